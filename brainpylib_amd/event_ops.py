"""Event-driven CSR operators (host side).

Mirrors brainpylib/event_ops.py: ``event_csr_matvec`` with the reference's signature, argument
checks and error conditions (brainpylib/_src/event_ops/event_csr_matvec.py:32-102), lowered to the
custom-call target the reference's GPU translation names (same file, :389-417).
"""
from typing import Tuple

import torch

from . import _lib, sparse_ops
from ._tensors import FLOAT_DTYPES, as_tensor, device_of, is_index_dtype, to_device

__all__ = ["event_csr_matvec", "event_csr_matvec_batching", "event_info"]


def _type_name(dt):
  return "_float" if dt == torch.float32 else "_double"


def event_csr_matvec(data, indices, indptr, events, *, shape: Tuple[int, int], transpose: bool = False):
  """Product of a CSR matrix (or its transpose) and an event vector.

  data     scalar / shape (1,) (homogeneous weight) or shape (nse,)
  indices  (nse,) int32 | uint32;  indptr  (shape[0] + 1,) int32 | uint32
  events   (shape[0] if transpose else shape[1],) bool, or the float dtype of ``data``
  returns  (shape[1] if transpose else shape[0],) tensor of ``data``'s dtype on the GPU.
  """
  data = as_tensor(data)
  indices = as_tensor(indices)
  indptr = as_tensor(indptr)
  events = as_tensor(events)
  # checking (conditions and messages of the reference wrapper)
  if data.ndim == 0:
    data = data.reshape(1)
  if data.ndim == 1:
    if data.shape[0] not in [1, indices.shape[0]]:
      raise ValueError('The size of data should be 1 or be consistent with indices.'
                       f'But we got {tuple(data.shape)} != {tuple(indices.shape)}, {tuple(data.shape)} != 1.')
  else:
    raise ValueError('data should be a scalar or 1D vector. '
                     f'But we got {data.ndim}-D array.')
  if indices.ndim != 1:
    raise ValueError('indices should be a 1D vector with integer type.')
  if indptr.ndim != 1:
    raise ValueError('indptr should be a 1D vector with integer type.')
  if not is_index_dtype(indices.dtype):
    raise ValueError('indices should be a 1D vector with int32 or uint32 type.')
  if not is_index_dtype(indptr.dtype):
    raise ValueError('indptr should be a 1D vector with int32 or uint32 type.')
  if events.ndim != 1:
    raise ValueError('events should be a 1D vector.')
  if len(shape) != 2:
    raise ValueError('shape should be a length-2 tuple.')
  if transpose:
    if events.shape[0] != shape[0]:
      raise ValueError(f'Shape mismatch, vec ({events.shape[0]},) @ mat {shape}.')
  else:
    if events.shape[0] != shape[1]:
      raise ValueError(f'Shape mismatch, mat {shape} @ vec ({events.shape[0]},).')
  # what the kernels additionally rely on
  if data.dtype not in FLOAT_DTYPES:
    raise TypeError(f'Only support float32 and float64. But we got {data.dtype}.')
  if indptr.shape[0] != shape[0] + 1:
    raise ValueError(f'indptr should have shape[0] + 1 = {shape[0] + 1} entries, got {indptr.shape[0]}.')

  if events.dtype != torch.bool and events.dtype != data.dtype:
    raise ValueError('events should be bool or have the dtype of data, '
                     f'but we got {events.dtype} != {data.dtype}.')
  device = device_of(data, indices, indptr, events)
  data, indices, indptr, events = (to_device(t, device) for t in (data, indices, indptr, events))
  if sparse_ops._wants_grad(data, events):
    return _EventCSRMatvec.apply(data, indices, indptr, events, tuple(shape), bool(transpose))
  return _launch(data, indices, indptr, events, shape, transpose)


def _launch(data, indices, indptr, events, shape, transpose):
  """The custom call itself, on checked device tensors; the target name is built as the
  reference's GPU translation builds it."""
  type_name = _type_name(data.dtype)
  data_name = '_homo' if data.shape[0] == 1 else '_heter'
  vec_type = '_bool' if events.dtype == torch.bool else type_name
  opaque = _lib.build_twouint_onebool_descriptor(shape[0], shape[1], transpose)
  out = torch.empty(shape[1] if transpose else shape[0], dtype=data.dtype, device=data.device)
  _lib.custom_call('event_csr_matvec' + data_name + type_name + vec_type,
                   [data, indices, indptr, events, out], opaque)
  return out


class _EventCSRMatvec(torch.autograd.Function):
  """Differentiation rules of event_csr_matvec
  (brainpylib/_src/event_ops/event_csr_matvec.py:439-463).  Tangent of the weights: the same
  operator on the tangent.  Tangent of float events: the dense CSR product with the tangent.
  Cotangent of the weights: ``events[row] * ct[col]`` per nonzero when transposed, else
  ``events[col] * ct[row]`` (summed for a homogeneous weight, as ``inner(ct, op(1))``).
  Cotangent of float events: the dense product of the weights with ``ct`` along the other
  orientation (the reference passes the operands of that product in another order, :449,
  which only type-checks for a homogeneous weight; the product meant is computed here)."""

  @staticmethod
  def forward(data, indices, indptr, events, shape, transpose):
    return _launch(data.detach(), indices, indptr, events.detach(), shape, transpose)

  @staticmethod
  def setup_context(ctx, inputs, output):
    data, indices, indptr, events, ctx.shape, ctx.transpose = inputs
    ctx.save_for_backward(data, indices, indptr, events)
    ctx.save_for_forward(data, indices, indptr, events)
    ctx.set_materialize_grads(False)

  @staticmethod
  def backward(ctx, ct):
    data, indices, indptr, events = ctx.saved_tensors
    g_data = g_events = None
    if ct is not None:
      ct = ct.contiguous()
      if ctx.needs_input_grad[3]:
        g_events = sparse_ops._launch(data.detach(), indices, indptr, ct, ctx.shape, not ctx.transpose)
      if ctx.needs_input_grad[0]:
        if data.shape[0] == 1:
          ones = torch.ones(1, dtype=data.dtype, device=ct.device)
          g_data = torch.inner(ct, _launch(ones, indices, indptr, events.detach(), ctx.shape, ctx.transpose)).reshape(1)
        else:
          row, col = sparse_ops.csr_to_coo(indices, indptr)
          row, col = sparse_ops._int64(row), sparse_ops._int64(col)
          ev = events.detach().to(data.dtype)
          g_data = ev[row] * ct[col] if ctx.transpose else ev[col] * ct[row]
    return g_data, None, None, g_events, None, None

  @staticmethod
  def jvp(ctx, d_data, d_indices, d_indptr, d_events, *_):
    data, indices, indptr, events = ctx.saved_tensors
    out = None
    if d_data is not None:
      out = _launch(d_data.contiguous(), indices, indptr, events, ctx.shape, ctx.transpose)
    if d_events is not None:
      t = sparse_ops._launch(data, indices, indptr, d_events.contiguous(), ctx.shape, ctx.transpose)
      out = t if out is None else out + t
    return out


def event_csr_matvec_batching(values, indices, indptr, events, *, batch_size: int, shape: Tuple[int, int],
                              transpose: bool = False):
  """The primitive behind ``vmap(event_csr_matvec)``: every operand carries a leading batch
  dimension and entry ``bi`` of the result uses row ``bi % dim`` of each operand
  (brainpylib/_src/event_ops/event_csr_matvec.py:112-193; the batching rule passes a dimension
  of 1 for operands that are not mapped).

  values   (B_v, 1) homogeneous or (B_v, nse);  indices (B_i, nse);  indptr (B_p, shape[0] + 1)
  events   (B_e, shape[0] if transpose else shape[1]) bool, or the float dtype of ``values``
  returns  (batch_size, shape[1] if transpose else shape[0]) tensor of ``values``' dtype.

  The reference has this operator on the CPU only.  Here one matrix shared by the whole batch
  (B_v = B_i = B_p = 1) with ``transpose=False`` streams the column indices once per eight event
  vectors; every other combination runs the single operator once per batch entry."""
  values = as_tensor(values)
  indices = as_tensor(indices)
  indptr = as_tensor(indptr)
  events = as_tensor(events)
  for name, t in (("values", values), ("indices", indices), ("indptr", indptr), ("events", events)):
    if t.ndim != 2:
      raise ValueError(f'{name} should be a 2D array with a leading batch dimension, got {t.ndim}-D.')
    if t.shape[0] < 1:
      raise ValueError(f'{name} has an empty batch dimension.')
  if len(shape) != 2:
    raise ValueError('shape should be a length-2 tuple.')
  if batch_size < 0:
    raise ValueError('batch_size should not be negative.')
  if values.dtype not in FLOAT_DTYPES:
    raise TypeError(f'Only support float32 and float64. But we got {values.dtype}.')
  if not is_index_dtype(indices.dtype) or not is_index_dtype(indptr.dtype):
    raise ValueError('indices and indptr should have int32 or uint32 type.')
  nse = indices.shape[1]
  if values.shape[1] not in (1, nse):
    raise ValueError('The size of data should be 1 or be consistent with indices.'
                     f'But we got {tuple(values.shape)} != {tuple(indices.shape)}, {tuple(values.shape)} != 1.')
  if indptr.shape[1] != shape[0] + 1:
    raise ValueError(f'indptr should have shape[0] + 1 = {shape[0] + 1} entries, got {indptr.shape[1]}.')
  n_in = shape[0] if transpose else shape[1]
  if events.shape[1] != n_in:
    if transpose:
      raise ValueError(f'Shape mismatch, vec ({events.shape[1]},) @ mat {shape}.')
    raise ValueError(f'Shape mismatch, mat {shape} @ vec ({events.shape[1]},).')
  type_name = _type_name(values.dtype)
  # (B, 1) values with a single nonzero are homogeneous, as in the reference (`values.shape[1] == 1`)
  data_name = '_homo' if values.shape[1] == 1 else '_heter'
  if events.dtype == torch.bool:
    vec_type = '_bool'
  else:
    if events.dtype != values.dtype:
      raise ValueError('events should be bool or have the dtype of data, '
                       f'but we got {events.dtype} != {values.dtype}.')
    vec_type = type_name
  device = device_of(values, indices, indptr, events)
  values, indices, indptr, events = (to_device(t, device).contiguous() for t in (values, indices, indptr, events))
  opaque = _lib.build_event_csr_batching_descriptor(shape[0], shape[1], batch_size, values.shape[0],
                                                    indices.shape[0], indptr.shape[0], events.shape[0], nse,
                                                    transpose)
  out = torch.empty((batch_size, shape[1] if transpose else shape[0]), dtype=values.dtype, device=device)
  _lib.custom_call('event_csr_matvec_batching' + data_name + type_name + vec_type,
                   [values, indices, indptr, events, out], opaque)
  return out


_NONZERO_SUFFIX = {torch.bool: 'bool', torch.int32: 'int', torch.int64: 'long', torch.float32: 'float',
                   torch.float64: 'double'}


def event_info(events):
  """Collects the event positions and their number (brainpylib/_src/event_ops/
  event_info_collection.py:24-45).

  events: 1-D vector (a leading batch dimension is accepted, as the reference's vmap rule
  produces).  Returns ``(event_ids, event_num)``: int32 positions in increasing order padded with
  -1 to the length of ``events``, and the count with shape (1,) (or (batch,))."""
  events = as_tensor(events)
  if events.ndim not in (1, 2):
    raise TypeError('Only support 1D boolean vector.')
  if events.dtype not in _NONZERO_SUFFIX:
    raise ValueError(f'events should be bool, int32, int64, float32 or float64, got {events.dtype}.')
  device = device_of(events)
  events = to_device(events, device)
  batch = 1 if events.ndim == 1 else events.shape[0]
  size = events.shape[-1]
  ids = torch.empty(events.shape, dtype=torch.int32, device=device)
  num = torch.empty((batch,), dtype=torch.int32, device=device)
  _lib.custom_call('nonzero_' + _NONZERO_SUFFIX[events.dtype], [events, ids, num],
                   _lib.build_nonzero_descriptor(size, batch))
  return ids, num
