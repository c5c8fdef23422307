"""Sparse CSR operators (host side).

Mirrors brainpylib/sparse_ops.py for the part on the hot path: ``csr_matvec`` with the reference's
signature and checks (brainpylib/_src/sparse_ops/sparse_csr_matvec.py:26-98), lowered to the
custom-call targets its GPU translations name (:129-210), and ``cusparse_csr_matvec``'s signature
(brainpylib/_src/sparse_ops/cusparse_matvec.py:31-94) for the transposed product, which the
reference hands to cuSPARSE and this package computes with its own scatter kernel.
"""
from typing import Tuple

import torch

from . import _lib
from ._tensors import FLOAT_DTYPES, as_tensor, device_of, is_index_dtype, to_device

__all__ = ["csr_matvec", "cusparse_csr_matvec", "csr_to_coo", "coo_to_csr", "csr_to_dense", "check_csr"]


def _prepare(data, indices, indptr, vector):
  data = as_tensor(data)
  if data.ndim == 0:
    data = data.reshape(1)
  return data, as_tensor(indices), as_tensor(indptr), as_tensor(vector)


def _move(*tensors):
  device = device_of(*tensors)
  return (device,) + tuple(to_device(t, device) for t in tensors)


def _check(data, indices, indptr, vector, shape):
  if data.dtype not in FLOAT_DTYPES:
    raise TypeError(f'Only support float32 and float64. But we got {data.dtype}.')
  if data.dtype != vector.dtype:
    raise TypeError('The types of data and vector should be the same. '
                    f'But we got {data.dtype} != {vector.dtype}.')
  assert data.ndim == indices.ndim == indptr.ndim == vector.ndim == 1
  if not (is_index_dtype(indices.dtype) and is_index_dtype(indptr.dtype)):
    raise ValueError('indices and indptr should be 1D vectors with int32 or uint32 type.')
  if data.shape[0] not in [1, indices.shape[0]]:
    raise ValueError('The size of data should be 1 or be consistent with indices.')
  if len(shape) != 2:
    raise ValueError('shape should be a length-2 tuple.')
  if indptr.shape[0] != shape[0] + 1:
    raise ValueError(f'indptr should have shape[0] + 1 = {shape[0] + 1} entries, got {indptr.shape[0]}.')


def _int64(t):
  return t.view(torch.int32).to(torch.int64) if t.dtype == torch.uint32 else t.to(torch.int64)


def check_csr(indices, indptr, *, shape: Tuple[int, int]):
  """Raises ValueError unless (indices, indptr) describe a CSR matrix of `shape`: indptr starts at 0,
  never decreases and ends at len(indices); every column index lies in [0, shape[1]).

  The operators trust their index arrays, as the reference's kernels do (an index beyond the
  matrix is read or written where it points: lib/gpu_event_csr_matvec.cu:47-70 has no check
  either), so that no call pays for a pass over them.  This check is that pass, for callers who
  build the arrays themselves; it runs where the arrays live and synchronises once."""
  indices, indptr = as_tensor(indices), as_tensor(indptr)
  if not (is_index_dtype(indices.dtype) and is_index_dtype(indptr.dtype)):
    raise ValueError('indices and indptr should be 1D vectors with int32 or uint32 type.')
  if indices.ndim != 1 or indptr.ndim != 1 or len(shape) != 2:
    raise ValueError('indices and indptr should be 1D vectors and shape a length-2 tuple.')
  if indptr.shape[0] != shape[0] + 1:
    raise ValueError(f'indptr should have shape[0] + 1 = {shape[0] + 1} entries, got {indptr.shape[0]}.')
  # (uint32 arrays are looked at as int32: an entry of 2^31 or more then reads as negative and fails below)
  ptr = indptr.view(torch.int32) if indptr.dtype == torch.uint32 else indptr
  idx = indices.view(torch.int32) if indices.dtype == torch.uint32 else indices
  nnz = indices.shape[0]
  bad_ptr = (ptr[0] != 0) | (ptr[-1] != nnz) | (ptr[1:] < ptr[:-1]).any()
  bad_idx = ((idx < 0) | (idx >= shape[1])).any() if nnz else torch.zeros((), dtype=torch.bool, device=idx.device)
  bad_ptr, bad_idx = bool(bad_ptr), bool(bad_idx)
  if bad_ptr:
    raise ValueError(f'indptr should start at 0, never decrease and end at len(indices) = {nnz}.')
  if bad_idx:
    raise ValueError(f'indices should lie in [0, {shape[1]}).')


def csr_to_coo(indices, indptr):
  """Given CSR (indices, indptr) return COO (row, col)
  (brainpylib/_src/sparse_ops/utils.py:47-54)."""
  indices = as_tensor(indices)
  indptr = _int64(as_tensor(indptr))
  counts = indptr[1:] - indptr[:-1]
  row = torch.repeat_interleave(torch.arange(counts.shape[0], device=counts.device, dtype=torch.int64), counts,
                                output_size=indices.shape[0])
  return row.to(device=indices.device, dtype=torch.int32), indices


def coo_to_csr(pre_ids, post_ids, *, num_row: int):
  """(pre_ids, post_ids) -> (indices, indptr), rows in increasing order and the order within a
  row kept (brainpylib/_src/sparse_ops/utils.py:22-44)."""
  pre_ids = _int64(as_tensor(pre_ids))
  post_ids = as_tensor(post_ids)
  order = torch.argsort(pre_ids, stable=True)
  indices = post_ids[order]
  counts = torch.bincount(pre_ids, minlength=num_row)
  indptr = torch.zeros(num_row + 1, dtype=torch.int64, device=pre_ids.device)
  indptr[1:] = torch.cumsum(counts, 0)
  return indices, indptr.to(torch.int32)


def csr_to_dense(data, indices, indptr, *, shape: Tuple[int, int]):
  """Dense (shape[0], shape[1]) array of a CSR matrix; entries given more than once add up
  (brainpylib/_src/sparse_ops/utils.py:70-88)."""
  data = as_tensor(data)
  row, col = csr_to_coo(indices, indptr)
  if data.ndim == 0 or data.shape[0] == 1:
    data = data.reshape(1).expand(col.shape[0])
  dense = torch.zeros(shape, dtype=data.dtype, device=data.device)
  dense.index_put_((_int64(row.to(data.device)), _int64(col.to(data.device))), data, accumulate=True)
  return dense


def _launch(data, indices, indptr, vector, shape, transpose, method='vector'):
  """The custom call itself, on checked arguments."""
  device, data, indices, indptr, vector = _move(data, indices, indptr, vector)
  type_name = 'float' if data.dtype == torch.float32 else 'double'
  data_name = 'homo' if data.shape[0] == 1 else 'heter'
  opaque = _lib.build_double_size_descriptor(shape[0], shape[1])
  out = torch.empty(shape[1] if transpose else shape[0], dtype=data.dtype, device=device)
  if transpose:
    opaque = _lib.build_csr_transpose_descriptor(shape[0], shape[1], indices.shape[0])
    _lib.custom_call('csr_matvec_transpose_' + data_name + '_' + type_name, [data, indices, indptr, vector, out],
                     opaque)
    return out
  if method == 'adaptive':
    # the reference's adaptive target takes a `row_blocks` operand before the vector
    # (lib/gpu_csr_matvec.cu:519-521); it is not read by this implementation.
    row_blocks = torch.zeros(1, dtype=torch.int32, device=device)
    buffers = [data, indices, indptr, row_blocks, vector, out]
  else:
    buffers = [data, indices, indptr, vector, out]
  _lib.custom_call('csr_matvec_' + data_name + '_' + method + '_' + type_name, buffers, opaque)
  return out


def _wants_grad(*tensors):
  """True if a floating-point argument takes part in reverse- or forward-mode differentiation."""
  for t in tensors:
    if t.requires_grad:
      return True
    # (outside a dual level unpack_dual returns at once with no tangent)
    if t.is_floating_point() and torch.autograd.forward_ad.unpack_dual(t).tangent is not None:
      return True
  return False


class _CSRMatvec(torch.autograd.Function):
  """Differentiation rules of the CSR matrix-vector product
  (brainpylib/_src/sparse_ops/cusparse_matvec.py:281-308): tangents go through the same
  operator; the cotangent of the vector is the product with the transposed matrix; the
  cotangent of the weights is ``vector[col] * ct[row]`` per nonzero (rows and columns swapped
  when transposed), or its sum for a homogeneous weight."""

  @staticmethod
  def forward(data, indices, indptr, vector, shape, transpose, method):
    return _launch(data.detach(), indices, indptr, vector.detach(), shape, transpose, method)

  @staticmethod
  def setup_context(ctx, inputs, output):
    data, indices, indptr, vector, ctx.shape, ctx.transpose, ctx.method = inputs
    ctx.save_for_backward(data, indices, indptr, vector)
    ctx.save_for_forward(data, indices, indptr, vector)
    ctx.set_materialize_grads(False)

  @staticmethod
  def backward(ctx, ct):
    data, indices, indptr, vector = ctx.saved_tensors
    g_data = g_vector = None
    if ct is not None:
      ct = ct.contiguous()
      if ctx.needs_input_grad[3]:
        g_vector = _launch(data.detach(), indices, indptr, ct, ctx.shape, not ctx.transpose)
      if ctx.needs_input_grad[0]:
        if data.shape[0] == 1:
          ones = torch.ones(1, dtype=data.dtype, device=ct.device)
          g_data = torch.inner(ct, _launch(ones, indices, indptr, vector.detach(), ctx.shape, ctx.transpose)).reshape(1)
        else:
          row, col = csr_to_coo(indices, indptr)
          row, col = _int64(row), _int64(col)
          v = vector.detach()
          g_data = v[row] * ct[col] if ctx.transpose else v[col] * ct[row]
    return g_data, None, None, g_vector, None, None, None

  @staticmethod
  def jvp(ctx, d_data, d_indices, d_indptr, d_vector, *_):
    data, indices, indptr, vector = ctx.saved_tensors
    out = None
    if d_data is not None:
      out = _launch(d_data.contiguous(), indices, indptr, vector, ctx.shape, ctx.transpose)
    if d_vector is not None:
      t = _launch(data, indices, indptr, d_vector.contiguous(), ctx.shape, ctx.transpose)
      out = t if out is None else out + t
    return out


def _csr_matvec(data, indices, indptr, vector, shape, transpose, method='vector'):
  if _wants_grad(data, vector):
    device, data, indices, indptr, vector = _move(data, indices, indptr, vector)
    return _CSRMatvec.apply(data, indices, indptr, vector, tuple(shape), bool(transpose), method)
  return _launch(data, indices, indptr, vector, shape, transpose, method)


def csr_matvec(data, indices, indptr, vector, *, shape: Tuple[int, int], method: str = 'vector'):
  """CSR sparse matrix times dense vector: ``y[shape[0]] = A @ vector``.

  ``method`` is one of 'scalar', 'vector', 'adaptive' and selects the custom-call target name as in
  the reference; on this device all three run the same kernel family, which picks the number
  of lanes per row from the mean row length."""
  if method not in ['scalar', 'vector', 'adaptive']:
    raise ValueError('Only support methods: scalar, vector, and adaptive. '
                     f'But we got {method}.')
  data, indices, indptr, vector = _prepare(data, indices, indptr, vector)
  _check(data, indices, indptr, vector, shape)
  if vector.shape[0] != shape[1]:
    raise ValueError(f'Shape mismatch, mat {shape} @ vec ({vector.shape[0]},).')
  return _csr_matvec(data, indices, indptr, vector, shape, False, method)


def cusparse_csr_matvec(data, indices, indptr, vector, *, shape: Tuple[int, int], transpose: bool = False):
  """``A @ vector`` (transpose=False) or ``A.T @ vector`` (transpose=True) for a CSR matrix."""
  if not transpose:
    return csr_matvec(data, indices, indptr, vector, shape=shape)
  data, indices, indptr, vector = _prepare(data, indices, indptr, vector)
  _check(data, indices, indptr, vector, shape)
  if vector.shape[0] != shape[0]:
    raise ValueError(f'Shape mismatch, vec ({vector.shape[0]},) @ mat {shape}.')
  return _csr_matvec(data, indices, indptr, vector, shape, True)
