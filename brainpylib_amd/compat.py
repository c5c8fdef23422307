"""The older operator names that brainpylib keeps for BrainPy models written against them
(brainpylib/_src/compat): ``csr_event_sum``, ``coo_event_sum``, ``coo_atomic_sum`` and the product
twins ``csr_event_prod`` and ``coo_atomic_prod``, with the reference's signatures and argument
checks, lowered to the custom-call targets its GPU translations name (event_sum.py:110-138,199-235,
atomic_sum.py:93-131, event_prod.py:107-127, atomic_prod.py:129-163)."""
import torch

from . import _lib
from ._tensors import FLOAT_DTYPES, as_tensor, device_of, to_device
from .event_ops import event_csr_matvec

__all__ = ["csr_event_sum", "coo_event_sum", "coo_atomic_sum", "csr_event_prod", "coo_atomic_prod"]

_INT_DTYPES = (torch.int32, torch.uint32, torch.int64, torch.uint64)


def _i_type(dt):
  return '_i32' if dt in (torch.int32, torch.uint32) else '_i64'


def _f_type(dt):
  return '_f32' if dt == torch.float32 else '_f64'


def _values(values):
  values = as_tensor(values)
  if values.ndim == 0:
    values = values.reshape(1)
  return values


def _csr_event_args(events, pre2post, post_num, values):
  """The argument checks csr_event_sum and csr_event_prod share (event_sum.py:33-62,
  event_prod.py:28-58)."""
  events = as_tensor(events)
  values = _values(values)
  indices, indptr = (as_tensor(a) for a in pre2post)
  post_num = int(post_num)
  if events.dtype != torch.bool:
    raise ValueError(f'"events" must be a vector of bool, while we got {events.dtype}')
  if len(events) + 1 != len(indptr):
    raise ValueError(f'The length of "events" must be equal to "len(pre2post[1]) - 1", '
                     f'while we get: {len(events)} + 1 != {len(indptr)}')
  if indices.dtype != indptr.dtype:
    raise ValueError(f"The dtype of pre2post[0] must be equal to that of pre2post[1], "
                     f"while we got {(indices.dtype, indptr.dtype)}")
  if indices.dtype not in _INT_DTYPES:
    raise ValueError(f'The dtype of pre2post must be integer, while we got {indices.dtype}')
  dtype = values.dtype
  if dtype not in FLOAT_DTYPES:
    raise ValueError(f'The dtype of "values" must be float32 or float64, while we got {dtype}.')
  if values.numel() not in [1, indices.numel()]:
    raise ValueError(f'The size of "values" must be 1 (a scalar) or len(pre2post[0]) (a vector), '
                     f'while we got {values.numel()} != 1 != {indices.numel()}')
  return events, indices, indptr, post_num, values.flatten()


def csr_event_sum(events, pre2post, post_num, values):
  """``out[post] += values`` over the synapses of every presynaptic neuron with an event
  (event_sum.py:33-63).  ``pre2post = (indices, indptr)``."""
  events, indices, indptr, post_num, values = _csr_event_args(events, pre2post, post_num, values)
  dtype = values.dtype
  if _i_type(indices.dtype) == '_i32':
    # the reference forwards to event_csr_matvec (event_sum.py:63)
    return event_csr_matvec(values, indices, indptr, events, shape=(events.shape[0], post_num), transpose=True)
  # 64-bit indices: event_csr_matvec takes 32-bit ones only, the older target does both
  device = device_of(values, indices, indptr, events)
  events, indices, indptr, values = (to_device(t, device) for t in (events, indices, indptr, values))
  out = torch.empty(post_num, dtype=dtype, device=device)
  name = 'gpu_csr_event_sum' + ('_homo' if values.shape[0] == 1 else '_heter') + _f_type(dtype) + '_i64'
  _lib.custom_call(name, [events, indices, indptr, values, out],
                   _lib.build_csr_event_sum_descriptor(events.shape[0], post_num))
  return out


def csr_event_prod(events, pre2post, post_num, values):
  """``out[post] *= values`` on a vector of ones, over the synapses of every presynaptic neuron
  with an event (event_prod.py:28-58; arithmetic of lib/cpu_event_prod.cc)."""
  events, indices, indptr, post_num, values = _csr_event_args(events, pre2post, post_num, values)
  device = device_of(values, indices, indptr, events)
  events, indices, indptr, values = (to_device(t, device) for t in (events, indices, indptr, values))
  out = torch.empty(post_num, dtype=values.dtype, device=device)
  name = ('gpu_csr_event_prod' + ('_homo' if values.shape[0] == 1 else '_heter') + _f_type(values.dtype) +
          _i_type(indices.dtype))
  _lib.custom_call(name, [events, indices, indptr, values, out],
                   _lib.build_csr_event_prod_descriptor(events.shape[0], post_num))
  return out


def coo_event_sum(events, pre_ids, post_ids, post_num, values):
  """``out[post_ids[i]] += values[i]`` for every connection ``i`` whose presynaptic neuron
  ``pre_ids[i]`` has an event (event_sum.py:151-178)."""
  events = as_tensor(events)
  pre_ids = as_tensor(pre_ids)
  post_ids = as_tensor(post_ids)
  values = _values(values)
  post_num = int(post_num)
  if events.dtype != torch.bool:
    raise ValueError(f'"events" must be a vector of bool, while we got {events.dtype}')
  if len(pre_ids) != len(post_ids):
    raise ValueError(f'The length of "pre_ids" must be equal to "post_ids", '
                     f'while we get: {len(pre_ids)} != {len(post_ids)}')
  if pre_ids.dtype != post_ids.dtype:
    raise ValueError(f'The dtype of "pre_ids" must be equal to that of "post_ids", '
                     f'while we got {(pre_ids.dtype, post_ids.dtype)}')
  if pre_ids.dtype not in _INT_DTYPES:
    raise ValueError(f'The dtype of "post_ids/pre_ids" must be a subtype of integer, '
                     f'while we got {pre_ids.dtype}')
  if values.dtype not in FLOAT_DTYPES:
    raise ValueError(f'The dtype of "values" must be float32 or float64, while we got {values.dtype}.')
  if values.numel() not in [1, pre_ids.numel()]:
    raise ValueError(f'The size of "values" must be 1 (a scalar) or len(pre_ids) (a vector), '
                     f'while we got {values.numel()} != 1 != {pre_ids.numel()}')
  values = values.flatten()
  device = device_of(values, pre_ids, post_ids, events)
  events, pre_ids, post_ids, values = (to_device(t, device) for t in (events, pre_ids, post_ids, values))
  out = torch.empty(post_num, dtype=values.dtype, device=device)
  name = ('gpu_coo_event_sum' + ('_homo' if values.shape[0] == 1 else '_heter') + _f_type(values.dtype) +
          _i_type(pre_ids.dtype))
  _lib.custom_call(name, [events, pre_ids, post_ids, values, out],
                   _lib.build_coo_event_sum_descriptor(pre_ids.shape[0], post_num))
  return out


def _coo_atomic(op, values, post_ids, post_num, pre_ids):
  """coo_atomic_sum and coo_atomic_prod: the same checks (atomic_sum.py:27-63,
  atomic_prod.py:28-62) and buffer order."""
  values = _values(values)
  post_ids = as_tensor(post_ids)
  post_num = int(post_num)
  if values.numel() != 1:
    assert pre_ids is not None, 'Must provide "pre_ids" when "values" is not a scalar.'
    pre_ids = as_tensor(pre_ids)
  else:
    pre_ids = post_ids
  if len(pre_ids) != len(post_ids):
    raise ValueError(f'The length of "pre_ids" and "post_ids" must be the same, '
                     f'while we got {len(pre_ids)} != {len(post_ids)}')
  if pre_ids.dtype != post_ids.dtype:
    raise ValueError(f"The dtype of pre_ids must be equal to that of post_ids, "
                     f"while we got {(pre_ids.dtype, post_ids.dtype)}")
  if post_ids.dtype not in _INT_DTYPES:
    raise ValueError(f'The dtype of post_ids must be a subtype of integer, while we got {post_ids.dtype}')
  if values.dtype not in FLOAT_DTYPES:
    raise ValueError(f'The dtype of "values" must be float32 or float64, while we got {values.dtype}.')
  values = values.flatten()
  homo = values.shape[0] == 1
  if not homo and pre_ids.numel() > 0:
    top = int(pre_ids.view(torch.int64 if _i_type(pre_ids.dtype) == '_i64' else torch.int32).max())
    if values.shape[0] <= top:
      raise ValueError(f'The size of "values" must be 1 (a scalar) or longer than pre_size (a vector), '
                       f'while we got {values.shape[0]} != 1 <= {top}')
  device = device_of(values, post_ids, pre_ids)
  values, post_ids, pre_ids = (to_device(t, device) for t in (values, post_ids, pre_ids))
  out = torch.empty(post_num, dtype=values.dtype, device=device)
  name = 'gpu_coo_atomic_' + op + ('_homo' if homo else '_heter') + _f_type(values.dtype) + _i_type(post_ids.dtype)
  buffers = [values, post_ids, out] if homo else [values, post_ids, pre_ids, out]
  build = _lib.build_coo_atomic_sum_descriptor if op == 'sum' else _lib.build_coo_atomic_prod_descriptor
  _lib.custom_call(name, buffers, build(post_ids.shape[0], post_num))
  return out


def coo_atomic_sum(values, post_ids, post_num, pre_ids=None):
  """``out[post_ids[i]] += values[pre_ids[i]]`` over all connections, or ``+= values`` for a
  scalar (atomic_sum.py:27-63)."""
  return _coo_atomic('sum', values, post_ids, post_num, pre_ids)


def coo_atomic_prod(values, post_ids, post_num, pre_ids=None):
  """``out[post_ids[i]] *= values[pre_ids[i]]`` on a vector of ones, over all connections, or
  ``*= values`` for a scalar (atomic_prod.py:28-62; arithmetic of lib/cpu_atomic_prod.cc)."""
  return _coo_atomic('prod', values, post_ids, post_num, pre_ids)
