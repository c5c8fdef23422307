"""Just-in-time-connectivity operators (host side).

Mirrors brainpylib/jitconn_ops.py: same function names, keyword arguments, defaults and checks as
brainpylib/_src/jitconn_ops/event_matvec.py:36-147 and matvec.py:29-284, lowered to the
custom-call targets their GPU translations name (event_matvec.py:201-239, matvec.py:338-368).

The matrix ``M`` of shape ``shape`` is never stored: ``transpose`` only swaps the roles of the two
dimensions before the kernel, ``outdim_parallel`` selects one generator stream per output element
(True) or per input element with atomic accumulation (False).  Flipping BOTH flags gives the
exact transpose of the same matrix (the reference's transpose rule, event_matvec.py:263-273).
"""
from typing import Optional, Tuple

import numpy as np
import torch

from . import _lib
from ._tensors import FLOAT_DTYPES, as_tensor, device_of, to_device

__all__ = [
  'event_matvec_prob_conn_homo_weight', 'event_matvec_prob_conn_uniform_weight',
  'event_matvec_prob_conn_normal_weight',
  'matvec_prob_conn_homo_weight', 'matvec_prob_conn_uniform_weight', 'matvec_prob_conn_normal_weight',
  'matmat_prob_conn_uniform_weight', 'matmat_prob_conn_normal_weight',
  'event_matvec_prob_conn_hashed',
]


def _log_p(conn_prob):
  # event_matvec.py:217
  return float(np.log((1 - conn_prob) if conn_prob < 1 else 1e-40))


def _check_vector(vec, shape, transpose, what):
  if vec.ndim != 1:
    raise ValueError(f'{what} should be a 1D vector.')
  if len(shape) != 2:
    raise ValueError('shape should be a length-2 tuple.')
  if transpose:
    if vec.shape[0] != shape[0]:
      raise ValueError(f'Shape mismatch, vec ({vec.shape[0]},) @ mat {shape}.')
  else:
    if vec.shape[0] != shape[1]:
      raise ValueError(f'Shape mismatch, mat {shape} @ vec ({vec.shape[0]},).')


def _seed(seed):
  if seed is None:
    seed = int(np.random.randint(0, int(1e8)))
  return int(seed)


def _uniform_range(w_low, w_high, dtype):
  """(w_min, w_range) of the uniform descriptor.  The range is formed in the result type, the
  way std::uniform_real_distribution<T>{a, b} forms b - a on the reference's CPU path."""
  np_dt = np.float32 if dtype == torch.float32 else np.float64
  lo, hi = np_dt(w_low), np_dt(w_high)
  return float(lo), float(np_dt(hi - lo))


def _apply_weight(r, weight):
  """r * weight with weight in r's dtype (event_matvec.py:67-68).  A Python / numpy scalar is
  multiplied in as a scalar, which needs no host-to-device copy (and so can be graph captured)."""
  if isinstance(weight, torch.Tensor):
    return r * weight.to(device=r.device, dtype=r.dtype)
  w = np.asarray(weight.value if hasattr(weight, 'value') else weight)
  if w.ndim == 0:
    np_dt = np.float32 if r.dtype == torch.float32 else np.float64
    return r * float(np_dt(w))
  return r * torch.from_numpy(np.ascontiguousarray(w)).to(device=r.device, dtype=r.dtype)


def _type_name(dt):
  return '_float' if dt == torch.float32 else '_double'


def _launch(fn_prefix, w_kind, inp, out_dtype, suffix, *, conn_prob, shape, seed, transpose, outdim_parallel,
            w_a=0.0, w_b=0.0, version='v2'):
  n_row, n_col = (shape[1], shape[0]) if transpose else (shape[0], shape[1])
  if not (conn_prob > 0):
    raise ValueError(f'conn_prob should be in (0, 1], got {conn_prob}.')
  name = fn_prefix + ('' if outdim_parallel else '_atomic') + '_prob_' + w_kind + '_' + version + suffix
  if version == 'v1' and not outdim_parallel:
    # matvec.py:355-358 builds this name, lib/gpu_ops.cc registers no such target
    raise _lib.GPUOperatorNotFound(name)
  device = device_of(inp)
  inp = to_device(inp, device)
  # version 1 descriptors carry conn_prob itself (matvec.py:338-343), version 2 log(1 - conn_prob)
  log_p = float(conn_prob) if version == 'v1' else _log_p(conn_prob)
  if w_kind == 'homo':
    opaque = _lib.build_jitconn_prob_homo_descriptor(n_row, n_col, seed, log_p)
  elif w_kind == 'uniform':
    opaque = _lib.build_jitconn_prob_uniform_descriptor(n_row, n_col, seed, log_p, w_a, w_b)
  else:
    opaque = _lib.build_jitconn_prob_normal_descriptor(n_row, n_col, seed, log_p, w_a, w_b)
  out = torch.empty(n_row, dtype=out_dtype, device=device)
  _lib.custom_call(name, [inp, out], opaque)
  return out


class _JitconnMatvec(torch.autograd.Function):
  """Differentiation rules of the jitconn matvec primitives with respect to the input vector
  (brainpylib/_src/jitconn_ops/event_matvec.py:242-273, matvec.py:371-409): the tangent goes
  through the dense-vector operator with the same matrix, the cotangent through the dense-vector
  operator with ``transpose`` and ``outdim_parallel`` both flipped, which walks the same random
  streams along the other axis and therefore is the exact transpose of the same matrix."""

  @staticmethod
  def forward(inp, fn_prefix, w_kind, out_dtype, suffix, kw):
    return _launch(fn_prefix, w_kind, inp.detach(), out_dtype, suffix, **kw)

  @staticmethod
  def setup_context(ctx, inputs, output):
    _, _, ctx.w_kind, ctx.out_dtype, _, ctx.kw = inputs
    ctx.set_materialize_grads(False)

  @staticmethod
  def backward(ctx, ct):
    if ct is None or not ctx.needs_input_grad[0]:
      return None, None, None, None, None, None
    kw = dict(ctx.kw, transpose=not ctx.kw['transpose'], outdim_parallel=not ctx.kw['outdim_parallel'], version='v2')
    g = _launch('gpu_matvec', ctx.w_kind, ct.contiguous(), ct.dtype, _type_name(ct.dtype), **kw)
    return g, None, None, None, None, None

  @staticmethod
  def jvp(ctx, d_inp, *_):
    if d_inp is None:
      return None
    d_inp = d_inp.to(ctx.out_dtype)
    return _launch('gpu_matvec', ctx.w_kind, d_inp.contiguous(), ctx.out_dtype, _type_name(ctx.out_dtype), **ctx.kw)


def _run(fn_prefix, w_kind, inp, out_dtype, suffix, **kw):
  if inp.is_floating_point() and (inp.requires_grad or
                                  torch.autograd.forward_ad.unpack_dual(inp).tangent is not None):
    # move first (differentiably), so that the gradient comes back on the caller's device
    return _JitconnMatvec.apply(to_device(inp, device_of(inp)), fn_prefix, w_kind, out_dtype, suffix, kw)
  return _launch(fn_prefix, w_kind, inp, out_dtype, suffix, **kw)


def _event_types(events):
  # event_matvec.py:206-214: bool events give the default float type, float events their own
  if events.dtype == torch.bool:
    return torch.float32, '_float_bool'
  if events.dtype not in FLOAT_DTYPES:
    raise TypeError(f'events should be bool, float32 or float64, got {events.dtype}.')
  t = _type_name(events.dtype)
  return events.dtype, t + t


def event_matvec_prob_conn_homo_weight(events, weight, *, conn_prob: float, shape: Tuple[int, int],
                                       seed: Optional[int] = None, transpose: bool = False,
                                       outdim_parallel: bool = True):
  """``y = M @ events`` with ``M`` drawn just in time: each entry is ``weight`` with probability
  ``conn_prob``.  The kernel counts the active synapses per output; the product with ``weight``
  is applied afterwards, as in the reference."""
  events = as_tensor(events)
  _check_vector(events, shape, transpose, 'events')
  out_dtype, suffix = _event_types(events)
  r = _run('gpu_event_matvec', 'homo', events, out_dtype, suffix, conn_prob=conn_prob, shape=shape, seed=_seed(seed),
           transpose=transpose, outdim_parallel=outdim_parallel)
  return _apply_weight(r, weight)


def event_matvec_prob_conn_uniform_weight(events, *, w_low: float, w_high: float, conn_prob: float,
                                          shape: Tuple[int, int], seed: Optional[int] = None,
                                          transpose: bool = False, outdim_parallel: bool = True):
  """``y = M @ events`` with each connection's weight drawn uniformly from [w_low, w_high)."""
  events = as_tensor(events)
  assert w_high > w_low
  _check_vector(events, shape, transpose, 'events')
  out_dtype, suffix = _event_types(events)
  w_min, w_range = _uniform_range(w_low, w_high, out_dtype)
  return _run('gpu_event_matvec', 'uniform', events, out_dtype, suffix, conn_prob=conn_prob, shape=shape,
              seed=_seed(seed), transpose=transpose, outdim_parallel=outdim_parallel, w_a=w_min, w_b=w_range)


def event_matvec_prob_conn_normal_weight(events, *, w_mu: float, w_sigma: float, conn_prob: float,
                                         shape: Tuple[int, int], seed: Optional[int] = None,
                                         transpose: bool = False, outdim_parallel: bool = True):
  """``y = M @ events`` with each connection's weight drawn from N(w_mu, w_sigma^2)."""
  events = as_tensor(events)
  _check_vector(events, shape, transpose, 'events')
  out_dtype, suffix = _event_types(events)
  return _run('gpu_event_matvec', 'normal', events, out_dtype, suffix, conn_prob=conn_prob, shape=shape,
              seed=_seed(seed), transpose=transpose, outdim_parallel=outdim_parallel, w_a=w_mu, w_b=w_sigma)


def _dense(vector):
  vector = as_tensor(vector)
  if vector.dtype not in FLOAT_DTYPES:
    raise TypeError(f'vector should be float32 or float64, got {vector.dtype}.')
  return vector


def event_matvec_prob_conn_hashed(events, *, w_kind: str = 'homo', weight=1.0, w_low: float = 0.0,
                                  w_high: float = 1.0, w_mu: float = 0.0, w_sigma: float = 1.0, conn_prob: float,
                                  shape: Tuple[int, int], seed: int, transpose: bool = False,
                                  dtype=torch.float32):
  """``y = M @ events`` with the stateless connectivity of the reference's first GPU kernel
  generation (targets ``gpu_event_matvec_prob_{homo,uniform,normal}_{float,double}``,
  lib/gpu_jitconn_event_matvec.cu:10-79,138-215,281-362): synapse (row, col) exists iff a hash of
  ``seed + n_col * row + col`` falls below ``conn_prob``.  The reference registers these targets
  but none of its Python functions builds their names; this wrapper collects the event positions
  with ``event_info`` and calls them.  A different matrix from ``event_matvec_prob_conn_*_weight``."""
  from .event_ops import event_info
  if w_kind not in ('homo', 'uniform', 'normal'):
    raise ValueError(f'w_kind should be homo, uniform or normal, got {w_kind}.')
  if dtype not in FLOAT_DTYPES:
    raise TypeError(f'Only support float32 and float64. But we got {dtype}.')
  events = as_tensor(events)
  if events.ndim != 1:
    raise ValueError('events should be a 1D vector.')
  n_row, n_col = (shape[1], shape[0]) if transpose else (shape[0], shape[1])
  if events.shape[0] != n_col:
    raise ValueError(f'Shape mismatch, mat {(n_row, n_col)} @ vec ({events.shape[0]},).')
  ids, num = event_info(events)
  if w_kind == 'homo':
    opaque = _lib.build_jitconn_prob_homo_descriptor(n_row, n_col, seed, float(conn_prob))
  elif w_kind == 'uniform':
    opaque = _lib.build_jitconn_prob_uniform_descriptor(n_row, n_col, seed, float(conn_prob), float(w_low),
                                                        float(w_high) - float(w_low))
  else:
    opaque = _lib.build_jitconn_prob_normal_descriptor(n_row, n_col, seed, float(conn_prob), float(w_mu),
                                                       float(w_sigma))
  out = torch.empty(n_row, dtype=dtype, device=ids.device)
  _lib.custom_call('gpu_event_matvec_prob_' + w_kind + _type_name(dtype), [ids, num, out], opaque)
  return _apply_weight(out, weight) if w_kind == 'homo' else out


def _check_version(version):
  """matvec.py:102.  Both versions give the matrix of the reference's CPU path, which has one kernel for
  either (matvec.py:296-308)."""
  assert version in ['v1', 'v2']


def matvec_prob_conn_homo_weight(vector, weight, *, conn_prob: float, shape: Tuple[int, int],
                                 seed: Optional[int] = None, transpose: bool = False, outdim_parallel: bool = True,
                                 version: str = 'v2'):
  """``y = M @ vector`` with ``M`` drawn just in time with the scalar ``weight`` at each connection."""
  vector = _dense(vector)
  _check_vector(vector, shape, transpose, 'vector')
  _check_version(version)
  r = _run('gpu_matvec', 'homo', vector, vector.dtype, _type_name(vector.dtype), conn_prob=conn_prob, shape=shape,
           seed=_seed(seed), transpose=transpose, outdim_parallel=outdim_parallel, version=version)
  return _apply_weight(r, weight)


def matvec_prob_conn_uniform_weight(vector, *, w_low: float, w_high: float, conn_prob: float, shape: Tuple[int, int],
                                    seed: Optional[int] = None, transpose: bool = False,
                                    outdim_parallel: bool = True, version: str = 'v2'):
  """``y = M @ vector`` with each connection's weight drawn uniformly from [w_low, w_high)."""
  vector = _dense(vector)
  assert w_high > w_low
  _check_vector(vector, shape, transpose, 'vector')
  _check_version(version)
  w_min, w_range = _uniform_range(w_low, w_high, vector.dtype)
  return _run('gpu_matvec', 'uniform', vector, vector.dtype, _type_name(vector.dtype), conn_prob=conn_prob, shape=shape,
              seed=_seed(seed), transpose=transpose, outdim_parallel=outdim_parallel, w_a=w_min, w_b=w_range,
              version=version)


def matvec_prob_conn_normal_weight(vector, *, w_mu: float, w_sigma: float, conn_prob: float, shape: Tuple[int, int],
                                   seed: Optional[int] = None, transpose: bool = False,
                                   outdim_parallel: bool = True, version: str = 'v2'):
  """``y = M @ vector`` with each connection's weight drawn from N(w_mu, w_sigma^2)."""
  vector = _dense(vector)
  _check_vector(vector, shape, transpose, 'vector')
  _check_version(version)
  return _run('gpu_matvec', 'normal', vector, vector.dtype, _type_name(vector.dtype), conn_prob=conn_prob, shape=shape,
              seed=_seed(seed), transpose=transpose, outdim_parallel=outdim_parallel, w_a=w_mu, w_b=w_sigma,
              version=version)


def _matmat(w_kind, matrix, w_a, w_b, conn_prob, shape, seed, version):
  # checks of brainpylib/_src/jitconn_ops/matmat.py:226-235
  matrix = as_tensor(matrix)
  if matrix.ndim != 2:
    raise ValueError('vector should be a 2D matrix.')
  if len(shape) != 2:
    raise ValueError('shape should be a length-2 tuple.')
  if matrix.shape[1] != shape[0]:
    raise ValueError(f'Shape mismatch, X {tuple(matrix.shape)} @ M ({shape},).')
  if seed is None:
    raise ValueError('Seed cannot be none.')
  if matrix.dtype not in FLOAT_DTYPES:
    raise TypeError(f'matrix should be float32 or float64, got {matrix.dtype}.')
  if version != 'v1':
    raise _lib.GPUOperatorNotFound(f'matmat_prob_{w_kind} version {version}: only v1 generates the matrix the '
                                   'matvec operators generate')
  if not (conn_prob > 0):
    raise ValueError(f'conn_prob should be in (0, 1], got {conn_prob}.')
  device = device_of(matrix)
  matrix = to_device(matrix, device)
  m, k = matrix.shape
  n = shape[1]
  opaque = _lib.build_matmat_jit_prob_descriptor1(m, k, n, int(seed), _log_p(conn_prob), w_a, w_b)
  out = torch.empty((m, n), dtype=matrix.dtype, device=device)
  _lib.custom_call('gpu_matmat_prob_prob_' + w_kind + _type_name(matrix.dtype) + '_v1', [matrix, out], opaque)
  return out


def matmat_prob_conn_uniform_weight(matrix, *, w_low: float, w_high: float, conn_prob: float, shape: Tuple[int, int],
                                    seed: Optional[int] = None, version: str = 'v1'):
  """``Y = X @ M`` with ``M`` of shape ``shape`` drawn just in time, weights uniform in [w_low, w_high)."""
  assert w_high > w_low
  dt = as_tensor(matrix).dtype
  w_min, w_range = _uniform_range(w_low, w_high, dt if dt in FLOAT_DTYPES else torch.float32)
  return _matmat('uniform', matrix, w_min, w_range, conn_prob, shape, seed, version)


def matmat_prob_conn_normal_weight(matrix, *, w_mu: float, w_sigma: float, conn_prob: float, shape: Tuple[int, int],
                                   seed: Optional[int] = None, version: str = 'v1'):
  """``Y = X @ M`` with ``M`` of shape ``shape`` drawn just in time, weights N(w_mu, w_sigma^2).

  ``Y[i, :]`` equals ``matvec_prob_conn_normal_weight(X[i, :], shape=shape, transpose=True)``."""
  return _matmat('normal', matrix, w_mu, w_sigma, conn_prob, shape, seed, version)
