"""CPU oracle for the event-driven sparse operator path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the CPU-baseline leg of ``bench.py`` may import
this package.  The shipped package ``brainpylib_amd`` never does.

``liboracle.so`` is a plain-C restatement (``oracle.c``) of the reference's CPU algorithms;
``oracle.ref`` binds the reference's own C++ CPU kernels when they were compiled into
``_ref/libref_cpu.so`` (possible only where the reference tree is mounted).

Parity status of each oracle function (what pins it, beyond retyping the formula):

==============================  ==============================================================
function                        pinned by
==============================  ==============================================================
mt19937_words                   ISO C++ known answer (10000th output of seed 5489 = 4123659995)
canonical_f64 / canonical_f32   the reference's compiled C++ (libstdc++ 11.4), via the skip
                                and weight streams below
jitconn_matvec (sequential)     bit-exact vs the reference's compiled lib/cpu_jitconn_*.cpp on
                                the reference tests' shapes, all 4 walks x 3 weight kinds x
                                bool/float/double inputs; committed fixtures tests/golden/
jitconn_matvec (per-stream)     row r == compiled reference with one stream and seed+r;
                                closed form at conn_prob >= 1; geometric-gap statistics;
                                adjoint identity <y, Mx> == <M^T y, x>; shape-swap identity
jitconn_matmat                  reference test identity matmat == vmap(matvec(transpose=True));
                                no reference CPU kernel exists for it.  The one-pass form
                                (each stream generated once) == that definition bit for bit
                                (tests/test_oracle_jitconn.py); abs sums == float64 numpy on the
                                explicit matrix
event_csr_matvec                dense matmul brute force, scipy.sparse, homo == heter(ones*w),
                                bool == float events, compiled lib/cpu_event_sum.cc (transpose,
                                bool events)
csr_matvec                      dense matmul brute force, scipy.sparse (both orientations)
event_info                      numpy.flatnonzero
coo_atomic_sum, csr_event_sum   compiled lib/cpu_atomic_sum.cc, lib/cpu_event_sum.cc (fixtures),
(64-bit ids), coo_event_sum     the reference tests' known answers, numpy.bincount
coo_atomic_prod,                compiled lib/cpu_atomic_prod.cc, lib/cpu_event_prod.cc
csr_event_prod                  (fixtures), the reference tests' known answers, numpy
                                multiply.at / powers of the weight
event_matvec_hash, lfsr113,     the reference holds this algorithm as CUDA only.  Maximal period
taus88                          of every component recurrence (2^31-1, 2^29-1, 2^28-1, 2^25-1:
                                no wrong shift or mask constant survives that), GF(2)-linearity,
                                synapse fraction and weight moments, closed forms at prob 0 / 1
==============================  ==============================================================
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

W_HOMO, W_UNIFORM, W_NORMAL = 0, 1, 2
_W_KINDS = {"homo": W_HOMO, "uniform": W_UNIFORM, "normal": W_NORMAL}


def build(ref=True):
  """Compile liboracle.so (and the reference CPU kernels when the reference tree is present)."""
  subprocess.check_call(["make", "-s", "-C", _HERE, "-B", "liboracle.so"])
  if ref and os.path.isdir(os.environ.get("REFERENCE", "/root/reference") + "/lib"):
    subprocess.check_call(["make", "-s", "-C", _HERE, "ref"])


def lib():
  global _lib
  if _lib is None:
    if not os.path.exists(_LIB_PATH):
      build(ref=False)
    _lib = ctypes.CDLL(_LIB_PATH)
    _lib.oracle_jitconn_stream_indices.restype = ctypes.c_uint32
    _lib.oracle_jitconn_stream_weights_f32.restype = ctypes.c_uint32
    _lib.oracle_jitconn_stream_weights_f64.restype = ctypes.c_uint32
    _lib.oracle_get_threads.restype = ctypes.c_int
    _lib.oracle_lfsr_component_step.restype = ctypes.c_uint32
    _lib.oracle_lfsr_component_period.restype = ctypes.c_uint64
    _lib.oracle_lfsr113_word.restype = ctypes.c_uint32
  return _lib


def _p(a):
  return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
  a = np.ascontiguousarray(a, dtype=dtype)
  return a


def set_threads(n):
  lib().oracle_set_threads(ctypes.c_int(int(n)))


def log_p_of(conn_prob):
  """log(1 - p), or log(1e-40) when p >= 1 (brainpylib/_src/jitconn_ops/event_matvec.py:162)."""
  return float(np.log((1 - conn_prob) if conn_prob < 1 else 1e-40))


# ---------------------------------------------------------------------------------------------
# generator primitives
# ---------------------------------------------------------------------------------------------
def mt19937_words(seed, n, skip=0):
  out = np.empty(n, dtype=np.uint32)
  lib().oracle_mt19937_words(ctypes.c_uint32(seed), ctypes.c_uint32(skip), ctypes.c_uint32(n), _p(out))
  return out


def canonical_f64(seed, n):
  out = np.empty(n, dtype=np.float64)
  lib().oracle_canonical_f64(ctypes.c_uint32(seed), ctypes.c_uint32(n), _p(out))
  return out


def canonical_f32(seed, n):
  out = np.empty(n, dtype=np.float32)
  lib().oracle_canonical_f32(ctypes.c_uint32(seed), ctypes.c_uint32(n), _p(out))
  return out


def normal_stream(seed, mu, sigma, n, dtype=np.float32):
  out = np.empty(n, dtype=dtype)
  if np.dtype(dtype) == np.float32:
    lib().oracle_normal_f32(ctypes.c_uint32(seed), ctypes.c_float(mu), ctypes.c_float(sigma),
                            ctypes.c_uint32(n), _p(out))
  else:
    lib().oracle_normal_f64(ctypes.c_uint32(seed), ctypes.c_double(mu), ctypes.c_double(sigma),
                            ctypes.c_uint32(n), _p(out))
  return out


def jitconn_stream_indices(seed, log_p, n, cap=None):
  """Indices connected by the single generator stream std::mt19937{seed} over [0, n)."""
  if cap is None:
    cap = int(n)
  out = np.empty(max(cap, 1), dtype=np.uint32)
  cnt = lib().oracle_jitconn_stream_indices(ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_double(log_p),
                                            ctypes.c_uint32(n), _p(out), ctypes.c_uint32(cap))
  return out[:min(cnt, cap)].copy(), int(cnt)


def jitconn_stream_weights(seed, w_kind, w_a, w_b, log_p, n, dtype=np.float32, cap=None):
  if cap is None:
    cap = int(n)
  idx = np.empty(max(cap, 1), dtype=np.uint32)
  w = np.empty(max(cap, 1), dtype=dtype)
  f32 = np.dtype(dtype) == np.float32
  fn = lib().oracle_jitconn_stream_weights_f32 if f32 else lib().oracle_jitconn_stream_weights_f64
  ft = ctypes.c_float if f32 else ctypes.c_double
  cnt = fn(ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_int(_W_KINDS[w_kind]), ft(w_a), ft(w_b),
           ctypes.c_double(log_p), ctypes.c_uint32(n), _p(idx), _p(w), ctypes.c_uint32(cap))
  cnt = min(cnt, cap)
  return idx[:cnt].copy(), w[:cnt].copy()


# ---------------------------------------------------------------------------------------------
# jitconn operators
# ---------------------------------------------------------------------------------------------
def jitconn_matvec(inp, *, w_kind="homo", w_a=0.0, w_b=0.0, log_p, seed, n_row, n_col,
                   col_walk=False, per_stream_seed=True, out_dtype=None, dense=None, return_abs=False):
  """Kernel-level jitconn (event) matvec: returns the custom call's result (for ``homo`` that is
  the count / plain sum; the weight is applied by the caller as the reference does).
  ``return_abs=True`` returns ``(result, abs_sum)``, abs_sum[o] = sum of |addend| over the
  addends of output o in float64 (what bounds the effect of another order of the additions).

  ``inp`` bool -> event input; float with dense=False -> float events (truthiness);
  float with dense=True -> dense vector.  ``n_row`` outputs, ``n_col`` inputs.
  ``per_stream_seed=False`` is the reference CPU backend's single sequential generator."""
  inp = np.ascontiguousarray(inp)
  assert inp.ndim == 1 and inp.shape[0] == n_col
  if inp.dtype == np.bool_:
    in_kind = 0
    out_dtype = np.dtype(out_dtype or np.float32)
    buf = inp.view(np.uint8)
  else:
    if dense is None:
      raise ValueError("say whether a float input is a dense vector or float events")
    in_kind = 2 if dense else 1
    out_dtype = inp.dtype
    buf = inp
  assert out_dtype in (np.dtype(np.float32), np.dtype(np.float64))
  out = np.empty(n_row, dtype=out_dtype)
  f32 = out_dtype == np.float32
  ft = ctypes.c_float if f32 else ctypes.c_double
  args = (_p(buf), ctypes.c_int(in_kind), ctypes.c_int(_W_KINDS[w_kind]), ft(w_a), ft(w_b),
          ctypes.c_double(log_p), ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_uint32(n_row),
          ctypes.c_uint32(n_col), ctypes.c_int(int(col_walk)), ctypes.c_int(int(per_stream_seed)), _p(out))
  if return_abs:
    abs_sum = np.empty(n_row, dtype=np.float64)
    (lib().oracle_jitconn_matvec_abs_f32 if f32 else lib().oracle_jitconn_matvec_abs_f64)(*args, _p(abs_sum))
    return out, abs_sum
  (lib().oracle_jitconn_matvec_f32 if f32 else lib().oracle_jitconn_matvec_f64)(*args)
  return out


def jitconn_matmat(X, *, w_kind="normal", w_a, w_b, log_p, seed, n, return_abs=False, by_rows=False):
  """Y[m, n] = X[m, k] @ M[k, n]; column j of M is generator stream seed + j.

  ``by_rows=True`` is the definition taken literally (one matvec per row of X, the identity of
  brainpylib/_src/jitconn_ops/tests/matmat_testcase.py:133-138); the default generates every
  stream once and applies it to all rows, bit for bit the same result.  ``return_abs=True``
  returns ``(Y, abs_sum)`` with abs_sum[mi, j] = sum of |w * X[mi, i]| over column j's synapses."""
  X = np.ascontiguousarray(X)
  m, k = X.shape
  Y = np.empty((m, n), dtype=X.dtype)
  f32 = X.dtype == np.float32
  ft = ctypes.c_float if f32 else ctypes.c_double
  args = (_p(X), ctypes.c_int(_W_KINDS[w_kind]), ft(w_a), ft(w_b), ctypes.c_double(log_p),
          ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_uint32(m), ctypes.c_uint32(k), ctypes.c_uint32(n), _p(Y))
  if by_rows:
    assert not return_abs
    (lib().oracle_jitconn_matmat_by_rows_f32 if f32 else lib().oracle_jitconn_matmat_by_rows_f64)(*args)
    return Y
  abs_sum = np.empty((m, n), dtype=np.float64) if return_abs else None
  (lib().oracle_jitconn_matmat_f32 if f32 else lib().oracle_jitconn_matmat_f64)(
    *args, _p(abs_sum) if return_abs else ctypes.c_void_p(None))
  return (Y, abs_sum) if return_abs else Y


# ---------------------------------------------------------------------------------------------
# CSR operators
# ---------------------------------------------------------------------------------------------
def _csr_args(data, indices, indptr):
  data = np.atleast_1d(np.ascontiguousarray(data))
  assert data.dtype in (np.float32, np.float64)
  indices = np.ascontiguousarray(indices).view(np.uint32) if indices.dtype != np.uint32 else np.ascontiguousarray(indices)
  indptr = np.ascontiguousarray(indptr).view(np.uint32) if indptr.dtype != np.uint32 else np.ascontiguousarray(indptr)
  return data, indices, indptr


def event_csr_matvec(data, indices, indptr, events, *, shape, transpose=False):
  data, indices, indptr = _csr_args(data, indices, indptr)
  events = np.ascontiguousarray(events)
  if events.dtype == np.bool_:
    ev_kind, ev = 0, events.view(np.uint8)
  else:
    assert events.dtype == data.dtype
    ev_kind, ev = 1, events
  out = np.empty(shape[1] if transpose else shape[0], dtype=data.dtype)
  fn = lib().oracle_event_csr_matvec_f32 if data.dtype == np.float32 else lib().oracle_event_csr_matvec_f64
  fn(_p(data), ctypes.c_uint32(data.shape[0]), _p(indices), _p(indptr), _p(ev), ctypes.c_int(ev_kind),
     ctypes.c_uint32(shape[0]), ctypes.c_uint32(shape[1]), ctypes.c_int(int(transpose)), _p(out))
  return out


def event_csr_matvec_batching(values, indices, indptr, events, *, batch_size, shape, transpose=False):
  """2-D operands with a leading batch dimension; entry bi reads row bi % dim of each."""
  values = np.ascontiguousarray(values)
  assert values.ndim == 2 and values.dtype in (np.float32, np.float64)
  indices = np.ascontiguousarray(indices).view(np.uint32) if indices.dtype == np.int32 else np.ascontiguousarray(
    indices, dtype=np.uint32)
  indptr = np.ascontiguousarray(indptr).view(np.uint32) if indptr.dtype == np.int32 else np.ascontiguousarray(
    indptr, dtype=np.uint32)
  events = np.ascontiguousarray(events)
  assert indices.ndim == 2 and indptr.ndim == 2 and events.ndim == 2
  assert indptr.shape[1] == shape[0] + 1 and values.shape[1] in (1, indices.shape[1])
  assert events.shape[1] == (shape[0] if transpose else shape[1])
  if events.dtype == np.bool_:
    ev_kind, ev = 0, events.view(np.uint8)
  else:
    assert events.dtype == values.dtype
    ev_kind, ev = 1, events
  out = np.empty((batch_size, shape[1] if transpose else shape[0]), dtype=values.dtype)
  fn = (lib().oracle_event_csr_matvec_batching_f32 if values.dtype == np.float32
        else lib().oracle_event_csr_matvec_batching_f64)
  u = ctypes.c_uint32
  fn(_p(values), u(values.shape[0]), u(values.shape[1]), _p(indices), u(indices.shape[0]), u(indices.shape[1]),
     _p(indptr), u(indptr.shape[0]), _p(ev), ctypes.c_int(ev_kind), u(events.shape[0]), u(batch_size),
     u(shape[0]), u(shape[1]), ctypes.c_int(int(transpose)), _p(out))
  return out


def csr_matvec(data, indices, indptr, vector, *, shape, transpose=False):
  data, indices, indptr = _csr_args(data, indices, indptr)
  vector = np.ascontiguousarray(vector, dtype=data.dtype)
  out = np.empty(shape[1] if transpose else shape[0], dtype=data.dtype)
  fn = lib().oracle_csr_matvec_f32 if data.dtype == np.float32 else lib().oracle_csr_matvec_f64
  fn(_p(data), ctypes.c_uint32(data.shape[0]), _p(indices), _p(indptr), _p(vector),
     ctypes.c_uint32(shape[0]), ctypes.c_uint32(shape[1]), ctypes.c_int(int(transpose)), _p(out))
  return out


def _wide(ids):
  ids = np.ascontiguousarray(ids)
  if ids.dtype == np.int32:
    ids = ids.view(np.uint32)
  return ids.astype(np.uint64)


def coo_atomic_sum(values, post_ids, post_num, pre_ids=None):
  values = np.atleast_1d(np.ascontiguousarray(values))
  assert values.dtype in (np.float32, np.float64)
  post = _wide(post_ids)
  pre = post if values.shape[0] == 1 else _wide(pre_ids)
  assert pre.shape == post.shape
  out = np.empty(post_num, dtype=values.dtype)
  fn = lib().oracle_coo_atomic_sum_f32 if values.dtype == np.float32 else lib().oracle_coo_atomic_sum_f64
  fn(_p(values), ctypes.c_uint32(values.shape[0]), _p(post), _p(pre), ctypes.c_uint32(post.shape[0]),
     ctypes.c_uint32(post_num), _p(out))
  return out


def coo_atomic_prod(values, post_ids, post_num, pre_ids=None):
  values = np.atleast_1d(np.ascontiguousarray(values))
  assert values.dtype in (np.float32, np.float64)
  post = _wide(post_ids)
  pre = post if values.shape[0] == 1 else _wide(pre_ids)
  assert pre.shape == post.shape
  out = np.empty(post_num, dtype=values.dtype)
  fn = lib().oracle_coo_atomic_prod_f32 if values.dtype == np.float32 else lib().oracle_coo_atomic_prod_f64
  fn(_p(values), ctypes.c_uint32(values.shape[0]), _p(post), _p(pre), ctypes.c_uint32(post.shape[0]),
     ctypes.c_uint32(post_num), _p(out))
  return out


def csr_event_prod(events, pre2post, post_num, values):
  values = np.atleast_1d(np.ascontiguousarray(values))
  assert values.dtype in (np.float32, np.float64)
  events = np.ascontiguousarray(events)
  assert events.dtype == np.bool_
  indices, indptr = (_wide(a) for a in pre2post)
  assert indptr.shape[0] == events.shape[0] + 1 and values.shape[0] in (1, indices.shape[0])
  out = np.empty(post_num, dtype=values.dtype)
  fn = lib().oracle_csr_event_prod_f32 if values.dtype == np.float32 else lib().oracle_csr_event_prod_f64
  fn(_p(events.view(np.uint8)), _p(indices), _p(indptr), _p(values), ctypes.c_uint32(values.shape[0]),
     ctypes.c_uint32(events.shape[0]), ctypes.c_uint32(post_num), _p(out))
  return out


def coo_event_sum(events, pre_ids, post_ids, post_num, values):
  values = np.atleast_1d(np.ascontiguousarray(values))
  assert values.dtype in (np.float32, np.float64)
  events = np.ascontiguousarray(events)
  assert events.dtype == np.bool_
  pre, post = _wide(pre_ids), _wide(post_ids)
  assert pre.shape == post.shape and values.shape[0] in (1, pre.shape[0])
  out = np.empty(post_num, dtype=values.dtype)
  fn = lib().oracle_coo_event_sum_f32 if values.dtype == np.float32 else lib().oracle_coo_event_sum_f64
  fn(_p(events.view(np.uint8)), _p(pre), _p(post), _p(values), ctypes.c_uint32(values.shape[0]),
     ctypes.c_uint32(pre.shape[0]), ctypes.c_uint32(post_num), _p(out))
  return out


def csr_event_sum(events, pre2post, post_num, values):
  """The older name of the event scatter; 64-bit index arrays are narrowed (the index width of
  lib/cpu_event_sum.cc's template does not enter the arithmetic)."""
  indices, indptr = (np.ascontiguousarray(a).astype(np.uint32) for a in pre2post)
  return event_csr_matvec(values, indices, indptr, events, shape=(len(events), post_num), transpose=True)


_EVENT_KINDS = {np.dtype(np.bool_): 0, np.dtype(np.int32): 1, np.dtype(np.int64): 2,
                np.dtype(np.float32): 3, np.dtype(np.float64): 4}


def event_info(events):
  events = np.ascontiguousarray(events)
  ids = np.empty(events.shape[0], dtype=np.int32)
  num = np.empty(1, dtype=np.int32)
  buf = events.view(np.uint8) if events.dtype == np.bool_ else events
  lib().oracle_event_info(_p(buf), ctypes.c_int(_EVENT_KINDS[events.dtype]),
                          ctypes.c_uint32(events.shape[0]), _p(ids), _p(num))
  return ids, num


# ---- stateless ("hash") jitconn event matvec: lib/gpu_jitconn_event_matvec.cu:10-51,138-183,281-331 ----
def lfsr_component_step(gen, comp, z):
  """One step of component ``comp`` of taus88 (gen 0) or LFSR113 (gen 1)."""
  return int(lib().oracle_lfsr_component_step(ctypes.c_int(gen), ctypes.c_int(comp), ctypes.c_uint32(z)))


def lfsr_component_period(gen, comp, start, limit):
  return int(lib().oracle_lfsr_component_period(ctypes.c_int(gen), ctypes.c_int(comp), ctypes.c_uint32(start),
                                                ctypes.c_uint64(limit)))


def lfsr113_word(seed):
  """lfsr113_double(seed) * 2^32 (lib/kernel_helpers_random.cuh:55-71)."""
  return int(lib().oracle_lfsr113_word(ctypes.c_uint32(seed & 0xffffffff)))


def taus88_words(seed, n=2):
  out = (ctypes.c_uint32 * 2)()
  lib().oracle_taus88_words(ctypes.c_uint32(seed & 0xffffffff), ctypes.c_int(n), out)
  return [int(out[i]) for i in range(n)]


def event_matvec_hash(event_ids, event_num, *, w_kind="homo", w_a=0.0, w_b=0.0, prob, seed, n_row, n_col,
                      dtype=np.float32):
  """out[row] = sum over the first ``event_num`` listed columns c with
  lfsr113(seed + n_col * row + c) * 2^-32 < prob of the synapse's weight."""
  ids = _c(event_ids, np.int32)
  out = np.empty(n_row, dtype=dtype)
  fn = lib().oracle_event_matvec_hash_f32 if np.dtype(dtype) == np.float32 else lib().oracle_event_matvec_hash_f64
  fn(_p(ids), ctypes.c_int32(int(event_num)), ctypes.c_uint32(seed & 0xffffffff), ctypes.c_double(prob),
     ctypes.c_int(_W_KINDS[w_kind]), ctypes.c_double(w_a), ctypes.c_double(w_b), ctypes.c_uint32(n_row),
     ctypes.c_uint32(n_col), _p(out))
  return out
