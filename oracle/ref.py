"""ctypes binding of the reference's own CPU kernels -- TEST INFRASTRUCTURE ONLY.

``_ref/libref_cpu.so`` is built by ``make -C oracle ref`` straight from the reference's C++
sources (lib/cpu_jitconn_*.cpp, lib/cpu_event_sum.cc); it exists only where that build ran.
The exported symbols are the reference's ``brainpy_lib::name(void** out, const void** in)``
functions (``void* out`` for cpu_event_sum), addressed by their Itanium-mangled names; the
operand order follows the CPU custom-call translations
(brainpylib/_src/jitconn_ops/event_matvec.py:183-192, matvec.py:318-327,602-615).
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "_ref", "libref_cpu.so")
_lib = None


def available():
  return os.path.exists(_PATH)


def _load():
  global _lib
  if _lib is None:
    _lib = ctypes.CDLL(_PATH)
  return _lib


def _sym(name, tuple_out=True):
  mangled = "_ZN11brainpy_lib%d%sE%s" % (len(name), name, "PPvPPKv" if tuple_out else "PvPPKv")
  return getattr(_load(), mangled)


def _ptr(a):
  return ctypes.c_void_p(a.ctypes.data)


def _suffix(dt):
  return "float" if np.dtype(dt) == np.float32 else "double"


def jitconn_matvec(inp, *, w_kind="homo", w_a=0.0, w_b=0.0, log_p, seed, n_row, n_col,
                   col_walk=False, out_dtype=None, dense=None):
  """Run the reference CPU custom-call target for one (event) matvec; same argument meaning as
  ``oracle.jitconn_matvec`` with the reference's single sequential generator."""
  inp = np.ascontiguousarray(inp)
  assert inp.shape == (n_col,)
  if inp.dtype == np.bool_:
    out_dtype = np.dtype(out_dtype or np.float32)
    name = "event_matvec%s_prob_%s_%s_bool" % ("_atomic" if col_walk else "", w_kind, _suffix(out_dtype))
  elif not dense:
    out_dtype = inp.dtype
    name = "event_matvec%s_prob_%s_%s_%s" % ("_atomic" if col_walk else "", w_kind,
                                            _suffix(out_dtype), _suffix(out_dtype))
  else:
    out_dtype = inp.dtype
    name = "matvec%s_prob_%s_%s" % ("_atomic" if col_walk else "", w_kind, _suffix(out_dtype))
  out = np.empty(n_row, dtype=out_dtype)
  logp = np.array(log_p, dtype=np.float64)
  sd = np.array(seed & 0xFFFFFFFF, dtype=np.uint32)
  nr = np.array(n_row, dtype=np.uint32)
  nc = np.array(n_col, dtype=np.uint32)
  if w_kind == "homo":
    ins = [inp, logp, sd, nr, nc]
  else:
    ins = [inp, logp, np.array(w_a, dtype=out_dtype), np.array(w_b, dtype=out_dtype), sd, nr, nc]
  in_arr = (ctypes.c_void_p * len(ins))(*[_ptr(a) for a in ins])
  out_arr = (ctypes.c_void_p * 1)(_ptr(out))
  _sym(name)(out_arr, in_arr)
  return out


def _ids(a, wide):
  """Index array as the kernels read it: unsigned 32- or 64-bit."""
  a = np.ascontiguousarray(a)
  if wide:
    return a.astype(np.uint64)
  return a.view(np.uint32) if a.dtype == np.int32 else a.astype(np.uint32)


def coo_atomic_sum(values, post_ids, post_num, pre_ids=None, *, wide=False):
  """lib/cpu_atomic_sum.cc: out[post_ids[i]] += values[pre_ids[i]] (heter, :6-23) or
  += values[0] (homo, :25-42); `wide` selects the 64-bit index instantiation."""
  values = np.atleast_1d(np.ascontiguousarray(values))
  post_ids = _ids(post_ids, wide)
  f = "f32" if values.dtype == np.float32 else "f64"
  i = "i64" if wide else "i32"
  out = np.empty(post_num, dtype=values.dtype)
  conn = np.array(post_ids.shape[0], dtype=np.uint32)
  size = np.array(post_num, dtype=np.uint32)
  if values.shape[0] == 1:
    kind, ins = "homo", [values, post_ids, conn, size]
  else:
    kind, ins = "heter", [values, _ids(pre_ids, wide), post_ids, conn, size]
  in_arr = (ctypes.c_void_p * len(ins))(*[_ptr(a) for a in ins])
  _sym("cpu_coo_atomic_sum_%s_%s_%s" % (kind, f, i), tuple_out=False)(_ptr(out), in_arr)
  return out


def coo_atomic_prod(values, post_ids, post_num, pre_ids=None, *, wide=False):
  """lib/cpu_atomic_prod.cc: on ones, out[post_ids[i]] *= values[pre_ids[i]] (heter, :5-23) or
  *= values[0] (homo, :25-43)."""
  values = np.atleast_1d(np.ascontiguousarray(values))
  post_ids = _ids(post_ids, wide)
  f = "f32" if values.dtype == np.float32 else "f64"
  i = "i64" if wide else "i32"
  out = np.empty(post_num, dtype=values.dtype)
  conn = np.array(post_ids.shape[0], dtype=np.uint32)
  size = np.array(post_num, dtype=np.uint32)
  if values.shape[0] == 1:
    kind, ins = "homo", [values, post_ids, conn, size]
  else:
    kind, ins = "heter", [values, _ids(pre_ids, wide), post_ids, conn, size]
  in_arr = (ctypes.c_void_p * len(ins))(*[_ptr(a) for a in ins])
  _sym("cpu_coo_atomic_prod_%s_%s_%s" % (kind, f, i), tuple_out=False)(_ptr(out), in_arr)
  return out


def csr_event_prod(data, indices, indptr, events, *, shape, wide=False):
  """lib/cpu_event_prod.cc: on ones, out[post] *= w for every synapse of every pre with
  events[pre]."""
  data = np.atleast_1d(np.ascontiguousarray(data))
  events = np.ascontiguousarray(events)
  assert events.dtype == np.bool_
  indices = _ids(indices, wide)
  indptr = _ids(indptr, wide)
  kind = "homo" if data.shape[0] == 1 else "heter"
  f = "f32" if data.dtype == np.float32 else "f64"
  out = np.empty(shape[1], dtype=data.dtype)
  pre = np.array(shape[0], dtype=np.uint32)
  post = np.array(shape[1], dtype=np.uint32)
  ins = [pre, post, events, indices, indptr, data]
  in_arr = (ctypes.c_void_p * len(ins))(*[_ptr(a) for a in ins])
  _sym("cpu_csr_event_prod_%s_%s_%s" % (kind, f, "i64" if wide else "i32"), tuple_out=False)(_ptr(out), in_arr)
  return out


def csr_event_sum(data, indices, indptr, events, *, shape, wide=False):
  """lib/cpu_event_sum.cc: out[post] += w for every synapse of every pre with events[pre]
  (the transpose=True, bool-event case of event_csr_matvec); `wide` selects the 64-bit index
  instantiation."""
  data = np.atleast_1d(np.ascontiguousarray(data))
  events = np.ascontiguousarray(events)
  assert events.dtype == np.bool_
  indices = _ids(indices, wide)
  indptr = _ids(indptr, wide)
  kind = "homo" if data.shape[0] == 1 else "heter"
  f = "f32" if data.dtype == np.float32 else "f64"
  out = np.empty(shape[1], dtype=data.dtype)
  pre = np.array(shape[0], dtype=np.uint32)
  post = np.array(shape[1], dtype=np.uint32)
  ins = [pre, post, events, indices, indptr, data]
  in_arr = (ctypes.c_void_p * len(ins))(*[_ptr(a) for a in ins])
  _sym("cpu_csr_event_sum_%s_%s_%s" % (kind, f, "i64" if wide else "i32"), tuple_out=False)(_ptr(out), in_arr)
  return out
