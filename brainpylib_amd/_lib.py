"""Loader of libbrainpylib_amd.so (ctypes) and the custom-call harness.

The operators in this package are thin argument-checking wrappers around the library's XLA
custom-call targets; this module calls a target exactly the way XLA's GPU runtime does:
``target(stream, buffers, opaque, opaque_len)`` with device pointers in ``buffers``.  PyTorch
only supplies device memory and the current HIP stream.

There is no fallback: if the library is missing or a target is unknown, the call raises.
"""
import ctypes
import functools
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libbrainpylib_amd.so")

_lib = None
_TARGET_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_char_p,
                              ctypes.c_size_t)
_targets = {}


class GPUOperatorNotFound(Exception):
  """Raised when a custom-call target is not available (the reference raises an exception of
  the same name from its GPU translations, brainpylib/_src/errors.py)."""

  def __init__(self, name):
    super().__init__("GPU operator for '%s' is not found: libbrainpylib_amd.so is missing or does not "
                     "export it. Build it with `python -m brainpylib_amd.build`." % name)


def lib():
  """The loaded shared library; builds nothing, raises if it is absent."""
  global _lib
  if _lib is None:
    if not os.path.exists(LIB_PATH):
      raise GPUOperatorNotFound(LIB_PATH)
    l = ctypes.CDLL(LIB_PATH)
    l.bpl_num_targets.restype = ctypes.c_int
    l.bpl_target_name.restype = ctypes.c_char_p
    l.bpl_target_name.argtypes = [ctypes.c_int]
    l.bpl_target_function.restype = ctypes.c_void_p
    l.bpl_target_function.argtypes = [ctypes.c_int]
    l.bpl_find_target.restype = ctypes.c_void_p
    l.bpl_find_target.argtypes = [ctypes.c_char_p]
    l.bpl_last_error.restype = ctypes.c_char_p
    l.bpl_version.restype = ctypes.c_char_p
    for name in ("bpl_build_twouint_onebool_descriptor", "bpl_build_double_size_descriptor",
                 "bpl_build_nonzero_descriptor", "bpl_build_jitconn_prob_homo_descriptor",
                 "bpl_build_jitconn_prob_uniform_descriptor", "bpl_build_jitconn_prob_normal_descriptor",
                 "bpl_build_matmat_jit_prob_descriptor1"):
      getattr(l, name).restype = ctypes.c_size_t
    _lib = l
  return _lib


def target_names():
  l = lib()
  return [l.bpl_target_name(i).decode() for i in range(l.bpl_num_targets())]


def target(name):
  fn = _targets.get(name)
  if fn is None:
    addr = lib().bpl_find_target(name.encode() if isinstance(name, str) else name)
    if not addr:
      raise GPUOperatorNotFound(name)
    fn = _TARGET_FN(addr)
    _targets[name] = fn
  return fn


def last_error():
  return lib().bpl_last_error().decode()


_PTR_ARRAYS = {}


def custom_call(name, buffers, opaque, stream=None):
  """Enqueue custom-call target ``name`` on ``stream`` (default: torch's current stream).

  ``buffers``: torch CUDA tensors (operands, then results), contiguous.  Asynchronous."""
  import torch
  fn = target(name)
  if stream is None:
    # (the raw handle; torch.cuda.current_stream() builds a Stream object first, which costs
    # several microseconds per call)
    try:
      stream = torch._C._cuda_getCurrentRawStream(buffers[0].device.index)
    except (AttributeError, TypeError):
      stream = torch.cuda.current_stream(buffers[0].device).cuda_stream
  n = len(buffers)
  array_type = _PTR_ARRAYS.get(n)
  if array_type is None:
    array_type = _PTR_ARRAYS[n] = ctypes.c_void_p * n
  ptrs = array_type(*[b.data_ptr() for b in buffers])
  fn(stream, ptrs, opaque, len(opaque))
  # the error string is per thread and empty unless a target has just failed
  err = lib().bpl_last_error()
  if err:
    lib().bpl_clear_error()
    raise RuntimeError(err.decode())


# ---- descriptor builders (same names and argument order as the reference's gpu_ops module,
# lib/gpu_ops.cc:181-198) ---------------------------------------------------------------------
def _build(fn_name, *args):
  buf = ctypes.create_string_buffer(64)
  n = getattr(lib(), fn_name)(*args, buf, ctypes.c_size_t(64))
  if n == 0:
    raise RuntimeError(fn_name + " failed")
  return buf.raw[:n]


@functools.lru_cache(maxsize=256)
def build_twouint_onebool_descriptor(uint_x, uint_y, bool_x):
  return _build("bpl_build_twouint_onebool_descriptor", ctypes.c_uint32(uint_x), ctypes.c_uint32(uint_y),
                ctypes.c_int(bool(bool_x)))


@functools.lru_cache(maxsize=256)
def build_event_csr_batching_descriptor(n_row, n_col, batch_size, values_batch, indices_batch, indptr_batch,
                                        events_batch, nnz, transpose):
  u = ctypes.c_uint32
  return _build("bpl_build_event_csr_batching_descriptor", u(n_row), u(n_col), u(batch_size), u(values_batch),
                u(indices_batch), u(indptr_batch), u(events_batch), u(nnz), ctypes.c_int(bool(transpose)))


@functools.lru_cache(maxsize=256)
def build_csr_event_sum_descriptor(pre_size, post_size):
  return _build("bpl_build_csr_event_sum_descriptor", ctypes.c_uint32(pre_size), ctypes.c_uint32(post_size))


@functools.lru_cache(maxsize=256)
def build_coo_event_sum_descriptor(conn_size, post_size):
  return _build("bpl_build_coo_event_sum_descriptor", ctypes.c_uint32(conn_size), ctypes.c_uint32(post_size))


@functools.lru_cache(maxsize=256)
def build_coo_atomic_sum_descriptor(conn_size, post_size):
  return _build("bpl_build_coo_atomic_sum_descriptor", ctypes.c_uint32(conn_size), ctypes.c_uint32(post_size))


@functools.lru_cache(maxsize=256)
def build_coo_atomic_prod_descriptor(conn_size, post_size):
  return _build("bpl_build_coo_atomic_prod_descriptor", ctypes.c_uint32(conn_size), ctypes.c_uint32(post_size))


@functools.lru_cache(maxsize=256)
def build_csr_event_prod_descriptor(pre_size, post_size):
  return _build("bpl_build_csr_event_prod_descriptor", ctypes.c_uint32(pre_size), ctypes.c_uint32(post_size))


@functools.lru_cache(maxsize=256)
def build_csr_transpose_descriptor(n_row, n_col, nnz):
  return _build("bpl_build_csr_transpose_descriptor", ctypes.c_uint32(n_row), ctypes.c_uint32(n_col),
                ctypes.c_uint32(nnz))


@functools.lru_cache(maxsize=256)
def build_double_size_descriptor(size_x, size_y):
  return _build("bpl_build_double_size_descriptor", ctypes.c_uint32(size_x), ctypes.c_uint32(size_y))


@functools.lru_cache(maxsize=256)
def build_nonzero_descriptor(event_size, batch_size):
  return _build("bpl_build_nonzero_descriptor", ctypes.c_uint32(event_size), ctypes.c_uint32(batch_size))


@functools.lru_cache(maxsize=256)
def build_jitconn_prob_homo_descriptor(n_row, n_col, seed, prob):
  return _build("bpl_build_jitconn_prob_homo_descriptor", ctypes.c_uint32(n_row), ctypes.c_uint32(n_col),
                ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_double(prob))


@functools.lru_cache(maxsize=256)
def build_jitconn_prob_uniform_descriptor(n_row, n_col, seed, prob, w_min, w_range):
  return _build("bpl_build_jitconn_prob_uniform_descriptor", ctypes.c_uint32(n_row), ctypes.c_uint32(n_col),
                ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_double(prob), ctypes.c_double(w_min),
                ctypes.c_double(w_range))


@functools.lru_cache(maxsize=256)
def build_jitconn_prob_normal_descriptor(n_row, n_col, seed, prob, w_mu, w_sigma):
  return _build("bpl_build_jitconn_prob_normal_descriptor", ctypes.c_uint32(n_row), ctypes.c_uint32(n_col),
                ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_double(prob), ctypes.c_double(w_mu),
                ctypes.c_double(w_sigma))


@functools.lru_cache(maxsize=256)
def build_matmat_jit_prob_descriptor1(m, k, n, seed, log_p, w1, w2):
  return _build("bpl_build_matmat_jit_prob_descriptor1", ctypes.c_uint32(m), ctypes.c_uint32(k),
                ctypes.c_uint32(n), ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_double(log_p),
                ctypes.c_double(w1), ctypes.c_double(w2))
