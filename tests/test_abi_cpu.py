"""The C-ABI library loads without a GPU, exports every symbol include/brainpylib_amd.h
declares, its registry lists exactly those targets, descriptors have the reference's layout and
a bad opaque is rejected without unwinding."""
import ctypes
import os
import re
import struct

import pytest

from brainpylib_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "brainpylib_amd.h")


def _declared():
  text = open(HEADER).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  targets = re.findall(r"^BPL_TARGET\((\w+)\);", text, flags=re.M)
  funcs = re.findall(r"^\s*(?:size_t|int|const char \*|void|bpl_target_fn)\s*\*?\s*(bpl_\w+)\(", text, flags=re.M)
  return targets, funcs


def test_library_exports_every_declared_symbol():
  targets, funcs = _declared()
  assert len(targets) >= 24 and len(funcs) >= 14
  lib = _lib.lib()
  for name in targets + funcs:
    assert hasattr(lib, name), name


def test_registry_lists_exactly_the_declared_targets():
  targets, _ = _declared()
  assert sorted(_lib.target_names()) == sorted(targets)
  lib = _lib.lib()
  for name in targets:
    addr = lib.bpl_find_target(name.encode())
    assert addr == ctypes.cast(getattr(lib, name), ctypes.c_void_p).value
  assert not lib.bpl_find_target(b"no_such_target")


def test_reference_target_names_present():
  # names registered by the reference (lib/gpu_ops.cc:72-174) for the operators built so far
  names = set(_lib.target_names())
  for data in ("homo", "heter"):
    for t in ("float_bool", "float_float", "double_bool", "double_double"):
      assert "event_csr_matvec_%s_%s" % (data, t) in names
    for m in ("scalar", "vector", "adaptive"):
      for t in ("float", "double"):
        assert "csr_matvec_%s_%s_%s" % (data, m, t) in names


def test_reference_registry_keys_of_the_other_operators_present():
  # lib/gpu_ops.cc:27-69 (the older event / atomic sums and products), :72-174 (jitconn, matmat, nonzero)
  names = set(_lib.target_names())
  want = []
  for w in ("homo", "uniform", "normal"):
    for t in ("float_bool", "float_float", "double_bool", "double_double"):
      want += ["gpu_event_matvec_prob_%s_v2_%s" % (w, t), "gpu_event_matvec_atomic_prob_%s_v2_%s" % (w, t)]
    for t in ("float", "double"):
      want += ["gpu_matvec_prob_%s_v2_%s" % (w, t), "gpu_matvec_atomic_prob_%s_v2_%s" % (w, t),
               "gpu_event_matvec_prob_%s_%s" % (w, t),  # first-generation event kernels
               "gpu_matvec_prob_%s_v1_%s" % (w, t)]  # first-generation dense names (lib/gpu_ops.cc:143-148)
  for w in ("normal", "uniform"):
    for t in ("float", "double"):
      want.append("gpu_matmat_prob_prob_%s_%s_v1" % (w, t))
  want += ["nonzero_" + t for t in ("bool", "int", "long", "float", "double")]
  for op in ("gpu_csr_event_sum", "gpu_coo_event_sum", "gpu_coo_atomic_sum", "gpu_coo_atomic_prod"):
    for data in ("homo", "heter"):
      for f in ("f32", "f64"):
        for i in ("i32", "i64"):
          want.append("%s_%s_%s_%s" % (op, data, f, i))
  missing = [n for n in want if n not in names]
  assert not missing, missing
  assert len(want) == 36 + 6 + 6 + 4 + 5 + 32  # + the 20 csr keys above: 109 of the reference's 113


@pytest.mark.parametrize("name", sorted(_lib.target_names()))
def test_every_target_refuses_a_malformed_call(name):
  # wrong opaque size, then a null buffer table: the call returns, launches nothing, records an error
  lib = _lib.lib()
  fn = _lib.target(name)
  bufs = (ctypes.c_void_p * 8)()
  lib.bpl_clear_error()
  fn(None, bufs, b"\x00" * 3, 3)
  assert "invalid opaque object size" in _lib.last_error()
  lib.bpl_clear_error()


def test_descriptor_layouts():
  # lib/kernel_helper_descriptor.cuh: native alignment, little endian
  assert _lib.build_twouint_onebool_descriptor(3, 4, True) == struct.pack("<IIB3x", 3, 4, 1)
  assert _lib.build_twouint_onebool_descriptor(3, 4, False) == struct.pack("<IIB3x", 3, 4, 0)
  assert _lib.build_double_size_descriptor(5, 6) == struct.pack("<II", 5, 6)
  assert _lib.build_nonzero_descriptor(7, 8) == struct.pack("<II", 7, 8)
  assert _lib.build_jitconn_prob_homo_descriptor(1, 2, 3, -0.25) == struct.pack("<III4xd", 1, 2, 3, -0.25)
  assert _lib.build_jitconn_prob_uniform_descriptor(1, 2, 3, -0.25, 0.5, 1.5) == struct.pack(
    "<III4xddd", 1, 2, 3, -0.25, 0.5, 1.5)
  assert _lib.build_jitconn_prob_normal_descriptor(1, 2, 3, -0.25, 0.5, 1.5) == struct.pack(
    "<III4xddd", 1, 2, 3, -0.25, 0.5, 1.5)
  assert _lib.build_matmat_jit_prob_descriptor1(1, 2, 3, 4, -0.25, 0.5, 1.5) == struct.pack(
    "<IIIIddd", 1, 2, 3, 4, -0.25, 0.5, 1.5)
  # log_p keeps double precision (the reference's builders narrow it to float)
  lp = -0.0010005003335835344
  assert struct.unpack("<III4xd", _lib.build_jitconn_prob_homo_descriptor(1, 2, 3, lp))[3] == lp


def test_builder_rejects_short_buffer():
  buf = ctypes.create_string_buffer(4)
  assert _lib.lib().bpl_build_double_size_descriptor(ctypes.c_uint32(1), ctypes.c_uint32(2), buf,
                                                     ctypes.c_size_t(4)) == 0


@pytest.mark.parametrize("name", ["event_csr_matvec_homo_float_bool", "csr_matvec_heter_vector_float",
                                  "csr_matvec_transpose_homo_double"])
def test_bad_opaque_is_reported_not_thrown(name, capfd):
  # the reference throws std::runtime_error("Invalid opaque object size") through the C boundary
  # (lib/kernel_helpers.h:36-38); here the call returns, launches nothing and records the error.
  lib = _lib.lib()
  lib.bpl_clear_error()
  fn = _lib.target(name)
  bufs = (ctypes.c_void_p * 6)()
  fn(None, bufs, b"\x00" * 5, 5)
  assert "invalid opaque object size" in _lib.last_error()
  assert "invalid opaque object size" in capfd.readouterr().err
  lib.bpl_clear_error()
  assert _lib.last_error() == ""


def test_unknown_target_fails_loudly():
  with pytest.raises(_lib.GPUOperatorNotFound):
    _lib.target("gpu_no_such_op")


def test_gpu_ops_module_matches_reference_interface():
  # lib/gpu_ops.cc:179-198: registrations() -> {name: PyCapsule("xla._CUSTOM_CALL_TARGET")}, build_* -> bytes
  from brainpylib_amd import gpu_ops
  regs = gpu_ops.registrations()
  assert sorted(regs) == sorted(_lib.target_names())
  api = ctypes.pythonapi
  api.PyCapsule_GetName.restype = ctypes.c_char_p
  api.PyCapsule_GetName.argtypes = [ctypes.py_object]
  api.PyCapsule_GetPointer.restype = ctypes.c_void_p
  api.PyCapsule_GetPointer.argtypes = [ctypes.py_object, ctypes.c_char_p]
  lib = _lib.lib()
  for name, cap in regs.items():
    assert api.PyCapsule_GetName(cap) == b"xla._CUSTOM_CALL_TARGET"
    assert api.PyCapsule_GetPointer(cap, b"xla._CUSTOM_CALL_TARGET") == lib.bpl_find_target(name.encode())
  assert gpu_ops.build_twouint_onebool_descriptor(3, 4, True) == struct.pack("<IIB3x", 3, 4, 1)
  assert gpu_ops.build_double_size_descriptor(5, 6) == struct.pack("<II", 5, 6)
  assert gpu_ops.build_coo_atomic_prod_descriptor(5, 6) == struct.pack("<II", 5, 6)  # lib/gpu_atomic_prod.cuh:10-13
  assert gpu_ops.build_csr_event_prod_descriptor(7, 8) == struct.pack("<II", 7, 8)
  assert gpu_ops.build_nonzero_descriptor(7, 8) == struct.pack("<II", 7, 8)
  assert gpu_ops.build_jitconn_prob_homo_descriptor(1, 2, 3, -0.25) == struct.pack("<III4xd", 1, 2, 3, -0.25)
  assert gpu_ops.build_jitconn_prob_uniform_descriptor(1, 2, 3, -0.25, 0.5, 1.0) == struct.pack(
    "<III4xddd", 1, 2, 3, -0.25, 0.5, 1.0)
  assert gpu_ops.build_jitconn_prob_normal_descriptor(1, 2, 3, -0.25, 0.5, 1.5) == struct.pack(
    "<III4xddd", 1, 2, 3, -0.25, 0.5, 1.5)
  assert gpu_ops.build_matmat_jit_prob_descriptor1(1, 2, 3, 4, -0.25, 0.5, 1.5) == struct.pack(
    "<IIIIddd", 1, 2, 3, 4, -0.25, 0.5, 1.5)


def test_jax_registration_shim_needs_jax():
  from brainpylib_amd import jax_register
  try:
    import jax  # noqa: F401
  except ImportError:
    with pytest.raises(ImportError):
      jax_register.register()


def test_missing_library_fails_loudly(monkeypatch):
  # no fallback: without the built library every operator raises
  import numpy as np
  import brainpylib_amd as bpl
  monkeypatch.setattr(_lib, "_lib", None)
  monkeypatch.setattr(_lib, "_targets", {})
  monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libbrainpylib_amd.so")
  with pytest.raises(_lib.GPUOperatorNotFound):
    _lib.target("event_csr_matvec_homo_float_bool")
  with pytest.raises(_lib.GPUOperatorNotFound):
    _lib.build_double_size_descriptor(11, 12)
