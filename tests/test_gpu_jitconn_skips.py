"""The jitconn kernels' two ways to a geometric skip, ceil(log(U) / log_p), compared on the device.

The exact way is the CPU code's arithmetic (lib/cpu_jitconn_event_matvec.cpp:24: fp64 log, IEEE
division, ceil), which the golden vectors pin; the fast way (hardware fp32 log2 of the mantissa) is
used only where the quotient is further from an integer than a guard band.  Here both are evaluated
for the same U, hashed ones and ones a few units in the last place either side of exp(k * log_p),
where ceil() changes; wherever the fast way was trusted it must give the exact way's integer.  The
guard band's width rests on an error bound of the hardware log2, which the third word measures
over every fp32 in [0.5, 1).
"""
import ctypes
import math
import struct

import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu

# how much of the error that the guard band allows for the fast path's log2(U) the fp32 value of U's two
# words can use up (two roundings, 2^-23 relative)
WORDS_TO_FP32 = 2.0 ** -23 / math.log(2.0)


def _check(log_p, n_draws, near_boundaries, seed=1):
  from brainpylib_amd import _lib
  lib = _lib.lib()
  lib.bpl_selfcheck_jitconn_skips.restype = ctypes.c_int
  lib.bpl_selfcheck_jitconn_skips.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int,
                                              ctypes.c_double, ctypes.c_void_p]
  counts = torch.zeros(4, dtype=torch.int64, device="cuda:0")
  stream = torch.cuda.current_stream()
  rc = lib.bpl_selfcheck_jitconn_skips(ctypes.c_void_p(stream.cuda_stream), seed, n_draws, int(near_boundaries),
                                       float(log_p), ctypes.c_void_p(counts.data_ptr()))
  assert rc == 0, _lib.last_error()
  torch.cuda.synchronize()
  differ, untrusted, worst_bits, allowed_bits = (int(v) for v in counts.cpu().numpy())
  as_double = lambda bits: struct.unpack("<d", struct.pack("<q", bits))[0]
  return differ, untrusted, as_double(worst_bits), as_double(allowed_bits)


@pytest.mark.parametrize("conn_prob", [0.9, 0.5, 0.1, 0.01, 1e-3, 1e-4, 1e-6])
def test_trusted_fast_skips_equal_exact_skips_for_hashed_words(conn_prob):
  import oracle
  n = 1 << 27
  differ, untrusted, _, allowed = _check(oracle.log_p_of(conn_prob), n, False, seed=int(1 / conn_prob))
  assert differ == 0
  # the band is 2 * guard wide around every integer: a draw falls into it with that probability
  guard = allowed * math.log(2.0) / abs(oracle.log_p_of(conn_prob)) + 1e-9
  expect = min(1.0, 2 * guard)
  assert untrusted <= n * (expect * 1.2 + 1e-6), (untrusted / n, expect)
  if expect < 0.5:
    assert untrusted >= n * expect * 0.8 - 100, (untrusted / n, expect)


@pytest.mark.parametrize("conn_prob", [0.5, 0.1, 0.01, 1e-3, 1e-4])
def test_trusted_fast_skips_equal_exact_skips_next_to_every_boundary(conn_prob):
  import oracle
  log_p = oracle.log_p_of(conn_prob)
  boundaries = min(int(43.0 / abs(log_p)), 1 << 21)  # exp(k log_p) down to 2^-62
  differ, untrusted, _, _ = _check(log_p, 64 * boundaries, True)
  assert differ == 0
  assert untrusted >= 32 * boundaries  # values this close to a boundary are (nearly all) inside the band


def test_hardware_log2_of_a_mantissa_is_within_the_error_the_guard_band_assumes():
  _, _, worst, allowed = _check(-0.001, 64, False)
  print("largest |hardware log2(m) - log2(m)| over the fp32 m in [0.5, 1): %.3e; allowed for log2(U): %.3e" % (worst, allowed))
  assert 1e-7 < allowed < 1e-6
  assert 0.0 < worst <= allowed - WORDS_TO_FP32 - 2e-8
