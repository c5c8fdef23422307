"""The allocation-free entry point event_csr_matvec_heter_float_bool_noalloc (scratch memory in a
static device array) against event_csr_matvec_heter_float_bool (scratch memory from the cached
allocation), through the C ABI: same buffers, same descriptor, the same result.  Gather results
and integer-valued weights must agree bit for bit; scattered fp32 sums of real weights within
rel 1e-5 / abs 1e-6 plus the reordering bound (both targets add with atomics, in an order that
changes from run to run)."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from brainpylib_amd import _lib
import benchdata as synth
from util import assert_close_reordered

pytestmark = pytest.mark.gpu

PLAIN = "event_csr_matvec_heter_float_bool"
NOALLOC = "event_csr_matvec_heter_float_bool_noalloc"


def _call(name, data, indices, indptr, events, shape, transpose, stream=None):
  out = torch.full((shape[1] if transpose else shape[0],), float("nan"), dtype=torch.float32, device=data.device)
  opaque = _lib.build_twouint_onebool_descriptor(shape[0], shape[1], transpose)
  _lib.custom_call(name, [data, indices, indptr, events, out], opaque, stream=stream)
  return out


def _case(cuda, n_row, n_col, mean, rate, seed, transpose, integer):
  rng = np.random.default_rng(seed)
  counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
  indices, indptr = synth.counted_csr(counts, n_col, seed=seed)
  if integer:
    data = rng.integers(-3, 4, size=indices.shape[0]).astype(np.float32)
  else:
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
  ev = rng.random(n_row if transpose else n_col) < rate
  return [torch.from_numpy(a).to(cuda) for a in (data, indices, indptr, ev)]


def _abs_sum(args, shape):
  data, indices, indptr, ev = [a.cpu().numpy() for a in args]
  rows = np.repeat(np.arange(shape[0]), np.diff(indptr))
  keep = ev[rows]
  return np.bincount(indices[keep], weights=np.abs(data[keep]).astype(np.float64), minlength=shape[1])


# (rows, columns, mean row length, event rate): each pair is a call followed by a SMALLER call that
# takes the same path, so that the second one finds the first one's lists, counters and runs in the array
SCATTER_PAIRS = [
  # sorted scatter (more than 8,192 columns): list + fill counters + runs
  ((60_000, 50_000, 60, 0.2), (20_000, 30_000, 40, 0.1)),
  # so little activity that the rows are added directly from the list
  ((60_000, 50_000, 60, 0.001), (9_000, 9_000, 10, 0.002)),
  # window scatter with a device list of active rows and partial outputs (more than 32,768 rows, narrow output)
  ((50_000, 6_000, 30, 0.3), (40_000, 3_000, 20, 0.05)),
  # window scatter, rows tested by the workgroups (4,097 .. 32,768 rows), then the one-launch kernel
  ((20_000, 8_000, 30, 0.3), (4_000, 4_000, 80, 0.02)),
]


@pytest.mark.parametrize("pair", SCATTER_PAIRS)
def test_noalloc_scatter_matches_the_allocating_target_twice_in_a_row(cuda, oracle_mod, pair):
  for integer in (True, False):
    for i, (n_row, n_col, mean, rate) in enumerate(pair):
      shape = (n_row, n_col)
      args = _case(cuda, n_row, n_col, mean, rate, seed=100 + i, transpose=True, integer=integer)
      print("scatter", shape, mean, rate, "integer" if integer else "real", flush=True)
      want = _call(PLAIN, *args, shape, True)
      got = _call(NOALLOC, *args, shape, True)
      torch.cuda.synchronize()
      assert not torch.isnan(got).any(), "every output element is written"
      host = [a.cpu().numpy() for a in args]
      cpu = oracle_mod.event_csr_matvec(*host, shape=shape, transpose=True)  # the oracle itself, not only the sibling
      if integer:
        assert torch.equal(got, want)
        assert np.array_equal(got.cpu().numpy(), cpu)
      else:
        mag = _abs_sum(args, shape)
        assert_close_reordered(got.cpu().numpy(), want.cpu().numpy(), mag, np.float32, what="noalloc scatter %s" % (shape,))
        assert_close_reordered(got.cpu().numpy(), cpu, mag, np.float32, what="noalloc scatter %s vs oracle" % (shape,))


def test_noalloc_gather_matches_bit_for_bit_twice_in_a_row(cuda, oracle_mod):
  # no transpose: an LDS bitmap (no scratch memory at all), then the two-level bitmap of a very wide
  # event vector (packed bitmap + coarse bitmap in the array), a smaller one after a larger one
  for n_row, n_col, mean, rate in ((30_000, 40_000, 50, 0.05), (3_000, 5_000_000, 100, 0.1),
                                   (2_000, 2_000_000, 60, 0.1), (500, 300, 20, 0.3)):
    shape = (n_row, n_col)
    args = _case(cuda, n_row, n_col, mean, rate, seed=n_row, transpose=False, integer=False)
    print("gather", shape, flush=True)
    want = _call(PLAIN, *args, shape, False)
    got = _call(NOALLOC, *args, shape, False)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    cpu = oracle_mod.event_csr_matvec(*[a.cpu().numpy() for a in args], shape=shape, transpose=False)
    assert np.array_equal(got.cpu().numpy(), cpu)


def test_noalloc_captured_cold_into_a_graph(cuda):
  # in a process of its own, so that the capture is the library's first call on each path: the device
  # address of the static array, the kernels' attributes and occupancy are all looked up under the capture
  child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "noalloc_capture_child.py")
  r = subprocess.run([sys.executable, "-u", child], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                     timeout=110)
  print(r.stdout, flush=True)
  assert r.returncode == 0, r.stdout[-3000:]
  assert "cold captures ok" in r.stdout


def test_noalloc_leaves_the_cached_allocation_alone_and_rejects_what_does_not_fit(cuda):
  lib = _lib.lib()
  lib.bpl_stream_workspace_query.restype = ctypes.c_int
  lib.bpl_stream_workspace_query.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
  s = torch.cuda.Stream()
  args = _case(cuda, 30_000, 30_000, 30, 0.1, seed=7, transpose=True, integer=True)
  torch.cuda.synchronize()
  with torch.cuda.stream(s):
    got = _call(NOALLOC, *args, (30_000, 30_000), True, stream=s.cuda_stream)
  s.synchronize()
  assert lib.bpl_stream_workspace_query(ctypes.c_void_p(s.cuda_stream), None, None, None) == 0, \
      "the stream has no cached scratch allocation: the call took none"
  want = _call(PLAIN, *args, (30_000, 30_000), True)
  torch.cuda.synchronize()
  assert torch.equal(got, want)
  # 8 bytes per row of active-row list beyond the 64 MiB array: rejected before anything is enqueued
  # (the operands are never touched, so small stand-ins do)
  n_row = 9_000_000
  out = torch.zeros(20_000, dtype=torch.float32, device=cuda)
  opaque = _lib.build_twouint_onebool_descriptor(n_row, 20_000, True)
  with pytest.raises(RuntimeError, match="allocation-free entry point holds"):
    _lib.custom_call(NOALLOC, [args[0], args[1], args[2], args[3], out], opaque)
  torch.cuda.synchronize()
  assert float(out.abs().sum()) == 0.0
