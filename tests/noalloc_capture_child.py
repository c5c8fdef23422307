"""Run as a process of its own by tests/test_zz_no_alloc.py: the allocation-free entry point captured
into a HIP graph COLD -- the capture is the first call this process makes into the library on that
path (symbol lookup, kernel attributes and occupancy queries all happen under the capture), on a
stream the library has never seen.  Every replay is compared with the CPU oracle, then with the
allocating target.  Exit code 0 = every check passed."""
import ctypes
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from brainpylib_amd import _lib  # noqa: E402
import benchdata as synth        # noqa: E402
import oracle                    # noqa: E402
from util import assert_close_reordered  # noqa: E402

PLAIN = "event_csr_matvec_heter_float_bool"
NOALLOC = "event_csr_matvec_heter_float_bool_noalloc"

# (rows, columns, mean row length, event rate, transpose): one case per path of the entry point
CASES = [
  ("sorted scatter", 60_000, 50_000, 60, 0.2, True),
  ("rows added directly from the list", 60_000, 50_000, 60, 0.001, True),
  ("window scatter with a device list", 50_000, 6_000, 30, 0.3, True),
  ("window scatter, rows found by the workgroups", 20_000, 8_000, 30, 0.3, True),
  ("one-launch scatter", 4_000, 4_000, 80, 0.02, True),
  ("gather, two-level bitmap", 3_000, 5_000_000, 100, 0.1, False),
  ("gather, LDS bitmap", 30_000, 40_000, 50, 0.05, False),
]


def main():
  dev = torch.device("cuda:0")
  torch.cuda.set_device(dev)
  lib = _lib.lib()
  lib.bpl_stream_workspace_query.restype = ctypes.c_int
  lib.bpl_stream_workspace_query.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
  other = torch.cuda.Stream()  # eager work between the replays runs here, through the allocating target
  grown = 0
  for ci, (what, n_row, n_col, mean, rate, transpose) in enumerate(CASES):
    print("capture cold:", what, (n_row, n_col), flush=True)
    rng = np.random.default_rng(40 + ci)
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=40 + ci)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    ev = rng.random(n_row if transpose else n_col) < rate
    want = oracle.event_csr_matvec(data, indices, indptr, ev, shape=(n_row, n_col), transpose=transpose)
    mag = oracle.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=(n_row, n_col), transpose=transpose)
    args = [torch.from_numpy(a).to(dev) for a in (data, indices, indptr, ev)]
    out = torch.full((n_col if transpose else n_row,), float("nan"), dtype=torch.float32, device=dev)
    opaque = _lib.build_twouint_onebool_descriptor(n_row, n_col, transpose)
    s = torch.cuda.Stream()  # a stream of its own per case: never used before its capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
      _lib.custom_call(NOALLOC, args + [out], opaque)
    assert lib.bpl_stream_workspace_query(ctypes.c_void_p(s.cuda_stream), None, None, None) == 0, \
        "the captured call took no cached allocation"
    for replay in range(3):
      out.fill_(float("nan"))
      torch.cuda.synchronize()
      g.replay()
      torch.cuda.synchronize()
      got = out.cpu().numpy()
      assert not np.isnan(got).any(), (what, replay, "every output element is written")
      if transpose:
        assert_close_reordered(got, want, mag, np.float32, what="%s, replay %d" % (what, replay))
      else:
        assert np.array_equal(got, want), (what, replay)
      if replay == 0:
        # eager work on another stream that makes that stream's cached allocation grow: a larger
        # scatter through the allocating target
        big_rows = 80_000 + 40_000 * ci
        ix2, ip2 = synth.counted_csr(np.full(big_rows, 20), 70_000, seed=ci)
        a2 = [torch.from_numpy(a).to(dev) for a in (np.ones(ix2.shape[0], np.float32), ix2, ip2,
                                                    np.ones(big_rows, np.bool_))]
        o2 = torch.empty(70_000, dtype=torch.float32, device=dev)
        with torch.cuda.stream(other):
          _lib.custom_call(PLAIN, a2 + [o2], _lib.build_twouint_onebool_descriptor(big_rows, 70_000, True))
        other.synchronize()
        size = ctypes.c_size_t(0)
        assert lib.bpl_stream_workspace_query(ctypes.c_void_p(other.cuda_stream), None, ctypes.byref(size), None) == 1
        assert size.value >= grown
        grown = size.value
        assert float(o2.sum()) == 20.0 * big_rows
    # and the allocating target, eagerly, after the replays
    ref = torch.full_like(out, float("nan"))
    _lib.custom_call(PLAIN, args + [ref], opaque)
    torch.cuda.synchronize()
    if transpose:
      assert_close_reordered(out.cpu().numpy(), ref.cpu().numpy(), mag, np.float32, what=what + " vs allocating target")
    else:
      assert torch.equal(out, ref)
  print("cold captures ok: %d paths, 3 replays each" % len(CASES), flush=True)


if __name__ == "__main__":
  main()
