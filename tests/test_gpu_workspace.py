"""The library's scratch memory (one cached allocation per stream): a buffer that was handed out
is never freed when a larger one replaces it, and nothing is allocated while the stream is being
captured into a HIP graph (the call fails instead and enqueues nothing)."""
import ctypes

import numpy as np
import pytest
import torch

import brainpylib_amd as bpl
from brainpylib_amd import _lib
import benchdata as synth

pytestmark = pytest.mark.gpu


def _query(stream_handle):
  lib = _lib.lib()
  lib.bpl_stream_workspace_query.restype = ctypes.c_int
  lib.bpl_stream_workspace_query.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p),
                                             ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
  ptr, size, retired = ctypes.c_void_p(), ctypes.c_size_t(), ctypes.c_size_t()
  has = lib.bpl_stream_workspace_query(ctypes.c_void_p(stream_handle), ctypes.byref(ptr), ctypes.byref(size),
                                       ctypes.byref(retired))
  return bool(has), ptr.value, size.value, retired.value


def _scatter_inputs(cuda, n_row, n_col, seed, dtype=np.float32):
  rng = np.random.default_rng(seed)
  indices, indptr = synth.counted_csr(rng.poisson(30, size=n_row), n_col, seed=seed)
  data = torch.from_numpy(rng.standard_normal(indices.shape[0]).astype(dtype)).to(cuda)
  ev = torch.from_numpy(rng.random(n_row) < 0.1).to(cuda)
  return data, torch.from_numpy(indices).to(cuda), torch.from_numpy(indptr).to(cuda), ev


def test_outgrown_buffer_is_retired_not_freed(cuda):
  s = torch.cuda.Stream()
  small = _scatter_inputs(cuda, 20_000, 20_000, 1)     # sorted scatter: 4,096 pairs per row, 0.6 GB of runs
  large = _scatter_inputs(cuda, 100_000, 100_000, 2)   # 1 GB of runs: a larger buffer
  torch.cuda.synchronize()
  with torch.cuda.stream(s):
    assert not _query(s.cuda_stream)[0]
    a = bpl.event_csr_matvec(*small, shape=(20_000, 20_000), transpose=True)
    has, p1, n1, r1 = _query(s.cuda_stream)
    assert has and p1 and n1 > 0 and r1 == 0
    b = bpl.event_csr_matvec(*large, shape=(100_000, 100_000), transpose=True)
    has, p2, n2, r2 = _query(s.cuda_stream)
    assert has and p2 != p1 and n2 >= 2 * n1
    assert r2 == n1, "the first buffer is kept (retired), not freed"
    # the same sizes again: no further growth
    a2 = bpl.event_csr_matvec(*small, shape=(20_000, 20_000), transpose=True)
    assert _query(s.cuda_stream)[1:] == (p2, n2, r2)
  s.synchronize()
  assert torch.allclose(a, a2, rtol=1e-5, atol=1e-5)
  # the retired buffer is still a valid allocation of its old size
  hip = ctypes.CDLL("libamdhip64.so")
  base, size = ctypes.c_void_p(), ctypes.c_size_t()
  rc = hip.hipMemGetAddressRange(ctypes.byref(base), ctypes.byref(size), ctypes.c_void_p(p1))
  assert rc == 0 and base.value == p1 and size.value == n1
  del b


def test_growth_is_refused_during_capture_and_works_after_a_warm_up(cuda, oracle_mod):
  s = torch.cuda.Stream()
  args = _scatter_inputs(cuda, 30_000, 30_000, 3)
  torch.cuda.synchronize()
  g = torch.cuda.CUDAGraph()
  with torch.cuda.stream(s):
    out = torch.zeros(30_000, dtype=torch.float32, device=cuda)
  s.synchronize()
  # cold stream: the call would have to allocate inside the capture; it must fail loudly instead
  with pytest.raises(RuntimeError, match="being captured"):
    with torch.cuda.graph(g, stream=s):
      bpl.event_csr_matvec(*args, shape=(30_000, 30_000), transpose=True)
  torch.cuda.synchronize()
  assert not _query(s.cuda_stream)[0], "nothing was allocated"
  # warmed on the stream first, the same call is captured and replays onto the same buffer
  with torch.cuda.stream(s):
    want = bpl.event_csr_matvec(*args, shape=(30_000, 30_000), transpose=True).clone()
  s.synchronize()
  # (the stream's first call: its counters and scratch memory were allocated inside it)
  host = [a.cpu().numpy() for a in args]
  ref = oracle_mod.event_csr_matvec(*host, shape=(30_000, 30_000), transpose=True)
  assert np.allclose(want.cpu().numpy(), ref, rtol=1e-5, atol=1e-5)
  before = _query(s.cuda_stream)
  g2 = torch.cuda.CUDAGraph()
  with torch.cuda.graph(g2, stream=s):
    out = bpl.event_csr_matvec(*args, shape=(30_000, 30_000), transpose=True)
  for _ in range(3):
    out.zero_()
    g2.replay()
    torch.cuda.synchronize()
    assert torch.allclose(out, want, rtol=1e-5, atol=1e-6)
  # a larger eager call on that stream afterwards moves on to a new buffer and leaves the graph's alone
  big = _scatter_inputs(cuda, 100_000, 120_000, 4, np.float64)  # (2 GB of float64 pairs)
  with torch.cuda.stream(s):
    bpl.event_csr_matvec(*big, shape=(100_000, 120_000), transpose=True)
  s.synchronize()
  after = _query(s.cuda_stream)
  assert after[1] != before[1] and after[3] >= before[2]
  out.zero_()
  g2.replay()
  torch.cuda.synchronize()
  assert torch.allclose(out, want, rtol=1e-5, atol=1e-6)
