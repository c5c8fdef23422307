"""GPU parity of event_csr_matvec_batching against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

import brainpylib_amd as bpl
import benchdata as synth
from util import assert_close, assert_close_reordered, batched_csr

pytestmark = pytest.mark.gpu


def _check(oracle_mod, values, indices, indptr, events, batch, shape, transpose, what):
  want = oracle_mod.event_csr_matvec_batching(values, indices, indptr, events, batch_size=batch, shape=shape,
                                              transpose=transpose)
  got = bpl.event_csr_matvec_batching(values, indices, indptr, events, batch_size=batch, shape=shape,
                                      transpose=transpose).cpu().numpy()
  assert got.shape == want.shape and got.dtype == want.dtype
  if transpose:
    mag = oracle_mod.event_csr_matvec_batching(np.abs(values), indices, indptr, events, batch_size=batch,
                                               shape=shape, transpose=True)
    assert_close_reordered(got, want, mag, values.dtype.type, what=what)
  else:
    assert_close(got, want, what=what)
  return got, want


@pytest.mark.parametrize("shape", [(100, 200), (200, 100), (10, 1000), (1000, 10), (3000, 2500)])
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_batching_broadcast_combinations(cuda, oracle_mod, shape, transpose, dtype):
  rng = np.random.default_rng(11)
  n_in = shape[0] if transpose else shape[1]
  for dims, batch in (((1, 1, 1, 5), 5), ((1, 1, 1, 9), 9), ((1, 1, 1, 1), 1), ((1, 1, 1, 3), 20), ((1, 1, 1, 1), 4),
                      ((1, 3, 3, 1), 3), ((4, 1, 1, 4), 4), ((3, 3, 3, 3), 3), ((2, 1, 1, 3), 6)):
    vb, ib, pb, eb = dims
    print("case", shape, transpose, dtype.__name__, dims, batch, flush=True)
    data, indices, indptr = batched_csr(shape, 40 if shape[1] >= 100 else 5, max(vb, ib), seed=shape[0] + batch,
                                        dtype=dtype)
    events = rng.random((eb, n_in)) < 0.15
    _check(oracle_mod, data[:vb], indices[:ib], indptr[:pb], events, batch, shape, transpose, "heter bool")
    fev = (events * rng.uniform(0.5, 2.0, events.shape)).astype(dtype)
    _check(oracle_mod, data[:vb], indices[:ib], indptr[:pb], fev, batch, shape, transpose, "heter float")
    w = rng.standard_normal((vb, 1)).astype(dtype)
    # homogeneous weights are added once per synapse, as the reference adds them: its bits, whatever the order
    got, want = _check(oracle_mod, w, indices[:ib], indptr[:pb], events, batch, shape, transpose, "homo bool")
    assert np.array_equal(got, want)
    one = np.full((1, 1), 0.6, dtype=dtype)
    got, want = _check(oracle_mod, one, indices[:ib], indptr[:pb], events, batch, shape, transpose, "counts")
    assert np.array_equal(got, want)


def test_batching_short_and_long_rows_and_wide_matrices(cuda, oracle_mod):
  # mean row length below / above 32 selects 8 lanes / one wave per row; 200,000 columns do not
  # fit the LDS copy of the event masks (global probes)
  rng = np.random.default_rng(12)
  for n_row, n_col, mean in ((20000, 3000, 6), (2000, 3000, 300), (500, 200_000, 900), (30000, 200_000, 10)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    shape = (n_row, n_col)
    print("shape", shape, flush=True)
    events = rng.random((11, n_col)) < 0.05
    got, want = _check(oracle_mod, data[None], indices[None], indptr[None], events, 11, shape, False, "heter")
    one = np.full((1, 1), 0.7, dtype=np.float32)
    got, want = _check(oracle_mod, one, indices[None], indptr[None], events, 11, shape, False, "homo")
    assert np.array_equal(got, want), "homogeneous gather is bit-exact"


def test_batching_transposed_through_one_sorted_scatter(cuda, oracle_mod):
  # transpose=True with one matrix for all entries: the active rows of all entries go through one
  # coarse sort over batch * n_col virtual columns.  Many virtual rows (several row tiles per
  # producer), wide virtual outputs (sliced windows above 2^21), events broadcast (3 vectors for 6 entries).
  rng = np.random.default_rng(13)
  for n_row, n_col, mean, batch, eb, rate in ((20_000, 30_000, 30, 8, 8, 0.05), (300_000, 5000, 4, 6, 3, 0.6),
                                              (2000, 1_500_000, 200, 4, 4, 0.3)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    shape = (n_row, n_col)
    print("shape", shape, "batch", batch, flush=True)
    events = rng.random((eb, n_row)) < rate
    _check(oracle_mod, data[None], indices[None], indptr[None], events, batch, shape, True, "heter")
    one = np.full((1, 1), 0.6, dtype=np.float32)
    got, want = _check(oracle_mod, one, indices[None], indptr[None], events, batch, shape, True, "counts")
    assert np.array_equal(got, want)
    # twice in a row (the list's counter is back at zero), float events
    fev = (events * rng.uniform(0.5, 2.0, events.shape)).astype(np.float32)
    _check(oracle_mod, data[None], indices[None], indptr[None], fev, batch, shape, True, "heter float events")


def test_batching_equals_single_operator(cuda):
  # every row of the batched result is the single operator's result (exactly so for the
  # homogeneous weight, to rounding of one float64 sum otherwise)
  c = synth.config_event_csr_small()
  rng = np.random.default_rng(13)
  shape = c["shape"]
  events = rng.random((10, shape[1])) < 0.02
  got = bpl.event_csr_matvec_batching(np.full((1, 1), 0.6, np.float32), c["indices"][None], c["indptr"][None],
                                      events, batch_size=10, shape=shape)
  for bi in range(10):
    single = bpl.event_csr_matvec(np.float32(0.6), c["indices"], c["indptr"], events[bi], shape=shape)
    assert torch.equal(got[bi], single)


def test_batching_edge_cases(cuda, oracle_mod):
  indptr = np.array([[0, 0, 3, 3, 5]], dtype=np.int32)
  indices = np.array([[0, 2, 4, 1, 4]], dtype=np.int32)
  data = np.array([[1, 2, 3, 4, 5]], dtype=np.float32)
  shape = (4, 5)
  for tr in (False, True):
    n_in = shape[0] if tr else shape[1]
    for ev in (np.zeros((3, n_in), bool), np.ones((3, n_in), bool)):
      got, want = _check(oracle_mod, data, indices, indptr, ev, 3, shape, tr, "edge")
      assert np.array_equal(got, want)
  # empty batch, empty matrix
  out = bpl.event_csr_matvec_batching(data, indices, indptr, np.ones((1, 5), bool), batch_size=0, shape=shape)
  assert tuple(out.shape) == (0, 4)
  e = np.zeros((1, 0), dtype=np.int32)
  out = bpl.event_csr_matvec_batching(np.ones((1, 1), np.float32), e, np.zeros((1, 4), np.int32),
                                      np.ones((5, 7), bool), batch_size=5, shape=(3, 7)).cpu().numpy()
  assert out.shape == (5, 3) and not out.any()
  with pytest.raises(ValueError):
    bpl.event_csr_matvec_batching(data[0], indices, indptr, np.ones((1, 5), bool), batch_size=1, shape=shape)
  with pytest.raises(ValueError):
    bpl.event_csr_matvec_batching(data, indices, indptr, np.ones((1, 4), bool), batch_size=1, shape=shape)


def test_full_size_batching_rows_equal_single_operator(cuda):
  # 100,000 x 100,000, ~1e8 nnz, nine event vectors (two tiles of eight): every row of the batched
  # result against the single operator; the homogeneous weight bit for bit
  c = synth.config_event_csr_large()
  shape = c["shape"]
  dev = cuda
  data = torch.from_numpy(c["data"]).to(dev)
  indices = torch.from_numpy(c["indices"]).to(dev)
  indptr = torch.from_numpy(c["indptr"]).to(dev)
  rng = np.random.default_rng(17)
  events = torch.from_numpy(rng.random((9, shape[1])) < 0.05).to(dev)
  w = torch.full((1, 1), 0.6, dtype=torch.float32, device=dev)
  het = bpl.event_csr_matvec_batching(data[None], indices[None], indptr[None], events, batch_size=9, shape=shape)
  hom = bpl.event_csr_matvec_batching(w, indices[None], indptr[None], events, batch_size=9, shape=shape)
  for bi in range(9):
    single = bpl.event_csr_matvec(data, indices, indptr, events[bi], shape=shape)
    assert_close(het[bi].cpu().numpy(), single.cpu().numpy(), what="heter entry %d" % bi)
    single = bpl.event_csr_matvec(w[0], indices, indptr, events[bi], shape=shape)
    assert torch.equal(hom[bi], single)
