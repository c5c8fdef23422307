"""Pins the oracle of the batched event_csr_matvec (the CPU kernels behind
vmap(event_csr_matvec), brainpylib/_src/event_ops/event_csr_matvec.py:112-193) against dense
float64 products and against the single operator applied entry by entry, the identity that the
reference's own vmap tests check (brainpylib/_src/event_ops/tests/test_event_csr_matvec.py:
76-126, vmap of the operator against vmap of the dense product)."""
import numpy as np
import pytest

from util import assert_close, batched_csr, to_dense

SHAPES = [(100, 200), (200, 100), (10, 1000), (1000, 10)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("dims", [(1, 1, 1, 5), (1, 3, 3, 1), (4, 1, 1, 4), (3, 3, 3, 3), (2, 1, 1, 3)])
def test_batching_vs_dense_and_single(oracle_mod, shape, transpose, dims):
  vb, ib, pb, eb = dims
  assert ib == pb
  batch = max(dims) if dims != (2, 1, 1, 3) else 6  # 6: both operands wrap around (bi % dim)
  nb = max(vb, ib)
  data, indices, indptr = batched_csr(shape, 6, nb, seed=shape[0] + 7 * batch)
  rng = np.random.default_rng(5)
  n_in = shape[0] if transpose else shape[1]
  events = rng.random((eb, n_in)) < 0.2
  for homo in (False, True):
    if homo:
      values = rng.standard_normal((vb, 1)).astype(np.float32)
    else:
      values = data[:vb]
    got = oracle_mod.event_csr_matvec_batching(values, indices[:ib], indptr[:pb], events, batch_size=batch,
                                               shape=shape, transpose=transpose)
    assert got.shape == (batch, shape[1] if transpose else shape[0]) and got.dtype == np.float32
    for bi in range(batch):
      v, ix, ip, ev = values[bi % vb], indices[bi % ib], indptr[bi % pb], events[bi % eb]
      dense = to_dense(v.astype(np.float64), ix, ip, shape)
      want = (ev.astype(np.float64) @ dense) if transpose else (dense @ ev.astype(np.float64))
      assert_close(got[bi], want, rtol=1e-5, atol=1e-5, what="entry %d" % bi)
      single = oracle_mod.event_csr_matvec(v, ix, ip, ev, shape=shape, transpose=transpose)
      assert np.array_equal(got[bi], single)
  # float events are tested for truthiness, as in the single operator
  fev = (events * rng.uniform(0.5, 2.0, events.shape)).astype(np.float32)
  a = oracle_mod.event_csr_matvec_batching(data[:vb], indices[:ib], indptr[:pb], fev, batch_size=batch, shape=shape,
                                           transpose=transpose)
  b = oracle_mod.event_csr_matvec_batching(data[:vb], indices[:ib], indptr[:pb], events, batch_size=batch,
                                           shape=shape, transpose=transpose)
  assert np.array_equal(a, b)


def test_batching_float64_and_empty_batch(oracle_mod):
  shape = (50, 70)
  data, indices, indptr = batched_csr(shape, 5, 1, seed=3, dtype=np.float64)
  events = np.random.default_rng(1).random((4, 70)) < 0.3
  got = oracle_mod.event_csr_matvec_batching(data, indices, indptr, events, batch_size=4, shape=shape)
  dense = to_dense(data[0], indices[0], indptr[0], shape)
  assert got.dtype == np.float64
  assert_close(got, events.astype(np.float64) @ dense.T, rtol=1e-12, atol=1e-12)
  got = oracle_mod.event_csr_matvec_batching(data, indices, indptr, events, batch_size=0, shape=shape)
  assert got.shape == (0, 50)
