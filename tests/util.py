"""Helpers shared by the tests: seeded inputs, dense brute force, tolerance check."""
import numpy as np

import benchdata as synth

# north_star tolerance for fp32 outputs (atomics may reorder additions)
RTOL, ATOL = 1e-5, 1e-6

# shapes of the reference's own operator tests
# (brainpylib/_src/event_ops/tests/test_event_csr_matvec.py:36-44)
CSR_SHAPES = [(100, 200), (200, 200), (200, 100), (10, 1000), (2, 10000), (1000, 10), (10000, 2)]
# (brainpylib/_src/jitconn_ops/tests/test_event_matvec.py:10-14)
JIT_SHAPES = [(100, 200), (10, 1000), (2, 1000), (1000, 10), (1000, 2)]


def assert_close(got, want, rtol=RTOL, atol=ATOL, what=""):
  got = np.asarray(got, dtype=np.float64)
  want = np.asarray(want, dtype=np.float64)
  assert got.shape == want.shape, (what, got.shape, want.shape)
  err = np.abs(got - want)
  bad = err > atol + rtol * np.abs(want)
  assert not bad.any(), "%s: %d of %d elements off; max abs err %.3e, max rel err %.3e" % (
    what, int(bad.sum()), bad.size, float(err.max()), float((err / np.maximum(np.abs(want), 1e-30)).max()))


def random_csr(shape, p, seed, dtype=np.float32, weights="normal"):
  indices, indptr = synth.bernoulli_csr(shape[0], shape[1], p, seed)
  rng = np.random.default_rng(seed + 77)
  nnz = indices.shape[0]
  if weights == "normal":
    data = rng.standard_normal(nnz).astype(dtype)
  elif weights == "uniform":
    data = rng.random(nnz).astype(dtype)
  else:  # integers in {-1, 0, 1}: sums are exact in any order
    data = rng.integers(-1, 2, size=nnz).astype(dtype)
  return data, indices, indptr


def to_dense(data, indices, indptr, shape):
  dense = np.zeros(shape, dtype=np.float64)
  data = np.atleast_1d(data)
  for r in range(shape[0]):
    s, e = indptr[r], indptr[r + 1]
    dense[r, indices[s:e]] += (data[s:e] if data.shape[0] > 1 else data[0])
  return dense


def assert_close_reordered(got, want, abs_sum, dtype=np.float32, what=""):
  """Tolerance for sums whose addends are accumulated in another ORDER in the same precision
  (atomic scatter vs the oracle's sequential loop): rel 1e-5 / abs 1e-6, plus the reordering
  bound 4 * eps * sum(|addends|) that two correctly rounded summation orders can differ by when
  the addends cancel.  `abs_sum` is that sum of magnitudes per output element."""
  got = np.asarray(got, dtype=np.float64)
  want = np.asarray(want, dtype=np.float64)
  err = np.abs(got - want)
  bound = ATOL + RTOL * np.abs(want) + 4 * np.finfo(dtype).eps * np.asarray(abs_sum, dtype=np.float64)
  bad = err > bound
  assert not bad.any(), "%s: %d of %d elements off; max abs err %.3e" % (what, int(bad.sum()), bad.size, float(err.max()))


def batched_csr(shape, mean, batch, seed, dtype=np.float32):
  """`batch` different CSR matrices of one shape with the same number of nonzeros (the same row
  counts in another order), as 2-D arrays: data (batch, nnz), indices (batch, nnz),
  indptr (batch, shape[0] + 1)."""
  rng = np.random.default_rng(seed)
  counts = np.minimum(rng.poisson(mean, size=shape[0]), shape[1])
  data, indices, indptr = [], [], []
  for b in range(batch):
    ix, ip = synth.counted_csr(rng.permutation(counts), shape[1], seed=seed * 31 + b)
    indices.append(ix)
    indptr.append(ip)
    data.append(rng.standard_normal(ix.shape[0]).astype(dtype))
  return np.stack(data), np.stack(indices), np.stack(indptr)
