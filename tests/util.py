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


# What assert_close_reordered saw, per label: elements checked, elements outside the PLAIN bound
# (rel 1e-5 / abs 1e-6) that passed only through the reordering term.  conftest.py prints the
# totals at the end of a run, so the width of the gate is on record with every run.
REORDER_STATS = {}


def assert_close_reordered(got, want, abs_sum, dtype=np.float32, what="", max_outside_plain=None):
  """Tolerance for sums whose addends are accumulated in another ORDER in the same precision
  (atomic scatter vs the oracle's sequential loop): rel 1e-5 / abs 1e-6, plus the reordering
  bound 4 * eps * sum(|addends|) that two correctly rounded summation orders can differ by when
  the addends cancel.  `abs_sum` is that sum of magnitudes per output element.  The number of
  elements that lie outside the plain rel 1e-5 / abs 1e-6 bound (and pass through the extra term
  only) is recorded in REORDER_STATS and returned; `max_outside_plain` caps it."""
  got = np.asarray(got, dtype=np.float64)
  want = np.asarray(want, dtype=np.float64)
  err = np.abs(got - want)
  plain = ATOL + RTOL * np.abs(want)
  bound = plain + 4 * np.finfo(dtype).eps * np.asarray(abs_sum, dtype=np.float64)
  bad = err > bound
  outside_plain = int((err > plain).sum())
  seen = REORDER_STATS.setdefault(what or "unnamed", [0, 0])
  seen[0] += got.size
  seen[1] += outside_plain
  assert not bad.any(), "%s: %d of %d elements off; max abs err %.3e" % (what, int(bad.sum()), bad.size, float(err.max()))
  if max_outside_plain is not None:
    assert outside_plain <= max_outside_plain, "%s: %d elements outside rel 1e-5 / abs 1e-6 (allowed %d)" % (
      what, outside_plain, max_outside_plain)
  return outside_plain


def exact_scatter(indices, indptr, scale_per_row, data, n_col):
  """out[c] = sum over nonzeros j of column c of scale_per_row[row(j)] * data[j], where each product is
  rounded to the type of `data` first (as the operators form it) and the products are then summed
  in float64 and with math.fsum-like accuracy (float64 addends of 24-bit products: the float64 sum
  of a few thousand of them is exact to far below one unit in the last place of float32)."""
  dt = data.dtype.type
  rows = np.repeat(np.arange(indptr.shape[0] - 1), np.diff(indptr.astype(np.int64)))
  d = data if data.shape[0] == indices.shape[0] else np.full(indices.shape[0], data[0], dtype=dt)
  prod = (np.asarray(scale_per_row, dtype=dt)[rows] * d).astype(dt)
  keep = np.asarray(scale_per_row)[rows] != 0
  out = np.zeros(n_col, dtype=np.float64)
  np.add.at(out, indices[keep], prod[keep].astype(np.float64))
  return out


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
