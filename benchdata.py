"""Seeded synthetic inputs for the operator benchmarks and tests (numpy, host side).

Every generator is a pure function of its seed (numpy ``default_rng`` / PCG64), so the CPU
oracle and the GPU kernels can be fed identical arrays on any machine.  The reference takes its
test inputs from ``brainpy.conn.FixedProb`` and an unseeded ``brainpy.math.random``
(brainpylib/_src/event_ops/tests/test_event_csr_matvec.py:46-52); these generators stand in
for them.
"""
import numpy as np


def bernoulli_csr(n_row, n_col, p, seed):
  """CSR structure of an n_row x n_col matrix whose entries are present independently with
  probability p: per-row nnz ~ Binomial(n_col, p), columns sorted, unique and uniform.

  Drawn as geometric gaps along the flattened matrix, so the cost is O(nnz)."""
  rng = np.random.default_rng(seed)
  cells = int(n_row) * int(n_col)
  if cells == 0 or p <= 0:
    return np.zeros(0, np.int32), np.zeros(n_row + 1, np.int32)
  pos_chunks = []
  last = -1
  expect = cells * p
  chunk = int(min(max(expect * 1.05 + 1000, 1024), 5e7))
  while last < cells:
    gaps = rng.geometric(p, size=chunk).astype(np.int64)
    pos = last + np.cumsum(gaps)
    last = int(pos[-1])
    pos_chunks.append(pos)
  pos = np.concatenate(pos_chunks)
  pos = pos[pos < cells]
  rows = pos // n_col
  indices = (pos - rows * n_col).astype(np.int32)
  counts = np.bincount(rows, minlength=n_row)
  indptr = np.zeros(n_row + 1, dtype=np.int64)
  np.cumsum(counts, out=indptr[1:])
  assert indptr[-1] < 2 ** 31
  return indices, indptr.astype(np.int32)


def fixed_count_csr(n_row, n_col, k, seed):
  """Exactly k distinct uniform-random sorted columns per row."""
  rng = np.random.default_rng(seed)
  keys = rng.random((n_row, n_col))
  cols = np.argpartition(keys, k - 1, axis=1)[:, :k] if k < n_col else np.tile(np.arange(n_col), (n_row, 1))
  cols = np.sort(cols, axis=1).astype(np.int32)
  indptr = (np.arange(n_row + 1, dtype=np.int64) * k).astype(np.int32)
  return cols.reshape(-1), indptr


def counted_csr(counts, n_col, seed):
  """Rows with the given nnz counts; columns distinct, sorted, uniform in [0, n_col)."""
  rng = np.random.default_rng(seed)
  counts = np.asarray(counts, dtype=np.int64)
  n_row = counts.shape[0]
  indptr = np.zeros(n_row + 1, dtype=np.int64)
  np.cumsum(counts, out=indptr[1:])
  total = int(indptr[-1])
  assert total < 2 ** 31 and counts.max(initial=0) <= n_col
  rows = np.repeat(np.arange(n_row, dtype=np.int64), counts)
  key = rows * n_col + rng.integers(0, n_col, size=total, dtype=np.int64)
  # rows that want more than half of the columns take the head of a shuffle of all columns: drawing
  # again until nothing repeats would need ~n_col * ln(n_col) rounds for a full row
  crowded = np.flatnonzero(counts * 2 > n_col)
  if crowded.size:
    shuffle = np.random.default_rng([int(seed), 0x5eed])
    r = np.repeat(crowded, n_col)
    c = np.tile(np.arange(n_col, dtype=np.int64), crowded.size)
    order = np.lexsort((shuffle.random(r.size), r))
    keep = (np.arange(r.size) % n_col) < counts[r]
    crowded_key = (r * n_col + c[order])[keep]  # r is already grouped by row, in rising order
    key[np.isin(rows, crowded)] = crowded_key
  key.sort()
  # re-draw the few duplicates until every row's columns are distinct
  while True:
    dup = np.flatnonzero(key[1:] == key[:-1]) + 1
    if dup.size == 0:
      break
    key[dup] = rows[dup] * n_col + rng.integers(0, n_col, size=dup.size, dtype=np.int64)
    key.sort()
  indices = (key - rows * n_col).astype(np.int32)
  return indices, indptr.astype(np.int32)


def poisson_csr(n_row, n_col, lam, seed, min_count=1):
  rng = np.random.default_rng(seed)
  counts = np.maximum(min_count, rng.poisson(lam, size=n_row))
  return counted_csr(counts, n_col, seed + 1_000_003)


# ---- the five benchmark configurations ------------------------------------------------------
def config_event_csr_small(seed=0):
  """4,000 x 4,000, exactly 80 per row, homogeneous weight 0.6, events Bernoulli(0.02), transpose."""
  n = 4000
  indices, indptr = fixed_count_csr(n, n, 80, seed)
  rng = np.random.default_rng(seed + 1)
  events = rng.random(n) < 0.02
  return dict(data=np.array([0.6], dtype=np.float32), indices=indices, indptr=indptr, events=events,
              shape=(n, n))


def config_event_csr_large(seed=1, n=100_000, p=0.01, event_rate=0.05):
  """100,000 x 100,000, nnz per row ~ Binomial(n, 0.01) (~1e8 nnz), weights N(0, 0.1^2),
  events Bernoulli(0.05); used with transpose=True and transpose=False (square matrix)."""
  indices, indptr = bernoulli_csr(n, n, p, seed)
  rng = np.random.default_rng(seed + 1)
  data = (rng.standard_normal(indices.shape[0], dtype=np.float32) * np.float32(0.1))
  events = rng.random(n) < event_rate
  return dict(data=data, indices=indices, indptr=indptr, events=events, shape=(n, n))


def config_csr_matvec(seed=2, n=1_000_000, lam=100):
  """1,000,000 x 1,000,000, nnz per row ~ max(1, Poisson(100)), data U[0,1), vector N(0,1)."""
  indices, indptr = poisson_csr(n, n, lam, seed)
  rng = np.random.default_rng(seed + 1)
  data = rng.random(indices.shape[0], dtype=np.float32)
  vector = rng.standard_normal(n, dtype=np.float32)
  return dict(data=data, indices=indices, indptr=indptr, vector=vector, shape=(n, n))


def config_jitconn_event(n=1_000_000, conn_prob=0.001, event_rate=0.01, event_seed=4):
  """1e6 x 1e6 implicit matrix, conn_prob 0.001, weight 0.1, events Bernoulli(0.01), seed 42."""
  rng = np.random.default_rng(event_seed)
  return dict(events=rng.random(n) < event_rate, weight=np.float32(0.1), conn_prob=conn_prob,
              shape=(n, n), seed=42)


def config_jitconn_matmat(n=10_000, cols=128, conn_prob=0.1, seed=7, data_seed=8):
  """10,000 x 10,000 implicit matrix with N(0, 0.01^2) weights times a dense N(0,1) 10,000 x 128
  matrix B.  In the reference's orientation (Y = X @ M) that is X = B.T, Y = out.T."""
  rng = np.random.default_rng(data_seed)
  B = rng.standard_normal((n, cols), dtype=np.float32)
  return dict(B=B, w_mu=0.0, w_sigma=0.01, conn_prob=conn_prob, shape=(n, n), seed=seed)
