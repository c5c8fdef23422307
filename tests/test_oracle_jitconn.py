"""Pins the jitconn oracle: against the golden vectors produced by the reference's compiled CPU
kernels, against those kernels live where they are built, and against what the mathematics
fixes (closed form at p >= 1, geometric gap law, adjoint identity, the reference tests' own
shape-swap and matmat identities)."""
import json
import os

import numpy as np
import pytest

from util import JIT_SHAPES, assert_close

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _cases():
  z = np.load(os.path.join(GOLD, "jitconn_cpu_reference.npz"))
  zs = np.load(os.path.join(GOLD, "jitconn_cpu_reference_streams.npz"))
  n = sum(1 for k in z.files if k.startswith("meta_"))
  for i in range(n):
    yield i, z["in_%d" % i], json.loads(str(z["meta_%d" % i])), z["out_%d" % i], zs["out_%d" % i]


def _oracle_call(oracle, inp, meta, per_stream):
  return oracle.jitconn_matvec(
    inp, w_kind=meta["w_kind"], w_a=meta["w_a"], w_b=meta["w_b"], log_p=oracle.log_p_of(meta["conn_prob"]),
    seed=meta["seed"], n_row=meta["n_row"], n_col=meta["n_col"], col_walk=meta["col_walk"],
    per_stream_seed=per_stream, out_dtype=np.dtype(meta["out_dtype"]) if meta["out_dtype"] else None,
    dense=meta["dense"])


def test_sequential_oracle_reproduces_reference_golden_bit_for_bit(oracle_mod):
  n = 0
  for i, inp, meta, out, _ in _cases():
    got = _oracle_call(oracle_mod, inp, meta, per_stream=False)
    assert got.dtype == out.dtype
    assert np.array_equal(got.view(np.uint8), out.view(np.uint8)), (i, meta)
    n += 1
  assert n == 450


def test_per_stream_oracle_reproduces_reference_one_stream_at_a_time(oracle_mod):
  for i, inp, meta, _, out_streams in _cases():
    got = _oracle_call(oracle_mod, inp, meta, per_stream=True)
    if not meta["col_walk"]:
      # element r is the reference's own result for (n_row=1, seed + r): bit-exact
      assert np.array_equal(got.view(np.uint8), out_streams.view(np.uint8)), (i, meta)
    elif meta["w_kind"] == "homo" and not meta["dense"]:
      assert np.array_equal(got.astype(np.float64), out_streams), (i, meta)  # counts
    else:
      # columns accumulate into shared outputs: same addends, float64 golden sum
      assert_close(got, out_streams, rtol=1e-5, atol=1e-5, what=str(meta))


def test_oracle_against_live_reference_build(oracle_mod, ref_mod):
  rng = np.random.default_rng(9)
  for (n_row, n_col) in [(37, 411), (411, 37)]:
    for p in (0.05, 0.3):
      for col_walk in (False, True):
        for wk, a, b in (("homo", 0, 0), ("uniform", 0.1, 0.9), ("normal", -1.0, 0.3)):
          for inp, dense in ((rng.random(n_col) < 0.2, None),
                             (rng.standard_normal(n_col).astype(np.float32), True),
                             (rng.standard_normal(n_col), True)):
            kw = dict(w_kind=wk, w_a=a, w_b=b, log_p=oracle_mod.log_p_of(p), seed=99, n_row=n_row, n_col=n_col,
                      col_walk=col_walk, dense=dense)
            want = ref_mod.jitconn_matvec(inp, **kw)
            got = oracle_mod.jitconn_matvec(inp, per_stream_seed=False, **kw)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_closed_form_full_connectivity(oracle_mod):
  # conn_prob >= 1: log_p = log(1e-40); every skip is 1, so a stream connects exactly
  # indices 1 .. n-1 (index 0 is never reached).
  lp = oracle_mod.log_p_of(1.0)
  idx, cnt = oracle_mod.jitconn_stream_indices(5, lp, 50)
  assert cnt == 49 and np.array_equal(idx, np.arange(1, 50))
  v = np.arange(1, 31, dtype=np.float64)
  for per_stream in (False, True):
    out = oracle_mod.jitconn_matvec(v, log_p=lp, seed=3, n_row=7, n_col=30, dense=True, per_stream_seed=per_stream)
    assert np.array_equal(out, np.full(7, v[1:].sum()))
    out = oracle_mod.jitconn_matvec(v, log_p=lp, seed=3, n_row=7, n_col=30, dense=True, col_walk=True,
                                    per_stream_seed=per_stream)
    want = np.full(7, v.sum())
    want[0] = 0
    assert np.array_equal(out, want)


def test_index_sets_follow_the_geometric_law(oracle_mod):
  # gaps between successive indices of a stream are Geometric(p) on {1,2,...}: P(gap=k) = p(1-p)^(k-1)
  p = 0.05
  lp = oracle_mod.log_p_of(p)
  gaps = []
  for s in range(200):
    idx, cnt = oracle_mod.jitconn_stream_indices(1000 + s, lp, 20000)
    assert cnt == idx.shape[0] and np.all(np.diff(idx.astype(np.int64)) > 0) and idx[0] >= 1
    gaps.append(np.diff(np.concatenate([[0], idx.astype(np.int64)])))
  gaps = np.concatenate(gaps)
  assert abs(gaps.mean() - 1 / p) < 0.2          # sd of the mean ~ 0.044
  ks = np.arange(1, 60)
  emp = np.array([(gaps == k).mean() for k in ks])
  assert np.abs(emp - p * (1 - p) ** (ks - 1)).max() < 2e-3


def test_sequential_and_per_stream_agree_on_the_first_stream(oracle_mod):
  ev = np.random.default_rng(0).random(500) < 0.5
  a = oracle_mod.jitconn_matvec(ev, log_p=oracle_mod.log_p_of(0.1), seed=42, n_row=9, n_col=500, per_stream_seed=False)
  b = oracle_mod.jitconn_matvec(ev, log_p=oracle_mod.log_p_of(0.1), seed=42, n_row=9, n_col=500, per_stream_seed=True)
  assert a[0] == b[0]


@pytest.mark.parametrize("shape", JIT_SHAPES)
@pytest.mark.parametrize("per_stream", [False, True])
def test_shape_swap_identity(oracle_mod, shape, per_stream):
  # brainpylib/_src/jitconn_ops/tests/test_event_matvec.py:80-87:
  # op(shape=(a,b), transpose=t) == op(shape=(b,a), transpose=not t); transpose only swaps
  # (n_row, n_col) before the kernel, so both calls see the same kernel arguments.
  ev = np.random.default_rng(1).random(shape[1]) < 0.1
  lp = oracle_mod.log_p_of(0.1)
  r1 = oracle_mod.jitconn_matvec(ev, log_p=lp, seed=1234, n_row=shape[0], n_col=shape[1], per_stream_seed=per_stream)
  n_row, n_col = (shape[1], shape[0])[::-1]  # shape=(b,a), transpose=True -> (n_row, n_col) = (a, b)
  r2 = oracle_mod.jitconn_matvec(ev, log_p=lp, seed=1234, n_row=n_row, n_col=n_col, per_stream_seed=per_stream)
  assert np.array_equal(r1, r2)


@pytest.mark.parametrize("w_kind,a,b", [("homo", 0, 0), ("uniform", -1.0, 1.0), ("normal", 0.0, 1.0)])
@pytest.mark.parametrize("per_stream", [False, True])
def test_row_walk_and_column_walk_are_adjoint(oracle_mod, w_kind, a, b, per_stream):
  # The reference's transpose rule flips both `transpose` and `outdim_parallel`
  # (brainpylib/_src/jitconn_ops/event_matvec.py:263-273): the row walk of M and the column walk
  # of the swapped shape consume the generator in the same order, so they are M and M^T:
  # <y, M x> == <M^T y, x>.
  n_out, n_in = 60, 90
  rng = np.random.default_rng(5)
  x = rng.integers(-3, 4, n_in).astype(np.float64)
  y = rng.integers(-3, 4, n_out).astype(np.float64)
  lp = oracle_mod.log_p_of(0.2)
  kw = dict(w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=11, dense=True, per_stream_seed=per_stream)
  Mx = oracle_mod.jitconn_matvec(x, n_row=n_out, n_col=n_in, col_walk=False, **kw)
  MTy = oracle_mod.jitconn_matvec(y, n_row=n_in, n_col=n_out, col_walk=True, **kw)
  assert abs(y @ Mx - MTy @ x) <= 1e-9 * max(1.0, abs(y @ Mx))


def test_dense_matvec_equals_explicit_matrix(oracle_mod):
  # build M row by row from the stream's (index, weight) lists and compare with numpy matmul
  n_out, n_in, seed = 40, 300, 21
  lp = oracle_mod.log_p_of(0.1)
  x = np.random.default_rng(2).standard_normal(n_in)
  for wk, a, b in (("homo", 0.0, 0.0), ("uniform", 0.5, 1.5), ("normal", 1.0, 0.1)):
    M = np.zeros((n_out, n_in))
    for r in range(n_out):
      idx, w = oracle_mod.jitconn_stream_weights(seed + r, wk, a, b, lp, n_in, dtype=np.float64)
      M[r, idx] = w
    out = oracle_mod.jitconn_matvec(x, w_kind=wk, w_a=a, w_b=b, log_p=lp, seed=seed, n_row=n_out, n_col=n_in,
                                    dense=True, per_stream_seed=True)
    assert_close(out, M @ x, rtol=1e-12, atol=1e-12)
    if wk == "uniform":
      assert M[M != 0].min() >= 0.5 and M[M != 0].max() < 1.5
    # event version == dense version on 0/1 input
    ev = x > 0.3
    out_e = oracle_mod.jitconn_matvec(ev, w_kind=wk, w_a=a, w_b=b, log_p=lp, seed=seed, n_row=n_out, n_col=n_in,
                                      per_stream_seed=True, out_dtype=np.float64)
    assert_close(out_e, M @ ev.astype(np.float64), rtol=1e-12, atol=1e-12)


def test_matmat_is_vmapped_transposed_matvec(oracle_mod):
  # brainpylib/_src/jitconn_ops/tests/matmat_testcase.py:133-138
  m, k, n = 5, 70, 40
  X = np.random.default_rng(3).standard_normal((m, k)).astype(np.float32)
  lp = oracle_mod.log_p_of(0.2)
  Y = oracle_mod.jitconn_matmat(X, w_kind="normal", w_a=0.0, w_b=0.01, log_p=lp, seed=7, n=n)
  for i in range(m):
    # matvec(X[i], shape=(k, n), transpose=True): n_row = n outputs, n_col = k inputs
    yi = oracle_mod.jitconn_matvec(X[i], w_kind="normal", w_a=0.0, w_b=0.01, log_p=lp, seed=7, n_row=n, n_col=k,
                                   dense=True, per_stream_seed=True)
    assert np.array_equal(Y[i], yi)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("w_kind,a,b", [("homo", 0.0, 0.0), ("uniform", -0.5, 1.5), ("normal", 0.0, 0.01)])
def test_matmat_one_pass_equals_the_definition_and_its_abs_sums(oracle_mod, dtype, w_kind, a, b):
  # the one-pass form (each stream generated once, applied to all rows of X) against the
  # definition taken literally, bit for bit; its abs sums against |M| @ |X| of the explicit matrix
  m, k, n, seed = 7, 90, 50, 13
  X = np.random.default_rng(4).standard_normal((m, k)).astype(dtype)
  lp = oracle_mod.log_p_of(0.15)
  kw = dict(w_kind=w_kind, w_a=a, w_b=b, log_p=lp, seed=seed, n=n)
  oracle_mod.set_threads(3)
  Y, mag = oracle_mod.jitconn_matmat(X, return_abs=True, **kw)
  oracle_mod.set_threads(1)
  assert np.array_equal(Y, oracle_mod.jitconn_matmat(X, by_rows=True, **kw))
  assert np.array_equal(Y, oracle_mod.jitconn_matmat(X, **kw))
  M = np.zeros((k, n))
  for j in range(n):
    idx, w = oracle_mod.jitconn_stream_weights(seed + j, w_kind, a, b, lp, k, dtype=dtype)
    M[idx, j] = w
  assert_close(mag, np.abs(X).astype(np.float64) @ np.abs(M), rtol=1e-6, atol=1e-12)
  assert_close(Y, X.astype(np.float64) @ M, rtol=1e-4, atol=1e-4 * float(mag.max()))


@pytest.mark.parametrize("col_walk", [False, True])
@pytest.mark.parametrize("kind", ["bool", "dense"])
def test_matvec_abs_sums(oracle_mod, col_walk, kind):
  # abs_sum[o] = sum |addend| == the same walk over |weights| and |input|; the result is unchanged
  n_out, n_in, seed = 35, 80, 3
  lp = oracle_mod.log_p_of(0.2)
  rng = np.random.default_rng(9)
  inp = (rng.random(n_in) < 0.4) if kind == "bool" else rng.standard_normal(n_in)
  kw = dict(w_kind="normal", w_a=0.0, w_b=1.0, log_p=lp, seed=seed, n_row=n_out, n_col=n_in, col_walk=col_walk,
            dense=(None if kind == "bool" else True), out_dtype=np.float64)
  out, mag = oracle_mod.jitconn_matvec(inp, return_abs=True, **kw)
  assert np.array_equal(out, oracle_mod.jitconn_matvec(inp, **kw))
  M = np.zeros((n_out, n_in))
  for s in range(n_in if col_walk else n_out):
    idx, w = oracle_mod.jitconn_stream_weights(seed + s, "normal", 0.0, 1.0, lp, n_out if col_walk else n_in,
                                               dtype=np.float64)
    if col_walk:
      M[idx, s] = w
    else:
      M[s, idx] = w
  assert_close(mag, np.abs(M) @ np.abs(inp.astype(np.float64)), rtol=1e-12, atol=1e-12)
