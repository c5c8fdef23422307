"""How close the GPU's sums are to the reference's, beyond the stated tolerance, through the C ABI.

* Homogeneous weights: the reference adds the weight once per delivered synapse (in place in the
  output's precision when it scatters, event_csr_matvec.py:313-331; into a float64 accumulator when
  it gathers, :334-357).  All addends being equal, the result depends on the synapse count alone,
  and the kernels, which count in integers, return the reference's bits: checked here with a weight
  that is not representable (0.6) and thousands of synapses per output, where `count * weight`
  rounded once is off by more than the tolerance.
* Heterogeneous weights and dense vectors: the addends arrive in another order than in the
  reference's sequential loop.  Against the exact sum (float64 sum of the products as the operators
  round them) the GPU result must not be farther off than the reference's own loop is, up to a
  stated number of units in the last place.
* Non-finite weights against zero inputs: 0 * inf is NaN in the reference's transposed dense
  product (cusparse_matvec.py:204-211), on every kernel path.
"""
import numpy as np
import pytest
import torch

import brainpylib_amd as bpl
import benchdata as synth
from util import assert_close_reordered, exact_scatter

pytestmark = pytest.mark.gpu


def _columns_in_a_corner(n_row, per_row, width, n_col, seed):
  """Rows of `per_row` distinct sorted columns drawn from the first `width` columns of n_col."""
  rng = np.random.default_rng(seed)
  keys = rng.random((n_row, width))
  cols = np.sort(np.argpartition(keys, per_row - 1, axis=1)[:, :per_row], axis=1).astype(np.int32)
  indptr = (np.arange(n_row + 1, dtype=np.int64) * per_row).astype(np.int32)
  return cols.reshape(-1), indptr


# (name, shape, structure, fraction of active rows): one case per kernel path of the event scatter
def _homo_scatter_cases():
  yield "one launch", (4000, 300), synth.bernoulli_csr(4000, 300, 0.5, seed=1), 1.0
  yield "windows, partial outputs", (20_000, 1000), synth.bernoulli_csr(20_000, 1000, 0.1, seed=2), 1.0
  yield "windows, active-row list", (40_000, 1000), synth.bernoulli_csr(40_000, 1000, 0.05, seed=3), 1.0
  yield "sorted by output window", (60_000, 12_000), synth.bernoulli_csr(60_000, 12_000, 1 / 30, seed=4), 1.0
  # 120,000 active nonzeros: below the threshold of the sort, rows are added to the output directly
  yield "little activity", (3000, 10_000), _columns_in_a_corner(3000, 40, 50, 10_000, seed=5), 1.0
  # 3e6 pairs into one window of 256 columns, whose runs hold about half of them: the rest is counted in the output
  yield "run overflow", (30_000, 20_000), _columns_in_a_corner(30_000, 100, 256, 20_000, seed=6), 1.0
  yield "sorted, part of the rows", (60_000, 12_000), synth.bernoulli_csr(60_000, 12_000, 1 / 30, seed=4), 0.3


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_homogeneous_scatter_is_the_reference_loop_bit_for_bit(cuda, oracle_mod, dtype):
  rng = np.random.default_rng(3)
  worst_gap = 0.0
  for name, shape, (indices, indptr), rate in _homo_scatter_cases():
    print("case", name, shape, dtype.__name__, flush=True)
    ev = rng.random(shape[0]) < rate
    for w in (0.6, -0.3, 1.0 + 2.0 ** -12):
      data = np.array([w], dtype=dtype)
      want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
      for _ in range(2):  # twice: counters and counts of the first call are gone
        got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
        assert np.array_equal(got, want), (name, w, int((got != want).sum()), got[got != want][:4], want[got != want][:4])
      # what one rounding of count * weight would have given: the gap this build used to have
      counts = np.bincount(indices[np.repeat(ev, np.diff(indptr.astype(np.int64)))], minlength=shape[1])
      assert counts.max() >= (2000 if rate == 1.0 else 500)
      once = (counts.astype(np.float64) * float(data[0])).astype(dtype)
      gap = np.abs(once.astype(np.float64) - want.astype(np.float64)) / np.maximum(np.abs(want.astype(np.float64)), 1e-30)
      if dtype == np.float32:
        worst_gap = max(worst_gap, float(gap.max()))
    # float events: any nonzero value is an event
    evf = (ev * rng.uniform(0.5, 2.0, shape[0])).astype(dtype)
    data = np.array([0.6], dtype=dtype)
    want = oracle_mod.event_csr_matvec(data, indices, indptr, evf, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(data, indices, indptr, evf, shape=shape, transpose=True).cpu().numpy()
    assert np.array_equal(got, want), name
  if dtype == np.float32:
    print("largest relative gap between count * weight rounded once and the reference's loop: %.3e" % worst_gap)
    assert worst_gap > 1e-5  # the inputs do reach the regime where the difference is outside the tolerance


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_homogeneous_gather_is_the_reference_loop_bit_for_bit(cuda, oracle_mod, dtype):
  # transpose=False: a float64 accumulator per row, rounded once (event_csr_matvec.py:334-357)
  rng = np.random.default_rng(4)
  for shape, p in (((3000, 6000), 0.5), ((300, 40_000), 0.4), ((20_000, 2000), 0.02)):
    indices, indptr = synth.bernoulli_csr(shape[0], shape[1], p, seed=shape[0])
    ev = rng.random(shape[1]) < 0.8
    for w in (0.6, -0.3):
      data = np.array([w], dtype=dtype)
      want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
      got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape).cpu().numpy()
      assert np.array_equal(got, want), (shape, w)


def _ulp(x, dtype):
  return np.spacing(np.abs(x).astype(dtype)).astype(np.float64)


def _closer_than_the_loop(got, want, exact, dtype, ulps, what, mag=None, k_eps=None):
  """Elementwise: |gpu - exact| <= |reference loop - exact| + `ulps` units in the last place of the result.
  With `mag` (sum of |addends| per element) instead: the result is the sum of up to 2 k_eps partial sums,
  each exact before it is rounded, so elementwise |gpu - exact| <= k_eps * eps * mag (the hard bound), and on
  the whole the GPU is not farther from the exact sums than the loop: root mean square error within 1.1 x
  and maximum error within 1.5 x the loop's (a margin: the order of these additions changes from run to run)."""
  e_gpu = np.abs(got.astype(np.float64) - exact)
  e_ref = np.abs(want.astype(np.float64) - exact)
  slack = ulps * _ulp(np.maximum(np.abs(exact), np.finfo(dtype).tiny), dtype)
  worse = e_gpu > e_ref + slack
  rms_gpu, rms_ref = np.sqrt((e_gpu ** 2).mean()), np.sqrt((e_ref ** 2).mean())
  print("%-46s gpu max err %.3e (rms %.3e), loop max err %.3e (rms %.3e), gpu worse than loop + %g ulp: %d of %d" % (
    what, e_gpu.max(), rms_gpu, e_ref.max(), rms_ref, ulps, int(worse.sum()), worse.size), flush=True)
  if mag is None:
    assert not worse.any(), (what, int(worse.sum()))
  else:
    # the hard bound is the elementwise one.  The comparison with the loop is a statistical statement about
    # additions whose order changes from run to run: asserted with a margin (the GPU's rms error has been
    # 0.4 to 0.7 of the loop's in every run so far)
    assert np.all(e_gpu <= k_eps * np.finfo(dtype).eps * mag + np.finfo(dtype).tiny), what
    assert rms_gpu <= 1.1 * rms_ref and e_gpu.max() <= 1.5 * e_ref.max(), what
  return e_gpu, e_ref


def test_event_scatter_sum_is_at_least_as_accurate_as_the_loop(cuda, oracle_mod):
  # the 1e8-nnz configuration at 1/16 scale (25,000 x 25,000, 6e6 nnz, 5 % events): sorted scatter,
  # float64 windows in LDS added to the output by at most a few workgroups per window
  c = synth.config_event_csr_large(n=25_000)
  ev = c["events"]
  exact = exact_scatter(c["indices"], c["indptr"], ev.astype(np.float32), c["data"], c["shape"][1])
  want = oracle_mod.event_csr_matvec(c["data"], c["indices"], c["indptr"], ev, shape=c["shape"], transpose=True)
  got = bpl.event_csr_matvec(c["data"], c["indices"], c["indptr"], ev, shape=c["shape"], transpose=True).cpu().numpy()
  _closer_than_the_loop(got, want, exact, np.float32, 1.0, "event scatter, sorted (25,000 columns)")
  mag = exact_scatter(c["indices"], c["indptr"], ev.astype(np.float32), np.abs(c["data"]), c["shape"][1])
  assert_close_reordered(got, want, mag, what="event scatter 1/16 scale")
  # narrow output: float32 windows in LDS, lanes add in the order they arrive: not more accurate than
  # the loop element by element, but as accurate on the whole, and far inside the summation bound
  indices, indptr = synth.bernoulli_csr(30_000, 6000, 0.02, seed=9)
  data = np.random.default_rng(9).standard_normal(indices.shape[0]).astype(np.float32)
  ev = np.random.default_rng(10).random(30_000) < 0.2
  shape = (30_000, 6000)
  exact = exact_scatter(indices, indptr, ev.astype(np.float32), data, shape[1])
  mag = exact_scatter(indices, indptr, ev.astype(np.float32), np.abs(data), shape[1])
  want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
  got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
  e_gpu = np.abs(got - exact)
  e_ref = np.abs(want - exact)
  print("event scatter, float32 windows: gpu rms err %.3e, loop rms err %.3e" % (
    np.sqrt((e_gpu ** 2).mean()), np.sqrt((e_ref ** 2).mean())), flush=True)
  assert np.sqrt((e_gpu ** 2).mean()) <= 1.5 * np.sqrt((e_ref ** 2).mean())
  counts = np.bincount(indices[np.repeat(ev, np.diff(indptr.astype(np.int64)))], minlength=shape[1])
  assert np.all(e_gpu <= counts * np.finfo(np.float32).eps * mag + 1e-30)  # (n - 1) eps sum|x|, Higham 4.4
  assert_close_reordered(got, want, mag, what="event scatter float32 windows")


def test_transposed_csr_matvec_sum_is_at_least_as_accurate_as_the_loop(cuda, oracle_mod):
  # wide output (bins of products, float64 windows) and a narrow one (float64 windows of the window kernel)
  for n_row, n_col, lam, what in ((120_000, 300_000, 40, "bins"), (50_000, 20_000, 30, "windows")):
    indices, indptr = synth.poisson_csr(n_row, n_col, lam, seed=n_row)
    rng = np.random.default_rng(n_col)
    data = rng.random(indices.shape[0], dtype=np.float32)
    v = rng.standard_normal(n_row, dtype=np.float32)
    shape = (n_row, n_col)
    exact = exact_scatter(indices, indptr, v, data, n_col)
    want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=True)
    got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
    # (up to 13 workgroups add their share of a window's bins, up to 64 row groups their partial windows:
    # each share is summed in float64 and rounded once, the shares are added in float32)
    mag = exact_scatter(indices, indptr, np.abs(v), data, n_col)
    _closer_than_the_loop(got, want, exact, np.float32, 2.0, "csr_matvec transposed, " + what, mag=mag, k_eps=32.0)
    assert_close_reordered(got, want, mag, what="csr_matvec transposed " + what)


def test_jitconn_column_walk_sum_is_at_least_as_accurate_as_the_loop(cuda, oracle_mod):
  # dense vector, uniform weights (the same bits on both sides), column walk through the bins:
  # out[row] += w * v in the reference (lib/cpu_jitconn_matvec_atomic.cpp)
  n_out, n_in, seed, p = 40_000, 3000, 5, 0.05
  lp = oracle_mod.log_p_of(p)
  v = np.random.default_rng(1).standard_normal(n_in).astype(np.float32)
  lo, hi = -1.0, 1.0
  exact, mag = np.zeros(n_out), np.zeros(n_out)
  for col in range(n_in):
    idx, w = oracle_mod.jitconn_stream_weights(seed + col, "uniform", lo, hi, lp, n_out, dtype=np.float32)
    np.add.at(exact, idx, (w * v[col]).astype(np.float32).astype(np.float64))
    np.add.at(mag, idx, np.abs((w * v[col]).astype(np.float32).astype(np.float64)))
  want = oracle_mod.jitconn_matvec(v, w_kind="uniform", w_a=lo, w_b=hi, log_p=lp, seed=seed, n_row=n_out,
                                   n_col=n_in, col_walk=True, dense=True, per_stream_seed=True)
  got = bpl.matvec_prob_conn_uniform_weight(v, w_low=lo, w_high=hi, conn_prob=p, shape=(n_out, n_in), seed=seed,
                                            outdim_parallel=False).cpu().numpy()
  # (several workgroups add their share of a window's bins: float64 sums rounded once, added in float32)
  _closer_than_the_loop(got, want, exact, np.float32, 2.0, "jitconn column walk, uniform weights", mag=mag, k_eps=32.0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_zero_input_times_non_finite_weight_is_nan_on_every_path(cuda, oracle_mod, dtype):
  # out[col] += vector[row] * values[j] has no test of the vector (cusparse_matvec.py:204-211):
  # 0 * inf and 0 * NaN reach the output.  Paths: direct atomics (tiny), float64 windows, bins.
  rng = np.random.default_rng(12)
  for n_row, n_col, lam in ((50, 70, 5), (3000, 5000, 20), (40_000, 60_000, 30), (40_000, 400_000, 40)):
    indices, indptr = synth.poisson_csr(n_row, n_col, lam, seed=n_row + 1)
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    v = rng.standard_normal(n_row).astype(dtype)
    rows = rng.choice(n_row, size=min(n_row // 4, 50), replace=False)
    v[rows] = 0
    first = indptr[rows[:2]]  # the first weight of two of the silent rows
    data[first[0]] = np.inf
    data[first[1]] = np.nan
    shape = (n_row, n_col)
    want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=True)
    got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
    assert np.isnan(want[indices[first]]).all()
    assert np.array_equal(np.isnan(got), np.isnan(want)), (shape, int(np.isnan(got).sum()), int(np.isnan(want).sum()))
    ok = ~np.isnan(want)
    mag = exact_scatter(indices, indptr, np.abs(v), np.abs(np.nan_to_num(data, nan=0.0, posinf=0.0)), n_col)
    assert_close_reordered(got[ok], want[ok], mag[ok], dtype, what="finite outputs beside the NaNs")
    # the untransposed product has no test either
    x = rng.standard_normal(n_col).astype(dtype)
    x[indices[first]] = 0
    want = oracle_mod.csr_matvec(data, indices, indptr, x, shape=shape)
    got = bpl.csr_matvec(data, indices, indptr, x, shape=shape).cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(want[rows[:2]]).all()
