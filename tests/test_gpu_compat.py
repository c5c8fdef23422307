"""GPU parity of the older operator family (csr_event_sum, coo_event_sum, coo_atomic_sum)
against the golden vectors of the reference's CPU kernels and against the CPU oracle."""
import os

import numpy as np
import pytest

import brainpylib_amd as bpl
import benchdata as synth
from util import assert_close_reordered

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden", "compat_cpu_reference.npz")


def test_coo_atomic_sum_golden(cuda):
  z = np.load(GOLD)
  n = sum(1 for k in z.files if k.startswith("as_out_"))
  for i in range(n):
    values, pre, post, num = z["as_values_%d" % i], z["as_pre_%d" % i], z["as_post_%d" % i], int(z["as_num_%d" % i])
    homo = values.shape[0] == 1
    print("case", i, values.dtype, pre.dtype, homo, flush=True)
    got = bpl.coo_atomic_sum(values, post, num, None if homo else pre).cpu().numpy()
    want = z["as_out_%d" % i]
    assert got.dtype == want.dtype
    mag = np.bincount(post, weights=np.abs(values[0] if homo else values[pre]) * np.ones(post.shape[0]), minlength=num)
    assert_close_reordered(got, want, mag, values.dtype.type, what="coo_atomic_sum %d" % i)


def test_csr_event_sum_wide_golden(cuda):
  z = np.load(GOLD)
  n = sum(1 for k in z.files if k.startswith("es_out_"))
  for i in range(n):
    shape = tuple(int(x) for x in z["es_shape_%d" % i])
    data, events = z["es_data_%d" % i], z["es_events_%d" % i]
    indices, indptr = z["es_indices_%d" % i], z["es_indptr_%d" % i]
    assert indices.dtype == np.int64
    print("case", i, shape, data.dtype, flush=True)
    got = bpl.csr_event_sum(events, (indices, indptr), shape[1], data).cpu().numpy()
    want = z["es_out_%d" % i]
    rows = np.repeat(np.arange(shape[0]), np.diff(indptr))
    w = np.abs(data[0] if data.shape[0] == 1 else data) * events[rows]
    mag = np.bincount(indices, weights=w, minlength=shape[1])
    assert_close_reordered(got, want, mag, data.dtype.type, what="csr_event_sum i64 %d" % i)
    # 32-bit indices go through event_csr_matvec
    got32 = bpl.csr_event_sum(events, (indices.astype(np.int32), indptr.astype(np.int32)), shape[1], data).cpu().numpy()
    assert_close_reordered(got32, want, mag, data.dtype.type, what="csr_event_sum i32 %d" % i)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_csr_event_sum_64_bit_ids_through_the_sorted_scatter(cuda, oracle_mod, dtype):
  # 64-bit index arrays and a result of more than 8,192 elements: the sorted event scatter reads the 64-bit
  # columns and offsets as they are.  Against the oracle (lib/cpu_event_sum.cc's loop): one weight bit for bit,
  # weights per connection within the reordered-sum bound; activity on both sides of the direct-atomics
  # threshold, empty rows, a result narrower and wider than the matrix has rows.
  for (pre, post, mean, rate) in ((30_000, 20_000, 40, 0.1), (30_000, 20_000, 40, 0.001), (5_000, 300_000, 300, 0.3),
                                  (200_000, 9_000, 10, 0.5)):
    rng = np.random.default_rng(pre + post)
    counts = np.minimum(rng.poisson(mean, size=pre), post)
    indices, indptr = synth.counted_csr(counts, post, seed=pre)
    events = rng.random(pre) < rate
    wide = (indices.astype(np.int64), indptr.astype(np.int64))
    print("case", pre, post, mean, rate, dtype.__name__, flush=True)
    for values in (np.array([0.6], dtype=dtype), rng.standard_normal(indices.shape[0]).astype(dtype)):
      want = oracle_mod.csr_event_sum(events, (indices, indptr), post, values)
      got = bpl.csr_event_sum(events, wide, post, values).cpu().numpy()
      if values.shape[0] == 1:
        assert np.array_equal(got, want)
      else:
        mag = oracle_mod.csr_event_sum(events, (indices, indptr), post, np.abs(values))
        assert_close_reordered(got, want, mag, dtype, what="csr_event_sum i64, sorted scatter")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("itype", [np.int32, np.uint32, np.int64])
def test_coo_event_sum_vs_oracle(cuda, oracle_mod, dtype, itype):
  rng = np.random.default_rng(9)
  for pre_n, post_n, conn in [(200, 200, 20000), (30, 500, 3000), (500, 3, 4000), (100000, 50000, 2_000_000)]:
    pre = rng.integers(0, pre_n, conn).astype(itype)
    post = rng.integers(0, post_n, conn).astype(itype)
    events = rng.random(pre_n) < 0.3
    print("case", pre_n, post_n, conn, flush=True)
    for values in (rng.standard_normal(conn).astype(dtype), dtype(0.25), np.ones(1, dtype=dtype)):
      want = oracle_mod.coo_event_sum(events, pre, post, post_n, values)
      got = bpl.coo_event_sum(events, pre, post, post_n, values).cpu().numpy()
      mag = oracle_mod.coo_event_sum(events, pre, post, post_n, np.abs(values))
      assert_close_reordered(got, want, mag, dtype, what="coo_event_sum")
      if np.ndim(values) and values.shape[0] == 1:
        assert np.array_equal(got, want)  # counts


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("itype", [np.int32, np.int64])
def test_coo_sums_through_windows_of_the_result(cuda, oracle_mod, dtype, itype):
  """Long connection lists are added in LDS windows of the result (one window, two slices, a connection count
  that is no multiple of a lane's four; with one weight up to 32 slices) or, with weights and a wider result,
  through bins (a fiftieth of the connections crowd into one window and overflow its bins); short lists and a
  single weight into a very wide result take the atomics."""
  rng = np.random.default_rng(21)
  for pre_n, post_n, conn in [(3000, 5000, 600_001), (70000, 16384, 400_003), (500, 20000, 300_002),
                              (1000, 32768, 262_147), (1000, 32769, 262_147), (40, 1, 140_000),
                              (2000, 100_000, 1_200_001), (50_000, 3_000_000, 1_100_003), (300, 40_000, 1_048_576)]:
    pre = rng.integers(0, pre_n, conn).astype(itype)
    post = rng.integers(0, post_n, conn).astype(itype)
    # a crowded end of the result (few enough additions per element for the oracle's float32 loop to stay within
    # the bound used below, enough for that window's bins to overflow)
    post[: conn // 50] = post_n - 1 - post[: conn // 50] % min(post_n, 7)
    events = rng.random(pre_n) < 0.3
    print("case", pre_n, post_n, conn, flush=True)
    for homo in (False, True):
      # coo_atomic_sum: a value per source
      values = np.full(1, 0.1, dtype) if homo else rng.standard_normal(pre_n).astype(dtype)
      got = bpl.coo_atomic_sum(values, post, post_n, None if homo else pre).cpu().numpy()
      want = oracle_mod.coo_atomic_sum(values, post, post_n, None if homo else pre)
      mag = np.bincount(post, weights=np.abs(values[0] if homo else values[pre]) * np.ones(conn), minlength=post_n)
      if homo:
        assert np.array_equal(got, want), "coo_atomic_sum of one weight: sums of that many additions"
      elif post_n == 1:
        # 140,000 additions to one element: the oracle's own float32 loop drifts by more than the bound below
        # allows for, so the sum is compared with the one taken in float64
        exact = np.array([values[pre].astype(np.float64).sum()])
        assert_close_reordered(got, exact, mag, dtype, what="coo_atomic_sum")
      else:
        assert_close_reordered(got, want, mag, dtype, what="coo_atomic_sum")
      # coo_event_sum: a value per connection
      values = np.full(1, 0.1, dtype) if homo else rng.standard_normal(conn).astype(dtype)
      got = bpl.coo_event_sum(events, pre, post, post_n, values).cpu().numpy()
      want = oracle_mod.coo_event_sum(events, pre, post, post_n, values)
      mag = oracle_mod.coo_event_sum(events, pre, post, post_n, np.abs(values))
      if homo:
        assert np.array_equal(got, want), "coo_event_sum of one weight: sums of that many additions"
      elif post_n == 1:
        exact = np.array([(values.astype(np.float64) * events[pre]).sum()])
        assert_close_reordered(got, exact, mag, dtype, what="coo_event_sum")
      else:
        assert_close_reordered(got, want, mag, dtype, what="coo_event_sum")


def test_coo_sums_of_fifty_million_connections_exact_on_integer_data(cuda):
  """At a size the CPU loop is not run at: small integers as weights add up exactly in any order, so the result
  must equal numpy's float64 bincount bit for bit, through the LDS windows (10,000 targets), the slices of a
  single weight and the bins (100,000 targets)."""
  rng = np.random.default_rng(33)
  conn, pre_n = 50_000_000, 100_000
  pre = rng.integers(0, pre_n, conn, dtype=np.int32)
  values = rng.integers(-3, 4, pre_n).astype(np.float32)
  events = rng.random(pre_n) < 0.2
  per_conn = values[pre]
  for post_n in (10_000, 100_000):
    post = rng.integers(0, post_n, conn, dtype=np.int32)
    print("targets", post_n, flush=True)
    got = bpl.coo_atomic_sum(values, post, post_n, pre).cpu().numpy()
    assert np.array_equal(got, np.bincount(post, weights=per_conn, minlength=post_n).astype(np.float32))
    got = bpl.coo_atomic_sum(np.float32(0.5), post, post_n).cpu().numpy()
    assert np.array_equal(got, (0.5 * np.bincount(post, minlength=post_n)).astype(np.float32))
    got = bpl.coo_event_sum(events, pre, post, post_n, per_conn).cpu().numpy()
    assert np.array_equal(got, np.bincount(post, weights=per_conn * events[pre], minlength=post_n).astype(np.float32))


def test_known_answers_and_argument_checks(cuda):
  # brainpylib/_src/compat/tests/test_atomic_sum_cpu.py:16-34
  size = 200
  ids = np.arange(size, dtype=np.uint32)
  sps = np.random.default_rng(12345).integers(0, 2, size).astype(np.float32)
  assert np.array_equal(bpl.coo_atomic_sum(sps, ids, size, ids).cpu().numpy(), sps)
  assert np.all(bpl.coo_atomic_sum(2., ids, size).cpu().numpy() == 2.)
  pre, post = np.divmod(np.arange(100, dtype=np.int32), 10)
  assert np.all(bpl.coo_atomic_sum(2., post, 10).cpu().numpy() == 20.)
  assert np.all(bpl.coo_atomic_sum(np.full(10, 2., np.float32), post, 10, pre).cpu().numpy() == 20.)
  # empty connection list: a zero vector
  e = np.zeros(0, np.int32)
  assert not bpl.coo_event_sum(np.ones(4, bool), e, e, 6, 1.0).cpu().numpy().any()
  with pytest.raises(ValueError):
    bpl.coo_event_sum(np.ones(4, np.float32), pre, post, 10, 1.0)  # events must be bool
  with pytest.raises(ValueError):
    bpl.coo_event_sum(np.ones(10, bool), pre, post[:5], 10, 1.0)
  with pytest.raises(ValueError):
    bpl.coo_atomic_sum(np.ones(5, np.float32), post, 10, pre)  # values shorter than max(pre_ids)
  with pytest.raises(ValueError):
    bpl.csr_event_sum(np.ones(4, bool), (post, np.zeros(4, np.int32)), 10, 1.0)  # len(indptr) != len(events) + 1


PROD_GOLD = os.path.join(os.path.dirname(__file__), "golden", "compat_prod_cpu_reference.npz")


def _assert_close_product(got, want, count, dtype, what):
  """A product of `count` factors rounds count - 1 times in either order (half an ulp each), so two
  orders differ by at most (count - 1) eps relative; equal factors give the same bits."""
  got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
  bound = np.abs(want) * np.finfo(dtype).eps * (count + 1)
  bad = np.abs(got - want) > bound
  assert not bad.any(), "%s: %d of %d off, worst %g" % (what, bad.sum(), bad.size, np.abs(got - want).max())


def test_coo_atomic_prod_golden(cuda):
  # lib/cpu_atomic_prod.cc, compiled
  z = np.load(PROD_GOLD)
  n = sum(1 for k in z.files if k.startswith("ap_out_"))
  assert n == 32
  for i in range(n):
    values, pre, post, num = z["ap_values_%d" % i], z["ap_pre_%d" % i], z["ap_post_%d" % i], int(z["ap_num_%d" % i])
    homo = values.shape[0] == 1
    got = bpl.coo_atomic_prod(values, post, num, None if homo else pre).cpu().numpy()
    want = z["ap_out_%d" % i]
    assert got.dtype == want.dtype
    if homo:
      assert np.array_equal(got, want), "case %d" % i  # equal factors: the order cannot matter
    else:
      _assert_close_product(got, want, np.bincount(post, minlength=num), values.dtype, "coo_atomic_prod %d" % i)


def test_csr_event_prod_golden(cuda):
  # lib/cpu_event_prod.cc, compiled
  z = np.load(PROD_GOLD)
  n = sum(1 for k in z.files if k.startswith("ep_out_"))
  assert n == 24
  for i in range(n):
    data, events, indices, indptr = (z["ep_%s_%d" % (k, i)] for k in ("data", "events", "indices", "indptr"))
    post_n = int(z["ep_shape_%d" % i][1])
    got = bpl.csr_event_prod(events, (indices, indptr), post_n, data).cpu().numpy()
    want = z["ep_out_%d" % i]
    assert got.dtype == want.dtype
    if data.shape[0] == 1:
      assert np.array_equal(got, want), "case %d" % i
    else:
      count = np.bincount(indices[np.repeat(events, np.diff(indptr))], minlength=post_n)
      _assert_close_product(got, want, count, data.dtype, "csr_event_prod %d" % i)


def test_prod_vs_oracle_larger(cuda, oracle_mod):
  rng = np.random.default_rng(77)
  for dtype in (np.float32, np.float64):
    for wide in (False, True):
      it = np.int64 if wide else np.int32
      pre_n, post_n, conn = 3000, 5000, 200000
      pre = rng.integers(0, pre_n, conn).astype(it)
      post = rng.integers(0, post_n, conn).astype(it)
      post[:2000] = 17  # one heavily shared target
      values = rng.uniform(0.99, 1.01, pre_n).astype(dtype)
      values[rng.integers(0, pre_n, 40)] *= -1
      got = bpl.coo_atomic_prod(values, post, post_n, pre).cpu().numpy()
      want = oracle_mod.coo_atomic_prod(values, post, post_n, pre)
      _assert_close_product(got, want, np.bincount(post, minlength=post_n), dtype, "coo_atomic_prod")
      assert np.array_equal(np.signbit(got), np.signbit(want))
      w = np.array([1.0009765625], dtype)  # 2,000 equal factors on one target: bit for bit
      got = bpl.coo_atomic_prod(w, post, post_n).cpu().numpy()
      assert got.dtype == dtype and np.array_equal(got, oracle_mod.coo_atomic_prod(w, post, post_n))
      indices, indptr = synth.bernoulli_csr(800, 1200, 0.1, seed=5)
      events = rng.random(800) < 0.4
      data = rng.uniform(0.98, 1.02, indices.shape[0]).astype(dtype)
      got = bpl.csr_event_prod(events, (indices.astype(it), indptr.astype(it)), 1200, data).cpu().numpy()
      want = oracle_mod.csr_event_prod(events, (indices, indptr), 1200, data)
      count = np.bincount(indices[np.repeat(events, np.diff(indptr))], minlength=1200)
      _assert_close_product(got, want, count, dtype, "csr_event_prod")
      assert np.all(got[count == 0] == 1)


def test_prod_known_answers_and_argument_checks(cuda):
  # brainpylib/_src/compat/tests/test_atomic_prod_cpu.py:16-53
  size = 200
  ids = np.arange(size, dtype=np.uint32)
  sps = np.random.default_rng(12345).integers(0, 2, size).astype(np.float32)
  assert np.array_equal(bpl.coo_atomic_prod(sps, ids, size, ids).cpu().numpy(), sps)
  assert np.all(bpl.coo_atomic_prod(2., ids, size).cpu().numpy() == 2.)
  pre, post = np.divmod(np.arange(100, dtype=np.int32), 10)
  assert np.all(bpl.coo_atomic_prod(2., post, 10).cpu().numpy() == 1024.)
  assert np.all(bpl.coo_atomic_prod(np.full(10, 2., np.float32), post, 10, pre).cpu().numpy() == 1024.)
  # a NaN weight reaches its target and nothing else
  v = np.ones(10, np.float64)
  v[3] = np.nan
  got = bpl.coo_atomic_prod(v, np.arange(10, dtype=np.int32), 10, np.arange(10, dtype=np.int32)).cpu().numpy()
  assert np.isnan(got[3]) and np.all(np.delete(got, 3) == 1)
  # no connections, no events: ones
  e = np.zeros(0, np.int32)
  assert np.all(bpl.coo_atomic_prod(3., e, 6).cpu().numpy() == 1.)
  indices = np.array([1, 2, 0, 2, 2], dtype=np.int32)
  indptr = np.array([0, 2, 2, 4, 5], dtype=np.int32)
  got = bpl.csr_event_prod(np.array([True, True, False, True]), (indices, indptr), 3, np.array([2., 3., 5., 7., 11.]))
  assert np.array_equal(got.cpu().numpy(), [1., 2., 33.])
  assert np.all(bpl.csr_event_prod(np.zeros(4, bool), (indices, indptr), 3, 3.).cpu().numpy() == 1.)
  with pytest.raises(ValueError):
    bpl.csr_event_prod(np.ones(4, np.float32), (indices, indptr), 3, 1.0)  # events must be bool
  with pytest.raises(ValueError):
    bpl.csr_event_prod(np.ones(3, bool), (indices, indptr), 3, 1.0)
  with pytest.raises(ValueError):
    bpl.coo_atomic_prod(np.ones(5, np.float32), post, 10, pre)  # values shorter than max(pre_ids)
