"""GPU parity of the older operator family (csr_event_sum, coo_event_sum, coo_atomic_sum)
against the golden vectors of the reference's CPU kernels and against the CPU oracle."""
import os

import numpy as np
import pytest

import brainpylib_amd as bpl
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
