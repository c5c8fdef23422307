"""Pins the oracles of the older operator family (coo_atomic_sum, coo_event_sum, csr_event_sum
with 64-bit indices) against the golden vectors written by the reference's own
lib/cpu_atomic_sum.cc and lib/cpu_event_sum.cc, against the known answers of the reference's
tests, and against numpy's bincount."""
import os

import numpy as np

from util import assert_close

GOLD = os.path.join(os.path.dirname(__file__), "golden", "compat_cpu_reference.npz")


def test_coo_atomic_sum_golden(oracle_mod):
  z = np.load(GOLD)
  n = sum(1 for k in z.files if k.startswith("as_out_"))
  assert n == 32
  for i in range(n):
    values, pre, post, num = z["as_values_%d" % i], z["as_pre_%d" % i], z["as_post_%d" % i], int(z["as_num_%d" % i])
    got = oracle_mod.coo_atomic_sum(values, post, num, None if values.shape[0] == 1 else pre)
    assert np.array_equal(got, z["as_out_%d" % i]), "case %d" % i


def test_csr_event_sum_wide_golden(oracle_mod):
  z = np.load(GOLD)
  n = sum(1 for k in z.files if k.startswith("es_out_"))
  assert n == 12
  for i in range(n):
    shape = tuple(int(x) for x in z["es_shape_%d" % i])
    got = oracle_mod.csr_event_sum(z["es_events_%d" % i], (z["es_indices_%d" % i], z["es_indptr_%d" % i]), shape[1],
                                   z["es_data_%d" % i])
    assert np.array_equal(got, z["es_out_%d" % i]), "case %d" % i


def test_known_answers_of_the_reference_tests(oracle_mod):
  # brainpylib/_src/compat/tests/test_atomic_sum_cpu.py:16-34: identity connections
  size = 200
  ids = np.arange(size, dtype=np.uint32)
  sps = np.random.default_rng(12345).integers(0, 2, size).astype(np.float32)
  assert np.array_equal(oracle_mod.coo_atomic_sum(sps, ids, size, ids), sps)
  assert np.all(oracle_mod.coo_atomic_sum(np.float32(2.), ids, size) == 2.)
  # :36-53: all-to-all, every post neuron receives `size` contributions
  pre, post = np.divmod(np.arange(100, dtype=np.int32), 10)
  assert np.all(oracle_mod.coo_atomic_sum(np.float32(2.), post, 10) == 20.)
  assert np.all(oracle_mod.coo_atomic_sum(np.full(10, 2., np.float32), post, 10, pre) == 20.)


def test_coo_event_sum_vs_bincount_and_csr(oracle_mod):
  rng = np.random.default_rng(8)
  for pre_n, post_n, conn in [(200, 200, 20000), (30, 500, 3000), (500, 3, 4000)]:
    pre = rng.integers(0, pre_n, conn).astype(np.int32)
    post = rng.integers(0, post_n, conn).astype(np.int32)
    events = rng.random(pre_n) < 0.5
    w = rng.standard_normal(conn)
    want = np.bincount(post, weights=w * events[pre], minlength=post_n)
    got = oracle_mod.coo_event_sum(events, pre, post, post_n, w)
    assert_close(got, want, rtol=1e-12, atol=1e-12)
    got = oracle_mod.coo_event_sum(events, pre.astype(np.int64), post.astype(np.int64), post_n, np.float64(0.5))
    assert_close(got, 0.5 * np.bincount(post, weights=events[pre].astype(float), minlength=post_n), rtol=1e-12,
                 atol=1e-12)
    # the same connections sorted by pre neuron are a CSR structure: csr_event_sum agrees
    order = np.argsort(pre, kind="stable")
    indptr = np.concatenate([[0], np.cumsum(np.bincount(pre, minlength=pre_n))]).astype(np.int32)
    csr = oracle_mod.csr_event_sum(events, (post[order], indptr), post_n, w[order])
    assert_close(csr, want, rtol=1e-12, atol=1e-12)
    want_as = np.bincount(post, weights=w[:pre_n][pre] if conn >= pre_n else None, minlength=post_n)
    got_as = oracle_mod.coo_atomic_sum(w[:pre_n].copy(), post, post_n, pre)
    assert_close(got_as, want_as, rtol=1e-12, atol=1e-12)


PROD_GOLD = os.path.join(os.path.dirname(__file__), "golden", "compat_prod_cpu_reference.npz")


def test_coo_atomic_prod_golden(oracle_mod):
  # lib/cpu_atomic_prod.cc, compiled: the restatement multiplies in the same order, so bit for bit
  z = np.load(PROD_GOLD)
  n = sum(1 for k in z.files if k.startswith("ap_out_"))
  assert n == 32
  for i in range(n):
    values, pre, post, num = z["ap_values_%d" % i], z["ap_pre_%d" % i], z["ap_post_%d" % i], int(z["ap_num_%d" % i])
    got = oracle_mod.coo_atomic_prod(values, post, num, None if values.shape[0] == 1 else pre)
    assert np.array_equal(got, z["ap_out_%d" % i]), "case %d" % i


def test_csr_event_prod_golden(oracle_mod):
  z = np.load(PROD_GOLD)
  n = sum(1 for k in z.files if k.startswith("ep_out_"))
  assert n == 24
  for i in range(n):
    got = oracle_mod.csr_event_prod(z["ep_events_%d" % i], (z["ep_indices_%d" % i], z["ep_indptr_%d" % i]),
                                    int(z["ep_shape_%d" % i][1]), z["ep_data_%d" % i])
    assert np.array_equal(got, z["ep_out_%d" % i]), "case %d" % i


def test_prod_known_answers_of_the_reference_tests(oracle_mod):
  # brainpylib/_src/compat/tests/test_atomic_prod_cpu.py:16-34: identity connections
  size = 200
  ids = np.arange(size, dtype=np.uint32)
  sps = np.random.default_rng(12345).integers(0, 2, size).astype(np.float32)
  assert np.array_equal(oracle_mod.coo_atomic_prod(sps, ids, size, ids), sps)
  assert np.all(oracle_mod.coo_atomic_prod(np.float32(2.), ids, size) == 2.)
  # :36-53: all-to-all of 10 x 10, every post neuron is multiplied by 2 ten times
  pre, post = np.divmod(np.arange(100, dtype=np.int32), 10)
  assert np.all(oracle_mod.coo_atomic_prod(np.float32(2.), post, 10) == 1024.)
  assert np.all(oracle_mod.coo_atomic_prod(np.full(10, 2., np.float32), post, 10, pre) == 1024.)


def test_prod_vs_numpy(oracle_mod):
  # an independent route: numpy's unbuffered multiply.at in float64, and powers of the weight
  rng = np.random.default_rng(21)
  for pre_n, post_n, conn in [(200, 200, 3000), (30, 500, 1000), (500, 3, 300)]:
    pre = rng.integers(0, pre_n, conn).astype(np.int32)
    post = rng.integers(0, post_n, conn).astype(np.int64)
    values = rng.uniform(0.9, 1.1, pre_n)
    values[rng.integers(0, pre_n, 5)] *= -1
    want = np.ones(post_n)
    np.multiply.at(want, post, values[pre])
    assert_close(oracle_mod.coo_atomic_prod(values, post, post_n, pre.astype(np.int64)), want, rtol=1e-12, atol=0)
    count = np.bincount(post, minlength=post_n)
    got = oracle_mod.coo_atomic_prod(np.float64(0.99), post, post_n)
    assert_close(got, 0.99 ** count, rtol=1e-12, atol=0)
    assert np.all(got[count == 0] == 1.0)
  # a dropped event test or a swapped indices/indptr would show here
  indices = np.array([1, 2, 0, 2, 2], dtype=np.int32)
  indptr = np.array([0, 2, 2, 4, 5], dtype=np.int32)
  events = np.array([True, True, False, True])
  got = oracle_mod.csr_event_prod(events, (indices, indptr), 3, np.array([2., 3., 5., 7., 11.]))
  assert np.array_equal(got, [1., 2., 33.])
  got = oracle_mod.csr_event_prod(events, (indices, indptr), 3, np.float32(3.))
  assert np.array_equal(got, [1., 3., 9.])
  assert np.all(oracle_mod.csr_event_prod(np.zeros(4, bool), (indices, indptr), 3, np.float32(3.)) == 1.)
