"""Pins the CSR oracles against dense brute force, scipy.sparse, the reference tests' own
cross-implementation identities and the golden vectors of the reference's lib/cpu_event_sum.cc."""
import os

import numpy as np
import pytest
import scipy.sparse as sp

from util import CSR_SHAPES, assert_close, random_csr, to_dense

GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("shape", CSR_SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_event_csr_matvec_vs_dense_and_identities(oracle_mod, shape, transpose, dtype):
  # brainpylib/_src/event_ops/tests/test_event_csr_matvec.py:57-73,205-217
  data, indices, indptr = random_csr(shape, 0.4, seed=shape[0] * 7 + shape[1], dtype=dtype)
  rng = np.random.default_rng(3)
  events = rng.random(shape[0] if transpose else shape[1]) < 0.1
  dense = to_dense(data, indices, indptr, shape)
  want = (events.astype(np.float64) @ dense) if transpose else (dense @ events.astype(np.float64))
  got = oracle_mod.event_csr_matvec(data, indices, indptr, events, shape=shape, transpose=transpose)
  assert got.dtype == dtype
  assert_close(got, want, rtol=1e-5, atol=1e-5)
  # float events: truthiness, not multiplication
  fev = (events * rng.uniform(0.5, 2.0, events.shape[0])).astype(dtype)
  got_f = oracle_mod.event_csr_matvec(data, indices, indptr, fev, shape=shape, transpose=transpose)
  assert np.array_equal(got_f, got)
  # homo == heter(ones * w)
  w = dtype(1.5)
  h1 = oracle_mod.event_csr_matvec(np.array([w]), indices, indptr, events, shape=shape, transpose=transpose)
  h2 = oracle_mod.event_csr_matvec(np.full(indices.shape[0], w, dtype=dtype), indices, indptr, events, shape=shape,
                                   transpose=transpose)
  if indices.shape[0] > 1:
    assert np.array_equal(h1, h2)
  # scipy
  A = sp.csr_matrix((data.astype(np.float64), indices, indptr), shape=shape)
  want_sp = (A.T @ events.astype(np.float64)) if transpose else (A @ events.astype(np.float64))
  assert_close(got, want_sp, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("shape", CSR_SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_csr_matvec_vs_dense_and_scipy(oracle_mod, shape, transpose, dtype):
  # brainpylib/_src/sparse_ops/tests/test_sparse_csr_matvec.py:31-42,66-73
  data, indices, indptr = random_csr(shape, 0.4, seed=shape[0] * 11 + shape[1], dtype=dtype, weights="uniform")
  v = np.random.default_rng(4).standard_normal(shape[0] if transpose else shape[1]).astype(dtype)
  A = sp.csr_matrix((data.astype(np.float64), indices, indptr), shape=shape)
  want = (A.T @ v.astype(np.float64)) if transpose else (A @ v.astype(np.float64))
  got = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=transpose)
  tol = 2e-5 if dtype == np.float32 else 1e-12
  assert_close(got, want, rtol=tol, atol=tol * 10)
  dense = to_dense(data, indices, indptr, shape)
  want_d = (v.astype(np.float64) @ dense) if transpose else (dense @ v.astype(np.float64))
  assert_close(got, want_d, rtol=tol, atol=tol * 10)
  # homo == heter(ones * w)
  w = dtype(0.75)
  h1 = oracle_mod.csr_matvec(np.array([w]), indices, indptr, v, shape=shape, transpose=transpose)
  h2 = oracle_mod.csr_matvec(np.full(indices.shape[0], w, dtype=dtype), indices, indptr, v, shape=shape,
                             transpose=transpose)
  if indices.shape[0] > 1:
    assert np.array_equal(h1, h2)


def test_event_scatter_matches_reference_cpu_event_sum_golden(oracle_mod):
  z = np.load(os.path.join(GOLD, "event_sum_cpu_reference.npz"))
  n = sum(1 for k in z.files if k.startswith("out_"))
  assert n == 24
  for i in range(n):
    shape = tuple(int(x) for x in z["shape_%d" % i])
    got = oracle_mod.event_csr_matvec(z["data_%d" % i], z["indices_%d" % i], z["indptr_%d" % i],
                                      z["events_%d" % i], shape=shape, transpose=True)
    want = z["out_%d" % i]
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), i


def test_event_scatter_matches_live_reference_build(oracle_mod, ref_mod):
  shape = (300, 170)
  data, indices, indptr = random_csr(shape, 0.2, seed=8)
  events = np.random.default_rng(1).random(shape[0]) < 0.3
  for d in (data, np.array([0.6], dtype=np.float32)):
    want = ref_mod.csr_event_sum(d, indices, indptr, events, shape=shape)
    got = oracle_mod.event_csr_matvec(d, indices, indptr, events, shape=shape, transpose=True)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_edge_cases(oracle_mod):
  # empty rows, an all-silent and an all-active event vector, an empty matrix
  indptr = np.array([0, 0, 3, 3, 5], dtype=np.int32)
  indices = np.array([0, 2, 4, 1, 4], dtype=np.int32)
  data = np.array([1, 2, 3, 4, 5], dtype=np.float32)
  shape = (4, 5)
  z = np.zeros(5, dtype=bool)
  assert not oracle_mod.event_csr_matvec(data, indices, indptr, z, shape=shape).any()
  o = np.ones(5, dtype=bool)
  assert np.array_equal(oracle_mod.event_csr_matvec(data, indices, indptr, o, shape=shape), [0, 6, 0, 9])
  assert np.array_equal(oracle_mod.event_csr_matvec(data, indices, indptr, np.ones(4, bool), shape=shape,
                                                    transpose=True), [1, 4, 2, 0, 8])
  e_ip = np.zeros(4, dtype=np.int32)
  e = np.zeros(0, dtype=np.int32)
  assert not oracle_mod.csr_matvec(np.zeros(0, np.float32), e, e_ip, np.ones(7, np.float32), shape=(3, 7)).any()


def test_event_info_is_ordered_compaction(oracle_mod):
  rng = np.random.default_rng(0)
  for dt in (np.bool_, np.int32, np.int64, np.float32, np.float64):
    ev = ((rng.random(1000) < 0.1) * rng.integers(1, 5, 1000)).astype(dt)
    ids, num = oracle_mod.event_info(ev)
    nz = np.flatnonzero(ev)
    assert num[0] == nz.size == (ev != 0).sum()
    assert np.array_equal(ids[:nz.size], nz) and (ids[nz.size:] == -1).all()
