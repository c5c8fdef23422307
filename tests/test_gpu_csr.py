"""GPU parity of event_csr_matvec / csr_matvec against the CPU oracle, through the C ABI
(the host wrappers call the custom-call targets of libbrainpylib_amd.so).

Bit-exact where the arithmetic allows it (homogeneous weights, integer-valued weights);
otherwise within the stated tolerance rel 1e-5 / abs 1e-6 (atomics reorder additions)."""
import os

import numpy as np
import pytest
import torch

import brainpylib_amd as bpl
import benchdata as synth
from util import CSR_SHAPES, assert_close, assert_close_reordered, random_csr

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _events(rng, n, kind, dtype, rate=0.1):
  ev = rng.random(n) < rate
  if kind == "bool":
    return ev
  return (ev * rng.uniform(0.5, 2.0, n)).astype(dtype)


@pytest.mark.parametrize("shape", CSR_SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("ev_kind", ["bool", "float"])
def test_event_csr_matvec_reference_test_shapes(cuda, oracle_mod, shape, transpose, dtype, ev_kind):
  data, indices, indptr = random_csr(shape, 0.4, seed=shape[0] * 3 + shape[1], dtype=dtype)
  rng = np.random.default_rng(5)
  events = _events(rng, shape[0] if transpose else shape[1], ev_kind, dtype)
  print("case", shape, transpose, dtype.__name__, ev_kind, flush=True)
  # heterogeneous weights
  want = oracle_mod.event_csr_matvec(data, indices, indptr, events, shape=shape, transpose=transpose)
  got = bpl.event_csr_matvec(data, indices, indptr, events, shape=shape, transpose=transpose).cpu().numpy()
  assert got.dtype == dtype
  if transpose:
    mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, events, shape=shape, transpose=True)
    assert_close_reordered(got, want, mag, dtype, what="heter scatter")
  else:
    assert_close(got, want, what="heter gather")
  # homogeneous weight: every addend is the same value, so the result is order independent
  w = np.array([0.6], dtype=dtype)
  want = oracle_mod.event_csr_matvec(w, indices, indptr, events, shape=shape, transpose=transpose)
  got = bpl.event_csr_matvec(w, indices, indptr, events, shape=shape, transpose=transpose).cpu().numpy()
  # the weight is added once per synapse (in place when scattering, into a float64 accumulator
  # when gathering): the result depends on the count alone and equals the reference's bit for bit
  assert np.array_equal(got, want), "homogeneous weight must be bit-exact"
  # integer-valued weights: exact in any order
  di = np.random.default_rng(6).integers(-1, 2, size=indices.shape[0]).astype(dtype)
  want = oracle_mod.event_csr_matvec(di, indices, indptr, events, shape=shape, transpose=transpose)
  got = bpl.event_csr_matvec(di, indices, indptr, events, shape=shape, transpose=transpose).cpu().numpy()
  assert np.array_equal(got, want), "integer weights must be bit-exact"


@pytest.mark.parametrize("shape", CSR_SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("method", ["scalar", "vector", "adaptive"])
def test_csr_matvec_reference_test_shapes(cuda, oracle_mod, shape, dtype, method):
  data, indices, indptr = random_csr(shape, 0.4, seed=shape[0] * 5 + shape[1], dtype=dtype, weights="uniform")
  v = np.random.default_rng(7).standard_normal(shape[1]).astype(dtype)
  print("case", shape, dtype.__name__, method, flush=True)
  want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape)
  got = bpl.csr_matvec(data, indices, indptr, v, shape=shape, method=method).cpu().numpy()
  assert_close(got, want, what="heter")
  w = np.array([0.75], dtype=dtype)
  want = oracle_mod.csr_matvec(w, indices, indptr, v, shape=shape)
  got = bpl.csr_matvec(w, indices, indptr, v, shape=shape, method=method).cpu().numpy()
  assert_close(got, want, what="homo")
  # integer data and vector: exact
  di = np.random.default_rng(8).integers(-2, 3, size=indices.shape[0]).astype(dtype)
  vi = np.random.default_rng(9).integers(-2, 3, size=shape[1]).astype(dtype)
  want = oracle_mod.csr_matvec(di, indices, indptr, vi, shape=shape)
  got = bpl.csr_matvec(di, indices, indptr, vi, shape=shape, method=method).cpu().numpy()
  assert np.array_equal(got, want)


@pytest.mark.parametrize("shape", CSR_SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_csr_matvec_transpose(cuda, oracle_mod, shape, dtype):
  data, indices, indptr = random_csr(shape, 0.4, seed=shape[0] * 9 + shape[1], dtype=dtype, weights="uniform")
  v = np.random.default_rng(7).standard_normal(shape[0]).astype(dtype)
  print("case", shape, dtype.__name__, flush=True)
  want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=True)
  got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
  # sums of up to shape[0] terms of mixed sign accumulated in another order: scale the
  # absolute tolerance by the magnitude of the sum of |terms|
  mag = oracle_mod.csr_matvec(data, indices, indptr, np.abs(v), shape=shape, transpose=True)  # data >= 0
  assert_close_reordered(got, want, mag, dtype, what="csr scatter")
  w = np.array([0.5], dtype=dtype)
  vi = np.random.default_rng(9).integers(-2, 3, size=shape[0]).astype(dtype)
  want = oracle_mod.csr_matvec(w, indices, indptr, vi, shape=shape, transpose=True)
  got = bpl.cusparse_csr_matvec(w, indices, indptr, vi, shape=shape, transpose=True).cpu().numpy()
  assert np.array_equal(got, want)


def test_event_scatter_against_reference_cpu_event_sum_golden(cuda):
  z = np.load(os.path.join(GOLD, "event_sum_cpu_reference.npz"))
  n = sum(1 for k in z.files if k.startswith("out_"))
  for i in range(n):
    shape = tuple(int(x) for x in z["shape_%d" % i])
    got = bpl.event_csr_matvec(z["data_%d" % i], z["indices_%d" % i], z["indptr_%d" % i], z["events_%d" % i],
                               shape=shape, transpose=True).cpu().numpy()
    want = z["out_%d" % i]
    if z["data_%d" % i].shape[0] == 1:
      assert np.array_equal(got, want), "golden homo %d" % i  # the compiled reference's bits
    else:
      mag = np.zeros(shape[1])
      ev, ip, ix, d = z["events_%d" % i], z["indptr_%d" % i], z["indices_%d" % i], z["data_%d" % i]
      for r in np.flatnonzero(ev):
        np.add.at(mag, ix[ip[r]:ip[r + 1]], np.abs(d[ip[r]:ip[r + 1]]))
      assert_close_reordered(got, want, mag, d.dtype.type, what="golden %d" % i)


def test_edge_cases(cuda, oracle_mod):
  # empty rows, silent / saturated event vectors, uint32 indices, empty matrix, zero rows
  indptr = np.array([0, 0, 3, 3, 5], dtype=np.int32)
  indices = np.array([0, 2, 4, 1, 4], dtype=np.int32)
  data = np.array([1, 2, 3, 4, 5], dtype=np.float32)
  shape = (4, 5)
  for tr in (False, True):
    n_in = shape[0] if tr else shape[1]
    for ev in (np.zeros(n_in, bool), np.ones(n_in, bool)):
      want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=tr)
      got = bpl.event_csr_matvec(data, indices.astype(np.uint32), indptr.astype(np.uint32), ev, shape=shape,
                                 transpose=tr).cpu().numpy()
      assert np.array_equal(got, want)
  e_ip = np.zeros(4, dtype=np.int32)
  e = np.zeros(0, dtype=np.int32)
  out = bpl.csr_matvec(np.zeros(0, np.float32), e, e_ip, np.ones(7, np.float32), shape=(3, 7)).cpu().numpy()
  assert out.shape == (3,) and not out.any()
  out = bpl.event_csr_matvec(1.0, e, e_ip, np.ones(3, bool), shape=(3, 7), transpose=True).cpu().numpy()
  assert out.shape == (7,) and not out.any()
  # NaN and -0.0 float events: NaN is an event, -0.0 is not
  ev = np.array([np.nan, -0.0, 0.0, 1e-30, 0.0], dtype=np.float32)
  want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
  got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape).cpu().numpy()
  assert np.array_equal(got, want)
  # output buffer is fully overwritten (results may be uninitialised on entry)
  t = torch.full((5,), 7.0, device=cuda)
  del t


def test_python_number_weights_keep_their_values(cuda, oracle_mod):
  # a homogeneous weight given as a Python number is copied to the device once per value:
  # alternating values must not alias each other
  shape = (50, 70)
  _, indices, indptr = random_csr(shape, 0.3, seed=11, dtype=np.float32)
  events = np.random.default_rng(3).random(shape[0]) < 0.5
  ix, ip, ev = (torch.from_numpy(a).cuda() for a in (indices, indptr, events))
  for w in (0.6, -1.25, 0.6, 3, -1.25, float("nan"), 0.6):
    want = oracle_mod.event_csr_matvec(np.float32(w), indices, indptr, events, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(w, ix, ip, ev, shape=shape, transpose=True).cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6, equal_nan=True)
  # zeros of either sign and NaN are values of their own (the copies are kept by bit pattern): the
  # sign bit of every output element is the oracle's, in both orientations, whichever came first
  for w in (0.0, -0.0, 0.0, float("nan"), -0.0):
    for transpose in (True, False):
      e, evt = (events, ev) if transpose else (np.resize(events, shape[1]), torch.from_numpy(np.resize(events, shape[1])).cuda())
      want = oracle_mod.event_csr_matvec(np.float32(w), indices, indptr, e, shape=shape, transpose=transpose)
      got = bpl.event_csr_matvec(w, ix, ip, evt, shape=shape, transpose=transpose).cpu().numpy()
      assert np.array_equal(got, want, equal_nan=True) and np.array_equal(np.signbit(got), np.signbit(want)), (w, transpose)


def test_ragged_rows_and_all_row_length_modes(cuda, oracle_mod):
  # mean row lengths that select each lanes-per-row mode (8 / 16 / 32 / 64), with ragged rows,
  # empty rows and one very long row
  rng = np.random.default_rng(11)
  n_col = 5000
  for mean in (3, 14, 30, 200):
    counts = rng.poisson(mean, size=3000)
    counts[::7] = 0
    counts[5] = 4000
    indices, indptr = synth.counted_csr(counts, n_col, seed=mean)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    ev = rng.random(n_col) < 0.2
    v = rng.standard_normal(n_col).astype(np.float32)
    shape = (counts.shape[0], n_col)
    print("mean row length", mean, flush=True)
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape).cpu().numpy()
    assert_close(got, want, what="event gather mean %d" % mean)
    want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape)
    got = bpl.csr_matvec(data, indices, indptr, v, shape=shape).cpu().numpy()
    assert_close(got, want, what="csr gather mean %d" % mean)
    evr = rng.random(shape[0]) < 0.3
    want = oracle_mod.event_csr_matvec(data, indices, indptr, evr, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(data, indices, indptr, evr, shape=shape, transpose=True).cpu().numpy()
    mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, evr, shape=shape, transpose=True)
    assert_close_reordered(got, want, mag, what="event scatter mean %d" % mean)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gather_long_rows_that_begin_at_different_steps(cuda, oracle_mod, dtype):
  # rows of 384 nonzeros or more take a wave each, in steps of 512 (float64: the same walk), and begin at a full
  # step chosen by the row's number: rows of exactly 1, 2, 3, 4 and 9 full steps, with and without a partial
  # last step, every row number modulo 4 among them.  Integer weights: the sums are exact whatever the order.
  rng = np.random.default_rng(21)
  n_col = 40_000
  lengths = [512, 1024, 1536, 2048, 4608, 513, 1023, 1025, 2049, 2047, 4096 + 5, 700, 385]
  counts = np.array([lengths[(i * 5 + i // 13) % len(lengths)] for i in range(416)])
  indices, indptr = synth.counted_csr(counts, n_col, seed=4)
  data = rng.integers(-8, 9, indices.shape[0]).astype(dtype)
  shape = (counts.shape[0], n_col)
  for rate in (0.05, 0.6):
    ev = rng.random(n_col) < rate
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape).cpu().numpy()
    assert np.array_equal(got, want), "heterogeneous, events %g" % rate
    w = np.array([3.0], dtype)
    want = oracle_mod.event_csr_matvec(w, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(w, indices, indptr, ev, shape=shape).cpu().numpy()
    assert np.array_equal(got, want), "one weight, events %g" % rate
  v = rng.integers(-4, 5, n_col).astype(dtype)
  want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape)
  got = bpl.csr_matvec(data, indices, indptr, v, shape=shape).cpu().numpy()
  assert np.array_equal(got, want), "dense vector"


def test_unaligned_event_vector_and_large_bitmap(cuda, oracle_mod):
  # an event vector that does not start on a 16-byte boundary, and one whose bitmap needs more
  # than 64 KiB of LDS (n_col > 524288)
  rng = np.random.default_rng(12)
  for n_col, offset in ((70001, 3), (700_000, 0), (1_400_000, 1)):
    counts = rng.poisson(40, size=2000)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_col)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    ev = rng.random(n_col) < 0.3
    shape = (2000, n_col)
    print("n_col", n_col, "offset", offset, flush=True)
    base = torch.zeros(n_col + 16, dtype=torch.bool, device=cuda)
    base[offset:offset + n_col] = torch.from_numpy(ev).to(cuda)
    ev_dev = base[offset:offset + n_col]
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(data, indices, indptr, ev_dev, shape=shape).cpu().numpy()
    assert_close(got, want)


def test_gather_row_length_modes_with_a_bitmap_that_fills_lds(cuda, oracle_mod):
  # more than 655,360 columns: the event bitmap leaves room for one workgroup per CU, and the
  # lanes-per-row modes of that regime are used (rows under 48 / 48 .. 383 / from 384 nonzeros)
  rng = np.random.default_rng(14)
  n_col = 700_000
  for n_row, mean in ((20_000, 5), (20_000, 40), (18_000, 120), (3000, 120), (17_000, 500)):
    counts = rng.poisson(mean, size=n_row)
    counts[::7] = 0
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row + mean)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    ev = rng.random(n_col) < 0.2
    shape = (n_row, n_col)
    print("shape", shape, "mean", mean, flush=True)
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape).cpu().numpy()
    assert_close(got, want)
    w = np.float32(0.37)
    want = oracle_mod.event_csr_matvec(w, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(w, indices, indptr, ev, shape=shape).cpu().numpy()
    assert_close(got, want)
    evf = (ev * rng.uniform(0.5, 2.0, n_col)).astype(np.float32)
    got = bpl.event_csr_matvec(data, indices, indptr, evf, shape=shape).cpu().numpy()
    want = oracle_mod.event_csr_matvec(data, indices, indptr, evf, shape=shape)
    assert_close(got, want)


@pytest.mark.parametrize("kind", ["ragged", "even", "step", "hub", "few", "dense_events", "offset"])
def test_gather_flat_walk_over_the_nonzeros_of_short_rows(cuda, oracle_mod, kind):
  # more than 655,360 columns and rows of 16 to 383 nonzeros on average: every wave walks a contiguous range of the
  # nonzeros that begins and ends at row boundaries and looks rows up for the hits only.  Integer weights: the sums
  # are exact, so every output is compared bit for bit (weights per nonzero, one weight, float events, float64).
  rng = np.random.default_rng(sum(map(ord, kind)))
  n_col, rate = 900_000, 0.05
  if kind == "ragged":      # empty rows, rows of one nonzero, rows of a thousand
    counts = rng.choice([0, 1, 3, 40, 150, 1000], size=60_000, p=[0.2, 0.1, 0.2, 0.3, 0.15, 0.05])
  elif kind == "even":      # every row 100 nonzeros: twelve rows and a bit per step of 1,280
    counts = np.full(200_000, 100)
  elif kind == "step":      # rows of exactly one step and of exactly one quad
    counts = np.where(np.arange(40_000) % 4 == 0, 1280, 4)
  elif kind == "hub":       # one row longer than a wave's whole share, between rows of 30
    counts = np.full(40_000, 30)
    counts[17_777] = 700_000
  elif kind == "few":       # fewer rows than waves
    counts = rng.integers(16, 200, size=1_500)
  elif kind == "dense_events":  # most nonzeros hit: the queue of hits is filled in several rounds per step
    counts, rate = rng.poisson(60, size=50_000), 0.9
  else:                     # many empty rows in a row, the matrix's last nonzeros in a partial quad
    counts = np.where((np.arange(90_001) // 500) % 2 == 0, 0, 70)
    counts[-1] = 3
  indices, indptr = synth.counted_csr(np.minimum(counts, n_col), n_col, seed=len(counts))
  nnz, n_row = indices.shape[0], len(counts)
  mean = nnz // n_row
  assert 16 <= mean < 384, mean
  shape = (n_row, n_col)
  ev = rng.random(n_col) < rate
  print("kind", kind, shape, "nnz", nnz, "mean", mean, flush=True)
  for dtype in (np.float32, np.float64):
    data = rng.integers(-3, 4, size=nnz).astype(dtype)
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape).cpu().numpy()
    assert np.array_equal(got, want), (kind, dtype, int((got != want).sum()), np.flatnonzero(got != want)[:5])
    w = np.array([0.37], dtype=dtype)
    want = oracle_mod.event_csr_matvec(w, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(w, indices, indptr, ev, shape=shape).cpu().numpy()
    assert np.array_equal(got, want), (kind, dtype, "one weight")
  evf = (ev * rng.uniform(0.5, 2.0, n_col)).astype(np.float64)
  got = bpl.event_csr_matvec(data, indices, indptr, evf, shape=shape).cpu().numpy()
  assert np.array_equal(got, oracle_mod.event_csr_matvec(data, indices, indptr, evf, shape=shape)), (kind, "float events")


@pytest.mark.parametrize("kind", ["ragged", "even", "dense_events"])
def test_gather_flat_walk_in_the_kernel_that_shares_its_cu(cuda, oracle_mod, kind):
  # A bitmap of at most 64 KB, weights per nonzero, rows of 16 to 255 nonzeros on average and 45 million nonzeros
  # or more: the same walk with three loads per lane and step, in the kernel that runs two workgroups per CU.
  # Integer weights: every output is compared bit for bit.  (Columns may repeat within a row: the sums do not care.)
  rng = np.random.default_rng(sum(map(ord, kind)) + 1)
  n_col, rate = 400_000, 0.05
  if kind == "ragged":      # empty rows, rows of one nonzero, rows of a thousand, one row longer than a wave's share
    counts = rng.choice([0, 1, 3, 40, 150, 1000], size=560_000, p=[0.2, 0.1, 0.2, 0.3, 0.15, 0.05])
    counts[333_333] = 300_000
  elif kind == "even":      # the widest bitmap that fits; runs of empty rows, also at the end; the last quad is partial
    n_col = 518_144
    counts = np.full(480_000, 100)
    counts[100_000:105_000] = 0
    counts[-3_000:] = 0
    counts[-3_001] = 3
  else:                     # most nonzeros hit: the queue of hits is filled in several rounds per step
    counts, rate = rng.poisson(60, size=800_000), 0.9
  counts = np.asarray(counts, dtype=np.int64)
  n_row = len(counts)
  indptr = np.zeros(n_row + 1, dtype=np.int32)
  indptr[1:] = np.cumsum(counts)
  nnz = int(indptr[-1])
  indices = rng.integers(0, n_col, size=nnz, dtype=np.int32)
  mean = nnz // n_row
  assert 16 <= mean < 256 and nnz >= 45_000_000, (mean, nnz)
  shape = (n_row, n_col)
  ev = rng.random(n_col) < rate
  print("kind", kind, shape, "nnz", nnz, "mean", mean, flush=True)
  for dtype in (np.float32, np.float64):
    data = rng.integers(-3, 4, size=nnz).astype(dtype)
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape).cpu().numpy()
    assert np.array_equal(got, want), (kind, dtype, int((got != want).sum()), np.flatnonzero(got != want)[:5])
  evf = (ev * rng.uniform(0.5, 2.0, n_col)).astype(np.float64)  # (events of the weights' type)
  got = bpl.event_csr_matvec(data, indices, indptr, evf, shape=shape).cpu().numpy()
  assert np.array_equal(got, oracle_mod.event_csr_matvec(data, indices, indptr, evf, shape=shape)), (kind, "float events")


def test_gather_with_a_two_level_event_bitmap(cuda, oracle_mod):
  # more columns than a bitmap in LDS can cover (1.3 million): a coarse bitmap (one bit per 2^g
  # columns) in LDS and the exact one in global memory; g = 2, 4 and 6 (both ways the coarse
  # bitmap is built), rows of all three length classes, bool and float events
  rng = np.random.default_rng(15)
  for n_col, n_row, mean in ((3_000_000, 20_000, 30), (3_000_000, 17_000, 450), (12_000_000, 3000, 120),
                             (45_000_001, 2000, 60)):
    counts = rng.poisson(mean, size=n_row)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row + mean)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    ev = rng.random(n_col) < 0.1
    ev[indices[::3]] = True  # (make sure many nonzeros do hit)
    shape = (n_row, n_col)
    print("shape", shape, "mean", mean, flush=True)
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape).cpu().numpy()
    assert_close(got, want)
    ones = np.array([0.6], dtype=np.float32)  # not representable: the sum depends on how it is formed
    want = oracle_mod.event_csr_matvec(ones, indices, indptr, ev, shape=shape)
    got = bpl.event_csr_matvec(ones, indices, indptr, ev, shape=shape).cpu().numpy()
    assert np.array_equal(got, want)
    if n_col <= 12_000_000:
      evf = (ev * rng.uniform(0.5, 2.0, n_col)).astype(np.float32)
      want = oracle_mod.event_csr_matvec(data, indices, indptr, evf, shape=shape)
      got = bpl.event_csr_matvec(data, indices, indptr, evf, shape=shape).cpu().numpy()
      assert_close(got, want)


def test_config_event_csr_small(cuda, oracle_mod):
  # 4,000 x 4,000, 80 per row, homogeneous 0.6, events 2 %, transpose
  c = synth.config_event_csr_small()
  want = oracle_mod.event_csr_matvec(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"],
                                     transpose=True)
  got = bpl.event_csr_matvec(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"],
                             transpose=True).cpu().numpy()
  assert_close(got, want)
  assert want.sum() > 0
  # the number of delivered synapses per target is exact: unit weight gives integer counts
  ones = np.array([0.6], dtype=np.float32)  # not representable: the sum depends on how it is formed
  want = oracle_mod.event_csr_matvec(ones, c["indices"], c["indptr"], c["events"], shape=c["shape"], transpose=True)
  got = bpl.event_csr_matvec(ones, c["indices"], c["indptr"], c["events"], shape=c["shape"], transpose=True).cpu().numpy()
  assert np.array_equal(got, want)


def test_config_event_csr_large_scaled_and_properties(cuda, oracle_mod):
  # the 1e8-nnz configuration at 1/16 scale against the oracle (25,000 x 25,000, ~6e6 nnz) ...
  c = synth.config_event_csr_large(n=25_000)
  for tr in (True, False):
    want = oracle_mod.event_csr_matvec(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"], transpose=tr)
    got = bpl.event_csr_matvec(c["data"], c["indices"], c["indptr"], c["events"], shape=c["shape"], transpose=tr)
    if tr:
      mag = oracle_mod.event_csr_matvec(np.abs(c["data"]), c["indices"], c["indptr"], c["events"], shape=c["shape"],
                                        transpose=True)
      assert_close_reordered(got.cpu().numpy(), want, mag, what="scatter")
    else:
      assert_close(got.cpu().numpy(), want, what="gather")


def test_full_size_event_csr_properties(cuda):
  # ... and at full size (100,000 x 100,000, ~1e8 nnz) through size-independent properties:
  #  * <y, A x> == <A^T y, x> with 0/1 vectors and integer weights (exact in fp32 up to 2^24)
  #  * linearity in the weights: f(2 * w) == 2 * f(w) bit for bit
  #  * all-ones events with unit weight give the row lengths / column counts exactly
  c = synth.config_event_csr_large()
  n = c["shape"][0]
  dev = cuda
  indices = torch.from_numpy(c["indices"]).to(dev)
  indptr = torch.from_numpy(c["indptr"]).to(dev)
  x = torch.from_numpy(c["events"]).to(dev)
  y = torch.from_numpy(np.random.default_rng(3).random(n) < 0.05).to(dev)
  ones = torch.ones(1, dtype=torch.float32, device=dev)
  Ax = bpl.event_csr_matvec(ones, indices, indptr, x, shape=c["shape"], transpose=False)
  ATy = bpl.event_csr_matvec(ones, indices, indptr, y, shape=c["shape"], transpose=True)
  lhs = float((Ax.double() * y.double()).sum())
  rhs = float((ATy.double() * x.double()).sum())
  assert lhs == rhs and lhs > 0
  row_len = np.diff(c["indptr"]).astype(np.float32)
  all_on = torch.ones(n, dtype=torch.bool, device=dev)
  got = bpl.event_csr_matvec(ones, indices, indptr, all_on, shape=c["shape"], transpose=False).cpu().numpy()
  assert np.array_equal(got, row_len)
  col_cnt = np.bincount(c["indices"], minlength=n).astype(np.float32)
  got = bpl.event_csr_matvec(ones, indices, indptr, all_on, shape=c["shape"], transpose=True).cpu().numpy()
  assert np.array_equal(got, col_cnt)
  data = torch.from_numpy(c["data"]).to(dev)
  f1 = bpl.event_csr_matvec(data, indices, indptr, x, shape=c["shape"], transpose=False)
  f2 = bpl.event_csr_matvec(data * 2, indices, indptr, x, shape=c["shape"], transpose=False)
  assert torch.equal(f1 * 2, f2)


def test_scatter_many_windows_and_row_chunks(cuda, oracle_mod):
  # transpose=True with (a) an output vector that needs several LDS windows and (b) row groups
  # larger than the active-row list, so that a workgroup walks its rows in several chunks
  rng = np.random.default_rng(21)
  # (mean row length below/above 64 selects direct atomics/LDS windows when there are many windows)
  for n_row, n_col, mean in ((5000, 700_000, 50), (600_000, 300, 3), (300_000, 200_000, 8),
                             (20_000, 400_000, 100)):
    counts = rng.poisson(mean, size=n_row)
    indices, indptr = synth.counted_csr(np.minimum(counts, n_col), n_col, seed=n_row)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    shape = (n_row, n_col)
    print("shape", shape, flush=True)
    for rate in (0.02, 0.9):
      ev = rng.random(n_row) < rate
      want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
      mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=shape, transpose=True)
      got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
      assert_close_reordered(got, want, mag, what="scatter %s rate %s" % (shape, rate))
      ones = np.array([0.6], dtype=np.float32)  # not representable: the sum depends on how it is formed
      want = oracle_mod.event_csr_matvec(ones, indices, indptr, ev, shape=shape, transpose=True)
      got = bpl.event_csr_matvec(ones, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
      assert np.array_equal(got, want)  # a homogeneous weight is added once per synapse: the reference's bits


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_event_scatter_sorted_by_output_window(cuda, oracle_mod, dtype):
  # event input and outputs wider than 131,072: the active rows' nonzeros are sorted coarsely by
  # output window.  Cases: more than 1,024 active rows per producer workgroup (several row tiles);
  # all columns in one window, more of them than the window's run holds (the rest goes through
  # direct atomics); float events; silent input; calls repeated (the counters are back at zero);
  # so little activity that the sort is skipped.
  rng = np.random.default_rng(41)
  cases = []
  counts = np.minimum(rng.poisson(3, size=1_200_000), 50)
  cases.append(("tiles", (1_200_000, 200_000), synth.counted_csr(counts, 200_000, seed=1), 0.9))
  # columns < 2,000: all 1.8 million pairs fall into one window (2,048 columns at this width), more than
  # its runs hold (8 x 171,000): the rest goes through direct atomics
  ix, ip = synth.counted_csr(np.full(3000, 600), 2000, seed=2)
  cases.append(("one window", (3000, 200_000), (ix, ip), 1.0))
  counts = rng.poisson(120, size=30_000)
  plain = synth.counted_csr(counts, 1_000_000, seed=3)
  cases.append(("plain", (30_000, 1_000_000), plain, 0.05))
  # some 7,000 active nonzeros: too few to be worth sorting, the active rows add them to y directly
  cases.append(("little activity", (30_000, 1_000_000), plain, 0.002))
  # above 2^21 columns a window is wider than its accumulators in LDS and is added in slices
  counts = rng.poisson(60, size=20_000)
  cases.append(("sliced windows", (20_000, 5_000_001), synth.counted_csr(counts, 5_000_001, seed=4), 0.3))
  for name, shape, (indices, indptr), rate in cases:
    print("case", name, shape, dtype.__name__, flush=True)
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    for kind in ("bool", "float", "silent"):
      ev = rng.random(shape[0]) < rate
      if kind == "silent":
        ev[:] = False
      elif kind == "float":
        ev = (ev * rng.uniform(0.5, 2.0, shape[0])).astype(dtype)
      for _ in range(2):
        want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
        mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=shape, transpose=True)
        got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
        assert got.dtype == dtype
        assert_close_reordered(got, want, mag, what="sorted event scatter %s %s" % (name, kind))
      ones = np.array([0.6], dtype=dtype)  # not representable: the sum depends on how it is formed
      want = oracle_mod.event_csr_matvec(ones, indices, indptr, ev, shape=shape, transpose=True)
      got = bpl.event_csr_matvec(ones, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
      assert np.array_equal(got, want)  # a homogeneous weight is added once per synapse: the reference's bits


def test_scatter_through_the_active_row_list(cuda, oracle_mod):
  # more than 32,768 rows: the active rows are first gathered into one list that the row groups
  # share; both input kinds, activity concentrated in one corner of the matrix, twice in a row
  # (the list's counter must be back at zero), silent input
  rng = np.random.default_rng(31)
  for n_row, n_col, mean in ((50_000, 3000, 20), (40_000, 150_000, 80), (70_000, 40_000, 5)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    data = rng.standard_normal(indices.shape[0]).astype(np.float32)
    shape = (n_row, n_col)
    print("shape", shape, flush=True)
    for kind in ("uniform", "corner", "silent"):
      ev = rng.random(n_row) < 0.05
      if kind == "corner":
        ev[n_row // 50:] = False
        ev[:n_row // 50] = True
      elif kind == "silent":
        ev[:] = False
      for _ in range(2):
        want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
        mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=shape, transpose=True)
        got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
        assert_close_reordered(got, want, mag, what="event scatter %s %s" % (shape, kind))
      ones = np.array([0.6], dtype=np.float32)  # not representable: the sum depends on how it is formed
      want = oracle_mod.event_csr_matvec(ones, indices, indptr, ev, shape=shape, transpose=True)
      got = bpl.event_csr_matvec(ones, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
      assert np.array_equal(got, want)
    if n_col <= 131072:  # dense input uses the windows up to four of them
      v = rng.standard_normal(n_row).astype(np.float32)
      v[rng.random(n_row) < 0.5] = 0
      want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=True)
      mag = oracle_mod.csr_matvec(np.abs(data), indices, indptr, np.abs(v), shape=shape, transpose=True)
      got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
      assert_close_reordered(got, want, mag, what="dense scatter %s" % (shape,))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_transposed_csr_matvec_wide_output_sorted_scatter(cuda, oracle_mod, dtype):
  # outputs beyond a few LDS windows with at least 2^20 nonzeros: products are binned by output
  # window first.  Even rows, one very long row (its bins overflow into direct atomics), few
  # rows, twice in a row, homogeneous weight.
  rng = np.random.default_rng(41)
  for n_row, n_col, mean, long_row in ((30_000, 300_000, 50, 0), (50_000, 400_000, 25, 250_000),
                                       (1500, 2_000_000, 1000, 0), (200_000, 140_000, 8, 0),
                                       # (fewer rows than producer workgroups: these take shares of the nonzeros, not rows)
                                       (40, 150_000, 50_000, 0), (12, 100_000, 0, 99_000),
                                       # (above 2^21 columns: windows wider than their LDS accumulators, added in slices)
                                       (4000, 5_000_001, 300, 0),
                                       # (above 2^23 columns: positions within a window beyond 16 bits, whole pairs)
                                       (3000, 9_000_000, 400, 0)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    if long_row:
      counts[7 % n_row] = long_row
      if n_row < 16:
        counts[:] = long_row
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    assert indices.shape[0] >= 1 << 20
    data = rng.random(indices.shape[0]).astype(dtype)
    shape = (n_row, n_col)
    print("shape", shape, dtype.__name__, flush=True)
    v = rng.standard_normal(n_row).astype(dtype)
    for _ in range(2):
      want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=True)
      mag = oracle_mod.csr_matvec(data, indices, indptr, np.abs(v), shape=shape, transpose=True)  # data >= 0
      got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
      assert_close_reordered(got, want, mag, dtype, what="sorted scatter %s" % (shape,))
    vi = rng.integers(-2, 3, size=n_row).astype(dtype)
    w = np.array([0.5], dtype=dtype)
    want = oracle_mod.csr_matvec(w, indices, indptr, vi, shape=shape, transpose=True)
    got = bpl.cusparse_csr_matvec(w, indices, indptr, vi, shape=shape, transpose=True).cpu().numpy()
    assert np.array_equal(got, want)  # multiples of 0.5: exact in any order


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_event_scatter_into_one_window_from_many_rows(cuda, oracle_mod, dtype):
  # more than 32,768 rows (the active rows go to a device list) and at most 8,192 columns: the listed rows'
  # nonzeros are walked flat into one window in LDS per workgroup.  Little and much activity, empty rows, a
  # row that holds a quarter of the nonzeros, bool and float events, both weight kinds (the homogeneous one
  # bit for bit), twice in a row (the list's counter must be back at zero).
  rng = np.random.default_rng(53)
  for n_row, n_col, mean, hub in ((100_000, 3000, 30, 0), (40_000, 8192, 12, 120_000), (300_000, 700, 3, 0),
                                  (33_000, 1, 2, 0)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    counts[rng.integers(0, n_row, size=n_row // 9)] = 0
    if hub:
      counts = counts.astype(np.int64)
      counts[n_row // 5] = min(hub, n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    shape = (n_row, n_col)
    print("shape", shape, dtype.__name__, flush=True)
    for rate in (0.0005, 0.05, 0.9):
      ev = rng.random(n_row) < rate
      if hub:
        ev[n_row // 5] = True
      want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
      mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=shape, transpose=True)
      for events in (ev, ev.astype(dtype) * 3):
        for _ in range(2):
          got = bpl.event_csr_matvec(data, indices, indptr, events, shape=shape, transpose=True).cpu().numpy()
          assert_close_reordered(got, want, mag, dtype, what="event scatter, one window %s rate %g" % (shape, rate))
      w = np.array([0.6], dtype=dtype)
      want = oracle_mod.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True)
      got = bpl.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
      assert np.array_equal(got, want), (shape, rate)  # the reference's repeated additions, bit for bit


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_event_scatter_of_one_weight_into_slices_of_the_output(cuda, oracle_mod, dtype):
  # a homogeneous weight, 32,769 to 65,536 rows and an output of up to four windows of 14,848 counts: the listed
  # rows are walked once per slice of the output into integer windows in LDS.  Widths at both ends of one, two
  # and four slices, the widths and row counts just beyond (the sorted scatter), little and much activity, empty
  # rows and a row that holds a large share of the nonzeros; bit for bit, twice in a row.  Weights per synapse
  # of the same matrices take the sorted scatter.
  rng = np.random.default_rng(61)
  # (up to 32,768 rows the workgroups find the active rows themselves: the same slices without the list)
  for n_row, n_col, mean, hub in ((40_000, 14_849, 20, 0), (65_536, 29_696, 9, 50_000), (33_000, 59_392, 25, 0),
                                  (50_000, 59_393, 10, 0), (65_537, 20_000, 12, 0), (45_000, 44_544, 40, 0),
                                  (20_000, 59_392, 30, 0), (32_768, 30_000, 15, 25_000), (5_000, 59_393, 50, 0)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    counts[rng.integers(0, n_row, size=n_row // 9)] = 0
    if hub:
      counts = counts.astype(np.int64)
      counts[n_row // 3] = min(hub, n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_col)
    shape = (n_row, n_col)
    print("shape", shape, dtype.__name__, flush=True)
    w = np.array([0.6], dtype=dtype)
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    for rate in (0.0005, 0.05, 0.9):
      ev = rng.random(n_row) < rate
      if hub:
        ev[n_row // 3] = True
      want = oracle_mod.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True)
      for events in (ev, ev.astype(dtype) * 3):
        for _ in range(2):
          got = bpl.event_csr_matvec(w, indices, indptr, events, shape=shape, transpose=True).cpu().numpy()
          assert np.array_equal(got, want), (shape, rate)  # the reference's repeated additions, bit for bit
      want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
      mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=shape, transpose=True)
      got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
      assert_close_reordered(got, want, mag, dtype, what="event scatter beside the sliced windows %s rate %g" % (shape, rate))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_event_scatter_into_one_window_rows_found_by_the_workgroups(cuda, oracle_mod, dtype):
  # 4,097 to 32,768 rows and at most 8,192 columns: no list, every workgroup numbers the active rows itself
  # (thread by thread, bit by bit).  The row counts at both ends, empty rows among the active ones, no event,
  # every row active, bool and float events (also -0.0 and NaN), both weight kinds (the homogeneous one bit
  # for bit), twice in a row.
  rng = np.random.default_rng(61)
  # Outputs of 7,425 to 14,848 columns are taken in two slices (with one weight in one); wider ones go to the sorted scatter.
  for n_row, n_col, mean in ((4097, 8192, 40), (32_768, 5000, 60), (20_000, 1, 1), (9000, 700, 300), (31_999, 8191, 5),
                             (9000, 7425, 30), (10_000, 14_848, 30), (32_768, 14_849, 20)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    counts[rng.integers(0, n_row, size=n_row // 5)] = 0
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    shape = (n_row, n_col)
    print("shape", shape, dtype.__name__, flush=True)
    for rate in (0.0, 0.002, 0.1, 1.0):
      ev = rng.random(n_row) < rate
      want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
      mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=shape, transpose=True)
      fev = ev.astype(dtype) * 3
      fev[~ev] = -0.0
      if ev.any():
        fev[np.flatnonzero(ev)[0]] = np.nan
      for events in (ev, fev):
        for _ in range(2):
          got = bpl.event_csr_matvec(data, indices, indptr, events, shape=shape, transpose=True).cpu().numpy()
          assert_close_reordered(got, want, mag, dtype, what="event scatter, rows found by the workgroups %s rate %g" % (shape, rate))
      w = np.array([0.6], dtype=dtype)
      want = oracle_mod.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True)
      got = bpl.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
      assert np.array_equal(got, want), (shape, rate)  # the reference's repeated additions, bit for bit


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_event_scatter_of_few_long_rows(cuda, oracle_mod, dtype):
  # fewer active rows than producer workgroups: several producers share a row, each a part of its nonzeros
  # (5 and about 20 active rows of 34,000; with half of the 700 rows active a producer per row and idle ones),
  # rows of unequal length, both weight kinds (the homogeneous one bit for bit), twice in a row
  rng = np.random.default_rng(59)
  n_row, n_col = 700, 60_000
  counts = np.full(n_row, 34_000)
  counts[::7] = 9
  counts[5] = 60_000
  indices, indptr = synth.counted_csr(counts, n_col, seed=3)
  data = rng.standard_normal(indices.shape[0]).astype(dtype)
  shape = (n_row, n_col)
  for active in (5, 20, 350):
    ev = np.zeros(n_row, dtype=bool)
    ev[rng.choice(n_row, size=active, replace=False)] = True
    ev[5] = True
    print("active rows", int(ev.sum()), dtype.__name__, flush=True)
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
    mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=shape, transpose=True)
    for _ in range(2):
      got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
      assert_close_reordered(got, want, mag, dtype, what="event scatter, %d long rows" % active)
    w = np.array([0.6], dtype=dtype)
    want = oracle_mod.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
    assert np.array_equal(got, want), active  # the reference's repeated additions, bit for bit


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_transposed_csr_matvec_one_output_window_flat_walk(cuda, oracle_mod, dtype):
  # outputs of at most 32,768 columns with at least 2^20 nonzeros: every workgroup walks an equal share of the
  # nonzeros into one float64 window of up to 16,384 columns.  Short rows, empty rows (also first and last), one row that holds a
  # third of the nonzeros, more than 1,024 rows per workgroup, the widest and a narrow window, twice in a row.
  rng = np.random.default_rng(47)
  for n_row, n_col, mean, hub in ((400_000, 16_384, 4, 0), (30_000, 16_000, 60, 600_000), (900_000, 700, 2, 0),
                                  (2000, 9000, 800, 0),
                                  # (two windows: every share of the nonzeros is walked once per window)
                                  (150_000, 32_768, 9, 0), (60_000, 16_385, 25, 0)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    counts[0] = counts[-1] = 0
    counts[rng.integers(0, n_row, size=n_row // 7)] = 0
    if hub:
      counts = counts.astype(np.int64)
      counts[n_row // 3] = min(hub, n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    assert indices.shape[0] >= 1 << 20
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    shape = (n_row, n_col)
    print("shape", shape, dtype.__name__, flush=True)
    v = rng.standard_normal(n_row).astype(dtype)
    want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=True)
    mag = oracle_mod.csr_matvec(np.abs(data), indices, indptr, np.abs(v), shape=shape, transpose=True)
    for _ in range(2):
      got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
      assert_close_reordered(got, want, mag, dtype, what="one-window flat walk %s" % (shape,))
    vi = rng.integers(-2, 3, size=n_row).astype(dtype)
    di = rng.integers(-3, 4, size=indices.shape[0]).astype(dtype)
    want = oracle_mod.csr_matvec(di, indices, indptr, vi, shape=shape, transpose=True)
    got = bpl.cusparse_csr_matvec(di, indices, indptr, vi, shape=shape, transpose=True).cpu().numpy()
    assert np.array_equal(got, want)  # small integers: exact in any order
    w = np.array([0.5], dtype=dtype)
    want = oracle_mod.csr_matvec(w, indices, indptr, vi, shape=shape, transpose=True)
    got = bpl.cusparse_csr_matvec(w, indices, indptr, vi, shape=shape, transpose=True).cpu().numpy()
    assert np.array_equal(got, want)  # multiples of 0.5


def test_transposed_csr_matvec_rows_taken_in_chunks(cuda, oracle_mod):
  # float64 pairs of 10 bytes: from 21 million nonzeros on the rows are binned and added in two or more
  # chunks, one after the other over the same scratch memory; uneven rows, so that the chunks differ
  rng = np.random.default_rng(43)
  n_row, n_col = 260_000, 300_000
  counts = rng.poisson(60, size=n_row)
  counts[n_row // 2:] *= 2
  counts[5] = 200_000
  indices, indptr = synth.counted_csr(counts, n_col, seed=3)
  assert indices.shape[0] * 10 > 200 << 20
  data = rng.random(indices.shape[0])
  v = rng.standard_normal(n_row)
  shape = (n_row, n_col)
  want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=True)
  mag = oracle_mod.csr_matvec(data, indices, indptr, np.abs(v), shape=shape, transpose=True)
  for _ in range(2):
    got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
    assert_close_reordered(got, want, mag, np.float64, what="sorted scatter in chunks %s" % (shape,))
  vi = rng.integers(-2, 3, size=n_row).astype(np.float64)
  w = np.array([0.5])
  want = oracle_mod.csr_matvec(w, indices, indptr, vi, shape=shape, transpose=True)
  got = bpl.cusparse_csr_matvec(w, indices, indptr, vi, shape=shape, transpose=True).cpu().numpy()
  assert np.array_equal(got, want)  # multiples of 0.5: exact in any order


def test_full_size_csr_matvec_both_orientations(cuda, oracle_mod):
  # 1,000,000 x 1,000,000, ~1e8 nnz (the transposed product runs the sorted scatter):
  #  * against the oracle on the configuration's own data,
  #  * <u, A v> == <A^T u, v> exactly with small integer data and vectors,
  #  * A^T 1 with unit weight gives the column counts exactly.
  c = synth.config_csr_matvec()
  shape = c["shape"]
  n = shape[0]
  dev = cuda
  data = torch.from_numpy(c["data"]).to(dev)
  indices = torch.from_numpy(c["indices"]).to(dev)
  indptr = torch.from_numpy(c["indptr"]).to(dev)
  vec = torch.from_numpy(c["vector"]).to(dev)
  print("full size csr_matvec", indices.shape[0], flush=True)
  want = oracle_mod.csr_matvec(c["data"], c["indices"], c["indptr"], c["vector"], shape=shape)
  got = bpl.csr_matvec(data, indices, indptr, vec, shape=shape).cpu().numpy()
  assert_close(got, want, what="csr_matvec full size")
  want = oracle_mod.csr_matvec(c["data"], c["indices"], c["indptr"], c["vector"], shape=shape, transpose=True)
  mag = oracle_mod.csr_matvec(c["data"], c["indices"], c["indptr"], np.abs(c["vector"]), shape=shape, transpose=True)
  got = bpl.cusparse_csr_matvec(data, indices, indptr, vec, shape=shape, transpose=True).cpu().numpy()
  assert_close_reordered(got, want, mag, what="csr_matvec transposed full size")
  rng = np.random.default_rng(5)
  di = torch.from_numpy(rng.integers(0, 3, size=indices.shape[0]).astype(np.float32)).to(dev)
  u = torch.from_numpy(rng.integers(-2, 3, size=n).astype(np.float32)).to(dev)
  v = torch.from_numpy(rng.integers(-2, 3, size=n).astype(np.float32)).to(dev)
  Av = bpl.csr_matvec(di, indices, indptr, v, shape=shape)
  ATu = bpl.cusparse_csr_matvec(di, indices, indptr, u, shape=shape, transpose=True)
  lhs = float((Av.double() * u.double()).sum())
  rhs = float((ATu.double() * v.double()).sum())
  assert lhs == rhs and lhs != 0
  ones = torch.ones(n, dtype=torch.float32, device=dev)
  cnt = bpl.cusparse_csr_matvec(torch.ones(1, device=dev), indices, indptr, ones, shape=shape, transpose=True)
  assert np.array_equal(cnt.cpu().numpy(), np.bincount(c["indices"], minlength=n).astype(np.float32))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_scatter_path_boundaries(cuda, oracle_mod, dtype):
  # shapes on both sides of every rule that picks a scatter kernel: 32,768 rows (active-row list),
  # 16,384 / 65,536 / 131,072 columns (one float64 window, four windows), 2^20 nonzeros (sorted
  # scatter), 64 nonzeros per row on average (device-side gate), event and dense input
  rng = np.random.default_rng(51)
  cases = [(32_768, 16_384, 40), (32_769, 16_385, 40), (20_000, 65_536, 60), (20_000, 65_537, 60),
           (9_000, 131_072, 130), (9_000, 131_073, 130), (40_000, 140_000, 63), (40_000, 140_000, 66),
           (3_000, 20_000, 349), (3_000, 20_000, 351), (70_000, 500, 20)]
  for n_row, n_col, mean in cases:
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row + mean)
    data = rng.random(indices.shape[0]).astype(dtype)
    shape = (n_row, n_col)
    print("shape", shape, "nnz", indices.shape[0], dtype.__name__, flush=True)
    ev = rng.random(n_row) < 0.1
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
    assert_close_reordered(got, want, want, dtype, what="event scatter %s" % (shape,))  # data >= 0: want is the bound
    w = np.array([0.3], dtype=dtype)
    want = oracle_mod.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(w, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
    assert_close(got, want, what="homogeneous event scatter %s" % (shape,))
    v = rng.standard_normal(n_row).astype(dtype)
    want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=True)
    mag = oracle_mod.csr_matvec(data, indices, indptr, np.abs(v), shape=shape, transpose=True)
    got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
    assert_close_reordered(got, want, mag, dtype, what="dense scatter %s" % (shape,))


@pytest.mark.parametrize("seed", [1, 2])
def test_random_shapes_all_operators_against_oracle(cuda, oracle_mod, seed):
  # shapes, row lengths (with an occasional very long row), activity, dtypes and event kinds drawn
  # at random over the ranges that select the different kernels; every operator of the family
  # against the oracle
  rng = np.random.default_rng(seed)
  done = 0
  for case in range(60):
    n_row = int(10 ** rng.uniform(0, 5.3))
    n_col = int(10 ** rng.uniform(0, 5.6))
    mean = float(10 ** rng.uniform(-0.5, 2.3))
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    if rng.random() < 0.3:
      counts[rng.integers(0, n_row)] = min(n_col, int(10 ** rng.uniform(2, 4.5)))
    if counts.sum() > 1e7:
      continue
    indices, indptr = synth.counted_csr(counts, n_col, seed=case)
    dtype = np.float32 if rng.random() < 0.7 else np.float64
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    rate = float(rng.choice([0.0, 0.001, 0.02, 0.2, 1.0]))
    shape = (n_row, n_col)
    print("case", case, shape, "mean %.1f" % mean, "nnz", indices.shape[0], "rate", rate, dtype.__name__, flush=True)
    for transpose in (True, False):
      n_in = n_row if transpose else n_col
      ev = rng.random(n_in) < rate
      if rng.random() < 0.3:
        ev = (ev * rng.uniform(0.5, 2, n_in)).astype(dtype)
      for d in (data, np.array([0.75], dtype=dtype)):
        want = oracle_mod.event_csr_matvec(d, indices, indptr, ev, shape=shape, transpose=transpose)
        got = bpl.event_csr_matvec(d, indices, indptr, ev, shape=shape, transpose=transpose).cpu().numpy()
        if d.shape[0] == 1:
          assert np.array_equal(got, want), ("homogeneous weight", shape, transpose)  # the reference's bits
        elif transpose:
          mag = oracle_mod.event_csr_matvec(np.abs(d), indices, indptr, ev, shape=shape, transpose=True)
          assert_close_reordered(got, want, mag, dtype, what="event scatter %s" % (shape,))
        else:
          assert_close(got, want, what="event gather %s" % (shape,))
      v = rng.standard_normal(n_in).astype(dtype)
      want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape, transpose=transpose)
      if transpose:
        got = bpl.cusparse_csr_matvec(data, indices, indptr, v, shape=shape, transpose=True).cpu().numpy()
        mag = oracle_mod.csr_matvec(np.abs(data), indices, indptr, np.abs(v), shape=shape, transpose=True)
        assert_close_reordered(got, want, mag, dtype, what="dense scatter %s" % (shape,))
      else:
        got = bpl.csr_matvec(data, indices, indptr, v, shape=shape).cpu().numpy()
        assert_close(got, want, what="dense gather %s" % (shape,))
    done += 1
  assert done >= 40



@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_csr_matvec_with_the_vector_staged_in_lds(cuda, oracle_mod, dtype):
  # at least 16,384 rows and a vector of at most 159 KB: the kernels gather it from LDS.  Every
  # row-length mode of that path, the largest vector that fits and the first that does not
  # (staged in part), empty rows, heterogeneous and homogeneous weights.
  rng = np.random.default_rng(61)
  limit = (160 * 1024 - 1024) // np.dtype(dtype).itemsize
  for n_row, n_col, mean in ((20_000, 5_000, 30), (17_000, limit, 5), (16_384, limit + 1, 5), (40_000, 3_000, 100),
                             (16_500, 20_000, 400), (30_000, 9_000, 14), (40_000, 1, 1),
                             # up to four times as long: the part that fits is staged, the rest comes from L2
                             (20_000, 100_000, 30), (17_000, 4 * limit, 8), (16_400, 70_000, 450)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    counts[rng.integers(0, n_row, 50)] = 0
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    v = rng.standard_normal(n_col).astype(dtype)
    shape = (n_row, n_col)
    print("shape", shape, flush=True)
    for d in (data, np.array([0.75], dtype=dtype)):
      want = oracle_mod.csr_matvec(d, indices, indptr, v, shape=shape)
      got = bpl.csr_matvec(d, indices, indptr, v, shape=shape).cpu().numpy()
      assert got.dtype == dtype
      assert_close(got, want, what="csr_matvec %s" % (shape,))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_small_event_scatter_in_one_launch(cuda, oracle_mod, dtype):
  # up to 4,096 rows and 8,192 columns one launch does the whole transposed product (every output
  # window's workgroup tests all events and walks all active rows); sizes on both sides of that
  # limit, windows of 1 .. 512 columns, every row active, empty rows, rows of several steps
  rng = np.random.default_rng(31)
  for n_row, n_col, mean, rate in ((4000, 4000, 80, 0.02), (4096, 8192, 20, 1.0), (4097, 8192, 20, 0.3),
                                   (4096, 8193, 20, 0.3), (300, 7, 5, 0.5), (3000, 257, 3, 0.9), (1, 1, 1, 1.0),
                                   (4000, 4097, 700, 0.01), (17, 8000, 3000, 0.5)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row + n_col)
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    ev = rng.random(n_row) < rate
    shape = (n_row, n_col)
    print("shape", shape, dtype.__name__, flush=True)
    want = oracle_mod.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True)
    mag = oracle_mod.event_csr_matvec(np.abs(data), indices, indptr, ev, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(data, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
    assert_close_reordered(got, want, mag, dtype, what="small scatter heter")
    evf = (ev * rng.uniform(0.5, 2.0, n_row)).astype(dtype)
    got = bpl.event_csr_matvec(data, indices, indptr, evf, shape=shape, transpose=True).cpu().numpy()
    assert_close_reordered(got, want, mag, dtype, what="small scatter heter, float events")
    # unit weight: counts, exact; integer weights: exact in any order
    ones = np.array([0.6], dtype=dtype)  # not representable: the sum depends on how it is formed
    want = oracle_mod.event_csr_matvec(ones, indices, indptr, ev, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(ones, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
    assert np.array_equal(got, want)
    di = rng.integers(-2, 3, size=indices.shape[0]).astype(dtype)
    want = oracle_mod.event_csr_matvec(di, indices, indptr, ev, shape=shape, transpose=True)
    got = bpl.event_csr_matvec(di, indices, indptr, ev, shape=shape, transpose=True).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_csr_matvec_with_16_byte_stream_loads(cuda, oracle_mod, dtype):
  # at least 16,384 rows, a vector too long for LDS and 4 nonzeros or more per row on average: the walk
  # that reads four consecutive nonzeros per lane and request.  Means from 30 to 900, means on both sides of
  # its limit (3: the other kernel runs; 4), nnz not a multiple of 4, empty
  # rows, rows of one nonzero, hub rows that go to the whole workgroup, both weight kinds.
  rng = np.random.default_rng(71)
  limit = 4 * (160 * 1024 - 1024) // np.dtype(dtype).itemsize + 1  # first length that is not staged at all
  for n_row, n_col, mean, hubs in ((20_000, limit, 30, 0), (16_384, limit + 3, 60, 2), (17_001, 400_000, 100, 3),
                                   (16_400, 300_000, 250, 1), (16_390, 200_000, 500, 0), (16_385, 170_000, 900, 1),
                                   (40_000, 1_000_000, 23, 0), (30_000, 250_000, 24, 40),
                                   (300_000, 170_000, 3, 0), (280_000, 170_000, 4, 2),
                                   # (a vector of which a part is staged in LDS: that walk from 24 per row on, below it the flat one)
                                   (40_000, 100_000, 9, 0), (30_000, 90_000, 40, 1), (50_000, 60_000, 23, 0)):
    counts = np.minimum(rng.poisson(mean, size=n_row), n_col)
    counts[rng.integers(0, n_row, 50)] = 0
    counts[rng.integers(0, n_row, 50)] = 1
    for h in range(hubs):
      counts[rng.integers(0, n_row)] = min(n_col, (5_000, 70_000, 150_000)[h % 3])
    if counts.sum() % 4 == 0:
      counts[0] += 1
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    data = rng.standard_normal(indices.shape[0]).astype(dtype)
    v = rng.standard_normal(n_col).astype(dtype)
    shape = (n_row, n_col)
    print("shape", shape, "nnz", indices.shape[0], flush=True)
    for d in (data, np.array([0.75], dtype=dtype)):
      want = oracle_mod.csr_matvec(d, indices, indptr, v, shape=shape)
      got = bpl.csr_matvec(d, indices, indptr, v, shape=shape).cpu().numpy()
      assert got.dtype == dtype
      assert_close(got, want, what="csr_matvec %s" % (shape,))
  # operands that do not start on a 16-byte boundary: the 4-byte walks take the call
  dev = torch.device("cuda:0")
  big_i = torch.from_numpy(np.concatenate([[0], indices]).astype(np.int32)).to(dev)[1:]
  big_d = torch.from_numpy(np.concatenate([[0], data]).astype(dtype)).to(dev)[1:]
  assert big_i.data_ptr() % 16 != 0
  got = bpl.csr_matvec(big_d, big_i, indptr, v, shape=shape).cpu().numpy()
  assert_close(got, oracle_mod.csr_matvec(data, indices, indptr, v, shape=shape), what="unaligned operands")


def test_csr_matvec_hub_row_time(cuda):
  # one row with a million nonzeros among 20,000 ordinary ones must not serialise the call: the whole
  # workgroup walks it (a single wave took milliseconds)
  rng = np.random.default_rng(5)
  n_row, n_col = 20_000, 2_000_000
  counts = np.full(n_row, 50)
  counts[777] = 1_000_000
  indices, indptr = synth.counted_csr(counts, n_col, seed=9)
  data = rng.integers(-2, 3, size=indices.shape[0]).astype(np.float32)
  v = rng.integers(-3, 4, size=n_col).astype(np.float32)
  dev = torch.device("cuda:0")
  args = [torch.from_numpy(a).to(dev) for a in (data, indices, indptr, v)]
  got = bpl.csr_matvec(*args, shape=(n_row, n_col))
  # small integers: exact in any order
  rows = np.repeat(np.arange(n_row), counts)
  want = np.bincount(rows, weights=data.astype(np.float64) * v[indices], minlength=n_row)
  assert np.array_equal(got.cpu().numpy().astype(np.float64), want)
  torch.cuda.synchronize()
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  e0.record()
  for _ in range(5):
    bpl.csr_matvec(*args, shape=(n_row, n_col))
  e1.record()
  torch.cuda.synchronize()
  per_call_us = e0.elapsed_time(e1) * 1e3 / 5
  print("hub row of 1e6 nonzeros: %.1f us per call" % per_call_us, flush=True)
  assert per_call_us < 500.0


def test_gather_hub_rows(cuda, oracle_mod):
  # rows that hold a large share of the nonzeros are left to the whole workgroup by every walk of the
  # gather (groups of 4, 8 or 32 lanes per row, a wave per row; LDS bitmap and two-level bitmap; the
  # dense product of matrices too small for its 16-byte walk): exact results on integer data, several
  # hub rows per workgroup, and a bound on the time of a row of a million nonzeros (one wave: 19 ms)
  rng = np.random.default_rng(8)
  cases = [  # n_row, n_col, ordinary rows, {row: nonzeros}
    (100_000, 100_000, 12, {777: 90_000, 778: 5000, 99_999: 2000, 0: 1025}),
    (30_000, 60_000, 30, {5: 50_000, 29_000: 4097}),
    (2000, 50_000, 500, {3: 40_000, 1999: 33_000}),
    (700, 60_000, 34_000, {0: 33_000, 699: 1}),  # every row but one goes to a whole workgroup, dealt one by one
    (20_000, 2_000_000, 50, {777: 1_000_000}),
  ]
  dev = torch.device("cuda:0")
  for n_row, n_col, base, hubs in cases:
    counts = np.full(n_row, base)
    for r, c in hubs.items():
      counts[r] = c
    indices, indptr = synth.counted_csr(counts, n_col, seed=n_row)
    print("case", n_row, n_col, base, hubs, flush=True)
    ev = rng.random(n_col) < 0.3
    for dtype in (np.float32, np.float64):
      data = rng.integers(-2, 3, size=indices.shape[0]).astype(dtype)
      for d in (data, np.array([0.6], dtype=dtype)):
        want = oracle_mod.event_csr_matvec(d, indices, indptr, ev, shape=(n_row, n_col))
        got = bpl.event_csr_matvec(d, indices, indptr, ev, shape=(n_row, n_col)).cpu().numpy()
        assert np.array_equal(got, want), (n_row, dtype.__name__, d.shape, np.flatnonzero(got != want)[:5])
      if n_row <= 30_000 and n_col <= 60_000:  # (dense product through the same kernel)
        v = rng.integers(-3, 4, size=n_col).astype(dtype)
        want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=(n_row, n_col))
        got = bpl.csr_matvec(data, indices, indptr, v, shape=(n_row, n_col)).cpu().numpy()
        assert np.array_equal(got, want), (n_row, dtype.__name__)
  # time of the last case (float32, heterogeneous weights)
  args = [torch.from_numpy(a).to(dev) for a in (data.astype(np.float32), indices, indptr, ev)]
  bpl.event_csr_matvec(*args, shape=(n_row, n_col))
  torch.cuda.synchronize()
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  e0.record()
  for _ in range(5):
    bpl.event_csr_matvec(*args, shape=(n_row, n_col))
  e1.record()
  torch.cuda.synchronize()
  per_call_us = e0.elapsed_time(e1) * 1e3 / 5
  print("event gather with a hub row of 1e6 nonzeros: %.1f us per call" % per_call_us, flush=True)
  assert per_call_us < 3000.0


def _flat_walk_counts(kind, n_row, rng):
  """Row lengths that exercise the flat walk of csr_matvec (mean of 4 or more, 16,384 rows or more)."""
  if kind == "poisson":
    return np.maximum(1, rng.poisson(100, n_row))
  if kind == "even":
    return np.full(n_row, 64)
  if kind == "ragged":  # two thirds of the rows empty, the others long: steps that meet several hundred rows
    c = np.zeros(n_row, dtype=np.int64)
    some = rng.random(n_row) < 0.33
    c[some] = rng.integers(1, 400, size=int(some.sum()))
    return c
  if kind == "empty ends":  # empty rows at both ends and in runs of more than a window of 64
    c = np.maximum(1, rng.poisson(60, n_row))
    c[:300] = 0
    c[-500:] = 0
    c[5000:5200] = 0
    return c
  if kind == "hubs":  # rows across many waves' ranges, next to rows of one nonzero
    c = np.full(n_row, 30)
    c[7] = 150_000
    c[8] = 1
    c[n_row // 2] = 70_000
    c[n_row - 1] = 40_000
    return c
  if kind == "steps":  # rows of exactly one step and of one quad, so that rows end where steps and ranges end
    c = np.full(n_row, 4)
    c[::3] = 1024
    return c
  if kind == "short":  # a mean just above the limit: a step of 1,024 nonzeros meets some 200 rows, four windows of indptr
    return rng.poisson(5, n_row)
  if kind == "ones":  # rows of one nonzero among rows of twelve: quads that meet four rows
    c = np.ones(n_row, dtype=np.int64)
    c[::3] = 12
    return c
  raise ValueError(kind)


@pytest.mark.parametrize("kind", ["poisson", "even", "ragged", "empty ends", "hubs", "steps", "short", "ones"])
def test_csr_matvec_flat_walk_over_the_nonzeros(cuda, oracle_mod, kind):
  # vectors too long for LDS (more than 162,816 elements) and rows of 4 nonzeros or more on average: every wave
  # owns a contiguous range of the nonzeros and tells the rows apart through windows of indptr
  # (csr_flat_gather.hip).  Integer data: every sum is exact in float64, so the result is the oracle's bit for bit.
  rng = np.random.default_rng(len(kind))
  n_row, n_col = 20_011, 170_003
  counts = np.minimum(_flat_walk_counts(kind, n_row, rng), n_col)
  indices, indptr = synth.counted_csr(counts, n_col, seed=3)
  assert indices.shape[0] // n_row >= 4
  for dtype in (np.float32, np.float64):
    data = rng.integers(-3, 4, size=indices.shape[0]).astype(dtype)
    v = rng.integers(-4, 5, size=n_col).astype(dtype)
    for d in (data, np.array([0.75], dtype=dtype)):
      want = oracle_mod.csr_matvec(d, indices, indptr, v, shape=(n_row, n_col))
      got = bpl.csr_matvec(d, indices, indptr, v, shape=(n_row, n_col)).cpu().numpy()
      assert np.array_equal(got, want), (kind, dtype.__name__, d.shape, np.flatnonzero(got != want)[:8])
  # real-valued data: within the tolerance of the gather paths
  data = rng.standard_normal(indices.shape[0]).astype(np.float32)
  v = rng.standard_normal(n_col).astype(np.float32)
  want = oracle_mod.csr_matvec(data, indices, indptr, v, shape=(n_row, n_col))
  got = bpl.csr_matvec(data, indices, indptr, v, shape=(n_row, n_col)).cpu().numpy()
  assert_close(got, want, what="flat walk " + kind)
