"""GPU parity of the stateless ("hash") jitconn event targets gpu_event_matvec_prob_{homo,uniform,
normal}_{float,double} against the CPU oracle, through the C ABI.  Connectivity and homogeneous
counts: exact.  Uniform weights: the same double arithmetic in the same order, exact in float64
and after rounding in float32.  Normal weights: device log / cos / sqrt differ from glibc's in the
last bits, rel 1e-5 / abs 1e-6 per output scaled by the number of addends."""
import numpy as np
import pytest
import torch

import brainpylib_amd as bpl
from brainpylib_amd import _lib

pytestmark = pytest.mark.gpu


def _call(ids, num, w_kind, a, b, prob, seed, n_row, n_col, dtype):
  """The custom-call target itself, on device tensors."""
  if w_kind == "homo":
    opaque = _lib.build_jitconn_prob_homo_descriptor(n_row, n_col, seed, prob)
  elif w_kind == "uniform":
    opaque = _lib.build_jitconn_prob_uniform_descriptor(n_row, n_col, seed, prob, a, b)
  else:
    opaque = _lib.build_jitconn_prob_normal_descriptor(n_row, n_col, seed, prob, a, b)
  tdt = torch.float32 if dtype == np.float32 else torch.float64
  out = torch.full((n_row,), float("nan"), dtype=tdt, device=ids.device)
  name = "gpu_event_matvec_prob_%s_%s" % (w_kind, "float" if dtype == np.float32 else "double")
  _lib.custom_call(name, [ids, num, out], opaque)
  return out.cpu().numpy()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n_row,n_col,rate", [(300, 257, 0.5), (1000, 5000, 0.3), (20, 3000, 1.0), (700, 40, 0.0)])
def test_hash_targets_against_oracle(cuda, oracle_mod, dtype, n_row, n_col, rate):
  rng = np.random.default_rng(n_row + n_col)
  ev = rng.random(n_col) < rate
  ids_h, num_h = oracle_mod.event_info(ev)
  ids = torch.from_numpy(ids_h).to(cuda)
  num = torch.from_numpy(np.asarray(num_h, dtype=np.int32).reshape(1)).to(cuda)
  for seed in (0, 12345, 0x9e3779b9, 0xfffffff0):  # (the last one wraps around 2^32)
    for prob in (0.02, 0.3):
      print("case", n_row, n_col, rate, dtype.__name__, seed, prob, flush=True)
      kw = dict(prob=prob, seed=seed, n_row=n_row, n_col=n_col)
      want = oracle_mod.event_matvec_hash(ids_h, int(np.asarray(num_h).reshape(-1)[0]), dtype=dtype, **kw)
      got = _call(ids, num, "homo", 0.0, 0.0, dtype=dtype, **kw)
      assert got.dtype == dtype and np.array_equal(got, want)
      want = oracle_mod.event_matvec_hash(ids_h, int(np.asarray(num_h).reshape(-1)[0]), w_kind="uniform", w_a=-0.5, w_b=2.0, dtype=dtype, **kw)
      got = _call(ids, num, "uniform", -0.5, 2.0, dtype=dtype, **kw)
      assert np.array_equal(got, want)
      cnt = oracle_mod.event_matvec_hash(ids_h, int(np.asarray(num_h).reshape(-1)[0]), dtype=np.float64, **kw)
      want = oracle_mod.event_matvec_hash(ids_h, int(np.asarray(num_h).reshape(-1)[0]), w_kind="normal", w_a=0.25, w_b=1.5, dtype=dtype, **kw)
      got = _call(ids, num, "normal", 0.25, 1.5, dtype=dtype, **kw)
      eps = np.finfo(dtype).eps
      bound = 1e-6 + 1e-5 * np.abs(want) + 8 * eps * cnt * (0.25 + 1.5 * 6)  # + rounding of the running sum
      # (small seeds make taus88 return 0: log(0) gives infinite weights, there as here)
      fin = np.isfinite(want)
      assert np.array_equal(np.isfinite(got), fin)
      assert np.array_equal(got[~fin], want[~fin], equal_nan=True)
      assert np.all(np.abs(got[fin].astype(np.float64) - want[fin]) <= bound[fin])


def test_hash_targets_edges(cuda, oracle_mod):
  n_row, n_col = 130, 600
  rng = np.random.default_rng(3)
  ev = rng.random(n_col) < 0.4
  ids_h, num_h = oracle_mod.event_info(ev)
  ids = torch.from_numpy(ids_h).to(cuda)
  n = int(np.asarray(num_h).reshape(-1)[0])
  for num_v, prob, want in ((n, 1.0, n), (n, 2.0, n), (n, 0.0, 0), (n, -1.0, 0), (0, 0.5, 0), (n // 3, 1.0, n // 3),
                            (-5, 1.0, 0), (10 ** 6, 1.0, n_col)):
    num = torch.tensor([num_v], dtype=torch.int32, device=cuda)
    # (a count beyond the list is cut to its length: the list holds n_col entries, -1 behind the events)
    got = _call(ids, num, "homo", 0.0, 0.0, prob=prob, seed=99, n_row=n_row, n_col=n_col, dtype=np.float32)
    if num_v > n:
      continue  # entries behind the events are -1: not an input the operator is defined for
    assert np.all(got == want), (num_v, prob)
  # more than one LDS tile of events
  n_col = 5000
  ids_h = np.arange(n_col, dtype=np.int32)
  ids = torch.from_numpy(ids_h).to(cuda)
  num = torch.tensor([n_col], dtype=torch.int32, device=cuda)
  kw = dict(prob=0.1, seed=0xabcdef12, n_row=77, n_col=n_col)
  want = oracle_mod.event_matvec_hash(ids_h, n_col, w_kind="uniform", w_a=0.0, w_b=1.0, dtype=np.float64, **kw)
  got = _call(ids, num, "uniform", 0.0, 1.0, dtype=np.float64, **kw)
  assert np.array_equal(got, want)


def test_hash_wrapper(cuda, oracle_mod):
  shape = (400, 900)
  rng = np.random.default_rng(4)
  for transpose in (False, True):
    n_row, n_col = (shape[1], shape[0]) if transpose else shape
    ev = rng.random(n_col) < 0.2
    ids_h, num_h = oracle_mod.event_info(ev)
    want = oracle_mod.event_matvec_hash(ids_h, int(np.asarray(num_h).reshape(-1)[0]), prob=0.05, seed=4242, n_row=n_row, n_col=n_col)
    got = bpl.event_matvec_prob_conn_hashed(ev, weight=0.5, conn_prob=0.05, shape=shape, seed=4242, transpose=transpose)
    assert got.shape == (n_row,) and np.array_equal(got.cpu().numpy(), want * np.float32(0.5))
    evf = torch.from_numpy(ev.astype(np.float32)).to(cuda)  # float events: same positions
    got = bpl.event_matvec_prob_conn_hashed(evf, w_kind="uniform", w_low=1.0, w_high=3.0, conn_prob=0.05, shape=shape,
                                            seed=4242, transpose=transpose, dtype=torch.float64)
    want = oracle_mod.event_matvec_hash(ids_h, int(np.asarray(num_h).reshape(-1)[0]), w_kind="uniform", w_a=1.0, w_b=2.0, prob=0.05, seed=4242,
                                        n_row=n_row, n_col=n_col, dtype=np.float64)
    assert np.array_equal(got.cpu().numpy(), want)
  with pytest.raises(ValueError):
    bpl.event_matvec_prob_conn_hashed(np.zeros(5, dtype=bool), conn_prob=0.1, shape=shape, seed=1)
