"""Pins of the oracle's restatement of the reference's stateless ("hash") jitconn generators and
event kernels (lib/kernel_helpers_random.cuh:12-71, lib/gpu_jitconn_event_matvec.cu:10-51,
138-183, 281-331).  The reference holds them as CUDA only and no file of it holds outputs, so
the pins are what the mathematics fixes."""
import numpy as np
import pytest

# published periods of the component recurrences (L'Ecuyer: taus88, LFSR113)
PERIODS = {(0, 0): 2 ** 31 - 1, (0, 1): 2 ** 29 - 1, (0, 2): 2 ** 28 - 1,
           (1, 0): 2 ** 31 - 1, (1, 1): 2 ** 29 - 1, (1, 2): 2 ** 28 - 1, (1, 3): 2 ** 25 - 1}


@pytest.mark.parametrize("gen,comp", sorted(PERIODS))
def test_component_recurrences_have_their_maximal_period(oracle_mod, gen, comp):
  # a wrong shift or mask constant gives a recurrence whose period is not the maximal one
  want = PERIODS[(gen, comp)]
  assert oracle_mod.lfsr_component_period(gen, comp, 12345 + 200, want + 10) == want


def test_component_steps_are_linear_over_gf2(oracle_mod):
  rng = np.random.default_rng(1)
  for (gen, comp) in PERIODS:
    for a, b in rng.integers(0, 2 ** 32, size=(50, 2), dtype=np.uint64):
      a, b = int(a), int(b)
      f = lambda z: oracle_mod.lfsr_component_step(gen, comp, z)
      assert f(a ^ b) == f(a) ^ f(b)
      assert f(0) == 0


def test_outputs_are_the_xor_of_the_component_steps(oracle_mod):
  # lfsr113: state seed + {1, 7, 15, 127}; taus88: seed + {1, 7, 15}, second output one step on
  m = 0xffffffff
  for seed in (0, 1, 12345, 0xfffffff0, 0xdeadbeef):
    z = [oracle_mod.lfsr_component_step(1, i, (seed + a) & m) for i, a in enumerate((1, 7, 15, 127))]
    assert oracle_mod.lfsr113_word(seed) == z[0] ^ z[1] ^ z[2] ^ z[3]
    s = [oracle_mod.lfsr_component_step(0, i, (seed + a) & m) for i, a in enumerate((1, 7, 15))]
    s2 = [oracle_mod.lfsr_component_step(0, i, s[i]) for i in range(3)]
    assert oracle_mod.taus88_words(seed) == [s[0] ^ s[1] ^ s[2], s2[0] ^ s2[1] ^ s2[2]]


def test_generators_are_uniform_over_random_seeds(oracle_mod):
  rng = np.random.default_rng(0)
  seeds = rng.integers(0, 2 ** 32, size=40000, dtype=np.uint64)
  w = np.array([oracle_mod.lfsr113_word(int(s)) for s in seeds], dtype=np.float64) / 2 ** 32
  n = w.size
  assert abs(w.mean() - 0.5) < 4 * (1 / np.sqrt(12)) / np.sqrt(n)
  for p in (0.01, 0.1, 0.5):
    assert abs((w < p).mean() - p) < 4 * np.sqrt(p * (1 - p) / n)
  t = np.array([oracle_mod.taus88_words(int(s)) for s in seeds], dtype=np.float64) / 2 ** 32
  assert np.all(np.abs(t.mean(0) - 0.5) < 4 * (1 / np.sqrt(12)) / np.sqrt(n))
  z = np.sqrt(-2 * np.log(t[:, 0])) * np.cos(2 * np.pi * t[:, 1])  # Box-Muller of the two outputs
  assert abs(z.mean()) < 4 / np.sqrt(n) and abs(z.std() - 1) < 0.02


def test_event_matvec_hash_closed_forms_and_structure(oracle_mod):
  rng = np.random.default_rng(2)
  n_row, n_col = 37, 500
  ev = rng.random(n_col) < 0.3
  ids, num = oracle_mod.event_info(ev)
  num = int(np.asarray(num).reshape(-1)[0])
  kw = dict(seed=0x9e3779b9, n_row=n_row, n_col=n_col)
  for dtype in (np.float32, np.float64):
    assert np.all(oracle_mod.event_matvec_hash(ids, num, prob=0.0, dtype=dtype, **kw) == 0)
    full = oracle_mod.event_matvec_hash(ids, num, prob=1.0, dtype=dtype, **kw)
    assert np.all(full == num) and full.dtype == dtype
    # uniform weights with zero range: count * w_min
    cnt = oracle_mod.event_matvec_hash(ids, num, prob=0.2, dtype=dtype, **kw)
    flat = oracle_mod.event_matvec_hash(ids, num, w_kind="uniform", w_a=0.25, w_b=0.0, prob=0.2, dtype=dtype, **kw)
    assert np.array_equal(flat, cnt * 0.25)
  # the count of a row is the number of listed columns whose hash word is below prob * 2^32
  cnt = oracle_mod.event_matvec_hash(ids, num, prob=0.2, dtype=np.float64, **kw)
  for row in (0, 5, 36):
    want = sum(oracle_mod.lfsr113_word((kw["seed"] + n_col * row + int(c)) & 0xffffffff) * 2.0 ** -32 < 0.2
               for c in ids[:num])
    assert cnt[row] == want
  # only the first event_num entries of the list count
  half = oracle_mod.event_matvec_hash(ids, num // 2, prob=1.0, **kw)
  assert np.all(half == num // 2)
  # weights: sum over a row == sum of the per-synapse formula
  got = oracle_mod.event_matvec_hash(ids, num, w_kind="uniform", w_a=-1.0, w_b=3.0, prob=0.5, dtype=np.float64, **kw)
  row = 3
  acc = 0.0
  for c in ids[:num]:
    s = (kw["seed"] + n_col * row + int(c)) & 0xffffffff
    if oracle_mod.lfsr113_word(s) * 2.0 ** -32 < 0.5:
      acc += oracle_mod.taus88_words(s)[0] * 2.0 ** -32 * 3.0 - 1.0
  assert abs(got[row] - acc) <= 1e-12 * max(1.0, abs(acc))
