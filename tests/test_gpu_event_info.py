"""GPU parity of event_info (the nonzero_* targets) against the ordered CPU oracle."""
import numpy as np
import pytest
import torch

import brainpylib_amd as bpl

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [np.bool_, np.int32, np.int64, np.float32, np.float64])
@pytest.mark.parametrize("size", [1, 63, 64, 1000, 1024, 1025, 100_000, 1_500_000])
def test_event_info_matches_oracle(cuda, oracle_mod, dtype, size):
  rng = np.random.default_rng(size)
  ev = ((rng.random(size) < 0.1) * rng.integers(1, 5, size)).astype(dtype)
  want_ids, want_num = oracle_mod.event_info(ev)
  ids, num = bpl.event_info(ev)
  assert ids.dtype == torch.int32 and num.dtype == torch.int32 and num.shape == (1,)
  assert np.array_equal(num.cpu().numpy(), want_num)
  assert np.array_equal(ids.cpu().numpy(), want_ids)
  # the reference's own check: event_num == sum(events != 0)
  # (brainpylib/_src/event_ops/tests/test_event_info_collection.py:39-40)
  assert int(num[0]) == int((ev != 0).sum())


def test_event_info_edges_and_batch(cuda, oracle_mod):
  for ev in (np.zeros(5000, bool), np.ones(5000, bool)):
    ids, num = bpl.event_info(ev)
    w_ids, w_num = oracle_mod.event_info(ev)
    assert np.array_equal(ids.cpu().numpy(), w_ids) and np.array_equal(num.cpu().numpy(), w_num)
  ev = np.random.default_rng(0).random((7, 3000)) < 0.2
  ids, num = bpl.event_info(ev)
  for b in range(7):
    w_ids, w_num = oracle_mod.event_info(ev[b])
    assert np.array_equal(ids[b].cpu().numpy(), w_ids) and int(num[b]) == int(w_num[0])


def test_event_info_with_more_batch_rows_than_a_grid_dimension(cuda, oracle_mod):
  # 65,600 rows of two tiles: more than the 65,535 a grid takes in its second dimension, taken in two passes
  ev = np.random.default_rng(2).random((65_600, 4100)) < 0.01
  ids, num = bpl.event_info(ev)
  num = num.cpu().numpy()
  assert np.array_equal(num.reshape(-1), ev.sum(axis=1))
  for b in (0, 65_534, 65_535, 65_536, 65_599):
    w_ids, w_num = oracle_mod.event_info(ev[b])
    assert np.array_equal(ids[b].cpu().numpy(), w_ids) and int(num[b]) == int(w_num[0])
  del ids


@pytest.mark.parametrize("size", [1, 37, 64, 65, 1000, 4096])
def test_event_info_of_many_short_rows(cuda, oracle_mod, size):
  # at least 64 rows of at most one tile: a wave per row
  ev = np.random.default_rng(size).random((70_000 if size == 37 else 300, size)) < 0.3
  ids, num = bpl.event_info(ev)
  ids, num = ids.cpu().numpy(), num.cpu().numpy()
  want_num = ev.sum(axis=1)
  assert np.array_equal(num.reshape(-1), want_num)
  for b in (0, 1, ev.shape[0] // 2, ev.shape[0] - 1):
    w_ids, w_num = oracle_mod.event_info(ev[b])
    assert np.array_equal(ids[b], w_ids) and int(num[b]) == int(w_num[0])
  # every row: its events in increasing order, then -1
  order = np.where(ev, np.arange(size), size + np.arange(size))
  want = np.sort(order, axis=1)
  want = np.where(want < size, want, -1)
  assert np.array_equal(ids, want)
  evf = np.where(ev, np.float32(-0.5), np.float32(0))  # float events: nonzero means event
  ids_f, num_f = bpl.event_info(evf)
  assert np.array_equal(ids_f.cpu().numpy(), want) and np.array_equal(num_f.cpu().numpy().reshape(-1), want_num)


@pytest.mark.parametrize("dtype", [np.bool_, np.float32])
def test_event_info_tiles_alignment_and_density(cuda, oracle_mod, dtype):
  # several 4,096-element tiles per row, rows that start at every alignment (one-byte events take a
  # 16-byte vector path only where the tile start is aligned), event densities from empty to full
  rng = np.random.default_rng(3)
  for size in (4095, 4096, 4097, 12_301, 65_536):
    for rate in (0.0, 0.03, 0.5, 1.0):
      ev = (rng.random((5, size)) < rate).astype(dtype)
      ids, num = bpl.event_info(ev)
      for b in range(5):
        w_ids, w_num = oracle_mod.event_info(ev[b])
        assert np.array_equal(ids[b].cpu().numpy(), w_ids), (size, rate, b)
        assert int(num[b]) == int(w_num[0])
  # a vector that starts 3 bytes into an allocation
  base = torch.from_numpy(rng.random(20_003) < 0.2).cuda()
  ids, num = bpl.event_info(base[3:])
  w_ids, w_num = oracle_mod.event_info(base[3:].cpu().numpy())
  assert np.array_equal(ids.cpu().numpy(), w_ids) and int(num[0]) == int(w_num[0])
