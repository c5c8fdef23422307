"""The custom calls can be captured into a HIP graph (no memset nodes, no allocation once the
scratch buffers are warm) and every replay reproduces the eager result."""
import numpy as np
import pytest
import torch

import brainpylib_amd as bpl
import benchdata as synth

pytestmark = pytest.mark.gpu


def _replay_check(fn, make_inputs, n_replays=4):
  out_eager = fn().clone()
  torch.cuda.synchronize()
  g = torch.cuda.CUDAGraph()
  s = torch.cuda.Stream()
  s.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(s):
    fn()  # warm the scratch buffers of this stream before capture
  torch.cuda.synchronize()
  with torch.cuda.graph(g, stream=s):
    out_graph = fn()
  for i in range(n_replays):
    make_inputs(i)          # eager work between replays: new inputs in the captured buffers
    want = fn().clone()     # eager result for these inputs
    torch.cuda.synchronize()
    out_graph.zero_()
    g.replay()
    torch.cuda.synchronize()
    assert torch.allclose(out_graph, want, rtol=1e-5, atol=1e-6), i
  return out_eager


def test_event_csr_matvec_graph_replays(cuda):
  c = synth.config_event_csr_small()
  d = {k: torch.from_numpy(v).to(cuda) for k, v in c.items() if isinstance(v, np.ndarray)}
  rng = np.random.default_rng(0)

  def new_events(i):
    d["events"].copy_(torch.from_numpy(rng.random(c["shape"][0]) < 0.02 * (i + 1)).to(cuda))

  for transpose in (True, False):
    _replay_check(lambda: bpl.event_csr_matvec(d["data"], d["indices"], d["indptr"], d["events"], shape=c["shape"],
                                               transpose=transpose), new_events)


def test_jitconn_graph_replays(cuda):
  n = 20000
  ev = torch.zeros(n, dtype=torch.bool, device=cuda)
  rng = np.random.default_rng(1)

  def new_events(i):
    ev.copy_(torch.from_numpy(rng.random(n) < 0.05).to(cuda))

  new_events(0)
  for odp in (True, False):
    _replay_check(lambda: bpl.event_matvec_prob_conn_homo_weight(ev, 0.5, conn_prob=0.01, shape=(n, n), seed=3,
                                                                 outdim_parallel=odp), new_events)


def test_sorted_event_scatter_and_two_level_walk_graph_replays(cuda):
  # the multi-kernel paths that pass counters and lists from kernel to kernel: the sorted event
  # scatter (more than 8,192 outputs), its batched form, and the row walk with a two-level bitmap
  rng = np.random.default_rng(2)
  n_row, n_col = 30_000, 50_000
  indices, indptr = synth.counted_csr(rng.poisson(40, size=n_row), n_col, seed=5)
  data = torch.from_numpy(rng.standard_normal(indices.shape[0]).astype(np.float32)).to(cuda)
  ix, ip = torch.from_numpy(indices).to(cuda), torch.from_numpy(indptr).to(cuda)
  ev = torch.zeros(n_row, dtype=torch.bool, device=cuda)
  evb = torch.zeros((5, n_row), dtype=torch.bool, device=cuda)

  def new_events(i):
    ev.copy_(torch.from_numpy(rng.random(n_row) < 0.03 * (i + 1)).to(cuda))
    evb.copy_(torch.from_numpy(rng.random((5, n_row)) < 0.03 * (i + 1)).to(cuda))

  new_events(0)
  _replay_check(lambda: bpl.event_csr_matvec(data, ix, ip, ev, shape=(n_row, n_col), transpose=True), new_events)
  _replay_check(lambda: bpl.event_csr_matvec_batching(data[None], ix[None], ip[None], evb, batch_size=5,
                                                      shape=(n_row, n_col), transpose=True), new_events)
  n_in = 400_000
  evj = torch.zeros(n_in, dtype=torch.bool, device=cuda)

  def new_inputs(i):
    evj.copy_(torch.from_numpy(rng.random(n_in) < 0.02 * (i + 1)).to(cuda))

  new_inputs(0)
  _replay_check(lambda: bpl.event_matvec_prob_conn_homo_weight(evj, 0.5, conn_prob=0.001, shape=(500, n_in), seed=9),
                new_inputs)
