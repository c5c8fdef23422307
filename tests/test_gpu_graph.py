"""The custom calls can be captured into a HIP graph (no memset nodes, no allocation once the
scratch buffers are warm) and every replay reproduces the eager result."""
import numpy as np
import pytest
import torch

import brainpylib_amd as bpl
from brainpylib_amd import synth

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
