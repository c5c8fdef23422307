"""Differentiation rules of the operators (the reference's JVP / transpose rules,
event_csr_matvec.py:439-463, cusparse_matvec.py:281-308, jitconn event_matvec.py:242-273),
checked against torch's own autograd through the equivalent dense float64 product on the CPU."""
import numpy as np
import pytest
import torch
import torch.autograd.forward_ad as fwAD

import brainpylib_amd as bpl
from util import random_csr

pytestmark = pytest.mark.gpu
SHAPES = [(60, 90), (90, 60), (200, 200)]


def _dense(data, indices, indptr, shape):
  """Differentiable dense float64 matrix on the CPU."""
  counts = np.diff(indptr)
  row = torch.from_numpy(np.repeat(np.arange(shape[0]), counts))
  col = torch.from_numpy(indices.astype(np.int64))
  vals = data if data.shape[0] > 1 else data.expand(col.shape[0])
  return torch.zeros(shape, dtype=torch.float64).index_put((row, col), vals, accumulate=True)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("homo", [False, True])
def test_event_csr_matvec_gradients(cuda, shape, transpose, homo):
  data_np, indices, indptr = random_csr(shape, 0.3, seed=shape[0] + 13, dtype=np.float64)
  if homo:
    data_np = np.array([0.8])
  rng = np.random.default_rng(2)
  n_in = shape[0] if transpose else shape[1]
  n_out = shape[1] if transpose else shape[0]
  ev_np = (rng.random(n_in) < 0.3) * rng.uniform(0.5, 2.0, n_in)
  ct_np = rng.standard_normal(n_out)
  # reference gradients: dense product with the events as a 0/1 vector for the weights ...
  d_ref = torch.tensor(data_np, requires_grad=True)
  M = _dense(d_ref, indices, indptr, shape)
  M = M.T if transpose else M
  (M @ torch.tensor((ev_np != 0).astype(np.float64)) @ torch.tensor(ct_np)).backward()
  # ... and the product that is linear in the events for the events (the rule's own definition)
  e_ref = torch.tensor(ev_np, requires_grad=True)
  (M.detach() @ e_ref @ torch.tensor(ct_np)).backward()

  data = torch.tensor(data_np, device="cuda", requires_grad=True)
  # weights: boolean events
  out = bpl.event_csr_matvec(data, indices, indptr, ev_np != 0, shape=shape, transpose=transpose)
  out.backward(torch.tensor(ct_np, device="cuda"))
  if homo:
    torch.testing.assert_close(data.grad.cpu(), d_ref.grad, rtol=1e-10, atol=1e-10)
  else:
    torch.testing.assert_close(data.grad.cpu(), d_ref.grad, rtol=1e-12, atol=1e-12)
  # events: float events carry a gradient
  events = torch.tensor(ev_np, device="cuda", requires_grad=True)
  out = bpl.event_csr_matvec(data.detach(), indices, indptr, events, shape=shape, transpose=transpose)
  out.backward(torch.tensor(ct_np, device="cuda"))
  torch.testing.assert_close(events.grad.cpu(), e_ref.grad, rtol=1e-10, atol=1e-10)
  # forward mode: tangents of weights and events together
  d_dot, e_dot = rng.standard_normal(data_np.shape), rng.standard_normal(n_in)
  with fwAD.dual_level():
    dd = fwAD.make_dual(data.detach(), torch.tensor(d_dot, device="cuda"))
    ee = fwAD.make_dual(events.detach(), torch.tensor(e_dot, device="cuda"))
    tangent = fwAD.unpack_dual(bpl.event_csr_matvec(dd, indices, indptr, ee, shape=shape, transpose=transpose)).tangent
  Md = _dense(torch.tensor(d_dot), indices, indptr, shape)
  Md = Md.T if transpose else Md
  want = Md @ torch.tensor((ev_np != 0).astype(np.float64)) + M.detach() @ torch.tensor(e_dot)
  torch.testing.assert_close(tangent.cpu(), want, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("homo", [False, True])
def test_csr_matvec_gradients(cuda, shape, transpose, homo):
  data_np, indices, indptr = random_csr(shape, 0.3, seed=shape[0] + 17, dtype=np.float64, weights="uniform")
  if homo:
    data_np = np.array([0.8])
  rng = np.random.default_rng(3)
  n_in = shape[0] if transpose else shape[1]
  n_out = shape[1] if transpose else shape[0]
  v_np, ct_np = rng.standard_normal(n_in), rng.standard_normal(n_out)
  d_ref = torch.tensor(data_np, requires_grad=True)
  v_ref = torch.tensor(v_np, requires_grad=True)
  M = _dense(d_ref, indices, indptr, shape)
  M = M.T if transpose else M
  (M @ v_ref @ torch.tensor(ct_np)).backward()
  data = torch.tensor(data_np, device="cuda", requires_grad=True)
  vec = torch.tensor(v_np, device="cuda", requires_grad=True)
  out = bpl.cusparse_csr_matvec(data, indices, indptr, vec, shape=shape, transpose=transpose)
  out.backward(torch.tensor(ct_np, device="cuda"))
  torch.testing.assert_close(data.grad.cpu(), d_ref.grad, rtol=1e-10, atol=1e-10)
  torch.testing.assert_close(vec.grad.cpu(), v_ref.grad, rtol=1e-10, atol=1e-10)
  d_dot, v_dot = rng.standard_normal(data_np.shape), rng.standard_normal(n_in)
  with fwAD.dual_level():
    dd = fwAD.make_dual(data.detach(), torch.tensor(d_dot, device="cuda"))
    vv = fwAD.make_dual(vec.detach(), torch.tensor(v_dot, device="cuda"))
    tangent = fwAD.unpack_dual(bpl.cusparse_csr_matvec(dd, indices, indptr, vv, shape=shape, transpose=transpose)).tangent
  Md = _dense(torch.tensor(d_dot), indices, indptr, shape)
  Md = Md.T if transpose else Md
  want = Md @ torch.tensor(v_np) + M.detach() @ torch.tensor(v_dot)
  torch.testing.assert_close(tangent.cpu(), want, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("kind", ["homo", "uniform", "normal"])
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("outdim_parallel", [False, True])
def test_jitconn_matvec_gradients(cuda, oracle_mod, kind, transpose, outdim_parallel):
  # the implicit matrix, made explicit column by column with unit vectors through the oracle
  shape = (70, 50)
  kw = dict(conn_prob=0.2, shape=shape, seed=99, transpose=transpose, outdim_parallel=outdim_parallel)
  n_in = shape[0] if transpose else shape[1]
  n_out = shape[1] if transpose else shape[0]
  if kind == "homo":
    call = lambda v: bpl.matvec_prob_conn_homo_weight(v, 1.5, **kw)
  elif kind == "uniform":
    call = lambda v: bpl.matvec_prob_conn_uniform_weight(v, w_low=-1.0, w_high=2.0, **kw)
  else:
    call = lambda v: bpl.matvec_prob_conn_normal_weight(v, w_mu=0.5, w_sigma=2.0, **kw)
  eye = torch.eye(n_in, dtype=torch.float64, device="cuda")
  M = torch.stack([call(eye[i]) for i in range(n_in)], dim=1)  # (n_out, n_in)
  rng = np.random.default_rng(4)
  v = torch.tensor(rng.standard_normal(n_in), device="cuda", requires_grad=True)
  ct = torch.tensor(rng.standard_normal(n_out), device="cuda")
  out = call(v)
  torch.testing.assert_close(out.detach(), M @ v.detach(), rtol=1e-10, atol=1e-10)
  out.backward(ct)
  torch.testing.assert_close(v.grad, M.T @ ct, rtol=1e-10, atol=1e-10)
  v_dot = torch.tensor(rng.standard_normal(n_in), device="cuda")
  with fwAD.dual_level():
    tangent = fwAD.unpack_dual(call(fwAD.make_dual(v.detach(), v_dot))).tangent
  torch.testing.assert_close(tangent, M @ v_dot, rtol=1e-10, atol=1e-10)
  # event operator with float events: same matrix applied to the 0/1 vector; gradient as above
  if kind == "homo":
    ecall = lambda e: bpl.event_matvec_prob_conn_homo_weight(e, 1.5, **kw)
  elif kind == "uniform":
    ecall = lambda e: bpl.event_matvec_prob_conn_uniform_weight(e, w_low=-1.0, w_high=2.0, **kw)
  else:
    ecall = lambda e: bpl.event_matvec_prob_conn_normal_weight(e, w_mu=0.5, w_sigma=2.0, **kw)
  ev = torch.tensor((rng.random(n_in) < 0.3) * rng.uniform(0.5, 2.0, n_in), device="cuda", requires_grad=True)
  out = ecall(ev)
  torch.testing.assert_close(out.detach(), M @ (ev.detach() != 0).double(), rtol=1e-10, atol=1e-10)
  out.backward(ct)
  torch.testing.assert_close(ev.grad, M.T @ ct, rtol=1e-10, atol=1e-10)


def test_homogeneous_jitconn_weight_gradient(cuda):
  w = torch.tensor(0.7, device="cuda", requires_grad=True)
  ev = np.random.default_rng(5).random(300) < 0.2
  out = bpl.event_matvec_prob_conn_homo_weight(ev, w, conn_prob=0.1, shape=(200, 300), seed=3)
  out.sum().backward()
  counts = bpl.event_matvec_prob_conn_homo_weight(ev, 1.0, conn_prob=0.1, shape=(200, 300), seed=3)
  torch.testing.assert_close(w.grad, counts.sum())


def test_csr_coo_utilities(cuda):
  data, indices, indptr = random_csr((40, 30), 0.3, seed=5)
  row, col = bpl.csr_to_coo(indices, indptr)
  assert np.array_equal(row.numpy(), np.repeat(np.arange(40), np.diff(indptr)))
  assert np.array_equal(col.numpy(), indices)
  perm = np.random.default_rng(6).permutation(indices.shape[0])
  ix, ip = bpl.coo_to_csr(row.numpy()[perm], indices[perm], num_row=40)
  assert np.array_equal(ip.numpy(), indptr)
  for r in range(40):  # same entries per row, in the order the COO arrays listed them
    assert np.array_equal(ix.numpy()[ip[r]:ip[r + 1]], indices[perm][row.numpy()[perm] == r])
  dense = bpl.csr_to_dense(data, indices, indptr, shape=(40, 30)).numpy()
  want = np.zeros((40, 30), np.float32)
  want[row.numpy(), indices] = data
  assert np.array_equal(dense, want)
