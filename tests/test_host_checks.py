"""Argument checking of the host-side operator wrappers (same conditions as the reference's
wrappers; no GPU needed: the checks run before a device is touched)."""
import numpy as np
import pytest
import torch

import brainpylib_amd as bpl

IDX = np.zeros(6, dtype=np.int32)
PTR = np.zeros(5, dtype=np.int32)  # shape[0] = 4


def test_event_csr_matvec_checks():
  # brainpylib/_src/event_ops/event_csr_matvec.py:75-99
  ev4, ev7 = np.zeros(4, bool), np.zeros(7, bool)
  with pytest.raises(ValueError, match="size of data"):
    bpl.event_csr_matvec(np.zeros(3, np.float32), IDX, PTR, ev7, shape=(4, 7))
  with pytest.raises(ValueError, match="scalar or 1D"):
    bpl.event_csr_matvec(np.zeros((2, 3), np.float32), IDX, PTR, ev7, shape=(4, 7))
  with pytest.raises(ValueError, match="indices should be a 1D vector with int32 or uint32"):
    bpl.event_csr_matvec(1.0, IDX.astype(np.int64), PTR, ev7, shape=(4, 7))
  with pytest.raises(ValueError, match="indptr should be a 1D vector with int32 or uint32"):
    bpl.event_csr_matvec(1.0, IDX, PTR.astype(np.int64), ev7, shape=(4, 7))
  with pytest.raises(ValueError, match="events should be a 1D"):
    bpl.event_csr_matvec(1.0, IDX, PTR, np.zeros((7, 1), bool), shape=(4, 7))
  with pytest.raises(ValueError, match="length-2"):
    bpl.event_csr_matvec(1.0, IDX, PTR, ev7, shape=(4, 7, 1))
  with pytest.raises(ValueError, match=r"Shape mismatch, mat \(4, 7\) @ vec \(4,\)"):
    bpl.event_csr_matvec(1.0, IDX, PTR, ev4, shape=(4, 7))
  with pytest.raises(ValueError, match=r"Shape mismatch, vec \(7,\) @ mat \(4, 7\)"):
    bpl.event_csr_matvec(1.0, IDX, PTR, ev7, shape=(4, 7), transpose=True)
  with pytest.raises(ValueError, match="events should be bool or have the dtype of data"):
    bpl.event_csr_matvec(np.zeros(6, np.float32), IDX, PTR, np.zeros(7, np.float64), shape=(4, 7))


def test_csr_matvec_checks():
  # brainpylib/_src/sparse_ops/sparse_csr_matvec.py:70-82
  v = np.zeros(7, np.float32)
  with pytest.raises(ValueError, match="Only support methods"):
    bpl.csr_matvec(1.0, IDX, PTR, v, shape=(4, 7), method="fast")
  with pytest.raises(TypeError, match="Only support float32 and float64"):
    bpl.csr_matvec(np.zeros(6, np.int32), IDX, PTR, v, shape=(4, 7))
  with pytest.raises(TypeError, match="types of data and vector"):
    bpl.csr_matvec(np.zeros(6, np.float64), IDX, PTR, v, shape=(4, 7))
  with pytest.raises(ValueError, match="Shape mismatch"):
    bpl.csr_matvec(np.zeros(6, np.float32), IDX, PTR, np.zeros(4, np.float32), shape=(4, 7))


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-device error")
def test_no_cpu_fallback():
  with pytest.raises(RuntimeError, match="no CPU path"):
    bpl.event_csr_matvec(1.0, IDX, PTR, np.zeros(7, bool), shape=(4, 7))
  with pytest.raises(RuntimeError, match="no CPU path"):
    bpl.csr_matvec(1.0, IDX, PTR, np.zeros(7, np.float32), shape=(4, 7))


def test_check_csr_accepts_a_matrix_and_names_what_is_wrong_with_the_others():
  # the operators trust their index arrays as the reference's kernels do; this is the opt-in pass over them
  idx = np.array([0, 6, 2, 2, 5, 1], dtype=np.int32)
  ptr = np.array([0, 2, 2, 5, 6], dtype=np.int32)
  bpl.check_csr(idx, ptr, shape=(4, 7))
  bpl.check_csr(idx.astype(np.uint32), ptr.astype(np.uint32), shape=(4, 7))
  bpl.check_csr(np.zeros(0, np.int32), np.zeros(5, np.int32), shape=(4, 7))
  with pytest.raises(ValueError, match=r"indices should lie in \[0, 6\)"):
    bpl.check_csr(idx, ptr, shape=(4, 6))
  with pytest.raises(ValueError, match="indices should lie"):
    bpl.check_csr(np.array([0, -1, 2, 2, 5, 1], dtype=np.int32), ptr, shape=(4, 7))
  with pytest.raises(ValueError, match="indices should lie"):
    bpl.check_csr(np.array([0, 2 ** 31 + 3, 2, 2, 5, 1], dtype=np.uint32), ptr, shape=(4, 7))
  with pytest.raises(ValueError, match="never decrease"):
    bpl.check_csr(idx, np.array([0, 3, 2, 5, 6], dtype=np.int32), shape=(4, 7))
  with pytest.raises(ValueError, match="end at len"):
    bpl.check_csr(idx, np.array([0, 2, 2, 5, 7], dtype=np.int32), shape=(4, 7))
  with pytest.raises(ValueError, match="start at 0"):
    bpl.check_csr(idx, np.array([1, 2, 2, 5, 6], dtype=np.int32), shape=(4, 7))
  with pytest.raises(ValueError, match="shape\\[0\\] \\+ 1 = 4 entries"):
    bpl.check_csr(idx, ptr, shape=(3, 7))
  with pytest.raises(ValueError, match="int32 or uint32"):
    bpl.check_csr(idx.astype(np.int64), ptr, shape=(4, 7))


def test_python_scalars_are_kept_by_bit_pattern():
  # 0.0 and -0.0 compare equal and NaN does not equal itself: the host copies of Python numbers are
  # looked up by the value's bits
  import math
  from brainpylib_amd import _tensors
  a, b = _tensors.as_tensor(0.0), _tensors.as_tensor(-0.0)
  assert not math.copysign(1.0, a.item()) < 0 and math.copysign(1.0, b.item()) < 0
  assert _tensors.as_tensor(-0.0) is b and _tensors.as_tensor(0.0) is a
  n1, n2 = _tensors.as_tensor(float("nan")), _tensors.as_tensor(float("nan"))
  assert n1 is n2 and math.isnan(n1.item())
  assert _tensors.as_tensor(True).dtype == torch.bool and _tensors.as_tensor(1).dtype == torch.float32
