"""Argument plumbing shared by the operator wrappers: everything becomes a contiguous torch
CUDA tensor (device memory is PyTorch-ROCm's; nothing is computed with torch)."""
import struct

import numpy as np
import torch

FLOAT_DTYPES = (torch.float32, torch.float64)
_INDEX_DTYPES = (torch.int32, torch.uint32)


_PY_SCALARS = {}  # host tensors of Python numbers seen as operands (read-only)


def as_tensor(a):
  """Unwraps brainpy-like arrays (objects with `.value`) and wraps numpy / python data as a torch
  tensor WITHOUT moving it, so that argument checks can run before a device is needed.
  Python floats become float32 (the reference's default float)."""
  if hasattr(a, "value") and not isinstance(a, (torch.Tensor, np.ndarray)):
    a = a.value
  if isinstance(a, torch.Tensor):
    return a
  if isinstance(a, (bool, int, float)):
    # keyed by the value's bits, so that 0.0 and -0.0 are two entries and a NaN finds its own
    key = (type(a), struct.pack("<d", a) if isinstance(a, float) else a)
    t = _PY_SCALARS.get(key)
    if t is None:
      if len(_PY_SCALARS) >= 256:
        _PY_SCALARS.clear()
      t = _PY_SCALARS[key] = torch.tensor(a, dtype=torch.bool if isinstance(a, bool) else torch.float32)
    return t
  arr = np.asarray(a)
  if arr.dtype == np.uint32:
    return torch.from_numpy(np.ascontiguousarray(arr).view(np.int32)).view(torch.uint32)
  if arr.ndim == 0:
    return torch.tensor(arr.item(), dtype=_np_to_torch(arr.dtype))
  return torch.from_numpy(np.ascontiguousarray(arr))


def device_of(*args):
  """The device the call runs on: that of the first CUDA tensor argument, else the current one."""
  for a in args:
    if isinstance(a, torch.Tensor) and a.is_cuda:
      return a.device
  if not torch.cuda.is_available():
    raise RuntimeError("brainpylib_amd needs a HIP device: there is no CPU path in this package.")
  return torch.device("cuda", torch.cuda.current_device())


_HOST_SCALARS = {}


def to_device(t, device):
  if t.device != device:
    if t.numel() == 1 and t.device.type == 'cpu' and not t.requires_grad:
      # A one-element host operand (a homogeneous weight given as a Python number): its device copy
      # is made once per value.  A pageable host-to-device copy per call would cost more than the
      # kernels of a small network.  The operators only read their operands.
      key = (t.numpy().tobytes(), t.dtype, tuple(t.shape), device)  # (the bits: -0.0 is not 0.0, NaN equals itself)
      hit = _HOST_SCALARS.get(key)
      if hit is None:
        if len(_HOST_SCALARS) >= 256:
          _HOST_SCALARS.clear()
        hit = _HOST_SCALARS[key] = t.to(device).contiguous()
      return hit
    t = t.to(device)
  return t.contiguous()


def _np_to_torch(dt):
  return {np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64,
          np.dtype(np.int32): torch.int32, np.dtype(np.int64): torch.int64,
          np.dtype(np.bool_): torch.bool, np.dtype(np.uint8): torch.uint8}.get(np.dtype(dt), torch.float32)


def is_index_dtype(dt):
  return dt in _INDEX_DTYPES
