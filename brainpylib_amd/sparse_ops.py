"""Sparse CSR operators (host side).

Mirrors brainpylib/sparse_ops.py for the part on the hot path: ``csr_matvec`` with the reference's
signature and checks (brainpylib/_src/sparse_ops/sparse_csr_matvec.py:26-98), lowered to the
custom-call targets its GPU translations name (:129-210), and ``cusparse_csr_matvec``'s signature
(brainpylib/_src/sparse_ops/cusparse_matvec.py:31-94) for the transposed product, which the
reference hands to cuSPARSE and this package computes with its own scatter kernel.
"""
from typing import Tuple

import torch

from . import _lib
from ._tensors import FLOAT_DTYPES, as_tensor, device_of, is_index_dtype, to_device

__all__ = ["csr_matvec", "cusparse_csr_matvec"]


def _prepare(data, indices, indptr, vector):
  data = as_tensor(data)
  if data.ndim == 0:
    data = data.reshape(1)
  return data, as_tensor(indices), as_tensor(indptr), as_tensor(vector)


def _move(*tensors):
  device = device_of(*tensors)
  return (device,) + tuple(to_device(t, device) for t in tensors)


def _check(data, indices, indptr, vector, shape):
  if data.dtype not in FLOAT_DTYPES:
    raise TypeError(f'Only support float32 and float64. But we got {data.dtype}.')
  if data.dtype != vector.dtype:
    raise TypeError('The types of data and vector should be the same. '
                    f'But we got {data.dtype} != {vector.dtype}.')
  assert data.ndim == indices.ndim == indptr.ndim == vector.ndim == 1
  if not (is_index_dtype(indices.dtype) and is_index_dtype(indptr.dtype)):
    raise ValueError('indices and indptr should be 1D vectors with int32 or uint32 type.')
  if data.shape[0] not in [1, indices.shape[0]]:
    raise ValueError('The size of data should be 1 or be consistent with indices.')
  if len(shape) != 2:
    raise ValueError('shape should be a length-2 tuple.')
  if indptr.shape[0] != shape[0] + 1:
    raise ValueError(f'indptr should have shape[0] + 1 = {shape[0] + 1} entries, got {indptr.shape[0]}.')


def csr_matvec(data, indices, indptr, vector, *, shape: Tuple[int, int], method: str = 'vector'):
  """CSR sparse matrix times dense vector: ``y[shape[0]] = A @ vector``.

  ``method`` is one of 'scalar', 'vector', 'adaptive' and selects the custom-call target name as in
  the reference; on this device all three run the same kernel family, which picks the number
  of lanes per row from the mean row length."""
  if method not in ['scalar', 'vector', 'adaptive']:
    raise ValueError('Only support methods: scalar, vector, and adaptive. '
                     f'But we got {method}.')
  data, indices, indptr, vector = _prepare(data, indices, indptr, vector)
  _check(data, indices, indptr, vector, shape)
  if vector.shape[0] != shape[1]:
    raise ValueError(f'Shape mismatch, mat {shape} @ vec ({vector.shape[0]},).')
  device, data, indices, indptr, vector = _move(data, indices, indptr, vector)
  type_name = 'float' if data.dtype == torch.float32 else 'double'
  data_name = 'homo' if data.shape[0] == 1 else 'heter'
  opaque = _lib.build_double_size_descriptor(shape[0], shape[1])
  out = torch.empty(shape[0], dtype=data.dtype, device=device)
  if method == 'adaptive':
    # the reference's adaptive target takes a `row_blocks` operand before the vector
    # (lib/gpu_csr_matvec.cu:519-521); it is not read by this implementation.
    row_blocks = torch.zeros(1, dtype=torch.int32, device=device)
    buffers = [data, indices, indptr, row_blocks, vector, out]
  else:
    buffers = [data, indices, indptr, vector, out]
  _lib.custom_call('csr_matvec_' + data_name + '_' + method + '_' + type_name, buffers, opaque)
  return out


def cusparse_csr_matvec(data, indices, indptr, vector, *, shape: Tuple[int, int], transpose: bool = False):
  """``A @ vector`` (transpose=False) or ``A.T @ vector`` (transpose=True) for a CSR matrix."""
  if not transpose:
    return csr_matvec(data, indices, indptr, vector, shape=shape)
  data, indices, indptr, vector = _prepare(data, indices, indptr, vector)
  _check(data, indices, indptr, vector, shape)
  if vector.shape[0] != shape[0]:
    raise ValueError(f'Shape mismatch, vec ({vector.shape[0]},) @ mat {shape}.')
  device, data, indices, indptr, vector = _move(data, indices, indptr, vector)
  type_name = 'float' if data.dtype == torch.float32 else 'double'
  data_name = 'homo' if data.shape[0] == 1 else 'heter'
  opaque = _lib.build_double_size_descriptor(shape[0], shape[1])
  out = torch.empty(shape[1], dtype=data.dtype, device=device)
  _lib.custom_call('csr_matvec_transpose_' + data_name + '_' + type_name,
                   [data, indices, indptr, vector, out], opaque)
  return out
