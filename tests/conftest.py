import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)


def pytest_configure(config):
  config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_mod():
  import oracle
  oracle.lib()
  return oracle


@pytest.fixture(scope="session")
def ref_mod():
  from oracle import ref
  if not ref.available():
    pytest.skip("oracle/_ref/libref_cpu.so was not built (the reference tree is not mounted here)")
  return ref


@pytest.fixture(scope="session")
def cuda():
  import torch
  if not torch.cuda.is_available():
    pytest.skip("no HIP device")
  return torch.device("cuda:0")
