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


def pytest_terminal_summary(terminalreporter):
  # how many elements passed a reordered-sum comparison only through the reordering term
  # (4 eps sum|addends| beyond rel 1e-5 / abs 1e-6), per comparison label
  try:
    import util
  except ImportError:
    return
  stats = getattr(util, "REORDER_STATS", {})
  if not stats:
    return
  checked = sum(v[0] for v in stats.values())
  outside = sum(v[1] for v in stats.values())
  terminalreporter.write_line("reordered-sum comparisons: %d elements checked, %d outside plain rel 1e-5 / abs 1e-6 "
                              "(passed through the reordering term)" % (checked, outside))
  for what, (n, k) in sorted(stats.items()):
    if k:
      terminalreporter.write_line("  %-60s %d of %d" % (what[:60], k, n))
