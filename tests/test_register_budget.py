"""Register budgets of the kernels that are meant to run two 1,024-thread workgroups per CU.

Eight waves per SIMD fit only while a wave holds at most 64 vector and at most 80 scalar registers
(measured on MI355X: with 81..96 scalar registers a 16-wave workgroup is alone on its CU although
the compiler still reports occupancy 8).  A kernel's allocation is the maximum over its branches,
so an unrelated edit can push a kernel over either line and cost a quarter of its speed without
any test of its results noticing.  This compiles the sources to assembly (device side only, no GPU
needed) and reads the counts from the code object metadata."""
import concurrent.futures
import os
import re
import subprocess

import pytest

from brainpylib_amd import build

SOURCES = ["csr_ops.hip", "csr_bin_scatter.hip", "jitconn_ops.hip"]
VGPR_MAX, SGPR_MAX = 64, 80

# (pattern on the demangled name, why it needs eight waves per SIMD)
TWO_PER_CU = [
  (r"csr_gather_kernel<\w+, [\w:]+, (true|false), 0, 1>", "event gather with the bitmap in LDS (the headline kernel)"),
  (r"csr_gather_kernel<float, float, (true|false), 1, 1>", "csr_matvec with the vector staged in LDS, float"),
  (r"csr_scatter_window_kernel<", "event scatter into LDS windows"),
  (r"bin_active_rows_kernel<", "producer of the sorted event scatter"),
  (r"jitconn_rowwalk_kernel<\w+, bpl::PackedBits, 0, \d, 2, (true|false)>", "jitconn row walk with the two-level bitmap"),
  (r"jitconn_rowwalk_kernel<float, [\w: ]+, \d, 2, \d, (true|false)>", "jitconn row walk, float normal weights"),
  (r"jitconn_colwalk_bins_kernel<float,", "jitconn column walk into bins, float"),
]


def _assembly(src, out_dir):
  out = os.path.join(out_dir, src[:-4] + ".s")
  flags = [f for f in build.HIP_FLAGS if f not in ("-fPIC", "-Wall")]
  cmd = [build.HIPCC] + flags + ["-S", "--cuda-device-only", "-I" + os.path.join(os.path.dirname(build.CSRC), "..", "include"),
                                 os.path.join(build.CSRC, src), "-o", out]
  r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
  assert r.returncode == 0, r.stdout[-2000:]
  return open(out).read()


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
  if not os.path.exists(build.HIPCC):
    pytest.skip("no hipcc")
  out_dir = str(tmp_path_factory.mktemp("asm"))
  with concurrent.futures.ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
    texts = list(ex.map(lambda s: _assembly(s, out_dir), SOURCES))
  found = {}
  pat = re.compile(r"\.name:\s+(\S+)\n(?:.*\n)*?\s+\.sgpr_count:\s+(\d+)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)\n\s+\.vgpr_spill_count:\s+(\d+)")
  for text in texts:
    for m in pat.finditer(text[text.index("amdhsa.kernels"):]):
      found[m.group(1)] = (int(m.group(2)), int(m.group(3)), int(m.group(4)))
  names = sorted(found)
  plain = subprocess.run(["c++filt"] + names, stdout=subprocess.PIPE, text=True, check=True).stdout.splitlines()
  return {p.replace("(anonymous namespace)::", ""): found[n] for n, p in zip(names, plain)}


def test_kernels_meant_to_share_a_cu_fit_twice(kernels):
  assert len(kernels) > 100
  over = []
  for pattern, why in TWO_PER_CU:
    hits = [k for k in kernels if re.search(pattern, k)]
    assert hits, "no kernel matches %s" % pattern
    for k in hits:
      sgpr, vgpr, _ = kernels[k]
      if sgpr > SGPR_MAX or vgpr > VGPR_MAX:
        over.append("%s: %d scalar, %d vector registers (%s)" % (k.split("(")[0], sgpr, vgpr, why))
  assert not over, "\n".join(over)


def test_no_kernel_spills_vector_registers_unexpectedly(kernels):
  # scratch-memory spills are tolerated only where the eight-wave budget was chosen knowingly, by exact
  # instantiation and with a cap on the count: double normal weights behind the two-level bitmap
  # (2 registers; 4 with the generators seeded inside the kernel)
  allowed = {"jitconn_rowwalk_kernel<double, bpl::PackedBits, 0, 2, 2, false>": 4,
             "jitconn_rowwalk_kernel<double, bpl::PackedBits, 0, 2, 2, true>": 8}
  spilled = []
  for k, (_, _, spill) in kernels.items():
    name = k.split("(")[0].replace("void ", "").replace("bpl::jitconn", "jitconn").strip()
    if spill and spill > allowed.get(name, 0):
      spilled.append("%s: %d" % (name, spill))
  assert not spilled, spilled
