"""Build recipe of libbrainpylib_amd.so (and the pybind11 `gpu_ops` module): plain hipcc for
gfx950, objects and libraries written in-tree next to the package.

    python -m brainpylib_amd.build            # build what is out of date
    python -m brainpylib_amd.build --force    # rebuild everything
"""
import concurrent.futures
import glob
import os
import subprocess
import sys
import sysconfig

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libbrainpylib_amd.so")
PYMOD_PATH = os.path.join(_HERE, "gpu_ops" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))

ARCH = "gfx950"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: the compiler must not form v_pk_*_f32 from ordinary float code.
# -ffp-contract=off: the jitconn generators must round exactly where the CPU path rounds.
HIP_FLAGS = [
  "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
  "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
  "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-pass-failed",
]


def _run(cmd):
  r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
  out = "\n".join(l for l in r.stdout.splitlines()
                  if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
  if r.returncode != 0:
    raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
  if out.strip():
    print(out)


def _newer(target, deps):
  if not os.path.exists(target):
    return True
  t = os.path.getmtime(target)
  return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True, jobs=8):
  os.makedirs(LIB_DIR, exist_ok=True)
  headers = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(_HERE, "..", "include", "*.h"))
  sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
  objs = []
  todo = []
  for src in sources:
    obj = os.path.join(LIB_DIR, os.path.basename(src)[:-4] + ".o")
    objs.append(obj)
    if force or _newer(obj, [src] + headers):
      todo.append([HIPCC] + HIP_FLAGS + ["-c", src, "-o", obj])
  if todo:
    if verbose:
      print("brainpylib_amd.build: compiling %d HIP source(s) for %s" % (len(todo), ARCH))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(jobs, len(todo))) as ex:
      list(ex.map(_run, todo))
  if force or todo or _newer(LIB_PATH, objs):
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB_PATH] + objs)
    if verbose:
      print("brainpylib_amd.build: linked", LIB_PATH)
  # pybind11 module `gpu_ops`: registrations() + build_*_descriptor(), as lib/gpu_ops.cc exports
  pysrc = os.path.join(CSRC, "gpu_ops_module.cc")
  if os.path.exists(pysrc) and (force or _newer(PYMOD_PATH, [pysrc, LIB_PATH] + headers)):
    import pybind11
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
          "-I" + pybind11.get_include(), "-I" + sysconfig.get_paths()["include"],
          pysrc, "-o", PYMOD_PATH, "-L" + LIB_DIR, "-lbrainpylib_amd", "-Wl,-rpath,$ORIGIN/lib"])
    if verbose:
      print("brainpylib_amd.build: built", PYMOD_PATH)
  return LIB_PATH


if __name__ == "__main__":
  build(force="--force" in sys.argv)
