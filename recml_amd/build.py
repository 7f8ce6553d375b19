"""Builds the HIP shared library for gfx950 in-tree (recml_amd/lib/)."""

from __future__ import annotations

import os
import shutil
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_HERE)
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libhstu_attn.so")
SOURCES = [os.path.join(_HERE, "csrc", "hstu_attn.hip")]
INCLUDE = os.path.join(ROOT, "include")

# -packed-fp32-ops is switched off for the device pass: packed fp32
# instructions are not wanted in these kernels.  The host pass does not know
# the feature and says so; that warning is harmless.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc() -> str:
  exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
  if not os.path.exists(exe):
    raise RuntimeError("hipcc not found; the HIP library cannot be built")
  return exe


def build_library(verbose: bool = False) -> str:
  """Compiles every HIP source into recml_amd/lib/libhstu_attn.so."""
  os.makedirs(LIB_DIR, exist_ok=True)
  tmp = LIB_PATH + ".tmp"
  cmd = [hipcc(), *HIPCC_FLAGS, "-I", INCLUDE, "-o", tmp, *SOURCES]
  res = subprocess.run(cmd, capture_output=True, text=True)
  if res.returncode != 0:
    raise RuntimeError("hipcc failed:\n" + res.stdout + res.stderr)
  if verbose:
    print(res.stderr)
  os.replace(tmp, LIB_PATH)
  return LIB_PATH


if __name__ == "__main__":
  print(build_library(verbose=True))
