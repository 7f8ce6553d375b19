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
# the block-side steps live in a library of their own: they bring hipBLASLt along, the attention does not
BLOCK_LIB_PATH = os.path.join(LIB_DIR, "libhstu_block.so")
BLOCK_SOURCES = [os.path.join(_HERE, "csrc", "hstu_block.hip")]
BLOCK_LINK = ["-lhipblaslt"]
INCLUDE = os.path.join(ROOT, "include")
# the block's microbenchmark: a stand-alone program (its own main), evidence for what bounds the kernel
MICRO_PATH = os.path.join(LIB_DIR, "micro_fwd_stream")
MICRO_SOURCES = [os.path.join(_HERE, "csrc", "micro_fwd_stream.hip")]

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


def _compile(sources, out, link=(), verbose=False) -> str:
  os.makedirs(LIB_DIR, exist_ok=True)
  tmp = out + ".tmp"
  cmd = [hipcc(), *HIPCC_FLAGS, "-I", INCLUDE, "-o", tmp, *sources, *link]
  res = subprocess.run(cmd, capture_output=True, text=True)
  if res.returncode != 0:
    raise RuntimeError("hipcc failed:\n" + res.stdout + res.stderr)
  if verbose:
    print(res.stderr)
  os.replace(tmp, out)
  return out


def build_library(verbose: bool = False) -> str:
  """Compiles the attention kernels into recml_amd/lib/libhstu_attn.so."""
  return _compile(SOURCES, LIB_PATH, verbose=verbose)


def build_block_library(verbose: bool = False) -> str:
  """Compiles the block-side steps into recml_amd/lib/libhstu_block.so."""
  return _compile(BLOCK_SOURCES, BLOCK_LIB_PATH, BLOCK_LINK, verbose=verbose)


def build_microbench(verbose: bool = False) -> str:
  """Compiles the forward block's microbenchmark into recml_amd/lib/micro_fwd_stream (an executable)."""
  os.makedirs(LIB_DIR, exist_ok=True)
  tmp = MICRO_PATH + ".tmp"
  flags = [f for f in HIPCC_FLAGS if f not in ("-fPIC", "-shared")]
  cmd = [hipcc(), *flags, "-o", tmp, *MICRO_SOURCES]
  res = subprocess.run(cmd, capture_output=True, text=True)
  if res.returncode != 0:
    raise RuntimeError("hipcc failed:\n" + res.stdout + res.stderr)
  if verbose:
    print(res.stderr)
  os.replace(tmp, MICRO_PATH)
  return MICRO_PATH


if __name__ == "__main__":
  print(build_library(verbose=True))
  print(build_block_library(verbose=True))
  print(build_microbench(verbose=True))
