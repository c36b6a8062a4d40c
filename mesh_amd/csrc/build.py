"""Builds libmesh_moe_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: python -m mesh_amd.csrc.build   (or build_library() from Python)
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["abi.hip", "route.hip", "dispatch.hip", "ffn.hip", "backward.hip",
           "expert_choice.hip", "ntlb.hip", "summaries.hip", "block.hip",
           "attention.hip"]
LIB_NAME = "libmesh_moe_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off",  # one rounding per written operation, as in the spec
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _compile(src):
  obj = os.path.join(HERE, "build", src.replace(".hip", ".o"))
  cmd = [HIPCC] + FLAGS + ["-c", os.path.join(HERE, src), "-o", obj]
  subprocess.run(cmd, check=True, cwd=HERE)
  return obj


def build_library(verbose=True):
  """Compiles every kernel source and links the shared library in-tree."""
  os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
  with ThreadPoolExecutor(max_workers=6) as pool:
    objs = list(pool.map(_compile, SOURCES))
  cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH]
  subprocess.run(cmd + objs, check=True, cwd=HERE)
  if verbose:
    print("built", LIB_PATH)
  return LIB_PATH


if __name__ == "__main__":
  build_library()
  sys.exit(0)
