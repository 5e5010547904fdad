"""Build recipe for libparrot_hip.so (hipcc, gfx950 only).

Run ``python -m parrotserve_amd.build`` or call ``build()``; the shared library
lands next to the sources' package (parrotserve_amd/libparrot_hip.so) so it
travels with the tree.  ``python -m parrotserve_amd.build --timeline`` also links the
profiling variant (libparrot_hip_timeline.so, what ``bench.py --timeline`` loads).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libparrot_hip.so")
# profiling variant: the same sources with the fused decode kernel's timeline marks switched on (csrc/timeline.hpp)
TIMELINE_LIB_PATH = os.path.join(PKG_DIR, "libparrot_hip_timeline.so")
SOURCES = ["move_tokens.hip", "gather_blocked.hip", "norm_rope.hip", "fused.hip", "sampler.hip", "tables.hip", "decode.hip", "prefix_mfma.hip", "attention_api.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    # packed-fp32 forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# The matrix-core kernels never produce NaNs from finite inputs (masked scores are -inf and every
# difference of two infinities is guarded), so their max trees may drop the NaN-quieting of each input.
EXTRA_FLAGS = {"prefix_mfma.hip": ["-fno-honor-nans"]}


def _compile(src: str, obj_dir: str, timeline: bool = False) -> str:
    obj = os.path.join(obj_dir, src.replace(".hip", ".timeline.o" if timeline else ".o"))
    extra = ["-include", os.path.join(CSRC, "timeline.hpp")] if timeline else []
    cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS.get(src, []), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    return obj


def build(verbose: bool = True, timeline: bool = False) -> str:
    """Compile and link the product library; ``timeline=True`` also links the profiling variant."""
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB_PATH}")
    if not timeline:
        return LIB_PATH
    # the profiling variant shares every object but the one that holds the marks
    tl_obj = _compile("prefix_mfma.hip", obj_dir, timeline=True)
    tl_objs = [tl_obj if o.endswith("prefix_mfma.o") else o for o in objs]
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", TIMELINE_LIB_PATH, *tl_objs],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {TIMELINE_LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build(timeline="--timeline" in sys.argv[1:])
    sys.exit(0)
