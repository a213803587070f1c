"""Builder and loader of the mixer-kernel library (`_mixops.so`).

The fp32-residual / delta-rule / linear-scan / attention kernels
(csrc/resid32.hip, csrc/delta_rule.hip, csrc/gated_delta.hip,
csrc/linear_scan.hip, csrc/talk_attention.hip, csrc/mixer_prep.hip,
csrc/mfma_attention.hip, csrc/moe_route.hip) expose a plain C ABI, so the
library needs hipcc only: no torch headers, seconds-to-minutes to build, and
a fresh checkout can compile just these files on first use without building
the large `_C` extension. Launchers receive raw device pointers and the
current HIP stream; shape checks live in the Python wrappers
(production_stack_amd/ops/__init__.py).
"""

from __future__ import annotations

import ctypes
import os
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROOT = os.path.dirname(PKG)
LIB_PATH = os.path.join(PKG, "_mixops.so")

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    # packed-fp32 instruction forms stay off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

# (source, extra defines): the delta-rule file is compiled once per element
# type so its many head-size instantiations build in parallel
UNITS = [
    ("resid32.hip", []),
    ("talk_attention.hip", []),
    ("delta_rule.hip", ["-DMX_ONLY_DTYPE=0"]),
    ("delta_rule.hip", ["-DMX_ONLY_DTYPE=1"]),
    ("mixer_prep.hip", []),
    ("mfma_attention.hip", []),
    ("moe_route.hip", []),
    ("gated_delta.hip", ["-DMX_ONLY_DTYPE=0"]),
    ("gated_delta.hip", ["-DMX_ONLY_DTYPE=1"]),
    # one unit per (decay law, element type)
    *[("linear_scan.hip", [f"-DLS_ONLY={i}"]) for i in range(6)],
]

_lib = None


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: cannot build _mixops.so")
    return exe


def build(force: bool = False) -> str:
    """Compile the library in-tree (atomic replace). Returns its path."""
    if os.path.exists(LIB_PATH) and not force:
        return LIB_PATH
    hipcc = _hipcc()
    src_dir = os.path.join(ROOT, "csrc")
    tmp = tempfile.mkdtemp(prefix="mixops-", dir=PKG)
    try:
        def compile_one(i_unit):
            i, (src, defs) = i_unit
            obj = os.path.join(tmp, f"u{i}.o")
            cmd = [hipcc, *HIPCC_FLAGS, *defs, "-I", src_dir, "-c",
                   os.path.join(src_dir, src), "-o", obj]
            r = subprocess.run(cmd, stdout=subprocess.PIPE,
                               stderr=subprocess.STDOUT, text=True)
            if r.returncode != 0:
                raise RuntimeError(
                    f"hipcc failed on {src}:\n{r.stdout[-4000:]}")
            return obj

        with ThreadPoolExecutor(max_workers=len(UNITS)) as ex:
            objs = list(ex.map(compile_one, enumerate(UNITS)))
        out = os.path.join(tmp, "lib.so")
        r = subprocess.run(
            [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *objs,
             "-o", out],
            stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout[-4000:]}")
        os.replace(out, LIB_PATH)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return LIB_PATH


def load():
    """ctypes handle of the library; builds it when nothing is built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        lib = ctypes.CDLL(LIB_PATH)
        for name in ("mx_delta_rule", "mx_talk_attention",
                     "mx_gated_delta", "mx_short_conv_silu",
                     "mx_mfma_attention", "mx_linear_scan",
                     "mx_linear_scan_splits",
                     "mx_moe_route"):
            getattr(lib, name).restype = ctypes.c_int
        for name in ("mx_embed_scale", "mx_add_rms_norm32",
                     "mx_add_group_norm32", "mx_group_norm_shift",
                     "mx_depth_mix", "mx_gated_act", "mx_kv_append",
                     "mx_attn_prep", "mx_latent_prep", "mx_norm_sum32",
                     "mx_moe_combine",
                     "mx_post_norm_add_norm32"):
            getattr(lib, name).restype = None
        _lib = lib
    return _lib


def available() -> bool:
    return os.path.exists(LIB_PATH)
