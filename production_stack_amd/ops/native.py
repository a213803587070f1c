"""Builder and loader of the mixer-kernel libraries (`_mixops*.so`).

The fp32-residual / delta-rule / linear-scan / attention kernels expose a
plain C ABI, so the libraries need hipcc only: no torch headers,
seconds-to-minutes to build, and a fresh checkout compiles on first use just
the group of files a model's ops live in, without building the large `_C`
extension. Launchers receive raw device pointers and the current HIP stream;
shape checks live in the Python wrappers
(production_stack_amd/ops/__init__.py).

Groups (one shared library each):
  core    resid32, norm_conv, mixer_prep, talk_attention, mfma_attention,
          moe_route, mingru_scan            -> _mixops.so
  delta   delta_rule                        -> _mixops_delta.so
  gdelta  gated_delta                       -> _mixops_gdelta.so
  scan    linear_scan                       -> _mixops_scan.so
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

# group -> [(source, extra defines)]: the recurrence files are compiled once
# per element type (or decay law) so their many head-size instantiations
# build in parallel
GROUPS = {
    "core": [
        ("resid32.hip", []),
        ("norm_conv.hip", []),
        ("talk_attention.hip", []),
        ("mixer_prep.hip", []),
        ("mfma_attention.hip", []),
        ("moe_route.hip", []),
        ("mingru_scan.hip", []),
    ],
    "delta": [
        ("delta_rule.hip", ["-DMX_ONLY_DTYPE=0"]),
        ("delta_rule.hip", ["-DMX_ONLY_DTYPE=1"]),
    ],
    "gdelta": [
        ("gated_delta.hip", ["-DMX_ONLY_DTYPE=0"]),
        ("gated_delta.hip", ["-DMX_ONLY_DTYPE=1"]),
    ],
    # one unit per (decay law, element type)
    "scan": [("linear_scan.hip", [f"-DLS_ONLY={i}"]) for i in range(6)],
}

LIB_PATHS = {
    "core": LIB_PATH,
    "delta": os.path.join(PKG, "_mixops_delta.so"),
    "gdelta": os.path.join(PKG, "_mixops_gdelta.so"),
    "scan": os.path.join(PKG, "_mixops_scan.so"),
}

# entry points outside the core group
SYMBOL_GROUP = {
    "mx_delta_rule": "delta",
    "mx_gated_delta": "gdelta",
    "mx_linear_scan": "scan",
    "mx_linear_scan_splits": "scan",
}

# entry points that return a status (the others return nothing)
INT_RESULT = {
    "mx_delta_rule", "mx_talk_attention", "mx_gated_delta",
    "mx_short_conv_silu", "mx_mfma_attention", "mx_linear_scan",
    "mx_linear_scan_splits", "mx_norm_conv32", "mx_moe_route",
}

# entry points that return a 64-bit count
LONG_RESULT = {"mx_mingru_scratch"}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: cannot build the mixer kernels")
    return exe


def _build_group(group: str) -> str:
    hipcc = _hipcc()
    src_dir = os.path.join(ROOT, "csrc")
    units = GROUPS[group]
    tmp = tempfile.mkdtemp(prefix=f"mixops-{group}-", dir=PKG)
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

        with ThreadPoolExecutor(max_workers=len(units)) as ex:
            objs = list(ex.map(compile_one, enumerate(units)))
        out = os.path.join(tmp, "lib.so")
        r = subprocess.run(
            [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *objs,
             "-o", out],
            stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout[-4000:]}")
        os.replace(out, LIB_PATHS[group])
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return LIB_PATHS[group]


def build(force: bool = False, groups=None) -> str:
    """Compile the libraries in-tree (atomic replace), all groups unless
    `groups` names some. Returns the core library's path."""
    todo = [g for g in (groups or GROUPS)
            if force or not os.path.exists(LIB_PATHS[g])]
    with ThreadPoolExecutor(max_workers=max(len(todo), 1)) as ex:
        list(ex.map(_build_group, todo))
    return LIB_PATH


class _Libs:
    """Attribute access resolves an entry point in its group's library,
    which is loaded (and built, when nothing is built) on first use."""

    def __init__(self) -> None:
        self._handles = {}

    def _handle(self, group: str):
        h = self._handles.get(group)
        if h is None:
            if not os.path.exists(LIB_PATHS[group]):
                _build_group(group)
            h = ctypes.CDLL(LIB_PATHS[group])
            self._handles[group] = h
        return h

    def __getattr__(self, name: str):
        if not name.startswith("mx_"):
            raise AttributeError(name)
        fn = getattr(self._handle(SYMBOL_GROUP.get(name, "core")), name)
        fn.restype = (ctypes.c_int if name in INT_RESULT else
                      ctypes.c_long if name in LONG_RESULT else None)
        setattr(self, name, fn)
        return fn


_lib = None


def load():
    """Handle of the libraries (see _Libs)."""
    global _lib
    if _lib is None:
        _lib = _Libs()
    return _lib


def available() -> bool:
    return all(os.path.exists(p) for p in LIB_PATHS.values())
