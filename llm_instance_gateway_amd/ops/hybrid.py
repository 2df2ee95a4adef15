"""Light native library for the hybrid-model kernels (grouped RMS norm, xIELU,
minGRU scan, general-size paged attention, shift norms, latent attention,
sum+norm residual step, q/k/v prep, head-mixed attention, matrix-state scan,
multi-stream residual step, grouped router and routed combine).

These kernels expose a plain C ABI and need no torch headers, so they are
compiled by one direct ``hipcc -shared`` call (seconds, not the minutes the
torch extension takes) into ``llm_instance_gateway_amd/_hybrid.so`` and
loaded with ctypes.  A model that needs only these kernels can therefore be
served from a fresh checkout after a short first-use build; nothing else is
compiled for it.

``build()`` always compiles; ``lib()`` loads what is built and builds only
when nothing is there (guarded by a file lock so concurrent processes build
once).
"""

from __future__ import annotations

import ctypes
import fcntl
import os
import shutil
import subprocess
import tempfile
from pathlib import Path
from typing import Optional

PKG = Path(__file__).resolve().parent.parent
CSRC = Path(__file__).resolve().parent / "csrc"
# Sources of the light library; setup.py leaves these out of the torch
# extension.
SOURCES = [
    "group_norm.hip", "xielu.hip", "mingru.hip", "attention_general.hip",
    "attention_prefill_tiles.hip", "shift_norm.hip", "latent_attention.hip", "ff_act.hip",
    "attention_latent_rows.hip", "post_norm.hip", "qkv_prep.hip", "attention_mixed_heads.hip",
    "matrix_state_scan.hip", "attention_mixed_heads_tiles.hip", "hyper_streams.hip",
    "routed.hip",
]
SO_PATH = PKG / "_hybrid.so"

_LIB: Optional[ctypes.CDLL] = None


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; cannot build the hybrid kernel library")


def build() -> Path:
    """Compile the light library for gfx950 (atomic replace of the .so)."""
    fd, tmp = tempfile.mkstemp(prefix="._hybrid-", suffix=".so", dir=str(PKG))
    os.close(fd)
    cmd = [
        _hipcc(), "-O3", "-std=c++17", "--offload-arch=gfx950",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-shared", "-fPIC", "-o", tmp,
    ] + [str(CSRC / s) for s in SOURCES]
    try:
        subprocess.run(cmd, check=True, cwd=str(CSRC), stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE)
        os.chmod(tmp, 0o755)
        os.replace(tmp, SO_PATH)
    except subprocess.CalledProcessError as e:
        raise RuntimeError(
            "building the hybrid kernel library failed:\n" + e.stderr.decode(errors="replace")[-4000:]
        ) from None
    finally:
        if os.path.exists(tmp):
            os.unlink(tmp)
    return SO_PATH


def _declare(lib: ctypes.CDLL) -> None:
    p, i, l, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float
    sigs = {
        "lig_embed_group_norm": [p, p, p, p, f, i, i, i, i, p],
        "lig_group_norm": [p, p, p, f, i, i, i, i, p],
        "lig_post_add_pre_norm": [p, p, p, p, p, f, i, i, i, i, p],
        "lig_xielu": [p, p, f, f, l, i, p],
        "lig_sigmoid_gate_mul": [p, p, l, i, i, i, p],
        "lig_mingru_scan": [p, p, p, p, l, p, p, p, p, p, p, i, i, i, i, p],
        "lig_paged_attention_general": [
            p, p, l, p, p, p, i, p, p, p, l, p, f, f, f, i, i, i, i, i, i, i, i, i,
            i, p, i, i, i, p,
        ],
        "lig_offset_norm_shift": [p, p, p, p, p, p, p, p, p, p, p, p, p, p, p, f, i, i, i, p],
        "lig_offset_rms_norm": [p, p, p, f, i, i, i, p],
        "lig_residual_add": [p, p, p, l, i, p],
        "lig_latent_kv_prep": [p, p, l, p, p, p, i, p, p, p, f, i, i, i, i, i, p],
        "lig_rotate_pack_queries": [p, p, p, i, p, i, i, i, i, i, i, p],
        "lig_scale_gather_rows": [p, p, p, p, l, i, i, p],
        "lig_relu_squared": [p, p, l, i, p],
        "lig_silu_mul": [p, p, l, i, i, p],
        "lig_kv_scatter": [p, p, l, p, p, p, i, i, i, i, i, i, p],
        "lig_temperature_scale_rows": [p, p, l, p, f, f, i, i, i, i, p],
        "lig_scaled_add_rms_norm": [p, p, p, p, p, f, f, f, f, i, i, i, p],
        "lig_qkv_norm_rope_cache": [
            p, p, p, l, p, p, p, i, p, p, f, p, p, p, f, i, i, i, i, i, i, i, i, i, i, i, p,
        ],
        "lig_token_shift_mix": [p, p, p, p, p, p, p, p, p, i, i, i, i, p],
        "lig_group_rms_norm_gate": [p, p, p, l, p, i, i, f, i, i, i, p],
        "lig_gelu_erf": [p, p, l, i, p],
        "lig_tanh_act": [p, p, l, i, p],
        "lig_tanh_softcap": [p, f, l, p],
        "lig_routed_combine": [p, p, p, p, p, i, p, i, i, i, i, p],
        "lig_glu_act": [p, p, l, i, i, f, f, i, p],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = None
    pt = lib.lig_paged_attention_prefill_tiles
    pt.argtypes = [
        p, p, l, p, p, p, l, p, p, p, p, p, p, f, f, f, i, i, i, i, i, i, i, i, i, i,
        i, p, i, i, p,
    ]
    pt.restype = ctypes.c_int
    hs = lib.lig_hyper_step
    hs.argtypes = [p, p, p, p, f, p, p, f, p, i, i, i, i, p]
    hs.restype = ctypes.c_int
    gr = lib.lig_grouped_topk_route
    gr.argtypes = [p, p, i, i, i, i, i, p, p, p]
    gr.restype = ctypes.c_int
    mh = lib.lig_paged_attention_mixed_heads
    mh.argtypes = [p, p, l, p, p, p, i, p, p, p, i, p, f, i, i, i, i, i, i, i, i, p]
    mh.restype = ctypes.c_int
    mt = lib.lig_paged_attention_mixed_heads_tiles
    mt.argtypes = [p, p, l, p, p, p, i, p, p, p, p, p, p, f, i, i, i, i, i, i, i, i, p]
    mt.restype = ctypes.c_int
    ms = lib.lig_matrix_state_scan
    ms.argtypes = [p, p, l, p, l, p, l, p, p, p, p, l, p, p, p, p, i, i, i, i, i, i, p]
    ms.restype = ctypes.c_int
    lr = lib.lig_latent_attention_rows
    lr.argtypes = [p, p, p, p, p, p, p, p, i, f, i, i, i, i, i, i, i, p, p]
    lr.restype = ctypes.c_int


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is not None:
        return _LIB
    if not SO_PATH.exists():
        lock = PKG / "._hybrid.lock"
        with open(lock, "w") as lf:
            fcntl.flock(lf, fcntl.LOCK_EX)
            try:
                if not SO_PATH.exists():
                    build()
            finally:
                fcntl.flock(lf, fcntl.LOCK_UN)
    _LIB = ctypes.CDLL(str(SO_PATH))
    _declare(_LIB)
    return _LIB


def available() -> bool:
    return SO_PATH.exists()
