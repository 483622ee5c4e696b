"""Host-side mirror of the reference's top-k sparse attention module
(src/shaders/attn/attention_topk/mod.rs): the same constants and entry names, driving the HIP
library through its C ABI.  torch is used for device memory and streams only."""
from __future__ import annotations

import ctypes as C
from typing import Sequence

import numpy as np

from . import capi
from .attention import AttnRig, Fixture, _torch, layer_offsets, step_params, stream_handle

# mod.rs:27-36
K_PAD = 64


def k_pad_for(k: int) -> int:
    """Slot capacity for a requested k: next power of two, clamped to [K_PAD, 1024] (mod.rs:34-36)."""
    k = max(k, 1)
    p = 1 << (k - 1).bit_length()
    return min(max(p, K_PAD), 1024)


def fixed_k(k: int) -> tuple:
    """k_cfg of the harness path: a fixed k, clamped like mod.rs:114-115."""
    kp = k_pad_for(k)
    return (min(max(k, 1), kp), 0, 0, 0)


def adaptive_k(grid: int = 256, divisor: int = 128, k_min: int = 64, k_max: int = 512) -> tuple:
    """k_cfg of the production path (src/flags/accessors.rs:210-221): k = clamp(t / 128, 64, 512) per row."""
    return (grid, divisor, k_min, k_max)


def _cfg(k_cfg: Sequence[int]):
    return (C.c_uint32 * 4)(*k_cfg)


def workspace_bytes(desc: capi.AttnDesc, k_cfg: Sequence[int]) -> int:
    n = C.c_size_t(0)
    capi.check(capi.load().dg_attn_topk_workspace_bytes(C.byref(desc), _cfg(k_cfg), C.byref(n)))
    return n.value


def alloc_workspace(desc: capi.AttnDesc, k_cfg: Sequence[int]):
    torch = _torch()
    return torch.empty(max(workspace_bytes(desc, k_cfg), 256), dtype=torch.uint8, device="cuda")


def forward(desc: capi.AttnDesc, k_cfg: Sequence[int], q, kv, out, workspace) -> None:
    """dg_attn_topk_forward on torch device tensors, on torch's current stream."""
    capi.check(capi.load().dg_attn_topk_forward(C.byref(desc), _cfg(k_cfg), q.data_ptr(), kv.data_ptr(),
                                                out.data_ptr(), workspace.data_ptr(),
                                                workspace.numel() * workspace.element_size(), stream_handle()))


def run_dispatch(rig: AttnRig, causal: bool, k_cfg: Sequence[int]) -> None:
    """The reference-shaped entry on an AttnRig (bf16 Q/out, f16 cache, truncating store)."""
    f = rig.fixture
    lib = capi.load()
    lo = layer_offsets(f, rig.kv_ring_mask)
    sp = step_params(f.kv_len)
    dims = capi.AttnDims(canvas=f.canvas, n_q_heads=f.n_q_heads, causal=1 if causal else 0, window=0)
    n = C.c_size_t(0)
    capi.check(lib.dg_attention_topk_state_bytes(C.byref(lo), C.byref(dims), f.kv_len, _cfg(k_cfg), C.byref(n)))
    key = ("topk", n.value)
    if key not in rig._ws:
        rig._ws[key] = _torch().empty(max(n.value, 256), dtype=_torch().uint8, device="cuda")
    st = rig._ws[key]
    capi.check(lib.dg_attention_topk_dispatch(rig.buf_q.data_ptr(), rig.buf_kv.data_ptr(), rig.buf_out.data_ptr(),
                                              C.byref(lo), C.byref(sp), C.byref(dims), _cfg(k_cfg),
                                              rig.buf_dbg.data_ptr(), st.data_ptr(), st.numel(), stream_handle()))


def gpu(f: Fixture, causal: bool, k: int) -> np.ndarray:
    """Top-k attention over a Fixture, bf16-rounded outputs as f32 (mod.rs:88-226, f16 cache path)."""
    rig = AttnRig.from_fixture(f)
    run_dispatch(rig, causal, fixed_k(k))
    return rig.read_out_f32()


def bench_gpu(f: Fixture, iters: int, k: int, causal: bool):
    """(min, median) ms per layer over warmed rounds (mod.rs:406-418)."""
    rig = AttnRig.from_fixture(f)
    cfg = fixed_k(k)
    run_dispatch(rig, causal, cfg)
    return rig.time_rounds(iters, lambda: run_dispatch(rig, causal, cfg))
