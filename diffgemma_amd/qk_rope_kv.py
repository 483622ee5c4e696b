"""Host side of the producer of the cache rows attention reads: per-head RMSNorm + RoPE + KV write.

Mirrors the reference module src/shaders/attn/qk_rope_kv/mod.rs: `Fixture`, its four fixture
generators, `layer_offsets`, `pack_out` and `gpu()` keep the reference's names and meaning, so a
parity test reads like the reference's `kernel_oracle_matrix!` cases (mod.rs:437-489).  `gpu()` here
drives the HIP kernel through the C ABI (`dg_qk_rope_kv_dispatch`); there is no CPU path.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from . import attention as A
from . import capi, rounding


@dataclass
class Fixture:
    """qk_rope_kv/mod.rs:41-53.  q [canvas][Hq][hd], k/v [canvas][Hkv][hd], f32 host values."""
    q: np.ndarray
    k: np.ndarray
    v: np.ndarray
    q_norm_w: np.ndarray
    k_norm_w: np.ndarray
    head_dim: int
    n_kv_heads: int
    is_full: bool
    canvas: int
    n_q_heads: int
    kv_len: int
    v_proj: int            # 0: V aliases the raw k projection (full-attention layers)
    kv_region: int = 0
    kv_ring_mask: int = 0
    kv_write_end: int = 0xFFFFFFFF
    kvcache: np.ndarray = field(default=None)   # f32 host image of the whole cache, reference layout

    def __post_init__(self):
        if self.kvcache is None:
            self.kvcache = np.zeros(self.kv_region // 2 + self.kv_slots(), np.float32)

    def n_slots(self) -> int:
        return (self.kv_ring_mask + 1) if self.kv_ring_mask else (self.kv_len + self.canvas)

    def kv_slots(self) -> int:          # mod.rs:68-70 (elements of the layer's region)
        return self.n_slots() * self.n_kv_heads * self.head_dim * 2

    def qk_grid_y(self) -> int:         # mod.rs:64-66
        return self.n_q_heads + 2 * self.n_kv_heads

    def out_len(self) -> int:           # mod.rs:72-74
        return self.q.size + self.k.size + self.canvas * self.n_kv_heads * self.head_dim * 2


def _gen(n, fn):
    i = np.arange(n, dtype=np.float32)
    return fn(i).astype(np.float32)


def tiny_fixture() -> Fixture:          # mod.rs:80-117
    canvas, nq, nkv, hd, kv_len = 2, 4, 2, 32, 2
    return Fixture(q=_gen(canvas * nq * hd, lambda i: np.sin(i * np.float32(0.13)) * np.float32(0.5)),
                   k=_gen(canvas * nkv * hd, lambda i: np.cos(i * np.float32(0.17)) * np.float32(0.4)),
                   v=_gen(canvas * nkv * hd, lambda i: np.sin(i * np.float32(0.11)) * np.float32(0.3)),
                   q_norm_w=np.ones(hd, np.float32), k_norm_w=np.ones(hd, np.float32), head_dim=hd,
                   n_kv_heads=nkv, is_full=False, canvas=canvas, n_q_heads=nq, kv_len=kv_len, v_proj=1)


def full_layer_fixture() -> Fixture:    # mod.rs:119-143
    canvas, nq, nkv, hd, kv_len = 2, 4, 2, 64, 2
    return Fixture(q=_gen(canvas * nq * hd, lambda i: np.sin(i * np.float32(0.07)) * np.float32(0.6)),
                   k=_gen(canvas * nkv * hd, lambda i: np.cos(i * np.float32(0.09)) * np.float32(0.5)),
                   v=_gen(canvas * nkv * hd, lambda i: np.sin(i * np.float32(0.08)) * np.float32(0.45)),
                   q_norm_w=np.ones(hd, np.float32), k_norm_w=np.ones(hd, np.float32), head_dim=hd,
                   n_kv_heads=nkv, is_full=True, canvas=canvas, n_q_heads=nq, kv_len=kv_len, v_proj=1)


def full_attn_v_alias_fixture() -> Fixture:   # mod.rs:145-150
    f = full_layer_fixture()
    f.v_proj = 0
    return f


def full_hd512_v_alias_fixture() -> Fixture:  # mod.rs:152-189
    canvas, nq, nkv, hd, kv_len = 1, 16, 2, 512, 22
    i = np.arange(hd, dtype=np.float32)
    return Fixture(q=_gen(canvas * nq * hd, lambda i: np.sin(i * np.float32(0.031)) * np.float32(0.55)),
                   k=_gen(canvas * nkv * hd, lambda i: np.cos(i * np.float32(0.029)) * np.float32(0.48)),
                   v=np.zeros(canvas * nkv * hd, np.float32),
                   q_norm_w=(np.float32(1.0) + i * np.float32(0.0001)).astype(np.float32),
                   k_norm_w=(np.float32(1.0) - i * np.float32(0.00005)).astype(np.float32), head_dim=hd,
                   n_kv_heads=nkv, is_full=True, canvas=canvas, n_q_heads=nq, kv_len=kv_len, v_proj=0)


def random_fixture(canvas, nq, nkv, hd, kv_len, *, is_full, v_proj, seed=0, kv_ring_mask=0,
                   kv_write_end=0xFFFFFFFF, kv_region=0) -> Fixture:
    """Layer-shaped inputs (projection outputs ~ N(0, 1), weights around 1)."""
    rng = np.random.default_rng(seed)
    return Fixture(q=rng.standard_normal(canvas * nq * hd, dtype=np.float32),
                   k=rng.standard_normal(canvas * nkv * hd, dtype=np.float32),
                   v=rng.standard_normal(canvas * nkv * hd, dtype=np.float32),
                   q_norm_w=(1.0 + 0.1 * rng.standard_normal(hd)).astype(np.float32),
                   k_norm_w=(1.0 + 0.1 * rng.standard_normal(hd)).astype(np.float32), head_dim=hd,
                   n_kv_heads=nkv, is_full=is_full, canvas=canvas, n_q_heads=nq, kv_len=kv_len, v_proj=v_proj,
                   kv_ring_mask=kv_ring_mask, kv_write_end=kv_write_end, kv_region=kv_region)


def layer_offsets(f: Fixture) -> capi.LayerOffsets:   # mod.rs:191-221
    L = capi.LayerOffsets()
    L.q_norm, L.k_norm = 0, f.head_dim * 2            # the blob holds q_norm_w then k_norm_w, bf16
    L.v_proj = f.v_proj
    L.kv_region = f.kv_region
    L.head_dim, L.n_kv_heads, L.is_full, L.kv_ring_mask = f.head_dim, f.n_kv_heads, int(f.is_full), f.kv_ring_mask
    return L


def pack_out(q, k, kvcache, f: Fixture) -> np.ndarray:   # mod.rs:223-236 (ring-aware slot)
    hd, nkv = f.head_dim, f.n_kv_heads
    rows = []
    base = f.kv_region // 2
    for tok in range(f.canvas):
        pos = f.kv_len + tok
        slot = (pos & f.kv_ring_mask) if f.kv_ring_mask else pos
        off = base + slot * nkv * hd * 2
        rows.append(kvcache[off:off + nkv * hd * 2])
    return np.concatenate([np.asarray(q).ravel(), np.asarray(k).ravel()] + rows).astype(np.float32)


def rope_desc(f: Fixture, *, kv_dtype=capi.DG_F16, truncate=True, layout="reference", t_cap=0) -> capi.RopeDesc:
    d = capi.RopeDesc()
    d.canvas, d.n_q_heads, d.n_kv_heads, d.head_dim = f.canvas, f.n_q_heads, f.n_kv_heads, f.head_dim
    d.kv_len, d.kv_write_end, d.kv_ring_mask = f.kv_len, f.kv_write_end, f.kv_ring_mask
    d.is_full, d.v_from_k, d.kv_dtype = int(f.is_full), int(f.v_proj == 0), kv_dtype
    d.flags = capi.DG_ROPE_F_QK_TRUNCATE if truncate else 0
    d.kv_region_bytes = f.kv_region
    row = f.n_kv_heads * f.head_dim
    if layout == "reference":
        d.k_tok_stride, d.k_head_stride = 2 * row, f.head_dim
        d.v_base_off, d.v_tok_stride, d.v_head_stride = row, 2 * row, f.head_dim
    else:   # two planes [Hkv][t_cap][d], K then V
        d.k_tok_stride, d.k_head_stride = f.head_dim, t_cap * f.head_dim
        d.v_base_off, d.v_tok_stride, d.v_head_stride = f.n_kv_heads * t_cap * f.head_dim, f.head_dim, t_cap * f.head_dim
    return d


class RopeRig:
    """Device buffers of one fixture, as the reference's gpu() allocates them (mod.rs:283-317)."""

    def __init__(self, f: Fixture):
        torch = A._torch()
        self.f = f
        self.buf_q = A.to_device_bits(rounding.f32_to_bf16_bits_trunc(f.q))     # write_bf16: truncating pack
        self.buf_k = A.to_device_bits(rounding.f32_to_bf16_bits_trunc(f.k))
        self.buf_v = A.to_device_bits(rounding.f32_to_bf16_bits_trunc(f.v))
        self.buf_kv = A.to_device_bits(rounding.f32_to_f16_bits_trunc(f.kvcache))
        blob = np.concatenate([rounding.f32_to_bf16_bits_trunc(f.q_norm_w), rounding.f32_to_bf16_bits_trunc(f.k_norm_w)])
        self.buf_blob = A.to_device_bits(blob)
        self.buf_dbg = torch.zeros(4, dtype=torch.int32, device="cuda")

    def run_dispatch(self) -> None:
        f = self.f
        L, P = layer_offsets(f), A.step_params(f.kv_len)
        P.kv_write_end = f.kv_write_end
        dims = capi.AttnDims(f.canvas, f.n_q_heads, 0, 0)
        capi.check(capi.load().dg_qk_rope_kv_dispatch(
            self.buf_q.data_ptr(), self.buf_k.data_ptr(), self.buf_v.data_ptr(), self.buf_kv.data_ptr(),
            self.buf_blob.data_ptr(), C.byref(L), C.byref(P), C.byref(dims), self.buf_dbg.data_ptr(),
            A.stream_handle()))
        A._torch().cuda.synchronize()

    def run_dispatch_dev(self) -> None:
        """run_dispatch with StepParams as a device buffer (qk_rope_kv.metal:30-38 binds it so): kv_len and
        kv_write_end are read when the kernel runs."""
        f = self.f
        L = layer_offsets(f)
        self.step_dev = A.device_step_params(f.kv_len, f.kv_write_end)
        dims = capi.AttnDims(f.canvas, f.n_q_heads, 0, 0)
        capi.check(capi.load().dg_qk_rope_kv_dispatch_dev(
            self.buf_q.data_ptr(), self.buf_k.data_ptr(), self.buf_v.data_ptr(), self.buf_kv.data_ptr(),
            self.buf_blob.data_ptr(), C.byref(L), self.step_dev.data_ptr(), C.byref(dims), self.buf_dbg.data_ptr(),
            A.stream_handle()))
        A._torch().cuda.synchronize()

    def read(self):
        """(q, k, kvcache) as f32 host arrays."""
        q = rounding.bf16_bits_to_f32(self.buf_q.cpu().numpy().view(np.uint16))
        k = rounding.bf16_bits_to_f32(self.buf_k.cpu().numpy().view(np.uint16))
        kv = rounding.f16_bits_to_f32(self.buf_kv.cpu().numpy().view(np.uint16))
        return q, k, kv


def gpu(f: Fixture) -> np.ndarray:      # mod.rs:283-426
    rig = RopeRig(f)
    rig.run_dispatch()
    q, k, kv = rig.read()
    return pack_out(q, k, kv, f)
