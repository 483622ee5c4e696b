"""Synthetic denoise-attention workloads: shapes, masks and seeded input generators.

The shapes are the model's (src/metal/step_kernel/mod.rs:64,127 and ARCHITECTURE.md:104-111
of the reference: canvas 256, 16 query heads; sliding layers hd 256 / 8 KV heads / window
1024; global layers hd 512 / 2 KV heads).  Inputs are numpy `default_rng(seed)` normals, so
the CPU oracle and the HIP kernel are fed identical bytes.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Optional, Tuple

import numpy as np

from . import capi, rounding
from .attention import make_desc

RMS_EPS = 1e-6


@dataclass(frozen=True)
class Workload:
    name: str
    canvas: int
    n_q_heads: int
    n_kv_heads: int
    head_dim: int
    kv_len: int
    causal_rows: int = 0
    window: int = 0
    t_lo: Optional[int] = None       # explicit first visible key for bidirectional rows
    dtype: str = "bf16"              # storage dtype of Q/K/V: "bf16" or "f32"
    layout: str = "head_major"       # "head_major" [Hkv,T,d] planes or "reference" slot-major
    rms_norm: bool = True            # per-head RMSNorm with unit gain after sampling
    q_std: float = 1.0
    kv_std: float = 1.0
    pre_scale: float = 1.0           # multiplies Q, K and V after sampling
    outlier_frac: float = 0.0        # fraction of prefix keys scaled by outlier_gain
    outlier_gain: float = 1.0
    seed: int = 0
    sees_masked: bool = False
    kv_f16: bool = False             # cache stored as f16 under bf16 queries (the reference's own pairing)

    @property
    def t_all(self) -> int:
        return self.kv_len + self.canvas

    def desc(self, **kw) -> capi.AttnDesc:
        dt = capi.DG_BF16 if self.dtype == "bf16" else capi.DG_F32
        flags = kw.pop("flags", 0)
        default_partials = kw.pop("default_partials", False)   # leave the partial-row format to the library
        t_lo = 0
        if self.t_lo is not None:
            flags |= capi.DG_ATTN_F_T_LO_EXPLICIT
            t_lo = self.t_lo
        if self.sees_masked:
            flags |= capi.DG_ATTN_F_CAUSAL_SEES_MASKED
        if not default_partials and not flags & capi.DG_ATTN_F_F32_PARTIALS:
            # every generator below draws V from N(0, kv_std^2) (RMS-normalised or not): far inside the
            # f16 range, as are the V rows a model's cache holds after the producer's RMSNorm
            flags |= capi.DG_ATTN_F_F16_PARTIALS
        args = dict(causal_rows=self.causal_rows, window=self.window, q_dtype=dt,
                    kv_dtype=capi.DG_F16 if self.kv_f16 else dt,
                    out_dtype=dt, flags=flags, t_lo=t_lo, layout=self.layout, t_cap=self.t_all)
        args.update(kw)
        return make_desc(self.canvas, self.n_q_heads, self.n_kv_heads, self.head_dim, self.kv_len, **args)


def config(name: str) -> Workload:
    """The benchmark configurations, by name."""
    if name == "cfg1_tiny":
        return Workload(name, 256, 8, 4, 128, 512, dtype="f32", layout="reference", rms_norm=False,
                        pre_scale=1.0 / np.sqrt(128.0), seed=0)
    if name == "cfg2_sliding":        # reference window rule: 1023 prefix keys + canvas
        return Workload(name, 256, 16, 8, 256, 4096, window=1024, seed=2)
    if name == "cfg2_sliding_768":    # the other reading: last 1024-256 prefix keys + canvas
        return Workload(name, 256, 16, 8, 256, 4096, window=1024, t_lo=4096 - (1024 - 256), seed=2)
    if name == "cfg3_global":         # committed rows never see the masked canvas tokens
        return Workload(name, 256, 16, 2, 512, 32768, causal_rows=128, seed=3)
    if name == "cfg3_global_b":       # committed rows additionally see canvas keys >= 128
        return Workload(name, 256, 16, 2, 512, 32768, causal_rows=128, sees_masked=True, seed=3)
    if name == "cfg3_global_f16kv":   # config 3 with the reference's storage: bf16 activations, f16 cache
        return Workload(name, 256, 16, 2, 512, 32768, causal_rows=128, seed=3, kv_f16=True)
    if name == "cfg3_global_flat":    # config 3's shape with a flat softmax: scores of unit spread (Q of std 1/sqrt(hd),
        # no RMSNorm), so that no softmax weight is negligible.  The headline workload's unit-RMS rows without a
        # 1/sqrt(hd) scale give scores of spread sqrt(hd) and rows so peaked that nearly all weights are stored as
        # exact zeros, which the power-limited matrix cores reward; this one shows the kernel without that help.
        return Workload(name, 256, 16, 2, 512, 32768, causal_rows=128, rms_norm=False, q_std=1.0 / np.sqrt(512.0),
                        seed=3)
    if name == "cfg3_global_flat_f16kv":   # the flat-softmax variant over an f16 cache: no row's maximum moves far
        # enough to outrun f16 probabilities, so the f16 kernel shows without its rescales of O
        return Workload(name, 256, 16, 2, 512, 32768, causal_rows=128, rms_norm=False, q_std=1.0 / np.sqrt(512.0),
                        seed=3, kv_f16=True)
    if name == "cfg4_long":
        return Workload(name, 256, 16, 2, 512, 131072, rms_norm=False, kv_std=0.5, outlier_frac=0.01,
                        outlier_gain=8.0, seed=4)
    if name == "cfg5_sliding_32k":    # sliding layer of the 30-layer schedule at prefix 32768
        return Workload(name, 256, 16, 8, 256, 32768, window=1024, seed=5)
    # causal extend of the committed prefix by 4 x 256 tokens in one call (the reference's batched
    # prefill super-chunk, src/metal/step_kernel/runtime.rs:370-389, enc.rs:2576-2585)
    if name == "prefill_global_super":
        return Workload(name, 1024, 16, 2, 512, 32768, causal_rows=1024, seed=6)
    if name == "prefill_sliding_super":
        return Workload(name, 1024, 16, 8, 256, 32768, causal_rows=1024, window=1024, seed=7)
    if name == "prefill_global_fresh":    # first super-chunk of a prompt: no prefix, triangular mask
        return Workload(name, 1024, 16, 2, 512, 0, causal_rows=1024, seed=8)
    raise KeyError(name)


def scaled(w: Workload, kv_len: int, name: Optional[str] = None) -> Workload:
    """Same workload at another prefix length (tests run the big ones scaled down too)."""
    t_lo = w.t_lo
    if t_lo is not None:
        t_lo = max(0, kv_len - (w.kv_len - w.t_lo))
    return replace(w, kv_len=kv_len, t_lo=t_lo, name=name or f"{w.name}@{kv_len}")


def _rms_norm_rows(x: np.ndarray) -> np.ndarray:
    ms = np.mean(x.astype(np.float32) ** 2, axis=-1, keepdims=True, dtype=np.float32)
    return (x / np.sqrt(ms + np.float32(RMS_EPS))).astype(np.float32)


def generate(w: Workload) -> Tuple[np.ndarray, np.ndarray]:
    """Returns (q, kv) as float32 holding storage-representable values.

    q: [canvas, Hq, hd].  kv: head_major -> [2, Hkv, T, hd] (K planes then V planes);
    reference -> [T, 2, Hkv, hd] (per slot: K heads then V heads)."""
    rng = np.random.default_rng(w.seed)
    q = rng.standard_normal((w.canvas, w.n_q_heads, w.head_dim), dtype=np.float32) * np.float32(w.q_std)
    kv = np.empty((2, w.n_kv_heads, w.t_all, w.head_dim), dtype=np.float32)
    for plane in range(2):
        for h in range(w.n_kv_heads):
            kv[plane, h] = rng.standard_normal((w.t_all, w.head_dim), dtype=np.float32) * np.float32(w.kv_std)
    if w.outlier_frac > 0.0:
        n = int(round(w.outlier_frac * w.kv_len))
        for h in range(w.n_kv_heads):
            idx = rng.choice(w.kv_len, size=n, replace=False)
            kv[0, h, idx] *= np.float32(w.outlier_gain)
    if w.rms_norm:
        q = _rms_norm_rows(q)
        for plane in range(2):
            for h in range(w.n_kv_heads):
                kv[plane, h] = _rms_norm_rows(kv[plane, h])
    if w.pre_scale != 1.0:
        q *= np.float32(w.pre_scale)
        kv *= np.float32(w.pre_scale)
    if w.dtype == "bf16":
        q = rounding.bf16_bits_to_f32(rounding.f32_to_bf16_bits_rne(q)).reshape(q.shape)
        for plane in range(2):
            for h in range(w.n_kv_heads):
                kv[plane, h] = rounding.bf16_bits_to_f32(rounding.f32_to_bf16_bits_rne(kv[plane, h])).reshape(
                    kv[plane, h].shape)
        if w.kv_f16:   # bf16 values are f16 values unless they are tiny: flush those the way the store does
            for plane in range(2):
                for h in range(w.n_kv_heads):
                    kv[plane, h] = rounding.f16_bits_to_f32(rounding.f32_to_f16_bits_rne(kv[plane, h])).reshape(
                        kv[plane, h].shape)
    if w.layout == "reference":
        kv = np.ascontiguousarray(kv.transpose(2, 0, 1, 3))  # [T, 2, Hkv, hd]
    return q, kv


def device_arrays(w: Workload, q: np.ndarray, kv: np.ndarray):
    """Upload (q, kv) in the workload's storage dtype; returns torch device tensors."""
    import torch
    if w.dtype == "bf16":
        qd = torch.from_numpy(rounding.f32_to_bf16_bits_trunc(q).view(np.int16).reshape(-1)).cuda()
        kd = torch.empty(kv.size, dtype=torch.int16, device="cuda")
        flat = kv.reshape(-1)
        step = 1 << 25
        to_bits = rounding.f32_to_f16_bits_rne if w.kv_f16 else rounding.f32_to_bf16_bits_trunc
        for o in range(0, flat.size, step):  # values are exactly representable: the conversion is exact
            kd[o:o + step] = torch.from_numpy(to_bits(flat[o:o + step]).view(np.int16)).cuda()
        return qd, kd
    return torch.from_numpy(q.reshape(-1)).cuda(), torch.from_numpy(kv.reshape(-1)).cuda()
