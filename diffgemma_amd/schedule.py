"""The attention schedule of one denoise iteration: 30 decoder layers, each the producer
(per-head RMSNorm + RoPE + KV write of the canvas rows) followed by the attention call, encoded
once into a HIP graph and replayed per iteration.

Reference shape: a denoise block runs `run_denoise_step` in a loop over one cached prefix
(src/metal/step_generate/turn.rs:575-623), each step one command buffer that walks the layers in
order (src/metal/step_kernel/runtime.rs:573-631), layers 5, 11, 17, 23, 29 being the full-attention
ones (src/metal/step_kernel/mod.rs:127): 25 sliding-window layers (8 KV heads, head_dim 256,
window 1024, ring cache) to 5 global layers (2 KV heads, head_dim 512, linear cache).  Only the
attention part of a layer is here; the canvas projections that feed it are regenerated between
iterations from `seed + iteration`, the prefix rows of the caches stay.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import attention as A, attention_topk as T, capi, qk_rope_kv as QR, rounding as R, step_kv


@dataclass
class ScheduleLayer:
    index: int
    full: bool
    head_dim: int
    n_kv_heads: int
    slots: int              # cache slots per KV head: prefix + canvas (global) or the ring (sliding)
    ring_mask: int
    window: int
    rope_desc: object
    attn_desc: capi.AttnDesc
    cache: object           # bf16 bits, head-major K planes then V planes
    q: object
    k: object
    v: object
    q_norm_w: object
    k_norm_w: object
    out: object
    lse: object             # [canvas][n_q_heads] fp32 log-sum-exp of the row's scores (dense layers)
    workspace: object
    flops: float = 0.0


@dataclass
class DenoiseSchedule:
    """Buffers, descriptors and the captured graph of one denoise iteration's attention work."""
    canvas: int = 256
    n_q_heads: int = 16
    kv_len: int = 32768
    kv_len_max: Optional[int] = None   # set: the committed prefix lives in device memory (a device StepParams the
                                       # kernels read when they run, as the reference binds it, enc.rs:2177-2220) and
                                       # may be advanced up to this value between replays of ONE recorded graph
    ring: int = 2048
    window: int = 1024
    n_layers: int = step_kv.N_LAYERS
    full_layers: tuple = step_kv.FULL_LAYERS
    global_topk: bool = False     # global layers as top-k sparse attention (the reference's default for them)
    seed: int = 1234
    layers: List[ScheduleLayer] = field(default_factory=list)
    flops_per_iteration: float = 0.0
    graph: Optional[object] = None
    topk_ws: Optional[object] = None
    step_dev: Optional[object] = None   # device StepParams (int32 x 12) when kv_len_max is set
    k_cfg: Optional[object] = None

    def build(self) -> "DenoiseSchedule":
        import torch
        self._lib = capi.load()
        self._gen = torch.Generator(device="cuda")
        self._gen.manual_seed(self.seed)
        self.k_cfg = T.adaptive_k()

        def unit_rows(n, hd):      # rows with unit RMS, bf16 bits: what a cache holds after the producer
            x = torch.randn(n, hd, device="cuda", generator=self._gen)
            x = x / x.pow(2).mean(-1, keepdim=True).sqrt()
            return x.to(torch.bfloat16).view(torch.int16).reshape(-1)

        canvas, nq = self.canvas, self.n_q_heads
        kv_len = self.kv_len_max if self.kv_len_max is not None else self.kv_len   # what the layers are planned for
        assert self.kv_len <= kv_len
        self.step_dev = A.device_step_params(self.kv_len) if self.kv_len_max is not None else None
        for i in range(self.n_layers):
            full = i in self.full_layers
            hd, nkv = (512, 2) if full else (256, 8)
            slots = kv_len + canvas if full else self.ring
            mask = 0 if full else self.ring - 1
            window = 0 if full else self.window
            f = QR.random_fixture(1, nq, nkv, hd, kv_len, is_full=full, v_proj=0 if full else 1, seed=100 + i,
                                  kv_ring_mask=mask)      # norm weights and flags only; the buffers are made below
            f.canvas = canvas
            rd = QR.rope_desc(f, kv_dtype=capi.DG_BF16, truncate=False, layout="head_major", t_cap=slots)
            ad = A.make_desc(canvas, nq, nkv, hd, kv_len, window=window, kv_ring_mask=mask,
                             q_dtype=capi.DG_BF16, kv_dtype=capi.DG_BF16, out_dtype=capi.DG_BF16,
                             layout="head_major", t_cap=slots,
                             # unit-RMS V rows: far inside the f16 range.  (The 30 caches add up to 1.1 GB per
                             # iteration, four times the memory-side cache, so a global layer's rows come from HBM:
                             # the library sees that by itself from what the calls before it streamed.)
                             flags=capi.DG_ATTN_F_F16_PARTIALS)
            lay = ScheduleLayer(
                index=i, full=full, head_dim=hd, n_kv_heads=nkv, slots=slots, ring_mask=mask, window=window,
                rope_desc=rd, attn_desc=ad,
                cache=unit_rows(2 * nkv * slots, hd),     # every slot live: prefix rows (ring: its window)
                q=torch.empty(canvas * nq * hd, dtype=torch.int16, device="cuda"),
                k=torch.empty(canvas * nkv * hd, dtype=torch.int16, device="cuda"),
                v=torch.empty(canvas * nkv * hd, dtype=torch.int16, device="cuda"),
                q_norm_w=A.to_device_bits(R.f32_to_bf16_bits_rne(f.q_norm_w)),
                k_norm_w=A.to_device_bits(R.f32_to_bf16_bits_rne(f.k_norm_w)),
                out=torch.zeros(canvas * nq * hd, dtype=torch.int16, device="cuda"),
                lse=torch.zeros(canvas * nq, dtype=torch.float32, device="cuda"),
                workspace=A.alloc_workspace(ad),
                flops=capi.visible_pairs(ad)[1])
            if full and self.global_topk and self.topk_ws is None:
                self.topk_ws = T.alloc_workspace(ad, self.k_cfg)      # one score plane, shared by the global layers
            self.layers.append(lay)
            self.flops_per_iteration += lay.flops
        return self

    def set_kv_len(self, kv_len: int) -> None:
        """A block was committed: the prefix grows.  Only the device word changes; a recorded graph stays valid."""
        assert self.step_dev is not None and kv_len <= self.kv_len_max
        self.kv_len = kv_len
        self.step_dev[0] = kv_len

    def regenerate(self, iteration: int) -> None:
        """Canvas projections of iteration `iteration`: N(0, 1) from the device generator keyed by seed + iteration."""
        import torch
        self._gen.manual_seed(self.seed + 4444 + iteration)
        for lay in self.layers:
            for t in (lay.q, lay.k, lay.v):
                t.copy_(torch.randn(t.numel(), device="cuda", generator=self._gen).to(torch.bfloat16).view(torch.int16))

    def encode(self) -> None:
        """Enqueue one iteration on the current stream: per layer the producer, then attention."""
        st = A.stream_handle()
        for lay in self.layers:
            if self.step_dev is not None:
                capi.check(self._lib.dg_qk_rope_kv_dev(C.byref(lay.rope_desc), self.step_dev.data_ptr(), lay.q.data_ptr(),
                                                       lay.k.data_ptr(), lay.v.data_ptr(), lay.cache.data_ptr(),
                                                       lay.q_norm_w.data_ptr(), lay.k_norm_w.data_ptr(), None, st))
                A.forward_dev(lay.attn_desc, self.step_dev, lay.q, lay.cache, lay.out, lay.lse, lay.workspace)
                continue
            capi.check(self._lib.dg_qk_rope_kv(C.byref(lay.rope_desc), lay.q.data_ptr(), lay.k.data_ptr(),
                                               lay.v.data_ptr(), lay.cache.data_ptr(), lay.q_norm_w.data_ptr(),
                                               lay.k_norm_w.data_ptr(), None, st))
            if lay.full and self.global_topk:
                T.forward(lay.attn_desc, self.k_cfg, lay.q, lay.cache, lay.out, self.topk_ws)
            else:
                A.forward(lay.attn_desc, lay.q, lay.cache, lay.out, lay.lse, lay.workspace)

    def run_eager(self) -> None:
        """One iteration as plain launches on a side stream (the stream a capture would use)."""
        import torch
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.encode()
        torch.cuda.current_stream().wait_stream(side)

    def capture(self) -> None:
        """Record one iteration into a HIP graph (the library records no memset nodes)."""
        import torch
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.encode()

    def replay(self) -> None:
        self.graph.replay()

    def outputs(self):
        return [lay.out.clone() for lay in self.layers]
