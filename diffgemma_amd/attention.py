"""Host side of the denoise-step attention op, shaped like the reference's module.

Mirrors src/shaders/attn/attention/mod.rs (Fixture, the closed-form fixture generators,
the gpu* harnesses, bench_path) and src/shaders/attn/harness.rs (AttnRig) of the
reference, over the HIP library instead of Metal.  Device memory and streams come from
torch; arithmetic never does.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Optional

import numpy as np

from . import capi, rounding

RMS_EPS = 1e-6
MMA_M_TILE = 128   # stacked query rows per workgroup of the HIP kernel
KV_SLACK_SLOTS = 8  # zero pad rows the reference appends (harness.rs:28-30); not needed here, kept for layout parity


@dataclass
class LayerAttnParams:
    """src/shaders/attn/cpu.rs:5-28"""
    head_dim: int
    n_kv_heads: int
    is_full: bool = False
    v_proj: int = 1
    kv_region: int = 0
    q_norm_off: int = 0
    k_norm_off: int = 0


@dataclass
class Fixture:
    """src/shaders/attn/attention/mod.rs:31-53.  q: [canvas][n_q_heads][hd] f32,
    kvcache: reference slot-major layout [t][K: nkv*hd | V: nkv*hd] f32."""
    q: np.ndarray
    kvcache: np.ndarray
    layer: LayerAttnParams
    canvas: int
    n_q_heads: int
    kv_len: int

    def head_dim(self) -> int:
        return self.layer.head_dim

    def n_kv(self) -> int:
        return self.layer.n_kv_heads

    def out_len(self) -> int:
        return self.canvas * self.n_q_heads * self.head_dim()

    def t_total(self) -> int:
        return self.kv_len + self.canvas


def _f32(x):
    return np.asarray(x, dtype=np.float32)


def tiny_fixture() -> Fixture:
    """attention/mod.rs:59-95"""
    canvas, nq, nkv, hd, kv_len = 2, 4, 2, 32, 2
    tt = kv_len + canvas
    t = np.arange(tt)[:, None, None]
    h = np.arange(nkv)[None, :, None]
    d = np.arange(hd)[None, None, :]
    k = np.sin(_f32(t * 17 + h * 3 + d) * _f32(0.05))
    v = np.cos(_f32(t * 13 + h * 5 + d) * _f32(0.04))
    kv = np.concatenate([k.reshape(tt, nkv * hd), v.reshape(tt, nkv * hd)], axis=1).astype(np.float32)
    q = (np.sin(_f32(np.arange(canvas * nq * hd)) * _f32(0.11)) * _f32(0.6)).astype(np.float32)
    return Fixture(q, kv.reshape(-1), LayerAttnParams(hd, nkv, False, 1), canvas, nq, kv_len)


def wide_fixture() -> Fixture:
    """attention/mod.rs:97-126"""
    canvas, nq, nkv, hd, kv_len = 4, 8, 2, 64, 4
    tt = kv_len + canvas
    kv = (np.sin(_f32(np.arange(tt * nkv * hd * 2)) * _f32(0.031)) * _f32(0.3)).astype(np.float32)
    q = (np.cos(_f32(np.arange(canvas * nq * hd)) * _f32(0.02)) * _f32(0.5)).astype(np.float32)
    return Fixture(q, kv, LayerAttnParams(hd, nkv, False, 1), canvas, nq, kv_len)


def model_attn_fixture(canvas: int, nq: int, nkv: int, hd: int, kv_len: int, is_full: bool) -> Fixture:
    """attention/mod.rs:128-167"""
    assert nq % nkv == 0
    tt = kv_len + canvas
    t = np.arange(tt, dtype=np.int64)[:, None, None]
    h = np.arange(nkv, dtype=np.int64)[None, :, None]
    d = np.arange(hd, dtype=np.int64)[None, None, :]
    k = np.sin(_f32(t * 19 + h * 7 + d) * _f32(0.0031)) * _f32(0.4)
    v = np.cos(_f32(t * 23 + h * 11 + d) * _f32(0.0027)) * _f32(0.35)
    kv = np.concatenate([k.reshape(tt, nkv * hd), v.reshape(tt, nkv * hd)], axis=1).astype(np.float32)
    i = np.arange(canvas * nq * hd, dtype=np.int64)
    q = (np.sin(_f32(i) * _f32(0.017)) * _f32(0.5) + _f32(0.02) * _f32(i % hd)).astype(np.float32)
    return Fixture(q, kv.reshape(-1), LayerAttnParams(hd, nkv, is_full, 0 if is_full else 1), canvas, nq, kv_len)


def full_hd512_fixture() -> Fixture:
    return model_attn_fixture(4, 16, 8, 512, 28, True)


def full_grp8_hd512_fixture() -> Fixture:
    return model_attn_fixture(16, 16, 2, 512, 28, True)


def sliding_hd256_fixture() -> Fixture:
    return model_attn_fixture(4, 16, 8, 256, 128, False)


def model_bench_fixture(hd: int, kv_len: int, is_full: bool) -> Fixture:
    """attention/mod.rs:689-691"""
    return model_attn_fixture(256, 16, 8, hd, kv_len, is_full)


def model_full_fixture(kv_len: int, canvas: int = 256) -> Fixture:
    """src/shaders/attn/attention_gemm/mod.rs:364-432"""
    nq, nkv, hd = 16, 2, 512
    tt = kv_len + canvas
    i = np.arange(tt * nkv * hd * 2, dtype=np.int64)
    kv = (np.sin(_f32(i % 4096) * _f32(0.0007)) * _f32(0.35)).astype(np.float32)
    j = np.arange(canvas * nq * hd, dtype=np.int64)
    q = (np.sin(_f32(j) * _f32(0.013)) * _f32(0.4)).astype(np.float32)
    return Fixture(q, kv, LayerAttnParams(hd, nkv, True, 0), canvas, nq, kv_len)


def layer_offsets(f: Fixture, kv_ring_mask: int = 0) -> capi.LayerOffsets:
    """attention/mod.rs:186-216"""
    lo = capi.LayerOffsets()
    lo.v_proj = f.layer.v_proj
    lo.kv_region = f.layer.kv_region
    lo.head_dim = f.layer.head_dim
    lo.n_kv_heads = f.layer.n_kv_heads
    lo.is_full = 1 if f.layer.is_full else 0
    lo.kv_ring_mask = kv_ring_mask
    return lo


def step_params(kv_len: int) -> capi.StepParams:
    """the StepParams literal the reference harnesses use (attention/mod.rs:417-430)"""
    return capi.StepParams(kv_len=kv_len, max_steps=8, entropy_bound=0.0, t_min=0.0, t_max=1.0,
                           conf_threshold=0.0, stability_threshold=0, min_early_stop_steps=0,
                           accept_plateau_threshold=0, plateau_prefix_mean_max=3.4028234663852886e38,
                           eos_token_id=1, kv_write_end=0xFFFFFFFF)


def make_desc(canvas: int, n_q_heads: int, n_kv_heads: int, head_dim: int, kv_len: int, *, causal_rows: int = 0,
              window: int = 0, kv_ring_mask: int = 0, q_dtype: int = capi.DG_BF16, kv_dtype: int = capi.DG_BF16,
              out_dtype: int = capi.DG_BF16, flags: int = 0, t_lo: int = 0, n_splits: int = 0,
              kernel: int = capi.DG_KERNEL_AUTO, softmax_scale: float = 0.0, kv_region_bytes: int = 0,
              layout: str = "reference", t_cap: Optional[int] = None) -> capi.AttnDesc:
    d = capi.AttnDesc(canvas=canvas, n_q_heads=n_q_heads, n_kv_heads=n_kv_heads, head_dim=head_dim, kv_len=kv_len,
                      causal_rows=causal_rows, window=window, kv_ring_mask=kv_ring_mask, q_dtype=q_dtype,
                      kv_dtype=kv_dtype, out_dtype=out_dtype, flags=flags, t_lo=t_lo, n_splits=n_splits,
                      kernel=kernel, softmax_scale=softmax_scale, kv_region_bytes=kv_region_bytes)
    lib = capi.load()
    if layout == "reference":
        lib.dg_attn_desc_reference_layout(C.byref(d))
    elif layout == "head_major":
        lib.dg_attn_desc_head_major_layout(C.byref(d), t_cap if t_cap is not None else kv_len + canvas)
    else:
        raise ValueError(layout)
    return d


# ---------------------------------------------------------------------------------------
# device plumbing (torch = memory + streams only)
# ---------------------------------------------------------------------------------------

def _torch():
    import torch
    if not torch.cuda.is_available():
        raise RuntimeError("no HIP device: the attention path runs only on a gfx950 GPU")
    return torch


def to_device_bits(bits: np.ndarray):
    """uint16 bit patterns -> device int16 tensor (bit-exact)."""
    torch = _torch()
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda()


def stream_handle() -> int:
    return _torch().cuda.current_stream().cuda_stream


def forward(desc: capi.AttnDesc, q, kv, out, lse=None, workspace=None) -> None:
    """dg_attn_forward on torch device tensors, on torch's current stream."""
    lib = capi.load()
    ws_ptr, ws_bytes = (workspace.data_ptr(), workspace.numel() * workspace.element_size()) if workspace is not None else (None, 0)
    capi.check(lib.dg_attn_forward(C.byref(desc), q.data_ptr(), kv.data_ptr(), out.data_ptr(),
                                   lse.data_ptr() if lse is not None else None, ws_ptr, ws_bytes, stream_handle()))


def forward_dev(desc: capi.AttnDesc, step_dev, q, kv, out, lse=None, workspace=None) -> None:
    """dg_attn_forward_dev: kv_len is read from the device StepParams `step_dev` (an int32 tensor of 12 words,
    kv_len first) when the kernels run; desc.kv_len is the largest prefix planned for."""
    lib = capi.load()
    ws_ptr, ws_bytes = (workspace.data_ptr(), workspace.numel() * workspace.element_size()) if workspace is not None else (None, 0)
    capi.check(lib.dg_attn_forward_dev(C.byref(desc), step_dev.data_ptr(), q.data_ptr(), kv.data_ptr(), out.data_ptr(),
                                       lse.data_ptr() if lse is not None else None, ws_ptr, ws_bytes, stream_handle()))


def device_step_params(kv_len: int, kv_write_end: int = 0xFFFFFFFF):
    """A device copy of the reference's StepParams (12 words; kv_len is word 0, kv_write_end word 11)."""
    torch = _torch()
    host = np.zeros(12, dtype=np.uint32)
    host[0], host[11] = kv_len, kv_write_end
    return torch.from_numpy(host.view(np.int32)).cuda()


def state_bytes(desc: capi.AttnDesc) -> int:
    n = C.c_size_t(0)
    capi.check(capi.load().dg_attn_state_bytes(C.byref(desc), C.byref(n)))
    return n.value


def alloc_state(desc: capi.AttnDesc):
    """Device memory for one attention state (m, l, acc) of `desc`."""
    return _torch().empty(state_bytes(desc), dtype=_torch().uint8, device="cuda")


def partial(desc: capi.AttnDesc, t_begin: int, t_end: int, q, kv, state) -> None:
    """State of the keys [t_begin, t_end) under desc's mask (dg_attn_partial); the workspace is made here."""
    torch = _torch()
    n = C.c_size_t(0)
    lib = capi.load()
    capi.check(lib.dg_attn_partial_workspace_bytes(C.byref(desc), t_begin, t_end, C.byref(n)))
    ws = torch.empty(max(n.value, 256), dtype=torch.uint8, device="cuda")
    capi.check(lib.dg_attn_partial(C.byref(desc), t_begin, t_end, q.data_ptr(), kv.data_ptr(), state.data_ptr(),
                                   state.numel(), ws.data_ptr(), ws.numel(), stream_handle()))
    torch.cuda.current_stream().synchronize()   # ws is released on return


def merge(desc: capi.AttnDesc, states, out=None, lse=None, state_out=None) -> None:
    """dg_attn_merge of a list of states into out (+ lse) and/or a state."""
    arr = (C.c_void_p * len(states))(*[s.data_ptr() for s in states])
    capi.check(capi.load().dg_attn_merge(C.byref(desc), arr, len(states), out.data_ptr() if out is not None else None,
                                         lse.data_ptr() if lse is not None else None,
                                         state_out.data_ptr() if state_out is not None else None, stream_handle()))


def read_state(desc: capi.AttnDesc, state):
    """(m [rows], l [rows], acc [rows, hd]) of a state, rows = canvas * n_q_heads, as numpy arrays."""
    rows = desc.canvas * desc.n_q_heads
    f = state.cpu().numpy().view(np.float32)
    off = (2 * rows + 3) & ~3
    return f[:rows].copy(), f[rows:2 * rows].copy(), f[off:off + rows * desc.head_dim].reshape(rows, desc.head_dim).copy()


def alloc_workspace(desc: capi.AttnDesc):
    torch = _torch()
    n = capi.workspace_bytes(desc)
    return torch.empty(max(n, 256), dtype=torch.uint8, device="cuda")


@dataclass
class AttnRig:
    """Fixture -> device buffers -> dispatch -> readback / timing (harness.rs:21-181)."""
    fixture: Fixture
    buf_q: object = None
    buf_kv: object = None
    buf_out: object = None
    buf_lse: object = None
    buf_dbg: object = None
    kv_ring_mask: int = 0
    _ws: dict = field(default_factory=dict)

    @classmethod
    def from_fixture(cls, f: Fixture, kv_slack_slots: int = KV_SLACK_SLOTS) -> "AttnRig":
        torch = _torch()
        rig = cls(f)
        rig.buf_q = to_device_bits(rounding.f32_to_bf16_bits_trunc(f.q))
        kstride = f.n_kv() * f.head_dim() * 2
        bits = rounding.f32_to_f16_bits_trunc(f.kvcache)
        bits = np.concatenate([bits, np.zeros(kv_slack_slots * kstride, dtype=np.uint16)])
        rig.buf_kv = to_device_bits(bits)
        rig.buf_out = torch.zeros(f.out_len(), dtype=torch.int16, device="cuda")
        rig.buf_lse = torch.zeros(f.canvas * f.n_q_heads, dtype=torch.float32, device="cuda")
        rig.buf_dbg = torch.zeros(4, dtype=torch.int32, device="cuda")
        return rig

    def desc(self, *, causal: int = 0, window: int = 0, kernel: int = capi.DG_KERNEL_AUTO,
             n_splits: int = 0, truncate: bool = True) -> capi.AttnDesc:
        f = self.fixture
        return make_desc(f.canvas, f.n_q_heads, f.n_kv(), f.head_dim(), f.kv_len,
                         causal_rows=f.canvas if causal else 0, window=window, kv_ring_mask=self.kv_ring_mask,
                         q_dtype=capi.DG_BF16, kv_dtype=capi.DG_F16, out_dtype=capi.DG_BF16,
                         flags=capi.DG_ATTN_F_OUT_TRUNCATE if truncate else 0, n_splits=n_splits, kernel=kernel,
                         kv_region_bytes=f.layer.kv_region)

    def workspace_for(self, desc: capi.AttnDesc):
        n = capi.workspace_bytes(desc)
        if n not in self._ws:
            self._ws[n] = _torch().empty(max(n, 256), dtype=_torch().uint8, device="cuda")
        return self._ws[n]

    def run_forward(self, desc: capi.AttnDesc) -> None:
        forward(desc, self.buf_q, self.buf_kv, self.buf_out, self.buf_lse, self.workspace_for(desc))

    def run_dispatch(self, *, causal: int = 0, window: int = 0) -> None:
        """The reference-shaped entry: the buffers encode_layer_attention_dispatch binds."""
        f = self.fixture
        lib = capi.load()
        lo = layer_offsets(f, self.kv_ring_mask)
        sp = step_params(f.kv_len)
        dims = capi.AttnDims(canvas=f.canvas, n_q_heads=f.n_q_heads, causal=causal, window=window)
        n = C.c_size_t(0)
        capi.check(lib.dg_attention_state_bytes(C.byref(lo), C.byref(dims), f.kv_len, C.byref(n)))
        key = ("state", n.value)
        if key not in self._ws:
            self._ws[key] = _torch().empty(max(n.value, 256), dtype=_torch().uint8, device="cuda")
        st = self._ws[key]
        capi.check(lib.dg_attention_dispatch(self.buf_q.data_ptr(), self.buf_kv.data_ptr(), self.buf_out.data_ptr(),
                                             C.byref(lo), C.byref(sp), C.byref(dims), self.buf_dbg.data_ptr(),
                                             st.data_ptr(), st.numel(), stream_handle()))

    def run_dispatch_dev(self, *, causal: int = 0, window: int = 0, kv_len_max: Optional[int] = None) -> None:
        """run_dispatch with StepParams bound as the reference binds it (enc.rs:2177-2220, buf4): a device buffer
        whose kv_len the kernels read when they run; the host only says how far the prefix can grow."""
        f = self.fixture
        lib = capi.load()
        lo = layer_offsets(f, self.kv_ring_mask)
        kv_len_max = f.kv_len if kv_len_max is None else kv_len_max
        self.step_dev = device_step_params(f.kv_len)
        dims = capi.AttnDims(canvas=f.canvas, n_q_heads=f.n_q_heads, causal=causal, window=window)
        n = C.c_size_t(0)
        capi.check(lib.dg_attention_state_bytes(C.byref(lo), C.byref(dims), kv_len_max, C.byref(n)))
        key = ("state", n.value)
        if key not in self._ws:
            self._ws[key] = _torch().empty(max(n.value, 256), dtype=_torch().uint8, device="cuda")
        st = self._ws[key]
        capi.check(lib.dg_attention_dispatch_dev(self.buf_q.data_ptr(), self.buf_kv.data_ptr(), self.buf_out.data_ptr(),
                                                 C.byref(lo), self.step_dev.data_ptr(), kv_len_max, C.byref(dims),
                                                 self.buf_dbg.data_ptr(), st.data_ptr(), st.numel(), stream_handle()))

    def time_rounds(self, iters: int, encode, rounds: int = 6):
        """6 rounds of `iters` back-to-back launches, round 0 discarded; returns
        (min, median) mean-ms-per-launch over the kept rounds (harness.rs:149-170)."""
        torch = _torch()
        per = []
        for rnd in range(rounds):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                encode()
            e1.record()
            e1.synchronize()
            if rnd > 0:
                per.append(e0.elapsed_time(e1) / iters)
        return min(per), float(np.median(per))

    def read_out_f32(self) -> np.ndarray:
        _torch().cuda.synchronize()
        bits = self.buf_out.cpu().numpy().view(np.uint16)
        return rounding.bf16_bits_to_f32(bits)

    def read_lse(self) -> np.ndarray:
        _torch().cuda.synchronize()
        return self.buf_lse.cpu().numpy().copy()

    def read_debug_status(self) -> capi.DebugStatus:
        _torch().cuda.synchronize()
        w = self.buf_dbg.cpu().numpy().view(np.uint32)
        return capi.DebugStatus(int(w[0]), int(w[1]), int(w[2]), int(w[3]))


def gpu(f: Fixture) -> np.ndarray:
    """Scalar cross-check kernel (the reference's `attention` kernel role, mod.rs:377-471)."""
    rig = AttnRig.from_fixture(f)
    rig.run_forward(rig.desc(kernel=capi.DG_KERNEL_SCALAR))
    return rig.read_out_f32()


def gpu_mma(f: Fixture, *, causal: int = 0, window: int = 0) -> np.ndarray:
    """MFMA kernel through the reference-shaped dispatch entry (roles of gpu_mma2 /
    gpu_mma_full, mod.rs:484-686: one kernel family covers hd<=256 and hd=512 here)."""
    rig = AttnRig.from_fixture(f)
    rig.run_dispatch(causal=causal, window=window)
    return rig.read_out_f32()


gpu_mma2 = gpu_mma
gpu_mma_full = gpu_mma


def bench_path(f: Fixture, iters: int, path: int) -> float:
    """mean ms/dispatch, min over rounds (attention/mod.rs:698-831). path 0 = scalar, else MFMA."""
    rig = AttnRig.from_fixture(f)
    desc = rig.desc(kernel=capi.DG_KERNEL_SCALAR if path == 0 else capi.DG_KERNEL_MFMA)
    rig.run_forward(desc)
    best, _ = rig.time_rounds(iters, lambda: rig.run_forward(desc))
    return best
