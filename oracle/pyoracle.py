"""ctypes binding of the CPU oracle (libdg_attn_oracle.so).  TEST INFRASTRUCTURE ONLY.

Imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg — never by the
diffgemma_amd package.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
LIB_PATH = ORACLE_DIR / "libdg_attn_oracle.so"


class Desc(C.Structure):
    _fields_ = [
        ("canvas", C.c_uint32), ("n_q_heads", C.c_uint32), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
        ("kv_len", C.c_uint32), ("causal_rows", C.c_uint32), ("window", C.c_uint32), ("kv_ring_mask", C.c_uint32),
        ("causal_sees_masked", C.c_uint32), ("strict_order", C.c_uint32),
        ("t_lo_override", C.c_int64),
        ("k_off", C.c_int64), ("k_tok_stride", C.c_int64), ("k_head_stride", C.c_int64),
        ("v_off", C.c_int64), ("v_tok_stride", C.c_int64), ("v_head_stride", C.c_int64),
        ("scale", C.c_float),
    ]


class RopeDesc(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("canvas", "n_q_heads", "n_kv_heads", "head_dim", "kv_len", "kv_write_end",
                                           "kv_ring_mask", "is_full", "v_from_k")] + \
               [(n, C.c_int64) for n in ("k_off", "k_tok_stride", "k_head_stride", "v_off", "v_tok_stride",
                                          "v_head_stride")]


def build(force: bool = False) -> Path:
    if force or not LIB_PATH.exists():
        subprocess.run(["make", "-C", str(ORACLE_DIR), "-B" if force else "-s"], check=True,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB_PATH


_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        build()
    lib = C.CDLL(str(LIB_PATH))
    P, VP = C.POINTER, C.c_void_p
    lib.dgo_desc_reference_layout.argtypes = [P(Desc)]
    lib.dgo_desc_head_major_layout.argtypes = [P(Desc), C.c_int64]
    lib.dgo_visible.argtypes = [P(Desc), C.c_uint32, C.c_uint32]
    lib.dgo_visible.restype = C.c_int
    lib.dgo_visible_pairs.argtypes = [P(Desc)]
    lib.dgo_visible_pairs.restype = C.c_uint64
    lib.dgo_attention_f32.argtypes = [P(Desc), VP, VP, VP, VP, VP, C.c_uint32, C.c_int]
    lib.dgo_attention_f64.argtypes = [P(Desc), VP, VP, VP, VP, VP, C.c_uint32, C.c_int]
    lib.dgo_attention_topk_f32.argtypes = [P(Desc), P(C.c_uint32), VP, VP, VP, VP, C.c_uint32, VP, VP, C.c_uint32, C.c_int]
    lib.dgo_topk_row_k.argtypes = [P(C.c_uint32), C.c_uint32, C.c_int]
    lib.dgo_topk_row_k.restype = C.c_uint32
    lib.dgo_fnv1a64.argtypes = [VP, C.c_size_t, C.c_uint64]
    lib.dgo_fnv1a64.restype = C.c_uint64
    lib.dgo_attention_blocked_f32.argtypes = [P(Desc), VP, VP, VP, VP, C.c_uint32, C.c_int]
    lib.dgo_attention_partial_f32.argtypes = [P(Desc), VP, VP, C.c_uint32, C.c_uint32, VP, VP, VP, C.c_int]
    lib.dgo_merge_partials_f32.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, VP, VP, VP, VP, VP]
    lib.dgo_attention_bitmap_f32.argtypes = [C.c_uint32] * 5 + [VP] * 5
    for name in ("dgo_f32_to_bf16_trunc", "dgo_f32_to_bf16_rne", "dgo_f32_to_f16_trunc", "dgo_f32_to_f16_rne"):
        getattr(lib, name).argtypes = [C.c_float]
        getattr(lib, name).restype = C.c_uint16
    lib.dgo_bf16_to_f32.argtypes = [C.c_uint16]
    lib.dgo_bf16_to_f32.restype = C.c_float
    lib.dgo_f16_to_f32.argtypes = [C.c_uint16]
    lib.dgo_f16_to_f32.restype = C.c_float
    lib.dgo_round_array.argtypes = [VP, C.c_size_t, C.c_int]
    lib.dgo_to_bits.argtypes = [VP, VP, C.c_size_t, C.c_int]
    lib.dgo_from_bits.argtypes = [VP, VP, C.c_size_t, C.c_int]
    lib.dgo_rms_norm_no_scale.argtypes = [VP, VP, C.c_size_t, C.c_float]
    lib.dgo_rms_norm_head.argtypes = [VP, VP, C.c_size_t, C.c_float]
    lib.dgo_fixture_tiny.argtypes = [VP, VP]
    lib.dgo_fixture_wide.argtypes = [VP, VP]
    lib.dgo_fixture_model_attn.argtypes = [C.c_uint32] * 5 + [VP, VP]
    lib.dgo_fixture_model_full.argtypes = [C.c_uint32] * 5 + [VP, VP]
    lib.dgo_synthetic_fill_kv.argtypes = [VP, C.c_size_t, C.c_uint64]
    lib.dgo_rope_split_half.argtypes = [VP, C.c_uint32, C.c_uint32, C.c_float, C.c_uint32]
    lib.dgo_rope_proportional.argtypes = [VP, C.c_uint32, C.c_uint32, C.c_float, C.c_uint32]
    lib.dgo_qk_rope_kv_f32.argtypes = [C.POINTER(RopeDesc), VP, VP, VP, VP, VP, VP]
    lib.dgo_fixture_rope.argtypes = [C.c_int, VP, VP, VP, VP, VP]
    lib.dgo_rms_norm_head.argtypes = [VP, VP, C.c_size_t, C.c_float]
    lib.dgo_max_threads.restype = C.c_int
    _lib = lib
    return lib


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def make_desc(canvas, n_q_heads, n_kv_heads, head_dim, kv_len, *, causal_rows=0, window=0, kv_ring_mask=0,
              causal_sees_masked=0, strict_order=0, t_lo_override=-1, scale=1.0, layout="reference", t_cap=None):
    d = Desc(canvas=canvas, n_q_heads=n_q_heads, n_kv_heads=n_kv_heads, head_dim=head_dim, kv_len=kv_len,
             causal_rows=causal_rows, window=window, kv_ring_mask=kv_ring_mask,
             causal_sees_masked=causal_sees_masked, strict_order=strict_order, t_lo_override=t_lo_override,
             scale=scale)
    lib = load()
    if layout == "reference":
        lib.dgo_desc_reference_layout(C.byref(d))
    elif layout == "head_major":
        lib.dgo_desc_head_major_layout(C.byref(d), t_cap if t_cap is not None else kv_len + canvas)
    else:
        raise ValueError(layout)
    return d


def _toks(tok_list):
    if tok_list is None:
        return None, 0
    t = np.ascontiguousarray(tok_list, dtype=np.uint32)
    return t, len(t)


def attention_f32(desc, q, kv, tok_list=None, n_threads=0):
    """Returns (out [canvas,Hq,hd] f32, lse [canvas,Hq] f32); rows not in tok_list stay 0."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    kv = np.ascontiguousarray(kv, dtype=np.float32)
    out = np.zeros((desc.canvas, desc.n_q_heads, desc.head_dim), dtype=np.float32)
    lse = np.zeros((desc.canvas, desc.n_q_heads), dtype=np.float32)
    t, n = _toks(tok_list)
    load().dgo_attention_f32(C.byref(desc), _ptr(q), _ptr(kv), _ptr(out), _ptr(lse), _ptr(t), n, n_threads)
    return out, lse


def topk_row_k(k_cfg, n_valid: int, causal_row: bool) -> int:
    cfg = (C.c_uint32 * 4)(*k_cfg)
    return int(load().dgo_topk_row_k(cfg, n_valid, 1 if causal_row else 0))


def attention_topk_f32(desc, k_cfg, q, kv, tok_list=None, sel_cap=0, n_threads=0):
    """Top-k sparse attention.  Returns out [canvas,Hq,hd] f32, or (out, sel_idx [canvas,Hq,sel_cap],
    sel_count [canvas,Hq]) when sel_cap > 0."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    kv = np.ascontiguousarray(kv, dtype=np.float32)
    out = np.zeros((desc.canvas, desc.n_q_heads, desc.head_dim), dtype=np.float32)
    cfg = (C.c_uint32 * 4)(*k_cfg)
    t, n = _toks(tok_list)
    if sel_cap > 0:
        idx = np.full((desc.canvas, desc.n_q_heads, sel_cap), 0xFFFFFFFF, dtype=np.uint32)
        cnt = np.zeros((desc.canvas, desc.n_q_heads), dtype=np.uint32)
        load().dgo_attention_topk_f32(C.byref(desc), cfg, _ptr(q), _ptr(kv), _ptr(out), _ptr(idx), sel_cap, _ptr(cnt),
                                      _ptr(t), n, n_threads)
        return out, idx, cnt
    load().dgo_attention_topk_f32(C.byref(desc), cfg, _ptr(q), _ptr(kv), _ptr(out), None, 0, None, _ptr(t), n, n_threads)
    return out


def attention_f64(desc, q, kv, tok_list=None, n_threads=0):
    q = np.ascontiguousarray(q, dtype=np.float32)
    kv = np.ascontiguousarray(kv, dtype=np.float32)
    out = np.zeros((desc.canvas, desc.n_q_heads, desc.head_dim), dtype=np.float64)
    lse = np.zeros((desc.canvas, desc.n_q_heads), dtype=np.float64)
    t, n = _toks(tok_list)
    load().dgo_attention_f64(C.byref(desc), _ptr(q), _ptr(kv), _ptr(out), _ptr(lse), _ptr(t), n, n_threads)
    return out, lse


def attention_blocked_f32(desc, q, kv, bk, n_threads=0):
    q = np.ascontiguousarray(q, dtype=np.float32)
    kv = np.ascontiguousarray(kv, dtype=np.float32)
    out = np.zeros((desc.canvas, desc.n_q_heads, desc.head_dim), dtype=np.float32)
    lse = np.zeros((desc.canvas, desc.n_q_heads), dtype=np.float32)
    load().dgo_attention_blocked_f32(C.byref(desc), _ptr(q), _ptr(kv), _ptr(out), _ptr(lse), bk, n_threads)
    return out, lse


def attention_partial_f32(desc, q, kv, t_begin, t_end, n_threads=0):
    q = np.ascontiguousarray(q, dtype=np.float32)
    kv = np.ascontiguousarray(kv, dtype=np.float32)
    rows = desc.canvas * desc.n_q_heads
    acc = np.zeros((rows, desc.head_dim), dtype=np.float32)
    m = np.zeros(rows, dtype=np.float32)
    l = np.zeros(rows, dtype=np.float32)
    load().dgo_attention_partial_f32(C.byref(desc), _ptr(q), _ptr(kv), t_begin, t_end, _ptr(acc), _ptr(m), _ptr(l),
                                     n_threads)
    return acc, m, l


def merge_partials_f32(parts, head_dim):
    """parts: list of (acc [rows,hd], m [rows], l [rows])."""
    n = len(parts)
    rows = parts[0][1].shape[0]
    arr = lambda i: (C.c_void_p * n)(*[p[i].ctypes.data for p in parts])
    out = np.zeros((rows, head_dim), dtype=np.float32)
    lse = np.zeros(rows, dtype=np.float32)
    load().dgo_merge_partials_f32(rows, head_dim, n, arr(0), arr(1), arr(2), _ptr(out), _ptr(lse))
    return out, lse


def attention_bitmap_f32(q, k, v, mask, n_heads, n_kv_heads, head_dim):
    """q [seq,Hq,hd], k/v [total_kv,Hkv,hd], mask [seq,total_kv] bool."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    mask = np.ascontiguousarray(mask, dtype=np.uint8)
    seq, total = mask.shape
    out = np.zeros((seq, n_heads, head_dim), dtype=np.float32)
    load().dgo_attention_bitmap_f32(seq, total, n_heads, n_kv_heads, head_dim, _ptr(q), _ptr(k), _ptr(v), _ptr(mask),
                                    _ptr(out))
    return out


def visible_matrix(desc):
    lib = load()
    t_all = desc.kv_len + desc.canvas
    m = np.zeros((desc.canvas, t_all), dtype=bool)
    for tok in range(desc.canvas):
        for t in range(t_all):
            m[tok, t] = bool(lib.dgo_visible(C.byref(desc), tok, t))
    return m


ROUND_BF16_TRUNC, ROUND_BF16_RNE, ROUND_F16_TRUNC, ROUND_F16_RNE = 0, 1, 2, 3


def round_array(x, mode):
    y = np.array(x, dtype=np.float32, copy=True, order="C")
    load().dgo_round_array(_ptr(y), y.size, mode)
    return y


def to_bits(x, mode):
    x = np.ascontiguousarray(x, dtype=np.float32)
    b = np.zeros(x.shape, dtype=np.uint16)
    load().dgo_to_bits(_ptr(x), _ptr(b), x.size, mode)
    return b


def from_bits(b, is_f16):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    x = np.zeros(b.shape, dtype=np.float32)
    load().dgo_from_bits(_ptr(b), _ptr(x), b.size, 1 if is_f16 else 0)
    return x


def rms_norm_no_scale(x, eps=1e-6):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros_like(x)
    load().dgo_rms_norm_no_scale(_ptr(out), _ptr(x), x.size, eps)
    return out


def fixture(name, *dims):
    """Reference fixture generators; returns (q, kv) flat f32 arrays."""
    lib = load()
    if name == "tiny":
        q, kv = np.zeros(2 * 4 * 32, np.float32), np.zeros(4 * 2 * 32 * 2, np.float32)
        lib.dgo_fixture_tiny(_ptr(q), _ptr(kv))
    elif name == "wide":
        q, kv = np.zeros(4 * 8 * 64, np.float32), np.zeros(8 * 2 * 64 * 2, np.float32)
        lib.dgo_fixture_wide(_ptr(q), _ptr(kv))
    elif name in ("model_attn", "model_full"):
        canvas, nq, nkv, hd, kv_len = dims
        q = np.zeros(canvas * nq * hd, np.float32)
        kv = np.zeros((kv_len + canvas) * nkv * hd * 2, np.float32)
        getattr(lib, "dgo_fixture_" + name)(canvas, nq, nkv, hd, kv_len, _ptr(q), _ptr(kv))
    else:
        raise ValueError(name)
    return q, kv


def make_rope_desc(canvas, n_q_heads, n_kv_heads, head_dim, kv_len, *, is_full=False, v_from_k=False,
                   kv_write_end=0xFFFFFFFF, kv_ring_mask=0, layout="reference", t_cap=0):
    """Producer descriptor; cache strides as in make_desc (reference slot-major or head-major planes)."""
    d = RopeDesc(canvas, n_q_heads, n_kv_heads, head_dim, kv_len, kv_write_end, kv_ring_mask, int(is_full),
                 int(v_from_k))
    row = n_kv_heads * head_dim
    if layout == "reference":
        d.k_off, d.k_tok_stride, d.k_head_stride = 0, 2 * row, head_dim
        d.v_off, d.v_tok_stride, d.v_head_stride = row, 2 * row, head_dim
    else:
        d.k_off, d.k_tok_stride, d.k_head_stride = 0, head_dim, t_cap * head_dim
        d.v_off, d.v_tok_stride, d.v_head_stride = n_kv_heads * t_cap * head_dim, head_dim, t_cap * head_dim
    return d


def qk_rope_kv_f32(d, q, k, v, kvcache, q_norm_w, k_norm_w):
    """Returns (q', k', kvcache') as new f32 arrays; inputs are not modified."""
    q = np.array(q, dtype=np.float32).ravel()
    k = np.array(k, dtype=np.float32).ravel()
    v = np.ascontiguousarray(v, dtype=np.float32).ravel()
    kvc = np.array(kvcache, dtype=np.float32).ravel()
    qw = np.ascontiguousarray(q_norm_w, dtype=np.float32)
    kw = np.ascontiguousarray(k_norm_w, dtype=np.float32)
    load().dgo_qk_rope_kv_f32(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(kvc), _ptr(qw), _ptr(kw))
    return q, k, kvc


def rope(x, rot, head_dim, theta, pos, proportional):
    x = np.array(x, dtype=np.float32)
    fn = load().dgo_rope_proportional if proportional else load().dgo_rope_split_half
    fn(_ptr(x), rot, head_dim, theta, pos)
    return x


def rms_norm_head(x, w=None, eps=1e-6):
    x = np.array(x, dtype=np.float32)
    wv = None if w is None else np.ascontiguousarray(w, dtype=np.float32)
    load().dgo_rms_norm_head(_ptr(x), None if wv is None else _ptr(wv), x.size, eps)
    return x


ROPE_FIXTURES = {  # name -> (which, canvas, Hq, Hkv, hd, kv_len, is_full, v_from_k); qk_rope_kv/mod.rs:80-189
    "tiny": (0, 2, 4, 2, 32, 2, False, False),
    "full_layer": (1, 2, 4, 2, 64, 2, True, False),
    "full_attn_v_alias": (1, 2, 4, 2, 64, 2, True, True),
    "full_hd512_v_alias": (2, 1, 16, 2, 512, 22, True, True),
}


def rope_fixture(name):
    """(dims dict, q, k, v, q_norm_w, k_norm_w) of one of the reference's producer fixtures."""
    which, canvas, nq, nkv, hd, kv_len, is_full, v_from_k = ROPE_FIXTURES[name]
    q = np.zeros(canvas * nq * hd, np.float32)
    k = np.zeros(canvas * nkv * hd, np.float32)
    v = np.zeros(canvas * nkv * hd, np.float32)
    qw, kw = np.zeros(hd, np.float32), np.zeros(hd, np.float32)
    load().dgo_fixture_rope(which, _ptr(q), _ptr(k), _ptr(v), _ptr(qw), _ptr(kw))
    dims = dict(canvas=canvas, n_q_heads=nq, n_kv_heads=nkv, head_dim=hd, kv_len=kv_len, is_full=is_full,
                v_from_k=v_from_k)
    return dims, q, k, v, qw, kw


def synthetic_fill_kv(n, seed):
    b = np.zeros(n, dtype=np.uint16)
    load().dgo_synthetic_fill_kv(_ptr(b), n, seed)
    return b


def max_threads():
    return load().dgo_max_threads()


# ---------------------------------------------------------------------------------------
# KV snapshots and the live-KV fingerprint, on a cache held in the reference's own layout
# (one byte buffer; per layer a region of `slots` positions, each [K: Hkv*hd | V: Hkv*hd] elements).
# `layers`: objects with kv_region (byte offset), n_kv_heads, head_dim, slots, kv_ring_mask.
# ---------------------------------------------------------------------------------------

FNV_OFFSET_BASIS = 0xcbf29ce484222325


def fnv1a64(data: bytes, seed_hash: int = FNV_OFFSET_BASIS) -> int:
    buf = np.frombuffer(bytes(data), dtype=np.uint8)
    return int(load().dgo_fnv1a64(_ptr(buf) if buf.size else None, buf.size, seed_hash))


def _group_bytes(l, elem_bytes):
    return 2 * l.n_kv_heads * l.head_dim * elem_bytes


def kv_gather_prefix(cache: np.ndarray, layers, kv_len: int, elem_bytes: int = 2) -> np.ndarray:
    """src/metal/step_kv/mod.rs:108-127: per layer the first min(kv_len, slots) slots of the region, concatenated."""
    out = []
    for l in layers:
        n = min(kv_len, l.slots) * _group_bytes(l, elem_bytes)
        out.append(cache[l.kv_region:l.kv_region + n])
    return np.concatenate(out) if out else np.zeros(0, np.uint8)


def kv_scatter_prefix(cache: np.ndarray, layers, kv_len: int, blob: np.ndarray, elem_bytes: int = 2) -> None:
    """src/metal/step_kv/mod.rs:133-151: the inverse; bytes past each layer's live prefix stay as they are."""
    off = 0
    for l in layers:
        n = min(kv_len, l.slots) * _group_bytes(l, elem_bytes)
        cache[l.kv_region:l.kv_region + n] = blob[off:off + n]
        off += n


def kv_live_stream(cache: np.ndarray, layers, kv_len: int, window: int, elem_bytes: int = 2) -> np.ndarray:
    """The bytes live_kv_fnv eats, in its order (src/metal/step_kernel/runtime.rs:135-147)."""
    out = []
    for l in layers:
        g = _group_bytes(l, elem_bytes)
        if l.kv_ring_mask == 0:
            out.append(cache[l.kv_region:l.kv_region + kv_len * g])
        else:
            for p in range(max(0, kv_len - window), kv_len):
                o = l.kv_region + (p & l.kv_ring_mask) * g
                out.append(cache[o:o + g])
    return np.concatenate(out) if out else np.zeros(0, np.uint8)


def kv_live_fnv(cache: np.ndarray, layers, kv_len: int, window: int, seed_hash: int, elem_bytes: int = 2) -> int:
    return fnv1a64(kv_live_stream(cache, layers, kv_len, window, elem_bytes).tobytes(), seed_hash)
