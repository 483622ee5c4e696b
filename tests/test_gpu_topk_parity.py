"""GPU parity of top-k sparse attention (topk_scores_kernel + topk_select_kernel through the C ABI)
against the CPU oracle.  The reference's own matrix (attention_topk/mod.rs:463-534) first, then
selection exactness on inputs whose scores are exact in fp32, model-shaped rows with the
context-adaptive k, and the size-independent properties (k >= visible keys is dense attention,
k = 1 is the arg-max key's V row, run-to-run bit equality)."""
import ctypes as C

import numpy as np
import pytest

from diffgemma_amd import attention as A
from diffgemma_amd import attention_topk as T
from diffgemma_amd import capi, rounding as R, workloads as W
from helpers import assert_oracle, max_abs_diff, mean_abs_diff

pytestmark = pytest.mark.gpu


def topk_cpu(po, f, k, causal):
    """cpu::topk_causal / topk_denoise with round_kv_f16 = true (cpu.rs:28-38): Q -> bf16, KV -> f16,
    output -> bf16, all by the reference's truncating conversions."""
    q = R.bf16_bits_to_f32(R.f32_to_bf16_bits_trunc(f.q))
    kv = R.f16_bits_to_f32(R.f32_to_f16_bits_trunc(f.kvcache))
    d = po.make_desc(f.canvas, f.n_q_heads, f.n_kv(), f.head_dim(), f.kv_len, causal_rows=f.canvas if causal else 0)
    out = po.attention_topk_f32(d, T.fixed_k(k), q, kv)
    return po.round_array(out, po.ROUND_BF16_TRUNC).ravel()


# ------------------------------------------------------------------ the reference's tests
@pytest.mark.parametrize("causal,k,cos", [(True, 64, 0.9999), (False, 64, 0.9999), (True, 1, 0.999), (True, 128, 0.9999)])
def test_reference_full_grp8_fixture(gpu_ready, po, causal, k, cos):
    f = A.full_grp8_hd512_fixture()
    assert_oracle(T.gpu(f, causal, k), topk_cpu(po, f, k, causal), 2e-2, cos)


def test_reference_model_fixture_midsize(gpu_ready, po):
    """model_full_fixture (attention_gemm/mod.rs:364-432) at a prefix of many key tiles, k = 64."""
    f = A.model_full_fixture(1500, canvas=64)
    assert_oracle(T.gpu(f, True, 64), topk_cpu(po, f, 64, True), 2e-2, 0.9999)


def test_ragged_causal_tail(gpu_ready, po):
    """cpu.rs:315-323: canvas 256 behind 4 keys, k = 64 > the keys early rows see."""
    f = A.model_bench_fixture(512, 4, True)
    got = T.gpu(f, True, 64)
    assert np.isfinite(got).all()
    assert_oracle(got, topk_cpu(po, f, 64, True), 2e-2, 0.9999)


# ------------------------------------------------------------------ generic runner
def run_topk(po, canvas, hq, hkv, hd, kv_len, k_cfg, *, causal_rows=0, window=0, q=None, kv=None, seed=0, toks=None,
             kv_dtype=capi.DG_BF16):
    """bf16 (or f16) storage, fp32 output: isolates selection and arithmetic from the output store."""
    import torch
    rng = np.random.default_rng(seed)
    t_all = kv_len + canvas
    if q is None:
        q = rng.standard_normal((canvas, hq, hd)).astype(np.float32)
        kv = rng.standard_normal((t_all, 2, hkv, hd)).astype(np.float32)
        rms = lambda x: x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + 1e-6)
        q, kv = rms(q).astype(np.float32), rms(kv).astype(np.float32)
    to_bits, from_bits = ((R.f32_to_bf16_bits_rne, R.bf16_bits_to_f32) if kv_dtype == capi.DG_BF16
                          else (R.f32_to_f16_bits_rne, R.f16_bits_to_f32))
    qb, kb = R.f32_to_bf16_bits_rne(q), to_bits(kv)
    d = A.make_desc(canvas, hq, hkv, hd, kv_len, causal_rows=causal_rows, window=window, q_dtype=capi.DG_BF16,
                    kv_dtype=kv_dtype, out_dtype=capi.DG_F32)
    out = torch.zeros(canvas * hq * hd, dtype=torch.float32, device="cuda")
    T.forward(d, k_cfg, A.to_device_bits(qb.reshape(-1)), A.to_device_bits(kb.reshape(-1)), out, T.alloc_workspace(d, k_cfg))
    torch.cuda.synchronize()
    od = po.make_desc(canvas, hq, hkv, hd, kv_len, causal_rows=causal_rows, window=window)
    ref = po.attention_topk_f32(od, k_cfg, R.bf16_bits_to_f32(qb).reshape(q.shape), from_bits(kb).reshape(kv.shape),
                                tok_list=toks)
    got = out.cpu().numpy().reshape(canvas, hq, hd)
    rows = np.arange(canvas) if toks is None else np.asarray(toks)
    return got[rows], ref[rows]


# ------------------------------------------------------------------ selection exactness
EXACT = [
    # canvas, hq, hkv, hd, kv_len, causal_rows, window, k
    (9, 4, 2, 32, 300, 0, 0, 16),
    (9, 4, 2, 64, 300, 9, 0, 16),
    (33, 8, 2, 128, 1000, 20, 0, 64),      # mixed rows
    (16, 16, 8, 256, 700, 16, 301, 40),    # causal + window
    (40, 16, 2, 512, 2100, 0, 0, 100),
    (5, 2, 1, 64, 9000, 0, 0, 700),        # threshold class larger than the candidate list
    (5, 2, 1, 64, 9000, 5, 0, 1024),
    (64, 16, 2, 512, 3, 64, 0, 64),        # ragged: early rows see fewer than k keys
    (3, 2, 2, 32, 5000, 0, 0, 1),
]


@pytest.mark.parametrize("case", EXACT)
def test_selection_is_exact_on_exact_scores(gpu_ready, po, case):
    """Q and K hold few-bit dyadic values: every dot product is exact in fp32 whatever the order of
    summation, so the kernel and the oracle see identical scores, full of ties; the kept sets and
    with them the outputs have to agree to fp32 summation error."""
    canvas, hq, hkv, hd, kvl, cr, win, k = case
    rng = np.random.default_rng(hash(case) & 0xFFFF)
    q = (rng.integers(-2, 3, (canvas, hq, hd)) / 4).astype(np.float32)
    kv = (rng.integers(-2, 3, (kvl + canvas, 2, hkv, hd)) / 4).astype(np.float32)
    kv[:, 1] = rng.standard_normal(kv[:, 1].shape).astype(np.float32)
    got, ref = run_topk(po, canvas, hq, hkv, hd, kvl, (k, 0, 0, 0), causal_rows=cr, window=win, q=q, kv=kv)
    assert np.isfinite(got).all()
    assert max_abs_diff(got, ref) < 2e-5


def test_all_scores_equal_keeps_the_first_k_positions(gpu_ready, po):
    """A zero query ties every key: the k lowest positions are kept (more ties than any list holds)."""
    canvas, hq, hkv, hd, kvl, k = 2, 2, 1, 64, 6000, 50
    q = np.zeros((canvas, hq, hd), np.float32)
    rng = np.random.default_rng(1)
    kv = rng.standard_normal((kvl + canvas, 2, hkv, hd)).astype(np.float32)
    got, ref = run_topk(po, canvas, hq, hkv, hd, kvl, (k, 0, 0, 0), q=q, kv=kv)
    want = R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(kv[:k, 1, 0])).reshape(k, hd).mean(axis=0)
    assert max_abs_diff(ref[0, 0], want) < 1e-5       # the oracle agrees with the closed form
    assert max_abs_diff(got, ref) < 1e-5


# ------------------------------------------------------------------ model-shaped inputs
@pytest.mark.parametrize("case", [
    # canvas, hq, hkv, hd, kv_len, causal_rows, k_cfg
    (64, 16, 2, 512, 4096, 0, T.adaptive_k()),        # denoise rows: k = 4160 / 128 -> 64 (k_min)
    (64, 16, 2, 512, 12000, 0, T.adaptive_k()),       # k = 94
    (64, 16, 2, 512, 12000, 64, T.adaptive_k()),      # causal rows: per-row k on the 256 grid
    (48, 16, 8, 256, 3000, 0, (200, 0, 0, 0)),
    (256, 8, 4, 128, 512, 128, (32, 0, 0, 0)),
])
def test_model_shaped_rows(gpu_ready, po, case):
    canvas, hq, hkv, hd, kvl, cr, k_cfg = case
    toks = np.unique(np.linspace(0, canvas - 1, 12).round().astype(np.uint32))
    got, ref = run_topk(po, canvas, hq, hkv, hd, kvl, k_cfg, causal_rows=cr, seed=hash(case[:6]) & 0xFFFF, toks=toks)
    assert np.isfinite(got).all()
    # the kernel's scores (MFMA summation order) and the oracle's (sequential) differ in the last
    # bits; keys whose scores are that close to the k-th carry the smallest kept weights
    assert max_abs_diff(got, ref) <= 2e-2 and mean_abs_diff(got, ref) <= 2e-3


def test_f16_cache_with_bf16_queries(gpu_ready, po):
    got, ref = run_topk(po, 32, 16, 2, 512, 2000, (64, 0, 0, 0), seed=4, kv_dtype=capi.DG_F16)
    assert max_abs_diff(got, ref) <= 2e-2 and mean_abs_diff(got, ref) <= 2e-3


def test_global_layer_at_32k_prefix_rows(gpu_ready, po):
    """The denoise shape of a global layer (canvas 256, 16 / 2 heads, hd 512, prefix 32768) with the
    production k rule (258 keys per row); the oracle runs a row sample."""
    import torch
    w = W.config("cfg3_global")
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc(causal_rows=0)
    d.out_dtype = capi.DG_F32
    k_cfg = T.adaptive_k()
    out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.float32, device="cuda")
    T.forward(d, k_cfg, qd, kd, out, T.alloc_workspace(d, k_cfg))
    torch.cuda.synchronize()
    toks = np.array([0, 63, 64, 130, 255], dtype=np.uint32)
    od = po.make_desc(w.canvas, w.n_q_heads, w.n_kv_heads, w.head_dim, w.kv_len, layout=w.layout, t_cap=w.t_all)
    ref, idx, cnt = po.attention_topk_f32(od, k_cfg, q, kv, tok_list=toks, sel_cap=512)
    assert (cnt[toks] == 258).all()
    got = out.cpu().numpy().reshape(w.canvas, w.n_q_heads, w.head_dim)
    assert np.isfinite(got).all()
    assert max_abs_diff(got[toks], ref[toks]) <= 2e-2 and mean_abs_diff(got[toks], ref[toks]) <= 2e-3


def test_long_context_rows(gpu_ready, po):
    """131072-key prefix with 1% of the keys scaled x8 (config 4's inputs): k = 512 (the cap), score rows of
    525 KB, sixteen blocks of canvas rows."""
    import torch
    w = W.config("cfg4_long")
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc()
    d.out_dtype = capi.DG_F32
    k_cfg = T.adaptive_k()
    out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.float32, device="cuda")
    T.forward(d, k_cfg, qd, kd, out, T.alloc_workspace(d, k_cfg))
    torch.cuda.synchronize()
    toks = np.array([0, 17, 128, 255], dtype=np.uint32)
    od = po.make_desc(w.canvas, w.n_q_heads, w.n_kv_heads, w.head_dim, w.kv_len, layout=w.layout, t_cap=w.t_all)
    ref, idx, cnt = po.attention_topk_f32(od, k_cfg, q, kv, tok_list=toks, sel_cap=512)
    assert (cnt[toks] == 512).all()
    got = out.cpu().numpy().reshape(w.canvas, w.n_q_heads, w.head_dim)
    assert np.isfinite(got).all()
    assert max_abs_diff(got[toks], ref[toks]) <= 2e-2 and mean_abs_diff(got[toks], ref[toks]) <= 2e-3


# ------------------------------------------------------------------ edge cases
EDGE = [
    # canvas, hq, hkv, hd, kv_len, causal_rows, window, k_cfg
    (1, 4, 2, 64, 0, 1, 0, (8, 0, 0, 0)),              # one row, one key
    (1, 16, 2, 512, 77, 0, 0, T.adaptive_k()),          # single denoise row, fewer keys than k_min
    (5, 2, 1, 32, 3, 0, 0, (1, 0, 0, 0)),               # less than one key tile in total
    (37, 12, 4, 64, 333, 20, 100, (17, 0, 0, 0)),       # ragged everything: group 3, mixed rows, window
    (256, 16, 8, 256, 0, 256, 0, T.adaptive_k()),       # prefill from an empty cache, per-row k
    (64, 16, 2, 512, 40000, 64, 0, (256, 128, 64, 512)),  # two blocks of canvas rows (score plane budget)
    (8, 8, 8, 128, 5000, 0, 0, (600, 0, 0, 0)),         # no GQA sharing
]


@pytest.mark.parametrize("case", EDGE)
def test_edge_cases(gpu_ready, po, case):
    canvas, hq, hkv, hd, kvl, cr, win, k_cfg = case
    toks = None if canvas <= 64 else np.unique(np.linspace(0, canvas - 1, 16).round().astype(np.uint32))
    got, ref = run_topk(po, canvas, hq, hkv, hd, kvl, k_cfg, causal_rows=cr, window=win, seed=hash(case[:7]) & 0xFFFF,
                        toks=toks)
    assert np.isfinite(got).all()
    assert max_abs_diff(got, ref) <= 2e-2 and mean_abs_diff(got, ref) <= 2e-3


def test_ring_cache(gpu_ready, po):
    """Top-k over a wrapped ring (a sliding layer's storage): kept positions map to slots for the gather."""
    import torch
    canvas, hq, hkv, hd, kvl, window, ring, k = 32, 4, 2, 128, 3000, 1000, 2048, 40
    rng = np.random.default_rng(77)
    t_all = kvl + canvas
    q = rng.standard_normal((canvas, hq, hd)).astype(np.float32)
    lin = rng.standard_normal((t_all, 2, hkv, hd)).astype(np.float32)
    qb, lb = R.f32_to_bf16_bits_rne(q), R.f32_to_bf16_bits_rne(lin).reshape(lin.shape)
    ringbits = np.full((ring, 2, hkv, hd), 0x7FC0, dtype=np.uint16)          # NaN in every dead slot
    for pos in range(kvl - (window - 1), t_all):
        ringbits[pos & (ring - 1)] = lb[pos]
    d = A.make_desc(canvas, hq, hkv, hd, kvl, window=window, kv_ring_mask=ring - 1, out_dtype=capi.DG_F32)
    out = torch.zeros(canvas * hq * hd, dtype=torch.float32, device="cuda")
    cfg = (k, 0, 0, 0)
    T.forward(d, cfg, A.to_device_bits(qb.reshape(-1)), A.to_device_bits(ringbits.reshape(-1)), out, T.alloc_workspace(d, cfg))
    torch.cuda.synchronize()
    od = po.make_desc(canvas, hq, hkv, hd, kvl, window=window)
    ref = po.attention_topk_f32(od, cfg, R.bf16_bits_to_f32(qb).reshape(q.shape), R.bf16_bits_to_f32(lb).reshape(lin.shape))
    got = out.cpu().numpy().reshape(ref.shape)
    assert np.isfinite(got).all()
    assert max_abs_diff(got, ref) <= 2e-2 and mean_abs_diff(got, ref) <= 2e-3


# ------------------------------------------------------------------ properties
def test_k_at_least_the_visible_keys_is_dense_attention(gpu_ready):
    import torch
    w = W.Workload("dense", 64, 16, 2, 512, 900, causal_rows=32, seed=9)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc()
    d.out_dtype = capi.DG_F32
    dense = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.float32, device="cuda")
    A.forward(d, qd, kd, dense, None, A.alloc_workspace(d))
    k_cfg = (1024, 0, 0, 0)
    sparse = torch.zeros_like(dense)
    T.forward(d, k_cfg, qd, kd, sparse, T.alloc_workspace(d, k_cfg))
    torch.cuda.synchronize()
    a, b = dense.cpu().numpy(), sparse.cpu().numpy()
    assert max_abs_diff(a, b) <= 8e-3 and mean_abs_diff(a, b) <= 3e-4    # the dense kernel rounds P to bf16


def test_k1_is_the_value_row_of_the_best_key(gpu_ready, po):
    canvas, hq, hkv, hd, kvl = 16, 8, 2, 128, 777
    rng = np.random.default_rng(12)
    q = rng.standard_normal((canvas, hq, hd)).astype(np.float32)
    kv = rng.standard_normal((kvl + canvas, 2, hkv, hd)).astype(np.float32)
    got, ref = run_topk(po, canvas, hq, hkv, hd, kvl, (1, 0, 0, 0), q=q, kv=kv)
    vb = R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(kv[:, 1])).reshape(kvl + canvas, hkv, hd)
    for tok in range(canvas):
        for h in range(hq):
            assert any(np.array_equal(got[tok, h], vb[t, h // 4]) for t in range(kvl + canvas))
    assert max_abs_diff(got, ref) == 0.0      # N(0,1) scores at hd 128: no near-ties at the top


def test_runs_are_bit_identical_and_replay_in_a_graph(gpu_ready):
    import torch
    w = W.Workload("rep", 64, 16, 2, 512, 5000, seed=31)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc()
    k_cfg = T.adaptive_k()
    ws = T.alloc_workspace(d, k_cfg)
    outs = []
    for _ in range(3):
        out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.int16, device="cuda")
        T.forward(d, k_cfg, qd, kd, out, ws)
        torch.cuda.synchronize()
        outs.append(out)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    gout = torch.zeros_like(outs[0])
    with torch.cuda.stream(side):
        T.forward(d, k_cfg, qd, kd, gout, ws)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        T.forward(d, k_cfg, qd, kd, gout, ws)
    for _ in range(3):
        gout.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(gout, outs[0])


def test_error_codes(gpu_ready):
    import torch
    d = A.make_desc(64, 16, 2, 512, 100)
    lib = capi.load()
    n = C.c_size_t(0)
    cfg = lambda *v: (C.c_uint32 * 4)(*v)
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), cfg(2000, 0, 0, 0), C.byref(n)) == capi.DG_ERR_SHAPE
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), cfg(256, 128, 64, 2048), C.byref(n)) == capi.DG_ERR_SHAPE
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), cfg(256, 128, 600, 512), C.byref(n)) == capi.DG_ERR_SHAPE
    d32 = A.make_desc(64, 16, 2, 512, 100, q_dtype=capi.DG_F32, kv_dtype=capi.DG_F32, out_dtype=capi.DG_F32)
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d32), cfg(64, 0, 0, 0), C.byref(n)) == capi.DG_ERR_UNSUPPORTED
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), cfg(64, 0, 0, 0), C.byref(n)) == capi.DG_OK and n.value > 0
    buf = torch.zeros(1 << 20, dtype=torch.int16, device="cuda")
    small = torch.zeros(256, dtype=torch.uint8, device="cuda")
    rc = lib.dg_attn_topk_forward(C.byref(d), cfg(64, 0, 0, 0), buf.data_ptr(), buf.data_ptr(), buf.data_ptr(),
                                  small.data_ptr(), small.numel(), A.stream_handle())
    assert rc == capi.DG_ERR_WORKSPACE
