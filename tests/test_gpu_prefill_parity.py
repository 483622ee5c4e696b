"""GPU parity of the causal prefill / committed-block extend through the same kernel: the
reference runs a prompt in causal 256-token chunks and batches up to four of them into one
super-chunk whose attention is still dispatched per sub-chunk with kv_len advancing by 256
(src/metal/step_kernel/runtime.rs:370-389, enc.rs:2576-2585, 2176-2183).  Here the whole
super-chunk is one call (canvas = n_subs * 256, every row causal), checked against the CPU oracle
and against the per-sub-chunk sequence the reference dispatches."""
import numpy as np
import pytest

from diffgemma_amd import attention as A
from diffgemma_amd import capi, rounding as R, workloads as W
from helpers import assert_oracle, max_abs_diff, mean_abs_diff
from test_gpu_parity import check_tolerances, reference_cpu, run_workload

pytestmark = pytest.mark.gpu

SUPER_CHUNKS = [
    # canvas, hq, hkv, hd, kv_len, window
    (1024, 16, 2, 512, 2048, 0),      # global layer, four sub-chunks behind a 2k prefix
    (1024, 16, 8, 256, 4096, 1024),   # sliding layer: row at pos sees [pos-1023, pos]
    (1024, 16, 2, 512, 0, 0),         # first super-chunk of a prompt (triangular mask)
    (1024, 16, 8, 256, 0, 1024),
    (512, 16, 2, 512, 1280, 0),       # two sub-chunks
    (768, 16, 8, 256, 768, 1024),     # three sub-chunks, window starts to bite inside the canvas
    (1024, 16, 8, 256, 256, 300),     # window shorter than one sub-chunk
]


@pytest.mark.parametrize("case", SUPER_CHUNKS)
def test_super_chunk_against_oracle(gpu_ready, po, case):
    c, hq, hkv, hd, kvl, win = case
    w = W.Workload("prefill", c, hq, hkv, hd, kvl, causal_rows=c, window=win, seed=hash(case) & 0xFFFF)
    check_tolerances(*run_workload(po, w))


@pytest.mark.parametrize("name", ["prefill_global_super", "prefill_sliding_super"])
def test_super_chunk_at_32k_prefix_rows(gpu_ready, po, name):
    """Full size (1024 causal rows behind a 32768-key prefix); the oracle runs a row sample that
    holds the first and last row of every sub-chunk."""
    toks = np.array([0, 1, 255, 256, 511, 512, 700, 767, 768, 1023], dtype=np.uint32)
    check_tolerances(*run_workload(po, W.config(name), toks=toks))


def test_reference_super_chunk_fixture_dispatch(gpu_ready, po):
    """The reference's production super-chunk fixture (attention_gemm/mod.rs:385-407: canvas 1024,
    16 Q / 2 KV heads, hd 512) through dg_attention_dispatch with causal = 1."""
    f = A.model_full_fixture(600, canvas=1024)
    want, _, _ = reference_cpu(po, f, causal_rows=f.canvas)
    rig = A.AttnRig.from_fixture(f)
    rig.run_dispatch(causal=1)
    assert_oracle(rig.read_out_f32(), want, 2e-2, 0.9999)
    assert rig.read_debug_status().code == 0


def _run(desc, q, kv, out, lse):
    A.forward(desc, q, kv, out, lse, A.alloc_workspace(desc))


@pytest.mark.parametrize("full", [True, False])
def test_super_chunk_equals_sequential_sub_chunks(gpu_ready, po, full):
    """One call over 4 x 256 rows == the four per-sub-chunk calls the reference encodes (Q/O planes
    offset by sub * 256 rows, kv_len = base + sub * 256), on a wrapped ring for the sliding layer."""
    import torch
    n_subs, sub, hq = 4, 256, 16
    hd, hkv, window, ring = (512, 2, 0, 0) if full else (256, 8, 1024, 2048)
    base = 2304 if full else 2816
    canvas = n_subs * sub
    t_all = base + canvas
    slots = t_all if full else ring
    rng = np.random.default_rng(17 + full)
    q = rng.standard_normal((canvas, hq, hd)).astype(np.float32)
    lin = rng.standard_normal((2, hkv, t_all, hd)).astype(np.float32)       # by absolute position
    qb, lb = R.f32_to_bf16_bits_rne(q), R.f32_to_bf16_bits_rne(lin).reshape(lin.shape)
    cache = np.full((2, hkv, slots, hd), 0x7FC0, dtype=np.uint16)           # NaN: dead slots must not be read
    first = 0 if full else base - (window - 1)
    for pos in range(first, t_all):
        cache[:, :, pos & (ring - 1) if ring else pos] = lb[:, :, pos]
    qd, kd = A.to_device_bits(qb.reshape(-1)), A.to_device_bits(cache.reshape(-1))

    def desc(c, kv_len):
        return A.make_desc(c, hq, hkv, hd, kv_len, causal_rows=c, window=window, kv_ring_mask=ring - 1 if ring else 0,
                           out_dtype=capi.DG_F32, layout="head_major", t_cap=slots)

    out = torch.zeros(canvas * hq * hd, dtype=torch.float32, device="cuda")
    lse = torch.zeros(canvas * hq, dtype=torch.float32, device="cuda")
    _run(desc(canvas, base), qd, kd, out, lse)
    seq = torch.zeros_like(out)
    seq_lse = torch.zeros_like(lse)
    n = sub * hq * hd
    for s in range(n_subs):
        _run(desc(sub, base + s * sub), qd[s * n:(s + 1) * n], kd, seq[s * n:(s + 1) * n],
             seq_lse[s * sub * hq:(s + 1) * sub * hq])
    torch.cuda.synchronize()
    a, b = out.cpu().numpy(), seq.cpu().numpy()
    la, lb_ = lse.cpu().numpy(), seq_lse.cpu().numpy()
    assert np.isfinite(a).all() and np.isfinite(b).all()
    # same arithmetic, different cuts of the key range: probabilities round to bf16 against
    # different running maxima, nothing more (values here are N(0,1), rows are sharply peaked)
    assert max_abs_diff(a, b) <= 2e-2 and mean_abs_diff(a, b) <= 1e-3
    assert np.max(np.abs(la - lb_) / np.maximum(np.abs(la), 1.0)) <= 2e-4
    od = po.make_desc(canvas, hq, hkv, hd, base, causal_rows=canvas, window=window, layout="head_major", t_cap=t_all)
    toks = np.array([0, 255, 256, 600, 1023], dtype=np.uint32)
    ref, ref_lse = po.attention_f32(od, R.bf16_bits_to_f32(qb).reshape(q.shape), R.bf16_bits_to_f32(lb).reshape(lin.shape),
                                    tok_list=toks)
    for got, got_lse in ((a, la), (b, lb_)):
        check_tolerances(got.reshape(canvas, hq, hd)[toks], got_lse.reshape(canvas, hq)[toks], ref[toks], ref_lse[toks])


def test_super_chunk_split_counts_agree(gpu_ready):
    """Each row tile cuts its own visible key range into the splits: any split count gives the
    same rows (to the rounding of the probabilities) and the same LSE."""
    import torch
    w = W.Workload("prefill", 1024, 16, 8, 256, 3000, causal_rows=1024, window=1024, seed=23)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    res = []
    for splits in (1, 2, 3, 7):
        d = w.desc(n_splits=splits)
        d.out_dtype = capi.DG_F32
        out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.float32, device="cuda")
        lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
        _run(d, qd, kd, out, lse)
        torch.cuda.synchronize()
        res.append((out.cpu().numpy(), lse.cpu().numpy()))
    for o, l in res[1:]:
        assert max_abs_diff(o, res[0][0]) < 1.6e-2 and mean_abs_diff(o, res[0][0]) < 4e-4   # two bf16-P roundings
        assert np.max(np.abs(l - res[0][1]) / np.maximum(np.abs(res[0][1]), 1.0)) <= 2e-4
