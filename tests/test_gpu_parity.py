"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on identical
seeded inputs.  Tolerances: the reference's per-fixture ones (attention/mod.rs:846-946:
max_abs 1e-2 / 2e-2, cosine >= 0.9999) on its own fixtures; max-abs <= 2e-2, mean-abs <= 2e-3
on bf16 outputs and per-row LSE within 1e-3 relative on the benchmark configurations."""
import ctypes as C

import numpy as np
import pytest

from diffgemma_amd import attention as A
from diffgemma_amd import capi, rounding as R, workloads as W
from helpers import assert_oracle, max_abs_diff, mean_abs_diff

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS, LSE_REL = 2e-2, 2e-3, 1e-3

FIXTURES = {
    "tiny": (A.tiny_fixture, 1e-2), "wide": (A.wide_fixture, 2e-2), "full_hd512": (A.full_hd512_fixture, 2e-2),
    "full_grp8_hd512": (A.full_grp8_hd512_fixture, 2e-2), "sliding_hd256": (A.sliding_hd256_fixture, 2e-2),
}


def reference_cpu(po, f, **kw):
    """The reference's test wrapper (attention/mod.rs:218-240): Q -> bf16, KV -> f16, both by
    truncation; run the oracle; output -> bf16 by truncation."""
    q = R.bf16_bits_to_f32(R.f32_to_bf16_bits_trunc(f.q))
    kv = R.f16_bits_to_f32(R.f32_to_f16_bits_trunc(f.kvcache))
    d = po.make_desc(f.canvas, f.n_q_heads, f.n_kv(), f.head_dim(), f.kv_len, **kw)
    out, lse = po.attention_f32(d, q, kv)
    return po.round_array(out, po.ROUND_BF16_TRUNC).ravel(), out.ravel(), lse.ravel()


# ------------------------------------------------------------------ the reference's Tier-1 matrix
@pytest.mark.parametrize("name", list(FIXTURES))
def test_reference_fixture_scalar_kernel(gpu_ready, po, name):
    fn, tol = FIXTURES[name]
    f = fn()
    want, _, _ = reference_cpu(po, f)
    assert_oracle(A.gpu(f), want, tol, 0.9999)


@pytest.mark.parametrize("name", list(FIXTURES))
@pytest.mark.parametrize("causal", [0, 1])
def test_reference_fixture_mfma_dispatch(gpu_ready, po, name, causal):
    """Through dg_attention_dispatch: the buffers encode_layer_attention_dispatch binds."""
    fn, tol = FIXTURES[name]
    f = fn()
    want, _, _ = reference_cpu(po, f, causal_rows=f.canvas if causal else 0)
    rig = A.AttnRig.from_fixture(f)
    rig.run_dispatch(causal=causal)
    assert_oracle(rig.read_out_f32(), want, tol, 0.9999)
    assert rig.read_debug_status().code == 0


@pytest.mark.parametrize("name", list(FIXTURES))
@pytest.mark.parametrize("causal", [0, 1])
def test_reference_fixture_dispatch_with_device_step_params(gpu_ready, po, name, causal):
    """dg_attention_dispatch_dev: StepParams bound as a device buffer (enc.rs:2177-2220), kv_len read when the
    kernels run.  Planned for exactly this prefix it gives the host-P entry's bits; planned for a longer one
    (the split plan then differs) it still meets the oracle."""
    fn, tol = FIXTURES[name]
    f = fn()
    want, _, _ = reference_cpu(po, f, causal_rows=f.canvas if causal else 0)
    host, dev = A.AttnRig.from_fixture(f), A.AttnRig.from_fixture(f)
    host.run_dispatch(causal=causal)
    dev.run_dispatch_dev(causal=causal)
    assert np.array_equal(host.read_out_f32().view(np.uint32), dev.read_out_f32().view(np.uint32))
    slack = 4096      # slots the cache buffer holds behind the fixture's rows: the plan may reach that far
    far = A.AttnRig.from_fixture(f, kv_slack_slots=slack)
    far.run_dispatch_dev(causal=causal, kv_len_max=f.kv_len + slack)
    assert_oracle(far.read_out_f32(), want, tol, 0.9999)
    assert dev.read_debug_status().code == 0 and far.read_debug_status().code == 0


@pytest.mark.parametrize("name", list(FIXTURES))
def test_reference_fixture_unrounded_and_lse(gpu_ready, po, name):
    import torch
    f = FIXTURES[name][0]()
    _, want, want_lse = reference_cpu(po, f)
    rig = A.AttnRig.from_fixture(f)
    d = rig.desc(kernel=capi.DG_KERNEL_MFMA, truncate=False)
    d.out_dtype = capi.DG_F32
    out = torch.zeros(f.out_len(), dtype=torch.float32, device="cuda")
    A.forward(d, rig.buf_q, rig.buf_kv, out, rig.buf_lse, rig.workspace_for(d))
    torch.cuda.synchronize()
    assert max_abs_diff(out.cpu().numpy(), want) < 2e-4
    lse = rig.read_lse()
    assert np.max(np.abs(lse - want_lse) / np.maximum(np.abs(want_lse), 1.0)) < LSE_REL


@pytest.mark.parametrize("name", ["tiny", "wide", "sliding_hd256"])
def test_f32_inputs_are_rounded_like_the_reference_wrapper(gpu_ready, po, name):
    """f32 queries and an f32 cache handed to dg_attn_forward are brought down on the device the way the
    reference's wrapper rounds them on the host (attention/mod.rs:218-240: Q -> bf16, K/V -> f16, both by
    truncation, f16 with clamp and subnormal flush): the result equals, bit for bit, the call fed the
    host-rounded bits, and meets the wrapper's own oracle."""
    import torch
    f = FIXTURES[name][0]()
    _, want, _ = reference_cpu(po, f)
    rig = A.AttnRig.from_fixture(f, kv_slack_slots=0)            # host-rounded bf16 Q / f16 cache
    d16 = rig.desc(kernel=capi.DG_KERNEL_MFMA, truncate=False)
    d16.out_dtype = capi.DG_F32
    out16 = torch.zeros(f.out_len(), dtype=torch.float32, device="cuda")
    A.forward(d16, rig.buf_q, rig.buf_kv, out16, rig.buf_lse, rig.workspace_for(d16))
    # the same fixture as f32, with values the f16 conversion has to clamp, flush and truncate
    q32 = torch.from_numpy(np.ascontiguousarray(f.q, dtype=np.float32)).cuda()
    kv32 = torch.from_numpy(np.ascontiguousarray(f.kvcache, dtype=np.float32)).cuda()
    d32 = A.make_desc(f.canvas, f.n_q_heads, f.n_kv(), f.head_dim(), f.kv_len, q_dtype=capi.DG_F32,
                      kv_dtype=capi.DG_F32, out_dtype=capi.DG_F32, kernel=capi.DG_KERNEL_MFMA,
                      kv_region_bytes=2 * f.layer.kv_region)   # the region offset is in bytes: f32 elements are twice as wide
    out32 = torch.zeros(f.out_len(), dtype=torch.float32, device="cuda")
    lse32 = torch.zeros(f.canvas * f.n_q_heads, dtype=torch.float32, device="cuda")
    A.forward(d32, q32, kv32, out32, lse32, A.alloc_workspace(d32))
    torch.cuda.synchronize()
    assert torch.equal(out16, out32)
    assert max_abs_diff(out32.cpu().numpy(), want) < 2e-4


def test_f32_cache_conversion_clamps_flushes_and_truncates(gpu_ready, po):
    """Values the three rules of the reference's f16 conversion act on (src/shaders/common/f16.rs:28-47):
    beyond +-65504 (clamped, not infinity), below 2^-14 (flushed to a signed zero), and mantissas that
    round-to-nearest would round up (truncated).  V carries them; the output of a one-key row is that V row."""
    import torch
    hd = 32
    v = np.zeros(hd, dtype=np.float32)
    v[:8] = [1e6, -1e6, 3e-5, -3e-5, 1.0 + 2.0 ** -11 + 2.0 ** -12, -(2.0 + 2.0 ** -10 + 2.0 ** -11), 65504.0, 7e-8]
    want = R.f16_bits_to_f32(R.f32_to_f16_bits_trunc(v))
    assert want[0] == 65504.0 and want[2] == 0.0 and want[4] == 1.0     # the rules do act on these values
    kv = np.zeros((1, 2, 1, hd), dtype=np.float32)               # one slot: [K head | V head]
    kv[0, 0, 0, 0] = 1.0
    kv[0, 1, 0] = v
    q = np.ones((1, 1, hd), dtype=np.float32)
    d = A.make_desc(1, 1, 1, hd, 0, q_dtype=capi.DG_F32, kv_dtype=capi.DG_F32, out_dtype=capi.DG_F32)
    out = torch.zeros(hd, dtype=torch.float32, device="cuda")
    A.forward(d, torch.from_numpy(q.ravel()).cuda(), torch.from_numpy(kv.ravel()).cuda(), out, None, A.alloc_workspace(d))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)


def test_model_full_fixture_midsize(gpu_ready, po):
    """The reference's bench fixture (attention_gemm/mod.rs:364-432) at a prefix that spans many key tiles."""
    f = A.model_full_fixture(1000, canvas=64)
    want, _, _ = reference_cpu(po, f)
    assert_oracle(A.gpu_mma(f), want, 2e-2, 0.9999)


# ------------------------------------------------------------------ generic runner
def run_workload(po, w, *, n_splits=0, kernel=capi.DG_KERNEL_AUTO, out_f32=False, toks=None, ring=None, flags=0,
                 kv_override=None, default_partials=False):
    import torch
    q, kv = W.generate(w)
    if kv_override is not None:
        kv = kv_override(kv)
    qd, kd = W.device_arrays(w, q, kv)
    desc = w.desc(n_splits=n_splits, kernel=kernel, flags=flags, default_partials=default_partials)
    if out_f32:
        desc.out_dtype = capi.DG_F32
    is_bf16_out = desc.out_dtype == capi.DG_BF16
    out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.int16 if is_bf16_out else torch.float32,
                      device="cuda")
    lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
    A.forward(desc, qd, kd, out, lse, A.alloc_workspace(desc))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    got = R.bf16_bits_to_f32(got.view(np.uint16)) if is_bf16_out else got
    got = got.reshape(w.canvas, w.n_q_heads, w.head_dim)
    got_lse = lse.cpu().numpy().reshape(w.canvas, w.n_q_heads)
    od = po.make_desc(w.canvas, w.n_q_heads, w.n_kv_heads, w.head_dim, w.kv_len, causal_rows=w.causal_rows,
                      window=w.window, causal_sees_masked=1 if w.sees_masked else 0,
                      t_lo_override=-1 if w.t_lo is None else w.t_lo, layout=w.layout, t_cap=w.t_all)
    ref, ref_lse = po.attention_f32(od, q, kv, tok_list=toks)
    rows = np.arange(w.canvas) if toks is None else np.asarray(toks)
    return got[rows], got_lse[rows], ref[rows], ref_lse[rows]


LSE_ABS = 2.0 ** -8


def check_tolerances(got, got_lse, ref, ref_lse, max_abs=MAX_ABS, mean_abs=MEAN_ABS, strict_lse=False):
    """The benchmark tolerances on the output.  Log-sum-exp: with strict_lse (the benchmark configurations)
    the stated bound, 1e-3 relative, on every row; otherwise (arbitrary shapes and data) the library's
    documented bound |lse - exact| <= max(1e-3 |exact|, 2^-8): the row sum is taken over the probabilities
    as rounded for the MFMA (the numbers P.V multiplies); bf16 keeps 8 significant bits, so each is within
    2^-8 of its value (unit roundoff), and on a row with one dominant key nothing averages out: ln(sum) moves
    by up to 2^-8 = 3.9e-3, so the relative bound alone would fail rows whose LSE is small in magnitude.
    Rows without a visible key: -inf."""
    assert np.all(np.isfinite(got))
    assert max_abs_diff(got, ref) <= max_abs
    assert mean_abs_diff(got, ref) <= mean_abs
    got_lse, ref_lse = np.asarray(got_lse), np.asarray(ref_lse)
    ok = np.isfinite(ref_lse)
    assert np.array_equal(np.isfinite(got_lse), ok)
    err = np.abs(got_lse[ok] - ref_lse[ok])
    assert np.all(err <= np.maximum(LSE_REL * np.abs(ref_lse[ok]), 0.0 if strict_lse else LSE_ABS))


# ------------------------------------------------------------------ benchmark configurations
def test_cfg1_tiny_fp32(gpu_ready, po):
    """fp32 in, fp32 out; the library computes in f16 after a conversion pass."""
    got, lse, ref, ref_lse = run_workload(po, W.config("cfg1_tiny"))
    check_tolerances(got, lse, ref, ref_lse, max_abs=2e-4, mean_abs=2e-5, strict_lse=True)


@pytest.mark.parametrize("over_workgroups", [False, True])
@pytest.mark.parametrize("name", ["cfg2_sliding", "cfg2_sliding_768"])
def test_cfg2_sliding_window(gpu_ready, po, name, over_workgroups):
    """A sliding layer runs as one launch (keys split over the waves of a workgroup, merged in LDS);
    DG_ATTN_F_SPLIT_OVER_WORKGROUPS asks for the general kernel (keys split over workgroups + merge launch)."""
    flags = capi.DG_ATTN_F_SPLIT_OVER_WORKGROUPS if over_workgroups else 0
    assert capi.resolved_splits(W.config(name).desc(flags=flags)) == ((6 if name == "cfg2_sliding" else 5) if over_workgroups else 1)
    check_tolerances(*run_workload(po, W.config(name), flags=flags), strict_lse=True)


@pytest.mark.parametrize("name", ["cfg3_global", "cfg3_global_b", "cfg3_global_f16kv"])
def test_cfg3_global_full_size(gpu_ready, po, name):
    """Full 32k-prefix shape, every row, mixed committed/bidirectional mask."""
    check_tolerances(*run_workload(po, W.config(name)), strict_lse=True)


def test_cfg3_global_with_the_library_default_partial_rows(gpu_ready, po):
    """The workload descriptors ask for f16 partial rows (DG_ATTN_F_F16_PARTIALS: the caller vouches for the
    range of V in a bf16 cache).  Without the flag a bf16 cache gets fp32 partial rows: same tolerances, and the
    two results differ by output roundings only."""
    w = W.config("cfg3_global")
    toks = np.arange(0, 256, 3, dtype=np.uint32)
    f32p = run_workload(po, w, toks=toks, default_partials=True)
    check_tolerances(*f32p, strict_lse=True)
    f16p = run_workload(po, w, toks=toks)
    diff = np.abs(f32p[0] - f16p[0])
    assert diff.max() <= 2.0 ** -7 * max(1.0, np.abs(f32p[0]).max()) and np.mean(diff > 0) < 0.1
    assert np.array_equal(f32p[1], f16p[1])


def test_cfg3_unrounded_output_error_budget(gpu_ready, po):
    """fp32 output isolates the kernel's own error (bf16 probabilities) from output rounding."""
    toks = np.arange(0, 256, 5, dtype=np.uint32)
    got, lse, ref, ref_lse = run_workload(po, W.config("cfg3_global"), out_f32=True, toks=toks)
    check_tolerances(got, lse, ref, ref_lse, max_abs=8e-3, mean_abs=3e-4, strict_lse=True)


def test_cfg4_long_context_rows(gpu_ready, po):
    """131072-key prefix with 1% of keys scaled x8 (peaked rows); oracle on a row sample."""
    toks = np.array([0, 1, 63, 64, 127, 128, 200, 255], dtype=np.uint32)
    check_tolerances(*run_workload(po, W.config("cfg4_long"), toks=toks), strict_lse=True)


@pytest.mark.parametrize("over_workgroups", [False, True])
def test_cfg5_sliding_layer_at_32k(gpu_ready, po, over_workgroups):
    flags = capi.DG_ATTN_F_SPLIT_OVER_WORKGROUPS if over_workgroups else 0
    check_tolerances(*run_workload(po, W.config("cfg5_sliding_32k"), flags=flags), strict_lse=True)


@pytest.mark.parametrize("hd,hq,hkv,canvas,kv_len,causal_rows,window", [
    (256, 16, 8, 256, 4096, 0, 1024),         # the model's sliding layer, denoise
    (256, 16, 8, 256, 9000, 256, 1024),       # the same rows causal (committed-block extend)
    (256, 16, 8, 100, 700, 50, 0),            # mixed rows, ragged canvas, no window
    (128, 8, 4, 77, 300, 0, 0), (64, 8, 8, 33, 0, 33, 0), (32, 4, 4, 20, 1500, 0, 200),
    (256, 2, 2, 1, 5, 0, 0),                  # one row, one tile: three of the four waves see no key
])
def test_one_launch_kernel_against_the_general_one(gpu_ready, po, hd, hq, hkv, canvas, kv_len, causal_rows, window):
    """The one-launch kernel for short key ranges (waves split the keys, merge in LDS) and the general kernel
    compute the same function: both meet the oracle, they differ from each other by the rounding of the
    probabilities only, and the one-launch kernel gives the same bits on every run (its merge always adds the
    waves in the same order)."""
    import torch
    w = W.Workload("ws", canvas, hq, hkv, hd, kv_len, causal_rows=causal_rows, window=window, seed=hd + canvas)
    assert capi.resolved_splits(w.desc()) == 1 and capi.workspace_bytes(w.desc()) == 0
    one = run_workload(po, w, out_f32=True)
    gen = run_workload(po, w, out_f32=True, flags=capi.DG_ATTN_F_SPLIT_OVER_WORKGROUPS, n_splits=3 if kv_len + canvas > 96 else 0)
    check_tolerances(*one)
    check_tolerances(*gen)
    assert max_abs_diff(one[0], gen[0]) <= 1.6e-2 and mean_abs_diff(one[0], gen[0]) <= 4e-4     # two bf16-P roundings
    ok = np.isfinite(one[3])
    assert np.max(np.abs(one[1][ok] - gen[1][ok]), initial=0.0) <= 2 * LSE_ABS      # each within 2^-8 of the exact value
    again = run_workload(po, w, out_f32=True)
    assert np.array_equal(one[0].view(np.uint32), again[0].view(np.uint32)) and np.array_equal(one[1].view(np.uint32), again[1].view(np.uint32))


# ------------------------------------------------------------------ size-independent properties at full size
def _device_run(w, q, kv, **kw):
    import torch
    qd, kd = W.device_arrays(w, q, kv)
    desc = w.desc(**kw)
    desc.out_dtype = capi.DG_F32
    out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.float32, device="cuda")
    lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
    A.forward(desc, qd, kd, out, lse, A.alloc_workspace(desc))
    torch.cuda.synchronize()
    return out.cpu().numpy().reshape(w.canvas, w.n_q_heads, w.head_dim), lse.cpu().numpy().reshape(w.canvas, -1)


def test_split_count_invariance_full_size(gpu_ready):
    """Split-KV + LSE merge: any split count gives the single-pass result (cfg 3 shape)."""
    w = W.config("cfg3_global")
    q, kv = W.generate(w)
    base, base_lse = _device_run(w, q, kv, n_splits=1)
    for s in (2, 8, 13, 64):
        out, lse = _device_run(w, q, kv, n_splits=s)
        assert max_abs_diff(out, base) < 1.6e-2 and mean_abs_diff(out, base) < 4e-4, s   # two bf16-P roundings
        assert np.max(np.abs(lse - base_lse) / np.abs(base_lse)) < 1e-4, s


@pytest.mark.parametrize("hd,hq,hkv,splits", [(32, 8, 4, 17), (64, 32, 4, 9), (128, 8, 4, 33), (256, 16, 8, 8), (256, 16, 8, 64),
                                              (512, 16, 2, 8), (512, 8, 1, 40)])
def test_split_partial_formats(gpu_ready, po, hd, hq, hkv, splits):
    """Split partial rows travel as normalised f16 rows with a 16-bit output when the cache is f16 or the
    caller vouches for the range of a bf16 one (DG_ATTN_F_F16_PARTIALS, which the workload descriptors set;
    DG_ATTN_F_F32_PARTIALS keeps fp32): both formats meet the oracle, they differ by output roundings
    only, and an f32 output keeps fp32 partials.  The split counts are larger than head_dim / 8 and
    head_dim / 4: the merge reads every split's weight whatever lanes its loads keep busy."""
    w = W.Workload("partials", 100, hq, hkv, hd, 2049, causal_rows=50, seed=11)
    half = run_workload(po, w, n_splits=splits)
    full = run_workload(po, w, n_splits=splits, flags=capi.DG_ATTN_F_F32_PARTIALS)
    check_tolerances(*half)
    check_tolerances(*full)
    diff = np.abs(half[0] - full[0])
    assert diff.max() <= 2.0 ** -7 * max(1.0, np.abs(full[0]).max())       # one bf16 step of the largest value
    assert np.mean(diff > 0) < 0.1                                         # and only where a rounding tipped
    assert np.max(np.abs(half[1] - full[1])) == 0.0                        # (m, l) travel in fp32 either way
    f32a = run_workload(po, w, n_splits=splits, out_f32=True)
    f32b = run_workload(po, w, n_splits=splits, out_f32=True, flags=capi.DG_ATTN_F_F32_PARTIALS)
    assert np.array_equal(f32a[0], f32b[0])


@pytest.mark.parametrize("hd,hq,hkv,splits,canvas", [(256, 16, 8, 6, 256), (256, 16, 8, 8, 100), (512, 16, 2, 8, 64),
                                                     (128, 8, 4, 3, 77), (64, 8, 8, 2, 33), (32, 4, 4, 5, 20)])
def test_both_merge_kernels_give_the_same_bits(gpu_ready, hd, hq, hkv, splits, canvas):
    """A few splits over a small workspace are merged by the kernel that fetches every partial row up front;
    DG_ATTN_F_STREAMED_MERGE asks for the streaming one instead.  Same weights, same cut of negligible
    splits, same order of the sums: output and LSE are bit-equal (peaked rows, so that the cut is taken)."""
    import torch
    w = W.Workload("merge_ab", canvas, hq, hkv, hd, 2049, causal_rows=canvas // 2, seed=13)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)

    def run(flags):     # bf16 output, f16 partial rows (the workload descriptor asks for them)
        desc = w.desc(n_splits=splits, flags=flags)
        out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.int16, device="cuda")
        lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
        A.forward(desc, qd, kd, out, lse, A.alloc_workspace(desc))
        torch.cuda.synchronize()
        return out.cpu().numpy().view(np.uint16), lse.cpu().numpy()

    a, a_lse = run(0)
    b, b_lse = run(capi.DG_ATTN_F_STREAMED_MERGE)
    assert np.array_equal(a, b)
    assert np.array_equal(a_lse.view(np.uint32), b_lse.view(np.uint32))
    assert np.isfinite(a_lse).all() and np.any(a != 0)


@pytest.mark.parametrize("layout", ["head_major", "reference"])
@pytest.mark.parametrize("canvas,hq,hkv,kv_len,splits", [(256, 16, 2, 32768, 0), (64, 16, 2, 1000, 0), (100, 8, 1, 2049, 3),
                                                         (33, 8, 2, 70, 1), (256, 16, 2, 4099, 8)])
def test_kv_from_hbm_hint_changes_no_bit(gpu_ready, canvas, hq, hkv, kv_len, splits, layout):
    """DG_ATTN_F_KV_FROM_HBM selects the head_dim 512 kernel that touches key/value tiles into the L2 ahead
    of their loads: a change in timing only.  Ragged last tiles, splits shorter than the look-ahead and a
    single tile included, with key rows contiguous per head and in the reference's slot-major layout (rows of
    a tile a whole slot apart)."""
    import torch
    w = W.Workload("hint", canvas, hq, hkv, 512, kv_len, causal_rows=canvas // 2, seed=17, layout=layout)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)

    def run(flags):
        desc = w.desc(n_splits=splits, flags=flags)
        out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.int16, device="cuda")
        lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
        A.forward(desc, qd, kd, out, lse, A.alloc_workspace(desc))
        torch.cuda.synchronize()
        return out.cpu().numpy().view(np.uint16), lse.cpu().numpy()

    a, a_lse = run(0)
    b, b_lse = run(capi.DG_ATTN_F_KV_FROM_HBM)
    assert np.array_equal(a, b) and np.array_equal(a_lse.view(np.uint32), b_lse.view(np.uint32))
    assert np.isfinite(a_lse).all() and np.any(a != 0)


def test_dropped_weights_stay_below_rounding(gpu_ready, po):
    """The kernel stores a softmax weight that is more than 2^40 below its row's running max as an exact
    zero.  Rows built to make the most of that: one key at the top, half of the others 2^39 below it (kept),
    half 2^41 below (dropped) and carrying values a thousand times larger than the rest.  The result still
    meets the oracle far inside the tolerances (what is left is the bf16 rounding of the kept weights, which
    moves ln(l) by up to 2^-8)."""
    import torch
    w = W.Workload("drop", 64, 8, 2, 64, 4096 - 64, rms_norm=False, seed=5)
    q, kv = W.generate(w)
    u = np.zeros(w.head_dim, dtype=np.float32)
    u[:4] = 0.5                                               # |u|^2 = 1, exact in bf16
    q[:] = u
    ln2 = np.float32(np.log(2.0))
    alpha = np.where(np.arange(w.t_all) % 2 == 0, (60.0 - 39.0) * ln2, (60.0 - 41.0) * ln2).astype(np.float32)
    alpha[1000] = 60.0 * ln2
    alpha = R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(alpha))
    kv[0] = alpha[None, :, None] * u[None, None, :]           # score of key t = alpha[t] for every row and head
    kv[0] = R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(kv[0])).reshape(kv[0].shape)
    kv[1, :, 1::2, :] *= np.float32(1000.0)                   # what the dropped keys would have brought in
    kv[1] = R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(kv[1])).reshape(kv[1].shape)
    qd, kd = W.device_arrays(w, q, kv)
    for splits in (1, 4):
        desc = w.desc(n_splits=splits)
        desc.out_dtype = capi.DG_F32
        out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.float32, device="cuda")
        lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
        A.forward(desc, qd, kd, out, lse, A.alloc_workspace(desc))
        torch.cuda.synchronize()
        od = po.make_desc(w.canvas, w.n_q_heads, w.n_kv_heads, w.head_dim, w.kv_len, layout=w.layout, t_cap=w.t_all)
        ref, ref_lse = po.attention_f32(od, q, kv)
        got = out.cpu().numpy().reshape(ref.shape)
        # the dropped half would add 2048 x 2^-41 x 1000 ~ 1e-6 of a value of order one
        assert max_abs_diff(got, ref) < 2e-3, splits              # bf16 rounding of the kept weights only
        assert np.max(np.abs(lse.cpu().numpy().reshape(ref_lse.shape) - ref_lse)) < 4e-3, splits


def test_f16_leading_reference_stays_inside_its_bound(gpu_ready, po):
    """With an f16 cache the one-launch kernel lets its reference lead the running max by 2^4, so a weight more
    than 2^20 below the row's largest is dropped or loses precision: at most 2^-21 of the largest weight per key,
    2^-10 of the row's mass over the 2048 keys that kernel can see.  Rows built to make the most of it: the
    largest key first in every wave's quarter of the keys (so that the reference is as high as it gets from the
    start), every other key 2^21.5 below it (all dropped), as many keys as the kernel takes.  The output stays
    inside the tolerances, and off the oracle by no more than the bound says."""
    import torch
    w = W.Workload("lead", 32, 2, 1, 64, 2048 - 32, rms_norm=False, seed=9, kv_f16=True)
    assert capi.resolved_splits(w.desc()) == 1 and capi.workspace_bytes(w.desc()) == 0      # the one-launch kernel
    q, kv = W.generate(w)
    u = np.zeros(w.head_dim, dtype=np.float32)
    u[:4] = 0.5                                                   # |u|^2 = 1, exact in bf16 and f16
    q[:] = u
    ln2 = np.float32(np.log(2.0))
    alpha = np.full(w.t_all, (10.0 - 21.5) * ln2, dtype=np.float32)
    alpha[[0, 512, 1024, 1536]] = 10.0 * ln2
    alpha = R.f16_bits_to_f32(R.f32_to_f16_bits_rne(alpha))
    kv[0] = alpha[None, :, None] * u[None, None, :]               # score of key t = alpha[t] for every row and head
    kv[0] = R.f16_bits_to_f32(R.f32_to_f16_bits_rne(kv[0])).reshape(kv[0].shape)
    kv[1] = R.f16_bits_to_f32(R.f32_to_f16_bits_rne(kv[1])).reshape(kv[1].shape)
    qd, kd = W.device_arrays(w, q, kv)
    desc = w.desc()
    desc.out_dtype = capi.DG_F32
    out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.float32, device="cuda")
    lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
    A.forward(desc, qd, kd, out, lse, A.alloc_workspace(desc))
    torch.cuda.synchronize()
    od = po.make_desc(w.canvas, w.n_q_heads, w.n_kv_heads, w.head_dim, w.kv_len, layout=w.layout, t_cap=w.t_all)
    ref, ref_lse = po.attention_f32(od, q, kv)
    got = out.cpu().numpy().reshape(ref.shape)
    dropped = (w.t_all - 4) * 2.0 ** -21.5 / 4.0                  # the mass of the small keys against the four large ones
    assert 5e-5 < dropped < 2.0 ** -10
    vmax = float(np.abs(kv[1]).max())
    assert max_abs_diff(got, ref) <= 2.0 * dropped * vmax + 2e-3  # what was dropped, and the f16 rounding of the kept weights
    assert max_abs_diff(got, ref) <= MAX_ABS and mean_abs_diff(got, ref) <= MEAN_ABS
    assert np.max(np.abs(lse.cpu().numpy().reshape(ref_lse.shape) - ref_lse)) <= dropped + 2.0 ** -11 + 1e-6


@pytest.mark.parametrize("hd,hq,hkv", [(128, 8, 4), (512, 16, 2)])
def test_wide_score_range_raises_reference(gpu_ready, po, hd, hq, hkv):
    """Scores that spread over hundreds of log2 units: a row's maximum climbs by more than the 2^120 the
    bf16 probabilities may lag behind it, so the reference is raised and the accumulators rescaled in the
    middle of rows (with unit-variance inputs that path never runs on a bf16 cache)."""
    w = W.Workload("wide", 64, hq, hkv, hd, 4096 - 64, rms_norm=False, q_std=12.0 * (128.0 / hd) ** 0.5, seed=17)
    q, kv = W.generate(w)
    s = np.einsum("d,td->t", q[0, 0], kv[0, 0]) * np.log2(np.e)          # one row's scores in log2 units
    run_max = np.maximum.accumulate(s.reshape(-1, 32).max(axis=1))
    assert run_max[-1] - run_max[0] > 120.0                              # the case is what it claims to be
    for splits in (1, 0):
        check_tolerances(*run_workload(po, w, n_splits=splits))


def test_scalar_and_mfma_kernels_agree_full_size(gpu_ready):
    w = W.scaled(W.config("cfg3_global"), 8192)
    q, kv = W.generate(w)
    a, la = _device_run(w, q, kv, kernel=capi.DG_KERNEL_SCALAR)
    b, lb = _device_run(w, q, kv, kernel=capi.DG_KERNEL_MFMA)
    assert max_abs_diff(a, b) < 8e-3 and mean_abs_diff(a, b) < 3e-4
    assert np.max(np.abs(la - lb) / np.abs(la)) < 1e-4


def test_constant_value_rows_pass_through(gpu_ready):
    """If every key's V row is the same vector the output is that vector, whatever the scores."""
    w = W.config("cfg3_global")
    q, kv = W.generate(w)
    vrow = kv[1, :, :1, :].copy()
    kv[1] = vrow
    out, _ = _device_run(w, q, kv)
    want = np.repeat(vrow[:, 0, :], w.n_q_heads // w.n_kv_heads, axis=0)[None]
    assert max_abs_diff(out, np.broadcast_to(want, out.shape)) < 1e-5 + 4e-3 * np.abs(vrow).max()


def test_linearity_in_v_full_size(gpu_ready):
    """out(V1 + V2) = out(V1) + out(V2) for fixed Q, K."""
    w = W.scaled(W.config("cfg3_global"), 16384)
    q, kv = W.generate(w)
    rng = np.random.default_rng(99)
    v2 = R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(rng.standard_normal(kv[1].shape).astype(np.float32) * 0.5)).reshape(kv[1].shape)
    kv1, kv2, kv12 = kv.copy(), kv.copy(), kv.copy()
    kv2[1] = v2
    kv12[1] = R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(kv[1] + v2)).reshape(v2.shape)
    o1, _ = _device_run(w, q, kv1)
    o2, _ = _device_run(w, q, kv2)
    o12, _ = _device_run(w, q, kv12)
    # bf16 rounding of V1+V2 costs up to 2^-9 relative per element
    assert max_abs_diff(o12, o1 + o2) < 3e-2 and mean_abs_diff(o12, o1 + o2) < 3e-3


def test_gqa_group_shares_keys(gpu_ready):
    """Heads of one group fed the same Q row produce the same output (kvh = qh / group)."""
    w = W.scaled(W.config("cfg3_global"), 2048)
    q, kv = W.generate(w)
    q[:] = q[:, :1, :]
    out, lse = _device_run(w, q, kv)
    for h in range(1, 8):
        assert np.array_equal(out[:, h], out[:, 0]) and np.array_equal(lse[:, h], lse[:, 0])
    assert max_abs_diff(out[:, 8], out[:, 0]) > 1e-3


# ------------------------------------------------------------------ edge cases
CASES = [
    # canvas, hq, hkv, hd, kv_len, causal_rows, window, splits
    (1, 4, 2, 64, 0, 0, 0, 0),          # single row, no prefix
    (1, 16, 2, 512, 77, 1, 0, 0),       # single causal row
    (64, 16, 8, 256, 100, 0, 0, 0),     # retry canvas 64
    (128, 16, 2, 512, 500, 64, 0, 0),   # retry canvas 128, mixed mask
    (256, 16, 8, 256, 0, 256, 0, 0),    # prefill from an empty cache
    (37, 16, 8, 256, 333, 20, 100, 2),  # ragged everything
    (256, 8, 4, 128, 512, 0, 0, 0),     # hd 128
    (256, 16, 8, 256, 5000, 256, 1024, 0),  # causal sliding prefill
    (33, 6, 3, 32, 95, 0, 40, 3),       # hd 32, group 2
    (200, 12, 4, 64, 1, 100, 0, 0),     # group 3, one prefix key
]


@pytest.mark.parametrize("case", CASES)
def test_edge_cases(gpu_ready, po, case):
    c, hq, hkv, hd, kvl, cr, win, splits = case
    w = W.Workload("edge", c, hq, hkv, hd, kvl, causal_rows=cr, window=win, seed=hash(case) & 0xFFFF)
    check_tolerances(*run_workload(po, w, n_splits=splits))
    check_tolerances(*run_workload(po, w, kernel=capi.DG_KERNEL_SCALAR))


def test_reference_layout_equals_head_major(gpu_ready):
    w = W.Workload("lay", 64, 16, 8, 256, 700, window=300, seed=5)
    q, kv = W.generate(w)
    a, la = _device_run(w, q, kv)
    w2 = W.Workload("lay", 64, 16, 8, 256, 700, window=300, seed=5, layout="reference")
    kv2 = np.ascontiguousarray(kv.transpose(2, 0, 1, 3))
    b, lb = _device_run(w2, q, kv2)
    assert np.array_equal(a, b) and np.array_equal(la, lb)


def test_f16_cache_with_bf16_queries(gpu_ready, po):
    """The reference's own pairing (bf16 activations, f16 cache) with values outside bf16's grid."""
    import torch
    rng = np.random.default_rng(21)
    c, hq, hkv, hd, kvl = 96, 16, 2, 512, 900
    q = rng.standard_normal((c, hq, hd)).astype(np.float32)
    kv = rng.standard_normal((kvl + c, 2, hkv, hd)).astype(np.float32)
    qb = R.f32_to_bf16_bits_rne(q)
    kb = R.f32_to_f16_bits_rne(kv)
    d = A.make_desc(c, hq, hkv, hd, kvl, q_dtype=capi.DG_BF16, kv_dtype=capi.DG_F16, out_dtype=capi.DG_F32)
    out = torch.zeros(c * hq * hd, dtype=torch.float32, device="cuda")
    lse = torch.zeros(c * hq, dtype=torch.float32, device="cuda")
    A.forward(d, A.to_device_bits(qb), A.to_device_bits(kb), out, lse, A.alloc_workspace(d))
    torch.cuda.synchronize()
    od = po.make_desc(c, hq, hkv, hd, kvl)
    ref, ref_lse = po.attention_f32(od, R.bf16_bits_to_f32(qb), R.f16_bits_to_f32(kb))
    check_tolerances(out.cpu().numpy().reshape(ref.shape), lse.cpu().numpy().reshape(ref_lse.shape), ref, ref_lse,
                     max_abs=2e-3, mean_abs=1e-4)


@pytest.mark.parametrize("hq,hkv,hd,flags", [(16, 8, 256, 0), (16, 8, 256, capi.DG_ATTN_F_SPLIT_OVER_WORKGROUPS),
                                             (16, 2, 512, capi.DG_ATTN_F_KV_FROM_HBM)])
def test_ring_cache_and_region_offset(gpu_ready, po, hq, hkv, hd, flags):
    """Sliding layer on a wrapped power-of-two ring placed at a non-zero region offset, through the one-launch
    kernel and through the general one (also at head_dim 512 with the instance that touches tiles ahead of
    their loads: the touches stay inside the ring)."""
    import torch
    rng = np.random.default_rng(31)
    c, kvl, window, ring = 256, 5000, 1024, 2048
    t_all = kvl + c
    row = 2 * hkv * hd
    q = rng.standard_normal((c, hq, hd)).astype(np.float32)
    lin = rng.standard_normal((t_all, row)).astype(np.float32)
    qb, lb = R.f32_to_bf16_bits_rne(q), R.f32_to_f16_bits_rne(lin)
    ringbits = np.full((ring, row), 0x7E00, dtype=np.uint16)      # NaN everywhere: dead slots must not be read
    t_lo = kvl - (window - 1)
    for pos in range(t_lo, t_all):
        ringbits[pos & (ring - 1)] = lb[pos]
    region = 4096
    buf = np.concatenate([np.full(region // 2, 0x7E00, np.uint16), ringbits.ravel()])
    d = A.make_desc(c, hq, hkv, hd, kvl, window=window, kv_ring_mask=ring - 1, q_dtype=capi.DG_BF16,
                    kv_dtype=capi.DG_F16, out_dtype=capi.DG_F32, kv_region_bytes=region, flags=flags)
    out = torch.zeros(c * hq * hd, dtype=torch.float32, device="cuda")
    lse = torch.zeros(c * hq, dtype=torch.float32, device="cuda")
    A.forward(d, A.to_device_bits(qb), A.to_device_bits(buf), out, lse, A.alloc_workspace(d))
    torch.cuda.synchronize()
    od = po.make_desc(c, hq, hkv, hd, kvl, window=window)
    ref, ref_lse = po.attention_f32(od, R.bf16_bits_to_f32(qb), R.f16_bits_to_f32(lb))
    check_tolerances(out.cpu().numpy().reshape(ref.shape), lse.cpu().numpy().reshape(ref_lse.shape), ref, ref_lse,
                     max_abs=2e-3, mean_abs=1e-4)


def test_truncating_store_matches_reference_rounding(gpu_ready):
    import torch
    f = A.model_full_fixture(300, canvas=32)
    rig = A.AttnRig.from_fixture(f)

    def desc(truncate):   # the same fp32 partial rows behind all three stores
        d = rig.desc(kernel=capi.DG_KERNEL_MFMA, truncate=truncate)
        d.flags |= capi.DG_ATTN_F_F32_PARTIALS
        return d
    d32 = desc(False)
    d32.out_dtype = capi.DG_F32
    out32 = torch.zeros(f.out_len(), dtype=torch.float32, device="cuda")
    A.forward(d32, rig.buf_q, rig.buf_kv, out32, rig.buf_lse, rig.workspace_for(d32))
    rig.run_forward(desc(True))
    trunc = rig.read_out_f32()
    rig.run_forward(desc(False))
    rne = rig.read_out_f32()
    full = out32.cpu().numpy()
    assert np.array_equal(trunc, R.bf16_bits_to_f32(R.f32_to_bf16_bits_trunc(full)))
    assert np.array_equal(rne, R.bf16_bits_to_f32(R.f32_to_bf16_bits_rne(full)))


@pytest.mark.parametrize("fixture", ["tiny", "full_grp8_hd512"])
def test_debug_status_reports_nonfinite_output(gpu_ready, fixture):
    """A NaN in a visible V row reaches the output; the debug status record (first writer wins) names
    the attention kernel, a (token, head) it happened at and a head_dim index, like the reference's
    per-step invariant check (runtime.rs:565-571).  The tiny fixture runs in one pass, the other through
    the split path and the merge."""
    f = FIXTURES[fixture][0]()
    clean = A.AttnRig.from_fixture(f)
    clean.run_dispatch(causal=0)
    assert clean.read_debug_status().code == 0
    kv = f.kvcache.copy()
    hd, nkv = f.head_dim(), f.n_kv()
    slot = f.kv_len                                          # first canvas key: visible to every row
    kv[slot * 2 * nkv * hd + nkv * hd + 3] = np.float32(np.nan)   # V of KV head 0, element 3
    bad = A.AttnRig.from_fixture(A.Fixture(q=f.q, kvcache=kv, layer=f.layer, canvas=f.canvas, n_q_heads=f.n_q_heads, kv_len=f.kv_len))
    bad.run_dispatch(causal=0)
    st = bad.read_debug_status()
    # DbgErrNonFinite = 4 in DbgKernelAttention = 26: what the reference's check_status decodes
    assert (st.code, st.kernel_id) == (4, 26) == (capi.DG_DBG_ERR_NONFINITE, capi.DG_DBG_KERNEL_ATTENTION)
    tok, head = st.tg_id >> 16, st.tg_id & 0xffff
    assert tok < f.canvas and head < f.n_q_heads // nkv       # a head of the group that reads KV head 0
    assert st.value <= 3 < st.value + 8
    assert np.isnan(bad.read_out_f32()).any()


def test_row_without_visible_keys(gpu_ready):
    """An empty key range stores zeros and LSE = -inf instead of NaN (attention_mma2.metal:297)."""
    import torch
    w = W.Workload("empty", 16, 4, 2, 64, 40, t_lo=56, seed=1)   # t_lo == t_all
    for kernel in (capi.DG_KERNEL_MFMA, capi.DG_KERNEL_SCALAR):
        q, kv = W.generate(w)
        qd, kd = W.device_arrays(w, q, kv)
        d = w.desc(kernel=kernel)
        out = torch.full((w.canvas * w.n_q_heads * w.head_dim,), 7, dtype=torch.int16, device="cuda")
        lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
        A.forward(d, qd, kd, out, lse, A.alloc_workspace(d))
        torch.cuda.synchronize()
        assert torch.all(out == 0) and torch.all(torch.isneginf(lse))


def test_runtime_error_codes(gpu_ready):
    import torch
    w = W.scaled(W.config("cfg3_global"), 4096)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc()
    out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.int16, device="cuda")
    lib = capi.load()
    small = torch.empty(1024, dtype=torch.uint8, device="cuda")
    rc = lib.dg_attn_forward(C.byref(d), qd.data_ptr(), kd.data_ptr(), out.data_ptr(), None, small.data_ptr(), 1024,
                             A.stream_handle())
    assert rc == capi.DG_ERR_WORKSPACE
    rc = lib.dg_attn_forward(C.byref(d), qd.data_ptr(), kd.data_ptr(), out.data_ptr(), None, None, 0, A.stream_handle())
    assert rc == capi.DG_ERR_WORKSPACE
    rc = lib.dg_attn_forward(C.byref(d), qd.data_ptr() + 2, kd.data_ptr(), out.data_ptr(), None, small.data_ptr(),
                             1 << 30, A.stream_handle())
    assert rc == capi.DG_ERR_LAYOUT
    with pytest.raises(capi.DgAttnError):
        A.forward(W.Workload("bad", 8, 4, 2, 96, 8).desc(), qd, kd, out)
    torch.cuda.synchronize()


def test_hip_graph_replay(gpu_ready):
    """The call is capturable: no allocation, no host sync, no memset nodes.  Replays with
    eager work in between must keep matching the eager result."""
    import torch
    w = W.scaled(W.config("cfg3_global"), 4096)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc()
    n = w.canvas * w.n_q_heads * w.head_dim
    out_e = torch.zeros(n, dtype=torch.int16, device="cuda")
    out_g = torch.zeros(n, dtype=torch.int16, device="cuda")
    ws = A.alloc_workspace(d)
    A.forward(d, qd, kd, out_e, None, ws)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        A.forward(d, qd, kd, out_g, None, ws)     # warm the side stream
    torch.cuda.current_stream().wait_stream(s)
    with torch.cuda.graph(g):
        A.forward(d, qd, kd, out_g, None, ws)
    for i in range(4):
        out_g.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), i
        A.forward(d, qd, kd, out_e, None, ws)     # eager work between replays
        torch.cuda.synchronize()


def test_two_host_threads_on_two_streams(gpu_ready):
    """The library keeps no state that two callers share (plans are made per call; the cache memo and the
    profiling state are per thread): two host threads, each on a stream of its own with buffers of its own,
    calling in a loop at the same time get the bits a single caller gets.  (The entry that allocates nothing
    is the documented exception: its scratch is one per GPU.)"""
    import threading
    import torch
    shapes = [W.Workload("thr_a", 64, 16, 2, 512, 3000, causal_rows=32, seed=41),      # splits + merge
              W.Workload("thr_b", 64, 16, 8, 256, 2000, window=1024, seed=42)]          # one launch
    want = []
    for w in shapes:
        q, kv = W.generate(w)
        qd, kd = W.device_arrays(w, q, kv)
        d = w.desc()
        out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.int16, device="cuda")
        lse = torch.zeros(w.canvas * w.n_q_heads, dtype=torch.float32, device="cuda")
        A.forward(d, qd, kd, out, lse, A.alloc_workspace(d))
        torch.cuda.synchronize()
        want.append((d, qd, kd, out.clone(), lse.clone()))
    errors = []

    def worker(order):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                bufs = [(torch.zeros_like(o), torch.zeros_like(l), A.alloc_workspace(d)) for d, _, _, o, l in want]
                for it in range(40):
                    i = order[it % 2]
                    d, qd, kd, o_ref, l_ref = want[i]
                    o, l, ws = bufs[i]
                    o.zero_()
                    A.forward(d, qd, kd, o, l, ws)
                    if it % 8 == 7 or it >= 38:
                        stream.synchronize()
                        if not (torch.equal(o, o_ref) and torch.equal(l, l_ref)):
                            errors.append((order, it, i))
                stream.synchronize()
        except Exception as e:   # a failure in a thread must fail the test
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(o,)) for o in ((0, 1), (1, 0))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
