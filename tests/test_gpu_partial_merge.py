"""Key-range partials and their merge (dg_attn_partial / dg_attn_merge) and the reference's
sequential kv-block dispatch built on them (dg_attention_dispatch_block): the reference's
attention_mma_full carries (m, l, O) in attn_state between block dispatches
(src/shaders/attn/attention/attention_mma_full.metal:107-118,151-186,355-368, host loop
src/metal/step_kernel/enc.rs:2261-2291); its CPU statement is cpu_flash_blocked
(src/shaders/attn/attention_flash/mod.rs:20-94)."""
import ctypes as C

import numpy as np
import pytest

from diffgemma_amd import attention as A, capi, rounding as R, workloads as W

pytestmark = pytest.mark.gpu

CASES = {
    # name: (workload, cuts of [0, t_all): arbitrary, unaligned, with an empty range and one past the end)
    "global_mixed_mask": (lambda: W.scaled(W.config("cfg3_global"), 4096), [0, 1000, 1000, 3333, 4200, 4352 + 50]),
    "sliding_window": (lambda: W.config("cfg2_sliding"), [0, 3100, 3500, 4100, 4352]),
    "causal_prefill": (lambda: W.Workload("pm1", 300, 8, 2, 128, 700, causal_rows=300, seed=31), [0, 64, 650, 777, 1000]),
    "hd64_window": (lambda: W.Workload("pm2", 96, 8, 4, 64, 2000, window=512, seed=32), [0, 1500, 1700, 2096]),
}


def _oracle_desc(po, w):
    return po.make_desc(w.canvas, w.n_q_heads, w.n_kv_heads, w.head_dim, w.kv_len, causal_rows=w.causal_rows,
                        window=w.window, layout=w.layout, t_cap=w.t_all)


@pytest.mark.parametrize("name", list(CASES))
def test_partials_match_the_oracle_and_merge_to_the_single_call(gpu_ready, po, name):
    """Each partial's state equals the oracle's partial over the same keys (as output row acc / l and
    log-sum-exp m + ln l; rows that see no key of the range: l = 0); merged, the states give the same
    rows as one dg_attn_forward call and as the oracle's merge, within the output tolerance."""
    import torch
    make, cuts = CASES[name]
    w = make()
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc()
    od = _oracle_desc(po, w)
    rows = w.canvas * w.n_q_heads
    states, oparts = [], []
    for a, b in zip(cuts[:-1], cuts[1:]):
        st = A.alloc_state(d)
        st.fill_(0x7f)            # whatever the buffer held must not matter
        A.partial(d, a, b, qd, kd, st)
        torch.cuda.synchronize()
        m, l, acc = A.read_state(d, st)
        oacc, om, ol = po.attention_partial_f32(od, q, kv, a, min(b, w.t_all))
        seen = ol > 0
        assert np.array_equal(l > 0, seen), (a, b)
        assert np.all(acc[~seen] == 0) and np.all(np.isneginf(m[~seen]))
        states.append(st)
        oparts.append((oacc, om, ol))
        if not seen.any():
            continue
        want = oacc[seen] / ol[seen, None]
        got = acc[seen] / l[seen, None]
        assert np.abs(got - want).max() <= 2e-2 and np.abs(got - want).mean() <= 2e-3, (a, b)
        want_lse = om[seen] + np.log(ol[seen])
        got_lse = m[seen] + np.log(l[seen])
        assert np.all(np.abs(got_lse - want_lse) <= np.maximum(1e-3 * np.abs(want_lse), 2.0 ** -8)), (a, b)
    out = torch.zeros(rows * w.head_dim, dtype=torch.int16, device="cuda")
    lse = torch.zeros(rows, dtype=torch.float32, device="cuda")
    A.merge(d, states, out, lse)
    one = torch.zeros_like(out)
    one_lse = torch.zeros_like(lse)
    A.forward(d, qd, kd, one, one_lse, A.alloc_workspace(d))
    torch.cuda.synchronize()
    got = R.bf16_bits_to_f32(out.cpu().numpy().view(np.uint16)).reshape(rows, w.head_dim)
    single = R.bf16_bits_to_f32(one.cpu().numpy().view(np.uint16)).reshape(rows, w.head_dim)
    ref, ref_lse = po.merge_partials_f32(oparts, w.head_dim)
    for other in (single, ref):
        diff = np.abs(got - other)
        assert diff.max() <= 2e-2 and diff.mean() <= 2e-3
    lg = lse.cpu().numpy()
    assert np.all(np.abs(lg - ref_lse) <= np.maximum(1e-3 * np.abs(ref_lse), 2.0 ** -8))
    assert np.all(np.abs(lg - one_lse.cpu().numpy()) <= np.maximum(1e-3 * np.abs(ref_lse), 2.0 ** -8))


def test_merge_into_a_state_in_place_equals_merge_of_all(gpu_ready):
    """Folding states one at a time into a carried state (state_out = an input) gives the rows a
    single merge of all of them gives, to fp32 rounding."""
    import torch
    w = W.scaled(W.config("cfg3_global"), 2048)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc()
    d.out_dtype = capi.DG_F32
    cuts = [0, 500, 1100, 1800, w.t_all]
    states = []
    for a, b in zip(cuts[:-1], cuts[1:]):
        st = A.alloc_state(d)
        A.partial(d, a, b, qd, kd, st)
        states.append(st)
    n = w.canvas * w.n_q_heads * w.head_dim
    all_at_once = torch.zeros(n, dtype=torch.float32, device="cuda")
    A.merge(d, states, all_at_once)
    carried = states[0].clone()
    for st in states[1:]:
        A.merge(d, [carried, st], state_out=carried)
    folded = torch.zeros(n, dtype=torch.float32, device="cuda")
    A.merge(d, [carried], folded)
    torch.cuda.synchronize()
    a, b = all_at_once.cpu().numpy(), folded.cpu().numpy()
    assert np.isfinite(a).all() and np.abs(a - b).max() <= 1e-5 * max(1.0, np.abs(a).max())


@pytest.mark.parametrize("block", [4096, 1000])
def test_block_dispatch_equals_single_dispatch(gpu_ready, po, block):
    """The reference's host loop over kv blocks (enc.rs:2261-2291) against this library: blocks in order
    with {t_begin, t_end, is_first, is_last}, the state carried in attn_state; the result must agree with
    the single dispatch and with the reference CPU attention."""
    import torch
    f = A.model_full_fixture(8192 - 256)
    rig = A.AttnRig.from_fixture(f)
    lib = capi.load()
    lo, sp = A.layer_offsets(f), A.step_params(f.kv_len)
    dims = capi.AttnDims(canvas=f.canvas, n_q_heads=f.n_q_heads, causal=0, window=0)
    rig.run_dispatch()
    torch.cuda.synchronize()
    single = rig.buf_out.clone()
    n = C.c_size_t(0)
    capi.check(lib.dg_attention_block_state_bytes(C.byref(lo), C.byref(dims), f.kv_len, C.byref(n)))
    st = torch.full((n.value,), 0x55, dtype=torch.uint8, device="cuda")
    rig.buf_out.fill_(-1)
    t_total = f.kv_len + f.canvas
    blocks = -(-t_total // block)
    assert blocks > 1
    for b in range(blocks):
        blk = capi.AttnBlockRange(b * block, min((b + 1) * block, t_total), int(b == 0), int(b + 1 == blocks))
        capi.check(lib.dg_attention_dispatch_block(rig.buf_q.data_ptr(), rig.buf_kv.data_ptr(), rig.buf_out.data_ptr(),
                                                   C.byref(lo), C.byref(sp), C.byref(dims), C.byref(blk),
                                                   rig.buf_dbg.data_ptr(), st.data_ptr(), st.numel(), A.stream_handle()))
    torch.cuda.synchronize()
    assert int(rig.buf_dbg.cpu()[0]) == 0
    got = R.bf16_bits_to_f32(rig.buf_out.cpu().numpy().view(np.uint16))
    want = R.bf16_bits_to_f32(single.cpu().numpy().view(np.uint16))
    # the truncating store moves a value by up to one bf16 step when the fp32 sums differ in their last bits
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -7 + 1e-6)
    assert np.mean(got != want) < 0.15   # (measured 6 %: the probabilities are rounded against other reference maxima per block)
    # and with the reference CPU attention on the stored values (attention/mod.rs:218-240)
    q = R.bf16_bits_to_f32(R.f32_to_bf16_bits_trunc(f.q))
    kv = R.f16_bits_to_f32(R.f32_to_f16_bits_trunc(f.kvcache))
    toks = np.array([0, 100, 255], dtype=np.uint32)
    ref, _ = po.attention_f32(po.make_desc(f.canvas, f.n_q_heads, f.n_kv(), f.head_dim(), f.kv_len), q, kv, tok_list=toks)
    g = got.reshape(f.canvas, f.n_q_heads, f.head_dim())[toks]
    assert np.abs(g - ref[toks]).max() <= 2e-2 and np.abs(g - ref[toks]).mean() <= 2e-3


def test_block_dispatch_replays_in_a_graph(gpu_ready):
    """The block sequence records no memset node, allocates nothing and synchronises nothing, so it can be
    captured; replays (with eager work and synchronisations between them) must give the eager bits."""
    import torch
    f = A.model_full_fixture(4096 - 256)
    rig = A.AttnRig.from_fixture(f)
    lib = capi.load()
    lo, sp = A.layer_offsets(f), A.step_params(f.kv_len)
    dims = capi.AttnDims(canvas=f.canvas, n_q_heads=f.n_q_heads, causal=0, window=0)
    n = C.c_size_t(0)
    capi.check(lib.dg_attention_block_state_bytes(C.byref(lo), C.byref(dims), f.kv_len, C.byref(n)))
    st = torch.zeros(n.value, dtype=torch.uint8, device="cuda")
    t_total, block = f.kv_len + f.canvas, 1500
    blocks = -(-t_total // block)

    def encode():
        for b in range(blocks):
            blk = capi.AttnBlockRange(b * block, min((b + 1) * block, t_total), int(b == 0), int(b + 1 == blocks))
            capi.check(lib.dg_attention_dispatch_block(rig.buf_q.data_ptr(), rig.buf_kv.data_ptr(), rig.buf_out.data_ptr(),
                                                       C.byref(lo), C.byref(sp), C.byref(dims), C.byref(blk), None,
                                                       st.data_ptr(), st.numel(), A.stream_handle()))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        encode()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    want = rig.buf_out.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        encode()
    for rep in range(3):
        rig.buf_out.fill_(-1)
        st.fill_(rep)                 # the carried state of an earlier sequence must not matter
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(rig.buf_out, want), rep


def test_partial_argument_checks(gpu_ready):
    import torch
    w = W.scaled(W.config("cfg3_global"), 1024)
    q, kv = W.generate(w)
    qd, kd = W.device_arrays(w, q, kv)
    d = w.desc()
    lib = capi.load()
    st = A.alloc_state(d)
    ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    call = lambda a, b, sb: lib.dg_attn_partial(C.byref(d), a, b, qd.data_ptr(), kd.data_ptr(), st.data_ptr(), sb,
                                                ws.data_ptr(), ws.numel(), None)
    assert call(100, 50, st.numel()) == capi.DG_ERR_MASK            # range backwards
    assert call(0, 100, st.numel() - 16) == capi.DG_ERR_WORKSPACE   # state too small
    arr = (C.c_void_p * 17)(*[st.data_ptr()] * 17)
    out = torch.zeros(w.canvas * w.n_q_heads * w.head_dim, dtype=torch.int16, device="cuda")
    assert lib.dg_attn_merge(C.byref(d), arr, 17, out.data_ptr(), None, None, None) == capi.DG_ERR_SHAPE
    assert lib.dg_attn_merge(C.byref(d), arr, 0, out.data_ptr(), None, None, None) == capi.DG_ERR_SHAPE
    assert lib.dg_attn_merge(C.byref(d), arr, 2, None, None, None, None) == capi.DG_ERR_NULL
    torch.cuda.synchronize()
