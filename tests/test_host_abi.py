"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the
header declares, the reference-shaped structs have the reference's sizes, descriptor
validation returns the documented status codes, and the KV layout arithmetic matches the
reference's (src/metal/step_kv/mod.rs:65-100, src/metal/step_kernel/mod.rs:511-587)."""
import ctypes as C
import os
import re

import pytest

from diffgemma_amd import attention as A
from diffgemma_amd import capi, step_kv, workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    inc = os.path.join(ROOT, "include")
    text = "".join(open(os.path.join(inc, f)).read() for f in sorted(os.listdir(inc)) if f.endswith(".h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = header_functions()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/*.h but not exported"
    assert set(names) == set(capi.EXPORTS)
    assert lib.dg_attn_abi_version() == 1


def test_headers_are_plain_c(tmp_path):
    """include/*.h is what a foreign-function generator (bindgen, cgo) reads: it has to be C, not C++."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "hdr.c"
    src.write_text('#include "dg_attn.h"\n#include "dg_attn_bench.h"\n'
                   "int main(void) { dg_attn_desc d; dg_rope_desc r; dg_layer_offsets l; (void)d; (void)r; (void)l; "
                   "return sizeof(dg_step_params) == 48 && sizeof(dg_attn_dims) == 16 ? 0 : 1; }\n")
    res = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                          str(src), "-o", str(tmp_path / "hdr")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout
    assert subprocess.run([str(tmp_path / "hdr")]).returncode == 0


def test_flag_constants_match_the_header():
    """The ctypes binding spells the desc.flags bits out again: they must be the header's."""
    text = open(os.path.join(ROOT, "include", "dg_attn.h")).read()
    defs = dict(re.findall(r"#define\s+(DG_ATTN_F_[A-Z0-9_]+)\s+(0x[0-9a-fA-F]+)u?", text))
    assert len(defs) >= 7
    for name, value in defs.items():
        assert getattr(capi, name) == int(value, 16), name
    assert len(set(defs.values())) == len(defs)          # no two flags share a bit


def test_debug_status_vocabulary_is_the_references():
    """The numbers the reference's host side decodes (src/metal/debug_status.rs:33-75): DbgErrorCode of
    src/shaders/include/debug_status.metal:8-19 and DbgKernelId of src/shaders/include/dgq_kernels.metal:33-34."""
    want = {"DG_DBG_ERR_SOFTMAX_NORM_ZERO": 3, "DG_DBG_ERR_NONFINITE": 4, "DG_DBG_ERR_BAD_DIM": 8,
            "DG_DBG_KERNEL_QK_ROPE_KV": 25, "DG_DBG_KERNEL_ATTENTION": 26}
    text = open(os.path.join(ROOT, "include", "dg_attn.h")).read()
    defs = {k: int(v) for k, v in re.findall(r"#define\s+(DG_DBG_[A-Z0-9_]+)\s+(\d+)u", text)}
    assert defs == want
    for name, value in want.items():
        assert getattr(capi, name) == value, name
    # the kernels' own spelling of the same numbers
    src = open(os.path.join(ROOT, "diffgemma_amd", "csrc", "attn_params.h")).read()
    dev = {k: int(v) for k, v in re.findall(r"(DBG_(?:ERR|KERNEL)_[A-Z0-9_]+) = (\d+)u", src)}
    assert dev == {k[3:]: v for k, v in want.items()}
    # no kernel source writes a literal code or kernel id
    for f in os.listdir(os.path.join(ROOT, "diffgemma_amd", "csrc")):
        body = open(os.path.join(ROOT, "diffgemma_amd", "csrc", f)).read()
        for call in re.findall(r"dbg_report\(([^;]*)\);", body):
            if "uint32_t* dbg" in call:
                continue
            args = [a.strip() for a in call.split(",")]
            assert args[1].startswith("DBG_ERR_") and args[2].startswith("DBG_KERNEL_"), (f, call)


def test_reference_struct_sizes():
    assert C.sizeof(capi.LayerOffsets) == 200     # 23 u64 + 4 u32, repr(C)
    assert C.sizeof(capi.StepParams) == 48
    assert C.sizeof(capi.AttnDims) == 16
    assert C.sizeof(capi.AttnBlockRange) == 16
    assert C.sizeof(capi.DebugStatus) == 16
    assert capi.LayerOffsets.kv_region.offset == 176 and capi.LayerOffsets.kv_ring_mask.offset == 196
    assert C.sizeof(capi.AttnDesc) == 112


def test_strerror_covers_every_status():
    seen = set()
    for code in range(0, -10, -1):
        text = capi.strerror(code)
        assert text and text != "unknown status"
        seen.add(text)
    assert len(seen) == 10
    assert capi.strerror(-99) == "unknown status"


def _status(desc):
    n = C.c_size_t(0)
    return capi.load().dg_attn_workspace_bytes(C.byref(desc), C.byref(n))


def test_descriptor_validation_codes():
    ok = A.make_desc(256, 16, 2, 512, 1024)
    assert _status(ok) == capi.DG_OK
    assert _status(A.make_desc(256, 16, 2, 96, 1024)) == capi.DG_ERR_SHAPE         # head_dim
    assert _status(A.make_desc(0, 16, 2, 512, 1024)) == capi.DG_ERR_SHAPE          # empty canvas
    assert _status(A.make_desc(256, 16, 3, 512, 1024)) == capi.DG_ERR_SHAPE        # Hq % Hkv
    assert _status(A.make_desc(65536, 128, 2, 512, 1024)) == capi.DG_ERR_SHAPE     # query rows past 4 GiB (32-bit row offsets)
    assert _status(A.make_desc(65536, 32, 2, 512, 1024)) == capi.DG_OK
    assert _status(A.make_desc(256, 16, 2, 512, 1024, causal_rows=257)) == capi.DG_ERR_MASK
    assert _status(A.make_desc(256, 16, 2, 512, 1024, kv_ring_mask=1000)) == capi.DG_ERR_LAYOUT
    assert _status(A.make_desc(256, 16, 2, 512, 1024, kv_ring_mask=15)) == capi.DG_ERR_LAYOUT  # ring < key tile
    # the ring must hold every visible position: window-1 + canvas of them
    assert _status(A.make_desc(1024, 16, 8, 256, 4096, causal_rows=1024, window=1024, kv_ring_mask=2047)) == capi.DG_OK
    assert _status(A.make_desc(1024, 16, 8, 256, 4096, causal_rows=1024, window=1026, kv_ring_mask=2047)) == capi.DG_ERR_LAYOUT
    assert _status(A.make_desc(256, 16, 8, 256, 4096, kv_ring_mask=2047)) == capi.DG_ERR_LAYOUT  # no window: 4352 positions
    assert _status(A.make_desc(256, 16, 2, 512, 1024, kv_dtype=7)) == capi.DG_ERR_DTYPE
    assert _status(A.make_desc(256, 16, 2, 512, 1024, q_dtype=capi.DG_F16, kv_dtype=capi.DG_BF16)) == capi.DG_ERR_DTYPE
    assert _status(A.make_desc(256, 16, 2, 512, 1024, out_dtype=capi.DG_F16)) == capi.DG_ERR_DTYPE
    assert _status(A.make_desc(256, 16, 2, 512, 1024, kernel=9)) == capi.DG_ERR_UNSUPPORTED
    assert _status(A.make_desc(256, 16, 2, 512, 1024, flags=capi.DG_ATTN_F_T_LO_EXPLICIT, t_lo=5000)) == capi.DG_ERR_MASK
    bad = A.make_desc(256, 16, 2, 512, 1024)
    bad.k_tok_stride = 1028                                                        # not 16-byte rows
    assert _status(bad) == capi.DG_ERR_LAYOUT
    bad = A.make_desc(256, 16, 2, 512, 1024)
    bad.kv_region_bytes = 8
    assert _status(bad) == capi.DG_ERR_LAYOUT
    assert capi.load().dg_attn_workspace_bytes(None, None) == capi.DG_ERR_NULL


def test_forward_rejects_null_pointers_before_touching_a_device():
    d = A.make_desc(4, 4, 2, 32, 8)
    assert capi.load().dg_attn_forward(C.byref(d), None, None, None, None, None, 0, None) == capi.DG_ERR_NULL
    assert capi.load().dg_attention_dispatch(None, None, None, None, None, None, None, None, 0, None) == capi.DG_ERR_NULL


def test_layout_helpers():
    d = A.make_desc(256, 16, 8, 256, 4096, layout="reference")
    assert (d.k_tok_stride, d.k_head_stride, d.v_base_off, d.v_tok_stride, d.v_head_stride) == (4096, 256, 2048, 4096, 256)
    d = A.make_desc(256, 16, 2, 512, 32768, layout="head_major")
    t = 32768 + 256
    assert (d.k_tok_stride, d.k_head_stride, d.v_base_off, d.v_tok_stride, d.v_head_stride) == (512, t * 512, 2 * t * 512, 512, t * 512)


def test_split_planning():
    assert capi.resolved_splits(W.config("cfg3_global").desc()) == 8          # 32 (tile, head) pairs x 8 = 256 workgroups
    assert capi.resolved_splits(W.config("cfg4_long").desc()) == 8
    # a sliding layer (head_dim 256, 40 visible key tiles) runs as one launch, keys split over the waves of a
    # workgroup: no splits over workgroups, no workspace; asked for the general kernel it takes 6 splits
    assert capi.resolved_splits(W.config("cfg2_sliding").desc()) == 1
    assert capi.workspace_bytes(W.config("cfg2_sliding").desc()) == 0
    over_wg = capi.DG_ATTN_F_SPLIT_OVER_WORKGROUPS
    assert capi.resolved_splits(W.config("cfg2_sliding").desc(flags=over_wg)) == 6        # 40 visible tiles, 7 to a split (none shorter than 6)
    assert capi.resolved_splits(W.config("cfg2_sliding_768").desc(flags=over_wg)) == 5    # 32 visible tiles, 7 to a split
    assert capi.workspace_bytes(W.config("cfg2_sliding").desc(flags=over_wg)) == 6 * 8 * 512 * (256 * 2 + 2 * 4)
    # the same head_dim over a long unwindowed range goes to the general kernel by itself
    assert capi.resolved_splits(A.make_desc(256, 16, 8, 256, 8192)) == 8
    assert capi.resolved_splits(A.make_desc(2, 4, 2, 32, 2)) == 1                 # one tile: nothing to split
    assert capi.resolved_splits(A.make_desc(256, 16, 2, 512, 32768, n_splits=3)) == 3
    assert capi.resolved_splits(A.make_desc(256, 16, 2, 512, 32768, kernel=capi.DG_KERNEL_SCALAR)) == 1
    # workspace: 8 splits x 2 heads x 2048 rows x (512 fp32 accumulators + (m, l)); the partial rows take
    # half of that as f16 (the workload descriptors vouch for the range of V)
    assert capi.workspace_bytes(W.config("cfg3_global").desc(flags=capi.DG_ATTN_F_F32_PARTIALS)) == 8 * 2 * 2048 * 514 * 4
    assert capi.workspace_bytes(W.config("cfg3_global").desc()) == 8 * 2 * 2048 * (512 * 2 + 2 * 4)
    assert capi.workspace_bytes(A.make_desc(256, 16, 2, 512, 32768)) == 8 * 2 * 2048 * 514 * 4                  # bf16 cache: fp32 unless asked
    assert capi.workspace_bytes(A.make_desc(256, 16, 2, 512, 32768, kv_dtype=capi.DG_F16)) == 8 * 2 * 2048 * (512 * 2 + 2 * 4)
    assert capi.workspace_bytes(A.make_desc(2, 4, 2, 32, 2)) == 0


def test_topk_planning_and_validation():
    from diffgemma_amd import attention_topk as T
    d = W.config("cfg3_global").desc()
    # score plane of one block of canvas rows: 64 rows x 16 heads x 33024 keys (a multiple of 32) x fp32 <= 144 MiB
    assert T.workspace_bytes(d, T.adaptive_k()) == 64 * 16 * 33024 * 4
    small = A.make_desc(8, 4, 2, 64, 100)
    assert T.workspace_bytes(small, T.fixed_k(64)) == 8 * 4 * 128 * 4            # whole canvas in one block, keys padded to 128
    lib = capi.load()
    n = C.c_size_t(0)
    cfg = lambda *v: (C.c_uint32 * 4)(*v)
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), cfg(1025, 0, 0, 0), C.byref(n)) == capi.DG_ERR_SHAPE
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), cfg(1024, 0, 0, 0), C.byref(n)) == capi.DG_OK
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), cfg(256, 128, 64, 1025), C.byref(n)) == capi.DG_ERR_SHAPE
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), cfg(256, 128, 513, 512), C.byref(n)) == capi.DG_ERR_SHAPE
    assert lib.dg_attn_topk_workspace_bytes(C.byref(d), None, C.byref(n)) == capi.DG_ERR_NULL
    scalar = A.make_desc(8, 4, 2, 64, 100, kernel=capi.DG_KERNEL_SCALAR)
    assert lib.dg_attn_topk_workspace_bytes(C.byref(scalar), cfg(8, 0, 0, 0), C.byref(n)) == capi.DG_ERR_UNSUPPORTED
    f32 = A.make_desc(8, 4, 2, 64, 100, q_dtype=capi.DG_F32, kv_dtype=capi.DG_F32, out_dtype=capi.DG_F32)
    assert lib.dg_attn_topk_workspace_bytes(C.byref(f32), cfg(8, 0, 0, 0), C.byref(n)) == capi.DG_ERR_UNSUPPORTED
    # the reference-shaped size query agrees with the general one (bf16 Q, f16 cache, slot-major)
    f = A.full_grp8_hd512_fixture()
    lo, dims = A.layer_offsets(f), capi.AttnDims(canvas=f.canvas, n_q_heads=f.n_q_heads, causal=1, window=0)
    assert lib.dg_attention_topk_state_bytes(C.byref(lo), C.byref(dims), f.kv_len, cfg(64, 0, 0, 0), C.byref(n)) == capi.DG_OK
    t_pad = -(-(f.kv_len + f.canvas) // 32) * 32
    assert n.value == f.canvas * f.n_q_heads * t_pad * 4
    assert T.k_pad_for(1) == 64 and T.k_pad_for(65) == 128 and T.k_pad_for(5000) == 1024     # mod.rs:34-36
    assert T.fixed_k(0) == (1, 0, 0, 0) and T.fixed_k(100) == (100, 0, 0, 0)


def test_visible_pairs_and_flops():
    pairs, flops = capi.visible_pairs(W.config("cfg3_global").desc())
    assert pairs == 8429632 and flops == 4.0 * 512 * 16 * 8429632
    assert capi.visible_pairs(W.config("cfg3_global_b").desc())[0] == 8446016
    assert capi.visible_pairs(W.config("cfg2_sliding").desc())[0] == 256 * 1279
    assert capi.visible_pairs(W.config("cfg2_sliding_768").desc())[0] == 256 * 1024
    assert capi.visible_pairs(W.config("cfg4_long").desc())[0] == 256 * 131328


def test_host_and_oracle_agree_on_pair_counts(po):
    import itertools
    lib = po.load()
    for c, kvl, cr, win, sees in itertools.product((1, 7, 64), (0, 5, 300), (0, 3, 64), (0, 2, 50), (0, 1)):
        if cr > c:
            continue
        d = A.make_desc(c, 4, 2, 32, kvl, causal_rows=cr, window=win,
                        flags=capi.DG_ATTN_F_CAUSAL_SEES_MASKED if sees else 0)
        od = po.make_desc(c, 4, 2, 32, kvl, causal_rows=cr, window=win, causal_sees_masked=sees)
        assert capi.visible_pairs(d)[0] == lib.dgo_visible_pairs(C.byref(od)), (c, kvl, cr, win, sees)


def test_kv_layout_arithmetic():
    assert step_kv.kv_row_bytes(256) == 512 and step_kv.kv_row_bytes(512) == 1024
    assert step_kv.kv_region_bytes(8, 256, 4096) == 4096 * 8 * 2 * 512          # 32 MiB ring
    assert step_kv.layer_kv_slots(True, 32768 + 256) == 33032                   # (max_seq + 8) rounded to 8
    assert step_kv.layer_kv_slots(False, 33024) == 4096                         # pow2 capped at the ring size
    assert step_kv.layer_kv_slots(False, 1000) == 1024
    assert step_kv.kv_slot(4095, 5000) == 5000 & 4095 and step_kv.kv_slot(0, 5000) == 5000
    layers = step_kv.build_layout(33024)
    assert [l.layer for l in layers if l.is_full] == [5, 11, 17, 23, 29]
    assert layers[0].kv_region == 0 and layers[1].kv_region == 32 << 20
    assert layers[6].kv_region == 6 * (32 << 20) - (32 << 20) + step_kv.kv_region_bytes(2, 512, 33032)
    assert all(l.kv_ring_mask == (0 if l.is_full else 4095) for l in layers)
    total = step_kv.kv_cache_total_bytes(layers)
    assert total == 25 * (32 << 20) + 5 * step_kv.kv_region_bytes(2, 512, 33032)
    lo = layers[5].offsets()
    assert (lo.head_dim, lo.n_kv_heads, lo.is_full, lo.kv_ring_mask) == (512, 2, 1, 0)


def test_profile_helpers_refuse_misuse():
    lib = capi.load()
    assert lib.dg_prof_end(None, None) == capi.DG_ERR_UNSUPPORTED   # not begun


def test_workload_table():
    w = W.config("cfg3_global")
    assert (w.canvas, w.n_q_heads, w.n_kv_heads, w.head_dim, w.kv_len, w.causal_rows) == (256, 16, 2, 512, 32768, 128)
    w = W.scaled(W.config("cfg2_sliding_768"), 2048)
    assert w.t_lo == 2048 - 768
    with pytest.raises(KeyError):
        W.config("nope")


def test_block_state_covers_every_block_partial():
    """dg_attention_block_state_bytes must hold the carried state, a fresh state and the workspace of the
    partial of ANY block [a, b) of the key range: the split count a range resolves to is not monotone in
    its length, so a shorter block can need more partial rows than the whole range."""
    lib = capi.load()
    for hd, nkv in ((512, 2), (256, 8)):
        L = capi.LayerOffsets()
        L.head_dim, L.n_kv_heads, L.is_full, L.kv_ring_mask = hd, nkv, int(hd == 512), 0
        dims = capi.AttnDims(256, 16, 0, 0)
        for kv_len in list(range(0, 4200, 97)) + [1287, 32768, 131072]:
            total, sb = C.c_size_t(0), C.c_size_t(0)
            capi.check(lib.dg_attention_block_state_bytes(C.byref(L), C.byref(dims), kv_len, C.byref(total)))
            d = A.make_desc(256, 16, nkv, hd, kv_len, q_dtype=capi.DG_BF16, kv_dtype=capi.DG_F16, out_dtype=capi.DG_BF16,
                            flags=capi.DG_ATTN_F_OUT_TRUNCATE)
            capi.check(lib.dg_attn_state_bytes(C.byref(d), C.byref(sb)))
            state = (sb.value + 255) // 256 * 256
            t_all = kv_len + 256
            ends = sorted(set(list(range(32, t_all + 64, max(32, t_all // 61))) + [t_all, 1536]))
            for b in ends:
                for a in (0, b // 3 // 8 * 8):
                    ws = C.c_size_t(0)
                    capi.check(lib.dg_attn_partial_workspace_bytes(C.byref(d), a, b, C.byref(ws)))
                    assert ws.value <= total.value - 2 * state, (hd, kv_len, a, b, ws.value, total.value, state)
