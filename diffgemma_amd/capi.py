"""ctypes binding of include/dg_attn.h and include/dg_attn_bench.h (libdg_attn_hip.so)."""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "libdg_attn_hip.so"

DG_BF16, DG_F16, DG_F32 = 0, 1, 2
DG_KERNEL_AUTO, DG_KERNEL_SCALAR, DG_KERNEL_MFMA = 0, 1, 2
DG_ATTN_F_OUT_TRUNCATE = 0x1
DG_ATTN_F_CAUSAL_SEES_MASKED = 0x2
DG_ATTN_F_T_LO_EXPLICIT = 0x4
DG_ATTN_F_F32_PARTIALS = 0x8
DG_ATTN_F_F16_PARTIALS = 0x10
DG_ATTN_F_STREAMED_MERGE = 0x20
DG_ATTN_F_KV_FROM_HBM = 0x40
DG_ATTN_F_SPLIT_OVER_WORKGROUPS = 0x80
DG_ATTN_F_KV_CACHED = 0x100
# the reference's DebugStatus vocabulary (debug_status.metal:8-19, dgq_kernels.metal:33-34)
DG_DBG_ERR_SOFTMAX_NORM_ZERO = 3
DG_DBG_ERR_NONFINITE = 4
DG_DBG_ERR_BAD_DIM = 8
DG_DBG_KERNEL_QK_ROPE_KV = 25
DG_DBG_KERNEL_ATTENTION = 26

DG_ROPE_F_QK_TRUNCATE = 0x1

DG_OK = 0
DG_ERR_NULL, DG_ERR_SHAPE, DG_ERR_DTYPE, DG_ERR_LAYOUT = -1, -2, -3, -4
DG_ERR_WORKSPACE, DG_ERR_MASK, DG_ERR_LAUNCH, DG_ERR_DEVICE, DG_ERR_UNSUPPORTED = -5, -6, -7, -8, -9
DG_ERR_SCRATCH_LIMIT = -10

# every symbol include/*.h declares
EXPORTS = (
    "dg_attn_desc_reference_layout", "dg_attn_desc_head_major_layout", "dg_attn_workspace_bytes",
    "dg_attn_resolved_splits", "dg_attn_forward", "dg_attn_strerror", "dg_attn_abi_version",
    "dg_attn_visible_pairs", "dg_attention_dispatch", "dg_attention_state_bytes", "dg_kv_row_bytes",
    "dg_kv_region_bytes", "dg_kv_slot", "dg_layer_kv_slots", "dg_prof_begin", "dg_prof_end",
    "dg_calib_copy", "dg_calib_mfma", "dg_qk_rope_kv", "dg_qk_rope_kv_dispatch",
    "dg_attn_topk_workspace_bytes", "dg_attn_topk_forward", "dg_attention_topk_state_bytes",
    "dg_attention_topk_dispatch", "dg_prof_end_split",
    "dg_kv_layer_reference_layout", "dg_kv_layer_head_major_layout", "dg_kv_snapshot_bytes", "dg_kv_snapshot_gather",
    "dg_kv_snapshot_scatter", "dg_kv_live_bytes", "dg_kv_live_gather", "dg_fnv1a64",
    "dg_attn_forward_static", "dg_attn_static_scratch_bytes",
    "dg_attn_state_bytes", "dg_attn_partial_workspace_bytes", "dg_attn_partial", "dg_attn_merge",
    "dg_attention_dispatch_block", "dg_attention_block_state_bytes",
    "dg_attn_forward_dev", "dg_attention_dispatch_dev", "dg_qk_rope_kv_dev", "dg_qk_rope_kv_dispatch_dev",
)


class AttnDesc(C.Structure):
    _fields_ = [
        ("canvas", C.c_uint32), ("n_q_heads", C.c_uint32), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
        ("kv_len", C.c_uint32), ("causal_rows", C.c_uint32), ("window", C.c_uint32), ("kv_ring_mask", C.c_uint32),
        ("q_dtype", C.c_uint32), ("kv_dtype", C.c_uint32), ("out_dtype", C.c_uint32), ("flags", C.c_uint32),
        ("t_lo", C.c_uint32), ("n_splits", C.c_uint32), ("kernel", C.c_uint32), ("softmax_scale", C.c_float),
        ("kv_region_bytes", C.c_uint64),
        ("k_tok_stride", C.c_int64), ("k_head_stride", C.c_int64),
        ("v_base_off", C.c_int64), ("v_tok_stride", C.c_int64), ("v_head_stride", C.c_int64),
    ]


class RopeDesc(C.Structure):
    """dg_rope_desc: the producer of the cache rows (RMSNorm + RoPE + KV write)."""
    _fields_ = [
        ("canvas", C.c_uint32), ("n_q_heads", C.c_uint32), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
        ("kv_len", C.c_uint32), ("kv_write_end", C.c_uint32), ("kv_ring_mask", C.c_uint32), ("is_full", C.c_uint32),
        ("v_from_k", C.c_uint32), ("kv_dtype", C.c_uint32), ("flags", C.c_uint32), ("reserved", C.c_uint32),
        ("kv_region_bytes", C.c_uint64),
        ("k_tok_stride", C.c_int64), ("k_head_stride", C.c_int64),
        ("v_base_off", C.c_int64), ("v_tok_stride", C.c_int64), ("v_head_stride", C.c_int64),
    ]


class KvLayer(C.Structure):
    """dg_kv_layer: one layer's region of the KV cache, for the snapshot calls."""
    _fields_ = [
        ("kv_region_bytes", C.c_uint64), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
        ("slots", C.c_uint32), ("kv_ring_mask", C.c_uint32), ("kv_dtype", C.c_uint32), ("reserved", C.c_uint32),
        ("k_tok_stride", C.c_int64), ("k_head_stride", C.c_int64),
        ("v_base_off", C.c_int64), ("v_tok_stride", C.c_int64), ("v_head_stride", C.c_int64),
    ]


class LayerOffsets(C.Structure):
    """Reference LayerOffsets (src/metal/step_kernel/mod.rs:132-167), repr(C), 200 bytes."""
    _fields_ = [(n, C.c_uint64) for n in (
        "input_ln", "q_proj", "q_norm", "k_proj", "k_norm", "v_proj", "o_proj", "post_attn_ln",
        "pre_ff_ln", "mlp_gate", "mlp_up", "mlp_down", "post_ff_ln_1",
        "router_scale", "router_proj", "per_expert_scale", "pre_ff_ln_2",
        "experts_gate_up", "experts_down", "post_ff_ln_2", "post_ff_ln", "layer_scalar", "kv_region")] + [
        ("head_dim", C.c_uint32), ("n_kv_heads", C.c_uint32), ("is_full", C.c_uint32), ("kv_ring_mask", C.c_uint32)]


class StepParams(C.Structure):
    """Reference StepParams (src/metal/step_kernel/mod.rs:189-213), 48 bytes."""
    _fields_ = [
        ("kv_len", C.c_uint32), ("max_steps", C.c_uint32), ("entropy_bound", C.c_float), ("t_min", C.c_float),
        ("t_max", C.c_float), ("conf_threshold", C.c_float), ("stability_threshold", C.c_uint32),
        ("min_early_stop_steps", C.c_uint32), ("accept_plateau_threshold", C.c_uint32),
        ("plateau_prefix_mean_max", C.c_float), ("eos_token_id", C.c_uint32), ("kv_write_end", C.c_uint32),
    ]


class AttnDims(C.Structure):
    """Reference AttnDims (src/shaders/attn/qk_rope_kv/mod.rs:15-38), 16 bytes."""
    _fields_ = [("canvas", C.c_uint32), ("n_q_heads", C.c_uint32), ("causal", C.c_uint32), ("window", C.c_uint32)]


class AttnBlockRange(C.Structure):
    _fields_ = [("t_begin", C.c_uint32), ("t_end", C.c_uint32), ("is_first", C.c_uint32), ("is_last", C.c_uint32)]


class DebugStatus(C.Structure):
    _fields_ = [("code", C.c_uint32), ("kernel_id", C.c_uint32), ("tg_id", C.c_uint32), ("value", C.c_uint32)]


class DgAttnError(RuntimeError):
    def __init__(self, status: int, text: str):
        super().__init__(f"dg_attn status {status}: {text}")
        self.status = status


_lib = None


def load():
    """Load the HIP library; raise (never fall back) when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = Path(os.environ.get("DG_ATTN_LIB", LIB_PATH))
    if not path.exists():
        raise RuntimeError(
            f"{path} is missing: build it with `python -m diffgemma_amd.build` (needs hipcc); "
            "there is no CPU fallback for the attention path")
    # One HIP runtime per process.  PyTorch brings its own libamdhip64.so.7 and the library was linked against the
    # system's, same soname: the dynamic loader gives every later user whichever copy came first.  The tensors this
    # package hands to the library are PyTorch's, so PyTorch's runtime has to be that copy: loaded the other way
    # round, the first launch fails with DG_ERR_DEVICE ("no gfx950 device current").  (A C or Rust host links one
    # runtime and has no such choice to make.)
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(str(path))
    P, VP = C.POINTER, C.c_void_p
    lib.dg_attn_desc_reference_layout.argtypes = [P(AttnDesc)]
    lib.dg_attn_desc_reference_layout.restype = None
    lib.dg_attn_desc_head_major_layout.argtypes = [P(AttnDesc), C.c_uint64]
    lib.dg_attn_desc_head_major_layout.restype = None
    lib.dg_attn_workspace_bytes.argtypes = [P(AttnDesc), P(C.c_size_t)]
    lib.dg_attn_workspace_bytes.restype = C.c_int
    lib.dg_attn_resolved_splits.argtypes = [P(AttnDesc), P(C.c_uint32)]
    lib.dg_attn_resolved_splits.restype = C.c_int
    lib.dg_attn_forward.argtypes = [P(AttnDesc), VP, VP, VP, VP, VP, C.c_size_t, VP]
    lib.dg_attn_forward.restype = C.c_int
    lib.dg_attn_forward_dev.argtypes = [P(AttnDesc), VP, VP, VP, VP, VP, VP, C.c_size_t, VP]
    lib.dg_attn_forward_dev.restype = C.c_int
    lib.dg_attention_dispatch_dev.argtypes = [VP, VP, VP, P(LayerOffsets), VP, C.c_uint32, P(AttnDims), VP, VP,
                                              C.c_size_t, VP]
    lib.dg_attention_dispatch_dev.restype = C.c_int
    lib.dg_qk_rope_kv_dev.argtypes = [P(RopeDesc), VP, VP, VP, VP, VP, VP, VP, VP, VP]
    lib.dg_qk_rope_kv_dev.restype = C.c_int
    lib.dg_qk_rope_kv_dispatch_dev.argtypes = [VP, VP, VP, VP, VP, P(LayerOffsets), VP, P(AttnDims), VP, VP]
    lib.dg_qk_rope_kv_dispatch_dev.restype = C.c_int
    lib.dg_attn_forward_static.argtypes = [P(AttnDesc), VP, VP, VP, VP, VP]
    lib.dg_attn_forward_static.restype = C.c_int
    lib.dg_attn_static_scratch_bytes.argtypes = []
    lib.dg_attn_static_scratch_bytes.restype = C.c_size_t
    lib.dg_attn_strerror.argtypes = [C.c_int]
    lib.dg_attn_strerror.restype = C.c_char_p
    lib.dg_attn_abi_version.argtypes = []
    lib.dg_attn_abi_version.restype = C.c_uint32
    lib.dg_attn_visible_pairs.argtypes = [P(AttnDesc), P(C.c_uint64), P(C.c_double)]
    lib.dg_attn_visible_pairs.restype = C.c_int
    lib.dg_attention_dispatch.argtypes = [VP, VP, VP, P(LayerOffsets), P(StepParams), P(AttnDims), VP, VP,
                                          C.c_size_t, VP]
    lib.dg_attention_dispatch.restype = C.c_int
    lib.dg_attention_state_bytes.argtypes = [P(LayerOffsets), P(AttnDims), C.c_uint32, P(C.c_size_t)]
    lib.dg_attention_state_bytes.restype = C.c_int
    lib.dg_attention_dispatch_block.argtypes = [VP, VP, VP, P(LayerOffsets), P(StepParams), P(AttnDims),
                                                P(AttnBlockRange), VP, VP, C.c_size_t, VP]
    lib.dg_attention_dispatch_block.restype = C.c_int
    lib.dg_attention_block_state_bytes.argtypes = [P(LayerOffsets), P(AttnDims), C.c_uint32, P(C.c_size_t)]
    lib.dg_attention_block_state_bytes.restype = C.c_int
    lib.dg_attn_state_bytes.argtypes = [P(AttnDesc), P(C.c_size_t)]
    lib.dg_attn_state_bytes.restype = C.c_int
    lib.dg_attn_partial_workspace_bytes.argtypes = [P(AttnDesc), C.c_uint32, C.c_uint32, P(C.c_size_t)]
    lib.dg_attn_partial_workspace_bytes.restype = C.c_int
    lib.dg_attn_partial.argtypes = [P(AttnDesc), C.c_uint32, C.c_uint32, VP, VP, VP, C.c_size_t, VP, C.c_size_t, VP]
    lib.dg_attn_partial.restype = C.c_int
    lib.dg_attn_merge.argtypes = [P(AttnDesc), P(VP), C.c_uint32, VP, VP, VP, VP]
    lib.dg_attn_merge.restype = C.c_int
    lib.dg_kv_row_bytes.argtypes = [C.c_uint32, C.c_uint32]
    lib.dg_kv_row_bytes.restype = C.c_uint64
    lib.dg_kv_region_bytes.argtypes = [C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint32]
    lib.dg_kv_region_bytes.restype = C.c_uint64
    lib.dg_kv_slot.argtypes = [C.c_uint32, C.c_uint64]
    lib.dg_kv_slot.restype = C.c_uint64
    lib.dg_layer_kv_slots.argtypes = [C.c_int, C.c_uint64, C.c_uint64]
    lib.dg_layer_kv_slots.restype = C.c_uint64
    lib.dg_calib_copy.argtypes = [VP, VP, C.c_size_t, VP]
    lib.dg_calib_copy.restype = C.c_int
    lib.dg_calib_mfma.argtypes = [VP, C.c_size_t, C.c_uint32, C.c_uint32, C.c_uint32, P(C.c_uint64), VP]
    lib.dg_calib_mfma.restype = C.c_int
    lib.dg_qk_rope_kv.argtypes = [P(RopeDesc), VP, VP, VP, VP, VP, VP, VP, VP]
    lib.dg_qk_rope_kv.restype = C.c_int
    lib.dg_qk_rope_kv_dispatch.argtypes = [VP, VP, VP, VP, VP, P(LayerOffsets), P(StepParams), P(AttnDims), VP, VP]
    lib.dg_qk_rope_kv_dispatch.restype = C.c_int
    lib.dg_attn_topk_workspace_bytes.argtypes = [P(AttnDesc), P(C.c_uint32), P(C.c_size_t)]
    lib.dg_attn_topk_workspace_bytes.restype = C.c_int
    lib.dg_attn_topk_forward.argtypes = [P(AttnDesc), P(C.c_uint32), VP, VP, VP, VP, C.c_size_t, VP]
    lib.dg_attn_topk_forward.restype = C.c_int
    lib.dg_attention_topk_state_bytes.argtypes = [P(LayerOffsets), P(AttnDims), C.c_uint32, P(C.c_uint32),
                                                  P(C.c_size_t)]
    lib.dg_attention_topk_state_bytes.restype = C.c_int
    lib.dg_attention_topk_dispatch.argtypes = [VP, VP, VP, P(LayerOffsets), P(StepParams), P(AttnDims),
                                               P(C.c_uint32), VP, VP, C.c_size_t, VP]
    lib.dg_attention_topk_dispatch.restype = C.c_int
    lib.dg_prof_begin.argtypes = [C.c_uint32]
    lib.dg_prof_begin.restype = C.c_int
    lib.dg_prof_end.argtypes = [P(C.c_double), P(C.c_uint32)]
    lib.dg_prof_end.restype = C.c_int
    lib.dg_kv_layer_reference_layout.argtypes = [P(KvLayer)]
    lib.dg_kv_layer_reference_layout.restype = None
    lib.dg_kv_layer_head_major_layout.argtypes = [P(KvLayer)]
    lib.dg_kv_layer_head_major_layout.restype = None
    lib.dg_kv_snapshot_bytes.argtypes = [P(KvLayer), C.c_uint32, C.c_uint64, P(C.c_uint64), P(C.c_uint64)]
    lib.dg_kv_snapshot_bytes.restype = C.c_int
    lib.dg_kv_snapshot_gather.argtypes = [VP, P(KvLayer), C.c_uint32, C.c_uint64, VP, C.c_size_t, VP]
    lib.dg_kv_snapshot_gather.restype = C.c_int
    lib.dg_kv_snapshot_scatter.argtypes = [VP, P(KvLayer), C.c_uint32, C.c_uint64, VP, C.c_size_t, VP]
    lib.dg_kv_snapshot_scatter.restype = C.c_int
    lib.dg_kv_live_bytes.argtypes = [P(KvLayer), C.c_uint32, C.c_uint64, C.c_uint32, P(C.c_uint64)]
    lib.dg_kv_live_bytes.restype = C.c_int
    lib.dg_kv_live_gather.argtypes = [VP, P(KvLayer), C.c_uint32, C.c_uint64, C.c_uint32, VP, C.c_size_t, VP]
    lib.dg_kv_live_gather.restype = C.c_int
    lib.dg_fnv1a64.argtypes = [VP, C.c_size_t, C.c_uint64]
    lib.dg_fnv1a64.restype = C.c_uint64
    lib.dg_prof_end_split.argtypes = [P(C.c_double), P(C.c_double), P(C.c_uint32)]
    lib.dg_prof_end_split.restype = C.c_int
    _lib = lib
    return lib


def strerror(status: int) -> str:
    return load().dg_attn_strerror(status).decode()


def check(status: int) -> None:
    if status != DG_OK:
        raise DgAttnError(status, strerror(status))


def workspace_bytes(desc: AttnDesc) -> int:
    n = C.c_size_t(0)
    check(load().dg_attn_workspace_bytes(C.byref(desc), C.byref(n)))
    return n.value


def resolved_splits(desc: AttnDesc) -> int:
    n = C.c_uint32(0)
    check(load().dg_attn_resolved_splits(C.byref(desc), C.byref(n)))
    return n.value


def visible_pairs(desc: AttnDesc):
    n, f = C.c_uint64(0), C.c_double(0.0)
    check(load().dg_attn_visible_pairs(C.byref(desc), C.byref(n), C.byref(f)))
    return n.value, f.value


def prof_begin(max_launches: int) -> None:
    check(load().dg_prof_begin(max_launches))


def prof_end_split():
    """Returns (ms of even-numbered event pairs, ms of odd-numbered ones, pairs recorded)."""
    a, b, n = C.c_double(0.0), C.c_double(0.0), C.c_uint32(0)
    check(load().dg_prof_end_split(C.byref(a), C.byref(b), C.byref(n)))
    return a.value, b.value, n.value


def prof_end():
    """Returns (summed main-kernel ms, launches recorded)."""
    ms, n = C.c_double(0.0), C.c_uint32(0)
    check(load().dg_prof_end(C.byref(ms), C.byref(n)))
    return ms.value, n.value
