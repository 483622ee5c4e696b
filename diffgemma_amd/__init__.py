"""MI355X-native denoise-step attention for diffgemma (one hot path, behind a C ABI).

The product is ``libdg_attn_hip.so`` (``csrc/``, declared in ``include/dg_attn.h``).  This
package is the Python host side: a ctypes binding, the reference-shaped harness
(``attention``), and the KV-cache layout arithmetic (``step_kv``).  There is no CPU
fallback: every compute call goes to the HIP library and raises if it is missing.
"""
from . import capi, rounding, step_kv, attention  # noqa: F401

__all__ = ["capi", "rounding", "step_kv", "attention"]
