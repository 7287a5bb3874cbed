"""MI355X-native OmniKV dynamic-context-selection decode path.

HIP kernels (omnikv_amd/csrc, built into libomnikv_hip.so) behind the reference's
torch-level interface: select_tokens_by_attn_universal and OmniKVMultiStageCache.
"""
from . import _lib, ops  # noqa: F401

__all__ = ["_lib", "ops"]
