"""ctypes binding of libnanovllm_hip.so (the C ABI declared in include/nanovllm_hip.h).

The library is built in-tree by ``make -C nano-vllm_amd/csrc`` (or ``__graft_entry__.build()``)
into ``nano-vllm_amd/lib/``.  There is no fallback: if it cannot be loaded, ``lib()`` raises.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libnanovllm_hip.so")
MIXERS_LIB_PATH = os.path.join(_HERE, "lib", "libnanovllm_hip_mixers.so")
ABI_VERSION = 11

_vp, _i32, _i64, _f32 = C.c_void_p, C.c_int, C.c_int64, C.c_float


class Tuning(C.Structure):
    """Mirror of `nv_tuning` (include/nanovllm_hip.h): launch-plan overrides, heuristics by default."""
    _fields_ = [("decode_target_waves", _i32), ("decode_chunk", _i32), ("decode_work_item", _i32),
                ("decode_score_path", _i32), ("decode_mfma_depth", _i32), ("decode_single_launch", _i32),
                ("prefill_split", _i32), ("prefill_kernel", _i32)]
    DEFAULTS = dict(decode_target_waves=0, decode_chunk=0, decode_work_item=-1, decode_score_path=-1,
                    decode_mfma_depth=-1, decode_single_launch=-1, prefill_split=0, prefill_kernel=-1)


# name -> (restype, argtypes); must mirror include/nanovllm_hip.h exactly
PROTOTYPES = {
    "nv_strerror": (C.c_char_p, [_i32]),
    "nv_last_error": (C.c_char_p, []),
    "nv_abi_version": (_i32, []),
    "nv_set_tuning": (_i32, [C.POINTER(Tuning)]),
    "nv_get_tuning": (_i32, [C.POINTER(Tuning)]),
    "nv_store_kvcache": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i64, _i32, _i64, _i64, _vp]),
    "nv_attn_decode_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32, _i32]),
    "nv_attn_decode_paged": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                    _i32, _i64, _i32, _f32, _i64, _i64, _vp, _i64, _vp]),
    "nv_attn_decode_suggest_chunk": (_i32, [_i32, _i32, _i32, _i32, _i64]),
    "nv_attn_decode_workspace_bytes_chunked": (_i64, [_i32, _i32, _i32, _i32, _i32, _i32]),
    "nv_attn_decode_paged_chunked": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                            _i32, _i64, _i32, _f32, _i64, _i64, _vp, _i64, _i32, _i32, _vp]),
    "nv_attn_decode_paged_fused_chunked": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                                  _i32, _i32, _i32, _i32, _i32, _i32, _i64, _i32, _i64, _f32, _f32,
                                                  _i64, _i64, _i64, _i64, _vp, _i64, _i32, _i32, _vp]),
    "nv_attn_decode_static_scratch_bytes": (_i64, []),
    "nv_attn_decode_paged_static": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                           _i32, _i64, _i32, _f32, _i64, _i64, _vp]),
    "nv_attn_decode_paged_fused": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32,
                                          _i32, _i32, _i32, _i32, _i32, _i64, _i32, _i64, _f32, _f32, _i64, _i64,
                                          _i64, _i64, _vp, _i64, _vp]),
    "nv_attn_prefill_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32, _i32, _i32, _i32]),
    "nv_attn_prefill_varlen": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                      _i32, _i32, _i64, _i32, _f32, _i64, _i64, _i32, _i32, _vp, _i64, _vp]),
    "nv_rmsnorm": (_i32, [_vp, _vp, _vp, _i64, _i32, _i64, _f32, _vp]),
    "nv_silu_and_mul": (_i32, [_vp, _vp, _i64, _i32, _i64, _vp]),
    "nv_add_rmsnorm": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _f32, _vp]),
    "nv_rope": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i64, _i64, _i64, _vp]),
    "nv_qknorm_rope_store": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32,
                                    _i32, _i32, _i32, _i64, _f32, _i64, _i32, _i64, _i64, _i64, _vp]),
}

# second library (`make mixers`): fp32-stream norms, score-modified attention, recurrent mixers
MIXERS_PROTOTYPES = {
    "nv_strerror": (C.c_char_p, [_i32]),
    "nv_last_error": (C.c_char_p, []),
    "nv_abi_version": (_i32, []),
    "nv_add_layernorm": (_i32, [_vp, _vp, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _f32, _vp]),
    "nv_gelu_tanh_and_mul": (_i32, [_vp, _vp, _i32, _i64, _i32, _i64, _vp]),
    "nv_qk_prep_store": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _f32, _i32, _i32, _i64, _i32, _i32,
                                _i32, _i32, _i64, _i64, _i64, _vp]),
    "nv_attn_scoremod_paged": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i64, _i32, _i32, _i32, _i32,
                                      _i64, _i32, _f32, _f32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i64, _i64,
                                      _vp, _i64, _vp]),
    "nv_attn_scoremod_paged_vld": (_i32, [_vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _i64, _i32, _i32, _i32, _i32,
                                          _i64, _i32, _f32, _f32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i64, _i64,
                                          _vp, _i64, _vp]),
    "nv_attn_scoremod_workspace_bytes": (_i64, [_i32, _i64, _i32, _i32, _i32, _i32]),
    "nv_causal_conv_silu": (_i32, [_vp, _i64, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp]),
    "nv_gated_delta_rule": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp,
                                   _vp, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp]),
    "nv_stream_boundary": (_i32, [_vp, _vp, _i64, _vp, _i32, _vp, _i64, _vp, _f32, _vp, _i32, _f32, _vp, _vp, _vp, _i32,
                                  _i64, _i32, _vp]),
    "nv_rms_norm_rows": (_i32, [_vp, _i64, _vp, _vp, _i32, _i64, _i32, _f32, _vp]),
    "nv_causal_conv_add": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp]),
    "nv_token_gate": (_i32, [_vp, _i64, _vp, _i64, _vp, _i32, _i32, _vp, _i32, _i64, _vp]),
    "nv_general_delta_rule": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp,
                                     _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _f32, _f32, _i32, _vp]),
    "nv_latent_prep_store": (_i32, [_vp, _i64, _i32, _vp, _i64, _i64, _vp, _i64, _vp, _vp, _f32, _i32, _vp, _vp, _vp, _vp,
                                    _vp, _i32, _i64, _i32, _i32, _i32, _f32, _vp]),
    "nv_moe_route": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _vp]),
    "nv_moe_tile_rows": (_i32, [_i64, _i32]),
    "nv_moe_max_tiles": (_i64, [_i64, _i32, _i32]),
    "nv_moe_align": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _vp]),
    "nv_moe_gate_up": (_i32, [_vp, _i64, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _i32, _vp]),
    "nv_moe_down": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _vp]),
    "nv_moe_gate_up_act": (_i32, [_vp, _i64, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _f32, _i32,
                                  _vp]),
    "nv_causal_conv_bias_silu": (_i32, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32,
                                        _vp]),
    "nv_hashed_bigram_embed": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp, _vp, _i32, _i64, _i32,
                                      _i32, _vp]),
    "nv_stream_boundary_pair": (_i32, [_vp, _vp, _i64, _vp, _i64, _vp, _i32, _f32, _vp, _i64, _vp, _vp, _i64, _vp, _f32, _vp,
                                       _vp, _f32, _vp, _vp, _i32, _i64, _i32, _vp]),
    "nv_relu_squared": (_i32, [_vp, _i64, _vp, _i32, _i64, _i32, _vp]),
    "nv_decay_memory": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp,
                               _vp, _vp, _i32, _i32, _i32, _i32, _f32, _i32, _vp]),
    "nv_state_space_scan": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64,
                                   _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "nv_token_shift_mix": (_i32, [_vp, _i64, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp]),
    "nv_group_rms_norm": (_i32, [_vp, _i64, _vp, _vp, _i64, _i32, _i64, _i32, _i32, _f32, _vp]),
    "nv_chunk_attn_prep_store": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _f32, _vp, _i32, _vp, _vp, _vp, _vp,
                                        _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _vp]),
    "nv_attn_chunk_sigmoid_tile_ok": (_i32, [_i32, _i32, _i32]),
    "nv_attn_chunk_sigmoid_paged": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i64, _i32, _i32, _i32, _i32,
                                           _i64, _i32, _f32, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i64, _i64,
                                           _vp]),
    "nv_causal_conv_act": (_i32, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32,
                                  _vp]),
    "nv_stream_boundary_scaled": (_i32, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i32, _vp, _vp, _f32, _vp, _vp, _i32,
                                         _i64, _i32, _vp]),
    "nv_poly_norm": (_i32, [_vp, _i64, _vp, _f32, _vp, _i32, _i64, _i32, _vp]),
    "nv_head_norm_rope_store": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp, _f32, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _i32,
                                       _i64, _i32, _i32, _i32, _vp]),
    "nv_mlstm_memory": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp,
                               _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _f32, _f32, _f32, _i32, _vp]),
    "nv_gated_write_memory": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i32,
                                     _i32, _i32, _i32, _f32, _i32, _vp]),
    "nv_moe_route_grouped": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _vp]),
    "nv_moe_up_relu2": (_i32, [_vp, _i64, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
}
DTYPE_BF16, DTYPE_F32 = 0, 1

_lock = threading.Lock()
_lib = None
_mixers = None


class NanoVllmHipError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


def load(path: str | None = None, prototypes: dict | None = None) -> C.CDLL:
    """Load the shared library and attach prototypes.  Raises if it is missing or stale."""
    path = path or os.environ.get("NANOVLLM_HIP_LIB", LIB_PATH)
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} not found: the HIP extension is not built. Run "
            "`make -C nano-vllm_amd/csrc` (needs hipcc, targets gfx950). There is no CPU fallback."
        )
    dll = C.CDLL(path)
    for name, (restype, argtypes) in (prototypes if prototypes is not None else PROTOTYPES).items():
        fn = getattr(dll, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    got = dll.nv_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"{path}: ABI version {got}, bindings expect {ABI_VERSION}; rebuild the library")
    return dll


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                _lib = load()
    return _lib


def mixers() -> C.CDLL:
    """The second library (libnanovllm_hip_mixers.so)."""
    global _mixers
    if _mixers is None:
        with _lock:
            if _mixers is None:
                _mixers = load(os.environ.get("NANOVLLM_HIP_MIXERS_LIB", MIXERS_LIB_PATH), MIXERS_PROTOTYPES)
    return _mixers


def build(target: str = "all") -> None:
    """Compile the in-tree libraries (`all`), or only the second one (`mixers`), with hipcc for gfx950."""
    import subprocess
    jobs = str(min(16, os.cpu_count() or 4))
    subprocess.run(["make", "-C", os.path.join(_HERE, "csrc"), "-j", jobs, target], check=True,
                   stdout=subprocess.DEVNULL)


def check(rc: int, what: str, dll: C.CDLL | None = None) -> None:
    if rc != 0:
        dll = dll if dll is not None else lib()
        raise NanoVllmHipError(
            f"{what}: {dll.nv_strerror(rc).decode()} ({rc}): {dll.nv_last_error().decode()}"
        )


def set_tuning(**fields) -> None:
    """Override launch-plan heuristics process-wide (`nv_set_tuning`); no arguments restores them.
    Unknown field names raise.  A measurement / test aid: the product path never calls it."""
    if not fields:
        check(lib().nv_set_tuning(None), "nv_set_tuning")
        return
    unknown = set(fields) - set(Tuning.DEFAULTS)
    if unknown:
        raise ValueError(f"unknown tuning fields: {sorted(unknown)}")
    t = Tuning(**{**Tuning.DEFAULTS, **fields})
    check(lib().nv_set_tuning(C.byref(t)), "nv_set_tuning")


def get_tuning() -> dict:
    t = Tuning()
    check(lib().nv_get_tuning(C.byref(t)), "nv_get_tuning")
    return {name: getattr(t, name) for name, _ in Tuning._fields_}
