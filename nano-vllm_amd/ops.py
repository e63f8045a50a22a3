"""Tensor-level wrappers over the C ABI: argument checking, output allocation, stream lookup.

torch is used here only as the owner of device memory and streams; every function hands raw
``data_ptr()`` values to libnanovllm_hip.so on torch's current stream.  Inputs must live on a
GPU; nothing here computes on the host.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib

_BF16 = torch.bfloat16
_workspaces: dict[tuple[int, int], torch.Tensor] = {}
_retired: list[torch.Tensor] = []   # outgrown workspaces stay alive: captured graphs may point at them


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _gpu_bf16(t: torch.Tensor, name: str) -> None:
    _need(t.is_cuda, f"{name} must be a GPU tensor (this path has no CPU implementation)")
    _need(t.dtype == _BF16, f"{name} must be bfloat16, got {t.dtype}")


def _i32(t: torch.Tensor, name: str) -> None:
    _need(t.is_cuda and t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be a contiguous int32 GPU tensor")


def _rows_ok(t: torch.Tensor, name: str) -> None:
    """[T, H, D] with (H, D) contiguous; the token stride may be larger (slice of a fused tensor)."""
    _need(t.dim() == 3, f"{name} must be [tokens, heads, head_dim]")
    _need(t.stride(2) == 1 and t.stride(1) == t.shape[2], f"{name}: heads and head_dim must be contiguous")


_small_decode_ws: dict[tuple[int, int], torch.Tensor] = {}
_SMALL_DECODE_PAIRS = 8            # (sequence, kv head) pairs up to which a decode launch combines in-launch
_COUNTERS_ZERO = 1                 # NV_DECODE_WS_COUNTERS_ZERO


def _decode_workspace(device: torch.device, nbytes: int, pairs: int) -> tuple[torch.Tensor, int]:
    """Workspace and flags of a decode launch.  Launches with at most 8 (sequence, kv head) pairs get a buffer of
    their own per (device, stream) whose arrival counters start at zero and that nothing else ever writes (the
    shared buffer below also holds the prefill launches' states): the library can then combine the key ranges
    inside the launch instead of in a second kernel, and leaves the counters at zero again."""
    if pairs > _SMALL_DECODE_PAIRS or nbytes <= 16:
        return _workspace(device, nbytes), 0
    idx = device.index if device.index is not None else torch.cuda.current_device()
    key = (idx, torch.cuda.current_stream(device).cuda_stream)
    ws = _small_decode_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            # zeroing a fresh buffer here would put a 16 MiB memset into the graph: such a capture keeps the merge
            # launch (captures on a stream that has run the step before, as the engine's do, find their buffer)
            return _workspace(device, nbytes), 0
        if ws is not None:
            _retired.append(ws)
        ws = torch.zeros(max(nbytes, 16 << 20), dtype=torch.uint8, device=device)
        _small_decode_ws[key] = ws
    return ws, _COUNTERS_ZERO


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Split-key scratch of the attention launches: one buffer per (device, stream), so launches on different
    streams of one device never share partial states (launches on one stream are ordered)."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    key = (idx, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired.append(ws)
        # the first buffer of a device is sized for the usual launches; side streams get what they ask for
        floor = (64 << 20) if not any(k[0] == idx for k in _workspaces) else (1 << 20)
        ws = torch.empty(max(nbytes, floor), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def store_kvcache(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor) -> None:
    """cache[slot // bs, slot % bs] = row, for K and V (bit-exact)."""
    for t, n in ((k, "k"), (v, "v"), (k_cache, "k_cache"), (v_cache, "v_cache")):
        _gpu_bf16(t, n)
    _rows_ok(k, "k")
    _rows_ok(v, "v")
    _need(k_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous(),
          "caches must be contiguous [num_blocks, block_size, H_kv, D]")
    _need(k_cache.shape == v_cache.shape and k.shape == v.shape, "k/v shape mismatch")
    nb, bs, hkv, d = k_cache.shape
    _need(k.shape[1:] == (hkv, d), "k rows do not match the cache rows")
    _i32(slot_mapping, "slot_mapping")
    _need(slot_mapping.numel() == k.shape[0], "slot_mapping length != number of tokens")
    rc = _lib.lib().nv_store_kvcache(k.data_ptr(), v.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                     slot_mapping.data_ptr(), k.shape[0], hkv, d, nb, bs,
                                     k.stride(0), v.stride(0), _stream(k))
    _lib.check(rc, "nv_store_kvcache")


def _attn_common(q, k_cache, v_cache, cu_seqlens_k, block_tables):
    _gpu_bf16(q, "q")
    _gpu_bf16(k_cache, "k_cache")
    _gpu_bf16(v_cache, "v_cache")
    _rows_ok(q, "q")
    _need(k_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous()
          and k_cache.shape == v_cache.shape, "caches must be contiguous [num_blocks, block_size, H_kv, D]")
    _i32(cu_seqlens_k, "cu_seqlens_k")
    _need(block_tables.is_cuda and block_tables.dtype == torch.int32 and block_tables.dim() == 2
          and block_tables.is_contiguous(), "block_tables must be a contiguous [B, max_blocks] int32 GPU tensor")
    B = cu_seqlens_k.numel() - 1
    _need(block_tables.shape[0] == B, "block_tables rows != number of sequences")
    return B


def attn_decode_paged(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      cu_seqlens_k: torch.Tensor, block_tables: torch.Tensor, max_seqlen_k: int,
                      scale: float, cu_seqlens_q: Optional[torch.Tensor] = None,
                      out: Optional[torch.Tensor] = None, chunk_keys: int = 0) -> torch.Tensor:
    """Paged decode attention; sequences with seqlen_q != 1 are left untouched in ``out``.
    `chunk_keys` > 0: the host's choice of keys per work item (`decode_suggest_chunk`), 0 = the plan's."""
    B = _attn_common(q, k_cache, v_cache, cu_seqlens_k, block_tables)
    nb, bs, hkv, d = k_cache.shape
    hq = q.shape[1]
    if cu_seqlens_q is not None:
        _i32(cu_seqlens_q, "cu_seqlens_q")
        _need(cu_seqlens_q.numel() == B + 1, "cu_seqlens_q / cu_seqlens_k length mismatch")
    else:
        _need(q.shape[0] == B, "without cu_seqlens_q there must be one query token per sequence")
    if out is None:
        out = torch.empty((q.shape[0], hq, d), dtype=_BF16, device=q.device)
    else:
        _gpu_bf16(out, "out")
        _rows_ok(out, "out")
        _need(out.shape == q.shape, "out shape != q shape")
    dll = _lib.lib()
    need = dll.nv_attn_decode_workspace_bytes_chunked(B, hq, hkv, d, int(max_seqlen_k), int(chunk_keys))
    ws, flags = _decode_workspace(q.device, need, B * hkv)
    rc = dll.nv_attn_decode_paged_chunked(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
                                          cu_seqlens_q.data_ptr() if cu_seqlens_q is not None else None,
                                          cu_seqlens_k.data_ptr(), block_tables.data_ptr(), B,
                                          block_tables.shape[1], int(max_seqlen_k), hq, hkv, d, nb, bs,
                                          float(scale), q.stride(0), out.stride(0), ws.data_ptr(), ws.numel(),
                                          int(chunk_keys), flags, _stream(q))
    _lib.check(rc, "nv_attn_decode_paged_chunked")
    return out


def decode_suggest_chunk(num_seqs: int, hq: int, hkv: int, max_seqlen_k: int, sum_seqlen_k: int) -> int:
    """Keys per decode work item for a batch whose lengths the host knows (0 = the plan's own choice stands):
    a few long sequences among many short ones are cut into pieces of about a mean sequence, so that their
    waves do not end the launch long after the others."""
    return int(_lib.lib().nv_attn_decode_suggest_chunk(int(num_seqs), int(hq), int(hkv), int(max_seqlen_k),
                                                       int(sum_seqlen_k)))


def attn_prefill_varlen(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                        cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                        block_tables: torch.Tensor, max_seqlen_q: int, max_seqlen_k: int, scale: float,
                        skip_single_query: bool = False,
                        out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Varlen (chunked-)prefill attention, bottom-right causal, K/V read through the block table."""
    B = _attn_common(q, k_cache, v_cache, cu_seqlens_k, block_tables)
    nb, bs, hkv, d = k_cache.shape
    hq = q.shape[1]
    _i32(cu_seqlens_q, "cu_seqlens_q")
    _need(cu_seqlens_q.numel() == B + 1, "cu_seqlens_q / cu_seqlens_k length mismatch")
    if out is None:
        out = torch.empty((q.shape[0], hq, d), dtype=_BF16, device=q.device)
    else:
        _gpu_bf16(out, "out")
        _rows_ok(out, "out")
        _need(out.shape == q.shape, "out shape != q shape")
    dll = _lib.lib()
    need = dll.nv_attn_prefill_workspace_bytes(B, q.shape[0], int(max_seqlen_q), int(max_seqlen_k), hq, hkv, d)
    ws = _workspace(q.device, need)
    rc = dll.nv_attn_prefill_varlen(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                    out.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                                    block_tables.data_ptr(), B, block_tables.shape[1],
                                    int(max_seqlen_q), int(max_seqlen_k), hq, hkv, d, nb, bs,
                                    float(scale), q.stride(0), out.stride(0),
                                    1 if skip_single_query else 0, q.shape[0], ws.data_ptr(), ws.numel(),
                                    _stream(q))
    _lib.check(rc, "nv_attn_prefill_varlen")
    return out


def decode_fused_supported(hq: int, hkv: int, block_size: int) -> bool:
    """Shapes nv_attn_decode_paged_fused takes (others run qknorm_rope_store + attn_decode_paged)."""
    return hq % hkv == 0 and hq // hkv <= 8 and block_size % 16 == 0


def attn_decode_paged_fused(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                            q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                            cos_sin: torch.Tensor, eps: float, slot_mapping: torch.Tensor,
                            k_cache: torch.Tensor, v_cache: torch.Tensor, cu_seqlens_k: torch.Tensor,
                            block_tables: torch.Tensor, max_seqlen_k: int, scale: float,
                            out: Optional[torch.Tensor] = None, chunk_keys: int = 0) -> torch.Tensor:
    """A pure decode step's q/k-norm + rotary + KV scatter + paged attention in one launch (token b is
    sequence b's only new token).  Bit-identical to qknorm_rope_store followed by attn_decode_paged."""
    _rope_common(positions, q, k, cos_sin)
    B = _attn_common(q, k_cache, v_cache, cu_seqlens_k, block_tables)
    nb, bs, hkv, d = k_cache.shape
    hq = q.shape[1]
    _need(q.shape[0] == B, "one query token per sequence")
    _need(k.shape[1:] == (hkv, d), "k rows do not match the cache rows")
    _gpu_bf16(v, "v")
    _rows_ok(v, "v")
    _need(v.shape == k.shape, "k/v shape mismatch")
    _i32(slot_mapping, "slot_mapping")
    _need(slot_mapping.numel() == B, "slot_mapping length != number of sequences")
    _need((q_weight is None) == (k_weight is None), "q_weight and k_weight go together")
    if q_weight is not None:
        _gpu_bf16(q_weight, "q_weight")
        _gpu_bf16(k_weight, "k_weight")
        _need(q_weight.numel() == d and k_weight.numel() == d, "norm weights must be [head_dim]")
    if out is None:
        out = torch.empty((B, hq, d), dtype=_BF16, device=q.device)
    else:
        _gpu_bf16(out, "out")
        _rows_ok(out, "out")
        _need(out.shape == q.shape, "out shape != q shape")
    dll = _lib.lib()
    need = dll.nv_attn_decode_workspace_bytes_chunked(B, hq, hkv, d, int(max_seqlen_k), int(chunk_keys))
    ws, flags = _decode_workspace(q.device, need, B * hkv)
    rc = dll.nv_attn_decode_paged_fused_chunked(
        q.data_ptr(), k.data_ptr(), v.data_ptr(),
        q_weight.data_ptr() if q_weight is not None else None,
        k_weight.data_ptr() if k_weight is not None else None,
        cos_sin.data_ptr(), positions.data_ptr(), slot_mapping.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        out.data_ptr(), cu_seqlens_k.data_ptr(), block_tables.data_ptr(), B, block_tables.shape[1],
        int(max_seqlen_k), hq, hkv, d, nb, bs, cos_sin.shape[0], float(eps), float(scale),
        q.stride(0), k.stride(0), v.stride(0), out.stride(0), ws.data_ptr(), ws.numel(), int(chunk_keys), flags,
        _stream(q))
    _lib.check(rc, "nv_attn_decode_paged_fused_chunked")
    return out


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """y = bf16(silu(f32(gate)) * f32(up)) for x = [gate | up] along the last dimension."""
    _need(x.is_cuda, "x must be a GPU tensor (this path has no CPU implementation)")
    _need(x.dtype == _BF16, f"x must be bfloat16, got {x.dtype}")
    _need(x.dim() >= 1 and x.shape[-1] % 16 == 0, "last dimension must be a multiple of 16")
    inter = x.shape[-1] // 2
    x2 = x.reshape(-1, x.shape[-1])
    _need(x2.stride(1) == 1 and x2.stride(0) % 8 == 0, "rows must be contiguous with a stride that is a multiple of 8")
    y = torch.empty(x.shape[:-1] + (inter,), dtype=_BF16, device=x.device)
    rc = _lib.lib().nv_silu_and_mul(x2.data_ptr(), y.data_ptr(), x2.shape[0], inter, x2.stride(0), _stream(x))
    _lib.check(rc, "nv_silu_and_mul")
    return y


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = bf16(f32(x) * rsqrt(mean(x^2) + eps) * f32(w)) over the last dimension."""
    _gpu_bf16(x, "x")
    _gpu_bf16(weight, "weight")
    cols = x.shape[-1]
    _need(weight.numel() == cols and weight.is_contiguous(), "weight must be [hidden] contiguous")
    x2 = x.reshape(-1, cols)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    y = torch.empty(x.shape, dtype=_BF16, device=x.device)
    rc = _lib.lib().nv_rmsnorm(x2.data_ptr(), weight.data_ptr(), y.data_ptr(), x2.shape[0], cols,
                               x2.stride(0) if x2.shape[0] > 1 else cols, float(eps), _stream(x))
    _lib.check(rc, "nv_rmsnorm")
    return y


def add_rmsnorm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    """(y, new_residual): new_residual = bf16(x + residual); y = rmsnorm of the unrounded sum."""
    _gpu_bf16(x, "x")
    _gpu_bf16(residual, "residual")
    _gpu_bf16(weight, "weight")
    cols = x.shape[-1]
    _need(x.shape == residual.shape, "x and residual shapes differ")
    _need(weight.numel() == cols and weight.is_contiguous(), "weight must be [hidden] contiguous")
    x2 = x.contiguous().view(-1, cols)
    r2 = residual.contiguous().view(-1, cols)
    y = torch.empty(x.shape, dtype=_BF16, device=x.device)
    new_res = torch.empty(x.shape, dtype=_BF16, device=x.device)
    rc = _lib.lib().nv_add_rmsnorm(x2.data_ptr(), r2.data_ptr(), weight.data_ptr(), y.data_ptr(),
                                   new_res.data_ptr(), x2.shape[0], cols, float(eps), _stream(x))
    _lib.check(rc, "nv_add_rmsnorm")
    return y, new_res


def _rope_common(positions, q, k, cos_sin):
    _gpu_bf16(q, "query")
    _gpu_bf16(k, "key")
    _rows_ok(q, "query")
    _rows_ok(k, "key")
    _need(positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous()
          and positions.numel() == q.shape[0] == k.shape[0], "positions must be a contiguous int64 [tokens] GPU tensor")
    _need(cos_sin.is_cuda and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
          and cos_sin.shape[-1] == q.shape[2], "cos_sin_cache must be contiguous fp32 [max_pos, (1,) head_dim]")


def rope(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, cos_sin: torch.Tensor):
    """NeoX rotary embedding of q [T,H_q,D] and k [T,H_kv,D]; returns new tensors."""
    _rope_common(positions, q, k, cos_sin)
    T, hq, d = q.shape
    hkv = k.shape[1]
    q_out = torch.empty((T, hq, d), dtype=_BF16, device=q.device)
    k_out = torch.empty((T, hkv, d), dtype=_BF16, device=q.device)
    rc = _lib.lib().nv_rope(q.data_ptr(), k.data_ptr(), q_out.data_ptr(), k_out.data_ptr(),
                            cos_sin.data_ptr(), positions.data_ptr(), T, hq, hkv, d, cos_sin.shape[0],
                            q.stride(0), k.stride(0), _stream(q))
    _lib.check(rc, "nv_rope")
    return q_out, k_out


def qknorm_rope_store(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: Optional[torch.Tensor],
                      q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                      cos_sin: torch.Tensor, eps: float, slot_mapping: Optional[torch.Tensor] = None,
                      k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
                      want_k: bool = True):
    """Fused per-head RMSNorm (optional) + rotary + KV scatter (optional).  Returns (q_out, k_out)."""
    _rope_common(positions, q, k, cos_sin)
    T, hq, d = q.shape
    hkv = k.shape[1]
    store = slot_mapping is not None
    nb = bs = 0
    if store:
        _need(v is not None and k_cache is not None and v_cache is not None, "scatter needs v, k_cache, v_cache")
        _gpu_bf16(v, "v")
        _rows_ok(v, "v")
        _i32(slot_mapping, "slot_mapping")
        _need(k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape
              and k_cache.shape[2:] == (hkv, d), "caches must be contiguous [num_blocks, block_size, H_kv, D]")
        nb, bs = k_cache.shape[0], k_cache.shape[1]
    if q_weight is not None:
        _gpu_bf16(q_weight, "q_weight")
        _gpu_bf16(k_weight, "k_weight")
        _need(q_weight.numel() == d and k_weight.numel() == d, "norm weights must be [head_dim]")
    q_out = torch.empty((T, hq, d), dtype=_BF16, device=q.device)
    k_out = torch.empty((T, hkv, d), dtype=_BF16, device=q.device) if (want_k or not store) else None
    rc = _lib.lib().nv_qknorm_rope_store(
        q.data_ptr(), k.data_ptr(), v.data_ptr() if store else None,
        q_weight.data_ptr() if q_weight is not None else None,
        k_weight.data_ptr() if k_weight is not None else None,
        cos_sin.data_ptr(), positions.data_ptr(),
        slot_mapping.data_ptr() if store else None,
        k_cache.data_ptr() if store else None, v_cache.data_ptr() if store else None,
        q_out.data_ptr(), k_out.data_ptr() if k_out is not None else None,
        T, hq, hkv, d, cos_sin.shape[0], float(eps), nb, bs,
        q.stride(0), k.stride(0), v.stride(0) if store else 0, _stream(q))
    _lib.check(rc, "nv_qknorm_rope_store")
    return q_out, k_out


# ---------------------------------------------------------------------------------------------------------
# Second library: fp32 residual stream + LayerNorm, tanh-GELU gate, score-modified paged attention with free
# head sizes, short convolution and gated delta rule with per-sequence state slots.  Activations and caches
# are bfloat16 or float32 (all tensors of one call the same), small per-head / per-channel constants float32.
# ---------------------------------------------------------------------------------------------------------
def _dt(t: torch.Tensor, name: str) -> int:
    _need(t.is_cuda, f"{name} must be a GPU tensor (this path has no CPU implementation)")
    if t.dtype == _BF16:
        return _lib.DTYPE_BF16
    _need(t.dtype == torch.float32, f"{name} must be bfloat16 or float32, got {t.dtype}")
    return _lib.DTYPE_F32


def _f32c(t: Optional[torch.Tensor], name: str) -> int:
    if t is None:
        return 0
    _need(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous(), f"{name} must be a contiguous float32 GPU tensor")
    return t.data_ptr()


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _rows2d(t: torch.Tensor, name: str) -> torch.Tensor:
    _need(t.dim() == 2 and t.stride(1) == 1, f"{name} must be [rows, cols] with contiguous columns")
    return t


def add_layernorm(resid: torch.Tensor, h: Optional[torch.Tensor] = None, post: Optional[tuple] = None,
                  extra: Optional[torch.Tensor] = None, pre: Optional[tuple] = None,
                  out_dtype: Optional[torch.dtype] = None, eps: float = 1e-5) -> Optional[torch.Tensor]:
    """One sublayer boundary of an fp32 residual stream, in place on `resid` [T, W]:
    resid += LN(h; *post) + extra (each part optional); returns y = LN(resid; *pre) in `out_dtype`, or None
    without `pre`.  post / pre are (weight, bias) float32 [W]."""
    _need(resid.is_cuda and resid.dtype == torch.float32 and resid.dim() == 2 and resid.is_contiguous(),
          "resid must be a contiguous float32 [tokens, width] GPU tensor")
    rows, cols = resid.shape
    h_dt, h_stride = _lib.DTYPE_F32, cols
    if h is not None:
        _rows2d(h, "h")
        _need(h.shape == resid.shape and post is not None, "h must match resid and come with its (weight, bias)")
        h_dt, h_stride = _dt(h, "h"), h.stride(0)
    if extra is not None:
        _need(extra.shape == resid.shape, "extra must match resid")
    y, y_dt = None, _lib.DTYPE_F32
    if pre is not None:
        y = torch.empty((rows, cols), dtype=out_dtype or torch.float32, device=resid.device)
        y_dt = _dt(y, "y")
    for pair, n in ((post, "post"), (pre, "pre")):
        if pair is not None:
            _need(pair[0].numel() == cols and pair[1].numel() == cols, f"{n} weight / bias must be [width]")
    dll = _lib.mixers()
    rc = dll.nv_add_layernorm(resid.data_ptr(), _ptr(h), h_dt, h_stride,
                              _f32c(post[0], "post weight") if post and h is not None else None,
                              _f32c(post[1], "post bias") if post and h is not None else None,
                              _f32c(extra, "extra") or None,
                              _f32c(pre[0], "pre weight") if pre else None, _f32c(pre[1], "pre bias") if pre else None,
                              _ptr(y), y_dt, rows, cols, float(eps), _stream(resid))
    _lib.check(rc, "nv_add_layernorm", dll)
    return y


def gelu_tanh_and_mul(x: torch.Tensor) -> torch.Tensor:
    """y = gelu_tanh(gate) * up for x = [gate | up] along the last dimension (fp32 arithmetic, one rounding)."""
    _rows2d(x, "x")
    dt = _dt(x, "x")
    inter = x.shape[1] // 2
    y = torch.empty((x.shape[0], inter), dtype=x.dtype, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_gelu_tanh_and_mul(x.data_ptr(), y.data_ptr(), dt, x.shape[0], inter, x.stride(0), _stream(x))
    _lib.check(rc, "nv_gelu_tanh_and_mul", dll)
    return y


def qk_prep_store(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  slot_mapping: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                  v_cache: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor] = None, rot_dims: int = 0,
                  temp_coef: float = 0.0, temp_every: int = 0) -> torch.Tensor:
    """Interleaved-pair rotary on the first rot_dims dimensions of q and k, optional query temperature, scatter of
    k / v into the paged cache; returns the prepared q [T, H, D]."""
    dt = _dt(q, "q")
    for t, n in ((q, "q"), (k, "k"), (v, "v")):
        _rows_ok(t, n)
        _need(t.dtype == q.dtype, "q, k, v must have one dtype")
    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    _need(k.shape == (T, G, D) and v.shape[:2] == (T, G), "k / v rows do not match q")
    _need(positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T,
          "positions must be a contiguous int64 [tokens] GPU tensor")
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        _need(slot_mapping.numel() == T, "slot_mapping length != number of tokens")
        _need(k_cache is not None and v_cache is not None and k_cache.is_contiguous() and v_cache.is_contiguous()
              and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype and k_cache.shape[2:] == (G, D)
              and v_cache.shape[2:] == (G, Dv) and k_cache.shape[:2] == v_cache.shape[:2],
              "caches must be contiguous [num_blocks, block_size, G, D] and [.., G, Dv] of q's dtype")
    if rot_dims:
        _need(inv_freq is not None and inv_freq.numel() == rot_dims // 2, "inv_freq must hold rot_dims / 2 frequencies")
    q_out = torch.empty((T, H, D), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    rc = dll.nv_qk_prep_store(q.data_ptr(), k.data_ptr(), v.data_ptr(), q_out.data_ptr(), _ptr(k_cache), _ptr(v_cache),
                              positions.data_ptr(), _ptr(slot_mapping), _f32c(inv_freq, "inv_freq") or None,
                              int(rot_dims), float(temp_coef), int(temp_every), dt, T, H, G, D, Dv, q.stride(0),
                              k.stride(0), v.stride(0), _stream(q))
    _lib.check(rc, "nv_qk_prep_store", dll)
    return q_out


def attn_scoremod_paged(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cu_seqlens_q: torch.Tensor,
                        cu_seqlens_k: torch.Tensor, block_tables: torch.Tensor, scale: float, softcap: float = 0.0,
                        sink: Optional[torch.Tensor] = None, dist_bias: Optional[torch.Tensor] = None,
                        max_seqlen_q: int = 0, max_seqlen_k: int = 0, single_rows: int = -1) -> torch.Tensor:
    """Causal paged attention with soft-capped scores, a per-head distance bias [H, n_dist] (the last column serves
    every larger distance) and a per-head sink in the softmax denominator; returns [T, H * Dv]."""
    dt = _dt(q, "q")
    _rows_ok(q, "q")
    T, H, D = q.shape
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.is_contiguous()
          and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype and k_cache.shape[:3] == v_cache.shape[:3]
          and k_cache.shape[3] == D, "caches must be [num_blocks, block_size, G, D | Dv] of q's dtype, the keys contiguous")
    nb, bs, G, _ = k_cache.shape
    Dv = v_cache.shape[3]
    # value rows: dense, or any layout with ONE stride between consecutive (slot, kv head) rows, e.g. a column range of
    # the key cache
    v_ld = v_cache.stride(2)
    _need(v_cache.stride(3) == 1 and v_ld >= Dv and v_cache.stride(1) == G * v_ld and v_cache.stride(0) == bs * G * v_ld,
          "value rows must be evenly spaced (a dense cache or a column range of one)")
    _i32(cu_seqlens_q, "cu_seqlens_q")
    _i32(cu_seqlens_k, "cu_seqlens_k")
    B = cu_seqlens_k.numel() - 1
    _need(cu_seqlens_q.numel() == B + 1, "cu_seqlens_q / cu_seqlens_k length mismatch")
    _need(block_tables.is_cuda and block_tables.dtype == torch.int32 and block_tables.dim() == 2
          and block_tables.is_contiguous() and block_tables.shape[0] == B,
          "block_tables must be a contiguous [B, max_blocks] int32 GPU tensor")
    if sink is not None:
        _need(sink.numel() == H, "sink must be [H]")
    n_dist = 0
    if dist_bias is not None:
        _need(dist_bias.dim() == 2 and dist_bias.shape[0] == H, "dist_bias must be [H, n_dist]")
        n_dist = dist_bias.shape[1]
    out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    need = dll.nv_attn_scoremod_workspace_bytes(B, T, H, G, Dv, int(max_seqlen_k))
    ws = _workspace(q.device, need) if need else None
    rc = dll.nv_attn_scoremod_paged_vld(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), v_ld, out.data_ptr(),
                                    cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), block_tables.data_ptr(), B,
                                    block_tables.shape[1], T, H, G, D, Dv, nb, bs, float(scale), float(softcap or 0.0),
                                    _f32c(sink, "sink") or None, _f32c(dist_bias, "dist_bias") or None, n_dist,
                                    int(max_seqlen_q), int(max_seqlen_k), int(single_rows), dt, q.stride(0),
                                    out.stride(0), _ptr(ws), ws.numel() if ws is not None else 0, _stream(q))
    _lib.check(rc, "nv_attn_scoremod_paged", dll)
    return out


def causal_conv_silu(x: torch.Tensor, weight: torch.Tensor, conv_state: torch.Tensor, cu_seqlens_q: torch.Tensor,
                     cu_seqlens_k: torch.Tensor, state_slots: torch.Tensor) -> torch.Tensor:
    """silu(causal conv over time) per channel of x [T, C]; weight [C, taps] float32; conv_state
    [num_slots, taps - 1, C] (x's dtype) carries each sequence's last inputs and is updated."""
    dt = _dt(x, "x")
    _rows2d(x, "x")
    T, Cc = x.shape
    taps = weight.shape[1]
    _need(weight.shape[0] == Cc, "weight must be [channels, taps]")
    _need(conv_state.is_cuda and conv_state.dtype == x.dtype and conv_state.is_contiguous()
          and conv_state.shape[1:] == (taps - 1, Cc), "conv_state must be contiguous [slots, taps - 1, C] of x's dtype")
    for t, n in ((cu_seqlens_q, "cu_seqlens_q"), (cu_seqlens_k, "cu_seqlens_k"), (state_slots, "state_slots")):
        _i32(t, n)
    B = state_slots.numel()
    _need(cu_seqlens_q.numel() == B + 1 and cu_seqlens_k.numel() == B + 1, "one state slot per sequence")
    y = torch.empty((T, Cc), dtype=x.dtype, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_causal_conv_silu(x.data_ptr(), x.stride(0), _f32c(weight, "weight"), conv_state.data_ptr(),
                                 y.data_ptr(), y.stride(0), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                                 state_slots.data_ptr(), B, T, Cc, taps, dt, _stream(x))
    _lib.check(rc, "nv_causal_conv_silu", dll)
    return y


def gated_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a_raw: torch.Tensor, b_raw: torch.Tensor,
                     gate_raw: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor, norm_weight: torch.Tensor,
                     state: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                     state_slots: torch.Tensor, eps: float) -> torch.Tensor:
    """Gated delta rule with per-channel decay over a step's rows, state [slots, H, D, Dv] float32 updated in
    place; q, k: [T, G, D]; v: [T, H, Dv]; a_raw: [T, H * D]; b_raw: [T, H]; gate_raw: [T, H * Dv];
    returns the normalised, gated read-out [T, H * Dv]."""
    dt = _dt(q, "q")
    _rows_ok(q, "q")
    _rows_ok(k, "k")
    _rows_ok(v, "v")
    T, G, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    _need(k.shape == q.shape and v.shape[0] == T, "q / k / v rows differ")
    for t, n, cols in ((a_raw, "a_raw", H * D), (b_raw, "b_raw", H), (gate_raw, "gate_raw", H * Dv)):
        _rows2d(t, n)
        _need(t.shape == (T, cols) and t.dtype == q.dtype, f"{n} must be [T, {cols}] of q's dtype")
    _need(k.dtype == q.dtype and v.dtype == q.dtype, "q, k, v must have one dtype")
    _need(state.is_cuda and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, Dv),
          "state must be contiguous float32 [slots, H, D, Dv]")
    _need(A_log.numel() == H and dt_bias.numel() == H * D and norm_weight.numel() == Dv, "constant shapes")
    for t, n in ((cu_seqlens_q, "cu_seqlens_q"), (cu_seqlens_k, "cu_seqlens_k"), (state_slots, "state_slots")):
        _i32(t, n)
    B = state_slots.numel()
    _need(cu_seqlens_q.numel() == B + 1 and cu_seqlens_k.numel() == B + 1, "one state slot per sequence")
    out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    rc = dll.nv_gated_delta_rule(q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(0), k.stride(0), v.stride(0),
                                 a_raw.data_ptr(), a_raw.stride(0), b_raw.data_ptr(), b_raw.stride(0),
                                 gate_raw.data_ptr(), gate_raw.stride(0), _f32c(A_log, "A_log"),
                                 _f32c(dt_bias, "dt_bias"), _f32c(norm_weight, "norm_weight"), state.data_ptr(),
                                 out.data_ptr(), out.stride(0), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                                 state_slots.data_ptr(), B, H, G, D, Dv, float(eps), dt, _stream(q))
    _lib.check(rc, "nv_gated_delta_rule", dll)
    return out


# ---------------------------------------------------------------------------------------------------------
# fp32 stream with a grouped RMS norm, input convolution, token gate, generalized delta rule, latent attention
# and routed experts (second library).
# ---------------------------------------------------------------------------------------------------------
def stream_boundary(x: torch.Tensor, add: Optional[torch.Tensor] = None, add_parts: Optional[torch.Tensor] = None,
                    normed: Optional[torch.Tensor] = None, normed_weight: Optional[torch.Tensor] = None,
                    mult: float = 1.0, norm: Optional[torch.Tensor] = None, groups: int = 1, eps: float = 1e-5,
                    out_dtype: Optional[torch.dtype] = None, want_f32: bool = False,
                    copy_dtype: Optional[torch.dtype] = None):
    """One boundary of an fp32 residual stream, in place on x [T, W]:
    x += mult * (add + add_parts.sum(1));  x += mult * rmsnorm(normed) * normed_weight  (each part optional).
    With `norm` (the weight of a grouped RMS norm) returns (h32 or None, h): the norm of x in float32 (if want_f32)
    and in out_dtype; else with `copy_dtype` returns x in that dtype; else None."""
    _need(x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(),
          "the stream must be a contiguous float32 [tokens, width] GPU tensor")
    rows, cols = x.shape
    dt_t = out_dtype or copy_dtype or (add.dtype if add is not None else normed.dtype if normed is not None else torch.float32)
    dt = _lib.DTYPE_BF16 if dt_t == _BF16 else _lib.DTYPE_F32
    _need(dt_t in (_BF16, torch.float32), "the matmul dtype must be bfloat16 or float32")
    for t, n in ((add, "add"), (normed, "normed")):
        if t is not None:
            _rows2d(t, n)
            _need(t.shape == x.shape and t.dtype == dt_t and t.is_cuda, f"{n} must match the stream's shape, in the matmul dtype")
    n_parts = 0
    if add_parts is not None:
        _need(add_parts.is_cuda and add_parts.dtype == torch.float32 and add_parts.is_contiguous() and add_parts.dim() == 3
              and add_parts.shape[0] == rows and add_parts.shape[2] == cols, "add_parts must be contiguous float32 [T, n, W]")
        n_parts = add_parts.shape[1]
    if normed is not None:
        _need(normed_weight is not None and normed_weight.numel() == cols, "normed needs its [width] weight")
    y32 = y = copy = None
    if norm is not None:
        _need(norm.numel() == cols, "norm weight must be [width]")
        y = torch.empty((rows, cols), dtype=dt_t, device=x.device)
        if want_f32:
            y32 = y if dt_t == torch.float32 else torch.empty((rows, cols), dtype=torch.float32, device=x.device)
    elif copy_dtype is not None:
        copy = torch.empty((rows, cols), dtype=dt_t, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_stream_boundary(x.data_ptr(), _ptr(add), add.stride(0) if add is not None else 0,
                                _ptr(add_parts) if n_parts else None, n_parts, _ptr(normed),
                                normed.stride(0) if normed is not None else 0,
                                _f32c(normed_weight, "normed_weight") if normed is not None else None, float(mult),
                                _f32c(norm, "norm") or None, int(groups), float(eps),
                                _ptr(y32) if (y32 is not None and y32 is not y) else None, _ptr(y), _ptr(copy), dt, rows,
                                cols, _stream(x))
    _lib.check(rc, "nv_stream_boundary", dll)
    if norm is not None:
        return y32, y
    return copy


def rms_norm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight per row (fp32 arithmetic), x [T, C] bfloat16 or float32."""
    dt = _dt(x, "x")
    _rows2d(x, "x")
    _need(weight.numel() == x.shape[1], "weight must be [cols]")
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_rms_norm_rows(x.data_ptr(), x.stride(0), _f32c(weight, "weight"), y.data_ptr(), dt, x.shape[0],
                              x.shape[1], float(eps), _stream(x))
    _lib.check(rc, "nv_rms_norm_rows", dll)
    return y


def causal_conv_add(x: torch.Tensor, weight: torch.Tensor, conv_state: torch.Tensor, out_dtype: torch.dtype,
                    cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor, state_slots: torch.Tensor) -> torch.Tensor:
    """x + causal convolution over time per channel, x [T, C] float32; weight [C, taps] float32; conv_state
    [num_slots, taps - 1, C] float32 carries each sequence's last inputs and is updated; result in out_dtype."""
    _need(x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "x must be contiguous float32 [T, C]")
    T, Cc = x.shape
    taps = weight.shape[1]
    _need(weight.shape[0] == Cc, "weight must be [channels, taps]")
    _need(conv_state.is_cuda and conv_state.dtype == torch.float32 and conv_state.is_contiguous()
          and conv_state.shape[1:] == (taps - 1, Cc), "conv_state must be contiguous float32 [slots, taps - 1, C]")
    for t, n in ((cu_seqlens_q, "cu_seqlens_q"), (cu_seqlens_k, "cu_seqlens_k"), (state_slots, "state_slots")):
        _i32(t, n)
    B = state_slots.numel()
    _need(cu_seqlens_q.numel() == B + 1 and cu_seqlens_k.numel() == B + 1, "one state slot per sequence")
    y = torch.empty((T, Cc), dtype=out_dtype, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_causal_conv_add(x.data_ptr(), _f32c(weight, "weight"), conv_state.data_ptr() if taps > 1 else None,
                                y.data_ptr(), _dt(y, "y"), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                                state_slots.data_ptr(), B, T, Cc, taps, _stream(x))
    _lib.check(rc, "nv_causal_conv_add", dll)
    return y


def token_gate(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, offset: int, dim: int) -> torch.Tensor:
    """gelu_tanh(z) * table[ids, offset : offset + dim]; z [T, dim] and table [V, n] of one dtype."""
    dt = _dt(z, "z")
    _rows2d(z, "z")
    _rows2d(table, "table")
    _need(table.dtype == z.dtype and table.is_cuda and z.shape[1] == dim and 0 <= offset and offset + dim <= table.shape[1],
          "table must be of z's dtype and hold the columns offset .. offset + dim")
    _need(ids.is_cuda and ids.dtype == torch.int64 and ids.is_contiguous() and ids.numel() == z.shape[0],
          "ids must be a contiguous int64 [tokens] GPU tensor")
    y = torch.empty((z.shape[0], dim), dtype=z.dtype, device=z.device)
    dll = _lib.mixers()
    rc = dll.nv_token_gate(z.data_ptr(), z.stride(0), table.data_ptr(), table.stride(0), ids.data_ptr(), int(offset),
                           int(dim), y.data_ptr(), dt, z.shape[0], _stream(z))
    _lib.check(rc, "nv_token_gate", dll)
    return y


def general_delta_rule(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, w_raw: torch.Tensor, a_raw: torch.Tensor,
                       gate_raw: torch.Tensor, w_bias: torch.Tensor, a_bias: torch.Tensor, norm_weight: torch.Tensor,
                       state: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                       state_slots: torch.Tensor, eps: float, decay_rate: float, key_eps: float) -> torch.Tensor:
    """Generalized delta rule over a step's rows, state [slots, H, D, D] float32 updated in place; r, k, v: [T, H, D];
    w_raw, a_raw, gate_raw: [T, H * D]; returns the normalised, gated read-out [T, H * D]."""
    dt = _dt(r, "r")
    T, H, D = r.shape
    for t, n in ((r, "r"), (k, "k"), (v, "v")):
        _rows_ok(t, n)
        _need(t.shape == (T, H, D) and t.dtype == r.dtype, "r, k, v must be [T, H, D] of one dtype")
    for t, n in ((w_raw, "w_raw"), (a_raw, "a_raw"), (gate_raw, "gate_raw")):
        _rows2d(t, n)
        _need(t.shape == (T, H * D) and t.dtype == r.dtype, f"{n} must be [T, H * D] of r's dtype")
    _need(state.is_cuda and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, D),
          "state must be contiguous float32 [slots, H, D, D]")
    _need(w_bias.numel() == H * D and a_bias.numel() == H * D and norm_weight.numel() == H * D, "constant shapes")
    for t, n in ((cu_seqlens_q, "cu_seqlens_q"), (cu_seqlens_k, "cu_seqlens_k"), (state_slots, "state_slots")):
        _i32(t, n)
    B = state_slots.numel()
    _need(cu_seqlens_q.numel() == B + 1 and cu_seqlens_k.numel() == B + 1, "one state slot per sequence")
    out = torch.empty((T, H * D), dtype=r.dtype, device=r.device)
    dll = _lib.mixers()
    rc = dll.nv_general_delta_rule(r.data_ptr(), k.data_ptr(), v.data_ptr(), r.stride(0), k.stride(0), v.stride(0),
                                   w_raw.data_ptr(), w_raw.stride(0), a_raw.data_ptr(), a_raw.stride(0),
                                   gate_raw.data_ptr(), gate_raw.stride(0), _f32c(w_bias, "w_bias"),
                                   _f32c(a_bias, "a_bias"), _f32c(norm_weight, "norm_weight"), state.data_ptr(),
                                   out.data_ptr(), out.stride(0), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                                   state_slots.data_ptr(), B, H, D, float(eps), float(decay_rate), float(key_eps), dt,
                                   _stream(r))
    _lib.check(rc, "nv_general_delta_rule", dll)
    return out


def latent_prep_store(q: torch.Tensor, q_lat: torch.Tensor, ckv: torch.Tensor, latent_weight: torch.Tensor,
                      freq: Optional[torch.Tensor], mag: float, interleaved: bool, positions: torch.Tensor,
                      slot_mapping: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                      v_cache: Optional[torch.Tensor], rot_dim: int, eps: float) -> torch.Tensor:
    """Normalises the latent, rotates the shared key part and the queries' rotated part, scatters [c | k_r] and c into
    the paged caches and returns the latent-space queries [T, H, rank + R].  q: [T, H, Dq] whose last R columns are
    rotated; q_lat: [T, H, rank] (any token / head strides); ckv: [T, rank + R]."""
    dt = _dt(q, "q")
    _rows_ok(q, "q")
    T, H, Dq = q.shape
    R, rank = int(rot_dim), q_lat.shape[2]
    _need(q_lat.shape[:2] == (T, H) and q_lat.stride(2) == 1 and q_lat.dtype == q.dtype and q_lat.is_cuda,
          "q_lat must be [T, H, rank] of q's dtype with contiguous columns")
    _rows2d(ckv, "ckv")
    _need(ckv.shape == (T, rank + R) and ckv.dtype == q.dtype, "ckv must be [T, rank + R] of q's dtype")
    _need(latent_weight.numel() == rank, "latent weight must be [rank]")
    _need(positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T,
          "positions must be a contiguous int64 [tokens] GPU tensor")
    if R:
        _need(freq is not None and freq.numel() == R // 2, "freq must hold R / 2 frequencies")
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        _need(slot_mapping.numel() == T, "slot_mapping length != number of tokens")
        _need(k_cache is not None and k_cache.is_contiguous() and k_cache.dtype == q.dtype
              and k_cache.shape[2:] == (1, rank + R), "k_cache must be contiguous [num_blocks, block_size, 1, rank + R] of q's dtype")
        if v_cache is not None and v_cache.data_ptr() == k_cache.data_ptr():
            _need(v_cache.shape == k_cache.shape[:3] + (rank,) and v_cache.stride() == k_cache.stride(),
                  "a value cache inside the key cache must be its first `rank` columns")
            v_cache = None                    # the values are the front of the key rows: nothing else to store
        else:
            _need(v_cache is not None and v_cache.is_contiguous() and v_cache.dtype == q.dtype
                  and v_cache.shape == k_cache.shape[:3] + (rank,), "v_cache must be contiguous [.., 1, rank] of q's dtype")
    q_full = torch.empty((T, H, rank + R), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    rc = dll.nv_latent_prep_store(q.data_ptr(), q.stride(0), Dq, q_lat.data_ptr(), q_lat.stride(0), q_lat.stride(1),
                                  ckv.data_ptr(), ckv.stride(0), _f32c(latent_weight, "latent_weight"),
                                  _f32c(freq, "freq") or None, float(mag), int(bool(interleaved)), positions.data_ptr(),
                                  _ptr(slot_mapping), q_full.data_ptr(), _ptr(k_cache),
                                  _ptr(v_cache) if slot_mapping is not None else None, dt, T, H, rank, R,
                                  float(eps), _stream(q))
    _lib.check(rc, "nv_latent_prep_store", dll)
    return q_full


def moe_experts(h: torch.Tensor, logits: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, top: int,
                limit: float, alpha: float) -> torch.Tensor:
    """Routed clamped-GLU experts: h [T, W]; logits [T, E] float32; gate_up [E, 2 ff, W]; down [E, W, ff].  Returns the
    weighted outputs of every token's `top` experts, [T, top, W] float32 (the stream update sums them)."""
    dt = _dt(h, "h")
    _rows2d(h, "h")
    T, W = h.shape
    E, ff = gate_up.shape[0], gate_up.shape[1] // 2
    _need(logits.is_cuda and logits.dtype == torch.float32 and logits.is_contiguous() and logits.shape == (T, E),
          "logits must be contiguous float32 [T, E]")
    _need(gate_up.is_cuda and down.is_cuda and gate_up.is_contiguous() and down.is_contiguous() and gate_up.dtype == h.dtype
          and down.dtype == h.dtype and gate_up.shape == (E, 2 * ff, W) and down.shape == (E, W, ff),
          "gate_up must be [E, 2 ff, W] and down [E, W, ff], contiguous, of h's dtype")
    dll = _lib.mixers()
    dev, P, s = h.device, T * top, _stream(h)
    ids = torch.empty((T, top), dtype=torch.int32, device=dev)
    wgt = torch.empty((T, top), dtype=torch.float32, device=dev)
    out = torch.empty((T, top, W), dtype=torch.float32, device=dev)
    if T == 0:
        return out
    _lib.check(dll.nv_moe_route(logits.data_ptr(), ids.data_ptr(), wgt.data_ptr(), T, E, int(top), s), "nv_moe_route", dll)
    rows = dll.nv_moe_tile_rows(P, E)
    tiles = dll.nv_moe_max_tiles(P, E, rows)
    sorted_pairs = torch.empty(P, dtype=torch.int32, device=dev)
    meta = torch.empty(1 + 3 * tiles, dtype=torch.int32, device=dev)
    _lib.check(dll.nv_moe_align(ids.data_ptr(), sorted_pairs.data_ptr(), meta.data_ptr(), P, E, rows, s), "nv_moe_align", dll)
    y = torch.empty((P, ff), dtype=h.dtype, device=dev)
    _lib.check(dll.nv_moe_gate_up(h.data_ptr(), h.stride(0), gate_up.data_ptr(), sorted_pairs.data_ptr(), meta.data_ptr(),
                                  y.data_ptr(), dt, P, E, int(top), W, ff, float(limit), float(alpha), rows, s),
               "nv_moe_gate_up", dll)
    _lib.check(dll.nv_moe_down(y.data_ptr(), down.data_ptr(), sorted_pairs.data_ptr(), meta.data_ptr(), wgt.data_ptr(),
                               out.data_ptr(), dt, P, E, W, ff, rows, s), "nv_moe_down", dll)
    return out


# ---------------------------------------------------------------------------------------------------------
# fp32 stream read through two RMS norms, hashed bigram embedding, decayed outer-product memories (bonus form and
# state-space scan), token-shift blends, chunked sigmoid attention with rotated values, table-routed experts.
# ---------------------------------------------------------------------------------------------------------
def _seq_meta(cu_seqlens_q, cu_seqlens_k, state_slots):
    for t, n in ((cu_seqlens_q, "cu_seqlens_q"), (cu_seqlens_k, "cu_seqlens_k"), (state_slots, "state_slots")):
        _i32(t, n)
    B = state_slots.numel()
    _need(cu_seqlens_q.numel() == B + 1 and cu_seqlens_k.numel() == B + 1, "one state slot per sequence")
    return B


def hashed_bigram_embed(ids: torch.Tensor, positions: torch.Tensor, embed: torch.Tensor, bigram: Optional[torch.Tensor],
                        mul_prev: int, mul_cur: int, norm_weight: Optional[torch.Tensor], eps: float,
                        prev_state: Optional[torch.Tensor], cu_seqlens_q: torch.Tensor,
                        state_slots: Optional[torch.Tensor]) -> torch.Tensor:
    """x = rmsnorm(embed[id] + bigram[hash(previous id, id)]) * norm_weight as a float32 stream [T, W] (norm_weight None:
    the sum as it is); the last row of the bigram table serves position 0; prev_state [slots] int64 carries each
    sequence's last id."""
    dt = _dt(embed, "embed")
    T, W = ids.numel(), embed.shape[1]
    for t, n in ((ids, "ids"), (positions, "positions")):
        _need(t.is_cuda and t.dtype == torch.int64 and t.is_contiguous() and t.numel() == T,
              f"{n} must be a contiguous int64 [tokens] GPU tensor")
    _need(embed.is_contiguous() and embed.dim() == 2, "embed must be contiguous [vocab, width]")
    _i32(cu_seqlens_q, "cu_seqlens_q")
    B = cu_seqlens_q.numel() - 1
    buckets = 0
    if bigram is not None:
        _need(bigram.is_cuda and bigram.is_contiguous() and bigram.dtype == embed.dtype and bigram.shape[1] == W
              and bigram.shape[0] >= 2, "bigram must be contiguous [buckets + 1, width] of embed's dtype")
        buckets = bigram.shape[0] - 1
        _need(prev_state is not None and prev_state.is_cuda and prev_state.dtype == torch.int64 and prev_state.is_contiguous(),
              "prev_state must be a contiguous int64 [slots] GPU tensor")
        _i32(state_slots, "state_slots")
        _need(state_slots.numel() == B, "one state slot per sequence")
    x = torch.empty((T, W), dtype=torch.float32, device=embed.device)
    dll = _lib.mixers()
    rc = dll.nv_hashed_bigram_embed(ids.data_ptr(), positions.data_ptr(), embed.data_ptr(), _ptr(bigram), buckets,
                                    int(mul_prev), int(mul_cur), _f32c(norm_weight, "norm_weight") or None, float(eps),
                                    _ptr(prev_state) if bigram is not None else None, x.data_ptr(),
                                    cu_seqlens_q.data_ptr(), _ptr(state_slots) if bigram is not None else None, B, T, W,
                                    dt, _stream(embed))
    _lib.check(rc, "nv_hashed_bigram_embed", dll)
    return x


def stream_boundary_pair(x: torch.Tensor, adds=(), parts: Optional[torch.Tensor] = None, parts_scale: float = 1.0,
                         normed=(), normed_mult: float = 1.0, norms=(), eps: float = 1e-5,
                         out_dtype: Optional[torch.dtype] = None, want_f32: bool = True):
    """One layer boundary of an fp32 stream x [T, W], in place:
    x += sum(adds) + parts_scale * parts.sum(1) + normed_mult * sum(rmsnorm(n) * w for (n, w) in normed).
    norms: up to two RMS-norm weights of the updated stream.  Returns (h32, h): the norms side by side in float32
    [T, len(norms) * W] (if want_f32) and the FIRST norm in out_dtype (if given); None for each part not asked for."""
    _need(x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(),
          "the stream must be a contiguous float32 [tokens, width] GPU tensor")
    rows, cols = x.shape
    adds, normed, norms = list(adds), list(normed), list(norms)
    _need(len(adds) <= 2 and len(normed) <= 2 and len(norms) <= 2, "at most two of each kind")
    ins = adds + [n for n, _ in normed]
    dt_t = out_dtype or (ins[0].dtype if ins else torch.float32)
    _need(dt_t in (_BF16, torch.float32), "the matmul dtype must be bfloat16 or float32")
    dt = _lib.DTYPE_BF16 if dt_t == _BF16 else _lib.DTYPE_F32
    for t in ins:
        _rows2d(t, "input")
        _need(t.shape == x.shape and t.dtype == dt_t and t.is_cuda, "inputs must match the stream's shape, in the matmul dtype")
    n_parts = 0
    if parts is not None:
        _need(parts.is_cuda and parts.dtype == torch.float32 and parts.is_contiguous() and parts.dim() == 3
              and parts.shape[0] == rows and parts.shape[2] == cols, "parts must be contiguous float32 [T, n, W]")
        n_parts = parts.shape[1]
    for _, w in normed:
        _need(w.numel() == cols, "a normed input needs its [width] weight")
    for w in norms:
        _need(w.numel() == cols, "norm weights must be [width]")
    y32 = y = None
    if norms:
        if want_f32:
            y32 = torch.empty((rows, len(norms) * cols), dtype=torch.float32, device=x.device)
        if out_dtype is not None:
            y = torch.empty((rows, cols), dtype=out_dtype, device=x.device)
        _need(y32 is not None or y is not None, "the norm needs an output")
    a1 = adds[0] if len(adds) > 0 else None
    a2 = adds[1] if len(adds) > 1 else None
    n1, w1 = normed[0] if len(normed) > 0 else (None, None)
    n2, w2 = normed[1] if len(normed) > 1 else (None, None)
    dll = _lib.mixers()
    rc = dll.nv_stream_boundary_pair(x.data_ptr(), _ptr(a1), a1.stride(0) if a1 is not None else 0, _ptr(a2),
                                     a2.stride(0) if a2 is not None else 0, _ptr(parts) if n_parts else None, n_parts,
                                     float(parts_scale), _ptr(n1), n1.stride(0) if n1 is not None else 0,
                                     _f32c(w1, "normed weight") or None, _ptr(n2), n2.stride(0) if n2 is not None else 0,
                                     _f32c(w2, "normed weight") or None, float(normed_mult),
                                     _f32c(norms[0], "norm") if norms else None,
                                     _f32c(norms[1], "norm") if len(norms) > 1 else None, float(eps), _ptr(y32), _ptr(y),
                                     dt, rows, cols, _stream(x))
    _lib.check(rc, "nv_stream_boundary_pair", dll)
    return y32, y


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    """max(x, 0)^2, x [T, C] bfloat16 or float32 (fp32 arithmetic, one rounding)."""
    dt = _dt(x, "x")
    _rows2d(x, "x")
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    dll = _lib.mixers()
    _lib.check(dll.nv_relu_squared(x.data_ptr(), x.stride(0), y.data_ptr(), dt, x.shape[0], x.shape[1], _stream(x)),
               "nv_relu_squared", dll)
    return y


def causal_conv_bias_silu(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], conv_state: torch.Tensor,
                          cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor, state_slots: torch.Tensor) -> torch.Tensor:
    """silu(causal conv over time + bias) per channel of x [T, C]; weight [C, taps] and bias [C] float32; conv_state
    [num_slots, taps - 1, C] (x's dtype) carries each sequence's last inputs and is updated."""
    dt = _dt(x, "x")
    _rows2d(x, "x")
    T, Cc = x.shape
    taps = weight.shape[1]
    _need(weight.shape[0] == Cc and (bias is None or bias.numel() == Cc), "weight must be [channels, taps], bias [channels]")
    _need(conv_state.is_cuda and conv_state.dtype == x.dtype and conv_state.is_contiguous()
          and conv_state.shape[1:] == (taps - 1, Cc), "conv_state must be contiguous [slots, taps - 1, C] of x's dtype")
    B = _seq_meta(cu_seqlens_q, cu_seqlens_k, state_slots)
    y = torch.empty((T, Cc), dtype=x.dtype, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_causal_conv_bias_silu(x.data_ptr(), x.stride(0), _f32c(weight, "weight"), _f32c(bias, "bias") or None,
                                      conv_state.data_ptr(), y.data_ptr(), y.stride(0), cu_seqlens_q.data_ptr(),
                                      cu_seqlens_k.data_ptr(), state_slots.data_ptr(), B, T, Cc, taps, dt, _stream(x))
    _lib.check(rc, "nv_causal_conv_bias_silu", dll)
    return y


def decay_memory(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, w_raw: torch.Tensor, gate_raw: torch.Tensor,
                 w_bias: torch.Tensor, bonus: torch.Tensor, norm_weight: torch.Tensor, state: torch.Tensor,
                 cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor, state_slots: torch.Tensor, eps: float) -> torch.Tensor:
    """Decayed outer-product memory read before it is written, with a bonus for the current token; state
    [slots, H, Dk, Dv] float32 updated in place; r, k: [T, H, Dk]; v: [T, H, Dv]; w_raw [T, H * Dk]; gate_raw [T, H * Dv];
    returns the per-head normalised, gated read-out [T, H * Dv]."""
    dt = _dt(r, "r")
    T, H, Dk = r.shape
    Dv = v.shape[2]
    for t, n in ((r, "r"), (k, "k"), (v, "v")):
        _rows_ok(t, n)
        _need(t.dtype == r.dtype, "r, k, v must have one dtype")
    _need(k.shape == (T, H, Dk) and v.shape[:2] == (T, H), "r / k / v rows differ")
    for t, n, cols in ((w_raw, "w_raw", H * Dk), (gate_raw, "gate_raw", H * Dv)):
        _rows2d(t, n)
        _need(t.shape == (T, cols) and t.dtype == r.dtype, f"{n} must be [T, {cols}] of r's dtype")
    _need(state.is_cuda and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, Dk, Dv),
          "state must be contiguous float32 [slots, H, Dk, Dv]")
    _need(w_bias.numel() == H * Dk and bonus.numel() == H * Dk and norm_weight.numel() == H * Dv, "constant shapes")
    B = _seq_meta(cu_seqlens_q, cu_seqlens_k, state_slots)
    out = torch.empty((T, H * Dv), dtype=r.dtype, device=r.device)
    dll = _lib.mixers()
    rc = dll.nv_decay_memory(r.data_ptr(), k.data_ptr(), v.data_ptr(), r.stride(0), k.stride(0), v.stride(0),
                             w_raw.data_ptr(), w_raw.stride(0), gate_raw.data_ptr(), gate_raw.stride(0),
                             _f32c(w_bias, "w_bias"), _f32c(bonus, "bonus"), _f32c(norm_weight, "norm_weight"),
                             state.data_ptr(), out.data_ptr(), out.stride(0), cu_seqlens_q.data_ptr(),
                             cu_seqlens_k.data_ptr(), state_slots.data_ptr(), B, H, Dk, Dv, float(eps), dt, _stream(r))
    _lib.check(rc, "nv_decay_memory", dll)
    return out


def state_space_scan(x: torch.Tensor, Bm: torch.Tensor, Cm: torch.Tensor, dt_raw: torch.Tensor, z: torch.Tensor,
                     dt_bias: torch.Tensor, A_log: torch.Tensor, D_skip: torch.Tensor, state: torch.Tensor,
                     cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor, state_slots: torch.Tensor) -> torch.Tensor:
    """State-space scan over a step's rows, state [slots, H, N, P] float32 updated in place; x: [T, H, P]; Bm, Cm:
    [T, G, N]; dt_raw [T, H]; z [T, H * P]; returns y * silu(z) as float32 [T, H * P]."""
    dt = _dt(x, "x")
    T, H, P = x.shape
    G, N = Bm.shape[1], Bm.shape[2]
    for t, n in ((x, "x"), (Bm, "B"), (Cm, "C")):
        _rows_ok(t, n)
        _need(t.dtype == x.dtype, "x, B, C must have one dtype")
    _need(Bm.shape == (T, G, N) and Cm.shape == (T, G, N) and H % G == 0, "B / C must be [T, G, N] with G dividing H")
    for t, n, cols in ((dt_raw, "dt_raw", H), (z, "z", H * P)):
        _rows2d(t, n)
        _need(t.shape == (T, cols) and t.dtype == x.dtype, f"{n} must be [T, {cols}] of x's dtype")
    _need(state.is_cuda and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, N, P),
          "state must be contiguous float32 [slots, H, N, P]")
    _need(dt_bias.numel() == H and A_log.numel() == H and D_skip.numel() == H, "constant shapes")
    B = _seq_meta(cu_seqlens_q, cu_seqlens_k, state_slots)
    out = torch.empty((T, H * P), dtype=torch.float32, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_state_space_scan(x.data_ptr(), Bm.data_ptr(), Cm.data_ptr(), x.stride(0), Bm.stride(0), Cm.stride(0),
                                 dt_raw.data_ptr(), dt_raw.stride(0), z.data_ptr(), z.stride(0), _f32c(dt_bias, "dt_bias"),
                                 _f32c(A_log, "A_log"), _f32c(D_skip, "D"), state.data_ptr(), out.data_ptr(), out.stride(0),
                                 cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), state_slots.data_ptr(), B, H, G, N, P,
                                 dt, _stream(x))
    _lib.check(rc, "nv_state_space_scan", dll)
    return out


def token_shift_mix(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, cu_seqlens_q: torch.Tensor,
                    cu_seqlens_k: torch.Tensor, state_slots: torch.Tensor) -> torch.Tensor:
    """out[s] = h + (previous row of h - h) * mu[s]; h [T, C] (row stride free); mu [n, C] float32; state [slots, C] of
    h's dtype carries each sequence's last row and is updated; returns [n, T, C]."""
    dt = _dt(h, "h")
    _rows2d(h, "h")
    T, Cc = h.shape
    _need(mu.dim() == 2 and mu.shape[1] == Cc, "mu must be [n, C]")
    _need(state.is_cuda and state.dtype == h.dtype and state.is_contiguous() and state.shape[1:] == (Cc,),
          "state must be contiguous [slots, C] of h's dtype")
    B = _seq_meta(cu_seqlens_q, cu_seqlens_k, state_slots)
    out = torch.empty((mu.shape[0], T, Cc), dtype=h.dtype, device=h.device)
    dll = _lib.mixers()
    rc = dll.nv_token_shift_mix(h.data_ptr(), h.stride(0), _f32c(mu, "mu"), mu.shape[0], state.data_ptr(), out.data_ptr(),
                                cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), state_slots.data_ptr(), B, T, Cc, dt,
                                _stream(h))
    _lib.check(rc, "nv_token_shift_mix", dll)
    return out


def group_rms_norm(x: torch.Tensor, weight: torch.Tensor, groups: int, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """Every row of x [T, C] float32 is cut into `groups` equal parts, each divided by its own root mean square; times
    weight; result in out_dtype."""
    _need(x.is_cuda and x.dtype == torch.float32, "x must be a float32 GPU tensor")
    _rows2d(x, "x")
    _need(weight.numel() == x.shape[1] and x.shape[1] % groups == 0, "weight must be [cols], groups must divide cols")
    y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_group_rms_norm(x.data_ptr(), x.stride(0), _f32c(weight, "weight"), y.data_ptr(), y.stride(0), _dt(y, "y"),
                               x.shape[0], x.shape[1], int(groups), float(eps), _stream(x))
    _lib.check(rc, "nv_group_rms_norm", dll)
    return y


def chunk_attn_prep_store(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_norm: torch.Tensor,
                          k_norm: torch.Tensor, eps: float, freq: Optional[torch.Tensor], rot_dims: int,
                          value_freq: torch.Tensor, slot_mapping: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                          v_cache: Optional[torch.Tensor]) -> torch.Tensor:
    """RMS norm over the whole q / k rows, rotate-half rotary on the first rot_dims dimensions of every head, values
    turned over all their dimensions, scatter of k / v into the paged cache; returns the prepared q [T, H, D]."""
    dt = _dt(q, "q")
    for t, n in ((q, "q"), (k, "k"), (v, "v")):
        _rows_ok(t, n)
        _need(t.dtype == q.dtype, "q, k, v must have one dtype")
    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    _need(k.shape == (T, G, D) and v.shape[:2] == (T, G), "k / v rows do not match q")
    _need(q_norm.numel() == H * D and k_norm.numel() == G * D, "the norm weights span the whole q / k rows")
    _need(positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T,
          "positions must be a contiguous int64 [tokens] GPU tensor")
    _need(value_freq.numel() == Dv // 2 and Dv % 2 == 0, "value_freq must hold Dv / 2 frequencies")
    if rot_dims:
        _need(freq is not None and freq.numel() == rot_dims // 2, "freq must hold rot_dims / 2 frequencies")
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        _need(slot_mapping.numel() == T, "slot_mapping length != number of tokens")
        _need(k_cache is not None and v_cache is not None and k_cache.is_contiguous() and v_cache.is_contiguous()
              and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype and k_cache.shape[2:] == (G, D)
              and v_cache.shape[2:] == (G, Dv) and k_cache.shape[:2] == v_cache.shape[:2],
              "caches must be contiguous [num_blocks, block_size, G, D] and [.., G, Dv] of q's dtype")
    q_out = torch.empty((T, H, D), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    rc = dll.nv_chunk_attn_prep_store(q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(0), k.stride(0), v.stride(0),
                                      _f32c(q_norm, "q_norm"), _f32c(k_norm, "k_norm"), float(eps),
                                      _f32c(freq, "freq") or None, int(rot_dims), _f32c(value_freq, "value_freq"),
                                      positions.data_ptr(), _ptr(slot_mapping), q_out.data_ptr(), _ptr(k_cache),
                                      _ptr(v_cache), dt, T, H, G, D, Dv, _stream(q))
    _lib.check(rc, "nv_chunk_attn_prep_store", dll)
    return q_out


def chunk_sigmoid_tile_ok(D: int, Dv: int, dtype: torch.dtype) -> bool:
    return bool(_lib.mixers().nv_attn_chunk_sigmoid_tile_ok(int(D), int(Dv), _lib.DTYPE_BF16 if dtype == _BF16 else _lib.DTYPE_F32))


def attn_chunk_sigmoid_paged(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cu_seqlens_q: torch.Tensor,
                             cu_seqlens_k: torch.Tensor, block_tables: torch.Tensor, scale: float,
                             head_bias: Optional[torch.Tensor], chunk: int, value_freq: torch.Tensor,
                             tiles: Optional[tuple] = None, single_rows: bool = True) -> torch.Tensor:
    """Sigmoid attention inside chunks of positions over a paged cache of rotated values (the sum is turned back by the
    query's position); returns [T, H * Dv].  tiles: (tile_seq, tile_q0) int32 GPU tensors that cut the rows of sequences
    with several rows into blocks of 64 for the MFMA kernel; None: every row on the one-wave-per-row kernel."""
    dt = _dt(q, "q")
    _rows_ok(q, "q")
    T, H, D = q.shape
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous()
          and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype and k_cache.shape[:3] == v_cache.shape[:3]
          and k_cache.shape[3] == D, "caches must be contiguous [num_blocks, block_size, G, D | Dv] of q's dtype")
    nb, bs, G, _ = k_cache.shape
    Dv = v_cache.shape[3]
    _i32(cu_seqlens_q, "cu_seqlens_q")
    _i32(cu_seqlens_k, "cu_seqlens_k")
    B = cu_seqlens_k.numel() - 1
    _need(cu_seqlens_q.numel() == B + 1, "cu_seqlens_q / cu_seqlens_k length mismatch")
    _need(block_tables.is_cuda and block_tables.dtype == torch.int32 and block_tables.dim() == 2
          and block_tables.is_contiguous() and block_tables.shape[0] == B,
          "block_tables must be a contiguous [B, max_blocks] int32 GPU tensor")
    _need(head_bias is None or head_bias.numel() == H, "head_bias must be [H]")
    _need(value_freq.numel() == Dv // 2, "value_freq must hold Dv / 2 frequencies")
    n_tiles = 0
    if tiles is not None:
        _i32(tiles[0], "tile_seq")
        _i32(tiles[1], "tile_q0")
        n_tiles = tiles[0].numel()
        _need(tiles[1].numel() == n_tiles, "tile tables differ in length")
    out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    rc = dll.nv_attn_chunk_sigmoid_paged(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
                                         cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), block_tables.data_ptr(), B,
                                         block_tables.shape[1], T, H, G, D, Dv, nb, bs, float(scale),
                                         _f32c(head_bias, "head_bias") or None, int(chunk),
                                         _f32c(value_freq, "value_freq"), _ptr(tiles[0]) if n_tiles else None,
                                         _ptr(tiles[1]) if n_tiles else None, n_tiles, int(bool(single_rows)), dt,
                                         q.stride(0), out.stride(0), _stream(q))
    _lib.check(rc, "nv_attn_chunk_sigmoid_paged", dll)
    return out


def moe_table_experts(h: torch.Tensor, ids: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """Experts chosen by a table: h [T, W]; ids [T, top] int32 (the experts of every token, distinct per row); gate_up
    [E, 2 ff, W]; down [E, W, ff].  Expert: D (silu(G h) * (U h)).  Returns the UNWEIGHTED outputs of every token's
    experts, [T, top, W] float32 (the stream update scales and sums them)."""
    dt = _dt(h, "h")
    _rows2d(h, "h")
    T, W = h.shape
    E, ff = gate_up.shape[0], gate_up.shape[1] // 2
    top = ids.shape[1]
    _need(ids.is_cuda and ids.dtype == torch.int32 and ids.is_contiguous() and ids.shape == (T, top),
          "ids must be contiguous int32 [T, top]")
    _need(gate_up.is_cuda and down.is_cuda and gate_up.is_contiguous() and down.is_contiguous() and gate_up.dtype == h.dtype
          and down.dtype == h.dtype and gate_up.shape == (E, 2 * ff, W) and down.shape == (E, W, ff),
          "gate_up must be [E, 2 ff, W] and down [E, W, ff], contiguous, of h's dtype")
    dll = _lib.mixers()
    dev, P, s = h.device, T * top, _stream(h)
    out = torch.empty((T, top, W), dtype=torch.float32, device=dev)
    if T == 0:
        return out
    wgt = torch.ones((T, top), dtype=torch.float32, device=dev)
    rows = dll.nv_moe_tile_rows(P, E)
    tiles = dll.nv_moe_max_tiles(P, E, rows)
    sorted_pairs = torch.empty(P, dtype=torch.int32, device=dev)
    meta = torch.empty(1 + 3 * tiles, dtype=torch.int32, device=dev)
    _lib.check(dll.nv_moe_align(ids.data_ptr(), sorted_pairs.data_ptr(), meta.data_ptr(), P, E, rows, s), "nv_moe_align", dll)
    y = torch.empty((P, ff), dtype=h.dtype, device=dev)
    _lib.check(dll.nv_moe_gate_up_act(h.data_ptr(), h.stride(0), gate_up.data_ptr(), sorted_pairs.data_ptr(),
                                      meta.data_ptr(), y.data_ptr(), dt, P, E, int(top), W, ff, float("inf"), 1.0, 0.0,
                                      rows, s), "nv_moe_gate_up_act", dll)
    _lib.check(dll.nv_moe_down(y.data_ptr(), down.data_ptr(), sorted_pairs.data_ptr(), meta.data_ptr(), wgt.data_ptr(),
                               out.data_ptr(), dt, P, E, W, ff, rows, s), "nv_moe_down", dll)
    return out


# ---------------------------------------------------------------------------------------------------------
# Pre-norm fp32 stream with per-column output scales, memories written before they are read (exponential-gate matrix
# memory, gated-write recurrence), attention whose values are its un-normed keys, polynomial-of-norms activation,
# sigmoid routing over groups of squared-ReLU experts.
# ---------------------------------------------------------------------------------------------------------
def stream_boundary_scaled(x: torch.Tensor, add: Optional[torch.Tensor] = None, gated: Optional[tuple] = None,
                           parts: Optional[torch.Tensor] = None, col_scale: Optional[torch.Tensor] = None,
                           norm: Optional[torch.Tensor] = None, eps: float = 1e-5,
                           out_dtype: Optional[torch.dtype] = None, want_f32: bool = False):
    """One sublayer boundary of a pre-norm fp32 stream x [T, W], in place:
    x += col_scale * (add + sigmoid(g) * a2 + parts.sum(1)) with gated = (a2 [T, W], g [T] raw gate, one per row);
    norm: the RMS-norm weight of the updated stream AS APPLIED (a one-plus weight is folded by the caller).
    Returns (h32, h): the norm in float32 (if want_f32) and in out_dtype (if given); None for each part not asked for."""
    _need(x.is_cuda and x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(),
          "the stream must be a contiguous float32 [tokens, width] GPU tensor")
    rows, cols = x.shape
    a2, g2 = gated if gated is not None else (None, None)
    ins = [t for t in (add, a2) if t is not None]
    dt_t = out_dtype or (ins[0].dtype if ins else torch.float32)
    _need(dt_t in (_BF16, torch.float32), "the matmul dtype must be bfloat16 or float32")
    dt = _lib.DTYPE_BF16 if dt_t == _BF16 else _lib.DTYPE_F32
    for t in ins:
        _rows2d(t, "input")
        _need(t.shape == x.shape and t.dtype == dt_t and t.is_cuda, "inputs must match the stream's shape, in the matmul dtype")
    if g2 is not None:
        _need(g2.is_cuda and g2.dtype == dt_t and g2.dim() == 1 and g2.numel() == rows, "the gate must be [T] of the matmul dtype")
    n_parts = 0
    if parts is not None:
        _need(parts.is_cuda and parts.dtype == torch.float32 and parts.is_contiguous() and parts.dim() == 3
              and parts.shape[0] == rows and parts.shape[2] == cols, "parts must be contiguous float32 [T, n, W]")
        n_parts = parts.shape[1]
    for w in (col_scale, norm):
        _need(w is None or w.numel() == cols, "column scale and norm weight must be [width]")
    y32 = y = None
    if norm is not None:
        if want_f32:
            y32 = torch.empty((rows, cols), dtype=torch.float32, device=x.device)
        if out_dtype is not None:
            y = torch.empty((rows, cols), dtype=out_dtype, device=x.device)
        _need(y32 is not None or y is not None, "the norm needs an output")
    dll = _lib.mixers()
    rc = dll.nv_stream_boundary_scaled(x.data_ptr(), _ptr(add), add.stride(0) if add is not None else 0, _ptr(a2),
                                       a2.stride(0) if a2 is not None else 0, _ptr(g2), g2.stride(0) if g2 is not None else 0,
                                       _ptr(parts) if n_parts else None, n_parts, _f32c(col_scale, "col_scale") or None,
                                       _f32c(norm, "norm") or None, float(eps), _ptr(y32), _ptr(y), dt, rows, cols,
                                       _stream(x))
    _lib.check(rc, "nv_stream_boundary_scaled", dll)
    return y32, y


def poly_norm(x: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """coef[0] x / rms(x) + coef[1] x^2 / rms(x^2) + coef[2] x^3 / rms(x^3) + coef[3] per row of x [T, C]; coef: 4 float32
    on the device."""
    dt = _dt(x, "x")
    _rows2d(x, "x")
    _need(coef.numel() == 4, "coef must hold four numbers")
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    dll = _lib.mixers()
    _lib.check(dll.nv_poly_norm(x.data_ptr(), x.stride(0), _f32c(coef, "coef"), float(eps), y.data_ptr(), dt, x.shape[0],
                                x.shape[1], _stream(x)), "nv_poly_norm", dll)
    return y


def causal_conv(x: torch.Tensor, weight: torch.Tensor, conv_state: torch.Tensor, cu_seqlens_q: torch.Tensor,
                cu_seqlens_k: torch.Tensor, state_slots: torch.Tensor, bias: Optional[torch.Tensor] = None,
                silu: bool = False) -> torch.Tensor:
    """Causal conv over time per channel of x [T, C] (+ bias, then SiLU if asked); weight [C, taps] float32; conv_state
    [num_slots, taps - 1, C] (x's dtype) carries each sequence's last inputs and is updated."""
    dt = _dt(x, "x")
    _rows2d(x, "x")
    T, Cc = x.shape
    taps = weight.shape[1]
    _need(weight.shape[0] == Cc and (bias is None or bias.numel() == Cc), "weight must be [channels, taps], bias [channels]")
    _need(conv_state.is_cuda and conv_state.dtype == x.dtype and conv_state.is_contiguous()
          and conv_state.shape[1:] == (taps - 1, Cc), "conv_state must be contiguous [slots, taps - 1, C] of x's dtype")
    B = _seq_meta(cu_seqlens_q, cu_seqlens_k, state_slots)
    y = torch.empty((T, Cc), dtype=x.dtype, device=x.device)
    dll = _lib.mixers()
    rc = dll.nv_causal_conv_act(x.data_ptr(), x.stride(0), _f32c(weight, "weight"), _f32c(bias, "bias") or None,
                                conv_state.data_ptr(), y.data_ptr(), y.stride(0), cu_seqlens_q.data_ptr(),
                                cu_seqlens_k.data_ptr(), state_slots.data_ptr(), B, T, Cc, taps, 1 if silu else 0, dt,
                                _stream(x))
    _lib.check(rc, "nv_causal_conv_act", dll)
    return y


def head_norm_rope_store(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, q_norm: torch.Tensor,
                         k_norm: torch.Tensor, eps: float, freq: Optional[torch.Tensor], rot_dims: int,
                         slot_mapping: Optional[torch.Tensor], k_cache: torch.Tensor, v_cache: torch.Tensor) -> torch.Tensor:
    """Per-head RMS norm of q [T, H, D] and k [T, G, D] (weights [D]), rotate-half rotary on the first rot_dims
    dimensions, scatter of the prepared k into k_cache and of k as given into v_cache; returns the prepared q."""
    dt = _dt(q, "q")
    for t, n in ((q, "q"), (k, "k")):
        _rows_ok(t, n)
        _need(t.dtype == q.dtype, "q, k must have one dtype")
    T, H, D = q.shape
    G = k.shape[1]
    _need(k.shape == (T, G, D), "k rows do not match q")
    _need(positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T,
          "positions must be a contiguous int64 [tokens] GPU tensor")
    _need(q_norm.numel() == D and k_norm.numel() == D, "norm weights must be [D]")
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        _need(slot_mapping.numel() == T, "slot_mapping length != number of tokens")
    for c in (k_cache, v_cache):
        _need(c.is_cuda and c.is_contiguous() and c.dtype == q.dtype and c.dim() == 4 and c.shape[2:] == (G, D),
              "caches must be contiguous [num_blocks, block_size, G, D] of q's dtype")
    if rot_dims:
        _need(freq is not None and freq.numel() == rot_dims // 2, "freq must hold rot_dims / 2 frequencies")
    q_out = torch.empty((T, H, D), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    rc = dll.nv_head_norm_rope_store(q.data_ptr(), k.data_ptr(), q.stride(0), k.stride(0), _f32c(q_norm, "q_norm"),
                                     _f32c(k_norm, "k_norm"), float(eps), _f32c(freq, "freq") or None, int(rot_dims),
                                     positions.data_ptr(), _ptr(slot_mapping), q_out.data_ptr(), k_cache.data_ptr(),
                                     v_cache.data_ptr(), dt, T, H, G, D, _stream(q))
    _lib.check(rc, "nv_head_norm_rope_store", dll)
    return q_out


def mlstm_memory(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gates_pre: torch.Tensor, gate_raw: torch.Tensor,
                 i_bias: torch.Tensor, f_bias: torch.Tensor, norm_weight: torch.Tensor, state: torch.Tensor,
                 norm_state: torch.Tensor, max_state: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                 state_slots: torch.Tensor, eps: float, gate_cap: float, q_scale: float) -> torch.Tensor:
    """Matrix memory with exponential gates over a step's rows; q, k: [T, H, Dk]; v: [T, H, Dv]; gates_pre [T, 2 H] float32
    (input-gate columns, then forget-gate columns, without bias); gate_raw [T, H * Dv]; state [slots, H, Dk, Dv],
    norm_state [slots, H, Dk], max_state [slots, H] float32, updated in place; returns [T, H * Dv]."""
    dt = _dt(q, "q")
    T, H, Dk = q.shape
    Dv = v.shape[2]
    for t, n in ((q, "q"), (k, "k"), (v, "v")):
        _rows_ok(t, n)
        _need(t.dtype == q.dtype, "q, k, v must have one dtype")
    _need(k.shape == (T, H, Dk) and v.shape[:2] == (T, H), "q / k / v rows differ")
    _rows2d(gate_raw, "gate_raw")
    _need(gate_raw.shape == (T, H * Dv) and gate_raw.dtype == q.dtype, "gate_raw must be [T, H * Dv] of q's dtype")
    _need(gates_pre.is_cuda and gates_pre.dtype == torch.float32 and gates_pre.dim() == 2 and gates_pre.stride(1) == 1
          and gates_pre.shape == (T, 2 * H), "gates_pre must be float32 [T, 2 H]")
    for t, n, shape in ((state, "state", (H, Dk, Dv)), (norm_state, "norm_state", (H, Dk)), (max_state, "max_state", (H,))):
        _need(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.shape[1:] == shape,
              f"{n} must be contiguous float32 [slots, {shape}]")
    _need(i_bias.numel() == H and f_bias.numel() == H and norm_weight.numel() == H * Dv, "constant shapes")
    B = _seq_meta(cu_seqlens_q, cu_seqlens_k, state_slots)
    out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    rc = dll.nv_mlstm_memory(q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(0), k.stride(0), v.stride(0),
                             gates_pre.data_ptr(), gates_pre.data_ptr() + 4 * H, gates_pre.stride(0), gate_raw.data_ptr(),
                             gate_raw.stride(0), _f32c(i_bias, "i_bias"), _f32c(f_bias, "f_bias"),
                             _f32c(norm_weight, "norm_weight"), state.data_ptr(), norm_state.data_ptr(),
                             max_state.data_ptr(), out.data_ptr(), out.stride(0), cu_seqlens_q.data_ptr(),
                             cu_seqlens_k.data_ptr(), state_slots.data_ptr(), B, H, Dk, Dv, float(eps), float(gate_cap),
                             float(q_scale), dt, _stream(q))
    _lib.check(rc, "nv_mlstm_memory", dll)
    return out


def gated_write_memory(q: torch.Tensor, f_raw: torch.Tensor, v: torch.Tensor, f_bias: torch.Tensor, lower: torch.Tensor,
                       norm_weight: torch.Tensor, state: torch.Tensor, cu_seqlens_q: torch.Tensor,
                       cu_seqlens_k: torch.Tensor, state_slots: torch.Tensor, eps: float) -> torch.Tensor:
    """Gated linear recurrence whose forget gate decides what is written; q, f_raw: [T, H, Dk] as projected; v: [T, H, Dv];
    f_bias, lower [H * Dk], norm_weight [Dv] float32; state [slots, H, Dk, Dv] float32 updated in place; returns
    [T, H * Dv]."""
    dt = _dt(q, "q")
    T, H, Dk = q.shape
    Dv = v.shape[2]
    for t, n in ((q, "q"), (f_raw, "f_raw"), (v, "v")):
        _rows_ok(t, n)
        _need(t.dtype == q.dtype, "q, f_raw, v must have one dtype")
    _need(f_raw.shape == (T, H, Dk) and v.shape[:2] == (T, H), "q / f_raw / v rows differ")
    _need(state.is_cuda and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, Dk, Dv),
          "state must be contiguous float32 [slots, H, Dk, Dv]")
    _need(f_bias.numel() == H * Dk and lower.numel() == H * Dk and norm_weight.numel() == Dv, "constant shapes")
    B = _seq_meta(cu_seqlens_q, cu_seqlens_k, state_slots)
    out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
    dll = _lib.mixers()
    rc = dll.nv_gated_write_memory(q.data_ptr(), f_raw.data_ptr(), v.data_ptr(), q.stride(0), f_raw.stride(0), v.stride(0),
                                   _f32c(f_bias, "f_bias"), _f32c(lower, "lower"), _f32c(norm_weight, "norm_weight"),
                                   state.data_ptr(), out.data_ptr(), out.stride(0), cu_seqlens_q.data_ptr(),
                                   cu_seqlens_k.data_ptr(), state_slots.data_ptr(), B, H, Dk, Dv, float(eps), dt, _stream(q))
    _lib.check(rc, "nv_gated_write_memory", dll)
    return out


def moe_route_grouped(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, n_groups: int,
                      keep_groups: int) -> tuple:
    """(ids [T, top] int32, weights [T, top] float32): sigmoid scores, choice on score + correction within the best
    groups, weights the plain scores of the chosen."""
    _need(logits.is_cuda and logits.dtype == torch.float32 and logits.is_contiguous() and logits.dim() == 2,
          "logits must be contiguous float32 [T, E]")
    T, E = logits.shape
    _need(correction is None or correction.numel() == E, "correction must be [E]")
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    wgt = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    dll = _lib.mixers()
    _lib.check(dll.nv_moe_route_grouped(logits.data_ptr(), _f32c(correction, "correction") or None, ids.data_ptr(),
                                        wgt.data_ptr(), T, E, int(top), int(n_groups), int(keep_groups), _stream(logits)),
               "nv_moe_route_grouped", dll)
    return ids, wgt


def moe_relu2_experts(h: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, up: torch.Tensor,
                      down: torch.Tensor) -> torch.Tensor:
    """Squared-ReLU experts for given choices: h [T, W]; ids [T, top] int32; weights [T, top] float32; up [E, ff, W];
    down [E, W, ff].  Returns the weighted outputs [T, top, W] float32 (the stream update sums them)."""
    dt = _dt(h, "h")
    _rows2d(h, "h")
    T, W = h.shape
    E, ff = up.shape[0], up.shape[1]
    top = ids.shape[1]
    _need(ids.is_cuda and ids.dtype == torch.int32 and ids.is_contiguous() and ids.shape == (T, top)
          and weights.is_cuda and weights.dtype == torch.float32 and weights.is_contiguous() and weights.shape == (T, top),
          "ids must be contiguous int32 [T, top], weights float32 [T, top]")
    _need(up.is_cuda and down.is_cuda and up.is_contiguous() and down.is_contiguous() and up.dtype == h.dtype
          and down.dtype == h.dtype and up.shape == (E, ff, W) and down.shape == (E, W, ff),
          "up must be [E, ff, W] and down [E, W, ff], contiguous, of h's dtype")
    dll = _lib.mixers()
    dev, P, s = h.device, T * top, _stream(h)
    out = torch.empty((T, top, W), dtype=torch.float32, device=dev)
    if T == 0:
        return out
    rows = dll.nv_moe_tile_rows(P, E)
    tiles = dll.nv_moe_max_tiles(P, E, rows)
    sorted_pairs = torch.empty(P, dtype=torch.int32, device=dev)
    meta = torch.empty(1 + 3 * tiles, dtype=torch.int32, device=dev)
    _lib.check(dll.nv_moe_align(ids.data_ptr(), sorted_pairs.data_ptr(), meta.data_ptr(), P, E, rows, s), "nv_moe_align", dll)
    y = torch.empty((P, ff), dtype=h.dtype, device=dev)
    _lib.check(dll.nv_moe_up_relu2(h.data_ptr(), h.stride(0), up.data_ptr(), sorted_pairs.data_ptr(), meta.data_ptr(),
                                   y.data_ptr(), dt, P, E, int(top), W, ff, rows, s), "nv_moe_up_relu2", dll)
    _lib.check(dll.nv_moe_down(y.data_ptr(), down.data_ptr(), sorted_pairs.data_ptr(), meta.data_ptr(), weights.data_ptr(),
                               out.data_ptr(), dt, P, E, W, ff, rows, s), "nv_moe_down", dll)
    return out
