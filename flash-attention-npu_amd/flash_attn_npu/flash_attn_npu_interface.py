"""Public API of flash_attn_npu on MI355X: the inference forward of the paged KV-cache path.

Signatures, argument order, defaults and return conventions follow the reference package
(flash_attn_npu/flash_attn_npu_interface.py:1344-1361 `flash_attn_varlen_func`,
:1438-1458 `flash_attn_with_kvcache`); the work is done by hand-written gfx950 kernels
behind the C ABI in include/fa_rocm.h.  Differences from the reference, all additive:
  * `k` / `v` are appended in place and `rotary_cos` / `rotary_sin` are applied, as the
    reference's docstring promises (its host code ignores k/v and rejects rotary);
  * `flash_attn_with_kvcache` takes keyword-only `k_scale_cache` / `v_scale_cache` for an int8
    latent cache with per-token fp32 scales;
  * `flash_attn_varlen_func` honours `block_table` (paged K/V, per-sequence lengths from
    cu_seqlens_k), which reference v2 rejects (flash_api.cpp:885).
Backward is not part of this build: tensors that require grad raise."""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

from . import flash_attn_npu  # operator layer (reference: the compiled extension of the same name)


def maybe_contiguous(x):
    return x.contiguous() if x is not None and x.stride(-1) != 1 else x


def round_multiple(x, m):
    return (x + m - 1) // m * m


# ------------------------------------------------------------------ varlen forward custom op
@torch.library.custom_op("flash_attn_npu::_flash_attn_varlen_forward", mutates_args=(), device_types="cuda")
def _flash_attn_varlen_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    dropout_p: float,
    softmax_scale: float,
    causal: bool,
    window_size_left: int = -1,
    window_size_right: int = -1,
    softcap: float = 0.0,
    alibi_slopes: Optional[torch.Tensor] = None,
    return_softmax: bool = False,
    block_table: Optional[torch.Tensor] = None,
    leftpad_k: Optional[torch.Tensor] = None,
    seqused_k: Optional[torch.Tensor] = None,
    zero_tensors: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    out, softmax_lse, S_dmask, rng_state = flash_attn_npu.varlen_fwd(
        q, k, v, None, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, block_table, alibi_slopes,
        max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, zero_tensors, causal,
        window_size_left, window_size_right, softcap, return_softmax, None,
    )
    return out, softmax_lse, S_dmask, rng_state


@torch.library.register_fake("flash_attn_npu::_flash_attn_varlen_forward")
def _flash_attn_varlen_forward_fake(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    dropout_p: float,
    softmax_scale: float,
    causal: bool,
    window_size_left: int = -1,
    window_size_right: int = -1,
    softcap: float = 0.0,
    alibi_slopes: Optional[torch.Tensor] = None,
    return_softmax: bool = False,
    block_table: Optional[torch.Tensor] = None,
    leftpad_k: Optional[torch.Tensor] = None,
    seqused_k: Optional[torch.Tensor] = None,
    zero_tensors: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    total_q, num_heads, _ = q.shape
    out = torch.empty_like(q, memory_format=torch.contiguous_format)
    softmax_lse = torch.empty((num_heads, total_q), dtype=torch.float32, device=q.device)
    p = torch.empty((0,), dtype=q.dtype, device=q.device)
    rng_state = torch.empty((2,), dtype=torch.int64, device=q.device)
    return out, softmax_lse, p, rng_state


_wrapped_flash_attn_varlen_forward = _flash_attn_varlen_forward


def _varlen_forward_eager(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale,
                          causal, window_size_left=-1, window_size_right=-1, softcap=0.0, alibi_slopes=None,
                          return_softmax=False, block_table=None, leftpad_k=None, seqused_k=None, zero_tensors=False):
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    return tuple(flash_attn_npu.varlen_fwd(
        q, k, v, None, cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, block_table, alibi_slopes,
        max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, zero_tensors, causal,
        window_size_left, window_size_right, softcap, return_softmax, None))


# ------------------------------------------------------------------ kvcache forward custom op
@torch.library.custom_op("flash_attn_npu::_flash_attn_kvcache_forward",
                         mutates_args=("k_cache", "v_cache", "k_scale_cache", "v_scale_cache"), device_types="cuda")
def _flash_attn_kvcache_forward(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k: Optional[torch.Tensor],
    v: Optional[torch.Tensor],
    cache_seqlens: Optional[torch.Tensor],
    rotary_cos: Optional[torch.Tensor],
    rotary_sin: Optional[torch.Tensor],
    cache_batch_idx: Optional[torch.Tensor],
    cache_leftpad: Optional[torch.Tensor],
    block_table: Optional[torch.Tensor],
    alibi_slopes: Optional[torch.Tensor],
    softmax_scale: float,
    causal: bool,
    window_size_left: int,
    window_size_right: int,
    softcap: float,
    rotary_interleaved: bool,
    num_splits: int,
    k_scale_cache: Optional[torch.Tensor],   # no defaults: the dispatcher drops trailing default arguments,
    v_scale_cache: Optional[torch.Tensor],   # and a mutated argument must be there to be version-bumped
) -> Tuple[torch.Tensor, torch.Tensor]:
    out, softmax_lse = flash_attn_npu.fwd_kvcache(
        q, k_cache, v_cache, k, v, cache_seqlens, rotary_cos, rotary_sin, cache_batch_idx, cache_leftpad,
        block_table, alibi_slopes, None, softmax_scale, causal, window_size_left, window_size_right, softcap,
        rotary_interleaved, num_splits, k_scale_cache, v_scale_cache,
    )
    return out, softmax_lse


@torch.library.register_fake("flash_attn_npu::_flash_attn_kvcache_forward")
def _flash_attn_kvcache_forward_fake(
    q, k_cache, v_cache, k, v, cache_seqlens, rotary_cos, rotary_sin, cache_batch_idx, cache_leftpad, block_table,
    alibi_slopes, softmax_scale, causal, window_size_left, window_size_right, softcap, rotary_interleaved, num_splits,
    k_scale_cache, v_scale_cache,
):
    B, sq, hq, _ = q.shape
    out = torch.empty((B, sq, hq, v_cache.shape[-1]), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, hq, sq), dtype=torch.float32, device=q.device)
    return out, lse


def _kvcache_forward_eager(q, k_cache, v_cache, k, v, cache_seqlens, rotary_cos, rotary_sin, cache_batch_idx,
                           cache_leftpad, block_table, alibi_slopes, softmax_scale, causal, window_size_left,
                           window_size_right, softcap, rotary_interleaved, num_splits, k_scale_cache=None,
                           v_scale_cache=None):
    out, softmax_lse = flash_attn_npu.fwd_kvcache(
        q, k_cache, v_cache, k, v, cache_seqlens, rotary_cos, rotary_sin, cache_batch_idx, cache_leftpad,
        block_table, alibi_slopes, None, softmax_scale, causal, window_size_left, window_size_right, softcap,
        rotary_interleaved, num_splits, k_scale_cache, v_scale_cache,
    )
    return out, softmax_lse


class FlashAttnVarlenFunc(torch.autograd.Function):
    """Forward half of the reference's autograd function (flash_attn_npu_interface.py:870-935)."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale,
                causal, window_size, softcap, alibi_slopes, deterministic, return_softmax, block_table,
                is_grad_enabled):
        is_grad = is_grad_enabled and any(x.requires_grad for x in [q, k, v])
        if is_grad:
            raise RuntimeError("flash_attn_npu (MI355X build) implements the inference forward only: "
                               "call it under torch.no_grad() or with tensors that do not require grad")
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        head_size_og = q.size(2)
        # As the reference does (flash_attn_npu_interface.py:897-901): a head dimension that is not a multiple of 8 is
        # padded with zeros to the next one (zero columns change neither QK^T nor the kept columns of PV); every
        # multiple of 8 up to 256 runs as it is.  Paged k / v are padded the same way, which copies the cache: rows
        # of such a width are not 16-byte pieces.
        head_size_pad = (head_size_og + 7) // 8 * 8
        if head_size_pad != head_size_og:
            q = torch.nn.functional.pad(q, [0, head_size_pad - head_size_og])
            k = torch.nn.functional.pad(k, [0, head_size_pad - head_size_og])
            v = torch.nn.functional.pad(v, [0, head_size_pad - head_size_og])
        fwd = _wrapped_flash_attn_varlen_forward if torch.compiler.is_compiling() else _varlen_forward_eager
        out_padded, softmax_lse, S_dmask, rng_state = fwd(
            q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale,
            causal=causal, window_size_left=window_size[0], window_size_right=window_size[1], softcap=softcap,
            alibi_slopes=alibi_slopes, return_softmax=return_softmax and dropout_p > 0, block_table=block_table,
        )
        out = out_padded[..., :head_size_og]
        return out if not return_softmax else (out, softmax_lse, S_dmask)

    @staticmethod
    def backward(ctx, *args):
        raise RuntimeError("flash_attn_npu (MI355X build) does not implement the backward pass")


def flash_attn_varlen_func(
    q,
    k,
    v,
    cu_seqlens_q,
    cu_seqlens_k,
    max_seqlen_q,
    max_seqlen_k,
    dropout_p=0.0,
    softmax_scale=None,
    causal=False,
    window_size=(-1, -1),  # -1 means infinite context window
    softcap=0.0,  # 0.0 means deactivated
    alibi_slopes=None,
    deterministic=False,
    return_attn_probs=False,
    block_table=None,
):
    """Variable-length attention forward over packed sequences.

    q: (total_q, nheads, headdim); k, v: (total_k, nheads_k, headdim), or, with `block_table`
    (batch, max_blocks) int32, paged (num_blocks, page_block_size, nheads_k, headdim) with the
    per-sequence key counts taken from cu_seqlens_k.  cu_seqlens_*: (batch+1,) int32.
    GQA/MQA: q head h reads kv head h // (nheads // nheads_k).  causal is aligned to the bottom
    right corner; window_size=(left, right) keeps keys in
    [i + seqlen_k - seqlen_q - left, i + seqlen_k - seqlen_q + right]; rows with no visible key
    give 0.  dropout_p must be 0, alibi_slopes None.
    Returns out (total_q, nheads, headdim), or (out, softmax_lse (nheads, total_q) fp32, S_dmask
    (empty)) when return_attn_probs=True.
    """
    return FlashAttnVarlenFunc.apply(
        q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, causal,
        window_size, softcap, alibi_slopes, deterministic, return_attn_probs, block_table, torch.is_grad_enabled(),
    )


_cu_cache = {}


def _even_cu_seqlens(batch: int, seqlen: int, device) -> torch.Tensor:
    """cu_seqlens of `batch` sequences of `seqlen` tokens each, built once per (batch, seqlen, device)."""
    key = (batch, seqlen, str(device))
    if key not in _cu_cache:
        _cu_cache[key] = torch.arange(batch + 1, dtype=torch.int32, device=device) * seqlen
    return _cu_cache[key]


def flash_attn_func(
    q,
    k,
    v,
    dropout_p=0.0,
    softmax_scale=None,
    causal=False,
    window_size=(-1, -1),  # -1 means infinite context window
    softcap=0.0,  # 0.0 means deactivated
    alibi_slopes=None,
    deterministic=False,
    return_attn_probs=False,
):
    """Attention forward over dense batches (reference flash_attn_npu_interface.py:1109-1183; forward only).

    q: (batch, seqlen_q, nheads, headdim); k, v: (batch, seqlen_k, nheads_k, headdim).  Runs on the
    varlen kernel as `batch` sequences of equal length; masks, GQA, softcap and softmax_scale as in
    flash_attn_varlen_func.  Returns out (batch, seqlen_q, nheads, headdim), or (out, softmax_lse
    (batch, nheads, seqlen_q) fp32, S_dmask (empty)) when return_attn_probs=True.
    """
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must be (batch, seqlen, nheads, headdim)"
    B, sq, hq, d = q.shape
    sk = k.shape[1]
    res = flash_attn_varlen_func(
        q.reshape(B * sq, hq, d), k.reshape(B * sk, k.shape[2], d), v.reshape(B * sk, v.shape[2], v.shape[3]),
        _even_cu_seqlens(B, sq, q.device), _even_cu_seqlens(B, sk, q.device), sq, sk, dropout_p, softmax_scale, causal,
        window_size, softcap, alibi_slopes, deterministic, return_attn_probs,
    )
    if not return_attn_probs:
        return res.reshape(B, sq, hq, -1)
    out, lse, s_dmask = res
    return out.reshape(B, sq, hq, -1), lse.reshape(hq, B, sq).permute(1, 0, 2).contiguous(), s_dmask


def flash_attn_kvpacked_func(q, kv, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1), softcap=0.0,
                             alibi_slopes=None, deterministic=False, return_attn_probs=False):
    """flash_attn_func with kv: (batch, seqlen_k, 2, nheads_k, headdim) (reference :1031-1106; forward only)."""
    return flash_attn_func(q, kv[:, :, 0], kv[:, :, 1], dropout_p, softmax_scale, causal, window_size, softcap,
                           alibi_slopes, deterministic, return_attn_probs)


def flash_attn_qkvpacked_func(qkv, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1), softcap=0.0,
                              alibi_slopes=None, deterministic=False, return_attn_probs=False):
    """flash_attn_func with qkv: (batch, seqlen, 3, nheads, headdim) (reference :972-1028; forward only)."""
    return flash_attn_func(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], dropout_p, softmax_scale, causal, window_size,
                           softcap, alibi_slopes, deterministic, return_attn_probs)


def flash_attn_varlen_kvpacked_func(q, kv, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p=0.0,
                                    softmax_scale=None, causal=False, window_size=(-1, -1), softcap=0.0,
                                    alibi_slopes=None, deterministic=False, return_attn_probs=False):
    """flash_attn_varlen_func with kv: (total_k, 2, nheads_k, headdim) (reference :1252-1341; forward only)."""
    return flash_attn_varlen_func(q, kv[:, 0], kv[:, 1], cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p,
                                  softmax_scale, causal, window_size, softcap, alibi_slopes, deterministic, return_attn_probs)


def flash_attn_varlen_qkvpacked_func(qkv, cu_seqlens, max_seqlen, dropout_p=0.0, softmax_scale=None, causal=False,
                                     window_size=(-1, -1), softcap=0.0, alibi_slopes=None, deterministic=False,
                                     return_attn_probs=False):
    """flash_attn_varlen_func with qkv: (total, 3, nheads, headdim) (reference :1186-1249; forward only)."""
    return flash_attn_varlen_func(qkv[:, 0], qkv[:, 1], qkv[:, 2], cu_seqlens, cu_seqlens, max_seqlen, max_seqlen, dropout_p,
                                  softmax_scale, causal, window_size, softcap, alibi_slopes, deterministic, return_attn_probs)


def flash_attn_with_kvcache(
    q,
    k_cache,
    v_cache,
    k=None,
    v=None,
    rotary_cos=None,
    rotary_sin=None,
    cache_seqlens: Optional[Union[(int, torch.Tensor)]] = None,
    cache_batch_idx: Optional[torch.Tensor] = None,
    cache_leftpad: Optional[torch.Tensor] = None,
    block_table: Optional[torch.Tensor] = None,
    softmax_scale=None,
    causal=False,
    window_size=(-1, -1),  # -1 means infinite context window
    softcap=0.0,  # 0.0 means deactivated
    rotary_interleaved=True,
    alibi_slopes=None,
    num_splits=0,
    return_softmax_lse=False,
    *,
    k_scale_cache: Optional[torch.Tensor] = None,
    v_scale_cache: Optional[torch.Tensor] = None,
):
    """Attention of q over a KV cache, with optional in-place append of k / v.

    q: (batch, seqlen, nheads, headdim).  k_cache / v_cache: (num_blocks, page_block_size, nheads_k,
    headdim) addressed through block_table (batch, max_num_blocks_per_seq) int32, or, without a
    block_table, (batch_cache, seqlen_cache, nheads_k, headdim) with row b of q using cache row b (or
    cache_batch_idx[b], (batch,) int32); cache_seqlens: int or (batch,) int32 keys already cached per
    row (a dense cache without it counts as full).  If k, v (batch, seqlen_new, nheads_k, headdim) are
    given they are written into the cache at positions cache_seqlens .. cache_seqlens+seqlen_new-1
    (the caller guarantees the pages exist) and attention sees cache_seqlens + seqlen_new keys;
    cache_seqlens itself is not changed.  With rotary_cos / rotary_sin (seqlen_ro, rotary_dim/2, dtype
    of q) k is rotated at those positions and q at cache_seqlens + i (causal or windowed) or at
    cache_seqlens (otherwise); rotary_interleaved pairs dims (2c, 2c+1), else (c, c + rotary_dim/2).
    GQA/MQA, bottom-right causal mask, window_size, softcap and softmax_scale (default
    headdim**-0.5) as in flash_attn_varlen_func.  num_splits: 0 = heuristic, 1 = no KV split,
    n > 1 = at most n splits.  cache_leftpad, alibi_slopes and cache_batch_idx with a block_table are
    not supported.
    An int8 k_cache (one latent kv head, 576 dims, v_cache = k_cache[..., :512]) needs
    k_scale_cache (num_blocks, page_block_size, 1) fp32 per-token scales; k (dtype of q, with
    v = k[..., :512]) is then quantised per token (scale = absmax / 127) and appended with its scale.

    Returns out (batch, seqlen, nheads, headdim_v), or (out, softmax_lse (batch, nheads, seqlen) fp32)
    when return_softmax_lse=True.  Does not support backward.
    """
    assert k_cache.stride(-1) == 1, "k_cache must have contiguous last dimension"
    assert v_cache.stride(-1) == 1, "v_cache must have contiguous last dimension"
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    if cache_seqlens is not None and isinstance(cache_seqlens, int):
        cache_seqlens = torch.full((q.shape[0],), cache_seqlens, dtype=torch.int32, device=k_cache.device)
        cache_seqlens = maybe_contiguous(cache_seqlens)
    cache_batch_idx = maybe_contiguous(cache_batch_idx)
    block_table = maybe_contiguous(block_table)
    # the registered custom op is for graph tracing; eager calls go straight to the operator layer
    fwd = _flash_attn_kvcache_forward if torch.compiler.is_compiling() else _kvcache_forward_eager
    out, softmax_lse = fwd(
        q, k_cache, v_cache, k, v, cache_seqlens, rotary_cos, rotary_sin, cache_batch_idx, cache_leftpad,
        block_table, alibi_slopes, float(softmax_scale), bool(causal), int(window_size[0]), int(window_size[1]),
        float(softcap), bool(rotary_interleaved), int(num_splits), k_scale_cache, v_scale_cache,
    )
    return (out, softmax_lse) if return_softmax_lse else out
