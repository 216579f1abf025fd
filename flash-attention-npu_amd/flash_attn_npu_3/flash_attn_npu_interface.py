"""Third-generation call surface of the KV-cache path on MI355X: `page_table`, token-major q with
`cu_seqlens_q`, explicit `num_splits` and `get_scheduler_metadata`.

Signatures, argument order, defaults and return conventions follow the reference
(flash_attn_npu_3/flash_attn_npu_interface.py:828-846 `flash_attn_func`, :911-934
`flash_attn_varlen_func`, :965-996 `flash_attn_with_kvcache`, :1129-1146 `get_scheduler_metadata`);
the checks of its host function (csrc/ascend910/flash_attn_npu_3/flash_api.cpp:104-161,216-218,
250-254,372) raise RuntimeError with the same text.  The work is done by the kernels behind
include/fa_rocm.h through the operator layer of flash_attn_npu.  Forward only.

Layouts of flash_attn_with_kvcache (tests/test_flash_attn_npu_v3.py:305-420):
  q (batch, seqlen, nheads, headdim), cache dense (batch, seqlen_cache, nheads_k, headdim) or paged
    behind `page_table`;
  q (total_q, nheads, headdim) with `cu_seqlens_q` and `max_seqlen_q`, cache paged, dense as above,
    or packed (total_k, nheads_k, headdim) holding cache_seqlens[b] keys per sequence back to back.
Differences from the reference, all additive: k / v are appended in place and rotary_cos /
rotary_sin are applied where the query blocks have one length (the reference ignores k / v and
rejects rotary, flash_api.cpp:150-151); num_splits > 1 is accepted for every paged or dense layout.

Scheduler metadata.  The reference precomputes its tiling and split plan on the device so that a
captured graph never reads lengths on the host (flash_api.cpp:506-569).  Here the kernels compute
the partition of the cached keys from cache_seqlens on the device at every launch, so a call is
capture-safe with or without metadata; the metadata tensor records the shape-dependent launch plan
and the signature of the call it was made for, and a call that passes it is checked against that
signature."""
from __future__ import annotations

import ctypes as C
from typing import Optional, Union

import torch

from flash_attn_npu import _lib
from flash_attn_npu import flash_attn_npu as _op
from flash_attn_npu.flash_attn_npu_interface import _even_cu_seqlens


def maybe_contiguous(x):
    return x.contiguous() if x is not None and x.stride(-1) != 1 else x


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _no_grad_inputs(*tensors) -> None:
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise RuntimeError("flash_attn_npu_3 (MI355X build) implements the forward only; detach the inputs")


def _max_splits(device) -> int:
    with torch.cuda.device(device):
        return int(_lib.load().fa_rocm_num_cus())


def _check_unsupported(qv, cache_leftpad, rotary_seqlens, q_descale, k_descale, v_descale, attention_chunk, pack_gqa,
                       softcap) -> None:
    # flash_api.cpp:149-161
    _require(cache_leftpad is None, "NPU FlashAttention does not support leftpad_k")
    _require(rotary_seqlens is None, "NPU FlashAttention does not support seqlens_rotary")
    _require(q_descale is None, "NPU FlashAttention does not support q_descale")
    _require(k_descale is None, "NPU FlashAttention does not support k_descale")
    _require(v_descale is None, "NPU FlashAttention does not support v_descale")
    _require(softcap >= 0.0, "softcap must be non-negative (0.0 disables softcap)")
    _require(attention_chunk == 0, "NPU FlashAttention does not support attention_chunk")
    _require(pack_gqa is None or not pack_gqa, "NPU FlashAttention does not support pack_gqa")
    _require(qv is None, "NPU FlashAttention does not support qv")


def _check_num_splits(num_splits: int, device) -> None:
    n = _max_splits(device)
    _require(0 <= num_splits <= n,
             f"NPU FlashAttention supports num_splits in [0, {n}] (0 = auto; upper bound = number of AI cores). ")


# ------------------------------------------------------------------ scheduler metadata
_META_MAGIC = 0x444D4146   # "FAMD"
_META_WORDS = 24
_META_FIELDS = ("batch", "max_seqlen_q", "num_heads_q", "num_heads_kv", "headdim", "headdim_v", "dtype", "varlen_q",
                "paged", "page_size", "causal")


def _dtype_code(dt) -> int:
    _require(dt in (torch.bfloat16, torch.float16), "FlashAttention only supports FP16 and BF16 data types")
    return _lib.FA_BF16 if dt == torch.bfloat16 else _lib.FA_FP16


def metadata_bytes() -> int:
    """Size of a scheduler-metadata record in bytes."""
    return _META_WORDS * 4


def get_scheduler_metadata(
    batch_size, max_seqlen_q, max_seqlen_k, num_heads_q, num_heads_kv, headdim,
    cache_seqlens: torch.Tensor,
    qkv_dtype=torch.bfloat16,
    headdim_v=None,
    cu_seqlens_q: Optional[torch.Tensor] = None,
    cu_seqlens_k_new: Optional[torch.Tensor] = None,
    cache_leftpad: Optional[torch.Tensor] = None,
    page_size: Optional[int] = None,
    max_seqlen_k_new=0,
    causal=False,
    window_size=(-1, -1),  # -1 means infinite context window
    attention_chunk=0,
    has_softcap=False,
    num_splits=0,    # Can be tuned for speed
    pack_gqa=None,   # Can be tuned for speed
    sm_margin=0,     # Can be tuned if some SMs are used for communication
):
    """Plan of a later flash_attn_with_kvcache / flash_attn_func / flash_attn_varlen_func call with
    these shapes, as a contiguous uint8 tensor on the device of cache_seqlens (reference
    flash_attn_npu_interface.py:1129-1169, flash_api.cpp:506-569).  Needs no host copy of the
    lengths: the split of the cached keys over the compute units is recomputed on the device from
    cache_seqlens by every launch.  The record: a tag, the call signature (batch, max_seqlen_q, head
    counts, head dimensions, dtype, layout, page size, causal) and the launch plan (mode, split
    count, keys per split, workgroups, workers, least share, workspace bytes)."""
    _require(cache_seqlens.dtype == torch.int32, "cache_seqlens must have dtype int32")
    _require(cache_seqlens.is_cuda, "cache_seqlens must be a device tensor")
    if cu_seqlens_q is not None:
        _require(cu_seqlens_q.dtype == torch.int32, "cu_seqlens_q must have dtype int32")
    _check_num_splits(int(num_splits), cache_seqlens.device)
    if headdim_v is None:
        headdim_v = headdim
    lib = _lib.load()
    a = _lib.KvcacheArgs()
    ps = int(page_size) if page_size is not None else max(int(max_seqlen_k), 1)
    a.batch, a.seqlen_q, a.nheads, a.nheads_k = int(batch_size), int(max_seqlen_q), int(num_heads_q), int(num_heads_kv)
    a.headdim_qk, a.headdim_v = int(headdim), int(headdim_v)
    a.page_size = ps
    a.max_blocks_per_seq = (int(max_seqlen_k) + ps - 1) // ps if page_size is not None else 1
    a.num_blocks = a.max_blocks_per_seq * int(batch_size)
    a.seqlen_new = int(max_seqlen_k_new)
    a.io_dtype = a.kv_dtype = _dtype_code(qkv_dtype)
    a.causal = int(bool(causal))
    a.window_left, a.window_right = int(window_size[0]), int(window_size[1])
    a.num_splits = int(num_splits)
    plan = _lib.SplitPlan()
    with torch.cuda.device(cache_seqlens.device):
        _lib.check(lib.fa_rocm_plan_kvcache(C.byref(a), lib.fa_rocm_num_cus(), C.byref(plan)))
    words = [0] * _META_WORDS
    words[0], words[1] = _META_MAGIC, lib.fa_rocm_abi_version()
    sig = (int(batch_size), int(max_seqlen_q), int(num_heads_q), int(num_heads_kv), int(headdim), int(headdim_v),
           _dtype_code(qkv_dtype), int(cu_seqlens_q is not None), int(page_size is not None),
           int(page_size) if page_size is not None else 0, int(bool(causal)))
    words[2:2 + len(sig)] = sig
    words[13] = int(num_splits)
    words[14:20] = [plan.mode, plan.nsplits, plan.split_keys, plan.num_wgs, plan.num_workers, plan.min_share]
    words[20], words[21] = plan.workspace_bytes & 0x7FFFFFFF, plan.workspace_bytes >> 31
    host = torch.tensor(words, dtype=torch.int32).view(torch.uint8)
    meta = host.to(cache_seqlens.device, non_blocking=False)
    meta._fa_signature = dict(zip(_META_FIELDS, sig))   # host copy: a call never reads the device record back
    return meta


def _check_metadata(meta, *, batch, max_seqlen_q, num_heads_q, num_heads_kv, headdim, headdim_v, dtype, varlen_q, paged,
                    page_size, causal) -> None:
    # flash_api.cpp:250-254
    _require(meta.dtype == torch.uint8, "scheduler_metadata must be a byte tensor")
    _require(meta.is_contiguous(), "scheduler_metadata must be contiguous")
    _require(meta.is_cuda, "scheduler_metadata must be a device tensor")
    _require(meta.numel() >= metadata_bytes(), "scheduler_metadata buffer is too small for this call's causal flag")
    sig = getattr(meta, "_fa_signature", None)
    if sig is None:
        return   # a copy of a record: its content is not read back on the host
    now = dict(batch=batch, max_seqlen_q=max_seqlen_q, num_heads_q=num_heads_q, num_heads_kv=num_heads_kv, headdim=headdim,
               headdim_v=headdim_v, dtype=_dtype_code(dtype), varlen_q=int(varlen_q), paged=int(paged),
               page_size=page_size if paged else 0, causal=int(bool(causal)))
    bad = [k for k in _META_FIELDS if sig[k] != now[k]]
    _require(not bad, "scheduler_metadata was computed for a different call: " +
             ", ".join(f"{k} {sig[k]} != {now[k]}" for k in bad))


# ------------------------------------------------------------------ dense and varlen forward
def _empty_accum(device):
    return torch.empty((0,), device=device), torch.empty((0,), device=device)


def flash_attn_func(
    q,
    k,
    v,
    softmax_scale=None,
    causal=False,
    qv=None,
    q_descale=None, k_descale=None, v_descale=None,
    window_size=(-1, -1),
    attention_chunk=0,
    softcap=0.0,
    num_splits=1,
    pack_gqa=None,
    deterministic=False,
    sm_margin=0,
    return_attn_probs=False,
    scheduler_metadata=None,
):
    """Attention forward over dense batches (reference flash_attn_npu_interface.py:828-908; forward only).

    q: (batch, seqlen_q, nheads, headdim); k, v: (batch, seqlen_k, nheads_k, headdim).  GQA/MQA,
    bottom-right causal mask, window_size and softcap as in flash_attn_with_kvcache.  Returns out, or
    (out, softmax_lse (batch, nheads, seqlen_q) fp32) when return_attn_probs=True."""
    _check_unsupported(qv, None, None, q_descale, k_descale, v_descale, attention_chunk, pack_gqa, softcap)
    _no_grad_inputs(q, k, v)
    _require(q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must be (batch, seqlen, nheads, headdim)")
    _check_num_splits(int(num_splits), q.device)
    _require(num_splits <= 1, "NPU FlashAttention num_splits>1 currently requires paged KV cache and varlen-q (TND) layout")
    B, sq, hq, d = q.shape
    sk, hk = k.shape[1], k.shape[2]
    if scheduler_metadata is not None:
        _check_metadata(scheduler_metadata, batch=B, max_seqlen_q=sq, num_heads_q=hq, num_heads_kv=hk, headdim=d,
                        headdim_v=v.shape[-1], dtype=q.dtype, varlen_q=False, paged=False, page_size=0, causal=causal)
    if softmax_scale is None:
        softmax_scale = d ** (-0.5)
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    out, lse, _, _ = _op.varlen_fwd(
        q.reshape(B * sq, hq, d), k.reshape(B * sk, hk, d), v.reshape(B * sk, hk, v.shape[-1]), None,
        _even_cu_seqlens(B, sq, q.device), _even_cu_seqlens(B, sk, q.device), None, None, None, None, sq, sk, 0.0,
        float(softmax_scale), False, bool(causal), int(window_size[0]), int(window_size[1]), float(softcap), False, None)
    out = out.reshape(B, sq, hq, -1)
    if not return_attn_probs:
        return out
    return out, lse.reshape(hq, B, sq).permute(1, 0, 2).contiguous()


def flash_attn_varlen_func(
    q,
    k,
    v,
    cu_seqlens_q,
    cu_seqlens_k,
    max_seqlen_q,
    max_seqlen_k,
    seqused_q=None,
    seqused_k=None,
    softmax_scale=None,
    causal=False,
    qv=None,
    q_descale=None, k_descale=None, v_descale=None,
    window_size=(-1, -1),
    attention_chunk=0,
    softcap=0.0,
    num_splits=1,
    pack_gqa=None,
    deterministic=False,
    sm_margin=0,
    return_attn_probs=False,
    scheduler_metadata=None,
):
    """Variable-length attention forward over packed sequences (reference
    flash_attn_npu_interface.py:911-958; forward only).  q: (total_q, nheads, headdim); k, v:
    (total_k, nheads_k, headdim); cu_seqlens_*: (batch+1,) int32.  Returns out, or (out, softmax_lse
    (nheads, total_q) fp32) when return_attn_probs=True.  seqused_k (batch,) int32: sequence b uses only the first
    seqused_k[b] of its cu_seqlens_k[b+1] - cu_seqlens_k[b] keys (the length vector of the reference's host,
    csrc/ascend910/flash_attn_npu_3/flash_api.cpp:143-147); the mask is aligned to that length.  seqused_q is not
    supported (the reference's host accepts and ignores it, flash_api.cpp:71)."""
    _check_unsupported(qv, None, None, q_descale, k_descale, v_descale, attention_chunk, pack_gqa, softcap)
    _no_grad_inputs(q, k, v)
    _require(seqused_q is None, "NPU FlashAttention (MI355X build) does not support seqused_q")
    if seqused_k is not None:
        _require(seqused_k.dtype == torch.int32, "seqused_k must have dtype int32")   # flash_api.cpp:146
    _require(cu_seqlens_q is not None and cu_seqlens_q.dtype == torch.int32, "cu_seqlens_q must have dtype int32")
    _require(cu_seqlens_k is not None and cu_seqlens_k.dtype == torch.int32, "cu_seqlens_k must have dtype int32")
    _require(max_seqlen_q is not None, "max_seqlen_q must be provided if cu_seqlens_q is provided")
    _check_num_splits(int(num_splits), q.device)
    _require(num_splits <= 1, "NPU FlashAttention num_splits>1 currently requires paged KV cache and varlen-q (TND) layout")
    if scheduler_metadata is not None:
        _check_metadata(scheduler_metadata, batch=cu_seqlens_q.numel() - 1, max_seqlen_q=int(max_seqlen_q),
                        num_heads_q=q.shape[1], num_heads_kv=k.shape[1], headdim=q.shape[2], headdim_v=v.shape[2],
                        dtype=q.dtype, varlen_q=True, paged=False, page_size=0, causal=causal)
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    out, lse, _, _ = _op._varlen_fwd(
        q, k, v, None, cu_seqlens_q, cu_seqlens_k, seqused_k, None, None, None, int(max_seqlen_q), int(max_seqlen_k), 0.0,
        float(softmax_scale), False, bool(causal), int(window_size[0]), int(window_size[1]), float(softcap), False, None)
    return (out, lse) if return_attn_probs else out


def flash_attn_combine(out_partial, lse_partial, out=None, out_dtype=None):
    """Merge of split-KV partial results (reference flash_attn_npu_interface.py:961-962).  The
    reference forwards to an extension function that its host library does not define
    (csrc/ascend910/flash_attn_npu_3/flash_api.cpp:829-835 registers fwd, bwd and
    get_scheduler_metadata only); the kernels here merge their partials inside the call, so there is
    nothing for a caller to combine."""
    raise RuntimeError("flash_attn_combine: split-KV partials are merged inside flash_attn_with_kvcache; "
                       "the library exports no separate combine")


# ------------------------------------------------------------------ KV cache
def flash_attn_with_kvcache(
    q,
    k_cache,
    v_cache,
    k=None,
    v=None,
    qv=None,
    rotary_cos=None,
    rotary_sin=None,
    cache_seqlens: Optional[Union[(int, torch.Tensor)]] = None,
    cache_batch_idx: Optional[torch.Tensor] = None,
    cache_leftpad: Optional[torch.Tensor] = None,
    page_table: Optional[torch.Tensor] = None,
    cu_seqlens_q: Optional[torch.Tensor] = None,
    cu_seqlens_k_new: Optional[torch.Tensor] = None,
    max_seqlen_q: Optional[int] = None,
    rotary_seqlens: Optional[torch.Tensor] = None,
    q_descale: Optional[torch.Tensor] = None,
    k_descale: Optional[torch.Tensor] = None,
    v_descale: Optional[torch.Tensor] = None,
    softmax_scale=None,
    causal=False,
    window_size=(-1, -1),  # -1 means infinite context window
    attention_chunk=0,
    softcap=0.0,  # 0.0 means deactivated
    rotary_interleaved=True,
    scheduler_metadata=None,
    num_splits=0,    # Can be tuned for speed
    pack_gqa=None,   # Can be tuned for speed
    sm_margin=0,     # Can be tuned if some SMs are used for communication
    return_softmax_lse=False,
):
    """Attention of q over a KV cache, with optional in-place append of k / v.

    q: (batch, seqlen, nheads, headdim), or (total_q, nheads, headdim) with cu_seqlens_q (batch+1,)
    int32 and max_seqlen_q.  k_cache / v_cache: (num_blocks, page_block_size, nheads_k, headdim)
    addressed through page_table (batch, max_num_blocks_per_seq) int32; or dense (batch_cache,
    seqlen_cache, nheads_k, headdim), row b of q using cache row b (or cache_batch_idx[b]); or, with
    token-major q only, packed (total_k, nheads_k, headdim) with the cache_seqlens[b] keys of
    sequence b back to back.  cache_seqlens: int or (batch,) int32, the keys cached per sequence.
    k, v (batch, seqlen_new, nheads_k, headdim): written into the cache at positions cache_seqlens ..
    cache_seqlens + seqlen_new - 1 before attention, which then sees cache_seqlens + seqlen_new
    keys; rotary_cos / rotary_sin (seqlen_ro, rotary_dim / 2) rotate k at those positions and q at
    cache_seqlens + i (causal or windowed) or cache_seqlens (otherwise).  Appending needs query
    blocks of one length (batch-major q, or total_q == batch * max_seqlen_q).
    GQA/MQA by head count; causal is aligned to the bottom right corner; window_size = (left, right)
    keeps keys in [i + seqlen_k - seqlen_q - left, i + seqlen_k - seqlen_q + right], a side at least
    as long as the longest cached sequence counts as unbounded; rows with no visible key give 0.
    num_splits: 0 = balanced split of the cached keys over all compute units, 1 = no split, n > 1 =
    at most n splits per sequence.  scheduler_metadata: a record from get_scheduler_metadata for
    this call's shapes (checked, see the module text).  qv, cache_leftpad, cu_seqlens_k_new,
    rotary_seqlens, the descale tensors, attention_chunk and pack_gqa=True are not supported.

    Returns out (the shape of q with headdim_v), or (out, softmax_lse, out_accum, softmax_lse_accum)
    when return_softmax_lse=True: softmax_lse fp32 (batch, nheads, seqlen) or (nheads, total_q), the
    two accumulators empty (partials live in a workspace of the call)."""
    assert k_cache.stride(-1) == 1, "k_cache must have contiguous last dimension"
    assert v_cache.stride(-1) == 1, "v_cache must have contiguous last dimension"
    _check_unsupported(qv, cache_leftpad, rotary_seqlens, q_descale, k_descale, v_descale, attention_chunk, pack_gqa,
                       softcap)
    _require(cu_seqlens_k_new is None, "NPU FlashAttention (MI355X build) does not support cu_seqlens_k_new")
    _require(q.dtype in (torch.bfloat16, torch.float16), "FlashAttention only supports FP16 and BF16 data types")
    _require(k_cache.dtype == q.dtype, "query and key must have the same dtype")
    _require(v_cache.dtype == q.dtype, "query and value must have the same dtype")
    _require(q.is_cuda, "flash_attn_npu_3 (MI355X build) needs tensors on a ROCm device; there is no CPU path")
    _check_num_splits(int(num_splits), q.device)
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    paged = page_table is not None
    varlen_q = cu_seqlens_q is not None
    if paged:
        _require(page_table.dtype == torch.int32, "page_table must have dtype int32")
        _require(page_table.stride(-1) == 1, "page_table must have contiguous last dimension")
    if varlen_q:
        _require(cu_seqlens_q.dtype == torch.int32, "cu_seqlens_q must have dtype int32")
        _require(cu_seqlens_q.is_contiguous(), "cu_seqlens_q must be contiguous")
        _require(max_seqlen_q is not None, "max_seqlen_q must be provided if cu_seqlens_q is provided")
        _require(q.dim() == 3, "q must be (total_q, nheads, headdim) when cu_seqlens_q is given")
        batch = cu_seqlens_q.numel() - 1
    else:
        _require(q.dim() == 4, "q must be (batch_size, seqlen, nheads, headdim)")
        batch = q.shape[0]
    _require(batch > 0, "batch size must be positive")
    _require(q.shape[-1] <= 256, "FlashAttention only supports head dimension at most 256")
    if cache_seqlens is not None and isinstance(cache_seqlens, int):
        cache_seqlens = torch.full((batch,), cache_seqlens, dtype=torch.int32, device=k_cache.device)
    if cache_seqlens is not None:
        _require(cache_seqlens.dtype == torch.int32, "seqused_k must have dtype int32")
    if scheduler_metadata is not None:
        _check_metadata(scheduler_metadata, batch=batch, max_seqlen_q=int(max_seqlen_q) if varlen_q else q.shape[1],
                        num_heads_q=q.shape[-2], num_heads_kv=k_cache.shape[-2], headdim=q.shape[-1],
                        headdim_v=v_cache.shape[-1], dtype=q.dtype, varlen_q=varlen_q, paged=paged,
                        page_size=k_cache.shape[1] if paged else 0, causal=causal)
    wl, wr = int(window_size[0]), int(window_size[1])
    common = (float(softmax_scale), bool(causal), wl, wr, float(softcap), bool(rotary_interleaved), int(num_splits))

    if not varlen_q:
        _require(k_cache.dim() == 4, "k_cache must be 4-D when q is (batch_size, seqlen, nheads, headdim)")
        out, lse = _op.fwd_kvcache(q, k_cache, v_cache, k, v, cache_seqlens, rotary_cos, rotary_sin, cache_batch_idx,
                                   None, page_table, None, None, *common)
    elif k_cache.dim() == 4 and q.shape[0] == batch * int(max_seqlen_q):
        # every query block has max_seqlen_q rows (each is at most that long and they sum to
        # batch * max_seqlen_q): the batch-major kernels run on a view of q
        sq = int(max_seqlen_q)
        out4, lse4 = _op.fwd_kvcache(q.view(batch, sq, q.shape[1], q.shape[2]), k_cache, v_cache, k, v, cache_seqlens,
                                     rotary_cos, rotary_sin, cache_batch_idx, None, page_table, None, None, *common)
        out = out4.view(batch * sq, q.shape[1], -1)
        lse = lse4.permute(1, 0, 2).reshape(q.shape[1], batch * sq)
    else:
        # ragged query blocks: the tiled kernel, which reads paged or packed keys
        _require(k is None and v is None, "appending k / v needs query blocks of one length")
        _require(rotary_cos is None and rotary_sin is None, "rotary embedding needs query blocks of one length")
        _require(cache_seqlens is not None and cache_seqlens.shape[0] == batch, "cache_seqlens must be (batch_size,) int32")
        if k_cache.dim() == 4:
            if paged:
                table = page_table
            elif cache_batch_idx is not None:
                _require(cache_batch_idx.dtype == torch.int32 and cache_batch_idx.shape[0] == batch,
                         "cache_batch_idx must be (batch_size,) int32")
                table = cache_batch_idx.contiguous().view(-1, 1)
            else:
                _require(k_cache.shape[0] >= batch, "batch size of the cache must be at least that of q")
                table = _op._identity_table(batch, q.device)
            _require(k_cache.shape[1] % 32 == 0 or table.shape[1] == 1, "page_block_size must be a positive multiple of 32")
            out, lse, _, _ = _op.varlen_fwd(q, k_cache, v_cache, None, cu_seqlens_q, None, cache_seqlens, None, table, None,
                                            int(max_seqlen_q), 0, 0.0, common[0], False, common[1], wl, wr, common[4],
                                            False, None, num_splits=common[6])
        else:
            _require(k_cache.dim() == 3 and not paged, "a packed cache must be (total_k, nheads_k, headdim) without page_table")
            _require(cache_batch_idx is None, "cache_batch_idx needs a dense (batch_cache, seqlen_cache, ...) cache")
            cu_k = torch.zeros(batch + 1, dtype=torch.int32, device=q.device)
            cu_k[1:] = torch.cumsum(cache_seqlens, 0)
            # the window sides are measured against the longest sequence (flash_api.cpp:300-306); it is
            # read back only when a window was asked for
            max_k = int(cache_seqlens.max()) if (wl >= 0 or wr >= 0) else k_cache.shape[0]
            out, lse, _, _ = _op.varlen_fwd(q, k_cache, v_cache, None, cu_seqlens_q, cu_k, None, None, None, None,
                                            int(max_seqlen_q), max(max_k, 1), 0.0, common[0], False, common[1], wl, wr,
                                            common[4], False, None)
    if not return_softmax_lse:
        return out
    return (out, lse) + _empty_accum(q.device)
