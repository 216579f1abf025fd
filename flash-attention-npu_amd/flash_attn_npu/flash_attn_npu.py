"""Operator layer: `fwd_kvcache` and `varlen_fwd` with the argument order of the reference's
extension module (csrc/ascend910/flash_attn_npu/flash_api.cpp:356-377, :848-869, exported at
:1335-1336).  Both are the compiled extension module `flash_attn_npu._C` (csrc/torch_binding.cpp: checks, argument
record, allocation and the call into the C ABI of libfa_rocm.so, all in C++); what stays in Python here is the
padded-copy path for head dimensions that are not multiples of 8, and `bind_kvcache` / `KvcacheCall`, a ctypes
binding of one call that can be run many times (benchmarks, graph capture).

Checks that the reference performs with TORCH_CHECK raise RuntimeError with the same text.
There is no fallback: tensors must live on a ROCm device and both the library and the module must be built."""
from __future__ import annotations

import ctypes as C
from typing import List, Optional

import torch

from . import _lib

_DT = {torch.bfloat16: _lib.FA_BF16, torch.float16: _lib.FA_FP16, torch.int8: _lib.FA_INT8}


_ext = None


def _C():
    """The compiled extension module; a missing build is an error, never a slower path."""
    global _ext
    if _ext is None:
        _lib.load()
        try:
            from . import _C as ext
        except ImportError as e:
            raise RuntimeError("flash_attn_npu._C (the compiled operator layer) is not built: run "
                               "`python flash-attention-npu_amd/build.py`; there is no CPU or PyTorch fallback") from e
        _ext = ext
    return _ext


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream(t: torch.Tensor):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _require_device(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("flash_attn_npu (MI355X build) needs tensors on a ROCm device; there is no CPU path")


class KvcacheCall:
    """One validated, fully bound kvcache call: the argument record, the output tensors and the
    tensors that must stay alive.  `run()` enqueues it on the current stream; a serving loop or a
    benchmark can bind once and run many times (the record holds raw pointers)."""

    def __init__(self, args, out, lse, keep, device):
        self.args, self.out, self.lse, self.keep, self.device = args, out, lse, keep, device

    def run(self, events=None) -> None:
        lib = _lib.load()
        with torch.cuda.device(self.device):
            stream = C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
            if events is None:
                _lib.check(lib.fa_rocm_fwd_kvcache(C.byref(self.args), stream))
            else:
                _lib.check(lib.fa_rocm_fwd_kvcache_profiled(C.byref(self.args), stream, events))


def fwd_kvcache(q, kcache, vcache, k_, v_, seqlens_k_, rotary_cos_, rotary_sin_, cache_batch_idx_, leftpad_k_,
                block_table_, alibi_slopes_, out_, softmax_scale, is_causal, window_size_left, window_size_right,
                softcap, is_rotary_interleaved, num_splits, k_scale_cache_=None, v_scale_cache_=None
                ) -> List[torch.Tensor]:
    """mha_fwd_kvcache (flash_api.cpp:356-637) on a paged cache.  Returns [out, softmax_lse]."""
    if (isinstance(q, torch.Tensor) and q.dim() == 4 and kcache.dtype != torch.int8
            and q.shape[-1] % 8 != 0 and q.shape[-1] <= 256 and q.shape[-1] == kcache.shape[-1]
            and q.dtype in (torch.bfloat16, torch.float16) and q.is_cuda and kcache.is_cuda):
        return _fwd_kvcache_padded(q, kcache, vcache, k_, v_, seqlens_k_, rotary_cos_, rotary_sin_, cache_batch_idx_,
                                   leftpad_k_, block_table_, alibi_slopes_, out_, softmax_scale, is_causal,
                                   window_size_left, window_size_right, softcap, is_rotary_interleaved, num_splits)
    return _C().fwd_kvcache(q, kcache, vcache, k_, v_, seqlens_k_, rotary_cos_, rotary_sin_, cache_batch_idx_, leftpad_k_,
                            block_table_, alibi_slopes_, out_, softmax_scale, is_causal, window_size_left, window_size_right,
                            softcap, is_rotary_interleaved, num_splits, k_scale_cache_, v_scale_cache_)


# Head dimensions that are not multiples of 8 are served through zero-padded COPIES (rows of such widths are not made of
# 16-byte pieces).  For q, k, v of a packed batch that is what the reference's front end does as well
# (flash_attn_npu_interface.py:897-901); for a KV cache it means copying the cache on every call, which is only
# acceptable while the cache is small (the reference's own test shapes with D = 1, 4, 111 are a few MB).  Beyond this many
# bytes (K and V caches together) the call is refused with a message that says what to do instead.
PADDED_CACHE_COPY_LIMIT = 256 << 20


def _check_padded_cache_copy(kcache, vcache) -> None:
    nbytes = kcache.numel() * kcache.element_size() + vcache.numel() * vcache.element_size()
    _require(nbytes <= PADDED_CACHE_COPY_LIMIT,
             f"head dimension {kcache.shape[-1]} is not a multiple of 8: this build serves such a KV cache through a zero-padded copy "
             f"of the whole cache on every call, and refuses to do that for {nbytes} bytes of cache (limit {PADDED_CACHE_COPY_LIMIT}). "
             "Allocate the cache with the head dimension rounded up to a multiple of 8 and zero columns behind the real ones "
             "(they change neither the scores nor the kept output columns), and pass q / k / v padded the same way")


def _fwd_kvcache_padded(q, kcache, vcache, k_, v_, seqlens_k_, rotary_cos_, rotary_sin_, cache_batch_idx_, leftpad_k_,
                        block_table_, alibi_slopes_, out_, softmax_scale, is_causal, window_size_left,
                        window_size_right, softcap, is_rotary_interleaved, num_splits) -> List[torch.Tensor]:
    """Head dimensions that are not a multiple of 8 (the reference's tests go down to 1 and 4,
    tests/test_flash_attn_npu_v2.py:178-183; every multiple of 8 up to 256 runs on the caller's cache as it is): the
    rows are not 16-byte pieces, so zero-padded COPIES of q and of the caches, to the next multiple of 8, go through
    the kernels (zero columns change neither the scores nor the kept output columns), then the rows the call
    appended are copied back into the caller's caches.  A slow path: it copies the whole cache."""
    import torch.nn.functional as F
    d, dv = q.shape[-1], vcache.shape[-1]
    dp = (max(d, dv) + 7) // 8 * 8
    _require(kcache.dim() == 4 and vcache.dim() == 4, "q, kcache and vcache must be 4-D")
    _require(dv == d, "k and v head dimensions must match")
    _check_padded_cache_copy(kcache, vcache)

    def pad(x):
        return None if x is None else F.pad(x, (0, dp - x.shape[-1]))

    kc_p, vc_p = pad(kcache), pad(vcache)
    out_p, lse = fwd_kvcache(pad(q), kc_p, vc_p, pad(k_), pad(v_), seqlens_k_, rotary_cos_, rotary_sin_,
                             cache_batch_idx_, leftpad_k_, block_table_, alibi_slopes_, None, softmax_scale, is_causal,
                             window_size_left, window_size_right, softcap, is_rotary_interleaved, num_splits)
    if k_ is not None:
        # positions the call wrote, computed on the device (no host sync); rows without capacity are
        # redirected to the first written row with that row's values, so duplicates agree
        B, snew = k_.shape[0], k_.shape[1]
        page, nblk = kcache.shape[1], kcache.shape[0]
        if block_table_ is None:
            table = (cache_batch_idx_.view(-1, 1) if cache_batch_idx_ is not None else _identity_table(B, q.device))
        else:
            table = block_table_
        pos = seqlens_k_.to(torch.int64).view(B, 1) + torch.arange(snew, device=q.device, dtype=torch.int64).view(1, snew)
        pg = pos // page
        blk = table.to(torch.int64).gather(1, pg.clamp(max=table.shape[1] - 1))
        ok = ((pg < table.shape[1]) & (blk >= 0) & (blk < nblk)).view(-1)
        n = ok.numel()
        first = torch.argmax(ok.to(torch.int32))
        sel = torch.where(ok, torch.arange(n, device=q.device), first)
        blk_s = blk.view(-1)[sel].clamp(0, nblk - 1)
        row_s = (pos % page).view(-1)[sel]
        any_ok = ok.any()
        for cache, cache_p, width in ((kcache, kc_p, d), (vcache, vc_p, dv)):
            new = cache_p[blk_s, row_s][..., :width]
            cache[blk_s, row_s] = torch.where(any_ok, new, cache[blk_s, row_s])
    out = out_p[..., :dv]
    if out_ is not None:
        _require(out_.dtype == q.dtype and tuple(out_.shape) == tuple(out.shape),
                 "out must have shape (batch_size, seqlen_q, num_heads, head_size_v) and the dtype of q")
        out_.copy_(out)
        out = out_
    else:
        out = out.contiguous()
    return [out, lse]


# Small constant tensors, one per (shape, device), never evicted: a captured HIP graph may hold
# their addresses long after the call that made them.
_tables = {}


def _identity_table(batch: int, device) -> torch.Tensor:
    """(batch, 1) int32 table 0..batch-1, built once per (device, batch)."""
    key = ("id", batch, str(device))
    if key not in _tables:
        _tables[key] = torch.arange(batch, dtype=torch.int32, device=device).view(batch, 1)
    return _tables[key]


def _full_lengths(batch: int, seqlen: int, device) -> torch.Tensor:
    key = ("len", batch, seqlen, str(device))
    if key not in _tables:
        _tables[key] = torch.full((batch,), seqlen, dtype=torch.int32, device=device)
    return _tables[key]


def bind_kvcache(q, kcache, vcache, k_, v_, seqlens_k_, rotary_cos_, rotary_sin_, cache_batch_idx_, leftpad_k_,
                 block_table_, alibi_slopes_, out_, softmax_scale, is_causal, window_size_left, window_size_right,
                 softcap, is_rotary_interleaved, num_splits, k_scale_cache_=None, v_scale_cache_=None) -> KvcacheCall:
    """Checks of mha_fwd_kvcache (flash_api.cpp:386-420,455-457) and binding of the C argument record."""
    lib = _lib.load()
    is_i8 = kcache.dtype == torch.int8
    _require(q.dtype in (torch.bfloat16, torch.float16), "FlashAttention only supports FP16 and BF16 data types")
    if not is_i8:
        _require(kcache.dtype == q.dtype, "query and key_cache must have the same dtype")
        _require(vcache.dtype == q.dtype, "query and value_cache must have the same dtype")
    else:
        _require(vcache.dtype == torch.int8, "key_cache and value_cache must have the same dtype")
        _require(k_scale_cache_ is not None, "int8 KV cache needs k_scale_cache")
    _require(q.stride(-1) == 1, "Input tensor q must have contiguous last dimension")
    _require(kcache.stride(-1) == 1, "Input tensor kcache must have contiguous last dimension")
    _require(vcache.stride(-1) == 1, "Input tensor vcache must have contiguous last dimension")
    # A dense cache (batch_cache, seqlen_cache, nheads_k, headdim) is a paged one with a single page
    # per row: the table is the identity, or cache_batch_idx (flash_attn_npu_interface.py:1516-1519).
    dense = block_table_ is None
    if dense:
        _require(q.dim() == 4 and kcache.dim() == 4, "q, kcache and vcache must be 4-D")
        if cache_batch_idx_ is not None:
            _require(cache_batch_idx_.dtype == torch.int32 and cache_batch_idx_.dim() == 1
                     and cache_batch_idx_.shape[0] == q.shape[0], "cache_batch_idx must be (batch_size,) int32")
            block_table_ = cache_batch_idx_.contiguous().view(-1, 1)
        else:
            _require(kcache.shape[0] >= q.shape[0], "batch size of the cache must be at least that of q")
            block_table_ = _identity_table(q.shape[0], q.device)
        if seqlens_k_ is None:
            _require(k_ is None, "cache_seqlens must be given to append k / v")
            seqlens_k_ = _full_lengths(q.shape[0], kcache.shape[1], q.device)
    else:
        _require(cache_batch_idx_ is None, "Paged KVcache does not support cache_batch_idx")
    _require(block_table_.dtype == torch.int32, "block_table must have dtype int32")
    _require(block_table_.dim() == 2, "block_table must be (batch_size, max_num_blocks_per_seq)")
    _require(block_table_.stride(-1) == 1, "block_table must have contiguous last dimension")
    _require(seqlens_k_ is not None, "cache_seqlens must be given with a paged KV cache")
    _require(seqlens_k_.dtype == torch.int32, "seqlens_k must have dtype int32")
    _require(seqlens_k_.dim() == 1, "seqlens_k must be (batch_size,)")
    _require(alibi_slopes_ is None, "NPU FlashAttention does not support alibi_slopes")
    _require(leftpad_k_ is None, "NPU FlashAttention does not support leftpad_k")
    _require(softcap >= 0.0, "softcap must be non-negative (0.0 disables softcap)")
    _require(q.dim() == 4 and kcache.dim() == 4 and vcache.dim() == 4, "q, kcache and vcache must be 4-D")
    # the rotation is part of the append (positions cache_seqlens .. + seqlen_new of q and k); without new tokens the
    # tables would be silently unused
    _require((k_ is not None or v_ is not None) or (rotary_cos_ is None and rotary_sin_ is None),
             "rotary_cos / rotary_sin are only applied together with new k / v")
    _require_device(q, kcache, vcache, k_, v_, seqlens_k_, block_table_, rotary_cos_, rotary_sin_)

    B, sq, hq, d = q.shape
    num_blocks, page, hk, dk = kcache.shape
    dv = vcache.shape[-1]
    _require(B > 0, "batch size must be positive")
    _require(d == dk, "q and kcache must have the same head dimension")
    _require(tuple(vcache.shape[:3]) == (num_blocks, page, hk),
             "vcache must have the num_blocks, page_block_size and nheads_k of kcache")
    _require(hq % hk == 0, "Number of heads in key/value must divide number of heads in query")
    _require(block_table_.shape[0] == B and seqlens_k_.shape[0] == B, "block_table / cache_seqlens batch mismatch")
    seqlens_k = seqlens_k_.contiguous()

    if out_ is not None:
        out = out_
        _require(out.dtype == q.dtype and tuple(out.shape) == (B, sq, hq, dv) and out.stride(-1) == 1,
                 "out must have shape (batch_size, seqlen_q, num_heads, head_size_v) and the dtype of q")
    else:
        out = torch.empty((B, sq, hq, dv), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, hq, sq), dtype=torch.float32, device=q.device)

    a = _lib.KvcacheArgs()
    a.q, a.out, a.softmax_lse = _ptr(q), _ptr(out), _ptr(lse)
    a.k_cache, a.v_cache = _ptr(kcache), _ptr(vcache)
    a.k_scale_cache, a.v_scale_cache = _ptr(k_scale_cache_), _ptr(v_scale_cache_)
    a.cache_seqlens, a.block_table = _ptr(seqlens_k), _ptr(block_table_)
    a.batch, a.seqlen_q, a.nheads, a.nheads_k = B, sq, hq, hk
    a.headdim_qk, a.headdim_v = d, dv
    a.num_blocks, a.page_size, a.max_blocks_per_seq = num_blocks, page, block_table_.shape[1]
    a.q_stride_b, a.q_stride_s, a.q_stride_h = q.stride(0), q.stride(1), q.stride(2)
    a.o_stride_b, a.o_stride_s, a.o_stride_h = out.stride(0), out.stride(1), out.stride(2)
    a.k_stride_block, a.k_stride_row, a.k_stride_h = kcache.stride(0), kcache.stride(1), kcache.stride(2)
    a.v_stride_block, a.v_stride_row, a.v_stride_h = vcache.stride(0), vcache.stride(1), vcache.stride(2)
    a.bt_stride_b = block_table_.stride(0)
    if k_scale_cache_ is not None:
        _require(k_scale_cache_.dtype == torch.float32 and k_scale_cache_.dim() == 3 and k_scale_cache_.stride(-1) == 1
                 and tuple(k_scale_cache_.shape) == (num_blocks, page, hk) and k_scale_cache_.is_cuda,
                 "k_scale_cache must be fp32 (num_blocks, page_block_size, nheads_k)")
        a.ks_stride_block, a.ks_stride_row = k_scale_cache_.stride(0), k_scale_cache_.stride(1)
        if v_scale_cache_ is not None:
            _require(v_scale_cache_.stride() == k_scale_cache_.stride() and v_scale_cache_.dtype == torch.float32
                     and v_scale_cache_.shape == k_scale_cache_.shape and v_scale_cache_.is_cuda,
                     "v_scale_cache must match k_scale_cache's layout")
    keep = [q, kcache, vcache, seqlens_k, block_table_, k_scale_cache_, v_scale_cache_]
    if k_ is not None or v_ is not None:
        _require(k_ is not None and v_ is not None, "k and v must be passed together")
        _require(k_.dtype == q.dtype and v_.dtype == q.dtype, "Key and value must have the same dtype as query")
        _require(k_.dim() == 4 and k_.shape[0] == B and k_.shape[2] == hk and k_.shape[3] == d
                 and tuple(v_.shape) == (B, k_.shape[1], hk, dv), "k / v must be (batch_size, seqlen_new, nheads_k, headdim)")
        if is_i8:
            # quantising append: the new latent rows come in the I/O dtype, v aliased like the cache
            _require(k_.stride(-1) == 1 and v_.data_ptr() == k_.data_ptr() and v_.stride() == k_.stride(),
                     "int8 KV cache: v must be the view k[..., :512] of the new latent rows")
            _require(rotary_cos_ is None and rotary_sin_ is None, "rotary embedding is not supported with an int8 KV cache")
        k_ = k_ if k_.stride(-1) == 1 else k_.contiguous()
        v_ = v_ if v_.stride(-1) == 1 else v_.contiguous()
        keep += [k_, v_]
        a.k_new, a.v_new, a.seqlen_new = _ptr(k_), _ptr(v_), k_.shape[1]
        a.kn_stride_b, a.kn_stride_s, a.kn_stride_h = k_.stride(0), k_.stride(1), k_.stride(2)
        a.vn_stride_b, a.vn_stride_s, a.vn_stride_h = v_.stride(0), v_.stride(1), v_.stride(2)
        if rotary_cos_ is not None or rotary_sin_ is not None:
            _require(rotary_cos_ is not None and rotary_sin_ is not None, "rotary_cos and rotary_sin must be passed together")
            _require(rotary_cos_.dtype == q.dtype and rotary_sin_.dtype == q.dtype,
                     "rotary_cos / rotary_sin must have the same dtype as query")
            _require(rotary_cos_.dim() == 2 and rotary_cos_.shape == rotary_sin_.shape, "rotary_cos / rotary_sin must be (seqlen_ro, rotary_dim / 2)")
            rc, rs = rotary_cos_.contiguous(), rotary_sin_.contiguous()
            keep += [rc, rs]
            a.rotary_cos, a.rotary_sin = _ptr(rc), _ptr(rs)
            a.seqlen_ro, a.rotary_dim = rc.shape[0], 2 * rc.shape[1]
            _require(a.rotary_dim <= d, "rotary_dim must be <= headdim")
            _require(a.rotary_dim % 16 == 0, "Only rotary dimensions divisible by 16 are currently supported")
    a.io_dtype = _DT[q.dtype]
    a.kv_dtype = _DT[kcache.dtype]
    a.softmax_scale, a.softcap = float(softmax_scale), float(softcap)
    a.causal = int(bool(is_causal))
    a.window_left, a.window_right = int(window_size_left), int(window_size_right)
    a.rotary_interleaved = int(bool(is_rotary_interleaved))
    a.num_splits = int(num_splits)

    _lib.check(lib.fa_rocm_kvcache_validate(C.byref(a)))
    with torch.cuda.device(q.device):
        cus = lib.fa_rocm_num_cus()
        need = lib.fa_rocm_kvcache_workspace_bytes(C.byref(a), cus)
        if need:
            ws = torch.empty((need + 3) // 4, dtype=torch.float32, device=q.device)
            keep.append(ws)
            a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel() * 4
    return KvcacheCall(a, out, lse, keep, q.device)


def varlen_fwd(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k_, leftpad_k_, block_table_, alibi_slopes_,
               max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal, window_size_left,
               window_size_right, softcap, return_softmax, gen_, *, num_splits: int = 0) -> List[torch.Tensor]:
    """mha_varlen_fwd (flash_api.cpp:848-1089).  Returns [out, softmax_lse (Hq, total_q), p, rng_state].
    num_splits (paged K/V only; not an argument of the reference's function): 0 cuts every sequence's keys into
    as many ranges as it takes to fill the device when the query tiles alone cannot, 1 never, n at most n."""
    # flash_api.cpp:886 (this generation's host takes seqused_k only as the lengths of paged K/V)
    _require(block_table_ is not None or seqused_k_ is None, "NPU FlashAttention does not support seqused_k.")
    return _varlen_fwd(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k_, leftpad_k_, block_table_, alibi_slopes_,
                       max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal, window_size_left,
                       window_size_right, softcap, return_softmax, gen_, num_splits=num_splits)


def _varlen_fwd(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k_, leftpad_k_, block_table_, alibi_slopes_,
                max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal, window_size_left,
                window_size_right, softcap, return_softmax, gen_, *, num_splits: int = 0) -> List[torch.Tensor]:
    """varlen_fwd without that generation's rejection of seqused_k for packed keys: with them, sequence b uses only
    its first seqused_k[b] keys (the third-generation surface, flash_attn_npu_3/flash_api.cpp:143-147)."""
    if (isinstance(q, torch.Tensor) and q.dim() == 3 and q.shape[-1] % 8 != 0 and q.shape[-1] <= 256 and q.is_cuda
            and k.shape[-1] == q.shape[-1] and v.shape[-1] == q.shape[-1]):
        # rows that are not 16-byte pieces: zero-padded copies to the next multiple of 8, as the reference's front end
        # does (flash_attn_npu_interface.py:897-901); with paged k / v this copies the cache
        import torch.nn.functional as F
        d = q.shape[-1]
        extra = (d + 7) // 8 * 8 - d
        if block_table_ is not None:
            _check_padded_cache_copy(k, v)
        res = _varlen_fwd(F.pad(q, (0, extra)), F.pad(k, (0, extra)), F.pad(v, (0, extra)), None, cu_seqlens_q, cu_seqlens_k,
                         seqused_k_, leftpad_k_, block_table_, alibi_slopes_, max_seqlen_q, max_seqlen_k, p_dropout,
                         softmax_scale, zero_tensors, is_causal, window_size_left, window_size_right, softcap, return_softmax,
                         gen_, num_splits=num_splits)
        out = res[0][..., :d]
        if out_ is not None:
            _require(out_.dtype == q.dtype and out_.shape == q.shape, "out must match q")
            out_.copy_(out)
            out = out_
        else:
            out = out.contiguous()
        return [out] + list(res[1:])
    return _C().varlen_fwd(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, seqused_k_, leftpad_k_, block_table_, alibi_slopes_,
                           int(max_seqlen_q), int(max_seqlen_k), float(p_dropout), float(softmax_scale), bool(zero_tensors),
                           bool(is_causal), int(window_size_left), int(window_size_right), float(softcap), bool(return_softmax),
                           gen_, int(num_splits))
