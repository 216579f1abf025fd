"""CPU oracle for the paged KV-cache attention path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain PyTorch on host cores, the algorithm that the
reference's own tests use as the forward golden, plus the documented-but-
unimplemented parts of its API (append, rotary) and the int8 latent format.
It is the checker for the HIP kernels: only tests, the smoke check and the
benchmark's cpu_baseline leg may import it.  The shipped package never does.

Reference anchors (paths relative to the reference checkout):
  * blocked forward golden `ref_flash_attention`      tests/test_flash_attn_npu_v2.py:84-143
  * GQA head mapping `group_matmul`                   tests/test_flash_attn_npu_v2.py:10-24
  * online softmax step `softmax1`                    tests/test_flash_attn_npu_v2.py:26-44
  * window normalisation (host)                       csrc/ascend910/flash_attn_npu/flash_api.cpp:483-505
                                                      tests/test_flash_attn_npu_v2.py:325-342
  * causal / window masks                             tests/test_flash_attn_npu_v2.py:356-386
                                                      tests/fa_small_op_golden.py:35-58
  * paged gather                                      tests/test_flash_attn_npu_v2.py:394-411
                                                      tests/test_flash_attn_npu_v4.py:529-535
  * fully masked rows -> out 0, lse +inf              tests/test_flash_attn_npu_v2.py:421-427
  * plain fp32 golden with fp64 LSE                   tests/test_flash_attn_npu_v4.py:194-218
  * split-KV combine                                  csrc/ascend910/flash_attn_npu/CombineScale.hpp:166-316
  * append / rotary semantics (docstring only)        flash_attn_npu/flash_attn_npu_interface.py:1460-1474,1508-1530
  * varlen layout, LSE (Hq, total_q)                  csrc/ascend910/flash_attn_npu/flash_api.cpp:998-1027

Pin status (what independent check holds each function; see tests/test_oracle_*.py):
  normalize_window      known-answer tables + equivalence with un-normalised closed form
  masked_matrix         docstring truth tables (2,5) and (5,2); element-wise closed form
  gather_paged          brute-force per-token loop, bit-exact
  ref_flash_attention   torch.softmax / torch.logsumexp in fp64 on the same inputs
  attention_fp32        same library routines
  combine_splits        logsumexp identity; split == unsplit
  append_kv             brute-force scalar loop, bit-exact; untouched bytes unchanged; the
                        quantising form: scalar-loop codes and scales per appended token,
                        attention equal to a cache quantised with the rows in place
  apply_rotary          complex-multiplication form, identity cases, norm preservation
  quantize_per_token    brute-force scalar loop, bit-exact codes
  The reference has no implementation or test of append, rotary or int8 KV: for
  those three the pins above are mathematical, not reference-derived
  (parity with the reference is unpinned because the reference rejects or
  ignores these arguments).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

KV_CHUNK = 512      # keys per online-softmax step   (tests/test_flash_attn_npu_v2.py:101)
DIM_SLICE = 128     # contraction slice of QK^T / PV  (tests/test_flash_attn_npu_v2.py:51,73)
MASK_ADD = -1e4     # additive mask value of the golden (tests/test_flash_attn_npu_v2.py:116)


# --------------------------------------------------------------------------- masks
def normalize_window(wl: int, wr: int, causal: bool, max_sk: int):
    """Host window normalisation (flash_api.cpp:483-505; test :325-342).

    Returns (wl, wr, is_causal, is_local).  `max_sk` is the batch maximum key
    length, as in the reference host code."""
    if max_sk > 0 and wl >= max_sk:
        wl = -1
    if max_sk > 0 and wr >= max_sk:
        wr = -1
    if causal:
        wr = 0
    is_causal = wl < 0 and wr == 0
    is_local = (wl >= 0 or wr >= 0) and not is_causal
    if is_local:
        if wl < 0:
            wl = max_sk
        if wr < 0:
            wr = max_sk
    return wl, wr, is_causal, is_local


def masked_matrix(sq: int, sk: int, is_causal: bool, is_local: bool, wl: int, wr: int) -> Optional[torch.Tensor]:
    """Boolean (sq, sk) matrix, True = key hidden.  None when nothing is masked.

    causal: torch.triu(ones, diagonal=sk-sq+1)          (test :380-384)
    local : (j-i) < sk-sq-wl  or  (j-i) > sk-sq+wr      (test :356-366, v4 :522-527)"""
    if is_causal:
        return torch.triu(torch.ones(sq, sk), diagonal=sk - sq + 1).bool()
    if is_local:
        i = torch.arange(sq)[:, None]
        j = torch.arange(sk)[None, :]
        lo = sk - sq - wl
        hi = sk - sq + wr
        return ((j - i) < lo) | ((j - i) > hi)
    return None


# --------------------------------------------------------------------------- paging
def gather_paged(cache: torch.Tensor, block_table_row: torch.Tensor, length: int) -> torch.Tensor:
    """Linearise one row's keys: out[j] = cache[bt[j // page], j % page]   (v4 test :529-535)."""
    page = cache.shape[1]
    pos = torch.arange(length)
    bt = block_table_row.to(torch.long)
    return cache[bt[pos // page], pos % page]


# --------------------------------------------------------------------------- rotary
def apply_rotary(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                 interleaved: bool) -> torch.Tensor:
    """Rotate x (T, H, d) at integer `positions` (T,).

    cos/sin: (seqlen_ro, rot/2) in any float dtype; rot = 2*cos.shape[1] <= d.
    Non-interleaved pairs (c, c+rot/2); interleaved pairs (2c, 2c+1)
    (flash_attn_npu_interface.py:1527-1530).  Arithmetic: every operand is
    widened to fp32, the two products and the add/sub are separately rounded
    fp32 operations (no fused multiply-add), the result is rounded to x.dtype
    with round-to-nearest-even; dims >= rot pass through untouched."""
    rot = 2 * cos.shape[1]
    d = x.shape[-1]
    assert rot <= d
    c = cos[positions.long()].to(torch.float32)[:, None, :]   # (T,1,rot/2)
    s = sin[positions.long()].to(torch.float32)[:, None, :]
    xf = x.to(torch.float32)
    out = xf.clone()
    if interleaved:
        x1 = xf[..., 0:rot:2]
        x2 = xf[..., 1:rot:2]
    else:
        x1 = xf[..., : rot // 2]
        x2 = xf[..., rot // 2: rot]
    # torch CPU elementwise ops are separately rounded (no contraction)
    o1 = x1 * c - x2 * s
    o2 = x1 * s + x2 * c
    if interleaved:
        out[..., 0:rot:2] = o1
        out[..., 1:rot:2] = o2
    else:
        out[..., : rot // 2] = o1
        out[..., rot // 2: rot] = o2
    return out.to(x.dtype)


# --------------------------------------------------------------------------- append
def append_kv(k_cache: torch.Tensor, v_cache: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
              cache_seqlens: torch.Tensor, block_table: torch.Tensor,
              rotary_cos: Optional[torch.Tensor] = None, rotary_sin: Optional[torch.Tensor] = None,
              rotary_interleaved: bool = True, k_scale_cache: Optional[torch.Tensor] = None,
              v_scale_cache: Optional[torch.Tensor] = None) -> None:
    """In-place paged append (flash_attn_npu_interface.py:1460-1467,1508-1510).

    For t < Snew: p = cache_seqlens[b] + t;
        k_cache[bt[b, p // page], p % page] = rope(k_new[b, t], pos=p);  v likewise without rope.
    int8 latent cache (k_scale_cache given; v_cache is a view of k_cache): the new rows are
    quantised per token (quantize_per_token) and codes and scale are written at the same place."""
    B, snew = k_new.shape[0], k_new.shape[1]
    page = k_cache.shape[1]
    for b in range(B):
        base = int(cache_seqlens[b])
        pos = base + torch.arange(snew)
        blk = block_table[b].to(torch.long)[pos // page]
        if k_scale_cache is not None:
            code, scale = quantize_per_token(k_new[b])          # (snew, Hk, d), (snew, Hk)
            k_cache[blk, pos % page] = code
            k_scale_cache[blk, pos % page] = scale
            if v_scale_cache is not None and v_scale_cache.data_ptr() != k_scale_cache.data_ptr():
                v_scale_cache[blk, pos % page] = scale
            continue
        kb = k_new[b]
        if rotary_cos is not None:
            kb = apply_rotary(kb, rotary_cos, rotary_sin, pos, rotary_interleaved)
        k_cache[blk, pos % page] = kb
        v_cache[blk, pos % page] = v_new[b]


# --------------------------------------------------------------------------- int8 latent format
def quantize_per_token(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Symmetric per-token int8: scale = absmax/127 (fp32), code = clamp(rne(x/scale), -127, 127).

    x: (..., d) any float dtype.  All-zero token -> scale 0, codes 0."""
    xf = x.to(torch.float32)
    absmax = xf.abs().amax(dim=-1, keepdim=True)
    scale = absmax / 127.0
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    code = torch.clamp(torch.round(xf / safe), -127, 127)   # torch.round is round-half-to-even
    code = torch.where(scale > 0, code, torch.zeros_like(code)).to(torch.int8)
    return code, scale.squeeze(-1)


def dequantize_per_token(code: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """fp32 value = code * scale (one correctly rounded fp32 multiply)."""
    return code.to(torch.float32) * scale.to(torch.float32)[..., None]


# --------------------------------------------------------------------------- attention cores
def _group_matmul(left: torch.Tensor, right: torch.Tensor) -> torch.Tensor:
    """left (Hq, M, K) x right (Hk, K, N) with q head h using kv head h // (Hq//Hk), fp32
    (tests/test_flash_attn_npu_v2.py:10-24)."""
    hq, hk = left.shape[0], right.shape[0]
    g = hq // hk
    lf = left.to(torch.float32).reshape(hk, g, left.shape[1], left.shape[2])
    rf = right.to(torch.float32)[:, None]
    return torch.matmul(lf, rf).reshape(hq, left.shape[1], right.shape[2])


def _sliced_matmul(left: torch.Tensor, right: torch.Tensor) -> torch.Tensor:
    """Accumulate the grouped product over 128-wide slices of the contraction dim
    (qkMM1 / pvMM2, tests/test_flash_attn_npu_v2.py:46-82)."""
    kdim = right.shape[1]
    acc = None
    for s in range(0, kdim, DIM_SLICE):
        part = _group_matmul(left[:, :, s:s + DIM_SLICE], right[:, s:s + DIM_SLICE, :])
        acc = part if acc is None else acc + part
    return acc


def ref_flash_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, scale: float,
                        mask: Optional[torch.Tensor], data_type: torch.dtype, softcap: float = 0.0):
    """Blocked golden (tests/test_flash_attn_npu_v2.py:84-143).

    query (Sq, Hq, d), key (Sk, Hk, d), value (Sk, Hk, dv), mask bool (Sq, Sk) True=hidden or None.
    512-key chunks, fp32 online max/sum, additive -1e4 mask, P cast to `data_type` before PV.
    Returns out (Sq, Hq, dv) in data_type and lse (Hq, Sq) fp32.  Rows hidden everywhere are NOT
    post-fixed here (the caller does that, as the reference test does)."""
    q = query.permute(1, 0, 2)            # (Hq, Sq, d)
    k = key.permute(1, 2, 0)              # (Hk, d, Sk)
    v = value.permute(1, 0, 2)            # (Hk, Sk, dv)
    sc = torch.tensor(scale, dtype=torch.float32)
    sk = k.shape[2]
    gm = gl = go = None
    for start in range(0, sk, KV_CHUNK):
        end = min(start + KV_CHUNK, sk)
        s = _sliced_matmul(q, k[:, :, start:end]) * sc
        if softcap > 0.0:
            s = softcap * torch.tanh(s / softcap)
        if mask is not None:
            s = s + mask[: q.shape[1], start:end].to(torch.float32) * MASK_ADD
        lm = s.max(dim=-1, keepdim=True)[0]
        if gm is None:
            hm = lm
            dm = None
        else:
            hm = torch.maximum(gm, lm)
            dm = torch.exp(gm - hm)
        gm = hm
        p = torch.exp(s - hm)
        row_sum = p.sum(dim=-1, keepdim=True)
        lo = _sliced_matmul(p.to(data_type), v[:, start:end, :])
        if dm is None:
            gl, go = row_sum, lo
        else:
            gl = gl * dm + row_sum
            go = go * dm + lo
    if go is None:      # no keys at all
        hq, sq = q.shape[0], q.shape[1]
        return (torch.zeros(sq, hq, value.shape[-1], dtype=data_type),
                torch.full((hq, sq), float("inf"), dtype=torch.float32))
    out = (go / gl).permute(1, 0, 2).to(data_type)
    lse = (torch.log(gl) + gm).squeeze(-1).to(torch.float32)
    return out, lse


def attention_fp32(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, scale: float,
                   mask: Optional[torch.Tensor], softcap: float = 0.0):
    """Unblocked fp32 reference with fp64 LSE (tests/test_flash_attn_npu_v4.py:194-218); P is NOT
    rounded to the I/O dtype.  Hidden keys are removed exactly (-inf), and rows with no visible key
    return out 0 / lse +inf.  Returns out (Sq, Hq, dv) fp32, lse (Hq, Sq) fp32."""
    q = query.permute(1, 0, 2)
    k = key.permute(1, 2, 0)
    v = value.permute(1, 0, 2)
    s = _group_matmul(q, k) * torch.tensor(scale, dtype=torch.float32)
    if softcap > 0.0:
        s = softcap * torch.tanh(s / softcap)
    if mask is not None:
        s = s.masked_fill(mask[None, : q.shape[1], : k.shape[2]], float("-inf"))
    if s.shape[-1] == 0:
        s = torch.full(s.shape[:-1] + (1,), float("-inf"))
        v = torch.zeros(v.shape[0], 1, v.shape[2])
    lse = torch.logsumexp(s.to(torch.float64), dim=-1)
    empty = torch.isinf(lse) & (lse < 0)
    p = torch.exp(s.to(torch.float64) - torch.where(empty, torch.zeros_like(lse), lse)[..., None]).to(torch.float32)
    p = torch.where(empty[..., None], torch.zeros_like(p), p)
    out = _group_matmul(p, v).permute(1, 0, 2)
    lse = torch.where(empty, torch.full_like(lse, float("inf")), lse).to(torch.float32)
    return out, lse


def _fix_hidden_rows(out: torch.Tensor, lse: torch.Tensor, mask: Optional[torch.Tensor]):
    """Rows whose every key is hidden: out = 0, lse = +inf (test :421-427; flash_api.cpp:570)."""
    if mask is not None and mask.numel() > 0:
        dead = mask.all(dim=-1)
        if dead.any():
            out[dead, :, :] = 0
            lse[:, dead] = float("inf")
    return out, lse


def combine_splits(o_parts: torch.Tensor, lse_parts: torch.Tensor):
    """Merge split-KV partials (CombineScale.hpp:166-194,249-316).

    o_parts (S, ..., dv) fp32, each already normalised by its own sum; lse_parts (S, ...) fp32 with
    +inf or -inf marking a split that saw no key.  Returns (out fp32, lse fp32); all-empty -> 0, +inf."""
    l = torch.where(torch.isinf(lse_parts) & (lse_parts > 0), torch.full_like(lse_parts, float("-inf")), lse_parts)
    m = l.max(dim=0)[0]
    dead = torch.isinf(m) & (m < 0)
    m0 = torch.where(dead, torch.zeros_like(m), m)
    w = torch.exp(l - m0)
    tot = w.sum(dim=0)
    lse = m0 + torch.log(tot)
    wn = torch.exp(l - torch.where(dead, torch.zeros_like(lse), lse))
    out = (wn[..., None] * torch.where(torch.isinf(l)[..., None], torch.zeros_like(o_parts), o_parts)).sum(dim=0)
    out = torch.where(dead[..., None], torch.zeros_like(out), out)
    lse = torch.where(dead, torch.full_like(lse, float("inf")), lse)
    return out, lse


# --------------------------------------------------------------------------- API-level oracles
def flash_attn_with_kvcache(q, k_cache, v_cache, k=None, v=None, rotary_cos=None, rotary_sin=None,
                            cache_seqlens=None, block_table=None, softmax_scale=None, causal=False,
                            window_size=(-1, -1), softcap=0.0, rotary_interleaved=True,
                            k_scale_cache=None, v_scale_cache=None, mode: str = "golden"):
    """API-level oracle of the paged kvcache call.

    mode "golden": blocked golden with P rounded to the I/O dtype (what the reference tests compare to).
    mode "fp32"  : plain fp32 reference (for the max-abs 2e-2 / mean-abs 2e-3 gate).
    Mutates k_cache / v_cache when k, v are given.  int8 caches (k_scale_cache given) are
    dequantised with the per-token fp32 scales before the same attention; for the latent (MLA)
    format v_cache is the narrow view k_cache[..., :dv] and v_scale_cache defaults to k_scale_cache."""
    B, sq, hq, d = q.shape
    assert block_table is not None, "oracle covers the paged path"
    if isinstance(cache_seqlens, int):
        cache_seqlens = torch.full((B,), cache_seqlens, dtype=torch.int32)
    snew = 0
    if k is not None:
        snew = k.shape[1]
        append_kv(k_cache, v_cache, k, v, cache_seqlens, block_table, rotary_cos, rotary_sin, rotary_interleaved,
                  k_scale_cache, v_scale_cache)
    if softmax_scale is None:
        softmax_scale = d ** (-0.5)
    lens = [int(x) + snew for x in cache_seqlens]
    wl, wr, is_causal, is_local = normalize_window(int(window_size[0]), int(window_size[1]), causal, max(lens))
    io_dtype = q.dtype
    dv = v_cache.shape[-1]
    out = torch.zeros(B, sq, hq, dv, dtype=io_dtype if mode == "golden" else torch.float32)
    lse = torch.empty(B, hq, sq, dtype=torch.float32)
    user_local = (int(window_size[0]) >= 0 or int(window_size[1]) >= 0)
    for b in range(B):
        lk = lens[b]
        kb = gather_paged(k_cache, block_table[b], lk)
        vb = gather_paged(v_cache, block_table[b], lk)
        if k_scale_cache is not None:
            kb = dequantize_per_token(kb, gather_paged(k_scale_cache, block_table[b], lk))
            vs = k_scale_cache if v_scale_cache is None else v_scale_cache
            vb = dequantize_per_token(vb, gather_paged(vs, block_table[b], lk))
        qb = q[b]
        if rotary_cos is not None and k is not None:
            base = int(cache_seqlens[b])
            if causal or user_local:
                pos = base + torch.arange(sq)
            else:
                pos = torch.full((sq,), base)
            qb = apply_rotary(qb, rotary_cos, rotary_sin, pos, rotary_interleaved)
        mask = masked_matrix(sq, lk, is_causal, is_local, wl, wr)
        if mode == "golden":
            o, l = ref_flash_attention(qb, kb, vb, softmax_scale, mask, io_dtype, softcap)
            o, l = _fix_hidden_rows(o, l, mask)
        else:
            o, l = attention_fp32(qb, kb, vb, softmax_scale, mask, softcap)
        out[b] = o
        lse[b] = l
    return out, lse


def flash_attn_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale=None,
                      causal=False, window_size=(-1, -1), softcap=0.0, mode: str = "golden"):
    """API-level oracle of the varlen forward: q (Tq, Hq, d), k/v (Tk, Hk, d); lse (Hq, Tq)
    (flash_api.cpp:998; per-sequence loop as in tests/test_flash_attn_npu_v2.py:610-650)."""
    tq, hq, d = q.shape
    if softmax_scale is None:
        softmax_scale = d ** (-0.5)
    io_dtype = q.dtype
    out = torch.zeros(tq, hq, v.shape[-1], dtype=io_dtype if mode == "golden" else torch.float32)
    lse = torch.empty(hq, tq, dtype=torch.float32)
    wl, wr, is_causal, is_local = normalize_window(int(window_size[0]), int(window_size[1]), causal, int(max_seqlen_k))
    nb = cu_seqlens_q.numel() - 1
    for b in range(nb):
        q0, q1 = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1])
        k0, k1 = int(cu_seqlens_k[b]), int(cu_seqlens_k[b + 1])
        sq, sk = q1 - q0, k1 - k0
        if sq == 0:
            continue
        mask = masked_matrix(sq, sk, is_causal, is_local, wl, wr)
        if mode == "golden":
            o, l = ref_flash_attention(q[q0:q1], k[k0:k1], v[k0:k1], softmax_scale, mask, io_dtype, softcap)
            o, l = _fix_hidden_rows(o, l, mask)
        else:
            o, l = attention_fp32(q[q0:q1], k[k0:k1], v[k0:k1], softmax_scale, mask, softcap)
        out[q0:q1] = o
        lse[:, q0:q1] = l
    return out, lse
