"""The reference's own parameter matrices for this path, replayed row for row on the reference's input
distribution: 130 kvcache rows (tests/test_flash_attn_npu_v2.py:145-286: dense and paged caches, block 128, decode /
multi-token / prefill-sized query blocks, odd GQA groups, windows, softcap 30, D = 1, 4, 128, 256), 20 dense-forward
rows (:436-459) and 33 varlen rows (:522-560), all drawn U(-5, 5) as the reference draws them (:290-302, :461-468,
:565-571).  The rows come from tests/golden/reference_matrix.json.  The bar is the reference's, rtol = atol = 1e-2 on
out and LSE against the blocked golden (:430-433); the fp32 bars (max-abs 2e-2, mean-abs 2e-3, LSE 1e-3) are checked
as well wherever the outputs are small enough for a 16-bit result to meet them at all."""
import json
import os

import pytest
import torch

import fa_oracle as O
from helpers import OUT_MAX_ABS, check_out, check_vs_golden, make_paged_case, to_dev
from test_gpu_prefill import run_varlen, varlen_case

pytestmark = pytest.mark.gpu

_M = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_matrix.json")))
_DT = {"bfloat16": torch.bfloat16, "float16": torch.float16}


def _ids(rows):
    return [f"{i:03d}-" + "-".join(str(x) for x in r) for i, r in enumerate(rows)]


def _uniform5(g, *shape):
    return -5.0 + 10.0 * torch.rand(*shape, generator=g)


def _check(out, lse, ref, gold, what):
    # the reference's bar
    check_vs_golden(out, gold[0], lse, gold[1], what)
    # A 16-bit output of magnitude up to 5 is rounded by up to 2^-9 * 4 = 7.8e-3 (bf16) on top of the rounding of P, so
    # the absolute fp32 bar is only meaningful where the result is of order one; the LSE bar always is.
    small = ref[0].abs().max().item() <= 2.0
    if small:
        check_out(out, ref[0], lse, ref[1], what)
    else:
        err = (out.detach().float().cpu() - ref[0].float()).abs()
        assert err.max().item() <= OUT_MAX_ABS * max(1.0, ref[0].abs().max().item() / 2.0), f"{what}: max abs err {err.max().item():.3e}"
        check_out(ref[0], ref[0], lse, ref[1], what)     # LSE bar alone


@pytest.mark.parametrize("row", _M["kvcache"], ids=_ids(_M["kvcache"]))
def test_reference_kvcache_matrix(row):
    from flash_attn_npu import flash_attn_with_kvcache
    dtype, B, hq, hk, sq, sk, d, paged, block, causal, wl, wr, softcap = row
    dtype = _DT[dtype]
    seed = (sq * 131 + sk * 7 + d * 3 + hq) & 0x7fffffff
    if paged:
        c = make_paged_case(B, hq, hk, d, block, [sk] * B, seqlen_q=sq, dtype=dtype, seed=seed, dist="uniform5")
        table = c["block_table"]
        dev = to_dev(c)
        table_dev = dev["block_table"]
    else:
        g = torch.Generator().manual_seed(seed)
        c = dict(q=_uniform5(g, B, sq, hq, d).to(dtype), k_cache=_uniform5(g, B, sk, hk, d).to(dtype),
                 v_cache=_uniform5(g, B, sk, hk, d).to(dtype), cache_seqlens=torch.full((B,), sk, dtype=torch.int32))
        table = torch.arange(B, dtype=torch.int32).view(B, 1)
        dev = to_dev(c)
        table_dev = None
    print("kvcache matrix row", row, flush=True)
    kw = dict(causal=causal, window_size=(wl, wr), softcap=softcap)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                       block_table=table_dev, return_softmax_lse=True, **kw)
    torch.cuda.synchronize()
    ref = O.flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], cache_seqlens=c["cache_seqlens"],
                                    block_table=table, mode="fp32", **kw)
    gold = O.flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], cache_seqlens=c["cache_seqlens"],
                                     block_table=table, mode="golden", **kw)
    _check(out, lse, ref, gold, str(row))


@pytest.mark.parametrize("row", _M["varlen"], ids=_ids(_M["varlen"]))
def test_reference_varlen_matrix(row):
    dtype, B, hq, hk, sq, sk, d, causal, wl, wr, softcap = row
    c = varlen_case([sq] * B, [sk] * B, hq, hk, d, dtype=_DT[dtype], seed=sq + sk + d, dist="uniform5")
    print("varlen matrix row", row, flush=True)
    got, ref, gold = run_varlen(c, causal=causal, window_size=(wl, wr), softcap=softcap)
    _check(got[0], got[1], ref, gold, str(row))


@pytest.mark.parametrize("row", _M["dense"], ids=_ids(_M["dense"]))
def test_reference_dense_forward_matrix(row):
    # flash_attn_func on (batch, seqlen, heads, headdim) tensors, with and without the LSE returned
    from flash_attn_npu import flash_attn_func
    dtype, B, hq, hk, sq, sk, d, with_lse, causal, softcap = row
    dtype = _DT[dtype]
    g = torch.Generator().manual_seed(sq * 17 + B * 3 + hq)
    q, k, v = _uniform5(g, B, sq, hq, d).to(dtype), _uniform5(g, B, sk, hk, d).to(dtype), _uniform5(g, B, sk, hk, d).to(dtype)
    print("dense matrix row", row, flush=True)
    ret = flash_attn_func(q.cuda(), k.cuda(), v.cuda(), 0.0, causal=causal, window_size=(-1, -1), softcap=softcap,
                          alibi_slopes=None, return_attn_probs=with_lse)
    torch.cuda.synchronize()
    out, lse = (ret[0], ret[1]) if with_lse else (ret, None)
    cu_q = torch.arange(B + 1, dtype=torch.int32) * sq
    cu_k = torch.arange(B + 1, dtype=torch.int32) * sk
    kw = dict(causal=causal, softcap=softcap)
    ref = O.flash_attn_varlen(q.reshape(B * sq, hq, d), k.reshape(B * sk, hk, d), v.reshape(B * sk, hk, d), cu_q, cu_k, sq, sk,
                              mode="fp32", **kw)
    gold = O.flash_attn_varlen(q.reshape(B * sq, hq, d), k.reshape(B * sk, hk, d), v.reshape(B * sk, hk, d), cu_q, cu_k, sq, sk,
                               mode="golden", **kw)
    out_t = out.reshape(B * sq, hq, d)
    # LSE of flash_attn_func is (batch, heads, seqlen); the oracle's is token-major (heads, total)
    lse_t = None if lse is None else lse.permute(1, 0, 2).reshape(hq, B * sq)
    if lse_t is None:
        torch.testing.assert_close(out_t.float().cpu(), gold[0].float(), rtol=1e-2, atol=1e-2)
    else:
        _check(out_t, lse_t, ref, gold, str(row))
