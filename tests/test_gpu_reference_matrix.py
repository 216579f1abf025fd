"""The reference's own parameter matrices for this path, replayed shape for shape against the oracle:
kvcache cases (tests/test_flash_attn_npu_v2.py:144-215: dense and paged caches, block 128, decode /
multi-token / prefill-sized query blocks, windows, D = 1, 4, 128, 256) and varlen cases (:522-560:
ragged-free batches of equal sequences, windows incl. negative sides, softcap 30, D = 64..256).
The bar is the reference's: rtol = atol = 1e-2 against the blocked golden, plus the fp32 bars."""
import pytest
import torch

import fa_oracle as O
from helpers import check_out, check_vs_golden, make_paged_case, to_dev
from test_gpu_prefill import run_varlen, varlen_case

pytestmark = pytest.mark.gpu

BF, FP = torch.bfloat16, torch.float16

# (dtype, batch, heads, kv_heads, q_seqlen, kv_seqlen, head_size, paged, block, causal, wl, wr, softcap)
KVCACHE_CASES = [
    (BF, 1, 1, 1, 1024, 1024, 128, 1, 128, False, -1, -1, 0.0),
    (BF, 5, 4, 4, 1024, 1024, 128, 0, 128, True, -1, -1, 0.0),
    (FP, 7, 1, 1, 512, 512, 128, 1, 128, False, -1, -1, 0.0),
    (BF, 1, 1, 1, 1, 1024, 128, 1, 128, True, -1, -1, 0.0),
    (BF, 1, 1, 1, 1, 4096, 128, 1, 128, False, -1, -1, 0.0),
    (FP, 2, 2, 1, 128, 128, 128, 1, 128, True, -1, -1, 0.0),
    (BF, 2, 6, 2, 2, 1024, 128, 1, 128, True, -1, -1, 0.0),
    (BF, 1, 1, 1, 1024, 1024, 128, 1, 128, True, 512, 0, 0.0),
    (BF, 1, 1, 1, 1024, 1024, 128, 1, 128, True, 512, 256, 0.0),
    (BF, 5, 4, 4, 1024, 1024, 128, 0, 128, True, -128, 864, 0.0),
    (BF, 1, 1, 1, 1024, 1024, 128, 1, 128, False, 0, 256, 0.0),
    (FP, 2, 2, 2, 512, 512, 128, 0, 128, False, 64, 128, 0.0),
    (FP, 1, 64, 1, 1, 1024, 128, 0, 128, True, 542, 647, 0.0),
    (FP, 1, 512, 1, 1, 1024, 128, 0, 128, True, 542, 647, 0.0),
    (BF, 1, 128, 1, 1, 1024, 128, 0, 128, True, 64, 0, 0.0),
    (FP, 16, 2, 2, 4096, 2, 128, 0, 128, False, 65, 412, 0.0),
    (FP, 1, 512, 1, 1, 1024, 4, 0, 128, True, 542, 647, 0.0),
    (FP, 4, 4, 2, 4, 4096, 1, 0, 128, True, 826, 973, 0.0),
    (FP, 4, 4, 2, 4, 4096, 1, 0, 128, False, 826, 973, 0.0),
    (BF, 4, 64, 16, 16, 1024, 128, 0, 128, True, -1, -1, 0.0),
    (BF, 8, 128, 16, 32, 2048, 128, 0, 128, False, -1, -1, 0.0),
    (BF, 4, 64, 8, 64, 4096, 128, 0, 128, False, -1, -1, 0.0),
    (BF, 8, 128, 8, 1, 4096, 128, 0, 128, False, -1, -1, 0.0),
    (BF, 4, 32, 4, 16, 1024, 256, 0, 128, False, -1, -1, 0.0),
    (BF, 2, 64, 8, 1, 4096, 256, 0, 128, False, -1, -1, 0.0),
    (BF, 1, 128, 4, 1, 2048, 128, 1, 128, True, -1, -1, 0.0),
    (BF, 1, 32, 8, 1, 2048, 256, 1, 128, False, -1, -1, 0.0),
    (BF, 1, 64, 4, 8, 2048, 128, 1, 128, True, -1, -1, 0.0),
    (BF, 2, 16, 2, 5, 4096, 128, 1, 128, True, -1, -1, 0.0),
    (BF, 1, 32, 4, 11, 4096, 128, 1, 128, False, -1, -1, 0.0),
    (BF, 1, 32, 8, 13, 2048, 256, 1, 128, False, -1, -1, 0.0),
    (BF, 2, 16, 2, 15, 2048, 128, 1, 128, True, -1, -1, 0.0),
]


@pytest.mark.parametrize("case", KVCACHE_CASES, ids=lambda c: "-".join(str(x).replace("torch.", "") for x in c))
def test_reference_kvcache_matrix(case):
    from flash_attn_npu import flash_attn_with_kvcache
    dtype, B, hq, hk, sq, sk, d, paged, block, causal, wl, wr, softcap = case
    g = torch.Generator().manual_seed(sq * 131 + sk + d)
    if paged:
        c = make_paged_case(B, hq, hk, d, block, [sk] * B, seqlen_q=sq, dtype=dtype, seed=sq + sk + d)
        table = c["block_table"]
        dev = to_dev(c)
        table_dev = dev["block_table"]
    else:
        c = dict(q=torch.randn(B, sq, hq, d, generator=g).to(dtype), k_cache=torch.randn(B, sk, hk, d, generator=g).to(dtype),
                 v_cache=torch.randn(B, sk, hk, d, generator=g).to(dtype), cache_seqlens=torch.full((B,), sk, dtype=torch.int32))
        table = torch.arange(B, dtype=torch.int32).view(B, 1)
        dev = to_dev(c)
        table_dev = None
    print("kvcache matrix case", case, flush=True)
    kw = dict(causal=causal, window_size=(wl, wr), softcap=softcap)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                       block_table=table_dev, return_softmax_lse=True, **kw)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], cache_seqlens=c["cache_seqlens"],
                                             block_table=table, mode="fp32", **kw)
    gold, gold_lse = O.flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], cache_seqlens=c["cache_seqlens"],
                                               block_table=table, mode="golden", **kw)
    check_out(out, ref, lse, ref_lse, str(case))
    check_vs_golden(out, gold, lse, gold_lse, str(case))


# (dtype, batch, heads, kv_heads, q_seqlen, kv_seqlen, head_size, causal, wl, wr, softcap)
VARLEN_CASES = [
    (BF, 1, 1, 1, 512, 1024, 128, True, -1, -1, 0.0),
    (BF, 2, 4, 4, 1024, 1024, 128, False, -1, -1, 0.0),
    (FP, 7, 5, 1, 512, 512, 128, True, -1, -1, 0.0),
    (FP, 7, 5, 1, 777, 888, 192, False, -1, -1, 0.0),
    (FP, 7, 5, 1, 1777, 1888, 256, True, -1, -1, 0.0),
    (BF, 1, 1, 1, 7777, 8192, 64, True, -1, -1, 0.0),
    (BF, 7, 5, 1, 711, 8192, 111, True, -1, -1, 0.0),
    (BF, 1, 1, 1, 512, 512, 128, True, 512, 0, 0.0),
    (BF, 1, 1, 1, 512, 512, 128, True, 256, 128, 0.0),
    (FP, 2, 4, 4, 256, 256, 128, False, 64, 128, 0.0),
    (BF, 1, 1, 1, 512, 512, 128, False, 0, 256, 0.0),
    (BF, 2, 6, 2, 128, 256, 128, True, 127, 0, 0.0),
    (BF, 2, 4, 4, 128, 512, 128, True, 511, 0, 0.0),
    (FP, 1, 2, 2, 64, 192, 128, False, 32, 64, 0.0),
    (BF, 1, 1, 1, 1, 1024, 128, True, 512, 0, 0.0),
    (FP, 2, 1, 1, 512, 512, 128, False, 508, -256, 0.0),
    (BF, 1, 1, 1, 1024, 1024, 128, True, -128, 864, 0.0),
    (BF, 2, 6, 2, 2, 1024, 128, True, 256, 0, 0.0),
    (FP, 1, 64, 1, 1, 1024, 128, True, 542, 647, 0.0),
    (FP, 1, 512, 1, 1, 1024, 128, True, 542, 647, 0.0),
    (BF, 1, 128, 1, 1, 1024, 128, True, 64, 0, 0.0),
    (FP, 7, 5, 1, 777, 888, 192, False, -1, -1, 30.0),
    (FP, 7, 5, 1, 1777, 1888, 256, True, -1, -1, 30.0),
    (BF, 7, 5, 1, 711, 8192, 111, True, -1, -1, 30.0),
    (FP, 1, 2, 2, 64, 192, 128, False, 32, 64, 30.0),
    (BF, 1, 1, 1, 1024, 1024, 128, True, 512, 0, 30.0),
    (FP, 2, 1, 1, 512, 512, 128, False, 508, -256, 30.0),
    (BF, 2, 6, 2, 2, 1024, 128, True, 256, 0, 30.0),
]


@pytest.mark.parametrize("case", VARLEN_CASES, ids=lambda c: "-".join(str(x).replace("torch.", "") for x in c))
def test_reference_varlen_matrix(case):
    dtype, B, hq, hk, sq, sk, d, causal, wl, wr, softcap = case
    c = varlen_case([sq] * B, [sk] * B, hq, hk, d, dtype=dtype, seed=sq + sk + d)
    print("varlen matrix case", case, flush=True)
    got, ref, gold = run_varlen(c, causal=causal, window_size=(wl, wr), softcap=softcap)
    check_out(got[0], ref[0], got[1], ref[1], str(case))
    check_vs_golden(got[0], gold[0], got[1], gold[1], str(case))
