"""Seeded random sweep over the argument space of the kvcache and varlen calls against the oracle:
every case draws shapes, lengths, masks, split counts, append / rotary and dtypes from a fixed seed,
so a failure names a reproducible case.  The bars are those of the other GPU tests."""
import random

import pytest
import torch

import fa_oracle as O
from helpers import check_out, make_paged_case, rotary_tables, to_dev
from test_gpu_prefill import run_varlen, varlen_case

pytestmark = pytest.mark.gpu


def draw_kvcache(seed):
    r = random.Random(seed)
    d = r.choice([64, 128, 128, 128, 256])
    hk = r.choice([1, 2, 4, 8])
    group = r.choice([1, 2, 4, 5, 8, 16])
    hq = hk * group
    sq = r.choice([1, 1, 1, 2, 3, 4, 7, 16])
    page = r.choice([32, 64, 128, 256])
    B = r.randint(1, 5)
    lens = [r.choice([0, 1, 31, 32, 33, r.randint(1, 300), r.randint(300, 3000)]) for _ in range(B)]
    snew = r.choice([0, 0, 1, 2, 5])
    causal = r.random() < 0.6
    window = r.choice([(-1, -1), (-1, -1), (r.randint(0, 200), 0), (r.randint(0, 500), r.randint(0, 100)), (-1, r.randint(0, 64)),
                       (r.randint(0, 64), -1)])
    softcap = r.choice([0.0, 0.0, 0.0, 15.0])
    num_splits = r.choice([0, 0, 0, 1, 2, 5])
    dtype = r.choice([torch.bfloat16, torch.bfloat16, torch.float16])
    rot = r.choice([0, 0, 32, d]) if snew else 0
    interleaved = r.random() < 0.5
    return dict(B=B, hq=hq, hk=hk, d=d, page=page, lens=lens, sq=sq, snew=snew, causal=causal, window=window, softcap=softcap,
                num_splits=num_splits, dtype=dtype, rot=rot, interleaved=interleaved)


@pytest.mark.parametrize("seed", range(60))
def test_random_kvcache(seed):
    from flash_attn_npu import flash_attn_with_kvcache
    c = draw_kvcache(1000 + seed)
    print("random kvcache", seed, c, flush=True)
    case = make_paged_case(c["B"], c["hq"], c["hk"], c["d"], c["page"], c["lens"], seqlen_q=c["sq"], seqlen_new=c["snew"],
                           dtype=c["dtype"], seed=seed, extra_table_cols=seed % 2)
    kw = dict(causal=c["causal"], window_size=c["window"], softcap=c["softcap"])
    if c["rot"]:
        cos, sin = rotary_tables(max(c["lens"]) + c["snew"] + c["sq"] + 8, c["rot"], dtype=c["dtype"])
        kw.update(rotary_cos=cos, rotary_sin=sin, rotary_interleaved=c["interleaved"])
    dev = to_dev(case)
    dkw = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"], cache_seqlens=dev["cache_seqlens"],
                                       block_table=dev["block_table"], num_splits=c["num_splits"], return_softmax_lse=True, **dkw)
    torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], mode="fp32", **kw)
    if c["snew"]:
        assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16)), "appended K bytes differ"
        assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16)), "appended V bytes differ"
    check_out(out, ref, lse, ref_lse, f"random kvcache {seed}")


@pytest.mark.parametrize("seed", range(30))
def test_random_varlen(seed):
    r = random.Random(5000 + seed)
    B = r.randint(1, 5)
    d = r.choice([64, 128, 128, 256, 96, 111])
    hk = r.choice([1, 2, 4])
    hq = hk * r.choice([1, 2, 4, 5])
    seqs_k = [r.choice([1, 63, 64, 65, r.randint(1, 200), r.randint(200, 1500)]) for _ in range(B)]
    seqs_q = [r.choice([k, k, max(1, k // 2), r.randint(1, 300)]) for k in seqs_k]
    causal = r.random() < 0.6
    window = r.choice([(-1, -1), (-1, -1), (r.randint(0, 200), 0), (r.randint(0, 300), r.randint(0, 100)), (-1, r.randint(0, 64))])
    softcap = r.choice([0.0, 0.0, 30.0])
    dtype = r.choice([torch.bfloat16, torch.float16])
    c = varlen_case(seqs_q, seqs_k, hq, hk, d, dtype=dtype, seed=seed)
    got, ref, gold = run_varlen(c, causal=causal, window_size=window, softcap=softcap)
    check_out(got[0], ref[0], got[1], ref[1], f"random varlen {seed}")
