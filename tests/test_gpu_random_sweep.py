"""Seeded random sweep over the argument space of the kvcache and varlen calls against the oracle:
every case draws shapes, lengths, masks, split counts, append / rotary and dtypes from a fixed seed,
so a failure names a reproducible case.  The bars are those of the other GPU tests."""
import random

import pytest
import torch

import fa_oracle as O
from helpers import check_out, make_paged_case, rotary_tables, to_dev
from test_gpu_dense import make_dense_case, run_dense
from test_gpu_mla import mla_case
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


def draw_odd_groups(seed):
    """GQA groups that are not powers of two and query blocks whose row count (tokens x group) lands on either side of
    the kernels' 16- and 32-row switches: 18, 30, 33, 50, 70 and their neighbours."""
    r = random.Random(seed)
    group = r.choice([3, 6, 7, 9, 12, 20])
    rows_target = r.choice([9, 15, 16, 18, 30, 32, 33, 50, 70])
    sq = max(1, round(rows_target / group))
    hk = r.choice([1, 2, 4])
    d = r.choice([64, 128, 128, 256])
    page = r.choice([32, 128, 256])
    B = r.randint(1, 4)
    lens = [r.choice([0, 1, 33, r.randint(1, 300), r.randint(300, 3000)]) for _ in range(B)]
    snew = r.choice([0, 0, 1, sq])
    causal = r.random() < 0.6
    window = r.choice([(-1, -1), (-1, -1), (r.randint(0, 300), 0), (r.randint(0, 300), r.randint(0, 64))])
    dtype = r.choice([torch.bfloat16, torch.bfloat16, torch.float16])
    rot = r.choice([0, 0, 32, d]) if snew else 0
    return dict(B=B, hq=hk * group, hk=hk, d=d, page=page, lens=lens, sq=sq, snew=snew, causal=causal, window=window,
                softcap=r.choice([0.0, 0.0, 30.0]), num_splits=r.choice([0, 0, 1, 3]), dtype=dtype, rot=rot,
                interleaved=r.random() < 0.5)


def draw_tall(seed):
    """Query blocks up to 257 tokens x 16 heads per kv head and batches up to 24 rows: the blocks that leave the
    decode kernels for the tiled one, its packed heads and its key-range split.  Sized so the oracle takes ~0.1 s."""
    r = random.Random(seed)
    while True:
        d = r.choice([64, 128, 128, 256])
        hk = r.choice([1, 2, 4, 8])
        group = r.choice([1, 2, 4, 8, 16])
        sq = r.choice([2, 5, 8, 16, 17, 33, 64, 100, 128, 130, 257])
        page = r.choice([32, 64, 128, 256])
        B = r.randint(1, 24)
        lens = [r.choice([0, 1, 33, r.randint(1, 300), r.randint(300, 2000), r.randint(2000, 6000)]) for _ in range(B)]
        if hk * group * sq * (sum(lens) + B * sq) * d <= 3e9:
            break
    snew = r.choice([0, 0, sq, 1, 3])
    causal = r.random() < 0.7
    window = r.choice([(-1, -1), (-1, -1), (-1, -1), (r.randint(0, 500), 0), (r.randint(0, 500), r.randint(0, 100)),
                       (-1, r.randint(0, 64)), (r.randint(0, 64), -1)])
    softcap = r.choice([0.0, 0.0, 0.0, 15.0])
    num_splits = r.choice([0, 0, 0, 1, 2, 4, 9])
    dtype = r.choice([torch.bfloat16, torch.bfloat16, torch.float16])
    rot = r.choice([0, 0, 32, d]) if snew else 0
    return dict(B=B, hq=hk * group, hk=hk, d=d, page=page, lens=lens, sq=sq, snew=snew, causal=causal, window=window,
                softcap=softcap, num_splits=num_splits, dtype=dtype, rot=rot, interleaved=r.random() < 0.5)


@pytest.mark.parametrize("seed", [*range(60), 324, *range(2000, 2060), *range(4000, 4048)])     # 324: an fp16 rotary result on an exact tie
def test_random_kvcache(seed):
    from flash_attn_npu import flash_attn_with_kvcache
    c = draw_kvcache(1000 + seed) if seed < 2000 else (draw_tall(seed - 2000) if seed < 4000 else draw_odd_groups(seed))
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


@pytest.mark.parametrize("seed", range(30))
def test_random_int8_latent(seed):
    from flash_attn_npu import flash_attn_with_kvcache
    r = random.Random(7000 + seed)
    B = r.randint(1, 40)
    hq = r.choice([64, 128])
    sq = r.choice([1, 1, 1, 2, 3, 4])
    page = r.choice([64, 128, 256])
    lens = [r.choice([0, 1, 255, 257, r.randint(1, 600), r.randint(600, 5000)]) for _ in range(B)]
    snew = r.choice([0, 0, sq])
    kw = dict(softmax_scale=192 ** -0.5, causal=r.random() < 0.7,
              window_size=r.choice([(-1, -1), (-1, -1), (r.randint(0, 600), 0), (-1, r.randint(0, 8))]), softcap=r.choice([0.0, 0.0, 20.0]))
    num_splits = r.choice([0, 0, 1, 3])
    print("random int8 latent", seed, dict(B=B, hq=hq, sq=sq, page=page, lens=lens, snew=snew, num_splits=num_splits), kw, flush=True)
    case = mla_case(B, hq, [l + snew for l in lens], page=page, seed=seed, spare=seed % 3)
    case["cache_seqlens"] = torch.tensor(lens, dtype=torch.int32)
    g = torch.Generator().manual_seed(seed + 7)
    q = torch.randn(B, sq, hq, 576, generator=g).to(torch.bfloat16)
    kn = torch.randn(B, snew, 1, 576, generator=g).to(torch.bfloat16) if snew else None
    kc, ks = case["k_cache"].cuda(), case["k_scale"].cuda()
    knd = kn.cuda() if snew else None
    out, lse = flash_attn_with_kvcache(q.cuda(), kc, kc[..., :512], knd, knd[..., :512] if snew else None,
                                       cache_seqlens=case["cache_seqlens"].cuda(), block_table=case["block_table"].cuda(),
                                       return_softmax_lse=True, k_scale_cache=ks, num_splits=num_splits, **kw)
    torch.cuda.synchronize()
    kc_o, ks_o = case["k_cache"].clone(), case["k_scale"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(q, kc_o, kc_o[..., :512], kn, kn[..., :512] if snew else None,
                                             cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                             k_scale_cache=ks_o, mode="fp32", **kw)
    assert torch.equal(kc.cpu(), kc_o), "codes differ"
    assert torch.equal(ks.cpu().view(torch.int32), ks_o.view(torch.int32)), "scales differ"
    check_out(out, ref, lse, ref_lse, f"random int8 latent {seed}")


@pytest.mark.parametrize("seed", range(30))
def test_random_dense(seed):
    r = random.Random(9000 + seed)
    B = r.randint(1, 8)
    d = r.choice([64, 128, 256])
    hk = r.choice([1, 2, 8])
    hq = hk * r.choice([1, 4, 8])
    sq = r.choice([1, 1, 2, 7, 40])
    s_cache = r.choice([64, 100, 512, 1111, 3000])
    snew = r.choice([0, 1, sq])
    lens = None if (snew == 0 and r.random() < 0.3) else [r.randint(0, s_cache - snew) for _ in range(B)]
    b_cache = B + r.choice([0, 0, 3])
    idx = torch.tensor(r.sample(range(b_cache), B), dtype=torch.int32) if r.random() < 0.5 else None
    causal, num_splits = r.random() < 0.6, r.choice([0, 0, 1, 3])
    dtype = r.choice([torch.bfloat16, torch.float16])
    case = make_dense_case(B, hq, hk, d, s_cache, lens, seqlen_q=sq, seqlen_new=snew, dtype=dtype, seed=seed, b_cache=b_cache)
    got, ref, gold, dev = run_dense(case, cache_batch_idx=idx, causal=causal, num_splits=num_splits)
    if snew:
        assert torch.equal(dev["k_cache"].cpu().view(torch.int16), ref[2].view(torch.int16)), "appended K bytes differ"
        assert torch.equal(dev["v_cache"].cpu().view(torch.int16), ref[3].view(torch.int16)), "appended V bytes differ"
    check_out(got[0], ref[0], got[1], ref[1], f"random dense {seed}")


def draw_ragged_paged(seed):
    r = random.Random(11000 + seed)
    B = r.randint(1, 12)
    d = r.choice([64, 128, 128, 256])
    hk = r.choice([1, 2, 4, 8])
    hq = hk * r.choice([1, 2, 4, 8])
    page = r.choice([32, 64, 256])
    while True:
        lens_k = [r.choice([0, 1, 40, r.randint(1, 600), r.randint(600, 3000), r.randint(3000, 9000)]) for _ in range(B)]
        lens_q = [r.choice([0, 1, 1, 1, 2, 17, r.randint(1, 150), r.randint(150, 600)]) for _ in range(B)]
        if sum(lens_q) > 0 and hq * d * sum(q * (k + 1) for q, k in zip(lens_q, lens_k)) <= 3e9:
            break
    causal = r.random() < 0.7
    window = r.choice([(-1, -1), (-1, -1), (-1, -1), (r.randint(0, 2000), 0), (r.randint(0, 2000), r.randint(0, 100)), (-1, r.randint(0, 64))])
    return dict(B=B, d=d, hk=hk, hq=hq, page=page, lens_k=lens_k, lens_q=lens_q, causal=causal, window=window,
                softcap=r.choice([0.0, 0.0, 25.0]), num_splits=r.choice([0, 0, 0, 1, 2, 7, 64]),
                dtype=r.choice([torch.bfloat16, torch.float16]))


@pytest.mark.parametrize("seed", range(40))
def test_random_ragged_blocks_over_pages(seed):
    # token-major query blocks of any length (empty ones, single decode rows, prompt chunks) over a paged cache:
    # packed heads per block, key ranges, the per-token merge
    from flash_attn_npu.flash_attn_npu import varlen_fwd
    c = draw_ragged_paged(seed)
    print("random ragged paged", seed, c, flush=True)
    B, d = c["B"], c["d"]
    case = make_paged_case(B, c["hq"], c["hk"], d, c["page"], c["lens_k"], dtype=c["dtype"], seed=seed, extra_table_cols=seed % 2)
    g = torch.Generator().manual_seed(seed + 1)
    q = torch.randn(sum(c["lens_q"]), c["hq"], d, generator=g).to(c["dtype"])
    cu_q = torch.tensor([0] + torch.tensor(c["lens_q"]).cumsum(0).tolist(), dtype=torch.int32)
    cu_k = torch.tensor([0] + torch.tensor(c["lens_k"]).cumsum(0).tolist(), dtype=torch.int32)
    kl = torch.cat([O.gather_paged(case["k_cache"], case["block_table"][b], c["lens_k"][b]) for b in range(B)])
    vl = torch.cat([O.gather_paged(case["v_cache"], case["block_table"][b], c["lens_k"][b]) for b in range(B)])
    max_q, max_k = max(c["lens_q"]), max(max(c["lens_k"]), 1)
    out, lse, _, _ = varlen_fwd(q.cuda(), case["k_cache"].cuda(), case["v_cache"].cuda(), None, cu_q.cuda(), None,
                                case["cache_seqlens"].cuda(), None, case["block_table"].cuda(), None, max_q, max_k, 0.0, d ** -0.5,
                                False, c["causal"], c["window"][0], c["window"][1], c["softcap"], False, None, num_splits=c["num_splits"])
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_varlen(q, kl, vl, cu_q, cu_k, max_q, max_k, causal=c["causal"], window_size=c["window"],
                                       softcap=c["softcap"], mode="fp32")
    check_out(out, ref, lse, ref_lse, f"random ragged paged {seed}")
