"""What the cache holds outside the visible keys must not matter, and where a page lies in the pool must not either.

A paged pool is allocated once and never cleared: slots past cache_seqlens and blocks no table names hold
whatever was there, NaN bit patterns included (0 * NaN = NaN in a P.V product that does not zero masked
keys).  Pools sized for a 288 GB device put blocks at byte offsets beyond 2^32."""
import pytest
import torch

import fa_oracle as O
from helpers import check_out, make_paged_case, rotary_tables, to_dev
from test_gpu_mla import mla_case

pytestmark = pytest.mark.gpu

LENS = [100, 1, 0, 777, 64, 65]


def visible_slots(case, lens):
    page = case["k_cache"].shape[1]
    used = torch.zeros(case["k_cache"].shape[0], page, dtype=torch.bool)
    for b, n in enumerate(lens):
        t = torch.arange(n)
        used[case["block_table"][b].long()[t // page], t % page] = True
    return used


@pytest.mark.parametrize("sq,snew,kw", [
    (1, 0, dict(causal=True)),                                  # wave-level decode
    (1, 1, dict(causal=True)),                                  # with the fused append
    (4, 0, dict(causal=True)),
    (1, 0, dict(causal=True, num_splits=3)),                    # grid of fixed splits
    (1, 0, dict(causal=True, num_splits=1)),
    (8, 0, dict(causal=True)),                                  # 32-row blocks
    (8, 3, dict(causal=False, num_splits=2)),
    (1, 0, dict(causal=True, window_size=(50, 0))),
    (64, 0, dict(causal=True)),                                 # tiled kernel, heads packed into the tile
    (64, 64, dict(causal=True)),
    (200, 0, dict(causal=False)),
    (64, 0, dict(causal=True, num_splits=4)),                   # tiled kernel, key ranges
])
def test_nan_outside_the_visible_keys(sq, snew, kw):
    from flash_attn_npu import flash_attn_with_kvcache
    lens = LENS + ([3000] if kw.get("num_splits", 0) == 4 else [])
    case = make_paged_case(len(lens), 32, 8, 128, 64, lens, seqlen_q=sq, seqlen_new=snew, seed=3)
    clean_k, clean_v = case["k_cache"].clone(), case["v_cache"].clone()
    unseen = ~visible_slots(case, lens)
    case["k_cache"][unseen] = float("nan")
    case["v_cache"][unseen] = float("nan")
    dev = to_dev(case)
    print("nan outside", sq, snew, kw, flush=True)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"], cache_seqlens=dev["cache_seqlens"],
                                       block_table=dev["block_table"], return_softmax_lse=True, **kw)
    torch.cuda.synchronize()
    okw = {k: v for k, v in kw.items() if k != "num_splits"}
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], clean_k, clean_v, case["k"], case["v"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], mode="fp32", **okw)
    check_out(out, ref, lse, ref_lse, "nan outside")
    seen_after = visible_slots(case, [n + snew for n in lens])
    assert torch.equal(dev["k_cache"].cpu()[seen_after].view(torch.int16), clean_k[seen_after].view(torch.int16))
    assert torch.isnan(dev["k_cache"].cpu()[~seen_after]).all() and torch.isnan(dev["v_cache"].cpu()[~seen_after]).all()


@pytest.mark.parametrize("sq,snew", [(1, 0), (2, 2)])
def test_nan_scales_outside_the_visible_keys(sq, snew):
    from flash_attn_npu import flash_attn_with_kvcache
    lens = [700, 1, 0, 257, 300]
    case = mla_case(5, 128, [n + snew for n in lens], seed=4)
    case["cache_seqlens"] = torch.tensor(lens, dtype=torch.int32)
    clean_scale = case["k_scale"].clone()
    case["k_scale"][~visible_slots(case, lens)] = float("nan")
    g = torch.Generator().manual_seed(5)
    q = torch.randn(5, sq, 128, 576, generator=g).to(torch.bfloat16)
    kn = torch.randn(5, snew, 1, 576, generator=g).to(torch.bfloat16) if snew else None
    kc, ks = case["k_cache"].cuda(), case["k_scale"].cuda()
    knd = kn.cuda() if snew else None
    kw = dict(softmax_scale=192 ** -0.5, causal=True)
    print("nan scales", sq, snew, flush=True)
    out, lse = flash_attn_with_kvcache(q.cuda(), kc, kc[..., :512], knd, knd[..., :512] if snew else None,
                                       cache_seqlens=case["cache_seqlens"].cuda(), block_table=case["block_table"].cuda(),
                                       return_softmax_lse=True, k_scale_cache=ks, **kw)
    torch.cuda.synchronize()
    kc_o = case["k_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(q, kc_o, kc_o[..., :512], kn, kn[..., :512] if snew else None, cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], k_scale_cache=clean_scale, mode="fp32", **kw)
    check_out(out, ref, lse, ref_lse, "nan scales")


def lift_pages(case, big_blocks, first):
    """The case's pools re-homed at blocks first, first+1, ... of NaN-filled pools of big_blocks blocks on the device."""
    small_k, small_v = case["k_cache"], case["v_cache"]
    n = small_k.shape[0]
    big = []
    for small in (small_k, small_v):
        pool = torch.empty((big_blocks,) + tuple(small.shape[1:]), dtype=small.dtype, device="cuda")
        pool.view(torch.int16 if small.element_size() == 2 else torch.int8).fill_(-1)       # 0xFFFF is a NaN in bf16 and fp16
        pool[first:first + n] = small.cuda()
        big.append(pool)
    return big[0], big[1], (case["block_table"] + first).cuda()


@pytest.mark.parametrize("sq,snew,num_splits", [(1, 1, 0), (1, 0, 2), (8, 2, 0), (64, 64, 0), (64, 0, 4)])
def test_pages_beyond_4_gib(sq, snew, num_splits):
    # 5 GiB per pool; the pages in use are its last ones
    from flash_attn_npu import flash_attn_with_kvcache
    lens = [1000, 33, 0, 2100]
    page, hk, d = 256, 8, 128
    case = make_paged_case(len(lens), 32, hk, d, page, lens, seqlen_q=sq, seqlen_new=snew, seed=6)
    n = case["k_cache"].shape[0]
    big_blocks = (5 << 30) // (page * hk * d * 2)
    first = big_blocks - n
    assert first * page * hk * d * 2 > (1 << 32)
    kc, vc, table = lift_pages(case, big_blocks, first)
    cos, sin = rotary_tables(4096, d)
    print("pages beyond 4 GiB", sq, snew, num_splits, "blocks", big_blocks, flush=True)
    kw = dict(causal=True, rotary_interleaved=False)
    out, lse = flash_attn_with_kvcache(case["q"].cuda(), kc, vc, case["k"].cuda() if snew else None, case["v"].cuda() if snew else None,
                                       rotary_cos=cos.cuda() if snew else None, rotary_sin=sin.cuda() if snew else None,
                                       cache_seqlens=case["cache_seqlens"].cuda(), block_table=table, num_splits=num_splits,
                                       return_softmax_lse=True, **kw)
    torch.cuda.synchronize()
    ok, ov = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], ok, ov, case["k"], case["v"], rotary_cos=cos if snew else None,
                                             rotary_sin=sin if snew else None, cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], mode="fp32", **kw)
    check_out(out, ref, lse, ref_lse, "pages beyond 4 GiB")
    assert torch.equal(kc[first:].cpu().view(torch.int16), ok.view(torch.int16)), "appended K bytes differ"
    assert torch.equal(vc[first:].cpu().view(torch.int16), ov.view(torch.int16)), "appended V bytes differ"
    assert bool((kc[first - 8:first].view(torch.int16) == -1).all()), "a block below the pages in use was written"
    del kc, vc
    torch.cuda.empty_cache()


def test_int8_pages_beyond_4_gib():
    from flash_attn_npu import flash_attn_with_kvcache
    lens, page, snew = [700, 1, 0, 2047], 256, 1
    case = mla_case(4, 128, [n + snew for n in lens], page=page, seed=8)
    case["cache_seqlens"] = torch.tensor(lens, dtype=torch.int32)
    n = case["k_cache"].shape[0]
    big_blocks = (5 << 30) // (page * 576)
    first = big_blocks - n
    assert first * page * 576 > (1 << 32)
    codes = torch.empty(big_blocks, page, 1, 576, dtype=torch.int8, device="cuda")
    codes.fill_(-1)
    codes[first:] = case["k_cache"].cuda()
    scales = torch.full((big_blocks, page, 1), float("nan"), dtype=torch.float32, device="cuda")
    scales[first:] = case["k_scale"].cuda()
    g = torch.Generator().manual_seed(9)
    q = torch.randn(4, 1, 128, 576, generator=g).to(torch.bfloat16)
    kn = torch.randn(4, snew, 1, 576, generator=g).to(torch.bfloat16)
    knd = kn.cuda()
    kw = dict(softmax_scale=192 ** -0.5, causal=True)
    print("int8 pages beyond 4 GiB, blocks", big_blocks, flush=True)
    out, lse = flash_attn_with_kvcache(q.cuda(), codes, codes[..., :512], knd, knd[..., :512], cache_seqlens=case["cache_seqlens"].cuda(),
                                       block_table=(case["block_table"] + first).cuda(), return_softmax_lse=True, k_scale_cache=scales, **kw)
    torch.cuda.synchronize()
    kc_o, ks_o = case["k_cache"].clone(), case["k_scale"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(q, kc_o, kc_o[..., :512], kn, kn[..., :512], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], k_scale_cache=ks_o, mode="fp32", **kw)
    check_out(out, ref, lse, ref_lse, "int8 pages beyond 4 GiB")
    assert torch.equal(codes[first:].cpu(), kc_o), "codes differ"
    assert torch.equal(scales[first:].cpu().view(torch.int32), ks_o.view(torch.int32)), "scales differ"
    del codes, scales
    torch.cuda.empty_cache()
