"""GPU parity of the int8 latent (MLA) decode against the CPU oracle (dequantise-then-golden)."""
import math

import pytest
import torch

import fa_oracle as O
from helpers import check_out, check_vs_golden

pytestmark = pytest.mark.gpu


def mla_case(B, hq, lens, page=256, seed=0, spare=2, zero_token=False):
    g = torch.Generator().manual_seed(seed)
    pages = [max(1, math.ceil(l / page)) for l in lens]
    pool = sum(pages) + spare
    perm = torch.randperm(pool, generator=g)
    bt = torch.zeros(B, max(pages), dtype=torch.int32)
    o = 0
    for b in range(B):
        bt[b, :pages[b]] = perm[o:o + pages[b]].to(torch.int32)
        o += pages[b]
    latent = torch.randn(pool, page, 1, 576, generator=g).to(torch.bfloat16)
    if zero_token:
        latent[bt[0, 0].item(), 3] = 0          # an all-zero token: scale 0, codes 0
    code, scale = O.quantize_per_token(latent)
    q = torch.randn(B, 1, hq, 576, generator=g).to(torch.bfloat16)
    return dict(q=q, k_cache=code, k_scale=scale, block_table=bt, cache_seqlens=torch.tensor(lens, dtype=torch.int32))


def run(case):
    from flash_attn_npu import flash_attn_with_kvcache
    kc = case["k_cache"].cuda()
    print("mla", tuple(case["q"].shape), case["cache_seqlens"].tolist(), flush=True)
    out, lse = flash_attn_with_kvcache(case["q"].cuda(), kc, kc[..., :512], cache_seqlens=case["cache_seqlens"].cuda(),
                                       block_table=case["block_table"].cuda(), softmax_scale=192 ** -0.5, causal=True,
                                       return_softmax_lse=True, k_scale_cache=case["k_scale"].cuda())
    torch.cuda.synchronize()
    res = {}
    for mode in ("fp32", "golden"):
        res[mode] = O.flash_attn_with_kvcache(case["q"], case["k_cache"], case["k_cache"][..., :512],
                                              cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                              softmax_scale=192 ** -0.5, causal=True, k_scale_cache=case["k_scale"], mode=mode)
    return (out, lse), res["fp32"], res["golden"]


@pytest.mark.parametrize("hq", [128, 64])
def test_mla_basic(hq):
    case = mla_case(3, hq, [700, 2048, 33], seed=1)
    got, ref, gold = run(case)
    check_out(got[0], ref[0], got[1], ref[1], "mla")
    check_vs_golden(got[0], gold[0], got[1], gold[1], "mla")


@pytest.mark.parametrize("page,hq", [(32, 128), (96, 16), (64, 192), (256, 200)])
def test_mla_page_sizes_and_head_counts(page, hq):
    """The chunk cursors carry page and in-page offset from chunk to chunk: pages of one chunk, of three, lengths that
    end inside a chunk and on a page boundary; head counts below, at and above one 128-head unit (the last unit partly
    empty), whose q rows are fetched row-wise."""
    case = mla_case(4, hq, [page, 3 * page + 1, 1500, 31], page=page, seed=20 + page)
    got, ref, gold = run(case)
    check_out(got[0], ref[0], got[1], ref[1], f"mla page {page} heads {hq}")
    check_vs_golden(got[0], gold[0], got[1], gold[1], f"mla page {page} heads {hq}")


def test_mla_q_with_padded_head_stride():
    """q as a view whose head stride is not the head dimension (each row still contiguous and 16-byte aligned)."""
    case = mla_case(2, 128, [1000, 77], seed=31)
    got_c, ref, gold = run(case)
    wide = torch.zeros(2, 1, 128, 640, dtype=torch.bfloat16)
    wide[..., :576] = case["q"]
    strided = dict(case)
    strided["q"] = wide[..., :576]                       # stride (128*640, 128*640, 640, 1)
    assert not strided["q"].is_contiguous()
    from flash_attn_npu import flash_attn_with_kvcache
    kc = case["k_cache"].cuda()
    out, lse = flash_attn_with_kvcache(wide.cuda()[..., :576], kc, kc[..., :512], cache_seqlens=case["cache_seqlens"].cuda(),
                                       block_table=case["block_table"].cuda(), softmax_scale=192 ** -0.5, causal=True,
                                       return_softmax_lse=True, k_scale_cache=case["k_scale"].cuda())
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), got_c[0].cpu()) and torch.equal(lse.cpu(), got_c[1].cpu())


def test_mla_ragged_and_empty():
    case = mla_case(5, 128, [1, 0, 255, 257, 5000], seed=2, zero_token=True)
    got, ref, gold = run(case)
    check_out(got[0], ref[0], got[1], ref[1], "mla ragged")


def test_mla_codes_and_scales_untouched():
    case = mla_case(2, 128, [900, 300], seed=3)
    from flash_attn_npu import flash_attn_with_kvcache
    kc, ks = case["k_cache"].cuda(), case["k_scale"].cuda()
    flash_attn_with_kvcache(case["q"].cuda(), kc, kc[..., :512], cache_seqlens=case["cache_seqlens"].cuda(),
                            block_table=case["block_table"].cuda(), softmax_scale=192 ** -0.5, causal=True, k_scale_cache=ks)
    assert torch.equal(kc.cpu(), case["k_cache"]) and torch.equal(ks.cpu(), case["k_scale"])


@pytest.mark.parametrize("snew", [1, 3])
def test_mla_quantising_append_bit_exact(snew):
    # new latent rows are quantised per token on the device: codes, scales and every untouched byte
    # must equal the oracle's; attention then sees cache_seqlens + snew keys
    from flash_attn_npu import flash_attn_with_kvcache
    lens = [700, 255, 0, 2047]
    case = mla_case(4, 128, [l + snew for l in lens], seed=5)      # pages sized for the appended rows
    case["cache_seqlens"] = torch.tensor(lens, dtype=torch.int32)
    g = torch.Generator().manual_seed(55)
    k_new = torch.randn(4, snew, 1, 576, generator=g).to(torch.bfloat16)
    k_new[1, 0] = 0                                                 # an all-zero new token
    kc, ks = case["k_cache"].cuda(), case["k_scale"].cuda()
    kn = k_new.cuda()
    out, lse = flash_attn_with_kvcache(case["q"].cuda(), kc, kc[..., :512], kn, kn[..., :512],
                                       cache_seqlens=case["cache_seqlens"].cuda(), block_table=case["block_table"].cuda(),
                                       softmax_scale=192 ** -0.5, causal=True, return_softmax_lse=True, k_scale_cache=ks)
    torch.cuda.synchronize()
    kc_o, ks_o = case["k_cache"].clone(), case["k_scale"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc_o, kc_o[..., :512], k_new, k_new[..., :512],
                                             cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                             softmax_scale=192 ** -0.5, causal=True, k_scale_cache=ks_o, mode="fp32")
    assert torch.equal(kc.cpu(), kc_o), "codes differ"
    assert torch.equal(ks.cpu().view(torch.int32), ks_o.view(torch.int32)), "scales differ"
    assert not torch.equal(kc_o, case["k_cache"])
    check_out(out, ref, lse, ref_lse, "mla append")


def test_mla_append_rejections():
    from flash_attn_npu import flash_attn_with_kvcache
    case = mla_case(1, 64, [40], seed=6)
    kc, ks = case["k_cache"].cuda(), case["k_scale"].cuda()
    kn = torch.zeros(1, 1, 1, 576, dtype=torch.bfloat16, device="cuda")
    vn = torch.zeros(1, 1, 1, 512, dtype=torch.bfloat16, device="cuda")
    kw = dict(cache_seqlens=case["cache_seqlens"].cuda(), block_table=case["block_table"].cuda(), k_scale_cache=ks)
    with pytest.raises(RuntimeError, match="v must be the view"):
        flash_attn_with_kvcache(case["q"].cuda(), kc, kc[..., :512], kn, vn, **kw)
    cos = torch.ones(64, 32, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="rotary embedding is not supported with an int8"):
        flash_attn_with_kvcache(case["q"].cuda(), kc, kc[..., :512], kn, kn[..., :512], rotary_cos=cos, rotary_sin=cos, **kw)


@pytest.mark.parametrize("sq,causal,window", [(2, True, (-1, -1)), (3, True, (-1, -1)), (2, False, (-1, -1)), (4, True, (300, 0))])
def test_mla_several_query_tokens(sq, causal, window):
    # multi-token decode (speculative / multi-token prediction): every query token is its own set
    # of units with its own causal / window bound
    from flash_attn_npu import flash_attn_with_kvcache
    lens = [700, 2, 1025, 64]
    case = mla_case(4, 128, lens, seed=7)
    g = torch.Generator().manual_seed(77)
    q = torch.randn(4, sq, 128, 576, generator=g).to(torch.bfloat16)
    kc = case["k_cache"].cuda()
    print("mla multi", sq, causal, window, lens, flush=True)
    out, lse = flash_attn_with_kvcache(q.cuda(), kc, kc[..., :512], cache_seqlens=case["cache_seqlens"].cuda(),
                                       block_table=case["block_table"].cuda(), softmax_scale=192 ** -0.5, causal=causal,
                                       window_size=window, return_softmax_lse=True, k_scale_cache=case["k_scale"].cuda())
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_with_kvcache(q, case["k_cache"], case["k_cache"][..., :512], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], softmax_scale=192 ** -0.5, causal=causal,
                                             window_size=window, k_scale_cache=case["k_scale"], mode="fp32")
    assert out.shape == (4, sq, 128, 512) and lse.shape == (4, 128, sq)
    check_out(out, ref, lse, ref_lse, f"mla sq={sq}")


def test_mla_multi_token_with_append():
    from flash_attn_npu import flash_attn_with_kvcache
    sq = 2
    lens = [300, 0, 511]
    case = mla_case(3, 64, [l + sq for l in lens], seed=8)
    case["cache_seqlens"] = torch.tensor(lens, dtype=torch.int32)
    g = torch.Generator().manual_seed(88)
    q = torch.randn(3, sq, 64, 576, generator=g).to(torch.bfloat16)
    k_new = torch.randn(3, sq, 1, 576, generator=g).to(torch.bfloat16)
    kc, ks, kn = case["k_cache"].cuda(), case["k_scale"].cuda(), k_new.cuda()
    out, lse = flash_attn_with_kvcache(q.cuda(), kc, kc[..., :512], kn, kn[..., :512], cache_seqlens=case["cache_seqlens"].cuda(),
                                       block_table=case["block_table"].cuda(), softmax_scale=192 ** -0.5, causal=True,
                                       return_softmax_lse=True, k_scale_cache=ks)
    torch.cuda.synchronize()
    kc_o, ks_o = case["k_cache"].clone(), case["k_scale"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(q, kc_o, kc_o[..., :512], k_new, k_new[..., :512], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], softmax_scale=192 ** -0.5, causal=True,
                                             k_scale_cache=ks_o, mode="fp32")
    assert torch.equal(kc.cpu(), kc_o) and torch.equal(ks.cpu().view(torch.int32), ks_o.view(torch.int32))
    check_out(out, ref, lse, ref_lse, "mla multi append")


def test_mla_softcap():
    from flash_attn_npu import flash_attn_with_kvcache
    case = mla_case(2, 128, [900, 130], seed=9)
    kc = case["k_cache"].cuda()
    out, lse = flash_attn_with_kvcache(case["q"].cuda(), kc, kc[..., :512], cache_seqlens=case["cache_seqlens"].cuda(),
                                       block_table=case["block_table"].cuda(), softmax_scale=192 ** -0.5, causal=True, softcap=20.0,
                                       return_softmax_lse=True, k_scale_cache=case["k_scale"].cuda())
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], case["k_cache"], case["k_cache"][..., :512], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], softmax_scale=192 ** -0.5, causal=True, softcap=20.0,
                                             k_scale_cache=case["k_scale"], mode="fp32")
    check_out(out, ref, lse, ref_lse, "mla softcap")


def test_mla_batch_larger_than_prefix_segments():
    import random
    r = random.Random(9)
    lens = [r.choice([0, 1, 40, 300]) for _ in range(270)]
    case = mla_case(270, 64, lens, page=64, seed=10)
    got, ref, gold = run(case)
    check_out(got[0], ref[0], got[1], ref[1], "mla B=270")


def test_mla_one_key_returns_that_key():
    # the output is a convex combination of the dequantised rows: the kernel rounds P * v_scale to bf16 and divides by
    # the sum of the weights it really applied, so a row that sees a single key gives that key's values, to the
    # rounding of the output alone
    from flash_attn_npu import flash_attn_with_kvcache
    case = mla_case(6, 128, [1, 1, 1, 1, 1, 1], seed=12)
    kc = case["k_cache"].cuda()
    out = flash_attn_with_kvcache(case["q"].cuda(), kc, kc[..., :512], cache_seqlens=case["cache_seqlens"].cuda(),
                                  block_table=case["block_table"].cuda(), softmax_scale=192 ** -0.5, causal=True,
                                  k_scale_cache=case["k_scale"].cuda())
    torch.cuda.synchronize()
    for b in range(6):
        blk = int(case["block_table"][b, 0])
        want = O.dequantize_per_token(case["k_cache"][blk, 0, 0, :512], case["k_scale"][blk, 0, 0]).to(torch.bfloat16)
        diff = (out[b, 0].cpu().float() - want.float().expand(128, 512)).abs()
        # 1 / sum and the product are two more fp32 roundings: an element within 1e-7 of a bf16 tie may land on the other side
        assert (diff <= want.float().abs() * 2.0 ** -7).all() and int((diff != 0).sum()) <= 8, f"row {b}: {int((diff != 0).sum())} differ"


@pytest.mark.parametrize("magnitude", [1e-3, 1.0, 3e3])
def test_mla_split_partials_keep_the_result_inside_their_value_range(magnitude):
    """Split units of the latent kernel leave their normalised partial outputs as fp16 rows, whatever the I/O type:
    outputs of magnitude 6e-5 .. 65504 keep 11 significant bits there (outside that range they lose bits, then flush
    to zero or saturate).  Inside it the result must not depend on the partition: one sequence as ONE whole unit on
    one workgroup (no partial is written) against the same call cut over every compute unit, with latent rows
    scaled so that the outputs are small, of order one, and in the thousands."""
    from flash_attn_npu import flash_attn_with_kvcache
    from helpers import library_env
    g = torch.Generator().manual_seed(77)
    page, n = 256, 6000
    pages = math.ceil(n / page)
    latent = (torch.randn(pages + 1, page, 1, 576, generator=g) * magnitude).to(torch.bfloat16)
    code, scale = O.quantize_per_token(latent)
    q = (torch.randn(1, 1, 128, 576, generator=g) / magnitude).to(torch.bfloat16)     # keeps the scores of order one
    table = torch.randperm(pages + 1, generator=g)[:pages].to(torch.int32).view(1, pages)
    lens = torch.tensor([n], dtype=torch.int32)
    kc = code.cuda()

    def call():
        out, lse = flash_attn_with_kvcache(q.cuda(), kc, kc[..., :512], cache_seqlens=lens.cuda(), block_table=table.cuda(),
                                           softmax_scale=192 ** -0.5, causal=True, return_softmax_lse=True, k_scale_cache=scale.cuda())
        torch.cuda.synchronize()
        return out.float().cpu(), lse.cpu()

    print("mla split vs whole, magnitude", magnitude, flush=True)
    split_out, split_lse = call()
    with library_env(FA_ROCM_DECODE_WGS=1):
        whole_out, whole_lse = call()
    ref, ref_lse = O.flash_attn_with_kvcache(q, code, code[..., :512], cache_seqlens=lens, block_table=table, softmax_scale=192 ** -0.5,
                                             causal=True, k_scale_cache=scale, mode="fp32")
    size = ref.abs().max().item()
    assert 0.02 * magnitude < size < 40 * magnitude
    # both within the output bars of the fp32 reference, relative to the magnitude of the result
    for name, o in (("split", split_out), ("whole", whole_out)):
        err = (o - ref).abs()
        assert err.max().item() <= 2e-2 * max(size, 1.0) and err.mean().item() <= 2e-3 * max(size, 1.0), (name, err.max().item(), size)
    # and the two partitions agree to the rounding of the I/O type (bf16: 2^-8 of the larger magnitude), never more
    assert (split_out - whole_out).abs().max().item() <= 2.0 ** -7 * size
    torch.testing.assert_close(split_lse, whole_lse, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(split_lse, ref_lse, rtol=1e-3, atol=1e-3)
