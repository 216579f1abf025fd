"""GPU parity of the tiled forward (varlen prefill, paged varlen, tall kvcache blocks) against the
CPU oracle.  Shapes follow the reference's varlen cases (tests/test_flash_attn_npu_v2.py:522-560)."""
import pytest
import torch

import fa_oracle as O
from helpers import check_compare_rule, check_out, check_vs_golden, library_env, make_paged_case, to_dev

pytestmark = pytest.mark.gpu


def varlen_case(seqs_q, seqs_k, hq, hk, d, dtype=torch.bfloat16, seed=0, dist="normal"):
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape):
        if dist == "normal":
            return torch.randn(*shape, generator=g)
        return -5.0 + 10.0 * torch.rand(*shape, generator=g)

    tq, tk = sum(seqs_q), sum(seqs_k)
    cu_q = torch.tensor([0] + list(torch.tensor(seqs_q).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(seqs_k).cumsum(0)), dtype=torch.int32)
    return dict(q=rnd(tq, hq, d).to(dtype), k=rnd(tk, hk, d).to(dtype), v=rnd(tk, hk, d).to(dtype),
                cu_q=cu_q, cu_k=cu_k, max_q=max(seqs_q), max_k=max(seqs_k))


def check_paged(out, ref, lse, ref_lse, what=""):
    """The bars of the paged-varlen tests: the fp32 bars plus the element-wise rule of the reference's own paged-varlen
    tests (its fourth API generation)."""
    check_out(out, ref, lse, ref_lse, what)
    check_compare_rule(out, ref, what)


def run_varlen(c, **kw):
    from flash_attn_npu import flash_attn_varlen_func
    print("varlen", tuple(c["q"].shape), tuple(c["k"].shape), c["cu_q"].tolist(), c["cu_k"].tolist(), kw, flush=True)
    out, lse, _ = flash_attn_varlen_func(c["q"].cuda(), c["k"].cuda(), c["v"].cuda(), c["cu_q"].cuda(), c["cu_k"].cuda(),
                                         c["max_q"], c["max_k"], return_attn_probs=True, **kw)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_varlen(c["q"], c["k"], c["v"], c["cu_q"], c["cu_k"], c["max_q"], c["max_k"], mode="fp32", **kw)
    gold, gold_lse = O.flash_attn_varlen(c["q"], c["k"], c["v"], c["cu_q"], c["cu_k"], c["max_q"], c["max_k"], mode="golden", **kw)
    return (out, lse), (ref, ref_lse), (gold, gold_lse)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
def test_varlen_basic(dtype, causal):
    c = varlen_case([128, 300, 77, 512], [128, 300, 77, 512], 8, 2, 128, dtype=dtype, seed=1)
    got, ref, gold = run_varlen(c, causal=causal)
    check_out(got[0], ref[0], got[1], ref[1], "varlen_basic")
    check_vs_golden(got[0], gold[0], got[1], gold[1], "varlen_basic")


@pytest.mark.parametrize("seqs_q,seqs_k", [([100, 257], [300, 257]), ([300, 64], [100, 700]), ([1, 129, 5], [64, 130, 1000])])
@pytest.mark.parametrize("causal", [False, True])
def test_varlen_sq_ne_sk(seqs_q, seqs_k, causal):
    c = varlen_case(seqs_q, seqs_k, 4, 4, 128, seed=2)
    got, ref, gold = run_varlen(c, causal=causal)
    check_out(got[0], ref[0], got[1], ref[1], "sq_ne_sk")


@pytest.mark.parametrize("d", [64, 256, 111, 192])
def test_varlen_headdims(d):
    c = varlen_case([200, 130], [200, 130], 5 if d == 111 else 4, 1, d, seed=3)
    got, ref, gold = run_varlen(c, causal=True)
    check_out(got[0], ref[0], got[1], ref[1], f"d={d}")


@pytest.mark.parametrize("window", [(64, 0), (100, 30), (-1, 17), (5, -1), (0, 0)])
def test_varlen_window(window):
    c = varlen_case([300, 150], [300, 400], 4, 2, 128, seed=4)
    got, ref, gold = run_varlen(c, causal=False, window_size=window)
    check_out(got[0], ref[0], got[1], ref[1], f"window={window}")


def test_varlen_softcap_and_uniform5():
    c = varlen_case([256, 100], [256, 100], 4, 2, 128, seed=5)
    got, ref, gold = run_varlen(c, causal=True, softcap=5.0)
    check_out(got[0], ref[0], got[1], ref[1], "softcap")
    c = varlen_case([512, 64], [512, 64], 4, 1, 128, seed=6, dist="uniform5")
    got, ref, gold = run_varlen(c, causal=True)
    check_vs_golden(got[0], gold[0], got[1], gold[1], "uniform5")


def test_varlen_per_sequence_independence():
    from flash_attn_npu import flash_attn_varlen_func
    c = varlen_case([150, 260, 33], [150, 260, 33], 4, 2, 128, seed=7)
    q, k, v = c["q"].cuda(), c["k"].cuda(), c["v"].cuda()
    full = flash_attn_varlen_func(q, k, v, c["cu_q"].cuda(), c["cu_k"].cuda(), c["max_q"], c["max_k"], causal=True)
    for b in range(3):
        a, e = int(c["cu_q"][b]), int(c["cu_q"][b + 1])
        cu = torch.tensor([0, e - a], dtype=torch.int32).cuda()
        one = flash_attn_varlen_func(q[a:e], k[a:e], v[a:e], cu, cu, e - a, e - a, causal=True)
        assert torch.equal(one, full[a:e])


def test_varlen_paged_kv():
    from flash_attn_npu import flash_attn_varlen_func
    lens_k = [700, 130, 1025]
    lens_q = [64, 130, 300]
    case = make_paged_case(3, 8, 2, 128, 256, lens_k, seed=8)
    g = torch.Generator().manual_seed(9)
    q = torch.randn(sum(lens_q), 8, 128, generator=g).to(torch.bfloat16)
    cu_q = torch.tensor([0, 64, 194, 494], dtype=torch.int32)
    cu_k = torch.tensor([0, 700, 830, 1855], dtype=torch.int32)
    out, lse, _ = flash_attn_varlen_func(q.cuda(), case["k_cache"].cuda(), case["v_cache"].cuda(), cu_q.cuda(), cu_k.cuda(),
                                         max(lens_q), max(lens_k), causal=True, return_attn_probs=True,
                                         block_table=case["block_table"].cuda())
    kl = torch.cat([O.gather_paged(case["k_cache"], case["block_table"][b], lens_k[b]) for b in range(3)])
    vl = torch.cat([O.gather_paged(case["v_cache"], case["block_table"][b], lens_k[b]) for b in range(3)])
    ref, ref_lse = O.flash_attn_varlen(q, kl, vl, cu_q, cu_k, max(lens_q), max(lens_k), causal=True, mode="fp32")
    check_paged(out, ref, lse, ref_lse, "paged varlen")


@pytest.mark.parametrize("sq,hq,hk", [(128, 8, 2), (1024, 4, 4), (33, 8, 1), (17, 16, 2)])
def test_kvcache_tall_query_blocks(sq, hq, hk):
    # chunked prefill through the kvcache call: seqlen_q * group > 32 runs on the tiled kernel
    from flash_attn_npu import flash_attn_with_kvcache
    case = make_paged_case(2, hq, hk, 128, 128, [2048, 1100], seqlen_q=sq, seqlen_new=0, seed=10)
    dev = to_dev(case)
    for causal in (True, False):
        out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                           block_table=dev["block_table"], causal=causal, return_softmax_lse=True)
        ref, ref_lse = O.flash_attn_with_kvcache(case["q"], case["k_cache"], case["v_cache"],
                                                 cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                                 causal=causal, mode="fp32")
        check_out(out, ref, lse, ref_lse, f"tall sq={sq} causal={causal}")


def test_kvcache_tall_with_append():
    from flash_attn_npu import flash_attn_with_kvcache
    case = make_paged_case(2, 8, 2, 128, 256, [500, 100], seqlen_q=200, seqlen_new=200, seed=11)
    dev = to_dev(case)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"],
                                       cache_seqlens=dev["cache_seqlens"], block_table=dev["block_table"], causal=True,
                                       return_softmax_lse=True)
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], causal=True, mode="fp32")
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    check_out(out, ref, lse, ref_lse, "tall append")


@pytest.mark.parametrize("window", [(0, -1), (-1, 1), (2, 2), (-1, 40)])
def test_varlen_window_more_queries_than_keys(window):
    c = varlen_case([200, 40], [30, 90], 4, 2, 128, seed=12)
    got, ref, gold = run_varlen(c, causal=False, window_size=window)
    check_out(got[0], ref[0], got[1], ref[1], f"sq>sk window={window}")


@pytest.mark.parametrize("causal", [False, True])
def test_dense_batch_functions(causal):
    # flash_attn_func and the packed wrappers (reference flash_attn_npu_interface.py:972-1341) are the
    # varlen kernel on equal-length sequences
    from flash_attn_npu import (flash_attn_func, flash_attn_kvpacked_func, flash_attn_qkvpacked_func,
                                flash_attn_varlen_kvpacked_func, flash_attn_varlen_qkvpacked_func)
    B, sq, sk, hq, hk, d = 3, 200, 333, 8, 2, 128
    c = varlen_case([sq] * B, [sk] * B, hq, hk, d, seed=40)
    ref, ref_lse = O.flash_attn_varlen(c["q"], c["k"], c["v"], c["cu_q"], c["cu_k"], sq, sk, mode="fp32", causal=causal)
    q4, k4, v4 = c["q"].view(B, sq, hq, d).cuda(), c["k"].view(B, sk, hk, d).cuda(), c["v"].view(B, sk, hk, d).cuda()
    out, lse, _ = flash_attn_func(q4, k4, v4, causal=causal, return_attn_probs=True)
    torch.cuda.synchronize()
    assert out.shape == (B, sq, hq, d) and lse.shape == (B, hq, sq)
    check_out(out.reshape(B * sq, hq, d), ref, lse.permute(1, 0, 2).reshape(hq, B * sq), ref_lse, "flash_attn_func")
    kv = torch.stack([k4, v4], dim=2)
    out2 = flash_attn_kvpacked_func(q4, kv, causal=causal)
    assert torch.equal(out2, out)
    out3 = flash_attn_varlen_kvpacked_func(q4.reshape(B * sq, hq, d), kv.reshape(B * sk, 2, hk, d), c["cu_q"].cuda(),
                                           c["cu_k"].cuda(), sq, sk, causal=causal)
    assert torch.equal(out3.reshape(B, sq, hq, d), out)
    # qkv packed needs equal head counts and lengths
    c2 = varlen_case([sq] * B, [sq] * B, 4, 4, d, seed=41)
    ref2, _ = O.flash_attn_varlen(c2["q"], c2["k"], c2["v"], c2["cu_q"], c2["cu_k"], sq, sq, mode="fp32", causal=causal)
    qkv = torch.stack([c2["q"], c2["k"], c2["v"]], dim=1).cuda()          # (total, 3, H, D)
    o4 = flash_attn_varlen_qkvpacked_func(qkv, c2["cu_q"].cuda(), sq, causal=causal)
    o5 = flash_attn_qkvpacked_func(qkv.view(B, sq, 3, 4, d), causal=causal)
    torch.cuda.synchronize()
    check_out(o4, ref2, None, None, "varlen_qkvpacked")
    assert torch.equal(o5.reshape(B * sq, 4, d), o4)


@pytest.mark.parametrize("interleaved,causal", [(False, True), (True, True), (False, False)])
def test_tall_query_block_with_append_and_rotary(interleaved, causal):
    # chunked prefill through the kvcache call: 40 new tokens x group 4 = 160 query rows go to the
    # tiled kernel; K is rotated by the append, q by a pre-pass into the workspace
    from flash_attn_npu import flash_attn_with_kvcache
    from helpers import rotary_tables
    case = make_paged_case(2, 8, 2, 128, 128, [300, 77], seqlen_q=40, seqlen_new=40, seed=50)
    cos, sin = rotary_tables(512, 64)
    dev = to_dev(case)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"], rotary_cos=cos.cuda(),
                                       rotary_sin=sin.cuda(), cache_seqlens=dev["cache_seqlens"], block_table=dev["block_table"],
                                       causal=causal, rotary_interleaved=interleaved, return_softmax_lse=True)
    torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], rotary_cos=cos, rotary_sin=sin,
                                             cache_seqlens=case["cache_seqlens"], block_table=case["block_table"], causal=causal,
                                             rotary_interleaved=interleaved, mode="fp32")
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))
    check_out(out, ref, lse, ref_lse, "tall rotary")


@pytest.mark.parametrize("sq,hq,hk,d", [(16, 64, 8, 128), (20, 12, 2, 128), (9, 24, 3, 64), (40, 10, 2, 256), (100, 6, 2, 128)])
@pytest.mark.parametrize("causal,window", [(True, (-1, -1)), (False, (-1, -1)), (False, (30, 3)), (True, (100, 0))])
def test_kvcache_short_blocks_packed_heads(sq, hq, hk, d, causal, window):
    # seqlen_q * group > 32 with fewer than 128 query rows per head: the tile rows are (query, head)
    # pairs of one kv head; groups that do not divide 128 (6, 8 of 3, 5) put a query's heads in two tiles
    from flash_attn_npu import flash_attn_with_kvcache
    case = make_paged_case(3, hq, hk, d, 64, [700, 64, sq], seqlen_q=sq, seed=31, dtype=torch.float16)
    dev = to_dev(case)
    print("packed heads", sq, hq, hk, d, causal, window, flush=True)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                       block_table=dev["block_table"], causal=causal, window_size=window,
                                       return_softmax_lse=True)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], case["k_cache"], case["v_cache"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], causal=causal, window_size=window, mode="fp32")
    check_out(out, ref, lse, ref_lse, f"packed sq={sq} g={hq // hk}")


@pytest.mark.parametrize("causal", [False, True])
def test_varlen_short_sequences_packed_heads(causal):
    # packed sequences all shorter than a tile, GQA group 5: ragged (query, head) rows, some
    # sequences with more queries than keys, one of a single token
    c = varlen_case([5, 40, 17, 1, 90], [300, 40, 9, 64, 1000], 10, 2, 128, seed=32)
    got, ref, gold = run_varlen(c, causal=causal)
    check_out(got[0], ref[0], got[1], ref[1], "varlen packed heads")
    check_vs_golden(got[0], gold[0], got[1], gold[1], "varlen packed heads")


@pytest.mark.parametrize("num_splits", [0, 2, 5])
@pytest.mark.parametrize("sq,hq,hk,d", [(16, 64, 8, 128), (128, 8, 2, 128), (300, 4, 4, 64), (70, 6, 2, 256)])
@pytest.mark.parametrize("causal,window", [(True, (-1, -1)), (False, (-1, -1)), (True, (700, 0))])
def test_kvcache_tall_blocks_split_keys(sq, hq, hk, d, causal, window, num_splits):
    # few sequences with tall query blocks over long contexts: the tiled kernel cuts every unit's
    # keys into ranges (num_splits 0: as many as fill the device, 2 / 5: at most that many) and the
    # combine kernel merges them; rows of very different lengths, one shorter than the query block
    from flash_attn_npu import flash_attn_with_kvcache
    lens = [5000, 40] if sq <= 128 else [3000, 301]
    case = make_paged_case(2, hq, hk, d, 128, lens, seqlen_q=sq, seed=41)
    dev = to_dev(case)
    print("tall split", sq, hq, hk, d, causal, window, num_splits, flush=True)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                       block_table=dev["block_table"], causal=causal, window_size=window,
                                       num_splits=num_splits, return_softmax_lse=True)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], case["k_cache"], case["v_cache"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], causal=causal, window_size=window, mode="fp32")
    check_out(out, ref, lse, ref_lse, f"tall split sq={sq} n={num_splits}")


def test_kvcache_tall_split_with_append_and_rotary():
    # the workspace holds the rotated q in front of the partials
    from flash_attn_npu import flash_attn_with_kvcache
    from helpers import rotary_tables
    case = make_paged_case(1, 16, 2, 128, 256, [6000], seqlen_q=24, seqlen_new=24, seed=42)
    cos, sin = rotary_tables(8192, 128)
    dev = to_dev(case)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"], rotary_cos=cos.cuda(),
                                       rotary_sin=sin.cuda(), cache_seqlens=dev["cache_seqlens"],
                                       block_table=dev["block_table"], causal=True, rotary_interleaved=False,
                                       return_softmax_lse=True)
    torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], rotary_cos=cos, rotary_sin=sin,
                                             cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                             causal=True, rotary_interleaved=False, mode="fp32")
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    check_out(out, ref, lse, ref_lse, "tall split append rotary")


def test_varlen_empty_sequences():
    # a sequence without query tokens, one without keys (its rows: 0 and +inf), one with neither
    from flash_attn_npu import flash_attn_varlen_func
    c = varlen_case([40, 0, 25, 0, 130], [40, 70, 0, 0, 300], 8, 2, 128, seed=51)
    for causal in (False, True):
        got, ref, gold = run_varlen(c, causal=causal)
        check_out(got[0], ref[0], got[1], ref[1], "empty sequences")
        a, e = int(c["cu_q"][2]), int(c["cu_q"][3])
        assert torch.count_nonzero(got[0][a:e]) == 0 and torch.isinf(got[1][:, a:e]).all()
    total0 = torch.zeros(0, 8, 128, dtype=torch.bfloat16, device="cuda")
    cu0 = torch.zeros(3, dtype=torch.int32, device="cuda")
    out = flash_attn_varlen_func(total0, c["k"].cuda(), c["v"].cuda(), cu0, c["cu_k"].cuda()[:3], 1, 70)
    assert out.shape == (0, 8, 128)


def paged_ragged(lens_q, lens_k, hq, hk, d, page, seed, dtype=torch.bfloat16):
    case = make_paged_case(len(lens_k), hq, hk, d, page, lens_k, dtype=dtype, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    q = torch.randn(sum(lens_q), hq, d, generator=g).to(dtype)
    cu_q = torch.tensor([0] + torch.tensor(lens_q).cumsum(0).tolist(), dtype=torch.int32)
    cu_k = torch.tensor([0] + torch.tensor(lens_k).cumsum(0).tolist(), dtype=torch.int32)
    kl = torch.cat([O.gather_paged(case["k_cache"], case["block_table"][b], lens_k[b]) for b in range(len(lens_k))])
    vl = torch.cat([O.gather_paged(case["v_cache"], case["block_table"][b], lens_k[b]) for b in range(len(lens_k))])
    return case, q, cu_q, cu_k, kl, vl


@pytest.mark.parametrize("num_splits", [0, 1, 3, 64])
@pytest.mark.parametrize("hq,hk,d", [(8, 2, 128), (4, 4, 64), (6, 1, 256)])
@pytest.mark.parametrize("causal,window", [(True, (-1, -1)), (False, (-1, -1)), (True, (900, 0)), (False, (2000, 100))])
def test_varlen_paged_ragged_blocks_split_keys(hq, hk, d, causal, window, num_splits):
    # a mixed batch over a paged cache: single-token rows, a chunk of a long prompt, an empty query block, a
    # sequence shorter than one range; every sequence's keys are cut into ranges and merged per token
    from flash_attn_npu.flash_attn_npu import varlen_fwd
    lens_q = [1, 300, 1, 0, 17, 40]
    lens_k = [5000, 3100, 40, 700, 2100, 0]
    case, q, cu_q, cu_k, kl, vl = paged_ragged(lens_q, lens_k, hq, hk, d, 64, seed=31)
    print("ragged split", hq, hk, d, causal, window, num_splits, flush=True)
    out, lse, _, _ = varlen_fwd(q.cuda(), case["k_cache"].cuda(), case["v_cache"].cuda(), None, cu_q.cuda(), None,
                                case["cache_seqlens"].cuda(), None, case["block_table"].cuda(), None, max(lens_q), max(lens_k),
                                0.0, d ** -0.5, False, causal, window[0], window[1], 0.0, False, None, num_splits=num_splits)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_varlen(q, kl, vl, cu_q, cu_k, max(lens_q), max(lens_k), causal=causal, window_size=window, mode="fp32")
    check_paged(out, ref, lse, ref_lse, "ragged split")


@pytest.mark.parametrize("causal,window,softcap", [(True, (-1, -1), 0.0), (False, (-1, -1), 0.0), (True, (1500, 0), 0.0),
                                                     (False, (3000, 7), 0.0), (True, (-1, -1), 20.0)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_varlen_paged_short_blocks_on_the_decode_kernels(causal, window, softcap, dtype):
    # a prompt chunk among decode rows and speculative blocks: blocks of 1 .. 4 tokens (16 rows of 4 q heads per kv
    # head) are computed by the decode kernels, the others by the tiled kernel; both against the oracle, and against
    # the same call with the routing switched off
    import os
    from flash_attn_npu.flash_attn_npu import varlen_fwd
    lens_q = [1, 1, 400, 1, 0, 4, 2, 1, 5, 3, 1, 2]
    lens_k = [4000, 1, 2500, 0, 300, 777, 64, 6000, 900, 2, 130, 1]
    hq, hk, d = 16, 4, 128
    case, q, cu_q, cu_k, kl, vl = paged_ragged(lens_q, lens_k, hq, hk, d, 128, seed=41, dtype=dtype)
    dev = [q.cuda(), case["k_cache"].cuda(), case["v_cache"].cuda(), cu_q.cuda(), case["cache_seqlens"].cuda(), case["block_table"].cuda()]

    def call():
        out, lse, _, _ = varlen_fwd(dev[0], dev[1], dev[2], None, dev[3], None, dev[4], None, dev[5], None, max(lens_q), max(lens_k),
                                    0.0, d ** -0.5, False, causal, window[0], window[1], softcap, False, None)
        torch.cuda.synchronize()
        return out, lse

    print("short blocks", causal, window, softcap, dtype, flush=True)
    out, lse = call()
    ref, ref_lse = O.flash_attn_varlen(q, kl, vl, cu_q, cu_k, max(lens_q), max(lens_k), causal=causal, window_size=window,
                                       softcap=softcap, mode="fp32")
    check_paged(out, ref, lse, ref_lse, "short blocks")
    with library_env(FA_ROCM_NO_SHORT_BLOCKS=1):
        out2, lse2 = call()
    check_paged(out2, ref, lse2, ref_lse, "short blocks, tiled kernel only")
    short = torch.tensor([1 <= n <= 4 for n in lens_q for _ in range(n)])
    assert torch.equal(out[~short].cpu(), out2[~short].cpu()), "rows of the tiled kernel changed with the routing"
    assert not torch.equal(out[short].cpu(), out2[short].cpu()), "the short blocks did not take the other path"


@pytest.mark.parametrize("causal,window", [(True, (-1, -1)), (False, (-1, -1)), (False, (500, 3))])
@pytest.mark.parametrize("lens_q,hq,hk", [([1, 1, 0, 1, 1], 8, 2), ([2, 4, 0, 1, 3], 8, 2), ([2, 1, 0, 2, 2], 16, 2), ([8, 3, 0, 1, 5], 4, 4)])
def test_varlen_paged_all_blocks_short(causal, window, lens_q, hq, hk):
    # no block is longer than the decode launch's slots: the whole call runs on the decode kernels (empty blocks
    # have no rows to write)
    from flash_attn_npu.flash_attn_npu import varlen_fwd
    lens_k = [3000, 1, 500, 0, 1025]
    d = 128
    case, q, cu_q, cu_k, kl, vl = paged_ragged(lens_q, lens_k, hq, hk, d, 64, seed=43)
    out, lse, _, _ = varlen_fwd(q.cuda(), case["k_cache"].cuda(), case["v_cache"].cuda(), None, cu_q.cuda(), None,
                                case["cache_seqlens"].cuda(), None, case["block_table"].cuda(), None, max(lens_q), max(lens_k),
                                0.0, d ** -0.5, False, causal, window[0], window[1], 0.0, False, None)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_varlen(q, kl, vl, cu_q, cu_k, max(lens_q), max(lens_k), causal=causal, window_size=window, mode="fp32")
    check_paged(out, ref, lse, ref_lse, "all blocks short")


def test_varlen_paged_small_mixed_batch():
    # one prompt chunk and two decode rows: the rule that calls a batch uneven looks at the blocks other than the longest
    import ctypes as C
    from flash_attn_npu.flash_attn_npu import varlen_fwd
    lens_q, lens_k = [1, 300, 1], [5000, 4000, 129]
    hq, hk, d = 8, 2, 128
    case, q, cu_q, cu_k, kl, vl = paged_ragged(lens_q, lens_k, hq, hk, d, 64, seed=47)
    out, lse, _, _ = varlen_fwd(q.cuda(), case["k_cache"].cuda(), case["v_cache"].cuda(), None, cu_q.cuda(), None,
                                case["cache_seqlens"].cuda(), None, case["block_table"].cuda(), None, max(lens_q), max(lens_k),
                                0.0, d ** -0.5, False, True, -1, -1, 0.0, False, None)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_varlen(q, kl, vl, cu_q, cu_k, max(lens_q), max(lens_k), causal=True, mode="fp32")
    check_paged(out, ref, lse, ref_lse, "small mixed batch")


@pytest.mark.parametrize("page", [32, 96, 160])
@pytest.mark.parametrize("d,dtype", [(128, torch.bfloat16), (64, torch.float16), (256, torch.bfloat16)])
def test_tall_query_block_over_pages_that_a_tile_straddles(page, d, dtype):
    """Pages that are no multiple of the 64-key tile: a tile then lies in two or three pages and every row of it takes
    its own page-table entry (the path of the ragged end of a sequence); pages of 64 keys and more give a whole tile
    one base address.  Lengths that end inside a tile, on a tile and on a page."""
    from flash_attn_npu import flash_attn_with_kvcache
    lens = [5 * page + 7, 64, page, 1000]
    case = make_paged_case(len(lens), 8, 2, d, page, lens, seqlen_q=40, seqlen_new=0, dtype=dtype, seed=60 + page)
    dev = to_dev(case)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                       block_table=dev["block_table"], causal=True, return_softmax_lse=True)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], case["k_cache"], case["v_cache"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], causal=True, mode="fp32")
    check_out(out, ref, lse, ref_lse, f"page {page} d {d}")
