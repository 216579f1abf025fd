"""GPU parity of the paged decode path (through the C ABI) against the CPU oracle."""
import pytest
import torch

import fa_oracle as O
from helpers import check_out, check_vs_golden, make_paged_case, rotary_tables, to_dev

pytestmark = pytest.mark.gpu


def run_both(case, **kw):
    from flash_attn_npu import flash_attn_with_kvcache
    dev = to_dev(case)
    print("case", {k: (tuple(v.shape) if isinstance(v, torch.Tensor) else v) for k, v in case.items()}, kw, flush=True)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"],
                                       cache_seqlens=dev["cache_seqlens"], block_table=dev["block_table"],
                                       return_softmax_lse=True, **kw)
    torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    okw = {k: v for k, v in kw.items() if k != "num_splits"}
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], mode="fp32", **okw)
    kc2, vc2 = case["k_cache"].clone(), case["v_cache"].clone()
    gold, gold_lse = O.flash_attn_with_kvcache(case["q"], kc2, vc2, case["k"], case["v"],
                                               cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                               mode="golden", **okw)
    return (out, lse), (ref, ref_lse), (gold, gold_lse), (dev, kc, vc)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hk", [(8, 2), (32, 8), (8, 8), (16, 1)])
def test_decode_basic(dtype, hq, hk):
    case = make_paged_case(3, hq, hk, 128, 256, [300, 511, 1025], dtype=dtype, seed=1)
    got, ref, gold, _ = run_both(case, causal=True)
    check_out(got[0], ref[0], got[1], ref[1], "decode_basic")
    check_vs_golden(got[0], gold[0], got[1], gold[1], "decode_basic")


@pytest.mark.parametrize("num_splits", [1, 2, 3, 7])
def test_decode_split_invariance(num_splits):
    case = make_paged_case(2, 16, 2, 128, 256, [4096, 2500], seed=2)
    got, ref, gold, _ = run_both(case, causal=True, num_splits=num_splits)
    check_out(got[0], ref[0], got[1], ref[1], f"splits={num_splits}")


@pytest.mark.parametrize("lens", [[1, 31, 32, 33], [255, 256, 257, 512], [0, 5, 0, 700]])
def test_decode_ragged_edges(lens):
    case = make_paged_case(4, 8, 2, 128, 256, lens, seed=3)
    got, ref, gold, _ = run_both(case, causal=True)
    check_out(got[0], ref[0], got[1], ref[1], f"lens={lens}")


def test_decode_uniform5_distribution():
    # the reference tests draw U(-5, 5): one dominant key per row
    case = make_paged_case(2, 8, 2, 128, 128, [2048, 777], seed=4, dist="uniform5")
    got, ref, gold, _ = run_both(case, causal=False)
    check_vs_golden(got[0], gold[0], got[1], gold[1], "uniform5")


@pytest.mark.parametrize("window", [(64, 0), (542, 647), (4095, 0), (0, 0), (-1, 3)])
def test_decode_window(window):
    case = make_paged_case(2, 8, 1, 128, 256, [5000, 1300], seed=5)
    got, ref, gold, _ = run_both(case, causal=False, window_size=window)
    check_out(got[0], ref[0], got[1], ref[1], f"window={window}")


@pytest.mark.parametrize("sq,hq,hk", [(2, 8, 2), (4, 4, 1), (3, 16, 8), (5, 8, 8), (2, 32, 1)])
def test_decode_multi_token_causal(sq, hq, hk):
    case = make_paged_case(2, hq, hk, 128, 256, [700, 259], seqlen_q=sq, seed=6)
    got, ref, gold, _ = run_both(case, causal=True)
    check_out(got[0], ref[0], got[1], ref[1], f"sq={sq}")


def test_decode_sq_longer_than_keys():
    # bottom-right causal with Sq > Sk: the first Sq-Sk rows see nothing -> 0 / +inf
    case = make_paged_case(1, 4, 2, 128, 256, [2], seqlen_q=5, seed=7)
    got, ref, gold, _ = run_both(case, causal=True)
    check_out(got[0], ref[0], got[1], ref[1], "sq>sk")
    assert torch.isinf(got[1][0, :, :3]).all() and (got[0][0, :3] == 0).all()


@pytest.mark.parametrize("d", [64, 256])
def test_decode_headdims(d):
    case = make_paged_case(2, 8, 2, d, 128, [900, 130], seed=8)
    got, ref, gold, _ = run_both(case, causal=True, num_splits=1)
    check_out(got[0], ref[0], got[1], ref[1], f"d={d}")
    got, ref, gold, _ = run_both(case, causal=True, num_splits=3)
    check_out(got[0], ref[0], got[1], ref[1], f"d={d} split")


def test_decode_softcap():
    case = make_paged_case(2, 8, 2, 128, 256, [600, 300], seed=9)
    got, ref, gold, _ = run_both(case, causal=True, softcap=3.0)
    check_out(got[0], ref[0], got[1], ref[1], "softcap")


@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("rot", [128, 64])
def test_append_rotary_bit_exact(interleaved, rot):
    B, hq, hk, d, page = 4, 8, 2, 128, 256
    lens = [300, 511, 256, 0]
    case = make_paged_case(B, hq, hk, d, page, lens, seqlen_new=1, seed=10)
    cos, sin = rotary_tables(1024, rot)
    got, ref, gold, (dev, kc, vc) = run_both(case, causal=True, rotary_cos=None, rotary_sin=None)
    # un-rotated append first: caches must match the oracle's bytes
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))
    check_out(got[0], ref[0], got[1], ref[1], "append")
    # rotary
    case = make_paged_case(B, hq, hk, d, page, lens, seqlen_new=1, seed=11)
    from flash_attn_npu import flash_attn_with_kvcache
    dev = to_dev(case)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"],
                                       rotary_cos=cos.cuda(), rotary_sin=sin.cuda(), cache_seqlens=dev["cache_seqlens"],
                                       block_table=dev["block_table"], causal=True, rotary_interleaved=interleaved,
                                       return_softmax_lse=True)
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], rotary_cos=cos, rotary_sin=sin,
                                             cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                             causal=True, rotary_interleaved=interleaved, mode="fp32")
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16)), "rotated K bytes differ"
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))
    check_out(out, ref, lse, ref_lse, "append+rotary")


def double_rounding_pairs(count, seed=0):
    """fp16 rotary inputs (x1, x2, sin; cos = 1) whose fp32 result x1 - x2*sin lies exactly half way between
    two fp16 values while the unrounded result does not: rounding once (a multiply-add that writes fp16
    directly) and rounding twice (fp32, then fp16) then disagree for about half of them."""
    g = torch.Generator().manual_seed(seed)
    n = 1 << 21
    x1 = (1 + torch.rand(n, generator=g)).to(torch.float16)
    x2 = (1 + torch.rand(n, generator=g)).to(torch.float16)
    sn = ((1 + torch.rand(n, generator=g)) * 2.0 ** -11).to(torch.float16)
    r32 = x1.float() - x2.float() * sn.float()                      # both operations exact or rounded once, unfused
    exact = x1.double() - x2.double() * sn.double()
    tie = ((r32.view(torch.int32) & 0x1FFF) == 0x1000) & (exact != r32.double())
    idx = tie.nonzero()[:count, 0]
    assert idx.numel() == count
    return x1[idx], x2[idx], sn[idx]


@pytest.mark.parametrize("num_splits", [0, 2])        # 0: rows appended by the attention kernel, 2: by the append kernel
@pytest.mark.parametrize("interleaved", [False, True])
def test_append_rotary_fp16_rounds_in_fp32_first(interleaved, num_splits):
    # the rotated row is defined as separately rounded fp32 operations followed by one conversion to fp16
    from flash_attn_npu import flash_attn_with_kvcache
    snew, half = 2, 64
    x1, x2, sn = double_rounding_pairs(snew * half)
    case = make_paged_case(1, 4, 1, 128, 64, [5], seqlen_q=snew, seqlen_new=snew, dtype=torch.float16, seed=21)
    k = case["k"]
    if interleaved:
        k[0, :, 0, 0::2] = x1.view(snew, half)
        k[0, :, 0, 1::2] = x2.view(snew, half)
    else:
        k[0, :, 0, :half] = x1.view(snew, half)
        k[0, :, 0, half:] = x2.view(snew, half)
    cos = torch.ones(16, half, dtype=torch.float16)
    sin = torch.zeros(16, half, dtype=torch.float16)
    sin[5:5 + snew] = sn.view(snew, half)
    dev = to_dev(case)
    flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"], rotary_cos=cos.cuda(),
                            rotary_sin=sin.cuda(), cache_seqlens=dev["cache_seqlens"], block_table=dev["block_table"],
                            causal=True, rotary_interleaved=interleaved, num_splits=num_splits)
    torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    O.append_kv(kc, vc, case["k"], case["v"], case["cache_seqlens"], case["block_table"], cos, sin, interleaved)
    rows = kc[case["block_table"][0, 0].item(), 5:5 + snew, 0]
    first = rows[:, 0::2] if interleaved else rows[:, :half]
    # numpy converts float64 to float16 in one rounding (torch goes through float32)
    once = torch.from_numpy((x1.double() - x2.double() * sn.double()).numpy().astype("float16")).view(snew, half)
    assert (first != once).sum() >= 16, "the inputs no longer tell one rounding from two"
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16)), "rotated K bytes differ"
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))


def test_append_multi_token_crosses_page():
    case = make_paged_case(2, 8, 2, 128, 256, [254, 510], seqlen_q=3, seqlen_new=3, seed=12)
    got, ref, gold, (dev, kc, vc) = run_both(case, causal=True)
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))
    check_out(got[0], ref[0], got[1], ref[1], "append3")


@pytest.mark.parametrize("window", [(0, -1), (-1, 1), (1, 1), (3, 0), (-1, 7)])
def test_decode_window_more_queries_than_keys(window):
    # Sq > Sk: the reference's host normalisation (side >= Sk unbounded, unbounded side := Sk) is not
    # mask-neutral here; kernel and oracle must agree on it
    case = make_paged_case(2, 4, 2, 128, 256, [2, 1], seqlen_q=5, seed=13)
    got, ref, gold, _ = run_both(case, causal=False, window_size=window)
    check_out(got[0], ref[0], got[1], ref[1], f"sq>sk window={window}")


@pytest.mark.parametrize("B,num_splits", [(300, 0), (700, 0), (300, 2)])
def test_decode_batch_larger_than_prefix_segments(B, num_splits):
    # the balanced partition scans the batch in 256 segments: more than 256 rows puts several rows
    # into one segment (rows with no key, short and long rows mixed)
    import random
    r = random.Random(B)
    lens = [r.choice([0, 1, 5, 33, 64, 100, 257, 600]) for _ in range(B)]
    case = make_paged_case(B, 8, 2, 128, 64, lens, seed=B)
    got, ref, gold, _ = run_both(case, causal=True, num_splits=num_splits)
    check_out(got[0], ref[0], got[1], ref[1], f"B={B}")


# Query blocks of 17-32 rows can run on three kernels; the built-in rule picks by head dimension, and the library's
# experiment settings force each of them in turn so that none goes untested whatever the rule is.
_TWO_TILE_KERNELS = {
    "rule": {},
    "wave-level, two tiles in a wave": dict(FA_ROCM_WAVE_TWO_TILES=1),
    "wave-level, tiles as units": dict(FA_ROCM_WAVE_MAX_ROWS=32),
    "workgroup-level, two tiles": dict(FA_ROCM_WAVE_MAX_ROWS=16, FA_ROCM_DECODE_MAX_ROWS=32),
    "tiled, heads packed": dict(FA_ROCM_WAVE_MAX_ROWS=16, FA_ROCM_DECODE_MAX_ROWS=16),
}


@pytest.mark.parametrize("kernel", list(_TWO_TILE_KERNELS))
@pytest.mark.parametrize("d,sq,hq,hk,kw", [
    (128, 1, 32, 1, dict(causal=True)),                              # MQA, 32 rows
    (128, 5, 8, 2, dict(causal=True)),                               # 20 rows: the second tile is partly empty
    (64, 4, 16, 2, dict(causal=True)),                               # 32 rows
    (256, 3, 18, 3, dict(causal=True)),                              # 18 rows, three kv heads
    (256, 1, 32, 1, dict(causal=False, window_size=(300, 0))),       # MQA with a window
    (128, 6, 12, 4, dict(causal=False, window_size=(100, 2))),       # 18 rows, two-sided window over several tokens
    (128, 4, 16, 2, dict(causal=True, softcap=30.0)),
])
def test_decode_two_tile_blocks_on_every_kernel(kernel, d, sq, hq, hk, kw):
    from helpers import library_env
    lens = [700, 31, 2600, 0, 259]
    case = make_paged_case(5, hq, hk, d, 64, lens, seqlen_q=sq, seqlen_new=sq, seed=40 + d + sq)
    with library_env(**_TWO_TILE_KERNELS[kernel]):
        got, ref, gold, (dev, kc, vc) = run_both(case, **kw)
    check_out(got[0], ref[0], got[1], ref[1], f"{kernel} d={d} sq={sq} {hq}q/{hk}kv")
    # the append that came with the call: bit-exact, whichever kernel followed it
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))


@pytest.mark.parametrize("kernel", list(_TWO_TILE_KERNELS))
@pytest.mark.parametrize("interleaved", [False, True])
def test_decode_two_tile_blocks_fp16_with_rotary(kernel, interleaved):
    """24 rows (three tokens x eight heads of one group) in fp16 with the rotation applied to q and to the appended keys:
    q rows of one tile belong to different tokens, i.e. different rotation angles and causal bounds."""
    from helpers import library_env
    from flash_attn_npu import flash_attn_with_kvcache
    lens = [515, 64, 0, 1300]
    case = make_paged_case(4, 16, 2, 128, 64, lens, seqlen_q=3, seqlen_new=3, dtype=torch.float16, seed=91)
    cos, sin = rotary_tables(2048, 64)
    cos, sin = cos.to(torch.float16), sin.to(torch.float16)
    dev = to_dev(case)
    print("case", kernel, interleaved, flush=True)
    with library_env(**_TWO_TILE_KERNELS[kernel]):
        out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"],
                                           rotary_cos=cos.cuda(), rotary_sin=sin.cuda(), cache_seqlens=dev["cache_seqlens"],
                                           block_table=dev["block_table"], causal=True, rotary_interleaved=interleaved,
                                           return_softmax_lse=True)
        torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], rotary_cos=cos, rotary_sin=sin,
                                             cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                             causal=True, rotary_interleaved=interleaved, mode="fp32")
    check_out(out, ref, lse, ref_lse, f"{kernel} fp16 rotary")
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))


@pytest.mark.parametrize("d", [256, 128, 64])
def test_decode_two_tile_blocks_split_over_many_workers(d):
    """One long sequence, 32 rows: every unit is cut over many workers and merged; the wave-level kernel (two tiles in
    one wave up to d = 128, 16-row units at d = 256) against the other kernels and the oracle."""
    from helpers import library_env
    case = make_paged_case(1, 32, 1, d, 256, [40000], seed=77)
    outs = {}
    for kernel, env in _TWO_TILE_KERNELS.items():
        with library_env(**env):
            got, ref, gold, _ = run_both(case, causal=True)
        check_out(got[0], ref[0], got[1], ref[1], kernel)
        outs[kernel] = got[0].float().cpu()
    for kernel, o in outs.items():
        assert (o - outs["rule"]).abs().max().item() <= 2e-3, kernel
