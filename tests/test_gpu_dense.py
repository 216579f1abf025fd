"""GPU parity of flash_attn_with_kvcache on dense (non-paged) caches: (batch_cache, seqlen_cache,
nheads_k, headdim) without a block_table, with and without cache_batch_idx.  Shapes follow the
reference's dense cases (tests/test_flash_attn_npu_v2.py:188-190).  The oracle sees the same cache
as one page per row behind an explicit table, which is what a dense cache is."""
import pytest
import torch

import fa_oracle as O
from helpers import check_out, check_vs_golden, rotary_tables

pytestmark = pytest.mark.gpu


def make_dense_case(B, hq, hk, d, s_cache, lens, seqlen_q=1, seqlen_new=0, dtype=torch.bfloat16, seed=0, b_cache=None):
    g = torch.Generator().manual_seed(seed)
    b_cache = B if b_cache is None else b_cache
    case = dict(
        q=torch.randn(B, seqlen_q, hq, d, generator=g).to(dtype),
        k_cache=torch.randn(b_cache, s_cache, hk, d, generator=g).to(dtype),
        v_cache=torch.randn(b_cache, s_cache, hk, d, generator=g).to(dtype),
        cache_seqlens=None if lens is None else torch.tensor(lens, dtype=torch.int32),
        k=None, v=None,
    )
    if seqlen_new:
        case["k"] = torch.randn(B, seqlen_new, hk, d, generator=g).to(dtype)
        case["v"] = torch.randn(B, seqlen_new, hk, d, generator=g).to(dtype)
    return case


def run_dense(case, cache_batch_idx=None, **kw):
    from flash_attn_npu import flash_attn_with_kvcache
    B = case["q"].shape[0]
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in case.items()}
    print("dense case", {k: (tuple(v.shape) if isinstance(v, torch.Tensor) else v) for k, v in case.items()},
          cache_batch_idx, kw, flush=True)
    idx_dev = None if cache_batch_idx is None else cache_batch_idx.cuda()
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"],
                                       cache_seqlens=dev["cache_seqlens"], cache_batch_idx=idx_dev,
                                       return_softmax_lse=True, **kw)
    torch.cuda.synchronize()
    table = (torch.arange(B, dtype=torch.int32) if cache_batch_idx is None else cache_batch_idx).view(B, 1)
    lens = case["cache_seqlens"]
    if lens is None:
        lens = torch.full((B,), case["k_cache"].shape[1], dtype=torch.int32)
    okw = {k: v for k, v in kw.items() if k != "num_splits"}
    res = []
    for mode in ("fp32", "golden"):
        kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
        res.append(O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], cache_seqlens=lens,
                                             block_table=table, mode=mode, **okw) + (kc, vc))
    return (out, lse), res[0], res[1], dev


@pytest.mark.parametrize("B,hq,hk,s_cache,causal", [(1, 8, 2, 512, True), (4, 32, 8, 2048, False), (8, 64, 8, 4096, False)])
def test_dense_decode_reference_shapes(B, hq, hk, s_cache, causal):
    # full caches, no cache_seqlens: every cached key counts
    case = make_dense_case(B, hq, hk, 128, s_cache, None, seed=B)
    got, ref, gold, _ = run_dense(case, causal=causal)
    check_out(got[0], ref[0], got[1], ref[1], "dense full")
    check_vs_golden(got[0], gold[0], got[1], gold[1], "dense full")


@pytest.mark.parametrize("s_cache", [511, 777, 1024])
def test_dense_ragged_lengths_any_cache_length(s_cache):
    # the cache length need not be a multiple of the 32-key chunk
    lens = [s_cache, 1, 300, 0][:4]
    case = make_dense_case(4, 8, 2, 128, s_cache, lens, seed=21)
    got, ref, gold, _ = run_dense(case, causal=True)
    check_out(got[0], ref[0], got[1], ref[1], f"dense s_cache={s_cache}")
    got, ref, gold, _ = run_dense(case, causal=True, num_splits=3)
    check_out(got[0], ref[0], got[1], ref[1], f"dense split s_cache={s_cache}")


def test_dense_cache_batch_idx():
    # rows of q use rows 5, 0, 3 of a larger cache
    idx = torch.tensor([5, 0, 3], dtype=torch.int32)
    case = make_dense_case(3, 16, 4, 128, 640, [640, 100, 333], seed=22, b_cache=7)
    got, ref, gold, _ = run_dense(case, cache_batch_idx=idx, causal=True)
    check_out(got[0], ref[0], got[1], ref[1], "cache_batch_idx")


@pytest.mark.parametrize("interleaved", [False, True])
def test_dense_append_rotary_bit_exact(interleaved):
    idx = torch.tensor([2, 0], dtype=torch.int32)
    case = make_dense_case(2, 8, 2, 128, 530, [400, 528], seqlen_new=2, seed=23, b_cache=3)
    cos, sin = rotary_tables(1024, 64)
    from flash_attn_npu import flash_attn_with_kvcache
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in case.items()}
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"],
                                       rotary_cos=cos.cuda(), rotary_sin=sin.cuda(), cache_seqlens=dev["cache_seqlens"],
                                       cache_batch_idx=idx.cuda(), causal=True, rotary_interleaved=interleaved,
                                       return_softmax_lse=True)
    torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], rotary_cos=cos, rotary_sin=sin,
                                             cache_seqlens=case["cache_seqlens"], block_table=idx.view(2, 1),
                                             causal=True, rotary_interleaved=interleaved, mode="fp32")
    # appended (and rotated) rows bit-exact, every other byte of the cache untouched
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))
    check_out(out, ref, lse, ref_lse, "dense append")


def test_dense_tall_query_block():
    # chunked prefill into a dense cache: the tiled kernel reads it through the same one-page table
    case = make_dense_case(2, 8, 2, 128, 700, [500, 690], seqlen_q=40, seed=24)
    got, ref, gold, _ = run_dense(case, causal=True)
    check_out(got[0], ref[0], got[1], ref[1], "dense tall")


def test_dense_rejections():
    from flash_attn_npu import flash_attn_with_kvcache
    case = make_dense_case(2, 8, 2, 128, 256, [10, 20], seqlen_new=1, seed=25)
    dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in case.items()}
    with pytest.raises(RuntimeError, match="cache_seqlens must be given to append"):
        flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"])
    with pytest.raises(RuntimeError, match="cache_batch_idx must be"):
        flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                cache_batch_idx=torch.zeros(2, dtype=torch.int64, device="cuda"))
    bt = torch.zeros(2, 1, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="Paged KVcache does not support cache_batch_idx"):
        flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                block_table=bt, cache_batch_idx=torch.zeros(2, dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("d,hq,hk,sq,s_cache,window", [(4, 512, 1, 1, 1024, (542, 647)), (4, 512, 1, 1, 1024, (-1, -1)),
                                                      (1, 4, 2, 4, 4096, (826, 973)), (96, 8, 2, 1, 640, (-1, -1)),
                                                      (192, 8, 4, 3, 300, (-1, -1))])
def test_dense_odd_head_dims(d, hq, hk, sq, s_cache, window):
    # head dimensions outside 64/128/256 (the reference's tests use 4 and 1,
    # tests/test_flash_attn_npu_v2.py:178-183) run on zero-padded copies
    case = make_dense_case(2, hq, hk, d, s_cache, [s_cache, s_cache // 3], seqlen_q=sq, dtype=torch.float16, seed=26)
    got, ref, gold, _ = run_dense(case, causal=True, window_size=window)
    assert got[0].shape[-1] == d
    check_out(got[0], ref[0], got[1], ref[1], f"d={d}")


def test_paged_odd_head_dim_append_written_back():
    from flash_attn_npu import flash_attn_with_kvcache
    from helpers import make_paged_case, to_dev
    case = make_paged_case(3, 6, 2, 80, 128, [100, 255, 128], seqlen_new=2, seed=27)
    case["cache_seqlens"][2] = 128   # second page of row 2 starts with the appended rows
    dev = to_dev(case)
    before_k = dev["k_cache"].clone()
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"],
                                       cache_seqlens=dev["cache_seqlens"], block_table=dev["block_table"], causal=True,
                                       return_softmax_lse=True)
    torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], causal=True, mode="fp32")
    assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
    assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))
    assert not torch.equal(dev["k_cache"], before_k)
    check_out(out, ref, lse, ref_lse, "d=80 append")
