"""GPU parity of the flash_attn_npu_3 call surface (page_table, token-major q with cu_seqlens_q,
num_splits, scheduler metadata) against the CPU oracle.  Cases follow the reference's own tests of
that surface: tests/test_flash_attn_npu_v3.py:236-420 (layouts BSND / TND x dense, packed, paged
caches, num_splits 0 and 2), tests/test_flash_attn_npu_v3_metadata.py:178-208 (metadata with every
entry point) and tests/test_flash_attn_npu_v3_graph.py:55-123 (capture and replay)."""
import pytest
import torch

import fa_oracle as O
from helpers import check_out, check_vs_golden, make_paged_case, rotary_tables, to_dev

pytestmark = pytest.mark.gpu

BF, FP = torch.bfloat16, torch.float16


def cu(lengths):
    out = [0]
    for n in lengths:
        out.append(out[-1] + n)
    return torch.tensor(out, dtype=torch.int32)


def packed_from_pages(case, lens):
    ks = [O.gather_paged(case["k_cache"], case["block_table"][b], lens[b]) for b in range(len(lens))]
    vs = [O.gather_paged(case["v_cache"], case["block_table"][b], lens[b]) for b in range(len(lens))]
    return torch.cat(ks), torch.cat(vs)


# (dtype, batch, heads, kv_heads, q_seqlen, kv_seqlen, head_size, causal, wl, wr, softcap): a cut of
# the reference's matrix that keeps every query-block height class, D = 128 / 256, windows, softcap
BSND_CASES = [
    (BF, 1, 32, 8, 128, 4096, 128, False, -1, -1, 0.0),
    (BF, 2, 16, 4, 256, 2048, 128, True, -1, -1, 0.0),
    (BF, 1, 32, 4, 65, 2048, 256, False, -1, -1, 0.0),
    (BF, 2, 24, 2, 6, 2048, 128, False, -1, -1, 0.0),
    (BF, 4, 32, 2, 10, 4096, 128, False, -1, -1, 0.0),
    (BF, 2, 24, 2, 6, 2048, 256, False, -1, -1, 0.0),
    (BF, 2, 64, 8, 1, 4096, 256, False, -1, -1, 30.0),
    (BF, 4, 64, 4, 32, 512, 128, False, -1, -1, 30.0),
    (BF, 1, 1, 1, 1024, 1024, 128, True, 512, 0, 30.0),
    (BF, 1, 1, 1, 1024, 1024, 128, False, -128, 1024, 30.0),
]


@pytest.mark.parametrize("paged", [0, 1])
@pytest.mark.parametrize("case", BSND_CASES, ids=lambda c: "-".join(str(x).replace("torch.", "") for x in c))
def test_v3_kvcache_bsnd(case, paged):
    from flash_attn_npu_3 import flash_attn_with_kvcache
    dtype, B, hq, hk, sq, sk, d, causal, wl, wr, softcap = case
    print("v3 bsnd", case, paged, flush=True)
    if paged:
        c = make_paged_case(B, hq, hk, d, 128, [sk] * B, seqlen_q=sq, dtype=dtype, seed=sq + sk, dist="uniform5")
        table = c["block_table"]
    else:
        g = torch.Generator().manual_seed(sq + sk)
        c = dict(q=(10 * torch.rand(B, sq, hq, d, generator=g) - 5).to(dtype),
                 k_cache=(10 * torch.rand(B, sk, hk, d, generator=g) - 5).to(dtype),
                 v_cache=(10 * torch.rand(B, sk, hk, d, generator=g) - 5).to(dtype),
                 cache_seqlens=torch.full((B,), sk, dtype=torch.int32))
        table = torch.arange(B, dtype=torch.int32).view(B, 1)
    dev = to_dev(c)
    out, lse, *rest = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], None, None, None,
                                              cache_seqlens=dev["cache_seqlens"],
                                              page_table=dev["block_table"] if paged else None, causal=causal,
                                              window_size=[wl, wr], softcap=softcap, return_softmax_lse=True)
    torch.cuda.synchronize()
    assert len(rest) == 2 and lse.shape == (B, hq, sq)
    kw = dict(cache_seqlens=c["cache_seqlens"], block_table=table, causal=causal, window_size=(wl, wr), softcap=softcap)
    gold, gold_lse = O.flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], mode="golden", **kw)
    check_vs_golden(out, gold, lse, gold_lse, str(case))


# (dtype, batch, heads, kv_heads, q_seqlen, kv_seqlen, head_size, causal, softcap)
TND_CASES = [
    (BF, 4, 32, 32, 48, 2048, 128, False, 0.0),
    (BF, 2, 32, 8, 65, 2048, 128, False, 0.0),
    (BF, 1, 64, 4, 2, 2048, 128, False, 0.0),
    (BF, 1, 64, 8, 4, 4096, 128, True, 0.0),
    (BF, 1, 32, 4, 7, 2048, 128, False, 0.0),
    (BF, 1, 32, 8, 16, 2048, 256, False, 0.0),
    (BF, 1, 10, 2, 15, 2048, 128, False, 0.0),
    (BF, 1, 10, 2, 10, 4096, 256, True, 0.0),
    (BF, 1, 32, 4, 1, 2048, 128, False, 30.0),
    (BF, 1, 64, 4, 8, 2048, 128, True, 30.0),
    (BF, 1, 32, 8, 13, 2048, 256, False, 30.0),
]


@pytest.mark.parametrize("num_splits", [0, 2])
@pytest.mark.parametrize("case", TND_CASES, ids=lambda c: "-".join(str(x).replace("torch.", "") for x in c))
def test_v3_kvcache_tnd_paged(case, num_splits):
    from flash_attn_npu_3 import flash_attn_with_kvcache
    dtype, B, hq, hk, sq, sk, d, causal, softcap = case
    print("v3 tnd paged", case, num_splits, flush=True)
    c = make_paged_case(B, hq, hk, d, 128, [sk] * B, seqlen_q=sq, dtype=dtype, seed=sq + sk + d, dist="uniform5")
    dev = to_dev(c)
    q_tnd = dev["q"].reshape(B * sq, hq, d)
    out, lse, *_ = flash_attn_with_kvcache(q_tnd, dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                           page_table=dev["block_table"], cu_seqlens_q=cu([sq] * B).cuda(),
                                           max_seqlen_q=sq, causal=causal, softcap=softcap, num_splits=num_splits,
                                           return_softmax_lse=True)
    torch.cuda.synchronize()
    assert out.shape == (B * sq, hq, d) and lse.shape == (hq, B * sq)
    gold, gold_lse = O.flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], cache_seqlens=c["cache_seqlens"],
                                               block_table=c["block_table"], causal=causal, softcap=softcap, mode="golden")
    check_vs_golden(out, gold.reshape(B * sq, hq, d), lse, gold_lse.permute(1, 0, 2).reshape(hq, B * sq), str(case))


@pytest.mark.parametrize("num_splits", [0, 1, 4])
def test_v3_kvcache_tnd_mixed_batch_long_contexts(num_splits):
    # decode rows and a prompt chunk in one token-major batch over long paged contexts: the keys of every
    # sequence are cut into ranges (num_splits 0 / 4) or not (1); same result either way
    from flash_attn_npu_3 import flash_attn_with_kvcache
    q_lens, k_lens = [1, 1, 200, 1], [6000, 129, 4500, 3000]
    B, hq, hk, d = 4, 16, 2, 128
    c = make_paged_case(B, hq, hk, d, 256, k_lens, seqlen_q=1, seed=93)
    g = torch.Generator().manual_seed(94)
    q = torch.randn(sum(q_lens), hq, d, generator=g).to(BF)
    k_packed, v_packed = packed_from_pages(c, k_lens)
    cu_q, cu_k = cu(q_lens), cu(k_lens)
    print("v3 mixed batch", num_splits, flush=True)
    out, lse, *_ = flash_attn_with_kvcache(q.cuda(), c["k_cache"].cuda(), c["v_cache"].cuda(), page_table=c["block_table"].cuda(),
                                           cache_seqlens=c["cache_seqlens"].cuda(), cu_seqlens_q=cu_q.cuda(), max_seqlen_q=max(q_lens),
                                           causal=True, num_splits=num_splits, return_softmax_lse=True)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_varlen(q, k_packed, v_packed, cu_q, cu_k, max(q_lens), max(k_lens), causal=True, mode="fp32")
    check_out(out, ref, lse, ref_lse, "v3 mixed batch")


@pytest.mark.parametrize("layout", ["paged", "packed", "dense"])
@pytest.mark.parametrize("causal,window", [(False, (-1, -1)), (True, (-1, -1)), (False, (300, 40))])
def test_v3_kvcache_tnd_ragged(layout, causal, window):
    # query blocks and caches of different lengths (the reference's is_varied cases,
    # tests/test_flash_attn_npu_v3.py:323-329): per-sequence oracle on the gathered keys
    from flash_attn_npu_3 import flash_attn_with_kvcache
    q_lens, k_lens = [5, 130, 1, 64], [700, 400, 33, 64]
    B, hq, hk, d = 4, 8, 2, 128
    c = make_paged_case(B, hq, hk, d, 128, k_lens, seqlen_q=1, seed=91)
    g = torch.Generator().manual_seed(92)
    q = torch.randn(sum(q_lens), hq, d, generator=g).to(BF)
    k_packed, v_packed = packed_from_pages(c, k_lens)
    cu_q, cu_k = cu(q_lens), cu(k_lens)
    print("v3 ragged", layout, causal, window, flush=True)
    kw = dict(cache_seqlens=c["cache_seqlens"].cuda(), cu_seqlens_q=cu_q.cuda(), max_seqlen_q=max(q_lens), causal=causal,
              window_size=window, return_softmax_lse=True)
    if layout == "paged":
        out, lse, *_ = flash_attn_with_kvcache(q.cuda(), c["k_cache"].cuda(), c["v_cache"].cuda(),
                                               page_table=c["block_table"].cuda(), **kw)
    elif layout == "packed":
        out, lse, *_ = flash_attn_with_kvcache(q.cuda(), k_packed.cuda(), v_packed.cuda(), **kw)
    else:
        cap = 704
        kd = torch.zeros(B, cap, hk, d, dtype=BF)
        vd = torch.zeros(B, cap, hk, d, dtype=BF)
        for b in range(B):
            kd[b, :k_lens[b]] = k_packed[cu_k[b]:cu_k[b + 1]]
            vd[b, :k_lens[b]] = v_packed[cu_k[b]:cu_k[b + 1]]
        out, lse, *_ = flash_attn_with_kvcache(q.cuda(), kd.cuda(), vd.cuda(), **kw)
    torch.cuda.synchronize()
    ref, ref_lse = O.flash_attn_varlen(q, k_packed, v_packed, cu_q, cu_k, max(q_lens), max(k_lens), causal=causal,
                                       window_size=window, mode="fp32")
    check_out(out, ref, lse, ref_lse, f"ragged {layout}")


def test_v3_append_rotary_bit_exact():
    # k / v appended through page_table with rotary, batch-major and token-major q: cache bytes
    # bit-exact against the oracle's append, outputs at the bar
    from flash_attn_npu_3 import flash_attn_with_kvcache
    B, hq, hk, d, sq = 3, 16, 4, 128, 2
    for tnd in (False, True):
        c = make_paged_case(B, hq, hk, d, 64, [100, 63, 640], seqlen_q=sq, seqlen_new=sq, seed=93)
        cos, sin = rotary_tables(1024, 64)
        dev = to_dev(c)
        q = dev["q"].reshape(B * sq, hq, d) if tnd else dev["q"]
        extra = dict(cu_seqlens_q=cu([sq] * B).cuda(), max_seqlen_q=sq) if tnd else {}
        print("v3 append", tnd, flush=True)
        out, lse, *_ = flash_attn_with_kvcache(q, dev["k_cache"], dev["v_cache"], dev["k"], dev["v"], rotary_cos=cos.cuda(),
                                               rotary_sin=sin.cuda(), cache_seqlens=dev["cache_seqlens"],
                                               page_table=dev["block_table"], causal=True, rotary_interleaved=False,
                                               return_softmax_lse=True, **extra)
        torch.cuda.synchronize()
        kc, vc = c["k_cache"].clone(), c["v_cache"].clone()
        ref, ref_lse = O.flash_attn_with_kvcache(c["q"], kc, vc, c["k"], c["v"], rotary_cos=cos, rotary_sin=sin,
                                                 cache_seqlens=c["cache_seqlens"], block_table=c["block_table"],
                                                 causal=True, rotary_interleaved=False, mode="fp32")
        assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16))
        assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16))
        if tnd:
            out, lse = out.view(B, sq, hq, d), lse.view(hq, B, sq).permute(1, 0, 2)
        check_out(out, ref, lse, ref_lse, f"v3 append tnd={tnd}")


@pytest.mark.parametrize("causal", [False, True])
def test_v3_kvcache_graph(causal):
    # the reference's graph test, shape for shape: metadata, one eager call, capture, replay
    from flash_attn_npu_3 import flash_attn_with_kvcache, get_scheduler_metadata
    B, hq, hk, sq, sk, d, page = 1, 4, 2, 16, 128, 128, 128
    g = torch.Generator().manual_seed(7)
    q = (2 * torch.rand(sq, hq, d, generator=g) - 1).to(BF)
    kc = (2 * torch.rand(B, page, hk, d, generator=g) - 1).to(BF)
    vc = (2 * torch.rand(B, page, hk, d, generator=g) - 1).to(BF)
    lens = torch.tensor([sk], dtype=torch.int32)
    table = torch.tensor([[0]], dtype=torch.int32)
    cu_q = torch.tensor([0, sq], dtype=torch.int32)
    dq, dk, dv, dl, dt, dcu = (x.cuda() for x in (q, kc, vc, lens, table, cu_q))
    meta = get_scheduler_metadata(batch_size=B, max_seqlen_q=sq, max_seqlen_k=sk, num_heads_q=hq, num_heads_kv=hk,
                                  headdim=d, cache_seqlens=dl, qkv_dtype=BF, cu_seqlens_q=dcu, page_size=page,
                                  causal=causal, window_size=(-1, -1))
    assert meta.dtype == torch.uint8 and meta.is_cuda and meta.is_contiguous()

    def run():
        return flash_attn_with_kvcache(dq, dk, dv, cache_seqlens=dl, page_table=dt, cu_seqlens_q=dcu, max_seqlen_q=sq,
                                       softmax_scale=d ** -0.5, causal=causal, window_size=(-1, -1),
                                       scheduler_metadata=meta, return_softmax_lse=True)
    print("v3 graph", causal, flush=True)
    run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out, lse, *_ = run()
    ref, ref_lse = O.flash_attn_with_kvcache(q.view(B, sq, hq, d), kc, vc, cache_seqlens=lens, block_table=table,
                                             causal=causal, mode="golden")
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        torch.testing.assert_close(out.cpu().float(), ref.view(sq, hq, d).float(), rtol=1e-2, atol=1e-2)


def test_v3_metadata_every_entry_point():
    from flash_attn_npu_3 import flash_attn_func, flash_attn_varlen_func, flash_attn_with_kvcache, get_scheduler_metadata
    # dense batch (tests/test_flash_attn_npu_v3_metadata.py:210-257)
    B, hq, hk, s, d = 2, 4, 4, 256, 128
    g = torch.Generator().manual_seed(11)
    q, k, v = ((10 * torch.rand(B, s, h, d, generator=g) - 5).to(BF) for h in (hq, hk, hk))
    lens = torch.full((B,), s, dtype=torch.int32).cuda()
    print("v3 metadata dense", flush=True)
    meta = get_scheduler_metadata(B, s, s, hq, hk, d, lens, qkv_dtype=BF, causal=True)
    out, lse = flash_attn_func(q.cuda(), k.cuda(), v.cuda(), softmax_scale=d ** -0.5, causal=True, num_splits=1,
                               return_attn_probs=True, scheduler_metadata=meta)
    torch.cuda.synchronize()
    gold, gold_lse = O.flash_attn_varlen(q.view(B * s, hq, d), k.view(B * s, hk, d), v.view(B * s, hk, d), cu([s] * B),
                                         cu([s] * B), s, s, causal=True, mode="golden")
    check_vs_golden(out.reshape(B * s, hq, d), gold, lse.permute(1, 0, 2).reshape(hq, B * s), gold_lse, "flash_attn_func")
    # packed sequences (:260-330)
    print("v3 metadata varlen", flush=True)
    cu_q = cu([s] * B).cuda()
    meta = get_scheduler_metadata(B, s, s, hq, hk, d, lens, qkv_dtype=BF, cu_seqlens_q=cu_q, causal=True)
    out = flash_attn_varlen_func(q.view(B * s, hq, d).cuda(), k.view(B * s, hk, d).cuda(), v.view(B * s, hk, d).cuda(), cu_q,
                                 cu_q, s, s, softmax_scale=d ** -0.5, causal=True, num_splits=1, scheduler_metadata=meta)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu().float(), gold.float(), rtol=1e-2, atol=1e-2)
    # a record made for other shapes is refused; so is one of the wrong dtype
    with pytest.raises(RuntimeError, match="computed for a different call"):
        flash_attn_func(q.cuda(), k.cuda(), v.cuda(), causal=False, scheduler_metadata=meta)
    with pytest.raises(RuntimeError, match="scheduler_metadata must be a byte tensor"):
        flash_attn_func(q.cuda(), k.cuda(), v.cuda(), causal=True, scheduler_metadata=meta.view(torch.int32))
    with pytest.raises(RuntimeError, match="scheduler_metadata buffer is too small"):
        flash_attn_func(q.cuda(), k.cuda(), v.cuda(), causal=True, scheduler_metadata=meta[:8].clone())


def test_v3_rejections():
    from flash_attn_npu_3 import flash_attn_with_kvcache
    c = to_dev(make_paged_case(2, 8, 2, 128, 128, [100, 200], seed=12))
    base = dict(cache_seqlens=c["cache_seqlens"], page_table=c["block_table"])
    one = torch.ones(1, device="cuda")
    for kw, msg in [(dict(cache_leftpad=c["cache_seqlens"]), "does not support leftpad_k"),
                    (dict(q_descale=one), "does not support q_descale"),
                    (dict(k_descale=one), "does not support k_descale"),
                    (dict(v_descale=one), "does not support v_descale"),
                    (dict(rotary_seqlens=c["cache_seqlens"]), "does not support seqlens_rotary"),
                    (dict(attention_chunk=4), "does not support attention_chunk"),
                    (dict(pack_gqa=True), "does not support pack_gqa"),
                    (dict(softcap=-1.0), "softcap must be non-negative"),
                    (dict(num_splits=100000), "supports num_splits in"),
                    (dict(cu_seqlens_q=torch.tensor([0, 1, 2], dtype=torch.int32, device="cuda")), "max_seqlen_q must be provided")]:
        with pytest.raises(RuntimeError, match=msg):
            flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], **{**base, **kw})
    with pytest.raises(RuntimeError, match="page_table must have dtype int32"):
        flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], cache_seqlens=c["cache_seqlens"],
                                page_table=c["block_table"].long())
    # pack_gqa=False is accepted, as in the reference (flash_api.cpp:161)
    flash_attn_with_kvcache(c["q"], c["k_cache"], c["v_cache"], pack_gqa=False, **base)
    torch.cuda.synchronize()
