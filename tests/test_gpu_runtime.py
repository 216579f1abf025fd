"""Runtime behaviour of the library boundary: calls on a side stream, calls from two host threads at
once (the C ABI keeps no mutable global state and its error text is thread-local), and caches larger
than 2^31 elements, whose block offsets need 64-bit arithmetic in every kernel."""
import threading

import pytest
import torch

import fa_oracle as O
from helpers import check_out, make_paged_case, to_dev

pytestmark = pytest.mark.gpu


def decode_once(dev, **kw):
    from flash_attn_npu import flash_attn_with_kvcache
    return flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], cache_seqlens=dev["cache_seqlens"],
                                   block_table=dev["block_table"], causal=True, return_softmax_lse=True, **kw)


def test_side_stream():
    dev = to_dev(make_paged_case(4, 32, 8, 128, 256, [3000, 17, 900, 5000], seed=81))
    out0, lse0 = decode_once(dev)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        out1, lse1 = decode_once(dev)
    side.synchronize()
    assert torch.equal(out1, out0) and torch.equal(lse1, lse0)


def test_two_host_threads():
    cases = [to_dev(make_paged_case(3, 16, 4, 128, 128, [2000 + 100 * t, 64, 999], seed=82 + t)) for t in range(2)]
    want = [decode_once(c) for c in cases]
    torch.cuda.synchronize()
    errors, results = [], [None, None]

    def worker(t):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(40):
                    results[t] = decode_once(cases[t])
                # an argument error in one thread must not disturb the other's calls or messages
                with pytest.raises(RuntimeError, match="block_table must have dtype int32"):
                    from flash_attn_npu import flash_attn_with_kvcache
                    flash_attn_with_kvcache(cases[t]["q"], cases[t]["k_cache"], cases[t]["v_cache"],
                                            cache_seqlens=cases[t]["cache_seqlens"], block_table=cases[t]["block_table"].long())
            stream.synchronize()
        except BaseException as exc:   # reported by the main thread
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors
    for t in range(2):
        assert torch.equal(results[t][0], want[t][0]) and torch.equal(results[t][1], want[t][1])


def high_pages_case(sq, lens, hq, hk, d, page, pool, dtype=torch.bfloat16, seed=0):
    """A pool of `pool` pages of which only the last few are used (and filled)."""
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    pages = [-(-l // page) for l in lens]
    used = sum(pages)
    ids = torch.arange(pool - used, pool)[torch.randperm(used, generator=g)]
    bt = torch.zeros(B, max(pages), dtype=torch.int32)
    o = 0
    for b in range(B):
        bt[b, :pages[b]] = ids[o:o + pages[b]].to(torch.int32)
        o += pages[b]
    return bt, ids


@pytest.mark.parametrize("sq,num_splits", [(1, 0), (1, 2), (8, 0), (24, 0)])
def test_cache_beyond_2_31_elements(sq, num_splits):
    # 9000 pages x 256 rows x 8 heads x 128 = 2.36e9 elements per cache: element offsets of the pages
    # in use do not fit 32 bits.  sq = 1: wave-level decode kernel, or the grid-split one with
    # num_splits = 2; sq = 8: 32 query rows per kv head, workgroup-level decode kernel; sq = 24: tiled kernel
    from flash_attn_npu import flash_attn_with_kvcache
    hq, hk, d, page, pool = 32, 8, 128, 256, 9000
    lens = [1500, 300]
    bt, ids = high_pages_case(sq, lens, hq, hk, d, page, pool, seed=83)
    kc = torch.empty(pool, page, hk, d, dtype=torch.bfloat16, device="cuda")
    vc = torch.empty(pool, page, hk, d, dtype=torch.bfloat16, device="cuda")
    assert kc.numel() > 2 ** 31 and int(ids.min()) * page * hk * d > 2 ** 31
    g = torch.Generator().manual_seed(84)
    k_used = torch.randn(len(ids), page, hk, d, generator=g).to(torch.bfloat16)
    v_used = torch.randn(len(ids), page, hk, d, generator=g).to(torch.bfloat16)
    kc[ids.cuda()], vc[ids.cuda()] = k_used.cuda(), v_used.cuda()
    q = torch.randn(2, sq, hq, d, generator=g).to(torch.bfloat16)
    k_new = torch.randn(2, sq, hk, d, generator=g).to(torch.bfloat16)
    v_new = torch.randn(2, sq, hk, d, generator=g).to(torch.bfloat16)
    cl = torch.tensor([l - sq for l in lens], dtype=torch.int32)
    print("big cache", sq, flush=True)
    out, lse = flash_attn_with_kvcache(q.cuda(), kc, vc, k_new.cuda(), v_new.cuda(), cache_seqlens=cl.cuda(),
                                       block_table=bt.cuda(), causal=True, num_splits=num_splits, return_softmax_lse=True)
    torch.cuda.synchronize()
    # oracle on the used pages only, renumbered
    renum = {int(p): i for i, p in enumerate(ids)}
    bt_small = torch.tensor([[renum.get(int(x), 0) for x in row] for row in bt], dtype=torch.int32)
    ks, vs = k_used.clone(), v_used.clone()
    ref, ref_lse = O.flash_attn_with_kvcache(q, ks, vs, k_new, v_new, cache_seqlens=cl, block_table=bt_small, causal=True,
                                             mode="fp32")
    check_out(out, ref, lse, ref_lse, "big cache")
    assert torch.equal(kc[ids.cuda()].cpu().view(torch.int16), ks.view(torch.int16)), "appended rows in high pages"
    del kc, vc
    torch.cuda.empty_cache()


def test_latent_cache_beyond_2_31_bytes():
    from flash_attn_npu import flash_attn_with_kvcache
    page, pool = 256, 15000                     # 15000 x 256 x 576 = 2.2e9 bytes
    lens = [1000, 260]
    bt, ids = high_pages_case(1, lens, 128, 1, 576, page, pool, seed=85)
    g = torch.Generator().manual_seed(86)
    latent = torch.randn(len(ids), page, 1, 576, generator=g).to(torch.bfloat16)
    code, scale = O.quantize_per_token(latent)
    kc = torch.empty(pool, page, 1, 576, dtype=torch.int8, device="cuda")
    sc = torch.empty(pool, page, 1, dtype=torch.float32, device="cuda")
    assert int(ids.min()) * page * 576 > 2 ** 31
    kc[ids.cuda()], sc[ids.cuda()] = code.cuda(), scale.cuda()
    q = torch.randn(2, 1, 128, 576, generator=g).to(torch.bfloat16)
    cl = torch.tensor(lens, dtype=torch.int32)
    out, lse = flash_attn_with_kvcache(q.cuda(), kc, kc[..., :512], cache_seqlens=cl.cuda(), block_table=bt.cuda(),
                                       softmax_scale=192 ** -0.5, causal=True, return_softmax_lse=True, k_scale_cache=sc)
    torch.cuda.synchronize()
    renum = {int(p): i for i, p in enumerate(ids)}
    bt_small = torch.tensor([[renum.get(int(x), 0) for x in row] for row in bt], dtype=torch.int32)
    ref, ref_lse = O.flash_attn_with_kvcache(q, code, code[..., :512], cache_seqlens=cl, block_table=bt_small,
                                             softmax_scale=192 ** -0.5, causal=True, k_scale_cache=scale, mode="fp32")
    check_out(out, ref, lse, ref_lse, "big latent cache")
    del kc, sc
    torch.cuda.empty_cache()


def test_validate_mode_checks_what_only_the_device_knows():
    """FA_ROCM_VALIDATE=1: page ids, capacities and rotary positions are checked by a kernel before anything is queued;
    a violation is an error naming the row and the cache is left as it was.  A valid call gives the usual result."""
    from flash_attn_npu import flash_attn_varlen_func, flash_attn_with_kvcache
    from helpers import library_env, rotary_tables
    lens = [100, 1, 0, 777, 64]
    case = make_paged_case(len(lens), 32, 8, 128, 64, lens, seqlen_q=1, seqlen_new=1, seed=9)
    dev = to_dev(case)

    def call(d, **kw):
        r = flash_attn_with_kvcache(d["q"], d["k_cache"], d["v_cache"], d["k"], d["v"], cache_seqlens=d["cache_seqlens"],
                                    block_table=d["block_table"], causal=True, return_softmax_lse=True, **kw)
        torch.cuda.synchronize()
        return r

    with library_env(FA_ROCM_VALIDATE=1):
        print("validate mode: valid call", flush=True)
        fresh = to_dev(case)
        out, lse = call(fresh)
        ref, ref_lse = O.flash_attn_with_kvcache(case["q"], case["k_cache"].clone(), case["v_cache"].clone(), case["k"], case["v"],
                                                 cache_seqlens=case["cache_seqlens"], block_table=case["block_table"], causal=True, mode="fp32")
        check_out(out, ref, lse, ref_lse, "validate mode")

        before_k = dev["k_cache"].clone()
        bad = dict(dev)
        bad["block_table"] = dev["block_table"].clone()
        bad["block_table"][3, 2] = dev["k_cache"].shape[0]           # one past the pool
        print("validate mode: page id beyond the pool", flush=True)
        with pytest.raises(RuntimeError, match=r"block_table row 3 names page \d+; the cache has num_blocks"):
            call(bad)
        bad["block_table"][3, 2] = -1
        with pytest.raises(RuntimeError, match="block_table row 3 names page -1"):
            call(bad)
        # an id behind the used pages of a row is never read: not an error
        ok = dict(dev)
        ok["block_table"] = dev["block_table"].clone()
        ok["k_cache"], ok["v_cache"] = dev["k_cache"].clone(), dev["v_cache"].clone()
        ok["block_table"][1, 1:] = 1 << 30
        call(ok)

        bad = dict(dev)
        bad["cache_seqlens"] = dev["cache_seqlens"].clone()
        cap = dev["block_table"].shape[1] * 64
        bad["cache_seqlens"][4] = cap                                # the appended token would fall behind the last page
        print("validate mode: append beyond the pages", flush=True)
        with pytest.raises(RuntimeError, match=rf"batch row 4 holds {cap + 1} keys .* addresses only {cap}"):
            call(bad)
        bad["cache_seqlens"][4] = -5
        with pytest.raises(RuntimeError, match=r"cache_seqlens\[4\] = -5 is negative"):
            call(bad)

        cos, sin = rotary_tables(778, 128, dtype=torch.bfloat16)           # positions 0..777: row 3 appends at 777, the last one
        cos, sin = cos.cuda(), sin.cuda()
        ok = dict(dev)
        ok["k_cache"], ok["v_cache"] = dev["k_cache"].clone(), dev["v_cache"].clone()
        call(ok, rotary_cos=cos, rotary_sin=sin)
        print("validate mode: position beyond the rotary tables", flush=True)
        with pytest.raises(RuntimeError, match="batch row 3 needs 778 rotary positions but rotary_cos / rotary_sin have seqlen_ro = 777"):
            call(dev, rotary_cos=cos[:777], rotary_sin=sin[:777])
        assert torch.equal(dev["k_cache"], before_k), "a rejected call wrote to the cache"

        # paged varlen: seqused_k and the table
        total = sum(lens)
        cu_q = torch.tensor([0, 3, 4, 4, 10, 12], dtype=torch.int32, device="cuda")
        q = torch.randn(12, 32, 128, dtype=torch.bfloat16, device="cuda")
        used = torch.tensor(lens, dtype=torch.int32, device="cuda")
        from flash_attn_npu.flash_attn_npu_interface import _varlen_forward_eager
        _varlen_forward_eager(q, dev["k_cache"], dev["v_cache"], cu_q, None, 6, 777, 0.0, 0.1, True, block_table=dev["block_table"], seqused_k=used)
        bt = dev["block_table"].clone()
        bt[0, 1] = dev["k_cache"].shape[0] + 7
        print("validate mode: paged varlen", flush=True)
        with pytest.raises(RuntimeError, match="block_table row 0 names page"):
            _varlen_forward_eager(q, dev["k_cache"], dev["v_cache"], cu_q, None, 6, 777, 0.0, 0.1, True, block_table=bt, seqused_k=used)
        used[2] = cap + 1
        with pytest.raises(RuntimeError, match="batch row 2 holds"):
            _varlen_forward_eager(q, dev["k_cache"], dev["v_cache"], cu_q, None, 6, 777, 0.0, 0.1, True, block_table=dev["block_table"],
                                  seqused_k=used)
        torch.cuda.synchronize()
    del total
