"""Pins for paged gather, in-place append, rotary and the int8 format: brute-force loops, bit-exact."""
import math

import torch

import fa_oracle as O
from helpers import make_paged_case, rotary_tables


def test_gather_matches_per_token_loop():
    c = make_paged_case(3, 4, 2, 16, 32, [70, 1, 96], dtype=torch.float32, seed=1)
    for b in range(3):
        n = int(c["cache_seqlens"][b])
        got = O.gather_paged(c["k_cache"], c["block_table"][b], n)
        for j in range(n):     # tests/test_flash_attn_npu_v2.py:401-409
            blk = int(c["block_table"][b][j // 32])
            assert torch.equal(got[j], c["k_cache"][blk, j % 32])


def test_append_brute_force_and_untouched_bytes():
    c = make_paged_case(3, 4, 2, 16, 32, [31, 32, 0], seqlen_new=3, dtype=torch.bfloat16, seed=2)
    kc, vc = c["k_cache"].clone(), c["v_cache"].clone()
    O.append_kv(kc, vc, c["k"], c["v"], c["cache_seqlens"], c["block_table"])
    touched = torch.zeros(kc.shape[:2], dtype=torch.bool)
    for b in range(3):
        for t in range(3):
            p = int(c["cache_seqlens"][b]) + t
            blk = int(c["block_table"][b][p // 32])
            assert torch.equal(kc[blk, p % 32], c["k"][b, t]) and torch.equal(vc[blk, p % 32], c["v"][b, t])
            touched[blk, p % 32] = True
    assert torch.equal(kc[~touched], c["k_cache"][~touched]) and torch.equal(vc[~touched], c["v_cache"][~touched])


def test_attention_after_append_equals_fresh_cache():
    c = make_paged_case(2, 4, 2, 16, 32, [40, 63], seqlen_new=2, seqlen_q=2, dtype=torch.float32, seed=3)
    kc, vc = c["k_cache"].clone(), c["v_cache"].clone()
    out, lse = O.flash_attn_with_kvcache(c["q"], kc, vc, c["k"], c["v"], cache_seqlens=c["cache_seqlens"],
                                         block_table=c["block_table"], causal=True)
    for b in range(2):
        n = int(c["cache_seqlens"][b])
        kl = torch.cat([O.gather_paged(c["k_cache"], c["block_table"][b], n), c["k"][b]])
        vl = torch.cat([O.gather_paged(c["v_cache"], c["block_table"][b], n), c["v"][b]])
        ref, ref_lse = O.attention_fp32(c["q"][b], kl, vl, 0.25, O.masked_matrix(2, n + 2, True, False, -1, 0))
        assert (out[b] - ref).abs().max() < 1e-5 and (lse[b] - ref_lse).abs().max() < 1e-5


def test_config1_cpu_plumbing():
    # BASELINE config 1: B=2, 8q/2kv heads, d=128, fp32, page 256, 8 pages, lens [300, 511], append 1, causal
    g = torch.Generator().manual_seed(0)
    q, kc, vc = torch.randn(2, 1, 8, 128, generator=g), torch.randn(8, 256, 2, 128, generator=g), torch.randn(8, 256, 2, 128, generator=g)
    bt = torch.randperm(8, generator=g).view(2, 4).to(torch.int32)
    lens = torch.tensor([300, 511], dtype=torch.int32)
    k, v = torch.randn(2, 1, 2, 128, generator=g), torch.randn(2, 1, 2, 128, generator=g)
    kc2, vc2 = kc.clone(), vc.clone()
    out, lse = O.flash_attn_with_kvcache(q, kc2, vc2, k, v, cache_seqlens=lens, block_table=bt, causal=True,
                                         softmax_scale=1 / math.sqrt(128))
    for b in range(2):
        p = int(lens[b])
        assert torch.equal(kc2[bt[b, p // 256], p % 256], k[b, 0]) and torch.equal(vc2[bt[b, p // 256], p % 256], v[b, 0])
    assert int((kc2 != kc).any(dim=-1).any(dim=-1).sum()) == 2          # exactly two rows written
    for b in range(2):
        n = int(lens[b]) + 1
        kl = torch.stack([kc2[bt[b, j // 256], j % 256] for j in range(n)]).double()
        vl = torch.stack([vc2[bt[b, j // 256], j % 256] for j in range(n)]).double()
        for h in range(8):
            s = (kl[:, h // 4] @ q[b, 0, h].double()) / math.sqrt(128)
            assert abs(float(torch.logsumexp(s, 0)) - float(lse[b, h, 0])) < 1e-5
            assert (torch.softmax(s, 0) @ vl[:, h // 4] - out[b, 0, h].double()).abs().max() < 1e-5


def test_rotary_closed_form_and_special_cases():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(6, 3, 64, generator=g)
    cos, sin = rotary_tables(50, 32, dtype=torch.float32)
    pos = torch.tensor([0, 1, 7, 20, 49, 3])
    for inter in (False, True):
        y = O.apply_rotary(x, cos, sin, pos, inter)
        assert torch.equal(y[..., 32:], x[..., 32:])                       # dims >= rotary_dim pass through
        assert torch.equal(y[0], x[0])                                      # position 0: angle 0
        x1, x2 = (x[..., 0:32:2], x[..., 1:32:2]) if inter else (x[..., :16], x[..., 16:32])
        y1, y2 = (y[..., 0:32:2], y[..., 1:32:2]) if inter else (y[..., :16], y[..., 16:32])
        z = torch.complex(x1.double(), x2.double()) * torch.complex(cos[pos].double(), sin[pos].double())[:, None, :]
        assert (y1.double() - z.real).abs().max() < 1e-6 and (y2.double() - z.imag).abs().max() < 1e-6
        assert ((y1 ** 2 + y2 ** 2) - (x1 ** 2 + x2 ** 2)).abs().max() < 1e-4   # rotation keeps the pair norm
    ident = O.apply_rotary(x, torch.ones(50, 16), torch.zeros(50, 16), pos, False)
    assert torch.equal(ident, x)
    # interleaved == non-interleaved on permuted dims
    perm = torch.cat([torch.arange(0, 32, 2), torch.arange(1, 32, 2)])
    a = O.apply_rotary(x[..., :32][..., perm], cos, sin, pos, False)
    b = O.apply_rotary(x[..., :32], cos, sin, pos, True)[..., perm]
    assert torch.equal(a, b)


def test_rotary_rounds_to_fp32_then_to_the_io_dtype():
    # known answer on an exact tie: x1 - x2 * sin = -1.559082081... lies just past the middle of the fp16 neighbours
    # -1.5595703125 and -1.55859375; the product and the difference each rounded to fp32 give the middle exactly
    # (-1.55908203125), which rounds to the even neighbour.  One rounding of the unrounded value gives the other one.
    x = torch.tensor([[[-1.560546875, -0.994140625]]], dtype=torch.float16)
    cos = torch.tensor([[1.0]], dtype=torch.float16)
    sin = torch.tensor([[0.0014734268188476562]], dtype=torch.float16)
    assert float(sin[0, 0]) == 0.0014734268188476562 and float(x[0, 0, 1]) == -0.994140625      # inputs are exact in fp16
    for inter in (False, True):
        y = O.apply_rotary(x, cos, sin, torch.tensor([0]), inter)
        assert float(y[0, 0, 0]) == -1.55859375


def test_rotary_q_positions_follow_docstring():
    # q at cache_seqlens + i when causal/local, all at cache_seqlens otherwise (interface docstring :1469-1474)
    c = make_paged_case(1, 2, 1, 32, 32, [10], seqlen_q=3, seqlen_new=3, dtype=torch.float32, seed=5)
    cos, sin = rotary_tables(64, 32, dtype=torch.float32)
    for causal in (True, False):
        out, _ = O.flash_attn_with_kvcache(c["q"], c["k_cache"].clone(), c["v_cache"].clone(), c["k"], c["v"], rotary_cos=cos,
                                           rotary_sin=sin, cache_seqlens=c["cache_seqlens"], block_table=c["block_table"],
                                           causal=causal, rotary_interleaved=False)
        pos_q = torch.tensor([10, 11, 12]) if causal else torch.tensor([10, 10, 10])
        qr = O.apply_rotary(c["q"][0], cos, sin, pos_q, False)
        kr = O.apply_rotary(c["k"][0], cos, sin, torch.tensor([10, 11, 12]), False)
        kl = torch.cat([O.gather_paged(c["k_cache"], c["block_table"][0], 10), kr])
        vl = torch.cat([O.gather_paged(c["v_cache"], c["block_table"][0], 10), c["v"][0]])
        mask = O.masked_matrix(3, 13, True, False, -1, 0) if causal else None
        ref, _ = O.attention_fp32(qr, kl, vl, 32 ** -0.5, mask)
        assert (out[0] - ref).abs().max() < 1e-5


def test_int8_codes_brute_force():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(5, 24, generator=g).bfloat16()
    x[2] = 0
    code, scale = O.quantize_per_token(x)
    for t in range(5):
        row = [float(v) for v in x[t]]
        amax = max(abs(v) for v in row)
        sc = torch.tensor(amax, dtype=torch.float32) / 127.0
        assert float(scale[t]) == float(sc)
        for c, v in enumerate(row):
            if amax == 0:
                assert int(code[t, c]) == 0
                continue
            r = float(torch.tensor(v, dtype=torch.float32) / sc)
            fl = math.floor(r)
            q = fl + 1 if r - fl > 0.5 else fl if r - fl < 0.5 else (fl if fl % 2 == 0 else fl + 1)   # half to even
            assert int(code[t, c]) == max(-127, min(127, q))
    deq = O.dequantize_per_token(code, scale)
    assert ((deq - x.float()).abs() <= scale[:, None] * 0.5 + 1e-7).all()
    assert int(code.abs().max()) == 127


def test_combine_splits_identity():
    g = torch.Generator().manual_seed(8)
    q, k, v = torch.randn(1, 4, 16, generator=g), torch.randn(90, 2, 16, generator=g), torch.randn(90, 2, 16, generator=g)
    full, full_lse = O.attention_fp32(q, k, v, 0.25, None)
    for cuts in ([0, 90], [0, 30, 90], [0, 1, 2, 50, 90], [0, 45, 45, 90]):
        parts, lses = [], []
        for a, e in zip(cuts[:-1], cuts[1:]):
            o, l = O.attention_fp32(q, k[a:e], v[a:e], 0.25, None)
            parts.append(o)
            lses.append(l.T)     # (Sq, Hq)
        out, lse = O.combine_splits(torch.stack(parts), torch.stack(lses))
        assert (out - full).abs().max() < 1e-5 and (lse.T - full_lse).abs().max() < 1e-5
    out, lse = O.combine_splits(torch.zeros(3, 1, 4, 16), torch.full((3, 1, 4), float("inf")))
    assert (out == 0).all() and torch.isinf(lse).all() and (lse > 0).all()


def test_quantising_append_brute_force():
    """int8 latent cache: appended rows hold the scalar-loop codes and scale of their token at
    p = cache_seqlens[b] + t, nothing else changes, and attention over the appended cache equals
    attention over a cache that was quantised with the rows already in place."""
    g = torch.Generator().manual_seed(7)
    B, page, d, snew = 2, 32, 576, 2
    lens = [30, 5]
    latent = torch.randn(4, page, 1, d, generator=g).to(torch.bfloat16)
    bt = torch.tensor([[2, 0], [3, 1]], dtype=torch.int32)
    k_new = torch.randn(B, snew, 1, d, generator=g).to(torch.bfloat16)
    k_new[1, 1] = 0
    code, scale = O.quantize_per_token(latent)
    kc, ks = code.clone(), scale.clone()
    O.append_kv(kc, kc[..., :512], k_new, k_new[..., :512], torch.tensor(lens, dtype=torch.int32), bt, k_scale_cache=ks)
    touched = torch.zeros(4, page, dtype=torch.bool)
    for b in range(B):
        for t in range(snew):
            p = lens[b] + t
            blk, row = int(bt[b][p // page]), p % page
            x = k_new[b, t, 0].to(torch.float32)
            absmax = float(x.abs().max())
            sc = torch.tensor(absmax, dtype=torch.float32) / 127.0
            assert ks[blk, row, 0].item() == sc.item()
            for e in range(0, d, 37):       # sampled scalar loop
                want = 0 if sc == 0 else max(-127, min(127, int(torch.round(x[e] / sc))))
                assert int(kc[blk, row, 0, e]) == want
            touched[blk, row] = True
    assert torch.equal(kc[~touched], code[~touched]) and torch.equal(ks[~touched], scale[~touched])
    # same attention as a cache built with the new rows in place before quantisation
    full = latent.clone()
    for b in range(B):
        for t in range(snew):
            p = lens[b] + t
            full[int(bt[b][p // page]), p % page] = k_new[b, t]
    code2, scale2 = O.quantize_per_token(full)
    q = torch.randn(B, 1, 8, d, generator=g).to(torch.bfloat16)
    kc3, ks3 = code.clone(), scale.clone()
    a, la = O.flash_attn_with_kvcache(q, kc3, kc3[..., :512], k_new, k_new[..., :512], cache_seqlens=torch.tensor(lens, dtype=torch.int32),
                                      block_table=bt, causal=True, k_scale_cache=ks3, mode="fp32")
    b2, lb = O.flash_attn_with_kvcache(q, code2, code2[..., :512], cache_seqlens=torch.tensor([l + snew for l in lens], dtype=torch.int32),
                                       block_table=bt, causal=True, k_scale_cache=scale2, mode="fp32")
    assert torch.equal(a, b2) and torch.equal(la, lb)
