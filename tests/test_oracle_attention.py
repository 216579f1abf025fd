"""Pins for the oracle's attention cores: library softmax / logsumexp in fp64, brute-force loops on
tiny inputs, the out/LSE identity of tests/fa_small_op_golden.py:104-135, fully hidden rows."""
import math

import pytest
import torch

import fa_oracle as O


def textbook(q, k, v, scale, keep, softcap=0.0):
    """fp64 attention with torch.softmax / torch.logsumexp.  q (Sq,Hq,d), k/v (Sk,Hk,*)."""
    hq, hk = q.shape[1], k.shape[1]
    g = hq // hk
    out = torch.zeros(q.shape[0], hq, v.shape[-1], dtype=torch.float64)
    lse = torch.zeros(hq, q.shape[0], dtype=torch.float64)
    for h in range(hq):
        s = (q[:, h].double() @ k[:, h // g].double().T) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if keep is not None:
            s = s.masked_fill(~keep, float("-inf"))
        lse[h] = torch.logsumexp(s, dim=-1)
        p = torch.softmax(s, dim=-1)
        p = torch.nan_to_num(p, nan=0.0)
        out[:, h] = p @ v[:, h // g].double()
    lse = torch.where(torch.isinf(lse) & (lse < 0), torch.full_like(lse, float("inf")), lse)
    return out, lse


@pytest.mark.parametrize("hq,hk", [(4, 4), (8, 2), (6, 1)])
@pytest.mark.parametrize("sq,sk", [(1, 700), (5, 1030), (33, 33)])
@pytest.mark.parametrize("causal", [False, True])
def test_blocked_golden_matches_library_softmax(hq, hk, sq, sk, causal):
    g = torch.Generator().manual_seed(sq * 1000 + sk + hq)
    q, k, v = torch.randn(sq, hq, 64, generator=g), torch.randn(sk, hk, 64, generator=g), torch.randn(sk, hk, 64, generator=g)
    wl, wr, ic, il = O.normalize_window(-1, -1, causal, sk)
    mask = O.masked_matrix(sq, sk, ic, il, wl, wr)
    out, lse = O.ref_flash_attention(q, k, v, 0.125, mask, torch.float32)
    ref, ref_lse = textbook(q, k, v, 0.125, None if mask is None else ~mask)
    assert (out.double() - ref).abs().max() < 2e-5
    assert (lse.double() - ref_lse).abs().max() < 2e-5
    o2, l2 = O.attention_fp32(q, k, v, 0.125, mask)
    assert (o2.double() - ref).abs().max() < 2e-5 and (l2.double() - ref_lse).abs().max() < 2e-5


def test_brute_force_tiny():
    # plain Python loops: catches a transposed operand, a dropped scale, a wrong head mapping
    g = torch.Generator().manual_seed(7)
    sq, sk, hq, hk, d = 2, 5, 4, 2, 3
    q, k, v = torch.randn(sq, hq, d, generator=g), torch.randn(sk, hk, d, generator=g), torch.randn(sk, hk, d, generator=g)
    scale = 0.37
    out, lse = O.ref_flash_attention(q, k, v, scale, O.masked_matrix(sq, sk, True, False, -1, 0), torch.float32)
    for i in range(sq):
        for h in range(hq):
            kv = h // (hq // hk)
            vis = [j for j in range(sk) if j <= i + sk - sq]
            s = [scale * sum(float(q[i, h, c]) * float(k[j, kv, c]) for c in range(d)) for j in vis]
            m = max(s)
            w = [math.exp(x - m) for x in s]
            tot = sum(w)
            assert abs(float(lse[h, i]) - (m + math.log(tot))) < 1e-5
            for c in range(d):
                o = sum(wj * float(v[j, kv, c]) for wj, j in zip(w, vis)) / tot
                assert abs(float(out[i, h, c]) - o) < 1e-5


def test_softcap_and_window_match_library():
    g = torch.Generator().manual_seed(3)
    q, k, v = torch.randn(4, 4, 32, generator=g) * 3, torch.randn(600, 2, 32, generator=g) * 3, torch.randn(600, 2, 32, generator=g)
    wl, wr, ic, il = O.normalize_window(100, 7, False, 600)
    mask = O.masked_matrix(4, 600, ic, il, wl, wr)
    out, lse = O.ref_flash_attention(q, k, v, 0.2, mask, torch.float32, softcap=4.0)
    ref, ref_lse = textbook(q, k, v, 0.2, ~mask, softcap=4.0)
    assert (out.double() - ref).abs().max() < 2e-5 and (lse.double() - ref_lse).abs().max() < 2e-5


def test_out_lse_identity():
    # P = exp(S*scale - LSE) sums to one and reproduces out (tests/fa_small_op_golden.py:104-135)
    g = torch.Generator().manual_seed(11)
    q, k, v = torch.randn(3, 2, 16, generator=g), torch.randn(40, 2, 16, generator=g), torch.randn(40, 2, 16, generator=g)
    out, lse = O.ref_flash_attention(q, k, v, 0.25, None, torch.float32)
    for h in range(2):
        p = torch.exp((q[:, h] @ k[:, h].T) * 0.25 - lse[h][:, None])
        assert (p.sum(-1) - 1).abs().max() < 1e-5
        assert (p @ v[:, h] - out[:, h]).abs().max() < 1e-5


def test_p_is_rounded_to_io_dtype_before_pv():
    # the golden casts P to the I/O dtype before PV (tests/test_flash_attn_npu_v2.py:127): with bf16 I/O
    # the blocked golden must differ from the fp32 reference by about bf16 rounding of P, not more
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(1, 4, 64, generator=g).bfloat16(), torch.randn(900, 1, 64, generator=g).bfloat16(),
               torch.randn(900, 1, 64, generator=g).bfloat16())
    gold, _ = O.ref_flash_attention(q, k, v, 0.125, None, torch.bfloat16)
    ref, _ = O.attention_fp32(q, k, v, 0.125, None)
    err = (gold.float() - ref).abs().max().item()
    assert 0 < err < 2e-2


def test_hidden_rows_and_empty_cache():
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.randn(5, 2, 8, generator=g), torch.randn(2, 2, 8, generator=g), torch.randn(2, 2, 8, generator=g)
    mask = O.masked_matrix(5, 2, True, False, -1, 0)
    out, lse = O.ref_flash_attention(q, k, v, 1.0, mask, torch.float32)
    out, lse = O._fix_hidden_rows(out, lse, mask)
    assert (out[:3] == 0).all() and torch.isinf(lse[:, :3]).all() and torch.isfinite(lse[:, 3:]).all()
    o2, l2 = O.attention_fp32(q, k, v, 1.0, mask)
    assert (o2[:3] == 0).all() and torch.isinf(l2[:, :3]).all()
    assert (o2[3:] - out[3:]).abs().max() < 1e-5
    o3, l3 = O.ref_flash_attention(q, k[:0], v[:0], 1.0, None, torch.float32)
    assert (o3 == 0).all() and torch.isinf(l3).all()


def test_varlen_equals_per_sequence():
    g = torch.Generator().manual_seed(9)
    lens = [5, 17, 9]
    cu = torch.tensor([0, 5, 22, 31], dtype=torch.int32)
    q, k, v = torch.randn(31, 4, 16, generator=g), torch.randn(31, 2, 16, generator=g), torch.randn(31, 2, 16, generator=g)
    out, lse = O.flash_attn_varlen(q, k, v, cu, cu, 17, 17, causal=True)
    assert lse.shape == (4, 31)
    for b in range(3):
        a, e = int(cu[b]), int(cu[b + 1])
        ref, ref_lse = textbook(q[a:e], k[a:e], v[a:e], 0.25, ~O.masked_matrix(e - a, e - a, True, False, -1, 0))
        assert (out[a:e].double() - ref).abs().max() < 1e-5 and (lse[:, a:e].double() - ref_lse).abs().max() < 1e-5
