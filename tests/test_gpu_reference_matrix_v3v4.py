"""The parameter matrices of the reference's third- and fourth-generation forward tests, replayed row for row.

  tests/test_flash_attn_npu_v3.py:148-316   145 kvcache rows x cache_mode {0, 1} x num_splits {0, 2}: batch-major ("BSND")
                                            and token-major ("TND") queries over dense, packed and paged (128-key pages)
                                            caches, `is_varied` per-sequence lengths, signed windows such as (508, -256)
                                            and (-128, 1024), softcap 30, D = 1, 4, 128, 256; U(-5, 5) inputs (:319-358)
  tests/test_flash_attn_npu_v3.py:545-567   20 dense-forward rows (flash_attn_func)
  tests/test_flash_attn_npu_v3.py:622-660   33 varlen rows (flash_attn_varlen_func)
  tests/test_flash_attn_npu_v4.py:220-406   137 rows x num_splits {0, 1, 2} of the paged / packed / dense varlen matrix,
                                            U(-1, 1) inputs (:416-419), paged gather as :529-535

The rows are data: tests/golden/reference_matrix_v3.json and reference_matrix_v4.json, written by
tests/golden/make_reference_matrix.py from the text of those files.  The skips are the reference's (num_splits > 1 needs
a paged cache and token-major q; `is_varied` needs token-major q).  Lengths of `is_varied` rows are drawn as the reference
draws them (seed 1234: q in [1, q_seqlen], then kv in [q, kv_seqlen]); its page tables are the reference's contiguous ones.
All rows run through the flash_attn_npu_3 surface (the fourth generation's call surface is not rebuilt; its matrix
exercises the same paged / packed / dense varlen path).  Bars: the reference's rtol = atol = 1e-2 on out and LSE against
the blocked golden (v3 :540-543, v4 :609-612), and for the fourth-generation rows its element-wise rule against both the
blocked and the plain fp32 golden (v4 :614-619).  The fourth generation's blocked golden moves its running maximum lazily
(rescale_threshold 4, v4 :46-48), which changes where P is rounded and nothing else; the oracle's blocked golden is the
plain one.  A row's golden is computed once and shared by its layout / split variants.

The inputs are seeded (the reference draws unseeded).  With U(-5, 5) inputs the scores have a standard deviation of about
8, a row's weight sits on one or two keys, and rounding P to bf16 (half an ulp = 2^-10 of a weight near 1/2, times values
of magnitude 5) moves an output by up to 5e-3 per such key: two correct evaluations that round P at different places can
differ by 1e-2 on an element, i.e. by the reference's bar.  One seed of the dense 5 x 1024 x 1024 causal row put a single
element of 2.6 million 3e-4 outside it (|golden| 0.044, difference 0.0107); the seeds used here do not."""
import json
import os

import pytest
import torch

import fa_oracle as O
from helpers import check_compare_rule, check_vs_golden

pytestmark = pytest.mark.gpu

_HERE = os.path.dirname(os.path.abspath(__file__))
_M3 = json.load(open(os.path.join(_HERE, "golden", "reference_matrix_v3.json")))
_M4 = json.load(open(os.path.join(_HERE, "golden", "reference_matrix_v4.json")))
_DT = {"bfloat16": torch.bfloat16, "float16": torch.float16}
PAGE = 128     # both test files overwrite the row's block size with 128 (v3 :323, v4 :420)


def _cu(lengths):
    out = [0]
    for n in lengths:
        out.append(out[-1] + int(n))
    return torch.tensor(out, dtype=torch.int32)


_golden = {}   # the last row's case and goldens: variants of a row follow each other


def _row_case(tag, idx, dtype, B, hq, hk, sq, sk, d, is_varied, lo, hi, causal, wl, wr, softcap):
    """Per-sequence q / k / v of a row (packed), its lengths, and the two goldens."""
    key = (tag, idx)
    if _golden.get("key") == key:
        return _golden["case"]
    gen = torch.Generator().manual_seed(1234)
    if is_varied:
        q_lens = torch.randint(low=1, high=sq + 1, size=(B,), generator=gen).tolist()
        k_lens = [int(torch.randint(low=q, high=sk + 1, size=(1,), generator=gen)) for q in q_lens]
    else:
        q_lens, k_lens = [sq] * B, [sk] * B
    q = (lo + (hi - lo) * torch.rand(sum(q_lens), hq, d, generator=gen)).to(dtype)
    k = (lo + (hi - lo) * torch.rand(sum(k_lens), hk, d, generator=gen)).to(dtype)
    v = (lo + (hi - lo) * torch.rand(sum(k_lens), hk, d, generator=gen)).to(dtype)
    cu_q, cu_k = _cu(q_lens), _cu(k_lens)
    kw = dict(causal=causal, window_size=(wl, wr), softcap=softcap)
    gold = O.flash_attn_varlen(q, k, v, cu_q, cu_k, sq, sk, mode="golden", **kw)
    ref = O.flash_attn_varlen(q, k, v, cu_q, cu_k, sq, sk, mode="fp32", **kw)
    case = dict(q=q, k=k, v=v, q_lens=q_lens, k_lens=k_lens, cu_q=cu_q, cu_k=cu_k, gold=gold, ref=ref)
    _golden["key"], _golden["case"] = key, case
    return case


def _run(case, B, hq, hk, sq, sk, d, dtype, layout, cache_mode, num_splits, causal, wl, wr, softcap):
    """One call of the third-generation kvcache surface in the row's layout; returns token-major (out, lse)."""
    from flash_attn_npu_3 import flash_attn_with_kvcache
    q, k, v, k_lens, cu_k = case["q"], case["k"], case["v"], case["k_lens"], case["cu_k"]
    table = None
    if cache_mode == 1:
        per_seq = (sk + PAGE - 1) // PAGE
        nblk = max(64, per_seq * B)
        kc = torch.zeros(nblk, PAGE, hk, d, dtype=dtype)
        vc = torch.zeros(nblk, PAGE, hk, d, dtype=dtype)
        table = torch.arange(per_seq * B, dtype=torch.int32).view(B, per_seq)
        for b in range(B):
            n = k_lens[b]
            kc.view(-1, hk, d)[b * per_seq * PAGE: b * per_seq * PAGE + n] = k[cu_k[b]:cu_k[b + 1]]
            vc.view(-1, hk, d)[b * per_seq * PAGE: b * per_seq * PAGE + n] = v[cu_k[b]:cu_k[b + 1]]
    elif layout == "BSND":
        kc, vc = k.view(B, sk, hk, d), v.view(B, sk, hk, d)
    else:
        kc, vc = k, v        # packed: the keys of the sequences back to back
    kw = dict(cache_seqlens=torch.tensor(k_lens, dtype=torch.int32).cuda(), page_table=None if table is None else table.cuda(),
              causal=causal, window_size=[wl, wr], softcap=softcap, rotary_interleaved=False, num_splits=num_splits,
              return_softmax_lse=True)
    if layout == "BSND":
        out, lse, *rest = flash_attn_with_kvcache(q.view(B, sq, hq, d).cuda(), kc.cuda(), vc.cuda(), None, None, None, **kw)
        torch.cuda.synchronize()
        assert out.shape == (B, sq, hq, d) and lse.shape == (B, hq, sq) and len(rest) == 2
        return out.reshape(B * sq, hq, d), lse.permute(1, 0, 2).reshape(hq, B * sq)
    out, lse, *rest = flash_attn_with_kvcache(q.cuda(), kc.cuda(), vc.cuda(), None, None, None, cu_seqlens_q=case["cu_q"].cuda(),
                                              max_seqlen_q=sq, **kw)
    torch.cuda.synchronize()
    assert out.shape == q.shape and lse.shape == (hq, q.shape[0]) and len(rest) == 2
    return out, lse


def _v3_params():
    out = []
    for i, r in enumerate(_M3["kvcache"]):
        layout, is_varied = r[9], r[10]
        if is_varied and layout != "TND":
            continue
        for cache_mode, num_splits in ((0, 0), (1, 0), (1, 2)):
            if num_splits > 1 and layout != "TND":
                continue
            out.append(pytest.param(i, cache_mode, num_splits, id=f"{i:03d}-" + "-".join(str(x) for x in r) + f"-cm{cache_mode}-ns{num_splits}"))
    return out


@pytest.mark.parametrize("idx,cache_mode,num_splits", _v3_params())
def test_reference_v3_kvcache_matrix(idx, cache_mode, num_splits):
    dtype, B, hq, hk, sq, sk, d, _block, causal, layout, is_varied, wl, wr, softcap = _M3["kvcache"][idx]
    dtype = _DT[dtype]
    print("v3 kvcache matrix row", idx, _M3["kvcache"][idx], "cache_mode", cache_mode, "num_splits", num_splits, flush=True)
    case = _row_case("v3", idx, dtype, B, hq, hk, sq, sk, d, is_varied, -5.0, 5.0, causal, wl, wr, softcap)
    out, lse = _run(case, B, hq, hk, sq, sk, d, dtype, layout, cache_mode, num_splits, causal, wl, wr, softcap)
    check_vs_golden(out, case["gold"][0], lse, case["gold"][1], f"v3 row {idx} cm{cache_mode} ns{num_splits}")


def _v4_params():
    out = []
    for i, r in enumerate(_M4["varlen"]):
        cache_mode, layout, is_varied = r[7], r[10], r[11]
        if is_varied and layout != "TND":
            continue
        for num_splits in (0, 1, 2):
            if num_splits > 1 and not (cache_mode == 1 and layout == "TND"):
                continue
            out.append(pytest.param(i, num_splits, id=f"{i:03d}-" + "-".join(str(x) for x in r) + f"-ns{num_splits}"))
    return out


@pytest.mark.parametrize("idx,num_splits", _v4_params())
def test_reference_v4_varlen_matrix(idx, num_splits):
    dtype, B, hq, hk, sq, sk, d, cache_mode, _block, causal, layout, is_varied, wl, wr = _M4["varlen"][idx]
    dtype = _DT[dtype]
    print("v4 varlen matrix row", idx, _M4["varlen"][idx], "num_splits", num_splits, flush=True)
    case = _row_case("v4", idx, dtype, B, hq, hk, sq, sk, d, is_varied, -1.0, 1.0, causal, wl, wr, 0.0)
    out, lse = _run(case, B, hq, hk, sq, sk, d, dtype, layout, cache_mode, num_splits, causal, wl, wr, 0.0)
    what = f"v4 row {idx} ns{num_splits}"
    check_vs_golden(out, case["gold"][0], lse, case["gold"][1], what)
    check_compare_rule(out, case["gold"][0], what + " (blocked golden)")
    check_compare_rule(out, case["ref"][0], what + " (fp32 golden)")


def _ids(rows):
    return [f"{i:03d}-" + "-".join(str(x) for x in r) for i, r in enumerate(rows)]


@pytest.mark.parametrize("row", _M3["dense"], ids=_ids(_M3["dense"]))
def test_reference_v3_dense_forward_matrix(row):
    from flash_attn_npu_3 import flash_attn_func
    dtype, B, hq, hk, sq, sk, d, with_lse, causal, softcap = row
    dtype = _DT[dtype]
    g = torch.Generator().manual_seed(sq * 17 + B * 3 + hq)
    q, k, v = ((-5.0 + 10.0 * torch.rand(B, s, h, d, generator=g)).to(dtype) for s, h in ((sq, hq), (sk, hk), (sk, hk)))
    print("v3 dense matrix row", row, flush=True)
    ret = flash_attn_func(q.cuda(), k.cuda(), v.cuda(), softmax_scale=d ** -0.5, causal=causal, window_size=[-1, -1], softcap=softcap,
                          return_attn_probs=with_lse)
    torch.cuda.synchronize()
    out, lse = (ret[0], ret[1]) if with_lse else (ret, None)
    gold = O.flash_attn_varlen(q.reshape(B * sq, hq, d), k.reshape(B * sk, hk, d), v.reshape(B * sk, hk, d), _cu([sq] * B), _cu([sk] * B),
                               sq, sk, causal=causal, softcap=softcap, mode="golden")
    out_t = out.reshape(B * sq, hq, d)
    if lse is None:
        torch.testing.assert_close(out_t.float().cpu(), gold[0].float(), rtol=1e-2, atol=1e-2)
    else:
        assert lse.shape == (B, hq, sq)
        check_vs_golden(out_t, gold[0], lse.permute(1, 0, 2).reshape(hq, B * sq), gold[1], str(row))


@pytest.mark.parametrize("row", _M3["varlen"], ids=_ids(_M3["varlen"]))
def test_reference_v3_varlen_matrix(row):
    from flash_attn_npu_3 import flash_attn_varlen_func
    dtype, B, hq, hk, sq, sk, d, causal, wl, wr, softcap = row
    dtype = _DT[dtype]
    g = torch.Generator().manual_seed(sq + 3 * sk + d)
    q = (-5.0 + 10.0 * torch.rand(B * sq, hq, d, generator=g)).to(dtype)
    k = (-5.0 + 10.0 * torch.rand(B * sk, hk, d, generator=g)).to(dtype)
    v = (-5.0 + 10.0 * torch.rand(B * sk, hk, d, generator=g)).to(dtype)
    cu_q, cu_k = _cu([sq] * B), _cu([sk] * B)
    print("v3 varlen matrix row", row, flush=True)
    out, lse = flash_attn_varlen_func(q.cuda(), k.cuda(), v.cuda(), cu_q.cuda(), cu_k.cuda(), sq, sk, softmax_scale=d ** -0.5,
                                      causal=causal, window_size=(wl, wr), softcap=softcap, return_attn_probs=True)
    torch.cuda.synchronize()
    gold = O.flash_attn_varlen(q, k, v, cu_q, cu_k, sq, sk, causal=causal, window_size=(wl, wr), softcap=softcap, mode="golden")
    check_vs_golden(out, gold[0], lse, gold[1], str(row))


def test_v3_varlen_seqused_k_limits_the_keys_of_each_sequence():
    """seqused_k with packed keys (reference host: flash_attn_npu_3/flash_api.cpp:143-147): sequence b uses the first
    seqused_k[b] keys of its cu_seqlens_k span, and the causal / window alignment follows that length.  Checked
    against the oracle on the truncated sequences; the keys behind the used ones are NaN."""
    from flash_attn_npu_3 import flash_attn_varlen_func
    hq, hk, d = 8, 2, 128
    q_lens, spans, used = [5, 130, 1, 64], [700, 400, 33, 64], [650, 130, 33, 1]
    g = torch.Generator().manual_seed(5)
    q = torch.randn(sum(q_lens), hq, d, generator=g).to(torch.bfloat16)
    k = torch.randn(sum(spans), hk, d, generator=g).to(torch.bfloat16)
    v = torch.randn(sum(spans), hk, d, generator=g).to(torch.bfloat16)
    cu_q, cu_span = _cu(q_lens), _cu(spans)
    kt = torch.cat([k[cu_span[b]:cu_span[b] + used[b]] for b in range(4)])
    vt = torch.cat([v[cu_span[b]:cu_span[b] + used[b]] for b in range(4)])
    for b in range(4):
        k[cu_span[b] + used[b]:cu_span[b + 1]] = float("nan")
        v[cu_span[b] + used[b]:cu_span[b + 1]] = float("nan")
    for causal, window in ((False, (-1, -1)), (True, (-1, -1)), (False, (100, 20))):
        print("v3 varlen seqused_k", causal, window, flush=True)
        out, lse = flash_attn_varlen_func(q.cuda(), k.cuda(), v.cuda(), cu_q.cuda(), cu_span.cuda(), max(q_lens), max(spans),
                                          seqused_k=torch.tensor(used, dtype=torch.int32).cuda(), causal=causal, window_size=window,
                                          return_attn_probs=True)
        torch.cuda.synchronize()
        ref, ref_lse = O.flash_attn_varlen(q, kt, vt, cu_q, _cu(used), max(q_lens), max(spans), causal=causal, window_size=window,
                                           mode="fp32")
        from helpers import check_out
        check_out(out, ref, lse, ref_lse, f"seqused_k causal={causal} window={window}")
