"""Strided inputs through the C ABI: q / k / v as slices of one fused projection output, a cache
whose memory is laid out (block, head, row, dim), a block table cut out of a wider one, an output
buffer inside a larger tensor, a latent cache with padded rows.  The library takes element strides,
so every such call must give the bits of the same call on contiguous copies."""
import pytest
import torch

from helpers import make_paged_case, rotary_tables, to_dev
from test_gpu_mla import mla_case
from test_gpu_prefill import varlen_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("sq,snew", [(1, 1), (3, 3), (40, 40)])
def test_kvcache_strided_everything(sq, snew):
    from flash_attn_npu import flash_attn_with_kvcache
    B, hq, hk, d = 3, 16, 4, 128
    case = to_dev(make_paged_case(B, hq, hk, d, 64, [100, 63, 640], seqlen_q=sq, seqlen_new=snew, seed=71))
    cos, sin = rotary_tables(1024, 64)
    cos, sin = cos.cuda(), sin.cuda()
    kw = dict(rotary_cos=cos, rotary_sin=sin, causal=True, rotary_interleaved=False, return_softmax_lse=True)
    # contiguous run
    kc0, vc0 = case["k_cache"].clone(), case["v_cache"].clone()
    out0, lse0 = flash_attn_with_kvcache(case["q"], kc0, vc0, case["k"], case["v"], cache_seqlens=case["cache_seqlens"],
                                         block_table=case["block_table"], **kw)
    # strided run: q, k, v inside one fused tensor, (block, head, row, dim) cache memory, table inside
    # a wider one, output inside a wider one
    fused = torch.zeros(B, sq, (hq + 2 * hk) * d + 8, dtype=torch.bfloat16, device="cuda")
    fused[..., :hq * d] = case["q"].reshape(B, sq, -1)
    fused[..., hq * d:(hq + hk) * d] = case["k"].reshape(B, sq, -1)
    fused[..., (hq + hk) * d:(hq + 2 * hk) * d] = case["v"].reshape(B, sq, -1)
    q = fused[..., :hq * d].view(B, sq, hq, d)
    k = fused[..., hq * d:(hq + hk) * d].view(B, sq, hk, d)
    v = fused[..., (hq + hk) * d:(hq + 2 * hk) * d].view(B, sq, hk, d)
    kc1 = case["k_cache"].permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    vc1 = case["v_cache"].permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    assert not q.is_contiguous() and not kc1.is_contiguous()
    wide = torch.full((B, case["block_table"].shape[1] + 5), -1, dtype=torch.int32, device="cuda")
    wide[:, :case["block_table"].shape[1]] = case["block_table"]
    table = wide[:, :case["block_table"].shape[1]]
    print("strided kvcache", sq, q.stride(), kc1.stride(), table.stride(), flush=True)
    out1, lse1 = flash_attn_with_kvcache(q, kc1, vc1, k, v, cache_seqlens=case["cache_seqlens"], block_table=table, **kw)
    torch.cuda.synchronize()
    assert torch.equal(out1, out0) and torch.equal(lse1, lse0)
    assert torch.equal(kc1, kc0) and torch.equal(vc1, vc0)


def test_operator_layer_strided_out():
    # the operator layer's out_ argument: a view with a batch stride larger than its rows
    from flash_attn_npu import flash_attn_npu as ops
    case = to_dev(make_paged_case(2, 8, 2, 128, 64, [300, 64], seed=72))
    args = (case["q"], case["k_cache"], case["v_cache"], None, None, case["cache_seqlens"], None, None, None, None,
            case["block_table"], None)
    tail = (128 ** -0.5, True, -1, -1, 0.0, True, 0)
    out0, lse0 = ops.fwd_kvcache(*args, None, *tail)
    big = torch.zeros(2, 1, 8, 256, dtype=torch.bfloat16, device="cuda")
    out1, lse1 = ops.fwd_kvcache(*args, big[..., :128], *tail)
    torch.cuda.synchronize()
    assert out1.data_ptr() == big.data_ptr() and torch.equal(out1, out0) and torch.equal(lse1, lse0)
    assert torch.count_nonzero(big[..., 128:]) == 0


def test_varlen_fused_qkv_views():
    from flash_attn_npu import flash_attn_varlen_func
    c = varlen_case([100, 300, 77], [100, 300, 77], 8, 2, 128, seed=73)
    cu = c["cu_q"].cuda()
    out0, lse0, _ = flash_attn_varlen_func(c["q"].cuda(), c["k"].cuda(), c["v"].cuda(), cu, cu, 300, 300, causal=True,
                                           return_attn_probs=True)
    qkv = torch.cat([c["q"], c["k"], c["v"]], dim=1).cuda()          # (total, 8 + 2 + 2, 128)
    q, k, v = qkv[:, :8], qkv[:, 8:10], qkv[:, 10:12]
    assert not k.is_contiguous()
    out1, lse1, _ = flash_attn_varlen_func(q, k, v, cu, cu, 300, 300, causal=True, return_attn_probs=True)
    torch.cuda.synchronize()
    assert torch.equal(out1, out0) and torch.equal(lse1, lse0)


def test_latent_cache_with_padded_rows():
    from flash_attn_npu import flash_attn_with_kvcache
    case = mla_case(2, 128, [700, 300], seed=74)
    kc = case["k_cache"].cuda()
    kw = dict(cache_seqlens=case["cache_seqlens"].cuda(), block_table=case["block_table"].cuda(), softmax_scale=192 ** -0.5,
              causal=True, return_softmax_lse=True, k_scale_cache=case["k_scale"].cuda())
    out0, lse0 = flash_attn_with_kvcache(case["q"].cuda(), kc, kc[..., :512], **kw)
    padded = torch.zeros(kc.shape[0], kc.shape[1], 1, 640, dtype=torch.int8, device="cuda")
    padded[..., :576] = kc
    kc1 = padded[..., :576]
    qbig = torch.zeros(2, 1, 128, 600, dtype=torch.bfloat16, device="cuda")
    qbig[..., :576] = case["q"].cuda()
    out1, lse1 = flash_attn_with_kvcache(qbig[..., :576], kc1, kc1[..., :512], **kw)
    torch.cuda.synchronize()
    assert torch.equal(out1, out0) and torch.equal(lse1, lse0)
