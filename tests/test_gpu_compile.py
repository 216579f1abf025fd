"""The two public calls traced by torch.compile (the reference registers its forward as a custom
op with a fake implementation for exactly this, flash_attn_npu_interface.py:137-224): dynamo must
capture them as single graph nodes without a graph break, the fake implementations must give the
real shapes and dtypes, and the compiled call must write the cache and return the same bits as the
eager one."""
import pytest
import torch

from helpers import make_paged_case, rotary_tables, to_dev
from test_gpu_prefill import varlen_case

pytestmark = pytest.mark.gpu


def test_kvcache_call_under_torch_compile():
    from flash_attn_npu import flash_attn_with_kvcache
    case = make_paged_case(3, 16, 4, 128, 64, [100, 63, 640], seqlen_q=1, seqlen_new=1, seed=61)
    cos, sin = rotary_tables(1024, 64)
    cos, sin = cos.cuda(), sin.cuda()

    def step(q, kc, vc, k, v, lens, table):
        return flash_attn_with_kvcache(q, kc, vc, k, v, rotary_cos=cos, rotary_sin=sin, cache_seqlens=lens, block_table=table,
                                       causal=True, rotary_interleaved=False, return_softmax_lse=True)

    eager = to_dev(case)
    out_e, lse_e = step(eager["q"], eager["k_cache"], eager["v_cache"], eager["k"], eager["v"], eager["cache_seqlens"],
                        eager["block_table"])
    comp = to_dev(case)
    print("compile kvcache", flush=True)
    compiled = torch.compile(step, backend="eager", fullgraph=True)
    out_c, lse_c = compiled(comp["q"], comp["k_cache"], comp["v_cache"], comp["k"], comp["v"], comp["cache_seqlens"],
                            comp["block_table"])
    torch.cuda.synchronize()
    assert torch.equal(out_c, out_e) and torch.equal(lse_c, lse_e)
    assert torch.equal(comp["k_cache"], eager["k_cache"]) and torch.equal(comp["v_cache"], eager["v_cache"])
    assert not torch.equal(comp["k_cache"].cpu(), case["k_cache"])      # the append really happened


def test_varlen_call_under_torch_compile():
    from flash_attn_npu import flash_attn_varlen_func
    c = varlen_case([100, 300, 77], [100, 300, 77], 8, 2, 128, seed=62)
    q, k, v, cu = c["q"].cuda(), c["k"].cuda(), c["v"].cuda(), c["cu_q"].cuda()

    def fwd(q, k, v, cu):
        return flash_attn_varlen_func(q, k, v, cu, cu, 300, 300, causal=True, return_attn_probs=True)

    out_e, lse_e, _ = fwd(q, k, v, cu)
    print("compile varlen", flush=True)
    out_c, lse_c, _ = torch.compile(fwd, backend="eager", fullgraph=True)(q, k, v, cu)
    torch.cuda.synchronize()
    assert torch.equal(out_c, out_e) and torch.equal(lse_c, lse_e)


def test_fake_implementations_match_the_ops():
    case = to_dev(make_paged_case(2, 8, 2, 128, 64, [100, 200], seqlen_q=2, seqlen_new=2, seed=63))
    args = (case["q"], case["k_cache"], case["v_cache"], case["k"], case["v"], case["cache_seqlens"], None, None, None, None,
            case["block_table"], None, 128 ** -0.5, True, -1, -1, 0.0, True, 0, None, None)
    import flash_attn_npu  # noqa: F401  registers the ops
    print("opcheck kvcache", flush=True)
    torch.library.opcheck(torch.ops.flash_attn_npu._flash_attn_kvcache_forward.default, args,
                          test_utils=("test_schema", "test_faketensor"))
    c = varlen_case([50, 70], [50, 70], 4, 2, 128, seed=64)
    cu = c["cu_q"].cuda()
    print("opcheck varlen", flush=True)
    torch.library.opcheck(torch.ops.flash_attn_npu._flash_attn_varlen_forward.default,
                          (c["q"].cuda(), c["k"].cuda(), c["v"].cuda(), cu, cu, 70, 70, 0.0, 128 ** -0.5, True),
                          test_utils=("test_schema", "test_faketensor"))
