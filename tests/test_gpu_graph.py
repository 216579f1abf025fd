"""A bound kvcache call records into a HIP graph: run() only enqueues kernels (no allocation, no host
sync, lengths read on the device), so a serving loop can capture one decode step and replay it while
cache_seqlens, the block table and the new k / v change in place."""
import pytest
import torch

import fa_oracle as O
from helpers import check_out, make_paged_case, rotary_tables, to_dev

pytestmark = pytest.mark.gpu


def test_decode_step_replays_from_a_graph():
    from flash_attn_npu import flash_attn_npu as op
    B, hq, hk, d, page = 6, 32, 8, 128, 64
    lens0 = [100, 64, 1, 500, 255, 0]
    steps = 4
    case = make_paged_case(B, hq, hk, d, page, [l + steps for l in lens0], seqlen_new=1, seed=60)
    case["cache_seqlens"] = torch.tensor(lens0, dtype=torch.int32)
    cos, sin = rotary_tables(1024, 64)
    dev = to_dev(case)
    cos_d, sin_d = cos.cuda(), sin.cuda()
    out = torch.empty(B, 1, hq, d, dtype=torch.bfloat16, device="cuda")
    call = op.bind_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"], dev["cache_seqlens"], cos_d, sin_d,
                           None, None, dev["block_table"], None, out, d ** -0.5, True, -1, -1, 0.0, False, 0)
    # warm up on a side stream, then capture one step
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    kc0, vc0 = dev["k_cache"].clone(), dev["v_cache"].clone()
    with torch.cuda.stream(s):
        call.run()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    dev["k_cache"].copy_(kc0)
    dev["v_cache"].copy_(vc0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call.run()
    dev["k_cache"].copy_(kc0)
    dev["v_cache"].copy_(vc0)
    torch.cuda.synchronize()

    g = torch.Generator().manual_seed(61)
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    lens = torch.tensor(lens0, dtype=torch.int32)
    for step in range(steps):
        q = torch.randn(B, 1, hq, d, generator=g).to(torch.bfloat16)
        kn = torch.randn(B, 1, hk, d, generator=g).to(torch.bfloat16)
        vn = torch.randn(B, 1, hk, d, generator=g).to(torch.bfloat16)
        # new inputs written in place, some eager work between replays
        dev["q"].copy_(q)
        dev["k"].copy_(kn)
        dev["v"].copy_(vn)
        dev["cache_seqlens"].copy_(lens)
        _ = (dev["q"].float() * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        ref, ref_lse = O.flash_attn_with_kvcache(q, kc, vc, kn, vn, rotary_cos=cos, rotary_sin=sin, cache_seqlens=lens,
                                                 block_table=case["block_table"], causal=True, rotary_interleaved=False, mode="fp32")
        print("graph step", step, lens.tolist(), flush=True)
        assert torch.equal(dev["k_cache"].cpu().view(torch.int16), kc.view(torch.int16)), f"step {step}: appended K differs"
        assert torch.equal(dev["v_cache"].cpu().view(torch.int16), vc.view(torch.int16)), f"step {step}: appended V differs"
        check_out(call.out, ref, call.lse, ref_lse, f"graph step {step}")
        lens = lens + 1
