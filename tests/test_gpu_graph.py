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


def test_mixed_token_major_batch_replays_from_a_graph():
    # a prompt chunk among decode rows through the third-generation surface: which block has one token, how long the
    # contexts are and where the key ranges fall are all read on the device, so the captured call follows lengths and
    # block boundaries that change in place (same total number of query tokens)
    from flash_attn_npu_3 import flash_attn_with_kvcache
    B, hq, hk, d, page = 6, 16, 4, 128, 128
    cap = 5000
    case = make_paged_case(B, hq, hk, d, page, [cap] * B, seed=70)
    total_q, max_q = 205, 200
    kc, vc, table = case["k_cache"].cuda(), case["v_cache"].cuda(), case["block_table"].cuda()
    q_d = torch.zeros(total_q, hq, d, dtype=torch.bfloat16, device="cuda")
    cu_d = torch.zeros(B + 1, dtype=torch.int32, device="cuda")
    lens_d = torch.zeros(B, dtype=torch.int32, device="cuda")

    def call():
        return flash_attn_with_kvcache(q_d, kc, vc, page_table=table, cache_seqlens=lens_d, cu_seqlens_q=cu_d, max_seqlen_q=max_q,
                                       causal=True, return_softmax_lse=True)[:2]

    settings = [([1, 1, 200, 1, 1, 1], [4000, 129, 4500, 3000, 1, 77]),
                ([1, 200, 1, 1, 1, 1], [300, 2500, 4999, 0, 640, 1024]),
                ([2, 1, 199, 1, 1, 1], [2000, 4000, 900, 33, 4100, 128])]

    def load(q_lens, k_lens, q):
        q_d.copy_(q)
        cu_d.copy_(torch.tensor([0] + torch.tensor(q_lens).cumsum(0).tolist(), dtype=torch.int32))
        lens_d.copy_(torch.tensor(k_lens, dtype=torch.int32))

    g = torch.Generator().manual_seed(71)
    load(*settings[0], torch.randn(total_q, hq, d, generator=g).to(torch.bfloat16))
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        call()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g, lse_g = call()
    for rep, (q_lens, k_lens) in enumerate(settings + settings[:1]):
        q = torch.randn(total_q, hq, d, generator=g).to(torch.bfloat16)
        load(q_lens, k_lens, q)
        _ = (q_d.float() * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        cu_q = torch.tensor([0] + torch.tensor(q_lens).cumsum(0).tolist(), dtype=torch.int32)
        cu_k = torch.tensor([0] + torch.tensor(k_lens).cumsum(0).tolist(), dtype=torch.int32)
        kl = torch.cat([O.gather_paged(case["k_cache"], case["block_table"][b], k_lens[b]) for b in range(B)])
        vl = torch.cat([O.gather_paged(case["v_cache"], case["block_table"][b], k_lens[b]) for b in range(B)])
        ref, ref_lse = O.flash_attn_varlen(q, kl, vl, cu_q, cu_k, max_q, max(k_lens), causal=True, mode="fp32")
        print("mixed graph replay", rep, q_lens, k_lens, flush=True)
        check_out(out_g, ref, lse_g, ref_lse, f"mixed graph replay {rep}")
        out_e, lse_e = call()
        torch.cuda.synchronize()
        assert torch.equal(out_e.cpu(), out_g.cpu()), "replay differs from the eager call"
