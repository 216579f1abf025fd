"""Head dimensions between the widths the kernels are compiled for (64, 128, 256): every multiple of 8 up to 256 runs on
the caller's tensors as they are - no padded copy of the cache - on every kernel family (wave-level decode, block-level
decode with fixed splits, tiled forward, their combines, the append with rotary).  Dimensions that are not multiples of
8 take the padded-copy path and still match."""
import pytest
import torch

import fa_oracle as O
from helpers import check_out, make_paged_case, rotary_tables, to_dev
from test_gpu_prefill import check_paged, paged_ragged

pytestmark = pytest.mark.gpu

DIMS = [8, 16, 24, 40, 48, 56, 72, 80, 96, 104, 112, 120, 136, 160, 192, 200, 224, 248]
LENS = [700, 1, 0, 2049, 64, 33]


def run_kvcache(d, sq, snew, dtype=torch.bfloat16, num_splits=0, rotary=0, nan_other_head=False, seed=0, **kw):
    from flash_attn_npu import flash_attn_with_kvcache
    hq, hk = 8, 2
    case = make_paged_case(len(LENS), hq, hk, d, 64, LENS, seqlen_q=sq, seqlen_new=snew, dtype=dtype, seed=seed)
    if nan_other_head:
        # kv head 1 holds NaN everywhere: a lane of head 0 that read behind its own row would pick it up
        case["k_cache"][:, :, 1] = float("nan")
        case["v_cache"][:, :, 1] = float("nan")
    dev = to_dev(case)
    rot = {}
    if rotary:
        cos, sin = rotary_tables(4096, rotary, dtype=dtype)
        rot = dict(rotary_cos=cos, rotary_sin=sin, rotary_interleaved=False)
    out, lse = flash_attn_with_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], dev["k"], dev["v"], cache_seqlens=dev["cache_seqlens"],
                                       block_table=dev["block_table"], return_softmax_lse=True, num_splits=num_splits,
                                       **{k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in rot.items()}, **kw)
    torch.cuda.synchronize()
    kc, vc = case["k_cache"].clone(), case["v_cache"].clone()
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], kc, vc, case["k"], case["v"], cache_seqlens=case["cache_seqlens"],
                                             block_table=case["block_table"], mode="fp32", **rot, **kw)
    if nan_other_head:
        g = hq // hk
        out, ref, lse, ref_lse = out[:, :, :g], ref[:, :, :g], lse[:, :g], ref_lse[:, :g]
        assert torch.isfinite(out.float()).all(), "NaN from the neighbouring head's rows"
    check_out(out, ref, lse, ref_lse, f"d={d} sq={sq} snew={snew} splits={num_splits}")
    if snew:
        # the appended rows, bit for bit (only the rows of head 0 when the other head is NaN)
        h = slice(0, 1) if nan_other_head else slice(None)
        assert torch.equal(dev["k_cache"].cpu()[:, :, h].view(torch.int16), kc[:, :, h].view(torch.int16)), "k_cache after the append"
        assert torch.equal(dev["v_cache"].cpu()[:, :, h].view(torch.int16), vc[:, :, h].view(torch.int16)), "v_cache after the append"


@pytest.mark.parametrize("d", DIMS)
def test_wave_decode(d):
    print("head dim: wave decode", d, flush=True)
    run_kvcache(d, 1, 1, causal=True, nan_other_head=True)
    run_kvcache(d, 3, 0, causal=False, dtype=torch.float16, seed=1)


@pytest.mark.parametrize("d", [d for d in DIMS if d <= 128])
def test_wave_decode_with_two_tiles_in_a_wave(d):
    """28 and 24 rows as two 16-row tiles carried by one wave (the rule takes that path when the call has at least as
    many units as the device has compute units; the knob takes it for these small cases)."""
    from helpers import library_env
    print("head dim: wave decode, two tiles", d, flush=True)
    with library_env(FA_ROCM_WAVE_TWO_TILES=1):
        run_kvcache(d, 7, 2, causal=True, nan_other_head=True)
        run_kvcache(d, 6, 0, causal=False, window_size=(300, 10), dtype=torch.float16, seed=5)


@pytest.mark.parametrize("d", DIMS)
def test_block_decode_and_fixed_splits(d):
    print("head dim: block decode", d, flush=True)
    run_kvcache(d, 7, 2, causal=True, nan_other_head=True)                     # 28 rows: the workgroup is the worker
    run_kvcache(d, 1, 0, causal=True, num_splits=3, seed=2)                    # grid of fixed splits + its combine
    run_kvcache(d, 6, 1, causal=False, num_splits=2, window_size=(300, 10), dtype=torch.float16, seed=3)


@pytest.mark.parametrize("d", DIMS)
def test_tiled_forward_over_the_cache(d):
    print("head dim: tiled", d, flush=True)
    run_kvcache(d, 40, 40, causal=True, nan_other_head=True)
    run_kvcache(d, 130, 0, causal=True, num_splits=4, softcap=15.0, seed=4)


@pytest.mark.parametrize("d,rot", [(96, 32), (96, 96), (192, 64), (72, 16), (48, 48), (200, 128)])
@pytest.mark.parametrize("sq", [1, 6, 40])
def test_rotary_append(d, rot, sq):
    print("head dim: rotary", d, rot, sq, flush=True)
    run_kvcache(d, sq, sq, causal=True, rotary=rot, seed=5)


@pytest.mark.parametrize("d", [3, 4, 9, 33, 100, 250])
def test_dimensions_that_are_not_multiples_of_8(d):
    print("head dim: padded copies", d, flush=True)
    run_kvcache(d, 1, 1, causal=True, seed=6)
    run_kvcache(d, 40, 0, causal=True, seed=7)


@pytest.mark.parametrize("d", [24, 72, 96, 160, 192, 100])
@pytest.mark.parametrize("causal", [True, False])
def test_varlen_packed_and_paged(d, causal):
    from flash_attn_npu import flash_attn_varlen_func
    from flash_attn_npu.flash_attn_npu import varlen_fwd
    print("head dim: varlen", d, causal, flush=True)
    lens_q = [1, 300, 1, 0, 17, 40]
    lens_k = [5000, 3100, 40, 700, 2100, 0]
    case, q, cu_q, cu_k, kl, vl = paged_ragged(lens_q, lens_k, 8, 2, d, 64, seed=40 + d)
    ref, ref_lse = O.flash_attn_varlen(q, kl, vl, cu_q, cu_k, max(lens_q), max(lens_k), causal=causal, mode="fp32")
    out, lse, _ = flash_attn_varlen_func(q.cuda(), kl.cuda(), vl.cuda(), cu_q.cuda(), cu_k.cuda(), max(lens_q), max(lens_k),
                                         causal=causal, return_attn_probs=True)
    check_paged(out, ref, lse, ref_lse, f"packed d={d}")
    for num_splits in (0, 1, 5):
        kc, vc = case["k_cache"].cuda(), case["v_cache"].cuda()
        out, lse, _, _ = varlen_fwd(q.cuda(), kc, vc, None, cu_q.cuda(), None, case["cache_seqlens"].cuda(), None,
                                    case["block_table"].cuda(), None, max(lens_q), max(lens_k), 0.0, d ** -0.5, False, causal, -1, -1,
                                    0.0, False, None, num_splits=num_splits)
        torch.cuda.synchronize()
        check_paged(out, ref, lse, ref_lse, f"paged d={d} splits={num_splits}")


@pytest.mark.parametrize("d", [96, 192])
def test_no_copy_of_the_cache(d):
    """A pool of ~0.4 GB per cache: the calls may allocate their outputs and split partials (tens of MB), never a padded
    copy of the pool."""
    from flash_attn_npu import flash_attn_with_kvcache
    from flash_attn_npu.flash_attn_npu import varlen_fwd
    hq, hk, page, B = 8, 2, 64, 8
    blocks = (400 << 20) // (page * hk * d * 2)
    g = torch.Generator(device="cuda").manual_seed(d)
    kc = torch.randn(blocks, page, hk, d, generator=g, device="cuda", dtype=torch.bfloat16)
    vc = torch.randn(blocks, page, hk, d, generator=g, device="cuda", dtype=torch.bfloat16)
    table = torch.randperm(blocks, device="cuda")[: B * 40].to(torch.int32).view(B, 40)
    lens = torch.tensor([2500, 17, 1, 2559, 640, 1000, 2000, 64], dtype=torch.int32, device="cuda")
    limit = 64 << 20
    for sq in (1, 6, 64):
        q = torch.randn(B, sq, hq, d, generator=g, device="cuda", dtype=torch.bfloat16)
        kn = torch.randn(B, 1, hk, d, generator=g, device="cuda", dtype=torch.bfloat16)
        print("head dim: no cache copy", d, sq, flush=True)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        out = flash_attn_with_kvcache(q, kc, vc, kn, kn, cache_seqlens=lens, block_table=table, causal=True)
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated() - before
        assert peak < limit, f"sq={sq}: the call allocated {peak} bytes beside a {kc.numel() * 2}-byte cache"
        # spot check against the oracle on one batch row (its keys gathered on the device, appended one included)
        b = 4
        n = int(lens[b]) + 1
        pos = torch.arange(n, device="cuda")
        ks = kc[table[b].long()[pos // page], pos % page].cpu()[None]
        vs = vc[table[b].long()[pos // page], pos % page].cpu()[None]
        ref, _ = O.flash_attn_with_kvcache(q[b:b + 1].cpu(), ks, vs, cache_seqlens=torch.tensor([n], dtype=torch.int32),
                                           block_table=torch.zeros(1, 1, dtype=torch.int32), causal=True, mode="fp32")
        assert (out[b:b + 1].float().cpu() - ref).abs().max() < 2e-2
    cu_q = torch.arange(B + 1, dtype=torch.int32, device="cuda") * 33
    q = torch.randn(B * 33, hq, d, generator=g, device="cuda", dtype=torch.bfloat16)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    varlen_fwd(q, kc, vc, None, cu_q, None, lens, None, table, None, 33, 2560, 0.0, d ** -0.5, False, True, -1, -1, 0.0, False, None)
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - before
    assert peak < limit, f"paged varlen allocated {peak} bytes beside a {kc.numel() * 2}-byte cache"


def test_abi_rejects_rows_that_are_not_16_byte_pieces():
    import ctypes as C
    from flash_attn_npu import _lib
    from test_abi import expect_error, good_args
    a = good_args(); a.headdim_qk = a.headdim_v = 100
    expect_error(a, "head dimension must be a positive multiple of 8")
    a = good_args(); a.headdim_qk = a.headdim_v = 96
    a.q_stride_h = a.o_stride_h = a.k_stride_h = a.v_stride_h = 96
    assert _lib.load().fa_rocm_kvcache_validate(C.byref(a)) == 0, _lib.last_error()
    plan = _lib.SplitPlan()
    _lib.load().fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.workspace_bytes == 2048 * 2 * 4 * (128 + 1) * 4 + 2048   # partial rows are as wide as the compiled kernel; + the partition header
