"""The entry point that allocates nothing (fa_rocm_fwd_kvcache_static): its split partials live in a static
device array instead of a caller-owned workspace.  Checked through the C ABI against fa_rocm_fwd_kvcache on
the same arguments, bit for bit, on two calls in a row, the second one smaller (so it runs over what the
first left in the array), and against the oracle."""
import ctypes as C

import pytest
import torch

import fa_oracle as O
from flash_attn_npu import _lib
from flash_attn_npu.flash_attn_npu import bind_kvcache
from helpers import check_out, make_paged_case, to_dev

pytestmark = pytest.mark.gpu


def _run_both(B, hq, hk, d, lens, seqlen_q, seed, window=(-1, -1)):
    lib = _lib.load()
    case = make_paged_case(B, hq, hk, d, 256, lens, seqlen_q=seqlen_q, seed=seed)
    dev = to_dev(case, "cuda")
    scale = d ** -0.5
    call = bind_kvcache(dev["q"], dev["k_cache"], dev["v_cache"], None, None, dev["cache_seqlens"], None, None, None,
                        None, dev["block_table"], None, None, scale, True, window[0], window[1], 0.0, False, 0)
    assert call.args.workspace_bytes > 0, "the case must split, or the scratch is not exercised"
    call.run()
    torch.cuda.synchronize()
    out_ref, lse_ref = call.out.clone(), call.lse.clone()
    # the same record, without a workspace, into fresh outputs
    out2 = torch.full_like(call.out, float("nan"))
    lse2 = torch.full_like(call.lse, float("nan"))
    a = _lib.KvcacheArgs()
    C.memmove(C.byref(a), C.byref(call.args), C.sizeof(a))
    a.out, a.softmax_lse = out2.data_ptr(), lse2.data_ptr()
    a.workspace, a.workspace_bytes = None, 0
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    before = torch.cuda.memory_allocated()
    _lib.check(lib.fa_rocm_fwd_kvcache_static(C.byref(a), stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(out2.view(torch.int16), out_ref.view(torch.int16)), "outputs differ from fa_rocm_fwd_kvcache"
    assert torch.equal(lse2, lse_ref), "LSEs differ from fa_rocm_fwd_kvcache"
    ref, ref_lse = O.flash_attn_with_kvcache(case["q"], case["k_cache"], case["v_cache"], None, None,
                                             cache_seqlens=case["cache_seqlens"], block_table=case["block_table"],
                                             causal=True, window_size=window, mode="fp32")
    check_out(out2, ref, lse2, ref_lse, f"static scratch B={B}")


def test_static_scratch_two_calls_second_smaller():
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(700, 3000, (12,), generator=g).tolist()
    _run_both(12, 32, 8, 128, lens, 1, seed=1)
    _run_both(3, 32, 8, 128, [900, 130, 1500], 1, seed=2)      # smaller: fewer rows, shorter, over the stale partials
    _run_both(2, 16, 2, 64, [2000, 77], 2, seed=3)             # other head dimension and block height, same array


def test_static_scratch_rejects_what_does_not_fit():
    lib = _lib.load()
    B, hq = 2, 128
    pool, page = 16, 256
    kc = torch.zeros(pool, page, 1, 576, dtype=torch.int8, device="cuda")
    sc = torch.ones(pool, page, 1, dtype=torch.float32, device="cuda")
    q = torch.zeros(B, 1, hq, 576, dtype=torch.bfloat16, device="cuda")
    lens = torch.tensor([1000, 2000], dtype=torch.int32, device="cuda")
    bt = torch.arange(pool, dtype=torch.int32, device="cuda").view(B, pool // B)
    call = bind_kvcache(q, kc, kc[..., :512], None, None, lens, None, None, None, None, bt, None, None, 192 ** -0.5,
                        True, -1, -1, 0.0, False, 0, sc, None)
    assert call.args.workspace_bytes > (36 << 20)
    a = _lib.KvcacheArgs()
    C.memmove(C.byref(a), C.byref(call.args), C.sizeof(a))
    a.workspace, a.workspace_bytes = None, 0
    rc = lib.fa_rocm_fwd_kvcache_static(C.byref(a), C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -5 and "static scratch" in _lib.last_error()
