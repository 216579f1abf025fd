"""Seeded input builders and tolerance checks shared by the tests, smoke() and bench.py."""
from __future__ import annotations

import math

import torch

# parity bars: 16-bit outputs vs the fp32 reference, LSE relative
OUT_MAX_ABS = 2e-2
OUT_MEAN_ABS = 2e-3
LSE_REL = 1e-3
# the reference's own test bar vs its blocked golden (tests/test_flash_attn_npu_v2.py:430-433)
REF_RTOL = 1e-2
REF_ATOL = 1e-2


def make_paged_case(B, hq, hk, d, page, lens, seqlen_q=1, seqlen_new=0, dtype=torch.bfloat16, seed=0,
                    spare_blocks=3, dist="normal", dv=None, extra_table_cols=0):
    """Random paged cache with a non-contiguous block table.

    Pages per row = ceil((len + seqlen_new) / page); pool = sum(pages) + spare; the table is
    slices of a seeded permutation of the pool.  dist: "normal" N(0,1) or "uniform5" U(-5,5)
    (the reference tests' distribution, tests/test_flash_attn_npu_v2.py:290-302)."""
    g = torch.Generator().manual_seed(seed)
    dv = d if dv is None else dv

    def rnd(*shape):
        if dist == "normal":
            return torch.randn(*shape, generator=g)
        return -5.0 + 10.0 * torch.rand(*shape, generator=g)

    lens = [int(x) for x in lens]
    pages = [max(1, math.ceil((l + seqlen_new) / page)) for l in lens]
    pool = sum(pages) + spare_blocks
    maxp = max(pages) + extra_table_cols
    perm = torch.randperm(pool, generator=g)
    bt = torch.zeros(B, maxp, dtype=torch.int32)
    o = 0
    for b in range(B):
        bt[b, :pages[b]] = perm[o:o + pages[b]].to(torch.int32)
        o += pages[b]
    case = dict(
        q=rnd(B, seqlen_q, hq, d).to(dtype),
        k_cache=rnd(pool, page, hk, d).to(dtype),
        v_cache=rnd(pool, page, hk, dv).to(dtype),
        cache_seqlens=torch.tensor(lens, dtype=torch.int32),
        block_table=bt,
        k=None, v=None,
    )
    if seqlen_new:
        case["k"] = rnd(B, seqlen_new, hk, d).to(dtype)
        case["v"] = rnd(B, seqlen_new, hk, dv).to(dtype)
    return case


def rotary_tables(seqlen_ro, rotary_dim, theta=500000.0, dtype=torch.bfloat16):
    inv = theta ** (-torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim)
    ang = torch.arange(seqlen_ro, dtype=torch.float64)[:, None] * inv[None, :]
    return torch.cos(ang).to(dtype), torch.sin(ang).to(dtype)


def to_dev(case, device="cuda"):
    return {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in case.items()}


def check_out(out, ref_fp32, lse, ref_lse, what=""):
    """Parity bars: max-abs 2e-2, mean-abs 2e-3 vs fp32; LSE 1e-3 relative."""
    out = out.detach().float().cpu()
    ref = ref_fp32.detach().float().cpu()
    err = (out - ref).abs()
    assert torch.isfinite(out).all(), f"{what}: non-finite output"
    assert err.max().item() <= OUT_MAX_ABS, f"{what}: max abs err {err.max().item():.3e}"
    assert err.mean().item() <= OUT_MEAN_ABS, f"{what}: mean abs err {err.mean().item():.3e}"
    if lse is not None:
        l = lse.detach().float().cpu()
        r = ref_lse.detach().float().cpu()
        inf_ref = torch.isinf(r)
        assert torch.equal(torch.isinf(l), inf_ref), f"{what}: +inf LSE rows differ"
        fin = ~inf_ref
        if fin.any():
            rel = ((l[fin] - r[fin]).abs() / r[fin].abs().clamp_min(1.0)).max().item()
            assert rel <= LSE_REL, f"{what}: LSE rel err {rel:.3e}"


def check_vs_golden(out, golden, lse, golden_lse, what=""):
    """The reference's own bar against its blocked golden (rtol = atol = 1e-2)."""
    torch.testing.assert_close(out.detach().float().cpu(), golden.float(), rtol=REF_RTOL, atol=REF_ATOL, msg=lambda m: f"{what}: {m}")
    l = lse.detach().float().cpu()
    fin = ~torch.isinf(golden_lse)
    assert torch.equal(torch.isinf(l), torch.isinf(golden_lse)), f"{what}: +inf LSE rows differ"
    torch.testing.assert_close(l[fin], golden_lse[fin], rtol=REF_RTOL, atol=REF_ATOL, msg=lambda m: f"{what} lse: {m}")


def check_compare_rule(out, ref_fp32, what="", rel=5e-3, floor=5e-3, share=0.995):
    """The element-wise rule of the reference's fourth-generation tests (tests/npu_precision_utils.py:130-164, used at
    tests/test_flash_attn_npu_v4.py:614-619): at least 99.5 % of the elements lie within max(5e-3 * |golden|, 5e-3)."""
    o = out.detach().float().cpu().flatten()
    g = ref_fp32.detach().float().cpu().flatten()
    limit = torch.maximum(g.abs() * rel, torch.tensor(floor))
    ok = ((o - g).abs() <= limit).float().mean().item()
    assert ok >= share, f"{what}: only {100 * ok:.3f} % of the elements within max({rel}*|g|, {floor})"


import contextlib


@contextlib.contextmanager
def library_env(**settings):
    """Set FA_ROCM_* variables for the calls inside the block.  The library reads its environment once, so it is told
    to read it again on the way in and on the way out."""
    import os
    from flash_attn_npu import _lib
    old = {k: os.environ.get(k) for k in settings}
    os.environ.update({k: str(v) for k, v in settings.items()})
    _lib.load().fa_rocm_reload_env()
    try:
        yield
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        _lib.load().fa_rocm_reload_env()
