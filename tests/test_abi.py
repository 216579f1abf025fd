"""CPU checks of the C ABI: the library loads without a GPU, exports every symbol the header
declares, agrees with the Python binding on the argument records, validates arguments with the
reference's messages, and plans splits consistently.  No compute call is made here."""
import ctypes as C
import os
import re

import pytest
import torch

from flash_attn_npu import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "fa_rocm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fa_rocm_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(_lib.LIB_PATH)
    names = header_functions()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/fa_rocm.h but not exported"
    assert set(names) == set(_lib.EXPORTS), "binding and header list different entry points"


def test_record_sizes_and_version():
    lib = _lib.load()
    assert lib.fa_rocm_abi_version() == _lib.ABI_VERSION == 2
    assert lib.fa_rocm_sizeof_kvcache_args() == C.sizeof(_lib.KvcacheArgs)
    assert lib.fa_rocm_sizeof_varlen_args() == C.sizeof(_lib.VarlenArgs)
    assert lib.fa_rocm_sizeof_split_plan() == C.sizeof(_lib.SplitPlan)


def good_args():
    a = _lib.KvcacheArgs()
    for f in ("q", "out", "softmax_lse", "k_cache", "v_cache", "cache_seqlens", "block_table"):
        setattr(a, f, 0x1000)
    a.batch, a.seqlen_q, a.nheads, a.nheads_k, a.headdim_qk, a.headdim_v = 64, 1, 32, 8, 128, 128
    a.num_blocks, a.page_size, a.max_blocks_per_seq = 1300, 256, 33
    a.q_stride_b, a.q_stride_s, a.q_stride_h = 4096, 4096, 128
    a.o_stride_b, a.o_stride_s, a.o_stride_h = 4096, 4096, 128
    a.k_stride_block, a.k_stride_row, a.k_stride_h = 256 * 1024, 1024, 128
    a.v_stride_block, a.v_stride_row, a.v_stride_h = 256 * 1024, 1024, 128
    a.bt_stride_b = 33
    a.io_dtype = a.kv_dtype = _lib.FA_BF16
    a.softmax_scale = 128 ** -0.5
    a.causal, a.window_left, a.window_right = 1, -1, -1
    return a


def expect_error(a, text):
    lib = _lib.load()
    assert lib.fa_rocm_kvcache_validate(C.byref(a)) != 0
    assert text in _lib.last_error(), _lib.last_error()


def test_validate_messages_follow_the_reference():
    lib = _lib.load()
    assert lib.fa_rocm_kvcache_validate(C.byref(good_args())) == 0
    a = good_args(); a.io_dtype = 7
    expect_error(a, "FlashAttention only supports FP16 and BF16 data types")          # flash_api.cpp:386
    a = good_args(); a.kv_dtype = _lib.FA_FP16
    expect_error(a, "query and key_cache must have the same dtype")                   # :387
    a = good_args(); a.nheads = 30
    expect_error(a, "Number of heads in key/value must divide number of heads in query")   # :457
    a = good_args(); a.headdim_qk = a.headdim_v = 512
    expect_error(a, "FlashAttention only supports head dimension at most 256")        # :456
    a = good_args(); a.batch = 0
    expect_error(a, "batch size must be positive")                                    # :455
    a = good_args(); a.softcap = -1.0
    expect_error(a, "softcap must be non-negative")                                   # :419
    a = good_args(); a.block_table = None
    expect_error(a, "block_table")
    a = good_args(); a.q = None
    expect_error(a, "non-NULL")
    a = good_args(); a.page_size = 100
    expect_error(a, "multiple of 32")
    a = good_args(); a.k_new = 0x1000
    expect_error(a, "k and v must be passed together")
    a = good_args(); a.rotary_cos = a.rotary_sin = 0x1000
    expect_error(a, "rotary embedding is only applied when k and v are passed")
    a = good_args(); a.kv_dtype = _lib.FA_INT8
    expect_error(a, "int8 KV cache needs k_scale_cache")
    assert lib.fa_rocm_kvcache_validate(None) != 0


def test_grid_extent_limits_are_rejected_with_a_message():
    # batch rows and the units of a row index the y / z extents of the explicit-split and combine grids (16 bits each)
    lib = _lib.load()
    a = good_args(); a.batch = 65535
    assert lib.fa_rocm_kvcache_validate(C.byref(a)) == 0
    a.batch = 65536
    expect_error(a, "batch size must be at most 65535")
    a = good_args(); a.nheads = a.nheads_k = 65536
    expect_error(a, "too many units per batch row")
    a = good_args(); a.k_cache = 0x1008
    expect_error(a, "tensor data must be 16-byte aligned")
    plan = _lib.SplitPlan()
    a = good_args(); a.batch = 1 << 20
    assert lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan)) == -3     # the planner accepts what the call accepts
    a = good_args(); a.page_size = 0
    assert lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan)) == -3
    assert lib.fa_rocm_kvcache_workspace_bytes(C.byref(a), 256) == 0


def test_environment_is_read_once_and_on_request(monkeypatch):
    lib = _lib.load()
    plan = _lib.SplitPlan()
    a = good_args()
    lib.fa_rocm_reload_env()
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.num_wgs == 512
    monkeypatch.setenv("FA_ROCM_DECODE_WGS", "100")
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.num_wgs == 512, "the environment was read again on the call path"
    lib.fa_rocm_reload_env()
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.num_wgs == 100
    monkeypatch.delenv("FA_ROCM_DECODE_WGS")
    lib.fa_rocm_reload_env()
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.num_wgs == 512


def test_split_plan_invariants():
    lib = _lib.load()
    plan = _lib.SplitPlan()
    a = good_args()
    assert lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan)) == 0
    assert plan.mode == 1 and plan.num_wgs == 512                      # balanced: two workgroups per CU
    assert plan.num_workers == 2048 and plan.min_share == 2            # one 16-row tile: every wave is a worker
    rows = 4
    assert plan.workspace_bytes == 2048 * 2 * rows * (128 + 1) * 4 + 2048 == lib.fa_rocm_kvcache_workspace_bytes(C.byref(a), 256)
    # 20 rows (two 16-row tiles): every wave is a worker; how it carries the tiles depends on the head dimension
    a.seqlen_q = 5
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))           # d = 128: both tiles in one wave, 20-row partial slots
    assert plan.mode == 1 and plan.num_wgs == 512 and plan.num_workers == 2048
    assert plan.workspace_bytes == 2048 * 2 * 20 * 129 * 4 + 2048
    a.headdim_qk = a.headdim_v = 64                                     # d = 64: the same
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.mode == 1 and plan.num_workers == 2048 and plan.workspace_bytes == 2048 * 2 * 20 * 65 * 4 + 2048
    a.num_splits = 2                                                    # explicit splits: the workgroup-level kernel's grid
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.mode == 0 and plan.num_workers == 0
    a.num_splits = 0
    a.headdim_qk = a.headdim_v = 256                                    # d = 256: two tiles do not fit a wave: the tiled kernel
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.mode == 0 and plan.num_workers == 0
    a.headdim_qk = a.headdim_v = 128
    a.batch = 16                                                        # fewer units (16 x 8) than compute units: the tiled kernel
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.mode == 0 and plan.num_workers == 0
    lib.fa_rocm_plan_kvcache(C.byref(a), 128, C.byref(plan))            # ... on a device of 128 compute units they fill it
    assert plan.mode == 1 and plan.num_workers == 128 * 2 * 4
    a.batch = 64
    a.headdim_qk = a.headdim_v = 128
    a.seqlen_q = 1
    a.num_splits = 1
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.mode == 0 and plan.nsplits == 1 and plan.workspace_bytes == 0 and plan.split_keys >= 33 * 256
    for n in (2, 3, 7, 33, 100):
        a.num_splits = n
        lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
        assert 1 <= plan.nsplits <= n and plan.split_keys % 256 == 0
        assert plan.nsplits * plan.split_keys >= 33 * 256               # the splits cover every addressable key
        assert plan.workspace_bytes == (64 * 8 * plan.nsplits * rows * 129 * 4 if plan.nsplits > 1 else 0)
    # a window bounds the live range: fewer keys per split
    a.num_splits, a.window_left, a.window_right, a.causal = 4, 4095, 0, 0
    lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan))
    assert plan.nsplits * plan.split_keys >= 4096 + 32 and plan.split_keys <= 1280


def test_operator_layer_fails_loudly_without_gpu_tensors():
    from flash_attn_npu import flash_attn_varlen_func, flash_attn_with_kvcache
    q = torch.zeros(1, 1, 8, 128, dtype=torch.bfloat16)
    kc = torch.zeros(4, 256, 2, 128, dtype=torch.bfloat16)
    bt = torch.zeros(1, 2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="ROCm device"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=5, block_table=bt)
    with pytest.raises(RuntimeError, match="FP16 and BF16"):
        flash_attn_with_kvcache(q.float(), kc.float(), kc.float(), cache_seqlens=5, block_table=bt)
    with pytest.raises(RuntimeError, match="ROCm device"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=5)   # dense cache: valid call, still no CPU path
    with pytest.raises(RuntimeError, match="Paged KVcache does not support cache_batch_idx"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=5, block_table=bt, cache_batch_idx=torch.zeros(1, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="alibi"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=5, block_table=bt, alibi_slopes=torch.zeros(8))
    with pytest.raises(RuntimeError, match="leftpad"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=5, block_table=bt, cache_leftpad=torch.zeros(1, dtype=torch.int32))
    cu = torch.tensor([0, 4], dtype=torch.int32)
    x = torch.zeros(4, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="dropout"):
        flash_attn_varlen_func(x, x, x, cu, cu, 4, 4, dropout_p=0.1)
    with pytest.raises(RuntimeError, match="ROCm device"):
        flash_attn_varlen_func(x, x, x, cu, cu, 4, 4)
    with pytest.raises(RuntimeError, match="inference forward only"):
        flash_attn_varlen_func(x.requires_grad_(), x, x, cu, cu, 4, 4)
    x = x.detach()
    # arguments that would otherwise be ignored without a word (reference flash_api.cpp:886,890)
    from flash_attn_npu.flash_attn_npu_interface import _varlen_forward_eager
    with pytest.raises(RuntimeError, match="does not support zero_tensors"):
        _varlen_forward_eager(x, x, x, cu, cu, 4, 4, 0.0, 0.1, False, zero_tensors=True)
    with pytest.raises(RuntimeError, match="does not support seqused_k"):
        _varlen_forward_eager(x, x, x, cu, cu, 4, 4, 0.0, 0.1, False, seqused_k=torch.tensor([4], dtype=torch.int32))
    with pytest.raises(RuntimeError, match="only applied together with new k / v"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=5, block_table=bt, rotary_cos=torch.zeros(8, 32, dtype=torch.bfloat16),
                                rotary_sin=torch.zeros(8, 32, dtype=torch.bfloat16))


def test_operator_layer_checks_every_shape_the_kernels_index_with():
    """The kernels index v_cache and the scale caches with k_cache's page ids, rows and heads, and the table and the
    lengths with the batch of q: a tensor that is smaller than that would be read out of bounds on the device, so it
    is refused on the host, before the device check (these run without a GPU)."""
    from flash_attn_npu import flash_attn_with_kvcache
    from flash_attn_npu.flash_attn_npu import _C
    q = torch.zeros(2, 1, 8, 128, dtype=torch.bfloat16)
    kc = torch.zeros(4, 256, 2, 128, dtype=torch.bfloat16)
    bt = torch.zeros(2, 2, dtype=torch.int32)
    lens = torch.tensor([5, 6], dtype=torch.int32)
    for bad_v in (kc[:3], kc[:, :128], kc[:, :, :1]):
        with pytest.raises(RuntimeError, match="vcache must have the num_blocks, page_block_size and nheads_k of kcache"):
            flash_attn_with_kvcache(q, kc, bad_v, cache_seqlens=lens, block_table=bt)
    with pytest.raises(RuntimeError, match=r"block_table must be \(batch_size, max_num_blocks_per_seq\)"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=lens, block_table=bt.view(-1))
    with pytest.raises(RuntimeError, match="block_table / cache_seqlens batch mismatch"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=lens, block_table=bt[:1])
    with pytest.raises(RuntimeError, match=r"seqlens_k must be \(batch_size,\)"):
        flash_attn_with_kvcache(q, kc, kc, cache_seqlens=lens.view(2, 1), block_table=bt)
    # int8 latent cache: scale caches must cover every (block, row, head) of the code cache
    q8 = torch.zeros(2, 1, 128, 576, dtype=torch.bfloat16)
    codes = torch.zeros(4, 256, 1, 576, dtype=torch.int8)
    scales = torch.ones(4, 256, 1)
    for bad_s in (scales[:3], scales[:, :64], scales.double(), scales.view(4, 256)):
        with pytest.raises(RuntimeError, match="k_scale_cache must be fp32"):
            flash_attn_with_kvcache(q8, codes, codes[..., :512], cache_seqlens=lens, block_table=bt, k_scale_cache=bad_s,
                                    v_scale_cache=scales)
    with pytest.raises(RuntimeError, match="v_scale_cache must match"):
        flash_attn_with_kvcache(q8, codes, codes[..., :512], cache_seqlens=lens, block_table=bt, k_scale_cache=scales,
                                v_scale_cache=scales[:2])
    # varlen: paged v against paged k, table and lengths against the batch
    cu = torch.tensor([0, 4, 8], dtype=torch.int32)
    x = torch.zeros(8, 8, 128, dtype=torch.bfloat16)
    ext = _C()
    tail = (4, 4, 0.0, 0.1, False, True, -1, -1, 0.0, False, None)
    with pytest.raises(RuntimeError, match="paged v must have"):
        ext.varlen_fwd(x, kc, kc[:3], None, cu, None, lens, None, bt, None, *tail)
    with pytest.raises(RuntimeError, match=r"block_table must be \(batch_size"):
        ext.varlen_fwd(x, kc, kc, None, cu, None, lens, None, bt[:1], None, *tail)
    with pytest.raises(RuntimeError, match=r"seqused_k must be \(batch_size,\)"):
        ext.varlen_fwd(x, kc, kc, None, cu, None, lens[:1], None, bt, None, *tail)
    with pytest.raises(RuntimeError, match="v must have the total_k and nheads_k of k"):
        ext.varlen_fwd(x, x, x[:4], None, cu, cu, None, None, None, None, *tail)
    with pytest.raises(RuntimeError, match=r"cu_seqlens_k must have batch_size \+ 1 entries"):
        ext.varlen_fwd(x, x, x, None, cu, cu[:2], None, None, None, None, *tail)


def test_extension_module_takes_the_reference_argument_lists():
    """flash_attn_npu.varlen_fwd is called by the reference's Python with 21 positional arguments, the last one the
    random generator, passed as None (flash_attn_npu_interface.py:160-185; flash_api.cpp:848-869); fwd_kvcache with 20
    (flash_attn_npu_interface.py:1556-1577).  Both argument lists must bind; num_splits of varlen_fwd is a trailing
    extra with a default."""
    from flash_attn_npu.flash_attn_npu import _C
    ext = _C()
    cu = torch.tensor([0, 4], dtype=torch.int32)
    x = torch.zeros(4, 8, 128, dtype=torch.bfloat16)
    ref_args = (x, x, x, None, cu, cu, None, None, None, None, 4, 4, 0.0, 0.1, False, True, -1, -1, 0.0, False, None)
    assert len(ref_args) == 21
    with pytest.raises(RuntimeError, match="ROCm device"):      # bound, checked, refused only for want of a GPU
        ext.varlen_fwd(*ref_args)
    with pytest.raises(RuntimeError, match="ROCm device"):
        ext.varlen_fwd(*ref_args, 2)
    with pytest.raises(RuntimeError, match="ROCm device"):
        ext.varlen_fwd(*ref_args[:20], torch.Generator())
    with pytest.raises(RuntimeError, match="ROCm device"):
        ext.varlen_fwd(*ref_args[:20], num_splits=1)
    q = torch.zeros(1, 1, 8, 128, dtype=torch.bfloat16)
    kc = torch.zeros(4, 256, 2, 128, dtype=torch.bfloat16)
    kv_args = (q, kc, kc, None, None, torch.tensor([5], dtype=torch.int32), None, None, None, None,
               torch.zeros(1, 2, dtype=torch.int32), None, None, 0.1, True, -1, -1, 0.0, True, 0)
    assert len(kv_args) == 20
    with pytest.raises(RuntimeError, match="ROCm device"):
        ext.fwd_kvcache(*kv_args)


def test_padded_copy_of_a_cache_is_bounded():
    """Head dimensions that are not multiples of 8 run through a padded copy of the cache; that is refused, with a
    message, once the cache is large (meta tensors: no memory is touched)."""
    from flash_attn_npu import flash_attn_npu as ops
    small = torch.empty(64, 128, 16, 111, dtype=torch.bfloat16, device="meta")
    ops._check_padded_cache_copy(small, small)
    big = torch.empty(4096, 256, 8, 111, dtype=torch.bfloat16, device="meta")     # 1.9 GB per cache
    with pytest.raises(RuntimeError, match="not a multiple of 8.*refuses.*rounded up to a multiple of 8"):
        ops._check_padded_cache_copy(big, big)


def test_even_cu_seqlens_of_empty_sequences():
    from flash_attn_npu.flash_attn_npu_interface import _even_cu_seqlens
    assert _even_cu_seqlens(3, 0, "cpu").tolist() == [0, 0, 0, 0]
    assert _even_cu_seqlens(3, 5, "cpu").tolist() == [0, 5, 10, 15]
    assert _even_cu_seqlens(1, 7, "cpu").dtype == torch.int32


def test_missing_library_is_an_error(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libfa_rocm.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_package_exports_reference_names():
    # reference flash_attn_npu/__init__.py:12-21
    import flash_attn_npu
    for name in ("flash_attn_func", "flash_attn_kvpacked_func", "flash_attn_qkvpacked_func", "flash_attn_varlen_func",
                 "flash_attn_varlen_kvpacked_func", "flash_attn_varlen_qkvpacked_func", "flash_attn_with_kvcache"):
        assert callable(getattr(flash_attn_npu, name)), name


def test_build_scans_the_assembly_of_hand_written_matrix_instructions():
    """The build reads the device assembly of the latent kernel: the compiler may not use an accumulation register
    of its own, and no hand-written matrix instruction may read what the vector instruction right in front of it
    wrote (the compiler inserts no wait states for instructions it does not know)."""
    import importlib.util
    import os
    spec = importlib.util.spec_from_file_location(
        "fa_build", os.path.join(os.path.dirname(__file__), "..", "flash-attention-npu_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    good = ["\tv_mov_b32_e32 v4, 0", "\t;;#ASMSTART", "\tv_mfma_f32_32x32x16_bf16 a[0:15], v[8:11], v[12:15], a[0:15]", "\t;;#ASMEND",
            "\tv_add_f32_e32 v1, v2, v3"]
    build.scan_assembly("k.hip", "k.s", good)
    stray = good + ["\tv_accvgpr_write_b32 a7, v1"]
    with pytest.raises(RuntimeError, match="accumulation register"):
        build.scan_assembly("k.hip", "k.s", stray)
    hazard = ["\tv_mov_b64_e32 v[8:9], s[0:1]", "\t;;#ASMSTART", "\tv_mfma_f32_32x32x16_bf16 a[0:15], v[8:11], v[8:11], 0", "\t;;#ASMEND"]
    with pytest.raises(RuntimeError, match="matrix instruction reads"):
        build.scan_assembly("k.hip", "k.s", hazard)
    spaced = ["\tv_mov_b64_e32 v[8:9], s[0:1]", "\t;;#ASMSTART", "\ts_nop 3", "\tv_mfma_f32_32x32x16_bf16 a[0:15], v[8:11], v[8:11], 0", "\t;;#ASMEND"]
    build.scan_assembly("k.hip", "k.s", spaced)
