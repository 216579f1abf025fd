"""Host plan of kvcache calls whose query block goes to the tiled kernel (no GPU needed): the keys
are cut into ranges only when the tiles alone cannot fill the device, never into ranges shorter than
256 keys, and the workspace holds the rotated q (rotary) in front of the partials."""
import ctypes as C

from flash_attn_npu import _lib


def plan_of(batch, sq, hq, hk, d, max_blocks, page=256, num_splits=0, rotary=False):
    lib = _lib.load()
    a = _lib.KvcacheArgs()
    a.batch, a.seqlen_q, a.nheads, a.nheads_k, a.headdim_qk, a.headdim_v = batch, sq, hq, hk, d, d
    a.page_size, a.max_blocks_per_seq, a.num_blocks = page, max_blocks, max_blocks * batch
    a.window_left = a.window_right = -1
    a.num_splits = num_splits
    if rotary:
        a.rotary_cos = a.rotary_sin = 256   # only tested for being non-NULL by the planner
        a.k_new = a.v_new = 256
        a.seqlen_new = sq
        a.rotary_dim, a.seqlen_ro = d, 1 << 20
    plan = _lib.SplitPlan()
    assert lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan)) == 0, _lib.last_error()
    return plan


def test_tall_plan():
    rows = 16 * 8
    # 64 sequences x 8 kv heads of packed 128-row tiles fill the 512 slots: no cut
    p = plan_of(64, 16, 64, 8, 128, 32)
    assert p.mode == 0 and p.nsplits == 1 and p.workspace_bytes == 0
    # one sequence: 8 tiles for 512 slots -> 64 ranges at most, 256 keys each at least
    p = plan_of(1, 16, 64, 8, 128, 512)
    assert p.nsplits == 64 and p.workspace_bytes == 1 * 8 * 64 * rows * 129 * 4
    p = plan_of(1, 16, 64, 8, 128, 16)          # 4096 addressable keys: 16 ranges
    assert p.nsplits == 16
    p = plan_of(1, 16, 64, 8, 128, 1)           # 256 keys: nothing to cut
    assert p.nsplits == 1 and p.workspace_bytes == 0
    # explicit counts: 1 = never, n = at most n
    assert plan_of(1, 16, 64, 8, 128, 512, num_splits=1).nsplits == 1
    assert plan_of(1, 16, 64, 8, 128, 512, num_splits=3).nsplits == 3
    # head dimension 256 runs one workgroup per compute unit
    assert plan_of(4, 128, 8, 8, 256, 512).nsplits == 8
    # rotary: the rotated q (rounded up to 256 bytes) comes first
    q_bytes = 1 * 24 * 16 * 128 * 2
    p = plan_of(1, 24, 16, 2, 128, 32, rotary=True)
    assert p.nsplits == 32 and p.workspace_bytes == q_bytes + 1 * 2 * 32 * (24 * 8) * 129 * 4


def test_varlen_split_plan():
    # the planner: paged only, never with num_splits = 1, at least 256 keys per range, at most 64 ranges
    import ctypes as C
    from flash_attn_npu import _lib
    lib = _lib.load()
    a = _lib.VarlenArgs()
    fake = 0x1000        # the planner and the checks never follow a pointer
    for f in ("q", "k", "v", "out", "softmax_lse", "cu_seqlens_q", "seqused_k", "block_table"):
        setattr(a, f, fake)
    a.batch, a.total_q, a.nheads, a.nheads_k, a.headdim = 2, 598, 8, 2, 128      # two blocks of 299 tokens
    a.max_seqlen_q, a.max_seqlen_k, a.page_size, a.max_blocks_per_seq, a.num_blocks = 299, 100000, 64, 2000, 4000
    a.q_stride_t = a.o_stride_t = 1024
    a.q_stride_h = a.o_stride_h = a.k_stride_h = a.v_stride_h = 128
    a.k_stride_t = a.v_stride_t = 256
    a.io_dtype = 0
    n = lib.fa_rocm_varlen_num_splits(C.byref(a), 256)
    assert 1 < n <= 64
    assert 0 <= lib.fa_rocm_varlen_workspace_bytes(C.byref(a), 256) - 598 * 8 * n * 129 * 4 < 256
    a.num_splits = 1
    assert lib.fa_rocm_varlen_num_splits(C.byref(a), 256) == 1 and lib.fa_rocm_varlen_workspace_bytes(C.byref(a), 256) == 0
    a.num_splits = 500
    assert lib.fa_rocm_varlen_num_splits(C.byref(a), 256) == 64
    a.num_splits, a.max_seqlen_k = 0, 700
    assert lib.fa_rocm_varlen_num_splits(C.byref(a), 256) == 3
    a.max_seqlen_k, a.total_q, a.max_seqlen_q = 100000, 40000, 20000          # the tiles fill the device: no cut
    assert lib.fa_rocm_varlen_num_splits(C.byref(a), 256) == 1
    a.total_q, a.max_seqlen_q, a.block_table = 598, 299, None
    a.cu_seqlens_k = fake
    assert lib.fa_rocm_varlen_num_splits(C.byref(a), 256) == 1
    # a workspace that is too small is refused before anything is launched
    a.block_table, a.num_splits = fake, 4
    a.workspace, a.workspace_bytes = fake, 16
    assert lib.fa_rocm_varlen_fwd(C.byref(a), None) == -5 and b"workspace" in lib.fa_rocm_last_error()


def test_varlen_short_blocks_workspace():
    # a prompt chunk among decode rows: the one-token blocks are computed by the decode kernels, whose batch-major
    # rows and own workspace follow the partials in the caller's workspace
    lib = _lib.load()
    a = _lib.VarlenArgs()
    fake = 0x1000
    for f in ("q", "k", "v", "out", "softmax_lse", "cu_seqlens_q", "seqused_k", "block_table"):
        setattr(a, f, fake)
    a.batch, a.total_q, a.nheads, a.nheads_k, a.headdim = 16, 527, 32, 8, 128
    a.max_seqlen_q, a.max_seqlen_k, a.page_size, a.max_blocks_per_seq, a.num_blocks = 512, 32768, 256, 128, 4096
    a.q_stride_t = a.o_stride_t = 4096
    a.q_stride_h = a.o_stride_h = a.k_stride_h = a.v_stride_h = 128
    a.k_stride_t = a.v_stride_t = 1024
    a.k_stride_block = a.v_stride_block = 1024 * 256
    a.io_dtype = 0
    n = lib.fa_rocm_varlen_num_splits(C.byref(a), 256)
    partials = 527 * 32 * n * 129 * 4 if n > 1 else 0
    rows = 16 * 32
    least = partials + 2 * rows * 128 * 2 + rows * 4 + 16 * 4
    with_rows = lib.fa_rocm_varlen_workspace_bytes(C.byref(a), 256)
    assert with_rows > least
    a.batch, a.total_q, a.max_seqlen_q = 3, 302, 300     # one chunk, two decode rows: uneven as well
    small = lib.fa_rocm_varlen_workspace_bytes(C.byref(a), 256)
    n3 = lib.fa_rocm_varlen_num_splits(C.byref(a), 256)
    assert small > (302 * 32 * n3 * 129 * 4 if n3 > 1 else 0) + 2 * 3 * 4 * 32 * 128 * 2
    a.batch, a.total_q, a.max_seqlen_q = 16, 527, 40     # blocks of similar length: nothing is routed
    assert lib.fa_rocm_varlen_workspace_bytes(C.byref(a), 256) < with_rows - partials + 527 * 32 * 64 * 129 * 4
    a.max_seqlen_q = 512
    a.nheads, a.nheads_k = 64, 1                       # 64 q heads per kv head: taller than the decode kernels take
    a.q_stride_t = a.o_stride_t = 8192
    n2 = lib.fa_rocm_varlen_num_splits(C.byref(a), 256)
    assert 0 <= lib.fa_rocm_varlen_workspace_bytes(C.byref(a), 256) - (527 * 64 * n2 * 129 * 4 if n2 > 1 else 0) < 256
