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
    plan = _lib.SplitPlan()
    assert lib.fa_rocm_plan_kvcache(C.byref(a), 256, C.byref(plan)) == 0
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
