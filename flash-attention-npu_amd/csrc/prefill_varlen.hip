// Tiled attention forward on the bf16/fp16 MFMA for gfx950: variable-length (token-major) prefill
// over dense or paged K/V, and kvcache calls whose query block is too tall for the decode kernel.
//
// Stands in for the reference's FAInfer kernel in TND layout (csrc/ascend910/flash_attn_npu/
// mha_fwd_kvcache.cpp:436-970 with per-sequence offsets :469-475,505-507; host mha_varlen_fwd,
// flash_api.cpp:848-1089).  Where the reference ping-pongs S, P and O_tmp between its matrix and
// vector cores through global memory, everything between the K/V tile loads and the final store
// stays in registers here:
//   * one workgroup = 128 query rows of one (sequence, q head); 4 waves x 32 rows.  Short query
//     blocks under GQA are packed instead (p.pack = group): the 128 rows are (query, head of the
//     group) pairs of one kv head, query-major, so a 16-token block of an 8-head group fills a tile
//     and K/V are read once per kv head (the reference packs heads the same way, flash_api.cpp:33-95);
//   * K/V tiles of 64 keys are fetched once per workgroup, 16 bytes per lane, straight from global memory
//     into LDS (no register holds them and no LDS store instruction moves them: such a store keeps the
//     wave from issuing anything else for ~50 cycles, and the tile stores were a tenth of the kernel's
//     time), double-buffered (K rows XOR-swizzled so MFMA operand reads are conflict free: the lane that
//     fills a piece's place in LDS fetches the piece that belongs there);
//   * S^T = K Q^T and O^T = V^T P^T on the 32x32x16 MFMA: a query row is one lane column in both
//     products, so the running max / sum / rescale never leave the lane (one xor-32 exchange);
//   * V^T operands come straight from the transposing LDS read (ds_read_b64_tr_b16);
//   * key tiles outside the causal / window range of the 128-row block are never loaded.
#include <type_traits>

#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {

constexpr int kBM = 128;  // query rows per workgroup
constexpr int kBN = 64;   // keys per tile

template <int D> struct PrefillCfg {
    static constexpr int kKSteps = D / 16;        // MFMA k-steps of QK^T
    static constexpr int kMT = D / 32;            // 32-column tiles of O^T
    static constexpr int kCPL = D / 32;           // V columns a lane owns per key row
    static constexpr int kChunks = D / 8;         // 16-byte pieces per row
    // XOR swizzle of the 16-byte pieces of a K row; the mask must not see the row step of the
    // tile stores (256 / kChunks rows), so it is 7 for D = 256
    static constexpr int kSwz = (kChunks == 16) ? 15 : 7;
    static constexpr int kTileBytes = kBN * D * 2;
    static constexpr int kVRowBytes = D * 2 + 64;        // padded V rows: transposing reads spread over all banks
    static constexpr int kVTileBytes = kBN * kVRowBytes;
    // A tile is filled by loads that go from global memory straight to LDS (global_load_lds_dwordx4): one instruction
    // of a wave fills 64 consecutive 16-byte pieces, lane l the piece at the instruction's LDS base + 16 l, from
    // whatever address the lane names.  The four waves share the pieces of a tile, instruction by instruction.
    static constexpr int kKLoads = kBN * kChunks / 256;            // per wave and K tile
    static constexpr int kVRowPieces = kVRowBytes / 16;            // data pieces and padding
    static constexpr int kVLoads = kBN * kVRowPieces / 256;        // per wave and V tile
    static_assert(kBN * kChunks % 256 == 0 && kBN * kVRowPieces % 256 == 0, "whole instructions per wave");
};

// EXT: packed heads and / or a split of the keys (p.pack, p.nsplits); without it both are compiled out
// One 128-row block of one (sequence, key range, kv head, q head) of the launch: `bid` is its place in the
// launch's order.  n_long < 0: the units are the launch's batch rows; otherwise they are the first n_long entries of
// p.long_ids (the sequences the tiled kernel computes, listed on the device).
// PART: the head dimension p.headdim is below D: pieces of the q / k / v rows behind it are zeros that nobody loads,
// k-steps and output tiles that only see such pieces are skipped, and the stores stop at the head dimension.
template <typename T, int D, bool PAGED, bool SOFTCAP, bool EXT, bool PART>
__device__ __forceinline__ void prefill_block(const PrefillParams &p, const unsigned bid, const int n_long,
                                              uint8_t (&s_k)[2][PrefillCfg<D>::kTileBytes],
                                              uint8_t (&s_v)[2][PrefillCfg<D>::kVTileBytes]) {
    using Cfg = PrefillCfg<D>;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lh = lane >> 5;   // half: MFMA k-slot
    const int ln = lane & 31;   // MFMA row / column
    const int hd = PART ? p.headdim : D;

    // Workgroup i of the 1-D grid runs on XCD i % 8.  The grid is ordered by 128-row block, tallest
    // first, and inside a block by position e: XCD lane e % 8 walks the units (sequence, key range,
    // kv head) congruent to it, the q heads of a unit one after the other.  Every XCD so gets the same
    // mix of tall and short causal blocks whatever the number of blocks is, and the heads that share
    // a unit's K/V meet in one L2.
    const int nsplits = EXT ? max(p.nsplits, 1) : 1;
    const int heads_per_unit = (EXT && p.pack > 1) ? 1 : p.group;
    const bool listed = EXT && n_long >= 0;
    const int n_units = (listed ? n_long : p.batch) * nsplits * p.nheads_k;
    const int units8 = listed ? (n_units + 7) / 8 * 8 : p.units8;
    int mb, unit, head_in_unit;
    if (p.num_mb > 2) {
        const int per_block = units8 * heads_per_unit;
        mb = p.num_mb - 1 - (int)(bid / per_block);
        const int e = bid % per_block;
        unit = ((e >> 3) / heads_per_unit) * 8 + (e & 7);
        head_in_unit = (e >> 3) % heads_per_unit;
    } else {
        // one or two blocks per unit (short sequences, all equally light): a unit's blocks stay
        // neighbours in their XCD's queue, so its K/V are fetched into that L2 once
        const int per_unit = p.num_mb * heads_per_unit;
        const int r = bid >> 3;
        unit = (r / per_unit) * 8 + (bid & 7);
        head_in_unit = (r % per_unit) / p.num_mb;
        mb = p.num_mb - 1 - r % p.num_mb;
    }
    if (unit >= n_units) return;
    const int z = unit / p.nheads_k;
    const int hk = unit - z * p.nheads_k;
    const int zb = z / nsplits;
    const int split = z - zb * nsplits;
    const int b = listed ? p.long_ids[zb] : zb;

    int q0, Sq, k0 = 0, Sk;
    if (p.cu_seqlens_q) {
        q0 = p.cu_seqlens_q[b];
        Sq = p.cu_seqlens_q[b + 1] - q0;
    } else {
        q0 = 0;
        Sq = p.seqlen_q_fixed;
    }
    if (EXT && Sq >= 1 && Sq <= p.skip_short) return;   // the decode kernels compute this sequence
    // tile row R is query R / pg of head h_base + R % pg.  pg is the launch's (every block packs the heads
    // of its group, or none does) unless the launch lets short blocks pack on their own: a block whose
    // (query, head) rows take at most three quarters of the tiles its heads would take one by one is
    // computed by the tiles of its first head alone, the tiles of the other heads leave
    int pg = EXT ? p.pack : 1;
    if (EXT && p.pack_short && pg == 1 && p.group > 1) {
        const int packed = (Sq * p.group + kBM - 1) / kBM;
        const int plain = p.group * ((Sq + kBM - 1) / kBM);
        if (packed * 4 <= plain * 3 && packed <= p.num_mb) {
            if (head_in_unit != 0) return;
            pg = p.group;
        }
    }
    const int h_base = hk * p.group + ((pg > 1) ? 0 : head_in_unit);
    if constexpr (PAGED) {
        Sk = p.seqused_k[b] + p.seqlen_k_add;
        Sk = min(Sk, p.max_blocks * p.page_size);
    } else {
        k0 = p.cu_seqlens_k[b];
        Sk = p.cu_seqlens_k[b + 1] - k0;
        if (p.seqused_k) Sk = max(0, min(Sk, p.seqused_k[b]));   // only the first seqused_k[b] keys of the sequence are used
    }
    // window normalisation: the varlen host passes max_seqlen_k as the reference does
    // (flash_api.cpp:938-943); the kvcache layout has the lengths on the device only, so the batch
    // maximum is reduced here when a window was requested
    int wl = p.window_left, wr_eff = p.window_right;
    int norm_m = p.window_norm_m;
    if constexpr (PAGED) {
        if (norm_m <= 0 && (wl >= 0 || wr_eff >= 0)) norm_m = block_max_keys(p.seqused_k, p.batch, p.seqlen_k_add);
    }
    if (norm_m <= 0) norm_m = max(Sk, 1);
    normalize_window(wl, wr_eff, p.causal, norm_m);
    int batch_max = 0;
    if constexpr (PAGED) {
        if (nsplits > 1) batch_max = min(block_max_keys(p.seqused_k, p.batch, p.seqlen_k_add), p.max_blocks * p.page_size);
    }
    const int n_rows = Sq * pg;
    const int R0 = mb * kBM;
    if (R0 >= n_rows) return;
    const int off = Sk - Sq;

    // split of the unit's visible keys: the same cut as the decode kernels' grid mode, so that the
    // same combine kernel merges the partials
    int range_lo = 0, range_hi = Sk;
    bool whole = true;
    int64_t slot = 0;
    if (nsplits > 1) {
        const int sk = adaptive_split_keys(batch_max, nsplits);
        const KeyRanges kr = key_ranges(Sq, Sk, wl, wr_eff, sk, nsplits);
        if (split >= kr.count) return;
        if (kr.hi > kr.lo) {
            range_lo = kr.begin(split, sk);
            range_hi = kr.end(split, sk);
        }
        whole = kr.count == 1;
        slot = ((int64_t)b * p.nheads_k + hk) * nsplits + split;
    }

    const int my_R = min(R0 + wave * 32 + ln, n_rows - 1);   // rows past the end repeat the last one and are dropped
    const bool row_ok = R0 + wave * 32 + ln < n_rows;
    const int my_row = my_R / pg;                            // query position of this lane column
    const int my_head = h_base + (my_R - my_row * pg);
    const uint16_t *q_row = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_stride_b +
                            (int64_t)my_head * p.q_stride_h + (int64_t)(q0 + my_row) * p.q_stride_t;
    uint16_t *o_row = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)my_head * p.o_stride_h +
                      (int64_t)(q0 + my_row) * p.o_stride_t;
    float *lse_row = p.lse + (int64_t)b * p.lse_stride_b + (int64_t)my_head * p.lse_stride_h + q0 + my_row;

    // key range the whole block (query positions r_lo .. r_hi) can see
    const int r_lo = R0 / pg;
    const int r_hi = (min(n_rows, R0 + kBM) - 1) / pg;
    int k_lo = 0, k_hi = Sk;
    if (wl >= 0) k_lo = max(0, r_lo + off - wl);
    if (wr_eff >= 0) k_hi = min(Sk, r_hi + off + wr_eff + 1);
    k_lo = max(k_lo, range_lo);
    k_hi = max(min(k_hi, range_hi), 0);
    // where this lane's row goes when the unit is cut: row (query, head of the group) of the slot
    float *part_row = nullptr, *part_lse = nullptr;
    if (!whole) {
        // kvcache layout: (batch row, kv head, range, query x head of the group); token-major q: (token, head, range)
        const int64_t prow = p.cu_seqlens_q ? ((int64_t)(q0 + my_row) * p.nheads + my_head) * nsplits + split
                                            : slot * p.rows + (int64_t)my_row * p.group + (my_head - hk * p.group);
        part_row = p.o_partial + prow * D;
        part_lse = p.lse_partial + prow;
    }

    if (k_hi <= k_lo) {
        // nothing visible for the whole block: out = 0, lse = +inf
        if (row_ok && whole) {
            for (int c = lh * (D / 2); c < min((lh + 1) * (D / 2), hd); c += 8) store16(o_row + c, u32x4_t{0, 0, 0, 0});
            if (lh == 0) *lse_row = INFINITY;
        } else if (row_ok) {
            for (int c = lh * (D / 2); c < (lh + 1) * (D / 2); c += 4) *reinterpret_cast<float4 *>(part_row + c) = make_float4(0.f, 0.f, 0.f, 0.f);
            if (lh == 0) *part_lse = -INFINITY;
        }
        return;
    }

    // per-lane visible interval of its row (inclusive bounds)
    int klo_r = 0, khi_r = Sk - 1;
    if (wl >= 0) klo_r = max(0, my_row + off - wl);
    if (wr_eff >= 0) khi_r = min(Sk - 1, my_row + off + wr_eff);
    klo_r = max(klo_r, range_lo);
    khi_r = min(khi_r, range_hi - 1);
    // bounds that decide, per wave, whether a tile needs element masks
    const int rw0 = min(R0 + wave * 32, n_rows - 1) / pg;        // first and last query position of the wave
    const int rw1 = (min(n_rows, R0 + wave * 32 + 32) - 1) / pg;
    const int wave_klo_max = max(range_lo, (wl >= 0) ? max(0, rw1 + off - wl) : 0);
    const int wave_khi_min = min(range_hi - 1, (wr_eff >= 0) ? min(Sk - 1, rw0 + off + wr_eff) : Sk - 1);

    // Q^T operand: lane (lh, ln) holds row ln, elements t*16 + lh*8 .. +7
    u32x4_t qreg[Cfg::kKSteps];
    {
        const uint16_t *src = q_row + lh * 8;
#pragma unroll
        for (int t = 0; t < Cfg::kKSteps; ++t) {
            if (PART && t * 16 + lh * 8 >= hd) {
                qreg[t] = u32x4_t{0, 0, 0, 0};
                continue;
            }
            qreg[t] = load16(src + t * 16);
            if (!row_ok) qreg[t] = u32x4_t{0, 0, 0, 0};
        }
    }

    // ---- K/V tile fetch ---------------------------------------------------------------------
    const uint16_t *kbase = reinterpret_cast<const uint16_t *>(p.k) + (int64_t)hk * p.k_stride_h;
    const uint16_t *vbase = reinterpret_cast<const uint16_t *>(p.v) + (int64_t)hk * p.v_stride_h;
    const int32_t *bt_row = PAGED ? p.block_table + (int64_t)b * p.bt_stride_b : nullptr;

    // Load i of this wave covers the LDS pieces 64 (wave + 4i) .. + 63 of the tile, piece = (row, place in the row);
    // a K row's place c' holds the row's piece c' ^ (row & kSwz), a V row is followed by its padding (nobody loads it).
    // Rows past the last key re-read the last key (never memory nobody wrote; they are masked); with PART the pieces
    // behind the head dimension are not loaded: their places hold the zeros written when the block started.
    int k_row[Cfg::kKLoads], v_row[Cfg::kVLoads];
    uint32_t k_col[Cfg::kKLoads], v_col[Cfg::kVLoads];          // byte offset of the lane's piece inside its row
    bool k_on[Cfg::kKLoads], v_on[Cfg::kVLoads];
#pragma unroll
    for (int i = 0; i < Cfg::kKLoads; ++i) {
        const int piece = 64 * (wave + 4 * i) + lane;
        k_row[i] = piece / Cfg::kChunks;
        const int c = (piece % Cfg::kChunks) ^ (k_row[i] & Cfg::kSwz);
        k_col[i] = c * 16;
        k_on[i] = !PART || c * 8 < hd;
    }
#pragma unroll
    for (int i = 0; i < Cfg::kVLoads; ++i) {
        const int piece = 64 * (wave + 4 * i) + lane;
        v_row[i] = piece / Cfg::kVRowPieces;
        const int c = piece % Cfg::kVRowPieces;
        v_col[i] = c * 16;
        v_on[i] = c < Cfg::kChunks && (!PART || c * 8 < hd);
    }
    // per-lane offsets of an interior tile of dense K/V (one wave-uniform base per tile serves all its loads)
    uint32_t k_off[Cfg::kKLoads], v_off[Cfg::kVLoads];
#pragma unroll
    for (int i = 0; i < Cfg::kKLoads; ++i) k_off[i] = (uint32_t)k_row[i] * (uint32_t)p.k_stride_t * 2u + k_col[i];
#pragma unroll
    for (int i = 0; i < Cfg::kVLoads; ++i) v_off[i] = (uint32_t)v_row[i] * (uint32_t)p.v_stride_t * 2u + v_col[i];
    auto lds_of = [](const void *ptr) -> uint32_t { return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)ptr; };
    // The loads are written out: the compiler would wait for such a load in front of every LDS read that follows (it
    // cannot tell the two buffers apart).  tiles_landed() is the wait that orders them.
    auto load_lds_base = [&](uint32_t lds, uint32_t off, const uint8_t *base) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(off), "s"(base) : "memory", "m0");
    };
    auto load_lds_addr = [&](uint32_t lds, const void *addr) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds), "v"(addr) : "memory", "m0");
    };
    auto tiles_landed = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
    auto fetch_tile = [&](int kt, int buf) {
        const uint32_t k_lds = lds_of(&s_k[buf][0]) + (uint32_t)wave * 1024u, v_lds = lds_of(&s_v[buf][0]) + (uint32_t)wave * 1024u;
        // A tile inside the sequence, of dense K/V or inside one page: one wave-uniform base serves all its loads
        if (kt * kBN + kBN <= Sk && (!PAGED || p.page_size % kBN == 0)) {
            int64_t koff, voff;
            if constexpr (PAGED) {
                const int page = (kt * kBN) / p.page_size;
                const int blk = min(max(__builtin_amdgcn_readfirstlane(bt_row[page]), 0), p.num_blocks - 1);
                const int inpage = kt * kBN - page * p.page_size;
                koff = (int64_t)blk * p.k_stride_block + (int64_t)inpage * p.k_stride_t;
                voff = (int64_t)blk * p.v_stride_block + (int64_t)inpage * p.v_stride_t;
            } else {
                koff = (int64_t)(k0 + kt * kBN) * p.k_stride_t;
                voff = (int64_t)(k0 + kt * kBN) * p.v_stride_t;
            }
            const uint8_t *kb = reinterpret_cast<const uint8_t *>(kbase + koff);
            const uint8_t *vb = reinterpret_cast<const uint8_t *>(vbase + voff);
#pragma unroll
            for (int i = 0; i < Cfg::kKLoads; ++i)
                if (k_on[i]) load_lds_base(k_lds + i * 4096u, k_off[i], kb);
#pragma unroll
            for (int i = 0; i < Cfg::kVLoads; ++i)
                if (v_on[i]) load_lds_base(v_lds + i * 4096u, v_off[i], vb);
            return;
        }
        // The ragged end of a sequence, or pages that a tile straddles: an address per row.  All addresses first (their
        // page-table entries are then fetched together), the loads behind them.
        auto row_addr = [&](int row, bool is_k) -> const uint8_t * {
            const int key = min(kt * kBN + row, Sk - 1);
            int64_t off;
            if constexpr (PAGED) {
                const int page = key / p.page_size;
                int blk = bt_row[page];
                blk = min(max(blk, 0), p.num_blocks - 1);
                const int inpage = key - page * p.page_size;
                off = is_k ? (int64_t)blk * p.k_stride_block + (int64_t)inpage * p.k_stride_t
                           : (int64_t)blk * p.v_stride_block + (int64_t)inpage * p.v_stride_t;
            } else {
                off = (int64_t)(k0 + key) * (is_k ? p.k_stride_t : p.v_stride_t);
            }
            return reinterpret_cast<const uint8_t *>((is_k ? kbase : vbase) + off);
        };
        const uint8_t *ka[Cfg::kKLoads], *va[Cfg::kVLoads];
#pragma unroll
        for (int i = 0; i < Cfg::kKLoads; ++i) ka[i] = row_addr(k_row[i], true) + k_col[i];
#pragma unroll
        for (int i = 0; i < Cfg::kVLoads; ++i) va[i] = row_addr(v_row[i], false) + v_col[i];
#pragma unroll
        for (int i = 0; i < Cfg::kKLoads; ++i)
            if (k_on[i]) load_lds_addr(k_lds + i * 4096u, ka[i]);
#pragma unroll
        for (int i = 0; i < Cfg::kVLoads; ++i)
            if (v_on[i]) load_lds_addr(v_lds + i * 4096u, va[i]);
    };
    if constexpr (PART) {
        // the places of the pieces that nobody loads
        for (int i = tid * 16; i < 2 * Cfg::kTileBytes; i += 256 * 16) *reinterpret_cast<u32x4_t *>(&s_k[0][0] + i) = u32x4_t{0, 0, 0, 0};
        for (int i = tid * 16; i < 2 * Cfg::kVTileBytes; i += 256 * 16) *reinterpret_cast<u32x4_t *>(&s_v[0][0] + i) = u32x4_t{0, 0, 0, 0};
        __syncthreads();
    }

    float m_run = -INFINITY, l_run = 0.f;
    float16_t o_acc[Cfg::kMT];
#pragma unroll
    for (int t = 0; t < Cfg::kMT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[t][r] = 0.f;

    const int kt_begin = k_lo / kBN;
    const int kt_end = (k_hi + kBN - 1) / kBN;
    const bool wave_live = __builtin_amdgcn_readfirstlane(R0 + wave * 32 < n_rows);
    fetch_tile(kt_begin, 0);
    tiles_landed();
    __syncthreads();

    int cur = 0;
    for (int kt = kt_begin; kt < kt_end; ++kt) {
        const bool more = kt + 1 < kt_end;
        if (more) fetch_tile(kt + 1, cur ^ 1);   // the other buffer: its readers passed the barrier that ended the last step
        __builtin_amdgcn_sched_barrier(0);

        // a wave whose 32 rows all lie past the block's end (short blocks: a decode row among prompt chunks
        // fills four rows of one wave) only helps to move the tiles, and leaves the matrix pipe to the others
        if (wave_live) {
        // ---- S^T = K Q^T for the two 32-key halves of the tile
        // the wave in a matrix phase goes first: its MFMAs then issue back to back and the vector work of the SIMD's other
        // wave fills the gaps between them (c5: 870 -> 856 us)
        __builtin_amdgcn_s_setprio(1);
        float16_t s[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[tt][r] = 0.f;
        // operand reads run kPf k-steps ahead of the MFMAs that use them
        constexpr int kPf = 2;
        u32x4_t ka[Cfg::kKSteps][2];
        auto read_k = [&](int t) {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const int row = tt * 32 + ln;
                ka[t][tt] = *reinterpret_cast<const u32x4_t *>(
                    &s_k[cur][row * (D * 2) + (((t * 2 + lh) ^ (row & Cfg::kSwz)) << 4)]);
            }
        };
#pragma unroll
        for (int t = 0; t < kPf; ++t) read_k(t);
#pragma unroll
        for (int t = 0; t < Cfg::kKSteps; ++t) {
            if (PART && t * 16 >= hd) break;   // wave-uniform; at least D/2 columns are live
            if (t + kPf < Cfg::kKSteps) read_k(t + kPf);
            s[0] = mfma32<T>(ka[t][0], qreg[t], s[0]);
            s[1] = mfma32<T>(ka[t][1], qreg[t], s[1]);
            __builtin_amdgcn_sched_barrier(0);
        }

        __builtin_amdgcn_s_setprio(0);
        // ---- online softmax; lane column = query row, register r of half tt = key
        //      kt*64 + tt*32 + 8*(r/4) + 4*lh + r%4
        const int tile0 = kt * kBN;
        // wave-uniform by construction; made scalar so the two softmax paths stay separate branches
        const bool need_mask = __builtin_amdgcn_readfirstlane((tile0 < wave_klo_max) || (tile0 + kBN - 1 > wave_khi_min));
        // Fast path (no softcap, no element masks, positive scale): the maximum is taken on the raw
        // scores and the scale rides in the exponent's fused multiply-add.
        const bool raw_path = !SOFTCAP && !need_mask && p.scale_log2 > 0.f;
        float mloc = -INFINITY;
        if (raw_path) {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, s[tt][r]);
            mloc *= p.scale_log2;
        } else if (!SOFTCAP && need_mask) {
            // masked tile (the diagonal of a causal block, window edges, the ragged end): element r
            // of half tt is key tile0 + 4*lh + e(tt, r) with e a compile-time constant, so the
            // row's bounds are compared in tile coordinates; a side that cannot bite is skipped
            const int lo_rel = klo_r - tile0 - 4 * lh;
            const int hi_rel = khi_r - tile0 - 4 * lh;
            const bool need_lo = __builtin_amdgcn_readfirstlane(tile0 < wave_klo_max);
            if (!need_lo) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int e = tt * 32 + 8 * (r >> 2) + (r & 3);
                        const float v = (e <= hi_rel) ? s[tt][r] * p.scale_log2 : -INFINITY;
                        s[tt][r] = v;
                        mloc = fmaxf(mloc, v);
                    }
            } else {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int e = tt * 32 + 8 * (r >> 2) + (r & 3);
                        const float v = (e >= lo_rel && e <= hi_rel) ? s[tt][r] * p.scale_log2 : -INFINITY;
                        s[tt][r] = v;
                        mloc = fmaxf(mloc, v);
                    }
            }
        } else {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float v = s[tt][r];
                    if constexpr (SOFTCAP) {
                        const float y = v * p.softcap_pre;
                        const float e2 = __expf(2.f * y);
                        v = p.softcap_post * (1.f - 2.f / (e2 + 1.f));
                    } else {
                        v *= p.scale_log2;
                    }
                    const int e = tt * 32 + 8 * (r >> 2) + (r & 3);
                    v = (!need_mask || (e >= klo_r - tile0 - 4 * lh && e <= khi_r - tile0 - 4 * lh)) ? v : -INFINITY;
                    s[tt][r] = v;
                    mloc = fmaxf(mloc, v);
                }
        }
        mloc = halves_max(mloc);
        // The accumulator rescale is skipped for the whole wave when no row of it saw a new maximum
        // (most tiles once a row is a few hundred keys in).  m_run stays the exact running maximum,
        // so the largest P of a row is exactly 1 as in the reference's golden.
        const bool bump = mloc > m_run;   // false for fully hidden tiles
        if (__any(bump)) {
            const float m_new = bump ? mloc : m_run;
            const float m_new_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = bump ? fast_exp2(m_run - m_new_use) : 1.f;
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < Cfg::kMT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[t][r] *= alpha;
        }
        const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
        float psum = 0.f;
        u32x4_t pk[2][2];
        if (raw_path) {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int r = 0; r < 16; ++r) s[tt][r] = fast_exp2(__builtin_fmaf(s[tt][r], p.scale_log2, -m_use));
        } else {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int r = 0; r < 16; ++r) s[tt][r] = fast_exp2(s[tt][r] - m_use);
        }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) psum += s[tt][r];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int u = 0; u < 4; ++u) pk[tt][ks][u] = pack2<T>(s[tt][8 * ks + 2 * u], s[tt][8 * ks + 2 * u + 1]);
        }
        l_run += psum;

        __builtin_amdgcn_s_setprio(1);
        // ---- O^T += V^T P^T, 16 keys per step.  The V^T operand comes from the transposing LDS read
        //      (ds_read_b64_tr_b16): in every 16-lane group, lane s points at 4 columns of key row
        //      s/4 and receives column s (of the group's 16) for the group's 4 key rows.  Column tile
        //      t is V columns t*32 .. t*32+31 in lane order.
        typedef short v4s_t __attribute__((ext_vector_type(4)));
        const int tr_row = 4 * lh + ((lane & 15) >> 2);
        const int tr_col = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                u32x4_t va[Cfg::kMT];
#pragma unroll
                for (int t = 0; t < Cfg::kMT; ++t)
#pragma unroll
                    for (int hv = 0; hv < 2; ++hv) {
                        if (PART && t * 32 >= hd) continue;
                        const int row = tt * 32 + 16 * ks + 8 * hv + tr_row;
                        const v4s_t r4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) v4s_t *)(&s_v[cur][row * Cfg::kVRowBytes + (t * 32 + tr_col) * 2]));
                        const uint2 r2 = __builtin_bit_cast(uint2, r4);
                        va[t][2 * hv] = r2.x;
                        va[t][2 * hv + 1] = r2.y;
                    }
#pragma unroll
                for (int t = 0; t < Cfg::kMT; ++t) {
                    if (PART && t * 32 >= hd) continue;
                    o_acc[t] = mfma32<T>(va[t], pk[tt][ks], o_acc[t]);
                }
            }
        __builtin_amdgcn_s_setprio(0);
        }   // wave_live

        tiles_landed();
        __syncthreads();
        cur ^= 1;
    }

    // ---- epilogue: O^T / l, store.  Register r of column tile t is V column
    //      t*32 + 8*(r/4) + 4*lh + r%4 of query row ln: four consecutive columns per (t, r/4).
    l_run = halves_sum(l_run);
    const float inv = (l_run > 0.f) ? 1.f / l_run : 0.f;
    if (!whole) {
        // one of several ranges of the unit: normalised fp32 partial and base-2 LSE for the combine
        if (row_ok) {
#pragma unroll
            for (int t = 0; t < Cfg::kMT; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    *reinterpret_cast<float4 *>(part_row + t * 32 + 8 * j + 4 * lh) =
                        make_float4(o_acc[t][4 * j] * inv, o_acc[t][4 * j + 1] * inv, o_acc[t][4 * j + 2] * inv,
                                    o_acc[t][4 * j + 3] * inv);
            if (lh == 0) *part_lse = (l_run > 0.f) ? m_run + fast_log2(l_run) : -INFINITY;
        }
        return;
    }
    if (row_ok && lh == 0) *lse_row = (l_run > 0.f) ? (m_run + fast_log2(l_run)) * kLn2 : INFINITY;
    // The lane owns 8-byte pieces of its row, 16 of them: stored as they are, one instruction would touch
    // 32 rows of the output.  The wave's 32 x D tile goes through LDS instead (the V tiles are free
    // after the last barrier of the loop; each wave uses its own part, so no workgroup barrier) and
    // leaves as whole rows, 16 bytes per lane.
    constexpr int kStageRow = D * 2 + 16;                      // padded: the 8-byte writes of a column spread over the banks
    static_assert(4 * 32 * kStageRow <= 2 * Cfg::kVTileBytes, "staging tile must fit the V tiles");
    uint8_t *stage = &s_v[0][0] + wave * (32 * kStageRow);
#pragma unroll
    for (int t = 0; t < Cfg::kMT; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint2 o2;
            o2.x = pack2<T>(o_acc[t][4 * j] * inv, o_acc[t][4 * j + 1] * inv);
            o2.y = pack2<T>(o_acc[t][4 * j + 2] * inv, o_acc[t][4 * j + 3] * inv);
            *reinterpret_cast<uint2 *>(stage + ln * kStageRow + (t * 32 + 8 * j + 4 * lh) * 2) = o2;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    constexpr int kLanesPerRow = D * 2 / 16;                   // lanes that cover one row with 16 bytes each
    constexpr int kStageRows = 64 / kLanesPerRow;              // rows a wave stores per instruction
    const int piece = lane % kLanesPerRow;
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += kStageRows) {
        const int rr = r0 + lane / kLanesPerRow;               // row of the wave's tile
        const int R = R0 + wave * 32 + rr;
        if (R < n_rows && (!PART || piece * 8 < hd)) {
            const int row = R / pg;
            const int head = h_base + (R - row * pg);
            uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)head * p.o_stride_h +
                            (int64_t)(q0 + row) * p.o_stride_t;
            store16(dst + piece * 8, *reinterpret_cast<const u32x4_t *>(stage + rr * kStageRow + piece * 16));
        }
    }
}

template <typename T, int D, bool PAGED, bool SOFTCAP, bool EXT, bool PART>
__global__ void __launch_bounds__(256, (D <= 128) ? 2 : 1) prefill_kernel(const PrefillParams p) {
    using Cfg = PrefillCfg<D>;
    __shared__ __attribute__((aligned(16))) uint8_t s_k[2][Cfg::kTileBytes];
    __shared__ __attribute__((aligned(16))) uint8_t s_v[2][Cfg::kVTileBytes];
    prefill_block<T, D, PAGED, SOFTCAP, EXT, PART>(p, blockIdx.x, -1, s_k, s_v);
}

// The same blocks for a launch whose live sequences are known on the device only (token-major batches whose
// short blocks went to the decode kernels: p.long_ids, p.list_state[0] of them).  A grid sized for every batch
// row would be mostly workgroups that find nothing to do, and dispatching those costs as much time as the live
// ones' work once the batch has many decode rows.  Here as many workgroups as the device holds take blocks from
// the ordered list until it ends: workgroup w (on XCD w % 8) takes the blocks congruent to w % 8, so that the heads
// of a unit still meet in one L2, through one counter per XCD (p.list_state[1 + x], zeroed by the kernel that
// wrote the list).  Every workgroup leaves when its counter passes the end of the list.
template <typename T, int D, bool SOFTCAP, bool PART>
__global__ void __launch_bounds__(256, (D <= 128) ? 2 : 1) prefill_list_kernel(const PrefillParams p) {
    using Cfg = PrefillCfg<D>;
    __shared__ __attribute__((aligned(16))) uint8_t s_k[2][Cfg::kTileBytes];
    __shared__ __attribute__((aligned(16))) uint8_t s_v[2][Cfg::kVTileBytes];
    __shared__ int s_item;
    const int n_long = p.list_state[0];
    const int heads_per_unit = (p.pack > 1) ? 1 : p.group;
    const int64_t units8 = ((int64_t)n_long * max(p.nsplits, 1) * p.nheads_k + 7) / 8 * 8;
    const int64_t total = (int64_t)p.num_mb * units8 * heads_per_unit;     // a multiple of 8
    const int x = blockIdx.x & 7;
    for (;;) {
        __syncthreads();   // the last block's LDS tiles and s_item are free
        if (threadIdx.x == 0) s_item = atomicAdd(&p.list_state[1 + x], 1);
        __syncthreads();
        const int64_t bid = (int64_t)s_item * 8 + x;
        if (bid >= total) break;
        prefill_block<T, D, true, SOFTCAP, true, PART>(p, (unsigned)bid, n_long, s_k, s_v);
    }
}

// Merge of the key ranges of token-major query blocks over a paged cache: one wave per (token, head).
// Partials are laid out (token, head, range): normalised fp32 rows and base-2 log-sum-exps, -inf for a
// range in which the row saw nothing.  out = sum_r e^{lse_r - LSE} O_r, LSE = log sum_r e^{lse_r}.
// grid: total_q * ceil(nheads / 4) workgroups of 256 threads: the four waves take four heads of one token,
// so what depends on the token alone (its sequence, the cut of that sequence's keys) is found once per
// workgroup and every early exit is taken by the whole workgroup.
template <typename T, int D>
__global__ void __launch_bounds__(256) prefill_combine_kernel(const PrefillParams p) {
    const int head_groups = (p.nheads + 3) >> 2;
    const int tok = blockIdx.x / head_groups;
    const int head = (blockIdx.x - tok * head_groups) * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    // the sequence of this token: last b with cu_seqlens_q[b] <= tok (empty sequences repeat an offset), counted by
    // the lanes side by side: one trip to memory where a bisection makes log2(batch) dependent ones
    int below = 0;
    for (int i = lane; i < p.batch; i += 64) below += (p.cu_seqlens_q[i] <= tok) ? 1 : 0;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) below += __shfl_xor(below, d, 64);
    const int b = max(below - 1, 0);
    const int Sq = p.cu_seqlens_q[b + 1] - p.cu_seqlens_q[b];
    const int Sk = min(p.seqused_k[b] + p.seqlen_k_add, p.max_blocks * p.page_size);
    if (Sq >= 1 && Sq <= p.skip_short) return;   // computed by the decode kernels (the whole workgroup: one token)
    const int longest = block_max_keys(p.seqused_k, p.batch, p.seqlen_k_add);
    int wl = p.window_left, wr = p.window_right;
    int norm_m = p.window_norm_m;
    if (norm_m <= 0 && (wl >= 0 || wr >= 0)) norm_m = longest;
    if (norm_m <= 0) norm_m = max(Sk, 1);
    normalize_window(wl, wr, p.causal, norm_m);
    const int sk = adaptive_split_keys(min(longest, p.max_blocks * p.page_size), p.nsplits);
    const KeyRanges kr = key_ranges(Sq, Sk, wl, wr, sk, p.nsplits);
    if (kr.count == 1) return;   // the tile that computed this row wrote it
    if (head >= p.nheads) return;
    const int64_t base = ((int64_t)tok * p.nheads + head) * p.nsplits;

    float mx = -INFINITY;
    for (int r = lane; r < kr.count; r += 64) mx = fmaxf(mx, p.lse_partial[base + r]);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
    const float mx_use = (mx == -INFINITY) ? 0.f : mx;
    constexpr int C = D / 64;        // columns per lane
    float acc[C];
#pragma unroll
    for (int c = 0; c < C; ++c) acc[c] = 0.f;
    float tot = 0.f;
    for (int r = 0; r < kr.count; ++r) {
        const float w = fast_exp2(p.lse_partial[base + r] - mx_use);
        tot += w;
        const float *o = p.o_partial + (base + r) * D + lane * C;
#pragma unroll
        for (int c = 0; c < C; ++c) acc[c] += w * o[c];
    }
    const float inv = (tot > 0.f) ? 1.f / tot : 0.f;
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)tok * p.o_stride_t + (int64_t)head * p.o_stride_h + lane * C;
    if (lane * C < p.headdim) {   // the partials are D wide; the output row ends at the head dimension
#pragma unroll
        for (int c = 0; c < C; ++c) dst[c] = from_float<T>(acc[c] * inv);
    }
    if (lane == 0) p.lse[(int64_t)head * p.lse_stride_h + tok] = (tot > 0.f) ? (mx + fast_log2(tot)) * kLn2 : INFINITY;
}

static_assert(kBM == kPrefillTileRows, "the planning rules in fa_kernels.h assume this tile height");

template <typename T, int D> static hipError_t launch_prefill_d(const PrefillParams &p_in, hipStream_t stream) {
    PrefillParams p = p_in;
    p.pack = prefill_pack(p.group, p.max_seqlen_q);
    p.num_mb = (p.max_seqlen_q * p.pack + kBM - 1) / kBM;
    if (p.nsplits > 1 && (!p.block_table || !p.o_partial || !p.lse_partial)) return hipErrorInvalidValue;
    const int64_t units = (int64_t)p.batch * max(p.nsplits, 1) * p.nheads_k;
    p.units8 = (int32_t)((units + 7) / 8 * 8);
    const int64_t wgs = (int64_t)p.num_mb * p.units8 * (p.pack > 1 ? 1 : p.group);
    if (wgs <= 0 || wgs >= (1ll << 31)) return hipErrorInvalidValue;
    dim3 grid((unsigned)wgs);
    dim3 block(256);
    const bool softcap = p.softcap_post != 0.f;
    const bool paged = p.block_table != nullptr;
    p.pack_short = p.cu_seqlens_q ? prefill_pack_short(p.group, p.max_seqlen_q, p.total_q, p.batch) : 0;
    if (p.headdim > D || p.headdim < 8 || p.headdim % 8 != 0) return hipErrorInvalidValue;
    const bool part = p.headdim < D;
    // a head dimension below the compiled width always takes the kernels with every extension compiled in
    const bool ext = part || p.pack > 1 || p.nsplits > 1 || p.pack_short || p.skip_short > 0;
    if (p.long_ids) {
        // live sequences listed on the device: workgroups that stay and take blocks from the list
        if (!paged || !p.list_state || p.list_wgs <= 0 || !p.cu_seqlens_q) return hipErrorInvalidValue;
        dim3 lgrid((unsigned)std::min<int64_t>(p.list_wgs, wgs));
        if (softcap) {
            if (part)
                hipLaunchKernelGGL((prefill_list_kernel<T, D, true, true>), lgrid, block, 0, stream, p);
            else
                hipLaunchKernelGGL((prefill_list_kernel<T, D, true, false>), lgrid, block, 0, stream, p);
        } else {
            if (part)
                hipLaunchKernelGGL((prefill_list_kernel<T, D, false, true>), lgrid, block, 0, stream, p);
            else
                hipLaunchKernelGGL((prefill_list_kernel<T, D, false, false>), lgrid, block, 0, stream, p);
        }
        return hipGetLastError();
    }
    auto launch = [&](auto paged_c, auto softcap_c, auto ext_c) {
        constexpr bool kExt = decltype(ext_c)::value;
        if constexpr (kExt) {
            if (part) {
                hipLaunchKernelGGL((prefill_kernel<T, D, decltype(paged_c)::value, decltype(softcap_c)::value, true, true>), grid, block,
                                   0, stream, p);
                return;
            }
        }
        hipLaunchKernelGGL((prefill_kernel<T, D, decltype(paged_c)::value, decltype(softcap_c)::value, kExt, false>), grid, block, 0,
                           stream, p);
    };
    auto pick_ext = [&](auto paged_c, auto softcap_c) {
        if (ext) launch(paged_c, softcap_c, std::true_type{}); else launch(paged_c, softcap_c, std::false_type{});
    };
    auto pick_softcap = [&](auto paged_c) {
        if (softcap) pick_ext(paged_c, std::true_type{}); else pick_ext(paged_c, std::false_type{});
    };
    if (paged) pick_softcap(std::true_type{}); else pick_softcap(std::false_type{});
    return hipGetLastError();
}

template <typename T> static hipError_t launch_prefill_t(const PrefillParams &p, int headdim, hipStream_t stream) {
    switch (headdim) {
        case 64: return launch_prefill_d<T, 64>(p, stream);
        case 128: return launch_prefill_d<T, 128>(p, stream);
        case 256: return launch_prefill_d<T, 256>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

template <typename T> static hipError_t launch_prefill_combine_t(const PrefillParams &p, int headdim, hipStream_t stream) {
    const int64_t wgs = (int64_t)p.total_q * ((p.nheads + 3) / 4);
    if (wgs <= 0 || wgs >= (1ll << 31)) return hipErrorInvalidValue;
    dim3 grid((unsigned)wgs), block(256);
    switch (headdim) {
        case 64: hipLaunchKernelGGL((prefill_combine_kernel<T, 64>), grid, block, 0, stream, p); break;
        case 128: hipLaunchKernelGGL((prefill_combine_kernel<T, 128>), grid, block, 0, stream, p); break;
        case 256: hipLaunchKernelGGL((prefill_combine_kernel<T, 256>), grid, block, 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_prefill_combine(const PrefillParams &p, int dtype, int headdim, hipStream_t stream) {
    if (p.nsplits <= 1 || p.total_q <= 0) return hipSuccess;
    if (!p.cu_seqlens_q || !p.block_table || !p.o_partial || !p.lse_partial) return hipErrorInvalidValue;
    return dtype == 0 ? launch_prefill_combine_t<BF16>(p, headdim, stream) : launch_prefill_combine_t<FP16>(p, headdim, stream);
}

hipError_t launch_prefill(const PrefillParams &p, int dtype, int headdim, hipStream_t stream) {
    if (p.max_seqlen_q <= 0 || p.batch <= 0) return hipSuccess;
    return dtype == 0 ? launch_prefill_t<BF16>(p, headdim, stream) : launch_prefill_t<FP16>(p, headdim, stream);
}

}  // namespace fa
