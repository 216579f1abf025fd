// Paged GQA/MQA decode for gfx950 with the wavefront as the unit of work: every wave owns a
// contiguous share of the balanced chunk list, streams it with its own running (max, sum, O) and
// writes its own final rows or partials.  After the one block-level prefix scan at kernel start
// there is no workgroup barrier: a wave that crosses from one (batch row, kv head) unit into the
// next only restarts its own pipeline while the other waves of the compute unit keep streaming.
//
// Same arithmetic as decode_paged.hip (the reference's hot loop, csrc/ascend910/flash_attn_npu/
// mha_fwd_kvcache.cpp:632-969): S^T = K Q^T and O^T = V^T P^T on the 16x16x32 MFMA with the query
// row in lane column lane%16; K rows through a wave-private swizzled LDS tile, which they reach
// straight from global memory (global_load_lds_dwordx4: no register holds them and no LDS store
// instruction moves them; two tiles per wave, the chunk being read and the chunk on its way); V rows
// loaded in operand order and transposed with v_perm; P rounded to the I/O dtype before PV.  Used
// when the query block (seqlen_q * group rows) fits one 16-row tile, or two where a wave's registers
// hold two sets of accumulators.
#include "decode_common.h"

namespace fa {

template <int D> struct WaveCfg {
    static constexpr int kLanesPerRow = D / 8;
    static constexpr int kRowsPerLoad = 64 / kLanesPerRow;
    static constexpr int kKLoads = kChunk / kRowsPerLoad;
    static constexpr int kKSteps = D / 32;
    static constexpr int kVW = (D >= 128) ? 8 : D / 16;
    static constexpr int kVH = D / (16 * kVW);
    static constexpr int kColTiles = D / 16;
    static constexpr int kSwzMask = (kLanesPerRow >= 16) ? 15 : kLanesPerRow - 1;
    static constexpr int kTileBytes = kChunk * D * 2;
    static constexpr int kPiecesPerRow = D / 8;   // 16-byte pieces of a query row
};

// Stage the 16-row query tile of unit (b, kvh), rotated if requested, into this wave's LDS rows.
// Work item = one 16-byte piece of one row; in the non-interleaved rotary region the item of a
// first-half piece also produces its partner piece rot/2 elements further on.
template <typename T, int D, bool PART>
__device__ __forceinline__ void stage_q_wave(const DecodeParams &p, int b, int kvh, int row0, int n_rows, int len_cache, uint16_t *sq) {
    using Cfg = WaveCfg<D>;
    const int lane = threadIdx.x & 63;
    const uint16_t *qbase = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_stride_b;
    const uint16_t *cosT = reinterpret_cast<const uint16_t *>(p.rotary_cos);
    const uint16_t *sinT = reinterpret_cast<const uint16_t *>(p.rotary_sin);
    const int rot = (cosT != nullptr) ? p.rotary_dim : 0;
    const int half = rot >> 1;
    for (int item = lane; item < 16 * Cfg::kPiecesPerRow; item += 64) {
        const int trow = item / Cfg::kPiecesPerRow;          // row of the tile; row0 + trow of the query block
        const int ci = item - trow * Cfg::kPiecesPerRow;
        const int d0 = ci * 8;
        uint16_t *dst = sq + trow * D + d0;
        const int row = row0 + trow;
        if (row >= n_rows || (PART && d0 >= p.headdim)) {   // padding rows, and the columns behind a head dimension below D
            *reinterpret_cast<u32x4_t *>(dst) = u32x4_t{0, 0, 0, 0};
            continue;
        }
        const int qi = row / p.group;
        const int g = row - qi * p.group;
        const uint16_t *src = qbase + (int64_t)qi * p.q_stride_s + (int64_t)(kvh * p.group + g) * p.q_stride_h;
        if (d0 >= rot) {
            *reinterpret_cast<u32x4_t *>(dst) = load16(src + d0);
            continue;
        }
        int pos = len_cache + (p.rotary_per_token ? qi : 0);
        pos = min(max(pos, 0), p.seqlen_ro - 1);
        const uint16_t *cs = cosT + (int64_t)pos * half;
        const uint16_t *sn = sinT + (int64_t)pos * half;
        if (p.rotary_interleaved) {
            // pairs (2c, 2c+1) live inside the piece: pair index d0/2 + j
            alignas(16) uint16_t x[8];
            alignas(16) uint16_t o[8];
            *reinterpret_cast<u32x4_t *>(x) = load16(src + d0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float c = to_float<T>(cs[d0 / 2 + j]), s = to_float<T>(sn[d0 / 2 + j]);
                const float x1 = to_float<T>(x[2 * j]), x2 = to_float<T>(x[2 * j + 1]);
                float r1, r2;
                rotate_pair(x1, x2, c, s, r1, r2);
                o[2 * j] = from_float<T>(r1);
                o[2 * j + 1] = from_float<T>(r2);
            }
            *reinterpret_cast<u32x4_t *>(dst) = *reinterpret_cast<const u32x4_t *>(o);
        } else if (d0 < half) {
            // pairs (c, c + rot/2): this piece and its partner
            alignas(16) uint16_t x1v[8];
            alignas(16) uint16_t x2v[8];
            alignas(16) uint16_t o1[8];
            alignas(16) uint16_t o2[8];
            *reinterpret_cast<u32x4_t *>(x1v) = load16(src + d0);
            *reinterpret_cast<u32x4_t *>(x2v) = load16(src + d0 + half);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float c = to_float<T>(cs[d0 + j]), s = to_float<T>(sn[d0 + j]);
                const float x1 = to_float<T>(x1v[j]), x2 = to_float<T>(x2v[j]);
                float r1, r2;
                rotate_pair(x1, x2, c, s, r1, r2);
                o1[j] = from_float<T>(r1);
                o2[j] = from_float<T>(r2);
            }
            *reinterpret_cast<u32x4_t *>(dst) = *reinterpret_cast<const u32x4_t *>(o1);
            *reinterpret_cast<u32x4_t *>(dst + half) = *reinterpret_cast<const u32x4_t *>(o2);
        }
        // second-half pieces of the non-interleaved region are written by their partner's item
    }
}

// In-place append of the new rows whose positions fall into [range_lo, range_hi), by the wave that
// is about to stream that range: same arithmetic as append_kv_kernel (separately rounded fp32
// products and sum, round-to-nearest-even), so the written bytes are identical.
template <typename T, int D>
__device__ __forceinline__ void append_rows_wave(const DecodeParams &p, int b, int kvh, int len_cache, int range_lo,
                                                 int range_hi) {
    const int lane = threadIdx.x & 63;
    const uint16_t *cosT = reinterpret_cast<const uint16_t *>(p.rotary_cos);
    const uint16_t *sinT = reinterpret_cast<const uint16_t *>(p.rotary_sin);
    const int rot = (cosT != nullptr) ? p.rotary_dim : 0;
    const int half = rot >> 1;
    for (int t = max(0, range_lo - len_cache); t < min(p.seqlen_new, range_hi - len_cache); ++t) {
        const int pos = len_cache + t;
        const int page = pos / p.page_size;
        if (page >= p.max_blocks) continue;
        const int blk = p.block_table[(int64_t)b * p.bt_stride_b + page];
        if (blk < 0 || blk >= p.num_blocks) continue;
        const int inpage = pos - page * p.page_size;
        uint16_t *kdst = const_cast<uint16_t *>(reinterpret_cast<const uint16_t *>(p.k_cache)) + (int64_t)blk * p.k_stride_block +
                         (int64_t)inpage * p.k_stride_row + (int64_t)kvh * p.k_stride_h;
        uint16_t *vdst = const_cast<uint16_t *>(reinterpret_cast<const uint16_t *>(p.v_cache)) + (int64_t)blk * p.v_stride_block +
                         (int64_t)inpage * p.v_stride_row + (int64_t)kvh * p.v_stride_h;
        const uint16_t *ksrc = reinterpret_cast<const uint16_t *>(p.k_new) + (int64_t)b * p.kn_stride_b +
                               (int64_t)t * p.kn_stride_s + (int64_t)kvh * p.kn_stride_h;
        const uint16_t *vsrc = reinterpret_cast<const uint16_t *>(p.v_new) + (int64_t)b * p.vn_stride_b +
                               (int64_t)t * p.vn_stride_s + (int64_t)kvh * p.vn_stride_h;
        const int rpos = min(pos, p.seqlen_ro - 1);
        for (int c = lane; c < p.headdim / 2; c += 64) {
            int d1, d2;
            if (c < half) {
                d1 = p.rotary_interleaved ? 2 * c : c;
                d2 = p.rotary_interleaved ? 2 * c + 1 : c + half;
            } else {
                d1 = rot + 2 * (c - half);
                d2 = d1 + 1;
            }
            uint16_t o1 = ksrc[d1], o2 = ksrc[d2];
            if (c < half) {
                const float cs = to_float<T>(cosT[(int64_t)rpos * half + c]);
                const float sn = to_float<T>(sinT[(int64_t)rpos * half + c]);
                const float x1 = to_float<T>(o1), x2 = to_float<T>(o2);
                float r1, r2;
                rotate_pair(x1, x2, cs, sn, r1, r2);
                o1 = from_float<T>(r1);
                o2 = from_float<T>(r2);
            }
            kdst[d1] = o1;
            kdst[d2] = o2;
        }
        for (int d = lane; d < p.headdim; d += 64) vdst[d] = vsrc[d];
    }
    // the wave's own later loads of these rows must find them
    __threadfence_block();
}

// PART: the head dimension p.headdim is below D (a multiple of 8 above D/2, or below 64 for D = 64).  The lanes whose
// 16-byte pieces of a K / V row lie behind it load nothing and hold zeros, the k-steps and output tiles that only
// see such pieces are skipped, and the stores stop at the head dimension.
// A query block of more than 16 rows (p.row_tiles > 1) is cut into 16-row tiles and every (kv head, tile) is a unit of
// its own: `row0` is the tile's first row, `n_rows` the rows of the block.  The tiles of a kv head are neighbouring
// units, i.e. neighbouring waves of one workgroup that walk the same keys at the same time: the second one finds
// them in the cache hierarchy, not in HBM.
// RT = 2: the wave carries TWO 16-row tiles (rows row0 .. row0 + 31) through one pass over the keys: every K operand it
// reads from its LDS tile and every V operand it builds feeds two matrix instructions, and the chunk in flight - what
// bounds a stream like this one - serves 32 rows.  The registers that the second set of accumulators takes are those
// that staged K: with RT = 2 the K rows of a chunk go from global memory straight to LDS (global_load_lds_dwordx4: lane
// l's 16 bytes land at the instruction's LDS base + 16 l, so the lane that fills a place of the swizzled tile fetches
// the piece that belongs there), into the one of the wave's two tiles that is not being read; `ktile` then points at
// both (2 * kTileBytes), and the second doubles as the staging area of the q rows before the first chunk uses it.
template <typename T, int D, bool SOFTCAP, bool PART, int RT>
__device__ __forceinline__ void wave_piece(const DecodeParams &p, const int b, const int kvh, const int row0, const int n_rows,
                                           const UnitRange &ur, const int range_lo, const int range_hi, const bool write_final,
                                           const int64_t slot, uint8_t *ktile) {
    using Cfg = WaveCfg<D>;
    const int lane = threadIdx.x & 63;
    const int lq = lane >> 4;
    const int ln = lane & 15;
    const int Lk = ur.Lk;
    const int Sq = p.seqlen_q;
    const int off = Lk - Sq;

    const uint8_t *kc_base = reinterpret_cast<const uint8_t *>(p.k_cache) + (int64_t)kvh * p.k_stride_h * 2;
    const uint8_t *vc_base = reinterpret_cast<const uint8_t *>(p.v_cache) + (int64_t)kvh * p.v_stride_h * 2;
    const int32_t *bt_row = p.block_table + (int64_t)b * p.bt_stride_b;
    const int c_begin = range_lo / kChunk;
    const int c_end = (range_hi + kChunk - 1) / kChunk;

    uint32_t vreg[8][Cfg::kVH][Cfg::kVW / 2];
    const int hd = PART ? p.headdim : D;
    bool v_live[Cfg::kVH];
#pragma unroll
    for (int hh = 0; hh < Cfg::kVH; ++hh) v_live[hh] = !PART || hh * 128 + ln * Cfg::kVW < hd;
    if constexpr (PART) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
#pragma unroll
            for (int hh = 0; hh < Cfg::kVH; ++hh)
#pragma unroll
                for (int w2 = 0; w2 < Cfg::kVW / 2; ++w2) vreg[e][hh][w2] = 0u;
    }
    const uint32_t k_row_bytes = (uint32_t)p.k_stride_row * 2u;
    const uint32_t v_row_bytes = (uint32_t)p.v_stride_row * 2u;
    const int k_lane_row = lane / Cfg::kLanesPerRow;
    const uint32_t v_lane_col = (uint32_t)(ln * Cfg::kVW) * 2u;
    // direct loads: load j fills the LDS pieces 64j .. 64j+63 of the tile = rows j * kRowsPerLoad .., the lane's place c' of
    // row r holds the row's piece c' ^ (r & kSwzMask); kd_col[j % kSwzRows]: that piece's byte offset in its row
    constexpr int kSwzRows = (Cfg::kSwzMask + 1 + Cfg::kRowsPerLoad - 1) / Cfg::kRowsPerLoad;   // loads after which the pattern repeats
    uint32_t kd_col[kSwzRows], kd_off[kSwzRows];   // ... and with the lane's row inside a load added (chunks inside the sequence)
    bool kd_live[kSwzRows];
#pragma unroll
    for (int j = 0; j < kSwzRows; ++j) {
        const int c = (lane % Cfg::kLanesPerRow) ^ ((j * Cfg::kRowsPerLoad + k_lane_row) & Cfg::kSwzMask);
        kd_col[j] = (uint32_t)c * 16u;
        kd_off[j] = (uint32_t)k_lane_row * k_row_bytes + kd_col[j];
        kd_live[j] = !PART || c * 8 < hd;
    }
    auto lds_of = [](const void *ptr) -> uint32_t { return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)ptr; };
    // (written out: the compiler would wait for such a load in front of every LDS read that follows)
    auto load_k_direct = [&](uint32_t lds, uint32_t off, const uint8_t *base) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds), "v"(off), "s"(base) : "memory", "m0");
    };
    const uint32_t v_lane_off = (uint32_t)(lq * 4) * v_row_bytes + v_lane_col;

    auto load_blk = [&](int c) -> int {   // the table entry as loaded (every lane the same address); not waited for
        if (c >= c_end) return 0;
        int page = (c * kChunk) / p.page_size;
        page = min(page, p.max_blocks - 1);
        return bt_row[page];
    };
    auto use_blk = [&](int raw) -> int { return min(max(__builtin_amdgcn_readfirstlane(raw), 0), p.num_blocks - 1); };
    auto load_v = [&](const uint8_t *s2, int e, int hh) {
        if constexpr (Cfg::kVW == 8) {
            const u32x4_t t4 = load16_stream(s2);
            vreg[e][hh][0] = t4[0];
            vreg[e][hh][1] = t4[1];
            vreg[e][hh][2] = t4[2];
            vreg[e][hh][3] = t4[3];
        } else if constexpr (Cfg::kVW == 4) {
            typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
            const u32x2_t t2 = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(s2));
            vreg[e][hh][0] = t2[0];
            vreg[e][hh][1] = t2[1];
        } else {
            vreg[e][hh][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(s2));
        }
    };
    auto issue_loads = [&](int c, int blk, int kbuf) {
        const int key0 = c * kChunk;
        const int inpage0 = key0 % p.page_size;
        const int last = Lk - 1 - key0;  // last written key relative to the chunk (>= 0)
        const uint8_t *kb = kc_base + (int64_t)blk * p.k_stride_block * 2 + (int64_t)inpage0 * k_row_bytes;
        const uint8_t *vb = vc_base + (int64_t)blk * p.v_stride_block * 2 + (int64_t)inpage0 * v_row_bytes;
        const uint32_t lds = lds_of(ktile + kbuf * Cfg::kTileBytes);
        if (last >= kChunk - 1) {
#pragma unroll
            for (int j = 0; j < Cfg::kKLoads; ++j)
                if (kd_live[j % kSwzRows])
                    load_k_direct(lds + j * 1024u, kd_off[j % kSwzRows], kb + (size_t)(j * Cfg::kRowsPerLoad) * k_row_bytes);
#pragma unroll
            for (int hh = 0; hh < Cfg::kVH; ++hh)
                if (v_live[hh]) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        load_v(vb + (size_t)((e >> 2) * 16 + (e & 3)) * v_row_bytes + hh * 256 + v_lane_off, e, hh);
                }
        } else {
            // tail chunk: rows past the last written key re-read that key (their scores are masked)
#pragma unroll
            for (int j = 0; j < Cfg::kKLoads; ++j) {
                const int row = min(j * Cfg::kRowsPerLoad + k_lane_row, last);
                if (kd_live[j % kSwzRows]) load_k_direct(lds + j * 1024u, (uint32_t)row * k_row_bytes + kd_col[j % kSwzRows], kb);
            }
#pragma unroll
            for (int hh = 0; hh < Cfg::kVH; ++hh)
                if (v_live[hh]) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int row = min((e >> 2) * 16 + lq * 4 + (e & 3), last);
                        load_v(vb + (uint32_t)row * v_row_bytes + v_lane_col + hh * 256, e, hh);
                    }
                }
        }
    };

    // (with row tiles several waves read a chunk, so the host does not fuse the append then)
    if (p.k_new != nullptr && range_hi > ur.len_cache) append_rows_wave<T, D>(p, b, kvh, ur.len_cache, range_lo, range_hi);

    if constexpr (PART) {
        // the places of the K pieces that nobody loads hold zeros: the first tile here, the second once the q rows have left it
        for (int i = lane * 16; i < Cfg::kTileBytes; i += 64 * 16) *reinterpret_cast<u32x4_t *>(ktile + i) = u32x4_t{0, 0, 0, 0};
        __builtin_amdgcn_wave_barrier();
    }
    // first chunk in flight while Q is staged
    int c = c_begin;
    int blk_next;
    {
        // Both table entries are asked for before the first chunk's loads.  Loads return in order: asked for behind
        // them, the second entry would only be there when the whole chunk is, and the q rows would be requested a
        // memory latency later than they need be.
        const int blk0 = load_blk(c);
        blk_next = load_blk(c + 1);
        if (c < c_end) issue_loads(c, use_blk(blk0), 0);
    }
    // the q rows are staged in the wave's second tile: the first chunk that lands there leaves after they have been read
    uint16_t *sq = reinterpret_cast<uint16_t *>(ktile + Cfg::kTileBytes);
    static_assert(RT * 16 * D * 2 <= Cfg::kTileBytes, "the q rows fit a tile");

#pragma unroll
    for (int r = 0; r < RT; ++r) stage_q_wave<T, D, PART>(p, b, kvh, row0 + 16 * r, n_rows, ur.len_cache, sq + r * 16 * D);
    __builtin_amdgcn_wave_barrier();
    u32x4_t qreg[RT][Cfg::kKSteps];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < Cfg::kKSteps; ++t) qreg[r][t] = *reinterpret_cast<const u32x4_t *>(&sq[(r * 16 + ln) * D + t * 32 + lq * 8]);
    // the q rows have left the second tile before the first load into it is issued
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

    if constexpr (PART) {
        // the places of the K pieces that nobody loads hold zeros (the q rows lay elsewhere in this tile)
        __builtin_amdgcn_wave_barrier();
        for (int i = lane * 16; i < Cfg::kTileBytes; i += 64 * 16) *reinterpret_cast<u32x4_t *>(ktile + Cfg::kTileBytes + i) = u32x4_t{0, 0, 0, 0};
        __builtin_amdgcn_wave_barrier();
    }
    // visible key interval of query row ln of every tile, clipped to this piece
    int row_lo[RT], row_hi[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        row_lo[r] = range_lo;
        row_hi[r] = range_hi - 1;
        const int row = row0 + 16 * r + ln;
        const int qi = row / p.group;
        if (ur.wl >= 0) row_lo[r] = max(row_lo[r], qi + off - ur.wl);
        if (ur.wr >= 0) row_hi[r] = min(row_hi[r], qi + off + ur.wr);
        if (row >= n_rows) row_hi[r] = -1;
    }

    float m_run[RT], l_run[RT];
    float4_t o_acc[RT][Cfg::kColTiles];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        m_run[r] = -INFINITY;
        l_run[r] = 0.f;
#pragma unroll
        for (int t = 0; t < Cfg::kColTiles; ++t) o_acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    // The two waves of a SIMD belong to different workgroups and stream independent shares; with
    // equal priority the older one (wave slot 0) wins every arbitration and finishes ~10 % earlier,
    // and the launch lasts as long as the slower.  The priority changes chunk by chunk: slot 1 has
    // the higher one two chunks out of three, slot 0 the third (measured: 1:1 leaves slot 1 ~4 %
    // behind, 2:1 brings the two within 2 %).
    const int hw_slot = __builtin_amdgcn_s_getreg((1 << 11) | 4) & 1;   // HW_ID.WAVE_ID bit 0
    while (c < c_end) {
        if ((c % 3 == 0) == (hw_slot == 0))
            __builtin_amdgcn_s_setprio(1);
        else
            __builtin_amdgcn_s_setprio(0);
        // staged chunk: K -> swizzled LDS tile, V -> transposed operand registers
        const int kbuf = (c - c_begin) & 1;
        const uint8_t *kt = ktile + kbuf * Cfg::kTileBytes;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the chunk's K rows are in their tile (and its V rows in their registers)
        u32x4_t vt[Cfg::kColTiles];
#pragma unroll
        for (int hh = 0; hh < Cfg::kVH; ++hh)
#pragma unroll
            for (int w2 = 0; w2 < Cfg::kVW / 2; ++w2)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t a = vreg[2 * u][hh][w2];
                    const uint32_t bb = vreg[2 * u + 1][hh][w2];
                    vt[hh * Cfg::kVW + 2 * w2][u] = __builtin_amdgcn_perm(bb, a, 0x05040100u);
                    vt[hh * Cfg::kVW + 2 * w2 + 1][u] = __builtin_amdgcn_perm(bb, a, 0x07060302u);
                }
        __builtin_amdgcn_wave_barrier();

        const int cn = c + 1;
        if (cn < c_end) issue_loads(cn, use_blk(blk_next), kbuf ^ 1);
        // asked for behind the chunk's loads, the next table entry is there when they all are: the wave rests here
        // until chunk cn has landed and only then works on chunk c
        blk_next = __builtin_amdgcn_readfirstlane(load_blk(cn + 1));
        __builtin_amdgcn_sched_barrier(0);

        // S^T = K Q^T, two 16-key tiles (for every row tile)
        float4_t s[RT][2];
#pragma unroll
        for (int r = 0; r < RT; ++r) s[r][0] = s[r][1] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < Cfg::kKSteps; ++t) {
            if (PART && t * 32 >= hd) continue;   // wave-uniform
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const int row = tt * 16 + ln;
                const u32x4_t a = *reinterpret_cast<const u32x4_t *>(
                    kt + row * (D * 2) + (((t * 4 + lq) ^ (row & Cfg::kSwzMask)) << 4));
#pragma unroll
                for (int r = 0; r < RT; ++r) s[r][tt] = mfma16<T>(a, qreg[r][t], s[r][tt]);
            }
        }

        // online softmax of query row ln of every tile; register i of key tile tt is key c*32 + tt*16 + lq*4 + i
        const int key_base = c * kChunk + lq * 4;
        u32x4_t pk[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            float x[8];
            float mloc = -INFINITY;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = key_base + (e >> 2) * 16 + (e & 3);
                float v = s[r][e >> 2][e & 3];
                if constexpr (SOFTCAP) {
                    const float y = v * p.softcap_pre;
                    const float e2 = __expf(2.f * y);
                    v = p.softcap_post * (1.f - 2.f / (e2 + 1.f));
                } else {
                    v *= p.scale_log2;
                }
                v = (key >= row_lo[r] && key <= row_hi[r]) ? v : -INFINITY;
                x[e] = v;
                mloc = fmaxf(mloc, v);
            }
            mloc = quad_rows_max(mloc);
            const float m_new = fmaxf(m_run[r], mloc);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run[r] - m_use);
            m_run[r] = m_new;
            float psum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[e] = fast_exp2(x[e] - m_use);
                psum += x[e];
            }
            l_run[r] = l_run[r] * alpha + psum;
            pk[r][0] = pack2<T>(x[0], x[1]);
            pk[r][1] = pack2<T>(x[2], x[3]);
            pk[r][2] = pack2<T>(x[4], x[5]);
            pk[r][3] = pack2<T>(x[6], x[7]);
#pragma unroll
            for (int t = 0; t < Cfg::kColTiles; ++t) {
                o_acc[r][t][0] *= alpha;
                o_acc[r][t][1] *= alpha;
                o_acc[r][t][2] *= alpha;
                o_acc[r][t][3] *= alpha;
            }
        }
        // (every column tile interleaves columns of the whole 128-column pass, so none is dead as a whole)
#pragma unroll
        for (int t = 0; t < Cfg::kColTiles; ++t)
#pragma unroll
            for (int r = 0; r < RT; ++r) o_acc[r][t] = mfma16<T>(vt[t], pk[r], o_acc[r][t]);
        c = cn;
    }

    // ---- write.  Register i of column tile t = hh*kVW + w is column hh*128 + (lq*4 + i)*kVW + w
    //      of query row ln: kVW consecutive columns per (hh, i).
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const float lr = quad_rows_sum(l_run[r]);
        const int trow = 16 * r + ln;                 // row of the unit
        if (row0 + trow < n_rows && trow >= dead_rows(p, b)) {
            const float inv = (lr > 0.f) ? 1.f / lr : 0.f;
            const int qi = (row0 + trow) / p.group;
            const int head = kvh * p.group + (row0 + trow - qi * p.group);
            if (write_final) {
                uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                                (int64_t)head * p.o_stride_h;
#pragma unroll
                for (int hh = 0; hh < Cfg::kVH; ++hh)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (PART && hh * 128 + (lq * 4 + i) * Cfg::kVW >= hd) continue;
                        uint16_t *d2 = dst + hh * 128 + (lq * 4 + i) * Cfg::kVW;
#pragma unroll
                        for (int w = 0; w < Cfg::kVW; w += 2)
                            *reinterpret_cast<uint32_t *>(d2 + w) =
                                pack2<T>(o_acc[r][hh * Cfg::kVW + w][i] * inv, o_acc[r][hh * Cfg::kVW + w + 1][i] * inv);
                    }
                if (lq == 0)
                    p.lse[((int64_t)b * p.nheads + head) * Sq + qi] = (lr > 0.f) ? (m_run[r] + fast_log2(lr)) * kLn2 : INFINITY;
            } else {
                const int64_t srow = slot * p.rows + trow;
                float *dst = p.o_partial + srow * D;
#pragma unroll
                for (int hh = 0; hh < Cfg::kVH; ++hh)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float *d2 = dst + hh * 128 + (lq * 4 + i) * Cfg::kVW;
#pragma unroll
                        for (int w = 0; w < Cfg::kVW; w += 2)
                            *reinterpret_cast<float2 *>(d2 + w) =
                                make_float2(o_acc[r][hh * Cfg::kVW + w][i] * inv, o_acc[r][hh * Cfg::kVW + w + 1][i] * inv);
                    }
                if (lq == 0) p.lse_partial[srow] = (lr > 0.f) ? m_run[r] + fast_log2(lr) : -INFINITY;
            }
        }
    }
    __builtin_amdgcn_wave_barrier();   // the wave's LDS rows are reused by its next piece
}

template <typename T, int D, bool SOFTCAP, bool PART, int RT>
__global__ void __launch_bounds__(256, (D <= 128) ? 2 : 1) decode_wave_kernel(const DecodeParams p) {
    using Cfg = WaveCfg<D>;
    __shared__ int s_pref[257];
    // two K tiles per wave: the chunk being read and the chunk on its way; the second also stages the q rows of a piece
    __shared__ __attribute__((aligned(16))) uint8_t s_k[4][2 * Cfg::kTileBytes];
    const Partition pt = make_partition(p, s_pref);
    publish_partition(p, pt, s_pref);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    walk_share(p, pt, s_pref, (int64_t)blockIdx.x * 4 + wave,
               [&](int b, int unit, const UnitRange &ur, int range_lo, int range_hi, bool whole, int64_t slot) {
                   int kvh = unit, row0 = 0, n_rows = p.rows;
                   if (RT == 1 && p.row_tiles > 1) {
                       kvh = unit / p.row_tiles;
                       row0 = (unit - kvh * p.row_tiles) * 16;
                       n_rows = p.rows_total;
                   }
                   wave_piece<T, D, SOFTCAP, PART, RT>(p, b, kvh, row0, n_rows, ur, range_lo, range_hi, whole, slot, s_k[wave]);
               });
    init_empty_units<D>(p, pt);
}

template <typename T, int D, int RT> static hipError_t launch_wave_rt(const DecodeParams &p, hipStream_t stream) {
    dim3 grid(p.num_wgs), block(256);
    if (p.headdim > D || p.headdim < 8 || p.headdim % 8 != 0) return hipErrorInvalidValue;
    const bool part = p.headdim < D;
    if (p.softcap_post != 0.f) {
        if (part)
            hipLaunchKernelGGL((decode_wave_kernel<T, D, true, true, RT>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((decode_wave_kernel<T, D, true, false, RT>), grid, block, 0, stream, p);
    } else {
        if (part)
            hipLaunchKernelGGL((decode_wave_kernel<T, D, false, true, RT>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((decode_wave_kernel<T, D, false, false, RT>), grid, block, 0, stream, p);
    }
    return hipGetLastError();
}

// Blocks of up to 16 rows: one tile per wave.  17 .. 32 rows: two tiles per wave where the registers allow it
// (wave_rows_per_unit(D) = 32); otherwise the host has cut the block into 16-row units (p.row_tiles > 1).
template <typename T, int D> static hipError_t launch_wave_d(const DecodeParams &p, hipStream_t stream) {
    if (p.rows > 16) {
        if constexpr (wave_rows_per_unit(D) >= 32)
            return launch_wave_rt<T, D, 2>(p, stream);
        else
            return hipErrorInvalidValue;
    }
    return launch_wave_rt<T, D, 1>(p, stream);
}

template <typename T> static hipError_t launch_wave_t(const DecodeParams &p, int headdim, hipStream_t stream) {
    switch (headdim) {
        case 64: return launch_wave_d<T, 64>(p, stream);
        case 128: return launch_wave_d<T, 128>(p, stream);
        case 256: return launch_wave_d<T, 256>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_decode_wave(const DecodeParams &p, int dtype, int headdim, hipStream_t stream) {
    if (p.rows > wave_rows_per_unit(headdim) || !p.balanced || !p.wave_workers || p.num_workers != p.num_wgs * 4) return hipErrorInvalidValue;
    if (p.rows > 16 && p.row_tiles > 1) return hipErrorInvalidValue;
    if (p.row_tiles > 1 && (p.rows != 16 || p.k_new != nullptr || p.q_live != nullptr || p.rows_total > 16 * p.row_tiles ||
                            p.nheads_k % p.row_tiles != 0))
        return hipErrorInvalidValue;
    return dtype == 0 ? launch_wave_t<BF16>(p, headdim, stream) : launch_wave_t<FP16>(p, headdim, stream);
}

}  // namespace fa
