// Paged GQA/MQA decode for gfx950: one workgroup per (batch row, kv head, KV split) that packs
// every query row of the group (seqlen_q * group <= 64) and streams the row's K/V pages once.
//
// It takes the place of the reference's FAInfer task loop for decode-shaped calls
// (csrc/ascend910/flash_attn_npu/mha_fwd_kvcache.cpp:436-970: paged addressing :496,527, key-range
// clipping :556-595, 512-key online-softmax loop :632-969) and of its flash-decode epilogue
// (CombineScale.hpp:76-357), with these differences of design:
//   * each of the NW wavefronts walks its own 32-key chunks with a private running (max, sum, O);
//     there is no workgroup barrier in the stream loop, waves merge once at the end through LDS;
//   * K rows are fetched as whole 16-byte-per-lane coalesced rows, staged through a swizzled LDS
//     tile and read back in MFMA operand order; V rows are fetched straight into the operand
//     order (lanes 16q..16q+15 read one whole row) and transposed in registers with v_perm;
//   * S^T = K Q^T and O^T = V^T P^T run on the 16x16x32 MFMA so the softmax state of a query row
//     lives in one lane column for both products (no cross-lane traffic for the rescale);
//   * lengths are read on the device; no host copy of cache_seqlens, no mask tensor.
#include "decode_common.h"

namespace fa {


template <int D> struct DecodeCfg {
    static constexpr int kLanesPerRow = D / 8;            // 16-byte pieces in one K row
    static constexpr int kRowsPerLoad = 64 / kLanesPerRow;
    static constexpr int kKLoads = kChunk / kRowsPerLoad;  // K load instructions per chunk
    static constexpr int kKSteps = D / 32;                 // MFMA k-steps of QK^T
    static constexpr int kVW = (D >= 128) ? 8 : D / 16;    // V columns one lane holds per key and pass
    static constexpr int kVH = D / (16 * kVW);             // column passes (128 columns each)
    static constexpr int kColTiles = D / 16;               // 16-column tiles of O^T
    static constexpr int kSwzMask = (kLanesPerRow >= 16) ? 15 : kLanesPerRow - 1;
};

// byte offset of 16-byte piece `ch` of row `row` in a wave's swizzled K tile
template <int D> __device__ __forceinline__ int k_tile_offset(int row, int ch) {
    return row * (D * 2) + ((ch ^ (row & DecodeCfg<D>::kSwzMask)) << 4);
}

// One piece of work: query block (b, kvh) against keys [range_lo, range_hi).  Writes the final
// output when `write_final`, else the normalised fp32 partial and its base-2 LSE into `slot`.
// PART: the head dimension p.headdim is below D.  Lanes whose 16-byte pieces of a K / V row lie behind it load nothing
// and hold zeros, k-steps that only see such pieces are skipped, and the stores stop at the head dimension.
template <typename T, int D, int RT, int NW, bool SOFTCAP, bool PART>
__device__ __forceinline__ void process_piece(const DecodeParams &p, const int b, const int kvh, const UnitRange &ur,
                                              const int range_lo, const int range_hi, const bool write_final,
                                              const int64_t slot) {
    using Cfg = DecodeCfg<D>;
    constexpr int ROWS = 16 * RT;
    constexpr int K_TILE_BYTES = kChunk * D * 2;
    constexpr int O_STAGE_BYTES = ROWS * D * 4;
    constexpr int MAIN_BYTES = (NW * K_TILE_BYTES > O_STAGE_BYTES) ? NW * K_TILE_BYTES : O_STAGE_BYTES;

    __shared__ __attribute__((aligned(16))) uint8_t s_main[MAIN_BYTES];  // K tiles, later the O merge buffer
    __shared__ __attribute__((aligned(16))) uint16_t s_q[ROWS * D];
    __shared__ float s_m[NW][ROWS];
    __shared__ float s_l[NW][ROWS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane >> 4;   // lane group: MFMA k-slot / key sub-block
    const int ln = lane & 15;   // MFMA row or column index

    const int len_cache = ur.len_cache;
    const int Lk = ur.Lk;
    const int Sq = p.seqlen_q;
    const int off = Lk - Sq;
    const int wr_eff = ur.wr;
    const int wl = ur.wl;

    // per-lane visible key interval of query row (r*16 + ln), clipped to this split
    int row_lo[RT], row_hi[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int row = r * 16 + ln;
        const int qi = row / p.group;
        int klo = range_lo, khi = range_hi - 1;
        if (wl >= 0) klo = max(klo, qi + off - wl);
        if (wr_eff >= 0) khi = min(khi, qi + off + wr_eff);
        if (row >= p.rows) khi = -1;
        row_lo[r] = klo;
        row_hi[r] = khi;
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

    uint8_t *ktile = s_main + wave * K_TILE_BYTES;
    const uint8_t *kc_base = reinterpret_cast<const uint8_t *>(p.k_cache) + (int64_t)kvh * p.k_stride_h * 2;
    const uint8_t *vc_base = reinterpret_cast<const uint8_t *>(p.v_cache) + (int64_t)kvh * p.v_stride_h * 2;
    const int32_t *bt_row = p.block_table + (int64_t)b * p.bt_stride_b;

    const int c_begin = range_lo / kChunk;
    const int c_end = (range_hi + kChunk - 1) / kChunk;

    u32x4_t kreg[Cfg::kKLoads];
    uint32_t vreg[8][Cfg::kVH][Cfg::kVW / 2];
    const int hd = PART ? p.headdim : D;
    const bool k_live = !PART || (lane % Cfg::kLanesPerRow) * 8 < hd;
    bool v_live[Cfg::kVH];
#pragma unroll
    for (int hh = 0; hh < Cfg::kVH; ++hh) v_live[hh] = !PART || hh * 128 + ln * Cfg::kVW < hd;
    if constexpr (PART) {
#pragma unroll
        for (int j = 0; j < Cfg::kKLoads; ++j) kreg[j] = u32x4_t{0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 8; ++e)
#pragma unroll
            for (int hh = 0; hh < Cfg::kVH; ++hh)
#pragma unroll
                for (int w2 = 0; w2 < Cfg::kVW / 2; ++w2) vreg[e][hh][w2] = 0u;
    }

    // per-lane byte offsets inside a page that do not change from chunk to chunk; the per-load
    // part is wave-uniform and folds into the scalar base address
    const uint32_t k_row_bytes = (uint32_t)p.k_stride_row * 2u;
    const uint32_t v_row_bytes = (uint32_t)p.v_stride_row * 2u;
    const int k_lane_row = lane / Cfg::kLanesPerRow;
    const uint32_t k_lane_col = (uint32_t)(lane % Cfg::kLanesPerRow) * 16u;
    const uint32_t v_lane_col = (uint32_t)(ln * Cfg::kVW) * 2u;
    const uint32_t k_lane_off = (uint32_t)k_lane_row * k_row_bytes + k_lane_col;
    const uint32_t v_lane_off = (uint32_t)(lq * 4) * v_row_bytes + v_lane_col;

    // page id of chunk c (clamped into the pool so a corrupt table cannot fault)
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

    auto issue_loads = [&](int c, int blk) {
        const int key0 = c * kChunk;
        const int inpage0 = key0 % p.page_size;
        const int last = Lk - 1 - key0;  // last initialised key, relative to the chunk (>= 0)
        const uint8_t *kb = kc_base + (int64_t)blk * p.k_stride_block * 2 + (int64_t)inpage0 * k_row_bytes;
        const uint8_t *vb = vc_base + (int64_t)blk * p.v_stride_block * 2 + (int64_t)inpage0 * v_row_bytes;
        if (last >= kChunk - 1) {
            if (k_live) {
#pragma unroll
                for (int j = 0; j < Cfg::kKLoads; ++j)
                    kreg[j] = load16_stream(kb + (size_t)(j * Cfg::kRowsPerLoad) * k_row_bytes + k_lane_off);
            }
#pragma unroll
            for (int hh = 0; hh < Cfg::kVH; ++hh)
                if (v_live[hh]) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        load_v(vb + (size_t)((e >> 2) * 16 + (e & 3)) * v_row_bytes + hh * 256 + v_lane_off, e, hh);
                }
        } else {
            // tail chunk: rows past the last written key re-read that key (their scores are masked)
            if (k_live) {
#pragma unroll
                for (int j = 0; j < Cfg::kKLoads; ++j) {
                    const int row = min(j * Cfg::kRowsPerLoad + k_lane_row, last);
                    kreg[j] = load16(kb + (uint32_t)row * k_row_bytes + k_lane_col);
                }
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

    int c = c_begin + wave;
    int blk_next;
    {
        // Both table entries are asked for before the first chunk's loads.  Loads return in order: asked for behind
        // them, the second entry would only be there when the whole chunk is, and the q rows would be requested a
        // memory latency later than they need be.
        const int blk0 = load_blk(c);
        blk_next = load_blk(c + NW);
        if (c < c_end) issue_loads(c, use_blk(blk0));
    }

    // (the first chunk is already in flight while Q is staged)
    // ---- stage Q (with rotary) into LDS as 16-bit rows -------------------------------------
    {
        const uint16_t *qbase = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_stride_b;
        const uint16_t *cosT = reinterpret_cast<const uint16_t *>(p.rotary_cos);
        const uint16_t *sinT = reinterpret_cast<const uint16_t *>(p.rotary_sin);
        const int rot = (cosT != nullptr) ? p.rotary_dim : 0;
        const int half = rot >> 1;
        for (int idx = tid; idx < ROWS * (D / 2); idx += NW * 64) {
            const int row = idx / (D / 2);
            const int c = idx - row * (D / 2);
            int d1, d2;
            if (c < half) {
                d1 = p.rotary_interleaved ? 2 * c : c;
                d2 = p.rotary_interleaved ? 2 * c + 1 : c + half;
            } else {
                d1 = rot + 2 * (c - half);
                d2 = d1 + 1;
            }
            uint16_t o1 = 0, o2 = 0;
            if (row < p.rows && (!PART || c < hd / 2)) {   // pairs behind the head dimension stay zero (c < hd/2 <=> d1, d2 < hd)
                const int qi = row / p.group;
                const int g = row - qi * p.group;
                const uint16_t *src = qbase + (int64_t)qi * p.q_stride_s + (int64_t)(kvh * p.group + g) * p.q_stride_h;
                o1 = src[d1];
                o2 = src[d2];
                if (c < half) {
                    int pos = len_cache + (p.rotary_per_token ? qi : 0);
                    pos = min(max(pos, 0), p.seqlen_ro - 1);
                    const float cs = to_float<T>(cosT[(int64_t)pos * half + c]);
                    const float sn = to_float<T>(sinT[(int64_t)pos * half + c]);
                    const float x1 = to_float<T>(o1), x2 = to_float<T>(o2);
                    float r1, r2;
                    rotate_pair(x1, x2, cs, sn, r1, r2);
                    o1 = from_float<T>(r1);
                    o2 = from_float<T>(r2);
                }
            }
            s_q[row * D + d1] = o1;
            s_q[row * D + d2] = o2;
        }
    }
    __syncthreads();

    // Q^T as MFMA B operand: lane (lq, ln) holds row ln, elements t*32 + lq*8 .. +7
    u32x4_t qreg[RT][Cfg::kKSteps];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < Cfg::kKSteps; ++t)
            qreg[r][t] = *reinterpret_cast<const u32x4_t *>(&s_q[(r * 16 + ln) * D + t * 32 + lq * 8]);

    while (c < c_end) {
        // ---- move the staged chunk: K -> swizzled LDS tile, V -> transposed operand registers
#pragma unroll
        for (int j = 0; j < Cfg::kKLoads; ++j) {
            const int row = j * Cfg::kRowsPerLoad + lane / Cfg::kLanesPerRow;
            const int ch = lane % Cfg::kLanesPerRow;
            *reinterpret_cast<u32x4_t *>(ktile + k_tile_offset<D>(row, ch)) = kreg[j];
        }
        // vt[T]: 8 keys of column tile T for this lane's column; dword u = keys (2u, 2u+1)
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

        const int cn = c + NW;
        if (cn < c_end) issue_loads(cn, use_blk(blk_next));
        // asked for behind the chunk's loads, the next table entry is there when they all are: the wave rests here
        // until chunk cn has landed and only then works on chunk c
        blk_next = __builtin_amdgcn_readfirstlane(load_blk(cn + NW));
        __builtin_amdgcn_sched_barrier(0);

        // ---- S^T = K Q^T : two 16-key tiles x RT row tiles
        float4_t s[2][RT];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < RT; ++r) s[tt][r] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < Cfg::kKSteps; ++t) {
            if (PART && t * 32 >= hd) continue;   // wave-uniform
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const u32x4_t a =
                    *reinterpret_cast<const u32x4_t *>(ktile + k_tile_offset<D>(tt * 16 + ln, t * 4 + lq));
#pragma unroll
                for (int r = 0; r < RT; ++r) s[tt][r] = mfma16<T>(a, qreg[r][t], s[tt][r]);
            }
        }

        // ---- online softmax per query row (lane column ln of tile r)
        const int key_base = c * kChunk + lq * 4;
        u32x4_t pk[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            float x[8];
            float mloc = -INFINITY;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = key_base + (e >> 2) * 16 + (e & 3);
                float v = s[e >> 2][r][e & 3];
                if constexpr (SOFTCAP) {
                    // cap * tanh(s*scale/cap), then to base 2
                    const float y = v * p.softcap_pre;
                    const float e2 = __expf(2.f * y);
                    v = p.softcap_post * (1.f - 2.f / (e2 + 1.f));
                } else {
                    v *= p.scale_log2;
                }
                const bool vis = (key >= row_lo[r]) && (key <= row_hi[r]);
                v = vis ? v : -INFINITY;
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

        // ---- O^T += V^T P^T
#pragma unroll
        for (int t = 0; t < Cfg::kColTiles; ++t)
#pragma unroll
            for (int r = 0; r < RT; ++r) o_acc[r][t] = mfma16<T>(vt[t], pk[r], o_acc[r][t]);

        c = cn;
    }

    // ---- merge the waves --------------------------------------------------------------------
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        l_run[r] = quad_rows_sum(l_run[r]);
        if (lq == 0) {
            s_m[wave][r * 16 + ln] = m_run[r];
            s_l[wave][r * 16 + ln] = l_run[r];
        }
    }
    __syncthreads();  // also: every wave is done with its K tile

    float fac[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        float mg = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) mg = fmaxf(mg, s_m[w][r * 16 + ln]);
        const float mg_use = (mg == -INFINITY) ? 0.f : mg;
        fac[r] = fast_exp2(m_run[r] - mg_use);
    }

    float *o_stage = reinterpret_cast<float *>(s_main);  // [ROWS][D], or [NW][ROWS][D] when RT == 1
    constexpr bool kParallelMerge = (RT == 1);
    if constexpr (kParallelMerge) {
        // every wave drops its rescaled accumulator into its own buffer; the writers add them up
        float *mine = o_stage + wave * (ROWS * D);
#pragma unroll
        for (int t = 0; t < Cfg::kColTiles; ++t) {
            const int hh = t / Cfg::kVW, w2 = t % Cfg::kVW;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = hh * 128 + (lq * 4 + i) * Cfg::kVW + w2;
                mine[ln * D + col] = o_acc[0][t][i] * fac[0];
            }
        }
        __syncthreads();
    } else {
        for (int w = 0; w < NW; ++w) {
            if (wave == w) {
#pragma unroll
                for (int r = 0; r < RT; ++r)
#pragma unroll
                    for (int t = 0; t < Cfg::kColTiles; ++t) {
                        const int hh = t / Cfg::kVW, w2 = t % Cfg::kVW;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int col = hh * 128 + (lq * 4 + i) * Cfg::kVW + w2;
                            float *dst = &o_stage[(r * 16 + ln) * D + col];
                            const float v = o_acc[r][t][i] * fac[r];
                            if (w == 0) *dst = v; else *dst += v;
                        }
                    }
            }
            __syncthreads();
        }
    }

    // ---- write: final output or split partial ------------------------------------------------
    constexpr int PIECES = D / 8;  // 8-column pieces per row
    for (int idx = tid; idx < p.rows * PIECES; idx += NW * 64) {
        const int row = idx / PIECES;
        const int piece = idx - row * PIECES;
        float mg = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) mg = fmaxf(mg, s_m[w][row]);
        const float mg_use = (mg == -INFINITY) ? 0.f : mg;
        float lg = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) lg += s_l[w][row] * fast_exp2(s_m[w][row] - mg_use);
        const float inv = (lg > 0.f) ? 1.f / lg : 0.f;
        const float *src = &o_stage[row * D + piece * 8];
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float a = src[e];
            if constexpr (kParallelMerge) {
#pragma unroll
                for (int w = 1; w < NW; ++w) a += src[w * (ROWS * D) + e];
            }
            v[e] = a * inv;
        }
        const int qi = row / p.group;
        const int g = row - qi * p.group;
        const int head = kvh * p.group + g;
        if (write_final) {
            if (PART && piece * 8 >= hd) continue;
            u32x4_t o4;
            o4[0] = pack2<T>(v[0], v[1]);
            o4[1] = pack2<T>(v[2], v[3]);
            o4[2] = pack2<T>(v[4], v[5]);
            o4[3] = pack2<T>(v[6], v[7]);
            uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                            (int64_t)head * p.o_stride_h + piece * 8;
            store16(dst, o4);
            if (piece == 0)
                p.lse[((int64_t)b * p.nheads + head) * Sq + qi] = (lg > 0.f) ? (mg + fast_log2(lg)) * kLn2 : INFINITY;
        } else {
            const int64_t srow = slot * p.rows + row;
            float *dst = p.o_partial + srow * D + piece * 8;
            *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4 *>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
            if (piece == 0) p.lse_partial[srow] = (lg > 0.f) ? mg + fast_log2(lg) : -INFINITY;
        }
    }
    __syncthreads();  // the LDS buffers may be reused by the next piece
}

// ---- grid mode: blockIdx = (split, kv head, batch row), fixed keys per split -------------------
template <typename T, int D, int RT, int NW, bool SOFTCAP, bool PART>
__global__ void __launch_bounds__(NW * 64, (D <= 128 && RT <= 2) ? 2 : 1)
decode_paged_kernel(const DecodeParams p) {
    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    const int b = blockIdx.z;
    const UnitRange ur = unit_range(p, b, window_norm_m(p));
    const bool empty = ur.nchunks == 0;
    const int lo_al = ur.c0 * kChunk;
    // splits this row really has; the grid was sized from shapes, so clamp and let the last split
    // run to the end of the range if the caller's lengths exceed what the shapes promised
    const int nsplits_row = empty ? 1 : min(p.nsplits, (ur.hi - lo_al + p.split_keys - 1) / p.split_keys);
    if (split >= nsplits_row) return;
    int range_lo = 0, range_hi = 0;
    if (!empty) {
        range_lo = max(ur.lo, lo_al + split * p.split_keys);
        range_hi = (split == nsplits_row - 1) ? ur.hi : min(ur.hi, lo_al + (split + 1) * p.split_keys);
    }
    const int64_t slot = ((int64_t)b * p.nheads_k + kvh) * p.nsplits + split;
    process_piece<T, D, RT, NW, SOFTCAP, PART>(p, b, kvh, ur, range_lo, range_hi, nsplits_row == 1, slot);
}

// ---- balanced mode ---------------------------------------------------------------------------
// The chunks of all (batch row, kv head) units, in (b, kvh) order, form one list of W chunks that
// is cut into gridDim.x equal contiguous shares, one per workgroup, cutting inside a unit where a
// share ends - the reference's flash-decode partition (flash_api.cpp:97-354, splitBN2S1GS2) done by
// every workgroup for itself from the device-resident lengths.  A workgroup writes the final
// output of every unit that lies wholly inside its share and at most two partials.

template <typename T, int D, int RT, int NW, bool SOFTCAP, bool PART>
__global__ void __launch_bounds__(NW * 64, (D <= 128 && RT <= 2) ? 2 : 1)
decode_balanced_kernel(const DecodeParams p) {
    static_assert(NW == 4, "the batch scan assumes 256 threads");
    balanced_driver<D>(p, blockIdx.x, [&](int b, int kvh, const UnitRange &ur, int range_lo, int range_hi, bool whole, int64_t slot) {
        process_piece<T, D, RT, NW, SOFTCAP, PART>(p, b, kvh, ur, range_lo, range_hi, whole, slot);
    });
}

// Split-KV combine (CombineScale.hpp:166-194,249-316), one wave per query row.
// Grid mode: one 64-thread workgroup per (query row, kv head, batch row).
template <typename T, int D>
__global__ void __launch_bounds__(64) splitkv_combine_kernel(const DecodeParams p) {
    const int row = blockIdx.x;
    const int kvh = blockIdx.y;
    const int b = blockIdx.z;
    const UnitRange ur = unit_range(p, b, window_norm_m(p));
    int split_keys = p.split_keys;
    if (p.split_adaptive)
        split_keys = adaptive_split_keys(min(block_max_keys(p.cache_seqlens, p.batch, p.seqlen_new), p.max_blocks * p.page_size),
                                         p.nsplits);
    const int lo_al = ur.c0 * kChunk;
    const int ns = (ur.nchunks == 0) ? 1 : min(p.nsplits, (ur.hi - lo_al + split_keys - 1) / split_keys);
    if (ns == 1) return;  // the kernel that computed this unit already wrote it
    combine_row_wave<T, D>(p, b, kvh, row, ns,
                           [&](int s) -> int64_t { return ((int64_t)b * p.nheads_k + kvh) * p.nsplits + s; });
}

// Merge of one query row by a whole 256-thread workgroup: D/4 column groups x (1024/D) piece
// lanes, reduced through LDS.  Every thread of the workgroup must call.
template <typename T, int D>
__device__ __forceinline__ void combine_row_block(const DecodeParams &p, int b, int kvh, int row, const UnitPieces &pcs) {
    constexpr int CG = D / 4;        // threads across the columns (4 columns each)
    constexpr int NPL = 256 / CG;    // piece lanes
    __shared__ float s_red[4];
    __shared__ float s_tot[NPL];
    __shared__ __attribute__((aligned(16))) float s_acc[NPL][D];
    const int tid = threadIdx.x;
    const int ns = pcs.ns;

    const int cg = tid % CG;
    const int pl = tid / CG;
    auto load_row = [&](int64_t srow) -> float4 {
        if constexpr (partials_are_half(D)) {
            const uint2 t = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p.o_partial) + srow * D + cg * 4);
            return make_float4(to_float<FP16>((uint16_t)(t.x & 0xffffu)), to_float<FP16>((uint16_t)(t.x >> 16)),
                               to_float<FP16>((uint16_t)(t.y & 0xffffu)), to_float<FP16>((uint16_t)(t.y >> 16)));
        } else {
            return *reinterpret_cast<const float4 *>(p.o_partial + srow * D + cg * 4);
        }
    };
    auto block_max = [&](float mx) -> float {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
        if ((tid & 63) == 0) s_red[tid >> 6] = mx;
        __syncthreads();
        return fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    };
    float tot = 0.f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float mx;
    constexpr int PL = 8;   // pieces of a thread in flight
    if (ns <= PL * NPL) {
        // The pieces were written by other compute units: every dependent load is a trip to memory.  All log-sum-exps
        // and rows of the unit are requested at once (a thread holds up to PL of each); the maximum is then taken
        // over what the threads hold, while the rows are still on their way.
        float lw[PL];
        float4 o[PL];
#pragma unroll
        for (int i = 0; i < PL; ++i) {
            const int s2 = pl + i * NPL;
            const int64_t srow = pcs.slot(min(s2, ns - 1)) * p.rows + row;
            lw[i] = (s2 < ns) ? p.lse_partial[srow] : -INFINITY;
            o[i] = load_row(srow);
        }
        mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < PL; ++i) mx = fmaxf(mx, lw[i]);
        mx = block_max(mx);
        const float mx_use = (mx == -INFINITY) ? 0.f : mx;
#pragma unroll
        for (int i = 0; i < PL; ++i) {
            const float w = fast_exp2(lw[i] - mx_use);   // 0 behind the last piece (-inf)
            tot += w;
            acc[0] += w * o[i].x;
            acc[1] += w * o[i].y;
            acc[2] += w * o[i].z;
            acc[3] += w * o[i].w;
        }
    } else {
        mx = -INFINITY;
        for (int s2 = tid; s2 < ns; s2 += 256) mx = fmaxf(mx, p.lse_partial[pcs.slot(s2) * p.rows + row]);
        mx = block_max(mx);
        const float mx_use = (mx == -INFINITY) ? 0.f : mx;
        // four of the thread's pieces are requested before the first is used (one trip to memory per four)
        for (int s0 = pl; s0 < ns; s0 += 4 * NPL) {
            float lw[4];
            float4 o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t srow = pcs.slot(min(s0 + i * NPL, ns - 1)) * p.rows + row;
                lw[i] = p.lse_partial[srow];
                o[i] = load_row(srow);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float w = (s0 + i * NPL < ns) ? fast_exp2(lw[i] - mx_use) : 0.f;
                tot += w;
                acc[0] += w * o[i].x;
                acc[1] += w * o[i].y;
                acc[2] += w * o[i].z;
                acc[3] += w * o[i].w;
            }
        }
    }
    *reinterpret_cast<float4 *>(&s_acc[pl][cg * 4]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    if (cg == 0) s_tot[pl] = tot;
    __syncthreads();
    if (pl == 0) {
        tot = 0.f;
        acc[0] = acc[1] = acc[2] = acc[3] = 0.f;
#pragma unroll
        for (int l = 0; l < NPL; ++l) {
            tot += s_tot[l];
            const float4 o = *reinterpret_cast<const float4 *>(&s_acc[l][cg * 4]);
            acc[0] += o.x;
            acc[1] += o.y;
            acc[2] += o.z;
            acc[3] += o.w;
        }
        const float inv = (tot > 0.f) ? 1.f / tot : 0.f;
        const RowId rid = row_id(p, kvh, row);
        const int qi = rid.qi, head = rid.head;
        uint16_t *out_row = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                            (int64_t)head * p.o_stride_h;
        uint2 o2;
        o2.x = pack2<T>(acc[0] * inv, acc[1] * inv);
        o2.y = pack2<T>(acc[2] * inv, acc[3] * inv);
        if (cg * 4 < p.headdim) *reinterpret_cast<uint2 *>(out_row + cg * 4) = o2;
        if (cg == 0)
            p.lse[((int64_t)b * p.nheads + head) * p.seqlen_q + qi] = (tot > 0.f) ? (mx + fast_log2(tot)) * kLn2 : INFINITY;
    }
    __syncthreads();   // s_acc / s_red are reused by the next row
}

// Balanced mode: blockIdx = (row group, kv head, batch row).  The workgroup recomputes the partition,
// finds the unit's pieces and merges its share of the query rows
template <typename T, int D>
__global__ void __launch_bounds__(256) splitkv_combine_balanced_kernel(const DecodeParams p) {
    __shared__ int s_pref[257];
    const int kvh = blockIdx.y;
    const int b = blockIdx.z;
    Partition pt;
    int pref_b;
    if (partition_published(p)) {   // launch-uniform
        pt = read_partition(p, b, &pref_b);
    } else {
        pt = make_partition(p, s_pref);
        pref_b = chunks_before(p, pt, s_pref, b);
    }
    const UnitRange ur = unit_range(p, b, pt.M);
    if (ur.nchunks == 0) return;   // the decode kernel initialised this unit
    const int64_t start = (int64_t)pref_b * pt.list_heads +
                          (pt.list_heads == 1 ? 0 : (int64_t)kvh * unit_cost(ur.nchunks, pt.cost));
    const UnitPieces pcs = unit_pieces(pt, start, ur.nchunks, kvh, p.nheads_k, pt.cost);
    if (pcs.ns == 1) return;       // written whole by one worker
    const int row0 = dead_rows(p, b);
    if (pcs.ns <= 16) {
        // few pieces: the four waves merge four rows side by side, no barrier and one chain of
        // dependent loads per row
        const int wave = threadIdx.x >> 6;
        for (int row = row0 + blockIdx.x * 4 + wave; row < p.rows; row += gridDim.x * 4)
            combine_row_wave<T, D>(p, b, kvh, row, pcs.ns, [&](int s) { return pcs.slot(s); });
        return;
    }
    // many pieces: the whole workgroup on one row at a time
    for (int row = row0 + blockIdx.x; row < p.rows; row += gridDim.x)
        if (row_id(p, kvh, row).head < p.nheads) combine_row_block<T, D>(p, b, kvh, row, pcs);   // block-uniform
}

template <typename T, int D, int RT, bool SOFTCAP, bool PART>
static hipError_t launch_decode_sp(const DecodeParams &p, hipStream_t stream) {
    constexpr int NW = 4;
    if (p.balanced)
        hipLaunchKernelGGL((decode_balanced_kernel<T, D, RT, NW, SOFTCAP, PART>), dim3(p.num_wgs), dim3(NW * 64), 0, stream, p);
    else
        hipLaunchKernelGGL((decode_paged_kernel<T, D, RT, NW, SOFTCAP, PART>), dim3(p.nsplits, p.nheads_k, p.batch), dim3(NW * 64), 0,
                           stream, p);
    return hipGetLastError();
}

template <typename T, int D, int RT>
static hipError_t launch_decode_rt(const DecodeParams &p, hipStream_t stream) {
    if (p.headdim > D || p.headdim < 8 || p.headdim % 8 != 0) return hipErrorInvalidValue;
    const bool softcap = p.softcap_post != 0.f;
    if (p.headdim < D) return softcap ? launch_decode_sp<T, D, RT, true, true>(p, stream) : launch_decode_sp<T, D, RT, false, true>(p, stream);
    return softcap ? launch_decode_sp<T, D, RT, true, false>(p, stream) : launch_decode_sp<T, D, RT, false, false>(p, stream);
}

template <typename T, int D> static hipError_t launch_decode_d(const DecodeParams &p, hipStream_t stream) {
    const int rt = (p.rows + 15) / 16;
    if (rt <= 1) return launch_decode_rt<T, D, 1>(p, stream);
    if (rt <= 2) return launch_decode_rt<T, D, 2>(p, stream);
    return hipErrorInvalidValue;   // taller blocks belong to the tiled kernel (kDecodeMaxRows)
}

template <typename T> static hipError_t launch_decode_t(const DecodeParams &p, int headdim, hipStream_t stream) {
    switch (headdim) {
        case 64: return launch_decode_d<T, 64>(p, stream);
        case 128: return launch_decode_d<T, 128>(p, stream);
        case 256: return launch_decode_d<T, 256>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_decode_paged(const DecodeParams &p, int dtype, int headdim, hipStream_t stream) {
    if (p.balanced && p.wave_workers) return launch_decode_wave(p, dtype, headdim, stream);
    return dtype == 0 ? launch_decode_t<BF16>(p, headdim, stream) : launch_decode_t<FP16>(p, headdim, stream);
}

template <typename T, int D> static void launch_combine_d(const DecodeParams &p, hipStream_t stream) {
    if (p.balanced) {
        // one workgroup per unit when there are many units, up to one per query row when there are few (units
        // of few pieces use the first quarter of them, four rows each)
        const int units = p.nheads_k * p.batch;
        const int row_groups = max(1, min(p.rows, 1024 / max(units, 1)));
        hipLaunchKernelGGL((splitkv_combine_balanced_kernel<T, D>), dim3(row_groups, p.nheads_k, p.batch), dim3(256), 0,
                           stream, p);
    } else {
        hipLaunchKernelGGL((splitkv_combine_kernel<T, D>), dim3(p.rows, p.nheads_k, p.batch), dim3(64), 0, stream, p);
    }
}

template <typename T> static hipError_t launch_combine_t(const DecodeParams &p, int headdim_v, hipStream_t stream) {
    switch (headdim_v) {
        case 64: launch_combine_d<T, 64>(p, stream); break;
        case 128: launch_combine_d<T, 128>(p, stream); break;
        case 256: launch_combine_d<T, 256>(p, stream); break;
        case 512: launch_combine_d<T, 512>(p, stream); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_splitkv_combine(const DecodeParams &p, int dtype, int headdim_v, hipStream_t stream) {
    return dtype == 0 ? launch_combine_t<BF16>(p, headdim_v, stream) : launch_combine_t<FP16>(p, headdim_v, stream);
}

}  // namespace fa
