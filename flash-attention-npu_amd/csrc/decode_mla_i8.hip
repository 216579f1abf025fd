// Latent-attention (MLA) decode over an int8 paged cache with per-token fp32 scales, gfx950.
//
// Layout: one latent kv head, 576 key dims, V = the first 512 of them (v_cache aliases k_cache);
// 128 q heads (any multiple of 64), any seqlen_q (each query token is its own set of units).  The reference has no quantised path
// (dtypes are limited to fp16/bf16 at csrc/ascend910/flash_attn_npu/flash_api.cpp:386-388 and
// descales are rejected at flash_attn_npu_3/flash_api.cpp:153-155); the attention arithmetic is
// the same as the bf16 decode kernel's (mha_fwd_kvcache.cpp:632-969 in the reference) applied to
// K^ = code * scale[token].
//
// A work unit is (batch row, 64-head half).  The 512-thread workgroup streams its share of the
// unit list (same balanced partition as the bf16 decode kernel): every 32-key chunk is fetched
// once as int8 with 8-byte loads, widened to the 16-bit type on the way into LDS (a code is an
// integer of magnitude <= 127, exact in bf16 and fp16) and shared by the eight waves, which come
// in two kinds, one of each per SIMD:
//   score waves  (0-3): they also stage the cache (loads two chunks ahead, the widening of chunk
//            c+2 interleaved with the products of chunk c+1); wave w owns heads 16w..16w+15 with
//            Q^T resident in registers: S^T = K Q^T over the chunk, per-token scale folded into
//            the scores, online softmax local to the lane column; P, the rescale factor and a
//            "new maximum" flag go to LDS;
//   output waves (4-7): wave w owns a 128-column slice of V for all 64 heads: O^T += V^T P^T, each
//            transposed V operand (rows read whole from the same LDS tile, v_perm in registers)
//            feeding four MFMAs; the V side of the dequantisation is folded into P.
// The kinds run one chunk apart (scores of chunk c+1 beside the output of chunk c), so the
// LDS-heavy score products, the conversions and the output products of one SIMD overlap instead
// of taking turns, with one barrier per chunk.
#include "decode_common.h"

namespace fa {

constexpr int kMlaDqk = 576;
constexpr int kMlaDv = 512;
constexpr int kMlaThreads = 512;
// LDS key rows are unpadded; the 16-byte units of a row are XOR-swizzled with (row & 7) inside
// their aligned groups of eight.  The LDS serves 16-byte reads eight lanes at a time and two
// neighbouring groups of eight lanes overlap in time, so any 16 consecutive lanes (from a
// multiple of 8) must hit 16 different units modulo 256 bytes: rows are 1152 = 4.5 * 256 bytes,
// so odd and even rows sit half a bank cycle apart and the swizzle spreads rows of equal parity.
constexpr int kMlaRowBytes = kMlaDqk * 2;                // 1152
constexpr int kMlaTileBytes = kChunk * kMlaRowBytes;     // 36864
constexpr int kMlaPiecesPerRow = kMlaDqk / 8;            // 72 8-byte int8 pieces per key = 16-byte units once widened
constexpr int kMlaStagers = 256;                         // threads of the score waves
constexpr int kMlaRounds = kChunk * kMlaPiecesPerRow / kMlaStagers;   // 9 pieces per staging thread per chunk
constexpr int kMlaHeadsPerUnit = 64;
static_assert(kChunk * kMlaPiecesPerRow == kMlaRounds * kMlaStagers, "chunk must split evenly over the staging threads");

struct __attribute__((aligned(4))) MlaCodes8 { uint32_t w[2]; };

// 4 signed bytes -> two dwords of 16-bit floats (lo = bytes 0,1 ; hi = bytes 2,3)
template <typename T> __device__ __forceinline__ void widen4(uint32_t w, uint32_t &lo, uint32_t &hi) {
    const float f0 = (float)(int8_t)(w & 0xff);
    const float f1 = (float)(int8_t)((w >> 8) & 0xff);
    const float f2 = (float)(int8_t)((w >> 16) & 0xff);
    const float f3 = (float)(int8_t)(w >> 24);
    lo = pack2<T>(f0, f1);
    hi = pack2<T>(f2, f3);
}

struct MlaShared {
    __attribute__((aligned(16))) uint8_t k[3][kMlaTileBytes];   // widened key tiles: scores, output, being filled
    __attribute__((aligned(16))) float ks[3][kChunk];            // per-token scales, K side
    __attribute__((aligned(16))) float vs[3][kChunk];            // per-token scales, V side
    __attribute__((aligned(16))) float vsi[3][kChunk];           // their inverses (0 for a zero scale)
    __attribute__((aligned(16))) u32x4_t pk[2][4][64];           // P^T operands of the four head groups, two chunks
    float alpha[2][4][16];                                       // accumulator rescale per head
    __attribute__((aligned(4))) uint8_t bump[2][4];              // head group saw a new maximum
    float l[4][16];                                              // final sum per head
};

template <typename T, bool SOFTCAP>
__device__ __forceinline__ void mla_piece(const DecodeParams &p, const int b, const int unit, const UnitRange &ur,
                                          const int range_lo, const int range_hi, const bool write_final,
                                          const int64_t slot, MlaShared &sh) {
    // unit = (query token qi, 64-head group `half`); the chunks walked are those of the whole query
    // block, the keys this token may not see (causal / window bounds of its own row) are masked
    const int qi = unit / p.units_per_token;
    const int half = unit - qi * p.units_per_token;
    const int row_off = ur.Lk - p.seqlen_q + qi;                       // key aligned with this query token
    const int mask_lo = max(range_lo, ur.wl >= 0 ? row_off - ur.wl : 0);
    const int mask_hi = min(range_hi, ur.wr >= 0 ? row_off + ur.wr + 1 : ur.Lk);
    constexpr int KSTEPS = kMlaDqk / 32;   // 18
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int role = wave >> 2;   // 0: scores, 1: output
    const int w4 = wave & 3;      // head group (scores) or 128-column slice (output)
    const int Lk = ur.Lk;

    const int8_t *kc = reinterpret_cast<const int8_t *>(p.k_cache);
    const int32_t *bt_row = p.block_table + (int64_t)b * p.bt_stride_b;
    const int c_begin = range_lo / kChunk;
    const int n = (range_hi + kChunk - 1) / kChunk - c_begin;   // chunks of this piece

    // Step j of a piece (j = 0 .. n + 1): chunk j is widened into tile j % 3 and chunk j + 2 loaded;
    // the score waves work on chunk j - 1 (tile (j + 2) % 3), the output waves on chunk j - 2
    // (tile (j + 1) % 3); one barrier ends the step.
    if (role == 0) {
        // =========================== score waves ===========================================
        const int lane0 = tid & 63;
        const int head = half * kMlaHeadsPerUnit + w4 * 16 + (lane0 & 15);   // head of this lane column
        // Q^T operand: lane (lq, ln) holds head `head` of query token qi, elements t*32 + lq*8 .. +7
        u32x4_t qreg[KSTEPS];
        {
            const uint16_t *src = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_stride_b +
                                  (int64_t)qi * p.q_stride_s + (int64_t)head * p.q_stride_h + (lane0 >> 4) * 8;
#pragma unroll
            for (int t = 0; t < KSTEPS; ++t) qreg[t] = load16(src + t * 32);
        }
        // ---- staging: int8 rows -> registers -> widened LDS tile.  Chunk j of the piece is loaded
        //      into register set j & 1 two steps before it is widened.  Thread -> (key row, 8-byte
        //      column): 8 threads per row, nine pieces 64 bytes apart each, so one address per chunk
        //      serves all loads and one LDS address all stores (the swizzle stays inside a group of
        //      eight units, the pieces of a thread are eight units apart).  Past the end of the piece the last
        //      chunk is named again: every step issues the same loads, so the compiler counts the
        //      loads in flight instead of waiting for all of them.  Page ids are loaded one step
        //      before the tile loads that use them and ahead of that step's tile loads, so waiting
        //      for a page id never waits for younger tile loads.  The thread index comes in as an
        //      argument: the step loop passes a copy the compiler cannot see through, so the few
        //      address terms are recomputed per chunk instead of held in registers.
        static_assert(kMlaStagers / 8 == kChunk && kMlaRounds * 8 == kMlaPiecesPerRow, "thread map of the staging");
        MlaCodes8 st[2][kMlaRounds];
        float st_ks[2] = {0.f, 0.f}, st_vs[2] = {0.f, 0.f};
        auto fetch_blk = [&](int j) -> int {
            int page = ((c_begin + min(j, n - 1)) * kChunk) / p.page_size;
            page = min(page, p.max_blocks - 1);
            return min(max(bt_row[page], 0), p.num_blocks - 1);
        };
        auto fetch = [&](int j_any, int blk, int set, int th) {
            const int j = min(j_any, n - 1);
            const int t_row = th >> 3;
            const int t_sub = th & 7;
            const int key0 = (c_begin + j) * kChunk;
            const int inpage0 = key0 % p.page_size;
            const int last = Lk - 1 - key0;
            // wave-uniform 64-bit base + 32-bit per-thread offset
            const int8_t *src = kc + (int64_t)blk * p.k_stride_block + (int64_t)inpage0 * p.k_stride_row;
            const uint32_t voff = (uint32_t)min(t_row, last) * (uint32_t)p.k_stride_row + t_sub * 8;
#pragma unroll
            for (int i = 0; i < kMlaRounds; ++i) st[set][i] = *reinterpret_cast<const MlaCodes8 *>(src + voff + i * 64);
            const int64_t so = (int64_t)blk * p.ks_stride_block + (int64_t)inpage0 * p.ks_stride_row;
            const uint32_t soff = (uint32_t)min(th & (kChunk - 1), last) * (uint32_t)p.ks_stride_row;
            st_ks[set] = (p.k_scale + so)[soff];
            st_vs[set] = (p.v_scale + so)[soff];
        };
        // piece i (0..8) of the staged chunk: eight codes -> eight 16-bit floats -> one LDS unit
        auto widen_piece = [&](int tile, int set, int th, int i) {
            const int row = th >> 3;
            uint8_t *dst = &sh.k[tile][row * kMlaRowBytes + (((th & 7) ^ (row & 7)) << 4)];
            u32x4_t w;
            uint32_t lo, hi;
            widen4<T>(st[set][i].w[0], lo, hi);
            w[0] = lo, w[1] = hi;
            widen4<T>(st[set][i].w[1], lo, hi);
            w[2] = lo, w[3] = hi;
            *reinterpret_cast<u32x4_t *>(dst + i * 128) = w;
        };
        auto stash_scales = [&](int tile, int set, int th) {
            if (th < kChunk) {
                sh.ks[tile][th] = st_ks[set];
                sh.vs[tile][th] = st_vs[set];
                sh.vsi[tile][th] = (st_vs[set] > 0.f) ? 1.f / st_vs[set] : 0.f;
            }
        };
        int blk_next;
        {
            const int b0 = fetch_blk(0), b1 = fetch_blk(1);
            blk_next = fetch_blk(2);
            fetch(0, b0, 0, tid);
            fetch(1, b1, 1, tid);
        }
        float m_run = -INFINITY, l_run = 0.f, l_norm = 0.f;

        auto score_step = [&](const int j, const int set, const int tile_j) {
            int th = tid;
            asm volatile("" : "+v"(th));
            const int lane = th & 63;
            const int lq = lane >> 4;
            const int ln = lane & 15;
            const bool do_stash = j < n;
            const bool do_score = j >= 1 && j <= n;
            const int tile = (tile_j == 0) ? 2 : tile_j - 1;   // (j + 2) % 3: tile of the scores
            float4_t s[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
            // per-token scales of the score chunk, read ahead of the products
            float4 ks4[2], vs4[2], vi4[2];
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                ks4[tt] = *reinterpret_cast<const float4 *>(&sh.ks[tile][tt * 16 + lq * 4]);
                vs4[tt] = *reinterpret_cast<const float4 *>(&sh.vs[tile][tt * 16 + lq * 4]);
                vi4[tt] = *reinterpret_cast<const float4 *>(&sh.vsi[tile][tt * 16 + lq * 4]);
            }
            if (do_score) {
                // ---- S^T = K Q^T : two 16-key tiles x this wave's 16 heads; operand reads run kPf
                //      k-steps ahead of the MFMAs that use them; one piece of the next-but-one chunk
                //      is widened beside every other k-step (in the last score step that is the last chunk
                //      once more, into a tile nobody reads: no branch inside the product loop)
                constexpr int kPf = 8;
                u32x4_t ka[KSTEPS][2];
                // unit 4t + lq of rows ln and 16 + ln (same row & 7), swizzled: two lane offsets by parity of t
                const uint8_t *k_rd = &sh.k[tile][ln * kMlaRowBytes];
                const int k_off[2] = {(lq ^ (ln & 7)) << 4, ((4 + lq) ^ (ln & 7)) << 4};
                auto read_k = [&](int t) {
                    ka[t][0] = *reinterpret_cast<const u32x4_t *>(k_rd + k_off[t & 1] + (t >> 1) * 128);
                    ka[t][1] = *reinterpret_cast<const u32x4_t *>(k_rd + 16 * kMlaRowBytes + k_off[t & 1] + (t >> 1) * 128);
                };
#pragma unroll
                for (int t = 0; t < kPf; ++t) read_k(t);
#pragma unroll
                for (int t = 0; t < KSTEPS; ++t) {
                    if (t + kPf < KSTEPS) read_k(t + kPf);
                    s[0] = mfma16<T>(ka[t][0], qreg[t], s[0]);
                    if (t & 1) widen_piece(tile_j, set, th, t >> 1);
                    s[1] = mfma16<T>(ka[t][1], qreg[t], s[1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else if (do_stash) {
#pragma unroll
                for (int i = 0; i < kMlaRounds; ++i) widen_piece(tile_j, set, th, i);
            }
            if (do_stash) stash_scales(tile_j, set, th);
            {
                const int blk_after = fetch_blk(j + 3);
                fetch(j + 2, blk_next, set, th);
                blk_next = blk_after;
            }
            __builtin_amdgcn_sched_barrier(0);
            if (do_score) {
                const int c = c_begin + j - 1;
                const int pb = set ^ 1;                              // (j - 1) & 1
                // ---- softmax; register i of tile tt is key c*32 + tt*16 + lq*4 + i
                const int key_base = c * kChunk + lq * 4;
                float x[8], vsc[8], vin[8];
                float mloc = -INFINITY;
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    const float ksv[4] = {ks4[tt].x, ks4[tt].y, ks4[tt].z, ks4[tt].w};
                    const float vsv[4] = {vs4[tt].x, vs4[tt].y, vs4[tt].z, vs4[tt].w};
                    const float viv[4] = {vi4[tt].x, vi4[tt].y, vi4[tt].z, vi4[tt].w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int key = key_base + tt * 16 + i;
                        float v = s[tt][i] * ksv[i];
                        if constexpr (SOFTCAP) {
                            const float e2 = __expf(2.f * v * p.softcap_pre);
                            v = p.softcap_post * (1.f - 2.f / (e2 + 1.f));
                        } else {
                            v *= p.scale_log2;
                        }
                        v = (key >= mask_lo && key < mask_hi) ? v : -INFINITY;
                        x[tt * 4 + i] = v;
                        vsc[tt * 4 + i] = vsv[i];
                        vin[tt * 4 + i] = viv[i];
                        mloc = fmaxf(mloc, v);
                    }
                }
                mloc = quad_rows_max(mloc);
                const bool bump = mloc > m_run;
                const float m_new = bump ? mloc : m_run;
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = bump ? fast_exp2(m_run - m_use) : 1.f;
                m_run = m_new;
                float psum = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float pe = fast_exp2(x[e] - m_use);
                    psum += pe;
                    x[e] = pe * vsc[e];   // V side of the dequantisation folded into P
                }
                l_run = l_run * alpha + psum;
                u32x4_t pk;
                pk[0] = pack2<T>(x[0], x[1]);
                pk[1] = pack2<T>(x[2], x[3]);
                pk[2] = pack2<T>(x[4], x[5]);
                pk[3] = pack2<T>(x[6], x[7]);
                // The weight a key really gets is round16(P * v_scale) / v_scale = P (1 + eps), |eps| <= 2^-8 (bf16).
                // The output is divided by the sum of THOSE weights, so that it stays a convex combination of
                // the dequantised values (a row that sees one key returns that key exactly); the LSE keeps the
                // sum of the unrounded P.
                float pcorr = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint32_t w = pk[e >> 1];
                    const float xr = to_float<T>((uint16_t)((e & 1) ? (w >> 16) : (w & 0xffffu)));
                    pcorr = __builtin_fmaf(xr - x[e], vin[e], pcorr);
                }
                l_norm = l_norm * alpha + (psum + pcorr);
                sh.pk[pb][w4][lane] = pk;
                if (lq == 0) sh.alpha[pb][w4][ln] = alpha;
                const int wave_bump = __any(bump) ? 1 : 0;
                if (lane == 0) sh.bump[pb][w4] = (uint8_t)wave_bump;
            }
            __syncthreads();
        };
        int tile_j = 0;
        for (int j = 0; j <= n + 1; j += 2) {
            score_step(j, 0, tile_j);
            tile_j = (tile_j == 2) ? 0 : tile_j + 1;
            if (j + 1 <= n + 1) {
                score_step(j + 1, 1, tile_j);
                tile_j = (tile_j == 2) ? 0 : tile_j + 1;
            }
        }

        // ---- publish the sums, write the LSE
        l_run = quad_rows_sum(l_run);
        l_norm = quad_rows_sum(l_norm);
        const int lane = tid & 63;
        const int ln = lane & 15;
        if ((lane >> 4) == 0) {
            sh.l[w4][ln] = (l_run > 0.f) ? l_norm : 0.f;
            const int row = w4 * 16 + ln;
            if (write_final)
                p.lse[((int64_t)b * p.nheads + head) * p.seqlen_q + qi] = (l_run > 0.f) ? (m_run + fast_log2(l_run)) * kLn2 : INFINITY;
            else
                p.lse_partial[slot * p.rows + row] = (l_run > 0.f) ? m_run + fast_log2(l_run) : -INFINITY;
        }
        __syncthreads();
    } else {
        // =========================== output waves ==========================================
        // o_acc[hg][t]: head group hg (16 heads), column tile t of this wave's 128-column slice
        float4_t o_acc[4][8];
#pragma unroll
        for (int hg = 0; hg < 4; ++hg)
#pragma unroll
            for (int t = 0; t < 8; ++t) o_acc[hg][t] = float4_t{0.f, 0.f, 0.f, 0.f};

        auto output_step = [&](const int j, const int set, const int tile_j) {
            int th = tid;
            asm volatile("" : "+v"(th));
            const int lane = th & 63;
            const int lq = lane >> 4;
            const int ln = lane & 15;
            if (j >= 2) {
                const int tile = (tile_j == 2) ? 0 : tile_j + 1;   // (j + 1) % 3
                const int pb = set;                                  // (j - 2) & 1
                // ---- O^T += V^T P^T on this wave's 128-column slice, all four head groups.
                //      k slot 8*lq + e of the MFMA is key (e >> 2) * 16 + lq * 4 + (e & 3) of the chunk.
                //      The V^T operands come from the transposing LDS read (ds_read_b64_tr_b16): in a
                //      16-lane group, lane s points at 4 columns (4*(s%4)..) of key row s/4 and receives
                //      column s of the group's 16 for its 4 key rows.  Column tile ct = columns ct*16..+15
                //      of the slice; the 16-byte unit of a row is swizzled with row & 7 = 4*(lq&1) + ln/4.
                typedef short v4s_t __attribute__((ext_vector_type(4)));
                const int tr_row = lq * 4 + (ln >> 2);
                const int tr_k = 4 * (lq & 1) + (ln >> 2);
                const uint8_t *tr_base = &sh.k[tile][tr_row * kMlaRowBytes + w4 * 256 + 8 * (ln & 1)];
                int tr_off[4];   // unit (2*(ct&3) + (ln&3)/2) ^ tr_k inside its aligned group of eight
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) tr_off[c4] = ((2 * c4 + ((ln & 3) >> 1)) ^ tr_k) << 4;
                u32x4_t pkg[4];
                const uint32_t bumps = *reinterpret_cast<const uint32_t *>(sh.bump[pb]);
#pragma unroll
                for (int hg = 0; hg < 4; ++hg) {
                    pkg[hg] = sh.pk[pb][hg][lane];
                    if ((bumps >> (8 * hg)) & 0xffu) {
                        const float ag = sh.alpha[pb][hg][ln];
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            o_acc[hg][t][0] *= ag;
                            o_acc[hg][t][1] *= ag;
                            o_acc[hg][t][2] *= ag;
                            o_acc[hg][t][3] *= ag;
                        }
                    }
                }
#pragma unroll
                for (int ct = 0; ct < 8; ++ct) {
                    u32x4_t va;
#pragma unroll
                    for (int hv = 0; hv < 2; ++hv) {
                        const v4s_t r4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) v4s_t *)(tr_base + hv * 16 * kMlaRowBytes + (ct >> 2) * 128 + tr_off[ct & 3]));
                        const uint2 r2 = __builtin_bit_cast(uint2, r4);
                        va[2 * hv] = r2.x;
                        va[2 * hv + 1] = r2.y;
                    }
#pragma unroll
                    for (int hg = 0; hg < 4; ++hg) o_acc[hg][ct] = mfma16<T>(va, pkg[hg], o_acc[hg][ct]);
                }
            }
            __syncthreads();
        };
        int tile_j = 0;
        for (int j = 0; j <= n + 1; j += 2) {
            output_step(j, 0, tile_j);
            tile_j = (tile_j == 2) ? 0 : tile_j + 1;
            if (j + 1 <= n + 1) {
                output_step(j + 1, 1, tile_j);
                tile_j = (tile_j == 2) ? 0 : tile_j + 1;
            }
        }

        // ---- write the column slice: register i of tile t of group hg is column
        //      w4*128 + t*16 + lq*4 + i of head hg*16 + ln
        __syncthreads();   // sums of all heads are in LDS
        const int lane = tid & 63;
        const int lq = lane >> 4;
        const int ln = lane & 15;
#pragma unroll
        for (int hg = 0; hg < 4; ++hg) {
            const int row = hg * 16 + ln;   // row of the unit (0..63)
            const int hd = half * kMlaHeadsPerUnit + row;
            const float lg = sh.l[hg][ln];
            const float inv = (lg > 0.f) ? 1.f / lg : 0.f;
            if (write_final) {
                uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                                (int64_t)hd * p.o_stride_h + w4 * 128;
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const uint2 o2 = make_uint2(pack2<T>(o_acc[hg][t][0] * inv, o_acc[hg][t][1] * inv),
                                                pack2<T>(o_acc[hg][t][2] * inv, o_acc[hg][t][3] * inv));
                    *reinterpret_cast<uint2 *>(dst + t * 16 + lq * 4) = o2;
                }
            } else {
                const int64_t srow = slot * p.rows + row;
                float *dst = p.o_partial + srow * kMlaDv + w4 * 128;
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    *reinterpret_cast<float4 *>(dst + t * 16 + lq * 4) =
                        make_float4(o_acc[hg][t][0] * inv, o_acc[hg][t][1] * inv, o_acc[hg][t][2] * inv, o_acc[hg][t][3] * inv);
            }
        }
    }
    __syncthreads();   // the LDS tiles and sums are reused by the next piece
}

template <typename T, bool SOFTCAP>
__global__ void __launch_bounds__(kMlaThreads) decode_mla_i8_kernel(const DecodeParams p) {
    __shared__ MlaShared sh;
    balanced_driver<kMlaDv>(p, [&](int b, int unit, const UnitRange &ur, int range_lo, int range_hi, bool whole, int64_t slot) {
        mla_piece<T, SOFTCAP>(p, b, unit, ur, range_lo, range_hi, whole, slot, sh);
    });
}

// p.nheads_k counts units per batch row here (seqlen_q * 64-head groups), p.group = p.rows = 64.
hipError_t launch_decode_mla_i8(const DecodeParams &p, int dtype, hipStream_t stream) {
    if (p.units_per_token <= 0 || p.rows != kMlaHeadsPerUnit || p.group != kMlaHeadsPerUnit || !p.balanced)
        return hipErrorInvalidValue;
    dim3 grid(p.num_wgs), block(kMlaThreads);
    const bool softcap = p.softcap_post != 0.f;
    if (dtype == 0) {
        if (softcap)
            hipLaunchKernelGGL((decode_mla_i8_kernel<BF16, true>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((decode_mla_i8_kernel<BF16, false>), grid, block, 0, stream, p);
    } else {
        if (softcap)
            hipLaunchKernelGGL((decode_mla_i8_kernel<FP16, true>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((decode_mla_i8_kernel<FP16, false>), grid, block, 0, stream, p);
    }
    return hipGetLastError();
}

}  // namespace fa
