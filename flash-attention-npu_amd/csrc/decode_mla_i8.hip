// Latent-attention (MLA) decode over an int8 paged cache with per-token fp32 scales, gfx950.
//
// Layout: one latent kv head, 576 key dims, V = the first 512 of them (v_cache aliases k_cache);
// 128 q heads (any multiple of 64), seqlen_q = 1.  The reference has no quantised path
// (dtypes are limited to fp16/bf16 at csrc/ascend910/flash_attn_npu/flash_api.cpp:386-388 and
// descales are rejected at flash_attn_npu_3/flash_api.cpp:153-155); the attention arithmetic is
// the same as the bf16 decode kernel's (mha_fwd_kvcache.cpp:632-969 in the reference) applied to
// K^ = code * scale[token].
//
// A work unit is (batch row, 64-head half).  The 256-thread workgroup streams its share of the
// unit list (same balanced partition as the bf16 decode kernel): every 32-key chunk is fetched
// once as int8 with 16-byte loads, widened to the 16-bit type on the way into LDS (a code is an
// integer of magnitude <= 127, exact in bf16 and fp16) and shared by the four waves, each of
// which owns 16 heads for the scores: S^T = K Q^T with Q^T resident in registers, per-token scale
// folded into the scores (K side) and into P (V side).  For O^T += V^T P^T the waves trade places:
// P of all 64 heads goes through LDS and every wave owns a 128-column slice of V for all heads,
// so each transposed V operand (rows read whole from the same LDS tile, v_perm in registers)
// feeds four MFMAs and is read from LDS once per workgroup instead of once per wave.
#include "decode_common.h"

namespace fa {

constexpr int kMlaDqk = 576;
constexpr int kMlaDv = 512;
constexpr int kMlaRowBytes = kMlaDqk * 2 + 16;           // padded LDS row: conflict-free operand reads
constexpr int kMlaTileBytes = kChunk * kMlaRowBytes;     // 37376
constexpr int kMlaPiecesPerRow = kMlaDqk / 16;           // 36 16-byte int8 pieces per key
constexpr int kMlaPieces = kChunk * kMlaPiecesPerRow;    // 1152 per chunk
constexpr int kMlaRounds = (kMlaPieces + 255) / 256;     // 5 (last one half full)
constexpr int kMlaHeadsPerUnit = 64;

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
    __attribute__((aligned(16))) uint8_t k[2][kMlaTileBytes];   // widened key tiles
    __attribute__((aligned(16))) float ks[2][kChunk];            // per-token scales, K side
    __attribute__((aligned(16))) float vs[2][kChunk];            // per-token scales, V side
    __attribute__((aligned(16))) u32x4_t pk[4][64];              // P^T operands of the four head groups
    float alpha[kMlaHeadsPerUnit];                               // accumulator rescale per head
    float m[kMlaHeadsPerUnit], l[kMlaHeadsPerUnit];              // final max / sum per head
    int bump[4];                                                 // head group saw a new maximum
};

template <typename T>
__device__ __forceinline__ void mla_piece(const DecodeParams &p, const int b, const int half, const UnitRange &ur,
                                          const int range_lo, const int range_hi, const bool write_final,
                                          const int64_t slot, MlaShared &sh) {
    constexpr int KSTEPS = kMlaDqk / 32;   // 18
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane >> 4;
    const int ln = lane & 15;
    const int head = half * kMlaHeadsPerUnit + wave * 16 + ln;   // query head whose scores this lane column holds
    const int Lk = ur.Lk;

    // Q^T operand (seqlen_q == 1): lane (lq, ln) holds head `head`, elements t*32 + lq*8 .. +7
    u32x4_t qreg[KSTEPS];
    {
        const uint16_t *src = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_stride_b +
                              (int64_t)head * p.q_stride_h + lq * 8;
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t) qreg[t] = load16(src + t * 32);
    }

    float m_run = -INFINITY, l_run = 0.f;
    // o_acc[g][t]: head group g (16 heads), column tile t of this wave's 128-column slice
    float4_t o_acc[4][8];
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int t = 0; t < 8; ++t) o_acc[g][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int8_t *kc = reinterpret_cast<const int8_t *>(p.k_cache);
    const int32_t *bt_row = p.block_table + (int64_t)b * p.bt_stride_b;
    const int c_begin = range_lo / kChunk;
    const int c_end = (range_hi + kChunk - 1) / kChunk;

    // ---- staging: int8 rows -> registers -> widened LDS tile --------------------------------
    u32x4_t st[kMlaRounds];
    float st_ks = 0.f, st_vs = 0.f;
    // page id of chunk c, fetched one chunk before the loads that need it
    auto fetch_blk = [&](int c) -> int {
        if (c >= c_end) return 0;
        int page = (c * kChunk) / p.page_size;
        page = min(page, p.max_blocks - 1);
        return min(max(bt_row[page], 0), p.num_blocks - 1);
    };
    auto fetch = [&](int c, int blk) {
        const int key0 = c * kChunk;
        const int inpage0 = key0 % p.page_size;
        const int last = Lk - 1 - key0;
        const int8_t *base = kc + (int64_t)blk * p.k_stride_block;
#pragma unroll
        for (int i = 0; i < kMlaRounds; ++i) {
            const int piece = tid + 256 * i;
            if (piece < kMlaPieces) {
                const int row = min(piece / kMlaPiecesPerRow, last);
                const int c16 = piece % kMlaPiecesPerRow;
                st[i] = load16(base + (int64_t)(inpage0 + row) * p.k_stride_row + c16 * 16);
            }
        }
        if (tid < kChunk) {
            const int row = min(tid, last);
            const int64_t so = (int64_t)blk * p.ks_stride_block + (int64_t)(inpage0 + row) * p.ks_stride_row;
            st_ks = p.k_scale[so];
            st_vs = p.v_scale[so];
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kMlaRounds; ++i) {
            const int piece = tid + 256 * i;
            if (piece < kMlaPieces) {
                const int row = piece / kMlaPiecesPerRow;
                const int c16 = piece % kMlaPiecesPerRow;
                uint32_t w[8];
                widen4<T>(st[i][0], w[0], w[1]);
                widen4<T>(st[i][1], w[2], w[3]);
                widen4<T>(st[i][2], w[4], w[5]);
                widen4<T>(st[i][3], w[6], w[7]);
                const u32x4_t a = {w[0], w[1], w[2], w[3]};
                const u32x4_t bq = {w[4], w[5], w[6], w[7]};
                uint8_t *dst = &sh.k[buf][row * kMlaRowBytes + c16 * 32];
                *reinterpret_cast<u32x4_t *>(dst) = a;
                *reinterpret_cast<u32x4_t *>(dst + 16) = bq;
            }
        }
        if (tid < kChunk) {
            sh.ks[buf][tid] = st_ks;
            sh.vs[buf][tid] = st_vs;
        }
    };

    int blk_next = fetch_blk(c_begin);
    if (c_begin < c_end) {
        fetch(c_begin, blk_next);
        blk_next = fetch_blk(c_begin + 1);
        stash(0);
    }
    __syncthreads();

    int cur = 0;
    for (int c = c_begin; c < c_end; ++c) {
        const bool more = c + 1 < c_end;
        if (more) fetch(c + 1, blk_next);
        blk_next = fetch_blk(c + 2);
        __builtin_amdgcn_sched_barrier(0);

        // ---- S^T = K Q^T : two 16-key tiles x this wave's 16 heads
        // operand reads run kPf k-steps ahead of the MFMAs that use them (one wave per SIMD here:
        // nothing else hides the LDS latency)
        constexpr int kPf = 4;
        float4_t s[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
        u32x4_t ka[KSTEPS][2];
        auto read_k = [&](int t) {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
                ka[t][tt] = *reinterpret_cast<const u32x4_t *>(&sh.k[cur][(tt * 16 + ln) * kMlaRowBytes + (t * 4 + lq) * 16]);
        };
#pragma unroll
        for (int t = 0; t < kPf; ++t) read_k(t);
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t) {
            if (t + kPf < KSTEPS) read_k(t + kPf);
            s[0] = mfma16<T>(ka[t][0], qreg[t], s[0]);
            s[1] = mfma16<T>(ka[t][1], qreg[t], s[1]);
            __builtin_amdgcn_sched_barrier(0);
        }

        // ---- softmax of this wave's heads; register i of tile tt is key c*32 + tt*16 + lq*4 + i
        const int key_base = c * kChunk + lq * 4;
        float x[8], vs[8];
        float mloc = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            const float4 ks4 = *reinterpret_cast<const float4 *>(&sh.ks[cur][tt * 16 + lq * 4]);
            const float4 vs4 = *reinterpret_cast<const float4 *>(&sh.vs[cur][tt * 16 + lq * 4]);
            const float ksv[4] = {ks4.x, ks4.y, ks4.z, ks4.w};
            const float vsv[4] = {vs4.x, vs4.y, vs4.z, vs4.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = key_base + tt * 16 + i;
                float v = s[tt][i] * ksv[i] * p.scale_log2;
                v = (key >= range_lo && key < range_hi) ? v : -INFINITY;
                x[tt * 4 + i] = v;
                vs[tt * 4 + i] = vsv[i];
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
            x[e] = pe * vs[e];   // V side of the dequantisation folded into P
        }
        l_run = l_run * alpha + psum;
        u32x4_t pk;
        pk[0] = pack2<T>(x[0], x[1]);
        pk[1] = pack2<T>(x[2], x[3]);
        pk[2] = pack2<T>(x[4], x[5]);
        pk[3] = pack2<T>(x[6], x[7]);
        sh.pk[wave][lane] = pk;
        if (lq == 0) sh.alpha[wave * 16 + ln] = alpha;
        const int wave_bump = __any(bump) ? 1 : 0;
        if (lane == 0) sh.bump[wave] = wave_bump;
        __syncthreads();   // P, alpha of all 64 heads are in LDS

        // ---- O^T += V^T P^T on this wave's 128-column slice, all four head groups
        u32x4_t pkg[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            pkg[g] = sh.pk[g][lane];
            if (sh.bump[g]) {
                const float ag = sh.alpha[g * 16 + ln];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    o_acc[g][t][0] *= ag;
                    o_acc[g][t][1] *= ag;
                    o_acc[g][t][2] *= ag;
                    o_acc[g][t][3] *= ag;
                }
            }
        }
        u32x4_t vr[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int row = (e >> 2) * 16 + lq * 4 + (e & 3);
            vr[e] = *reinterpret_cast<const u32x4_t *>(&sh.k[cur][row * kMlaRowBytes + (wave * 128 + ln * 8) * 2]);
        }
#pragma unroll
        for (int w2 = 0; w2 < 4; ++w2) {
            u32x4_t a_lo, a_hi;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                a_lo[u] = __builtin_amdgcn_perm(vr[2 * u + 1][w2], vr[2 * u][w2], 0x05040100u);
                a_hi[u] = __builtin_amdgcn_perm(vr[2 * u + 1][w2], vr[2 * u][w2], 0x07060302u);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                o_acc[g][2 * w2] = mfma16<T>(a_lo, pkg[g], o_acc[g][2 * w2]);
                o_acc[g][2 * w2 + 1] = mfma16<T>(a_hi, pkg[g], o_acc[g][2 * w2 + 1]);
            }
        }

        // keep the widening of the prefetched tile behind the products: it waits for the loads
        __builtin_amdgcn_sched_barrier(0);
        if (more) stash(cur ^ 1);
        __syncthreads();   // next tile staged; P buffer free again
        cur ^= 1;
    }

    // ---- write.  The score-owning waves publish max and sum; every wave then stores its column
    //      slice: register i of tile t of group g is column wave*128 + (lq*4 + i)*8 + t of head g*16 + ln.
    l_run = quad_rows_sum(l_run);
    if (lq == 0) {
        sh.m[wave * 16 + ln] = m_run;
        sh.l[wave * 16 + ln] = l_run;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int row = g * 16 + ln;   // row of the unit (0..63)
        const int hd = half * kMlaHeadsPerUnit + row;
        const float lg = sh.l[row];
        const float inv = (lg > 0.f) ? 1.f / lg : 0.f;
        if (write_final) {
            uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)hd * p.o_stride_h +
                            wave * 128;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                u32x4_t o4;
#pragma unroll
                for (int u = 0; u < 4; ++u) o4[u] = pack2<T>(o_acc[g][2 * u][i] * inv, o_acc[g][2 * u + 1][i] * inv);
                store16(dst + (lq * 4 + i) * 8, o4);
            }
        } else {
            const int64_t srow = slot * p.rows + row;
            float *dst = p.o_partial + srow * kMlaDv + wave * 128;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float *d2 = dst + (lq * 4 + i) * 8;
                *reinterpret_cast<float4 *>(d2) = make_float4(o_acc[g][0][i] * inv, o_acc[g][1][i] * inv, o_acc[g][2][i] * inv,
                                                              o_acc[g][3][i] * inv);
                *reinterpret_cast<float4 *>(d2 + 4) = make_float4(o_acc[g][4][i] * inv, o_acc[g][5][i] * inv,
                                                                  o_acc[g][6][i] * inv, o_acc[g][7][i] * inv);
            }
        }
    }
    if (lq == 0) {
        // this lane column's own head: LSE (final) or partial LSE
        const int row = wave * 16 + ln;
        if (write_final)
            p.lse[(int64_t)b * p.nheads + head] = (l_run > 0.f) ? (m_run + fast_log2(l_run)) * kLn2 : INFINITY;
        else
            p.lse_partial[slot * p.rows + row] = (l_run > 0.f) ? m_run + fast_log2(l_run) : -INFINITY;
    }
    __syncthreads();   // the LDS tiles are reused by the next piece
}

template <typename T> __global__ void __launch_bounds__(256, 1) decode_mla_i8_kernel(const DecodeParams p) {
    __shared__ MlaShared sh;
    balanced_driver<kMlaDv>(p, [&](int b, int half, const UnitRange &ur, int range_lo, int range_hi, bool whole, int64_t slot) {
        mla_piece<T>(p, b, half, ur, range_lo, range_hi, whole, slot, sh);
    });
}

// p.nheads_k counts 64-head halves here (units per batch row), p.group = p.rows = 64.
hipError_t launch_decode_mla_i8(const DecodeParams &p, int dtype, hipStream_t stream) {
    if (p.seqlen_q != 1 || p.rows != kMlaHeadsPerUnit || p.group != kMlaHeadsPerUnit || !p.balanced)
        return hipErrorInvalidValue;
    dim3 grid(p.num_wgs), block(256);
    if (dtype == 0)
        hipLaunchKernelGGL(decode_mla_i8_kernel<BF16>, grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL(decode_mla_i8_kernel<FP16>, grid, block, 0, stream, p);
    return hipGetLastError();
}

}  // namespace fa
