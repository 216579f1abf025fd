// Latent-attention (MLA) decode over an int8 paged cache with per-token fp32 scales, gfx950.
//
// Layout: one latent kv head, 576 key dims, V = the first 512 of them (v_cache aliases k_cache);
// 128 q heads (any multiple of 64), seqlen_q = 1.  The reference has no quantised path
// (dtypes are limited to fp16/bf16 at csrc/ascend910/flash_attn_npu/flash_api.cpp:386-388 and
// descales are rejected at flash_attn_npu_3/flash_api.cpp:153-155); the attention arithmetic is
// the same as the bf16 decode kernel's (mha_fwd_kvcache.cpp:632-969 in the reference) applied to
// K^ = code * scale[token].
//
// A work unit is (batch row, 64-head half).  The 512-thread workgroup (two waves per SIMD, so one
// wave's matrix products cover the other's conversions and LDS waits) streams its share of the
// unit list (same balanced partition as the bf16 decode kernel): every 32-key chunk is fetched
// once as int8 with 12-byte loads, widened to the 16-bit type on the way into LDS (a code is an
// integer of magnitude <= 127, exact in bf16 and fp16) and shared by the eight waves.
//   scores : wave (g, t) owns head group g (16 heads, Q^T resident in registers) and the 16-key
//            tile t of the chunk: S^T = K Q^T, per-token scale folded into the scores; the chunk
//            maximum of a head group is exchanged between its two waves through LDS;
//   output : the waves trade places: P of all 64 heads goes through LDS and every wave owns a
//            64-column slice of V for all heads, so each transposed V operand (rows read whole
//            from the same LDS tile, v_perm in registers) feeds four MFMAs; the V side of the
//            dequantisation is folded into P.
// Two barriers per chunk; the widening of the next chunk sits between them.
#include "decode_common.h"

namespace fa {

constexpr int kMlaDqk = 576;
constexpr int kMlaDv = 512;
constexpr int kMlaThreads = 512;
constexpr int kMlaRowBytes = kMlaDqk * 2 + 16;           // padded LDS row: conflict-free operand reads
constexpr int kMlaTileBytes = kChunk * kMlaRowBytes;     // 37376
constexpr int kMlaPiecesPerRow = kMlaDqk / 12;           // 48 12-byte int8 pieces per key
constexpr int kMlaRounds = kChunk * kMlaPiecesPerRow / kMlaThreads;   // 3 pieces per thread per chunk
constexpr int kMlaHeadsPerUnit = 64;
static_assert(kChunk * kMlaPiecesPerRow == kMlaRounds * kMlaThreads, "chunk must split evenly over the threads");

struct __attribute__((aligned(4))) MlaCodes12 { uint32_t w[3]; };

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
    __attribute__((aligned(16))) uint2 pk[4][64][2];             // P^T operands of the four head groups, by key tile
    // per head, indexed [head group][head in group] so the group is a constant address offset
    float mx[2][4][16];                                          // chunk maximum per key tile
    float alpha[4][16];                                          // accumulator rescale
    float m[4][16], l[2][4][16];                                 // final max, sum per key tile
    __attribute__((aligned(4))) uint8_t bump[4];                 // head group saw a new maximum
};

template <typename T>
__device__ __forceinline__ void mla_piece(const DecodeParams &p, const int b, const int half, const UnitRange &ur,
                                          const int range_lo, const int range_hi, const bool write_final,
                                          const int64_t slot, MlaShared &sh) {
    constexpr int KSTEPS = kMlaDqk / 32;   // 18
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = wave & 3;    // head group of the score phase
    const int kt = wave >> 2;  // 16-key tile of the score phase
    const int lq = lane >> 4;
    const int ln = lane & 15;
    const int head = half * kMlaHeadsPerUnit + g * 16 + ln;   // query head whose scores this lane column holds
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
    // o_acc[hg][t]: head group hg (16 heads), column tile t of this wave's 64-column slice
    float4_t o_acc[4][4];
#pragma unroll
    for (int hg = 0; hg < 4; ++hg)
#pragma unroll
        for (int t = 0; t < 4; ++t) o_acc[hg][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int8_t *kc = reinterpret_cast<const int8_t *>(p.k_cache);
    const int32_t *bt_row = p.block_table + (int64_t)b * p.bt_stride_b;
    const int c_begin = range_lo / kChunk;
    const int c_end = (range_hi + kChunk - 1) / kChunk;

    // ---- staging: int8 rows -> registers -> widened LDS tile.  Loads run two chunks ahead of the
    //      products (register sets st[0], st[1] by chunk parity within the piece): one chunk of
    //      arithmetic is shorter than a trip to memory.
    MlaCodes12 st[2][kMlaRounds];
    float st_ks[2] = {0.f, 0.f}, st_vs[2] = {0.f, 0.f};
    auto fetch_blk = [&](int c) -> int {
        if (c >= c_end) return 0;
        int page = (c * kChunk) / p.page_size;
        page = min(page, p.max_blocks - 1);
        return min(max(bt_row[page], 0), p.num_blocks - 1);
    };
    // thread -> (key row, 12-byte column) of the chunk: 16 threads per row, three pieces 192 bytes
    // apart each, so one address per chunk serves all three loads and one LDS address all stores
    static_assert(kMlaThreads / 16 == kChunk && kMlaRounds * 16 == kMlaPiecesPerRow, "thread map of the staging");
    // (the thread index comes in as an argument: the chunk loop passes a copy the compiler cannot
    //  see through, so these few address terms are recomputed per chunk instead of held in registers)
    auto fetch = [&](int c, int blk, int set, int th) {
        const int t_row = th >> 4;
        const int t_sub = th & 15;
        const int key0 = c * kChunk;
        const int inpage0 = key0 % p.page_size;
        const int last = Lk - 1 - key0;
        // wave-uniform 64-bit base + 32-bit per-thread offset
        const int8_t *src = kc + (int64_t)blk * p.k_stride_block + (int64_t)inpage0 * p.k_stride_row;
        const uint32_t voff = (uint32_t)min(t_row, last) * (uint32_t)p.k_stride_row + t_sub * 12;
#pragma unroll
        for (int i = 0; i < kMlaRounds; ++i) st[set][i] = *reinterpret_cast<const MlaCodes12 *>(src + voff + i * 192);
        // every thread loads a scale (no branch around a load: the waits stay counted in order)
        const int64_t so = (int64_t)blk * p.ks_stride_block + (int64_t)inpage0 * p.ks_stride_row;
        const uint32_t soff = (uint32_t)min(th & (kChunk - 1), last) * (uint32_t)p.ks_stride_row;
        st_ks[set] = (p.k_scale + so)[soff];
        st_vs[set] = (p.v_scale + so)[soff];
    };
    auto stash = [&](int buf, int set, int th) {
        uint8_t *dst = &sh.k[buf][(th >> 4) * kMlaRowBytes + (th & 15) * 24];
#pragma unroll
        for (int i = 0; i < kMlaRounds; ++i) {
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                uint2 w;
                widen4<T>(st[set][i].w[j], w.x, w.y);
                *reinterpret_cast<uint2 *>(dst + i * 384 + j * 8) = w;
            }
        }
        if (th < kChunk) {
            sh.ks[buf][th] = st_ks[set];
            sh.vs[buf][th] = st_vs[set];
        }
    };

    // page ids are loaded one step before the loads that use them and always ahead of that step's
    // tile loads, so waiting for a page id never waits for younger tile loads
    int blk_next = 0;
    if (c_begin < c_end) {
        fetch(c_begin, fetch_blk(c_begin), 0, tid);
        blk_next = fetch_blk(c_begin + 1);
        stash(0, 0, tid);
        const int blk2 = fetch_blk(c_begin + 2);
        if (c_begin + 1 < c_end) fetch(c_begin + 1, blk_next, 1, tid);
        blk_next = blk2;
    }
    __syncthreads();

    // one chunk; `set` = parity of the chunk within the piece (compile-time in the unrolled loop)
    auto chunk_step = [&](const int c, const int set) {
        const int cur = set;
        const bool more = c + 1 < c_end;
        // lane-derived LDS addresses are recomputed in every step (a few adds) instead of being kept
        // in registers across the whole piece, which the register budget cannot afford
        int tid_here = tid;
        asm volatile("" : "+v"(tid_here));
        const int lane = tid_here & 63;
        const int lq = lane >> 4;
        const int ln = lane & 15;
        {
            const int blk3 = fetch_blk(c + 3);
            if (c + 2 < c_end) fetch(c + 2, blk_next, set, tid_here);
            blk_next = blk3;
        }
        __builtin_amdgcn_sched_barrier(0);

        // ---- S^T = K Q^T : this wave's 16-key tile x 16 heads; operand reads run kPf k-steps
        //      ahead of the MFMAs that use them, two accumulators break the dependency chain
        constexpr int kPf = 4;
        float4_t s2[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
        u32x4_t ka[KSTEPS];
        const uint8_t *k_rd = &sh.k[cur][(kt * 16 + ln) * kMlaRowBytes + lq * 16];
#pragma unroll
        for (int t = 0; t < kPf; ++t) ka[t] = *reinterpret_cast<const u32x4_t *>(k_rd + t * 64);
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t) {
            if (t + kPf < KSTEPS) ka[t + kPf] = *reinterpret_cast<const u32x4_t *>(k_rd + (t + kPf) * 64);
            s2[t & 1] = mfma16<T>(ka[t], qreg[t], s2[t & 1]);
            __builtin_amdgcn_sched_barrier(0);
        }

        // ---- softmax; register i is key c*32 + kt*16 + lq*4 + i of head `head`
        const int key_base = c * kChunk + kt * 16 + lq * 4;
        const float4 ks4 = *reinterpret_cast<const float4 *>(&sh.ks[cur][kt * 16 + lq * 4]);
        const float4 vs4 = *reinterpret_cast<const float4 *>(&sh.vs[cur][kt * 16 + lq * 4]);
        const float ksv[4] = {ks4.x, ks4.y, ks4.z, ks4.w};
        const float vsv[4] = {vs4.x, vs4.y, vs4.z, vs4.w};
        float x[4];
        float mloc = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = key_base + i;
            float v = (s2[0][i] + s2[1][i]) * ksv[i] * p.scale_log2;
            v = (key >= range_lo && key < range_hi) ? v : -INFINITY;
            x[i] = v;
            mloc = fmaxf(mloc, v);
        }
        mloc = quad_rows_max(mloc);
        if (lq == 0) sh.mx[kt][g][ln] = mloc;
        __syncthreads();   // both key tiles' maxima are in LDS (and the previous chunk's products are done)

        mloc = fmaxf(mloc, sh.mx[kt ^ 1][g][ln]);
        const bool bump = mloc > m_run;
        const float m_new = bump ? mloc : m_run;
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = bump ? fast_exp2(m_run - m_use) : 1.f;
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float pe = fast_exp2(x[i] - m_use);
            psum += pe;
            x[i] = pe * vsv[i];   // V side of the dequantisation folded into P
        }
        l_run = l_run * alpha + psum;
        sh.pk[g][lane][kt] = make_uint2(pack2<T>(x[0], x[1]), pack2<T>(x[2], x[3]));
        if (kt == 0) {
            if (lq == 0) sh.alpha[g][ln] = alpha;
            const int wave_bump = __any(bump) ? 1 : 0;
            if (lane == 0) sh.bump[g] = (uint8_t)wave_bump;
        }
        // widening of the prefetched tile: its buffer was last read by the previous chunk's products
        if (more) stash(cur ^ 1, set ^ 1, tid_here);
        __syncthreads();   // P, alpha of all 64 heads and the next tile are in LDS

        // ---- O^T += V^T P^T on this wave's 64-column slice, all four head groups.
        //      k slot 8*lq + e of the MFMA is key (e >> 2) * 16 + lq * 4 + (e & 3) of the chunk.
        uint2 vr[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int row = (e >> 2) * 16 + lq * 4 + (e & 3);
            vr[e] = *reinterpret_cast<const uint2 *>(&sh.k[cur][row * kMlaRowBytes + (wave * 64 + ln * 4) * 2]);
        }
        u32x4_t pkg[4];
        const uint32_t bumps = *reinterpret_cast<const uint32_t *>(sh.bump);
#pragma unroll
        for (int hg = 0; hg < 4; ++hg) {
            pkg[hg] = *reinterpret_cast<const u32x4_t *>(&sh.pk[hg][lane][0]);
            if ((bumps >> (8 * hg)) & 0xffu) {
                const float ag = sh.alpha[hg][ln];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    o_acc[hg][t][0] *= ag;
                    o_acc[hg][t][1] *= ag;
                    o_acc[hg][t][2] *= ag;
                    o_acc[hg][t][3] *= ag;
                }
            }
        }
#pragma unroll
        for (int w2 = 0; w2 < 2; ++w2) {
            u32x4_t a_lo, a_hi;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t e0 = w2 ? vr[2 * u].y : vr[2 * u].x;
                const uint32_t e1 = w2 ? vr[2 * u + 1].y : vr[2 * u + 1].x;
                a_lo[u] = __builtin_amdgcn_perm(e1, e0, 0x05040100u);
                a_hi[u] = __builtin_amdgcn_perm(e1, e0, 0x07060302u);
            }
#pragma unroll
            for (int hg = 0; hg < 4; ++hg) {
                o_acc[hg][2 * w2] = mfma16<T>(a_lo, pkg[hg], o_acc[hg][2 * w2]);
                o_acc[hg][2 * w2 + 1] = mfma16<T>(a_hi, pkg[hg], o_acc[hg][2 * w2 + 1]);
            }
        }
    };
    for (int c = c_begin; c < c_end; c += 2) {
        chunk_step(c, 0);
        if (c + 1 < c_end) chunk_step(c + 1, 1);
    }

    // ---- write.  The score-owning waves publish max and sum; every wave then stores its column
    //      slice: register i of tile t of group hg is column wave*64 + (lq*4 + i)*4 + t of head hg*16 + ln.
    l_run = quad_rows_sum(l_run);
    if (lq == 0) {
        sh.m[g][ln] = m_run;      // identical in both key-tile waves
        sh.l[kt][g][ln] = l_run;
    }
    __syncthreads();
#pragma unroll
    for (int hg = 0; hg < 4; ++hg) {
        const int row = hg * 16 + ln;   // row of the unit (0..63)
        const int hd = half * kMlaHeadsPerUnit + row;
        const float lg = sh.l[0][hg][ln] + sh.l[1][hg][ln];
        const float inv = (lg > 0.f) ? 1.f / lg : 0.f;
        if (write_final) {
            uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)hd * p.o_stride_h +
                            wave * 64;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint2 o2 = make_uint2(pack2<T>(o_acc[hg][0][i] * inv, o_acc[hg][1][i] * inv),
                                            pack2<T>(o_acc[hg][2][i] * inv, o_acc[hg][3][i] * inv));
                *reinterpret_cast<uint2 *>(dst + (lq * 4 + i) * 4) = o2;
            }
        } else {
            const int64_t srow = slot * p.rows + row;
            float *dst = p.o_partial + srow * kMlaDv + wave * 64;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *reinterpret_cast<float4 *>(dst + (lq * 4 + i) * 4) =
                    make_float4(o_acc[hg][0][i] * inv, o_acc[hg][1][i] * inv, o_acc[hg][2][i] * inv, o_acc[hg][3][i] * inv);
        }
    }
    if (kt == 0 && lq == 0) {
        // this lane column's own head: LSE (final) or partial LSE
        const int row = g * 16 + ln;
        const float lg = sh.l[0][g][ln] + sh.l[1][g][ln];
        if (write_final)
            p.lse[(int64_t)b * p.nheads + head] = (lg > 0.f) ? (m_run + fast_log2(lg)) * kLn2 : INFINITY;
        else
            p.lse_partial[slot * p.rows + row] = (lg > 0.f) ? m_run + fast_log2(lg) : -INFINITY;
    }
    __syncthreads();   // the LDS tiles are reused by the next piece
}

template <typename T> __global__ void __launch_bounds__(kMlaThreads) decode_mla_i8_kernel(const DecodeParams p) {
    __shared__ MlaShared sh;
    balanced_driver<kMlaDv>(p, [&](int b, int half, const UnitRange &ur, int range_lo, int range_hi, bool whole, int64_t slot) {
        mla_piece<T>(p, b, half, ur, range_lo, range_hi, whole, slot, sh);
    });
}

// p.nheads_k counts 64-head halves here (units per batch row), p.group = p.rows = 64.
hipError_t launch_decode_mla_i8(const DecodeParams &p, int dtype, hipStream_t stream) {
    if (p.seqlen_q != 1 || p.rows != kMlaHeadsPerUnit || p.group != kMlaHeadsPerUnit || !p.balanced)
        return hipErrorInvalidValue;
    dim3 grid(p.num_wgs), block(kMlaThreads);
    if (dtype == 0)
        hipLaunchKernelGGL(decode_mla_i8_kernel<BF16>, grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL(decode_mla_i8_kernel<FP16>, grid, block, 0, stream, p);
    return hipGetLastError();
}

}  // namespace fa
