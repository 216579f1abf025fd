// Latent-attention (MLA) decode over an int8 paged cache with per-token fp32 scales, gfx950.
//
// Layout: one latent kv head, 576 key dims, V = the first 512 of them (v_cache aliases k_cache); any number of q
// heads, any seqlen_q (each query token is its own set of units).  The reference has no quantised path (dtypes are
// limited to fp16/bf16 at csrc/ascend910/flash_attn_npu/flash_api.cpp:386-388 and descales are rejected at
// flash_attn_npu_3/flash_api.cpp:153-155); the attention arithmetic is the same as the bf16 decode kernel's
// (mha_fwd_kvcache.cpp:632-969 in the reference) applied to K^ = code * scale[token].
//
// A work unit is (batch row, query token, group of 128 heads): ALL heads of a token share one pass over the cache,
// so every 32-key chunk is fetched from HBM once and widened to the 16-bit type once (a code is an integer of
// magnitude <= 127, exact in bf16 and fp16).  One 256-thread workgroup per compute unit, one wave per SIMD with the
// whole register file (512 registers): the fp32 accumulators of 128 heads x 512 columns fill the 256 accumulation
// registers of every wave, Q^T most of the ordinary ones.
//
//   scores  wave w owns heads 32w..32w+31 with Q^T resident (29 operands of the 32x32x16 MFMA in registers, the last
//           7 in LDS): S^T[32 keys x 32 heads] = K Q^T, the key-side scale folded into the exponent, online softmax local
//           to the lane column (one exchange between the two half-waves per chunk).  P^T, with the V-side scale folded
//           in and rounded to the 16-bit type, goes to LDS in MFMA operand order.
//   output  wave w owns columns 128w..128w+127 of V for ALL 128 heads: O^T[cols x heads] += V^T P^T; every
//           transposed V operand (ds_read_b64_tr_b16 from the same LDS tile) feeds four MFMAs, one per head group.
//   staging all four waves: the loads of chunk c+2 leave (global -> registers) piece by piece while chunk c+1 is
//           widened into LDS beside the score products of chunk c, and the softmax of chunk c stands beside the
//           output products of chunk c-1; one workgroup barrier per chunk, three LDS tiles.
// Measured on this machine, a wave that is alone on its SIMD issues one instruction per turn whatever its kind, and
// its matrix instructions overlap little with the rest: a chunk costs its 68 MFMAs plus 4-5 cycles for EVERY other
// instruction (vector, scalar, LDS, wait: ~540 of them), so what counts is the instruction count of the loop.
// Split units leave fp16 partial rows (partials_are_half), and neighbouring shares are dealt to one XCD (their q
// rows meet in one L2).
//
// The exponent reference of a head moves only when a chunk's maximum passes it by more than kLazy (the lazy rescale of
// the reference's fourth-generation kernels, csrc/ascend910/flash_attn_npu_4/online_softmax.hpp:633-666): rescaling
// the accumulators is then rare, and all of it (masks, the first chunk, a moved reference) lives on a slow path the
// common chunk never enters.  The weight a key really gets is round16(P * v_scale) / v_scale; the output is divided
// by the sum of THOSE weights, so it stays a convex combination of the dequantised rows whatever the reference is
// (a row that sees one key returns that key); the LSE uses the unrounded P.
#include <utility>

#include "decode_common.h"

// This file keeps its output accumulators in a0..a255 behind the compiler's back (see below).  Whether the compiler
// left those registers alone can only be read off the assembly it produced: build.py does that for every build
// (_check_acc_registers) and defines this macro; a build that does not run the check must not produce this kernel.
#ifndef FA_ROCM_ACC_REGISTERS_CHECKED
#error "decode_mla_i8.hip must be compiled by flash-attention-npu_amd/build.py, which checks the accumulation registers in the device assembly"
#endif

namespace fa {

constexpr int kMlaDqk = 576;
constexpr int kMlaDv = 512;
constexpr int kMlaThreads = 256;
constexpr int kMlaUnitHeads = 128;                       // heads of a unit, 32 per wave
constexpr int kMlaRowBytes = kMlaDqk * 2;                // 1152: a widened key row
constexpr int kMlaTileBytes = kChunk * kMlaRowBytes;     // 36864
constexpr int kMlaKSteps = kMlaDqk / 16;                 // 36 k-steps of the score product
constexpr int kMlaRounds = kMlaDqk / 64;                 // 9 eight-code pieces per staging thread and chunk
constexpr int kMlaQLds = 7;                              // Q^T operands of the last k-steps wait in LDS, not in registers
constexpr int kMlaQReg = kMlaKSteps - kMlaQLds;
static_assert(kMlaThreads / 8 == kChunk, "eight staging threads per key row");

// LDS key rows are unpadded (1152 B = 4.5 x 256 B: odd and even rows sit half a bank cycle apart); the 16-byte units
// of a row are XOR-swizzled inside their aligned groups of eight with the bit-reversed (row / 2) % 8.  The LDS serves
// 16 lanes per cycle, so: the 16 rows x same unit of a score operand read land on 16 different units modulo 256 B
// (eight rows of equal parity get eight different swizzles), and the 4 rows x 4 units of a transposed read as well
// (rows r and r + 2 differ in swizzle bit 2, i.e. in which aligned group of four units they use).
__device__ __forceinline__ int mla_swz(int row) {
    const int t = row >> 1;
    return ((t & 1) << 2) | (t & 2) | ((t >> 2) & 1);
}

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

template <typename T> struct MlaLazy;
// P <= 2^kLazy before the V-side scale is folded in: bf16 has the range; fp16 (max 65504) keeps 2^4 x scale inside it
template <> struct MlaLazy<BF16> { static constexpr float kLog2 = 8.f, kMax = 256.f; };
template <> struct MlaLazy<FP16> { static constexpr float kLog2 = 4.f, kMax = 16.f; };

// ---- the output accumulators live in the 256 accumulation registers a0..a255, addressed by number.
// The compiler's register allocator keeps loop-carried vector values in ordinary registers and copies them in and out
// of every hand-written matrix instruction; 128 heads x 512 columns only fit if they never leave the accumulation
// file.  So these registers are not C++ values at all: every instruction that touches them is written out with the
// register number in its text, and lists all 256 as clobbered, which (a) makes the kernel's register count include
// them and (b) keeps the compiler from parking anything of its own there across these instructions.
#define MLA_AD(p, d) "a" p #d
#define MLA_ATEN(p) MLA_AD(p, 0), MLA_AD(p, 1), MLA_AD(p, 2), MLA_AD(p, 3), MLA_AD(p, 4), MLA_AD(p, 5), MLA_AD(p, 6), MLA_AD(p, 7), MLA_AD(p, 8), MLA_AD(p, 9)
#define MLA_ALL_ACC                                                                                                          \
    MLA_ATEN(""), MLA_ATEN("1"), MLA_ATEN("2"), MLA_ATEN("3"), MLA_ATEN("4"), MLA_ATEN("5"), MLA_ATEN("6"), MLA_ATEN("7"),        \
        MLA_ATEN("8"), MLA_ATEN("9"), MLA_ATEN("10"), MLA_ATEN("11"), MLA_ATEN("12"), MLA_ATEN("13"), MLA_ATEN("14"), MLA_ATEN("15"), \
        MLA_ATEN("16"), MLA_ATEN("17"), MLA_ATEN("18"), MLA_ATEN("19"), MLA_ATEN("20"), MLA_ATEN("21"), MLA_ATEN("22"),          \
        MLA_ATEN("23"), MLA_ATEN("24"), MLA_AD("25", 0), MLA_AD("25", 1), MLA_AD("25", 2), MLA_AD("25", 3), MLA_AD("25", 4),      \
        MLA_AD("25", 5)

template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// a[BASE : BASE+15] += A * B (32x32x16).  Register numbers are printed digit by digit: an immediate of 64 or more
// would come out in hexadecimal.
template <typename T, int BASE> __device__ __forceinline__ void acc_mfma(const u32x4_t &a, const u32x4_t &b) {
    if constexpr (BASE == 0) {
        if constexpr (__is_same(T, BF16))
            asm volatile("v_mfma_f32_32x32x16_bf16 a[0:15], %0, %1, a[0:15]" ::"v"(a), "v"(b) : MLA_ALL_ACC);
        else
            asm volatile("v_mfma_f32_32x32x16_f16 a[0:15], %0, %1, a[0:15]" ::"v"(a), "v"(b) : MLA_ALL_ACC);
    } else {
        if constexpr (__is_same(T, BF16))
            asm volatile("v_mfma_f32_32x32x16_bf16 a[%2%3:%4%5], %0, %1, a[%2%3:%4%5]" ::"v"(a), "v"(b), "n"(BASE / 10),
                         "n"(BASE % 10), "n"((BASE + 15) / 10), "n"((BASE + 15) % 10)
                         : MLA_ALL_ACC);
        else
            asm volatile("v_mfma_f32_32x32x16_f16 a[%2%3:%4%5], %0, %1, a[%2%3:%4%5]" ::"v"(a), "v"(b), "n"(BASE / 10),
                         "n"(BASE % 10), "n"((BASE + 15) / 10), "n"((BASE + 15) % 10)
                         : MLA_ALL_ACC);
    }
}
// a[BASE : BASE+15] = 0 (z must hold zeros).  The wait states in front of the first one stand for those the compiler
// would put between the vector instruction that writes z and a matrix instruction it knows.
template <typename T, int BASE> __device__ __forceinline__ void acc_mfma_zero(const u32x4_t &z) {
    if constexpr (BASE == 0)
        asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_bf16 a[0:15], %0, %0, 0" ::"v"(z) : MLA_ALL_ACC);
    else
        asm volatile("v_mfma_f32_32x32x16_bf16 a[%1%2:%3%4], %0, %0, 0" ::"v"(z), "n"(BASE / 10), "n"(BASE % 10),
                     "n"((BASE + 15) / 10), "n"((BASE + 15) % 10)
                     : MLA_ALL_ACC);
}
template <int R> __device__ __forceinline__ float acc_read() {
    float v;
    if constexpr (R < 10)
        asm volatile("v_accvgpr_read_b32 %0, a%1" : "=v"(v) : "n"(R) : MLA_ALL_ACC);
    else
        asm volatile("v_accvgpr_read_b32 %0, a%1%2" : "=v"(v) : "n"(R / 10), "n"(R % 10) : MLA_ALL_ACC);
    return v;
}
template <int R> __device__ __forceinline__ void acc_scale(float f) {
    float t;
    if constexpr (R < 10)
        asm volatile("v_accvgpr_read_b32 %0, a%2\n\tv_mul_f32 %0, %0, %1\n\tv_accvgpr_write_b32 a%2, %0" : "=&v"(t) : "v"(f), "n"(R) : MLA_ALL_ACC);
    else
        asm volatile("v_accvgpr_read_b32 %0, a%2%3\n\tv_mul_f32 %0, %0, %1\n\tv_accvgpr_write_b32 a%2%3, %0"
                     : "=&v"(t)
                     : "v"(f), "n"(R / 10), "n"(R % 10)
                     : MLA_ALL_ACC);
}
// wait states between a matrix instruction and the first vector instruction that reads or writes its result
// registers (and back): the hazards the compiler would cover for instructions it knows
__device__ __forceinline__ void mfma_settle() { asm volatile("s_nop 15\n\ts_nop 3" ::: "memory", MLA_ALL_ACC); }

// Eight 16-byte LDS reads at constant offsets from one address, issued back to back, then one wait.  Written out by
// hand because the compiler pairs every such read with the store that uses it (sixteen exposed LDS latencies per pass
// of the epilogue) whatever the source order is.
template <int STRIDE> __device__ __forceinline__ void lds_read8x16(uint32_t addr, float4 (&v)[8]) {
    asm volatile(
        "ds_read_b128 %0, %8\n\t"
        "ds_read_b128 %1, %8 offset:%9\n\t"
        "ds_read_b128 %2, %8 offset:%10\n\t"
        "ds_read_b128 %3, %8 offset:%11\n\t"
        "ds_read_b128 %4, %8 offset:%12\n\t"
        "ds_read_b128 %5, %8 offset:%13\n\t"
        "ds_read_b128 %6, %8 offset:%14\n\t"
        "ds_read_b128 %7, %8 offset:%15\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
        : "v"(addr), "n"(STRIDE), "n"(2 * STRIDE), "n"(3 * STRIDE), "n"(4 * STRIDE), "n"(5 * STRIDE), "n"(6 * STRIDE), "n"(7 * STRIDE)
        : "memory");
}

// The small arrays come first: an LDS instruction carries a 16-bit byte offset, so everything below 64 KB is reached as
// (lane's register + constant); behind the 108 KB of key tiles every access needed an add of its own.
struct MlaShared {
    struct __attribute__((aligned(16))) Scales {                 // per-token scales of a tile, side by side: one LDS base address
        float ksl[kChunk];                                       // key-side scale x softmax scale (log2 units)
        float vs[kChunk];                                        // V-side scale
        float vsi[kChunk];                                       // its inverse (0 for a zero scale)
        uint16_t vsi_hi[kChunk];                                 // the inverse as two bf16 terms (hi + lo), for v_dot2_f32_bf16
        uint16_t vsi_lo[kChunk];
    } sc[3];
    __attribute__((aligned(16))) u32x4_t pk[2][4][2][64];        // P^T operands: [chunk parity][head group][k-step][lane]
    float alpha[2][kMlaUnitHeads];                               // accumulator rescale per head (slow path only)
    __attribute__((aligned(16))) int32_t moved[2][4];                                         // head group moved its reference in this chunk
    float l[kMlaUnitHeads];                                      // final normaliser per head
    __attribute__((aligned(16))) u32x4_t q[4][kMlaQLds][64];     // Q^T operands of the last k-steps: [wave][k-step][lane]
    __attribute__((aligned(16))) uint8_t k[3][kMlaTileBytes];   // widened key tiles
};

template <typename T, bool SOFTCAP>
__device__ __forceinline__ void mla_piece(const DecodeParams &p, const int b, const int unit, const UnitRange &ur,
                                          const int range_lo, const int range_hi, const bool write_final,
                                          const int64_t slot, MlaShared &sh) {
    // unit = (query token qi, 128-head group hgrp); the chunks walked are those of the whole query block, the keys
    // this token may not see (causal / window bounds of its own row) are masked
    const int qi = unit / p.units_per_token;
    const int hgrp = unit - qi * p.units_per_token;
    const int row_off = ur.Lk - p.seqlen_q + qi;                       // key aligned with this query token
    const int mask_lo = max(range_lo, ur.wl >= 0 ? row_off - ur.wl : 0);
    const int mask_hi = min(range_hi, ur.wr >= 0 ? row_off + ur.wr + 1 : ur.Lk);
    // The thread number is made opaque here: a worker walks the pieces of its share in a loop, and everything derived
    // from the lane (LDS offsets, swizzles, row numbers) would otherwise be computed once outside that loop and kept
    // alive through prologue and epilogue, where the registers are needed for other things.
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int ln = lane & 31;     // MFMA column: head of the wave's group (scores), head of a group (output)
    const int lh = lane >> 5;     // half-wave
    const int Lk = ur.Lk;
    const int c_begin = range_lo / kChunk;
    const int nch = (range_hi + kChunk - 1) / kChunk - c_begin;   // chunks of this piece (>= 1)

    const int8_t *kc = reinterpret_cast<const int8_t *>(p.k_cache);
    const int32_t *bt_row = p.block_table + (int64_t)b * p.bt_stride_b;

    // The chunks of a piece are consecutive, so the page of a chunk and its offset inside the page are carried along
    // from chunk to chunk (page sizes are multiples of the chunk, or the cache is one page): a division and four
    // 64-bit products per chunk were 90 scalar instructions, and in this loop of one wave per SIMD every instruction
    // of any kind costs its 4-5 cycles.  Two cursors: fb_* runs ahead and requests table entries, fs_* sets up the
    // loads.  Both stop at the piece's last chunk (requests past it repeat it).
    const uint32_t page_size = (uint32_t)p.page_size;
    uint32_t fb_page = (uint32_t)(c_begin * kChunk) / page_size;
    uint32_t fb_in = (uint32_t)(c_begin * kChunk) - fb_page * page_size;
    int fb_left = nch - 1;                                             // chunks the cursor may still advance
    uint32_t fs_in = fb_in;
    int fs_last = Lk - 1 - c_begin * kChunk;                           // last key of the sequence, relative to the chunk
    int fs_left = nch - 1;
    const int64_t row32_k = (int64_t)kChunk * p.k_stride_row, row32_s = (int64_t)kChunk * p.ks_stride_row;
    int64_t fs_off_k = (int64_t)fs_in * p.k_stride_row, fs_off_s = (int64_t)fs_in * p.ks_stride_row;
    auto fetch_blk = [&]() -> int {
        const int v = bt_row[min(fb_page, (uint32_t)p.max_blocks - 1)];   // clamped and made wave-uniform where it is used, an iteration later: no wait here
        if (fb_left > 0) {
            --fb_left;
            fb_in += kChunk;
            if (fb_in >= page_size) {
                fb_in -= page_size;
                ++fb_page;
            }
        }
        return v;
    };
    // page ids of the first two chunks: requested first, they come back while Q^T is loaded
    const int blk_first = fetch_blk();
    const int blk_second = fetch_blk();

    // ---- Q^T operands: lane (ln, lh) holds head 32*wave + ln, dims 16t + 8lh .. +7 of k-step t.  Loaded in that
    //      layout, one instruction would touch 32 rows of q, 32 bytes each (measured: 9 us of the kernel).  The wave's 32
    //      rows are fetched as they lie instead - a third of a row (384 bytes = 24 lanes) after the other, three rounds
    //      of 12 instructions, all requested here - and turned into the operand layout through a staging area of the
    //      wave's own (stage_q below, once the first chunk's loads are out as well).
    const int row_u = wave * 32 + ln;                                  // row of the unit
    const int head = hgrp * kMlaUnitHeads + row_u;
    constexpr int kQRounds = 3;
    constexpr int kQRoundSteps = kMlaKSteps / kQRounds;                // k-steps of a round
    constexpr int kQRoundBytes = kQRoundSteps * 32;                    // 384 bytes of a row
    constexpr int kQRowPieces = kQRoundBytes / 16;
    // staged rows lie 100 words apart: the 16 lanes the LDS serves per cycle, 4 banks each, then tile all 64 banks.
    // Unpadded, the reads of the operand layout were 4-way bank conflicts, and staging q cost the LDS 6 us per piece.
    constexpr int kQStageRow = kQRoundBytes + 16;
    static_assert(kQRounds * kQRoundSteps == kMlaKSteps && kQRoundSteps * 64 == 32 * kQRowPieces, "rounds tile q");
    static_assert(4 * 32 * kQStageRow <= 2 * kMlaTileBytes, "the Q staging areas live in key tiles 1 and 2");
    u32x4_t qreg[kMlaQReg];
    u32x4_t qraw[kQRounds][kQRoundSteps];
    {
        const uint16_t *src = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_stride_b + (int64_t)qi * p.q_stride_s;
        const int head0 = hgrp * kMlaUnitHeads + wave * 32;
#pragma unroll
        for (int r = 0; r < kQRounds; ++r)
#pragma unroll
            for (int i = 0; i < kQRoundSteps; ++i) {
                const int j = i * 64 + lane;                           // 16-byte piece j of the round: row j / 24
                const int row = j / kQRowPieces;
                const int c = j - row * kQRowPieces;
                qraw[r][i] = load16(src + (int64_t)min(head0 + row, p.nheads - 1) * p.q_stride_h + r * (kQRoundBytes / 2) + c * 8);
            }
    }
    auto stage_q = [&]() {
        uint8_t *stg = &sh.k[1][0] + wave * (32 * kQStageRow);         // tiles 1 and 2 are written from the first step on
#pragma unroll
        for (int r = 0; r < kQRounds; ++r) {
#pragma unroll
            for (int i = 0; i < kQRoundSteps; ++i) {
                const int j = i * 64 + lane;
                const int row = j / kQRowPieces;
                *reinterpret_cast<u32x4_t *>(stg + row * kQStageRow + (j - row * kQRowPieces) * 16) = qraw[r][i];
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int t = 0; t < kQRoundSteps; ++t) {
                const u32x4_t v = *reinterpret_cast<const u32x4_t *>(stg + ln * kQStageRow + t * 32 + lh * 16);
                const int tt = r * kQRoundSteps + t;
                if (tt < kMlaQReg)
                    qreg[tt < kMlaQReg ? tt : 0] = v;
                else
                    sh.q[wave][tt >= kMlaQReg ? tt - kMlaQReg : 0][lane] = v;   // wave-private
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();   // the area is rewritten by the next round
        }
    };

    // ---- staging: thread -> (key row tid / 8, eight-code pieces tid % 8 + 8i): one address per chunk serves all
    //      loads and one LDS address all stores.  Rows past the last key of the sequence re-read the last key
    //      (never memory nobody wrote); they are masked.
    MlaCodes8 st[kMlaRounds];
    float st_ks = 0.f, st_vs = 0.f;
    // the loads of a chunk leave piece by piece (fetch_piece), right behind the widening of the piece that held the
    // registers before: they have a whole step to come back
    const int8_t *f_src = nullptr;
    const float *f_ks = nullptr, *f_vs = nullptr;
    // per-thread offsets of a chunk that lies wholly inside the sequence; only the sequence's last chunk clamps its rows
    uint32_t f_voff = (uint32_t)(tid >> 3) * (uint32_t)p.k_stride_row + (tid & 7) * 8;
    uint32_t f_soff = (uint32_t)(tid & (kChunk - 1)) * (uint32_t)p.ks_stride_row;
    auto fetch_setup = [&](int blk_raw) {
        const int blk = __builtin_amdgcn_readfirstlane(min(max(blk_raw, 0), p.num_blocks - 1));
        f_src = kc + (int64_t)blk * p.k_stride_block + fs_off_k;
        const int64_t so = (int64_t)blk * p.ks_stride_block + fs_off_s;
        f_ks = p.k_scale + so;
        f_vs = p.v_scale + so;
        if (fs_last < kChunk - 1) {   // wave-uniform, the end of the sequence
            f_voff = (uint32_t)min(tid >> 3, fs_last) * (uint32_t)p.k_stride_row + (tid & 7) * 8;
            f_soff = (uint32_t)min(tid & (kChunk - 1), fs_last) * (uint32_t)p.ks_stride_row;
        }
        if (fs_left > 0) {
            --fs_left;
            fs_last -= kChunk;
            fs_in += kChunk;
            fs_off_k += row32_k;
            fs_off_s += row32_s;
            if (fs_in >= page_size) {   // only with pages that are multiples of the chunk: the next page starts at 0
                fs_in = 0;
                fs_off_k = fs_off_s = 0;
            }
        }
    };
    auto fetch_piece = [&](int i) { st[i] = *reinterpret_cast<const MlaCodes8 *>(f_src + f_voff + i * 64); };
    auto fetch_scales = [&]() {
        st_ks = f_ks[f_soff];
        st_vs = f_vs[f_soff];
    };
    const int st_row = tid >> 3;
    const int st_off = st_row * kMlaRowBytes + (((tid & 7) ^ mla_swz(st_row)) << 4);
    // widening of eight-code piece i in four steps (q = 0..3: two codes each ... the last one stores the unit)
    u32x4_t wide;
    auto widen_quarter = [&](int tile, int i, int q) {
        const uint32_t w = st[i].w[q >> 1];
        if ((q & 1) == 0) {
            wide[q] = pack2<T>((float)(int8_t)(w & 0xff), (float)(int8_t)((w >> 8) & 0xff));
        } else {
            wide[q] = pack2<T>((float)(int8_t)((w >> 16) & 0xff), (float)(int8_t)(w >> 24));
            if (q == 3) *reinterpret_cast<u32x4_t *>(&sh.k[tile][st_off + i * 128]) = wide;
        }
    };
    auto stash_scales = [&](int tile) {
        if (tid < kChunk) {
            sh.sc[tile].ksl[tid] = st_ks * (SOFTCAP ? p.softcap_pre : p.scale_log2);
            sh.sc[tile].vs[tid] = st_vs;
            const float inv = (st_vs > 0.f) ? __builtin_amdgcn_rcpf(st_vs) : 0.f;
            sh.sc[tile].vsi[tid] = inv;
            const uint16_t hi = from_float<BF16>(inv);
            sh.sc[tile].vsi_hi[tid] = hi;
            sh.sc[tile].vsi_lo[tid] = from_float<BF16>(inv - to_float<BF16>(hi));
        }
    };

    // All matrix instructions of the loop are written out: the accumulator of the score product is pinned to ordinary
    // vector registers (the softmax reads it there), and the products stand in the instruction stream exactly where
    // the vector work beside them is written (the wave issues in order: a product, then the few vector instructions
    // that run in its shadow).
    // (the result of the first product is written while the operands are still being read: it may share no register
    // with them, hence the early-clobber constraint; the accumulating form reads and writes the same registers)
    auto mfma_first = [&](float16_t &d, const u32x4_t &a, const u32x4_t &bq) {
        if constexpr (__is_same(T, BF16))
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(bq));
        else
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(bq));
    };
    auto mfma_v = [&](float16_t &d, const u32x4_t &a, const u32x4_t &bq) {
        if constexpr (__is_same(T, BF16))
            asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(bq));
        else
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(bq));
    };
    // ---- S^T = K Q^T: operand t is unit 2t + lh of key row ln.  A quarter of an eight-code piece of the next chunk is
    //      widened beside every product.
    float16_t s_acc;
    const int sc_row = ln * kMlaRowBytes;
    int sc_off[4];
    {
        const int sw = mla_swz(ln);
#pragma unroll
        for (int k = 0; k < 4; ++k) sc_off[k] = sc_row + (((2 * k + lh) ^ sw) << 4);
    }
    auto scores = [&](int tile, int tile_w) {
        constexpr int kPf = 4;
        const uint8_t *base = &sh.k[tile][0];
        u32x4_t ka[kMlaKSteps];
        u32x4_t ql[kMlaQLds];
        auto issue = [&](int t) {
            ka[t] = *reinterpret_cast<const u32x4_t *>(base + sc_off[t & 3] + (t >> 2) * 128);
            if (t >= kMlaQReg) ql[t - kMlaQReg] = sh.q[wave][t - kMlaQReg][lane];
        };
#pragma unroll
        for (int t = 0; t < kPf; ++t) issue(t);
#pragma unroll
        for (int t = 0; t < kMlaKSteps; ++t) {
            if (t + kPf < kMlaKSteps) issue(t + kPf);
            const u32x4_t &bq = (t < kMlaQReg) ? qreg[t < kMlaQReg ? t : 0] : ql[t >= kMlaQReg ? t - kMlaQReg : 0];
            if (t == 0)
                mfma_first(s_acc, ka[t], bq);
            else
                mfma_v(s_acc, ka[t], bq);
            widen_quarter(tile_w, t >> 2, t & 3);
            if ((t & 3) == 3) fetch_piece(t >> 2);   // chunk i+2 into the registers just widened
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- softmax of chunk j on s_acc, in place: register r of a lane is key 8*(r/4) + 4*lh + r%4 of the chunk
    float m_ref = -INFINITY, l_run = 0.f, l_norm = 0.f;   // per lane: its 16 keys of every chunk; halves summed at the end
    float psum = 0.f, nsum = 0.f;
    u32x4_t pk[2];
    // the scale vectors of slice g: registers 4g .. 4g+3 are keys 8g + 4*lh + 0..3
    auto load_ksl = [&](int tile, int g) { return *reinterpret_cast<const float4 *>(&sh.sc[tile].ksl[4 * lh + 8 * g]); };
    auto load_vs = [&](int tile, int g) { return *reinterpret_cast<const float4 *>(&sh.sc[tile].vs[4 * lh + 8 * g]); };
    auto load_vsi = [&](int tile, int g) { return *reinterpret_cast<const float4 *>(&sh.sc[tile].vsi[4 * lh + 8 * g]); };
    auto load_vsi_hi = [&](int tile, int g) { return *reinterpret_cast<const uint2 *>(&sh.sc[tile].vsi_hi[4 * lh + 8 * g]); };
    auto load_vsi_lo = [&](int tile, int g) { return *reinterpret_cast<const uint2 *>(&sh.sc[tile].vsi_lo[4 * lh + 8 * g]); };
    // scores in log2 units RELATIVE TO THE STANDING REFERENCE, in place, and their maximum (registers 4g .. 4g+3): the
    // subtraction rides in the scaling's fused multiply-add, and the common chunk exponentiates what it finds here
    float xmax = -INFINITY;
    auto softmax_scale4 = [&](int g, const float4 &kq) {
        const float kv[4] = {kq.x, kq.y, kq.z, kq.w};
        const float m_std = (m_ref == -INFINITY) ? 0.f : m_ref;
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
            const int r = 4 * g + e;
            float v0, v1;
            if constexpr (SOFTCAP) {
                const float y0 = s_acc[r] * kv[e], y1 = s_acc[r + 1] * kv[e + 1];
                v0 = p.softcap_post * (1.f - 2.f / (__expf(2.f * y0) + 1.f)) - m_std;
                v1 = p.softcap_post * (1.f - 2.f / (__expf(2.f * y1) + 1.f)) - m_std;
            } else {
                v0 = __builtin_fmaf(s_acc[r], kv[e], -m_std);
                v1 = __builtin_fmaf(s_acc[r + 1], kv[e + 1], -m_std);
            }
            s_acc[r] = v0;
            s_acc[r + 1] = v1;
            xmax = fmaxf(fmaxf(xmax, v0), v1);   // one three-input maximum
        }
    };
    // The common chunk keeps the standing reference.  Anything else (the first chunk: the reference is -inf; a maximum
    // beyond the lazy bound; a chunk with masked keys) goes through here: masks, a moved reference, the rescale
    // factors for the column owners; the scores are then re-expressed relative to the reference the exponentials use.
    auto softmax_check = [&](int j) {
        const int pb = j & 1;
        const int key0 = (c_begin + j) * kChunk;
        const bool edge = key0 < mask_lo || key0 + kChunk > mask_hi;   // wave-uniform
        xmax = halves_max(xmax);
        const bool slow = edge || __any(m_ref == -INFINITY || !(xmax <= MlaLazy<T>::kLog2));
        int moved = 0;
        if (__builtin_expect(slow, 0)) {
            const float m_std = (m_ref == -INFINITY) ? 0.f : m_ref;
            float mloc = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = key0 + 8 * (r >> 2) + 4 * lh + (r & 3);
                s_acc[r] = (key >= mask_lo && key < mask_hi) ? s_acc[r] + m_std : -INFINITY;   // absolute again
                mloc = fmaxf(mloc, s_acc[r]);
            }
            mloc = halves_max(mloc);
            const bool bump = mloc > m_ref + MlaLazy<T>::kLog2;   // a reference of -inf moves to any finite maximum
            const float m_new = bump ? mloc : m_ref;
            const float alpha = bump ? fast_exp2(m_ref - ((m_new == -INFINITY) ? 0.f : m_new)) : 1.f;
            moved = __any(bump && m_ref != -INFINITY) ? 1 : 0;      // somebody's accumulators hold something to rescale
            if (moved && lh == 0) sh.alpha[pb][row_u] = alpha;
            l_run *= alpha;
            l_norm *= alpha;
            m_ref = m_new;
            const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref;
#pragma unroll
            for (int r = 0; r < 16; ++r) s_acc[r] -= m_use;
        }
        if (lane == 0) sh.moved[pb][wave] = moved;
        xmax = -INFINITY;
    };
    // exponentials (registers 4g .. 4g+3)
    auto softmax_exp4 = [&](int g) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s_acc[4 * g + e] = fast_exp2(s_acc[4 * g + e]);
    };
    // sums, V-side scale, rounding to the 16-bit type (registers 4g .. 4g+3); the weights really applied are summed
    // with the inverse scales: exactly for fp16, with a two-term bf16 inverse (2^-17 relative) on the dot-product path
    auto softmax_pack4 = [&](int g, const float4 &vq, const float4 &vi, const uint2 &ih, const uint2 &il) {
        const float vv[4] = {vq.x, vq.y, vq.z, vq.w};
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
            const int r = 4 * g + e;
            psum += s_acc[r] + s_acc[r + 1];
            const uint32_t d = pack2<T>(s_acc[r] * vv[e], s_acc[r + 1] * vv[e + 1]);   // V side of the dequantisation folded into P
            pk[r >> 3][(r & 7) >> 1] = d;
            if constexpr (__is_same(T, BF16)) {
                const uint32_t h2 = e ? ih.y : ih.x, l2 = e ? il.y : il.x;
                nsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, d), __builtin_bit_cast(bf16x2_t, h2), nsum, false);
                nsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, d), __builtin_bit_cast(bf16x2_t, l2), nsum, false);
            } else {
                const float iv[4] = {vi.x, vi.y, vi.z, vi.w};
                nsum = __builtin_fmaf(to_float<T>((uint16_t)(d & 0xffffu)), iv[e], nsum);
                nsum = __builtin_fmaf(to_float<T>((uint16_t)(d >> 16)), iv[e + 1], nsum);
            }
        }
    };
    auto softmax_store = [&](int j) {
        const int pb = j & 1;
        l_run += psum;
        l_norm += nsum;
        psum = nsum = 0.f;
        sh.pk[pb][wave][0][lane] = pk[0];
        sh.pk[pb][wave][1][lane] = pk[1];
    };

    // ---- O^T += V^T P^T on this wave's 128 columns, all four head groups.  o_acc[cc][hg]: column tile cc (32 columns)
    //      x head group hg; register r of a lane is column 128*wave + 32*cc + 8*(r/4) + 4*lh + r%4 of head 32*hg + ln.
    //      k slot 8*lh + i of k-step s2 is key 16*s2 + 8*(i/4) + 4*lh + i%4 (the order the score registers come in).
    //      The V^T operand comes from two transposing reads: in a 16-lane group, lane s points at 4 columns
    //      (4*(s%4)..) of key row s/4 and receives column s of the group's 16 for its 4 key rows.
    // accumulator tile (cc, hg) = a[16 * (4*cc + hg) .. +15]
    // zeroed sixteen registers at a time: a product of zero operands with a zero addend
    {
        const u32x4_t z = {0u, 0u, 0u, 0u};
        static_for<0, 16>([&](auto t_) { acc_mfma_zero<T, 16 * decltype(t_)::value>(z); });
    }
    int tr_off[2][2];   // [second four keys][odd column tile]
    {
        const int g16 = lane >> 4, s16 = lane & 15;
        const int rbase = 4 * (g16 >> 1) + (s16 >> 2);           // key row of this lane inside an 8-row block
        const int ub = 2 * (g16 & 1) + ((s16 & 3) >> 1);         // 16-byte unit inside the 64 bytes of a column tile
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int row = 8 * jj + rbase;
            const int sw = mla_swz(row);                          // rows 16 apart share it
#pragma unroll
            for (int c1 = 0; c1 < 2; ++c1)
                tr_off[jj][c1] = row * kMlaRowBytes + (((4 * c1 + ub) ^ sw) << 4) + wave * 256 + 8 * (s16 & 1);
        }
    }
    // accumulators of head groups whose reference moved in chunk j (rare)
    auto rescale_moved = [&](int j) {
        const int pb = j & 1;
        const int4 mv = *reinterpret_cast<const int4 *>(sh.moved[pb]);
        if (__builtin_expect((mv.x | mv.y | mv.z | mv.w) != 0, 0)) {
            mfma_settle();
            const int mvs[4] = {mv.x, mv.y, mv.z, mv.w};
            static_for<0, 4>([&](auto hg_) {
                constexpr int hg = decltype(hg_)::value;
                if (mvs[hg]) {
                    const float ag = sh.alpha[pb][hg * 32 + ln];
                    static_for<0, 4>([&](auto cc_) {
                        constexpr int cc = decltype(cc_)::value;
                        static_for<0, 16>([&](auto r_) { acc_scale<16 * (4 * cc + hg) + decltype(r_)::value>(ag); });
                    });
                }
            });
            mfma_settle();
        }
    };
    typedef short v4s_t __attribute__((ext_vector_type(4)));
    // LDS addresses that depend on the tile or the parity of the chunk are formed once per step and HELD (made opaque):
    // left to itself the compiler re-adds the tile's base to the lane's offset in front of every read, and an add
    // costs this loop as much as any other instruction.
    auto lds_addr = [](const void *ptr) -> uint32_t {
        return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)ptr;
    };
    uint32_t va_addr[2][2];   // V^T operand reads of the output chunk's tile: [second four keys][odd column tile]
    auto read_va = [&](int half, int cc) -> u32x4_t {
        u32x4_t va;
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const v4s_t r4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) v4s_t *)(uintptr_t)(va_addr[jj][cc & 1] + half * (16 * kMlaRowBytes) + (cc >> 1) * 128));
            const uint2 r2 = __builtin_bit_cast(uint2, r4);
            va[2 * jj] = r2.x;
            va[2 * jj + 1] = r2.y;
        }
        return va;
    };
    // ---- the second half of a step: the 32 output products of chunk j_out (OUT) beside the softmax of chunk j_sm
    //      (SM), product by product.  Operands are requested from LDS a few products before they are used: the four
    //      P^T operands of a 16-key half stay for its 16 products (in the half's last quarter the products run
    //      head group by head group, and each operand is replaced by the next half's as soon as it is done with); two
    //      pairs of V^T operands alternate, the idle pair being filled for the next quarter; the scale vectors of a
    //      softmax slice arrive one slice ahead.  The one rare branch (softmax_check) sits after the first quarter.
    auto phase_b = [&](auto out_, auto sm_, int j_out, int tile_out, int j_sm, int tile_sm) {
        constexpr bool OUT = decltype(out_)::value, SM = decltype(sm_)::value;
        const int pb = j_out & 1;
        constexpr int tb0 = 0, tb1 = 1;   // the tile's two 16-key halves
        if constexpr (OUT) {
            const uint32_t tb = lds_addr(&sh.k[tile_out][0]);
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int c1 = 0; c1 < 2; ++c1) {
                    va_addr[jj][c1] = tb + (uint32_t)tr_off[jj][c1];
                    asm volatile("" : "+v"(va_addr[jj][c1]));
                }
        }
        u32x4_t pkg[4], va[2], vb[2];
        float4 sc0, sc1, sc2;
        uint2 sh2, sl2;
        if constexpr (OUT) {
            rescale_moved(j_out);
#pragma unroll
            for (int hg = 0; hg < 4; ++hg) pkg[hg] = sh.pk[pb][hg][0][lane];
            va[0] = read_va(tb0, 0);
            va[1] = read_va(tb0, 1);
        }
        if constexpr (SM) sc0 = load_ksl(tile_sm, 0);
        // quarter 0: half 0, column tiles 0 and 1; scaled scores and their maximum
        static_for<0, 8>([&](auto slot_) {
            constexpr int slot = decltype(slot_)::value;
            constexpr int c = slot >> 2, hg = slot & 3;
            if constexpr (OUT) {
                acc_mfma<T, 16 * (4 * c + hg)>(va[c], pkg[hg]);
                if constexpr (slot == 0) vb[0] = read_va(tb0, 2);
                if constexpr (slot == 2) vb[1] = read_va(tb0, 3);
            }
            if constexpr (SM && (slot & 1)) {
                constexpr int g = slot >> 1;
                const float4 cur = sc0;
                if constexpr (g < 3) sc0 = load_ksl(tile_sm, g + 1);
                softmax_scale4(g, cur);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (SM) {
            softmax_check(j_sm);
            sc1 = load_vs(tile_sm, 0);
            if constexpr (__is_same(T, BF16)) {
                sh2 = load_vsi_hi(tile_sm, 0);
                sl2 = load_vsi_lo(tile_sm, 0);
            } else {
                sc2 = load_vsi(tile_sm, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // quarter 1: half 0, column tiles 2 and 3, head group by head group; exponentials
        static_for<0, 8>([&](auto slot_) {
            constexpr int slot = decltype(slot_)::value;
            constexpr int hg = slot >> 1, c = slot & 1;
            if constexpr (OUT) {
                acc_mfma<T, 16 * (4 * (2 + c) + hg)>(vb[c], pkg[hg]);
                if constexpr (c == 1) pkg[hg] = sh.pk[pb][hg][1][lane];
                if constexpr (slot == 2) va[0] = read_va(tb1, 0);
                if constexpr (slot == 4) va[1] = read_va(tb1, 1);
            }
            if constexpr (SM && (slot & 1)) softmax_exp4(slot >> 1);
            __builtin_amdgcn_sched_barrier(0);
        });
        // quarters 2 and 3: half 1; sums, V-side scale, rounding
        static_for<0, 16>([&](auto slot_) {
            constexpr int slot = decltype(slot_)::value;
            constexpr int cc = slot >> 2, hg = slot & 3;
            if constexpr (OUT) {
                if constexpr (cc < 2)
                    acc_mfma<T, 16 * (4 * cc + hg)>(va[cc], pkg[hg]);
                else
                    acc_mfma<T, 16 * (4 * cc + hg)>(vb[cc - 2], pkg[hg]);
                if constexpr (slot == 0) vb[0] = read_va(tb1, 2);
                if constexpr (slot == 2) vb[1] = read_va(tb1, 3);
            }
            if constexpr (SM && (slot & 3) == 3) {
                constexpr int g = slot >> 2;
                const float4 cv = sc1, ci = sc2;
                const uint2 ch = sh2, cl = sl2;
                if constexpr (g < 3) {
                    sc1 = load_vs(tile_sm, g + 1);
                    if constexpr (__is_same(T, BF16)) {
                        sh2 = load_vsi_hi(tile_sm, g + 1);
                        sl2 = load_vsi_lo(tile_sm, g + 1);
                    } else {
                        sc2 = load_vsi(tile_sm, g + 1);
                    }
                }
                softmax_pack4(g, cv, ci, ch, cl);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (SM) softmax_store(j_sm);
    };
    using Yes = std::true_type;
    using No = std::false_type;

    // ---- the pipeline.  Chunk j lives in tile j % 3.
    //      step i: scores of chunk i beside the widening of chunk i+1 (the loads of chunk i+2 leave piece by piece),
    //              softmax of chunk i beside the output products of chunk i-1, one barrier.
    int blk_next;
    {
        fetch_setup(blk_first);
#pragma unroll
        for (int i = 0; i < kMlaRounds; ++i) fetch_piece(i);
        fetch_scales();
        blk_next = blk_second;
        stage_q();   // q was requested before the chunk: it is here first
#pragma unroll
        for (int i = 0; i < kMlaRounds; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) widen_quarter(0, i, q);
        stash_scales(0);
        fetch_setup(blk_next);
#pragma unroll
        for (int i = 0; i < kMlaRounds; ++i) fetch_piece(i);
        fetch_scales();
        blk_next = fetch_blk();
    }
    __syncthreads();
    int t_cur = 0;   // tile of chunk i
    for (int i = 0; i < nch; ++i) {
        const int t_nxt = (t_cur == 2) ? 0 : t_cur + 1;
        const int t_prv = (t_cur == 0) ? 2 : t_cur - 1;
        stash_scales(t_nxt);                // chunk i+1 (past the end: the last chunk again, into a tile nobody reads)
        fetch_setup(blk_next);
        fetch_scales();
        scores(t_cur, t_nxt);
        blk_next = fetch_blk();
        mfma_settle();
        __builtin_amdgcn_sched_barrier(0);
        if (i > 0)
            phase_b(Yes{}, Yes{}, i - 1, t_prv, i, t_cur);
        else
            phase_b(No{}, Yes{}, 0, 0, i, t_cur);
        __syncthreads();
        t_cur = t_nxt;
    }
    phase_b(Yes{}, No{}, nch - 1, (t_cur == 0) ? 2 : t_cur - 1, 0, 0);
    mfma_settle();

    // ---- sums of the two half-waves, LSE, normaliser to LDS for the column owners
    l_run = halves_sum(l_run);
    l_norm = halves_sum(l_norm);
    if (lh == 0) {
        sh.l[row_u] = (l_run > 0.f) ? l_norm : 0.f;
        if (head < p.nheads) {
            if (write_final)
                p.lse[((int64_t)b * p.nheads + head) * p.seqlen_q + qi] = (l_run > 0.f) ? (m_ref + fast_log2(l_run)) * kLn2 : INFINITY;
            else
                p.lse_partial[slot * p.rows + row_u] = (l_run > 0.f) ? m_ref + fast_log2(l_run) : -INFINITY;
        }
    }
    __syncthreads();
    // ---- write this wave's 128-column slice of every head.  A lane holds 16-byte pieces of 32 different rows: stored as
    //      they are, every instruction would touch 32 rows of the output.  The slice of one head group (32 rows x 128
    //      columns, fp32) goes through a staging area of the wave's own inside the key tiles (free after the barrier
    //      above) and leaves as whole rows, 16 bytes per lane.
    constexpr int kStageRowBytes = 128 * 4 + 16;                     // padded: the 16 lanes the LDS serves per cycle hit 64 banks
    static_assert(4 * 32 * kStageRowBytes <= 3 * kMlaTileBytes, "the staging areas must fit the key tiles");
    uint8_t *stage = &sh.k[0][0] + wave * (32 * kStageRowBytes);
    // Everything the stores need is derived from the lane number HERE: the walk over the pieces of a share is a loop,
    // and per-lane constants computed outside it would be kept alive through the main loop, where there is no
    // register to spare (they were spilled, and every reload waited for the store before it).
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int ln_e = lane_e & 31, lh_e = lane_e >> 5;
    static_for<0, 4>([&](auto hg_) {
        constexpr int hg = decltype(hg_)::value;
        const float lg = sh.l[hg * 32 + ln_e];
        const float inv = (lg > 0.f) ? 1.f / lg : 0.f;
        static_for<0, 16>([&](auto t_) {
            constexpr int cc = decltype(t_)::value >> 2, g = decltype(t_)::value & 3;
            constexpr int base = 16 * (4 * cc + hg) + 4 * g;
            const float o0 = acc_read<base>() * inv, o1 = acc_read<base + 1>() * inv;
            const float o2 = acc_read<base + 2>() * inv, o3 = acc_read<base + 3>() * inv;
            *reinterpret_cast<float4 *>(stage + ln_e * kStageRowBytes + (cc * 32 + g * 8 + 4 * lh_e) * 4) = make_float4(o0, o1, o2, o3);
        });
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int hd0 = hgrp * kMlaUnitHeads + hg * 32;               // head of the staged row 0
        // all LDS reads of the pass first (constant offsets from one address), then the stores (one pointer, constant
        // strides); a head group that is complete - every one but possibly the unit's last - needs no per-row test
        const bool full = hd0 + 32 <= p.nheads;                       // wave-uniform
        // 128 columns of a 16-bit type = 256 bytes = 16 lanes: four rows per instruction.  The final output is in the
        // I/O type; the partial rows of a split unit are fp16 (partials_are_half), clamped to its range.
        const int c = lane_e & 15, r0 = lane_e >> 4;
        const uint8_t *src = stage + r0 * kStageRowBytes + c * 32;
        const uint32_t src_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t *)src;
        float4 x[8], y[8];
        lds_read8x16<4 * kStageRowBytes>(src_lds, x);
        lds_read8x16<4 * kStageRowBytes>(src_lds + 16, y);
        uint16_t *dst;
        int64_t step;
        if (write_final) {
            dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                  (int64_t)(hd0 + r0) * p.o_stride_h + wave * 128 + c * 8;
            step = 4 * p.o_stride_h;
        } else {
            static_assert(partials_are_half(kMlaDv), "the merge reads these rows as fp16");
            dst = reinterpret_cast<uint16_t *>(p.o_partial) + (slot * p.rows + hg * 32 + r0) * kMlaDv + wave * 128 + c * 8;
            step = 4 * kMlaDv;
        }
        auto put = [&](int i) {
            if (write_final) {
                store16(dst + i * step, u32x4_t{pack2<T>(x[i].x, x[i].y), pack2<T>(x[i].z, x[i].w), pack2<T>(y[i].x, y[i].y),
                                                pack2<T>(y[i].z, y[i].w)});
            } else {
                auto cl = [](float v) { return __builtin_amdgcn_fmed3f(v, -65504.f, 65504.f); };
                store16(dst + i * step, u32x4_t{pack2<FP16>(cl(x[i].x), cl(x[i].y)), pack2<FP16>(cl(x[i].z), cl(x[i].w)),
                                                pack2<FP16>(cl(y[i].x), cl(y[i].y)), pack2<FP16>(cl(y[i].z), cl(y[i].w))});
            }
        };
        if (full) {
#pragma unroll
            for (int i = 0; i < 8; ++i) put(i);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (hd0 + r0 + 4 * i < p.nheads) put(i);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();   // the staging area is rewritten by the next head group
    });
    __syncthreads();   // the LDS tiles and sums are reused by the next piece
}

template <typename T, bool SOFTCAP>
__global__ void __launch_bounds__(kMlaThreads) decode_mla_i8_kernel(const DecodeParams p) {
    __shared__ MlaShared sh;
    // Neighbouring shares are mostly pieces of one batch row and read the same 147 KB of Q.  Workgroup x runs on XCD
    // x % 8 (each XCD has its own L2): the shares are dealt so that eight neighbours meet in one L2.
    const int G = gridDim.x;
    const int worker = (G & 7) ? (int)blockIdx.x : (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3);
    balanced_driver<kMlaDv>(p, worker, [&](int b, int unit, const UnitRange &ur, int range_lo, int range_hi, bool whole, int64_t slot) {
        mla_piece<T, SOFTCAP>(p, b, unit, ur, range_lo, range_hi, whole, slot, sh);
    });
}

// p.nheads_k counts units per batch row here (seqlen_q * 128-head groups), p.group = p.rows = 128.
hipError_t launch_decode_mla_i8(const DecodeParams &p, int dtype, hipStream_t stream) {
    if (p.units_per_token <= 0 || p.rows != kMlaUnitHeads || p.group != kMlaUnitHeads || !p.balanced)
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
