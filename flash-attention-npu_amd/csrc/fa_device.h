// Device-side helpers shared by the gfx950 attention kernels: 16-bit element traits,
// MFMA wrappers for the two I/O dtypes, packing, wave-level exchanges.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fa {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 half8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float float4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float float16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

struct BF16 {};
struct FP16 {};

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---- scalar conversions (round-to-nearest-even) ------------------------------------------
template <typename T> __device__ __forceinline__ float to_float(uint16_t bits);
template <> __device__ __forceinline__ float to_float<BF16>(uint16_t bits) {
    return __uint_as_float(static_cast<uint32_t>(bits) << 16);
}
template <> __device__ __forceinline__ float to_float<FP16>(uint16_t bits) {
    _Float16 h;
    __builtin_memcpy(&h, &bits, 2);
    return static_cast<float>(h);
}

template <typename T> __device__ __forceinline__ uint16_t from_float(float f);
template <> __device__ __forceinline__ uint16_t from_float<BF16>(float f) {
    __bf16 h = static_cast<__bf16>(f);   // RNE on gfx950 (v_cvt_pk_bf16_f32)
    uint16_t b;
    __builtin_memcpy(&b, &h, 2);
    return b;
}
template <> __device__ __forceinline__ uint16_t from_float<FP16>(float f) {
    _Float16 h = static_cast<_Float16>(f);
    uint16_t b;
    __builtin_memcpy(&b, &h, 2);
    return b;
}

// two floats -> one dword holding (lo = a, hi = b) in the 16-bit type, round-to-nearest-even
// (bf16: one v_cvt_pk_bf16_f32)
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 half2_t;
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<BF16>(float a, float b) {
    const bf16x2_t v = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
    return __builtin_bit_cast(uint32_t, v);
}
template <> __device__ __forceinline__ uint32_t pack2<FP16>(float a, float b) {
    const half2_t v = {static_cast<_Float16>(a), static_cast<_Float16>(b)};
    return __builtin_bit_cast(uint32_t, v);
}

// ---- MFMA 16x16x32: D(16x16) += A(16x32) * B(32x16), 16-bit inputs, fp32 accumulate -------
// Lane l holds A[l%16][8*(l/16) .. +7], B[8*(l/16) .. +7][l%16], D[4*(l/16) + r][l%16], r = 0..3.
template <typename T>
__device__ __forceinline__ float4_t mfma16(const u32x4_t &a, const u32x4_t &b, const float4_t &c);
template <>
__device__ __forceinline__ float4_t mfma16<BF16>(const u32x4_t &a, const u32x4_t &b, const float4_t &c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
}
template <>
__device__ __forceinline__ float4_t mfma16<FP16>(const u32x4_t &a, const u32x4_t &b, const float4_t &c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0,
                                                  0, 0);
}

// ---- MFMA 32x32x16: D(32x32) += A(32x16) * B(16x32) ---------------------------------------
// Lane l holds A[l%32][8*(l/32) .. +7], B[8*(l/32) .. +7][l%32],
// D[8*(r/4) + 4*(l/32) + r%4][l%32], r = 0..15.
template <typename T>
__device__ __forceinline__ float16_t mfma32(const u32x4_t &a, const u32x4_t &b, const float16_t &c);
template <>
__device__ __forceinline__ float16_t mfma32<BF16>(const u32x4_t &a, const u32x4_t &b, const float16_t &c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
}
template <>
__device__ __forceinline__ float16_t mfma32<FP16>(const u32x4_t &a, const u32x4_t &b, const float16_t &c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0,
                                                  0, 0);
}

// ---- wave-level exchanges -------------------------------------------------------------------
__device__ __forceinline__ float xor_shuffle(float v, int lane_mask) { return __shfl_xor(v, lane_mask, 64); }

// max / sum over the four lanes {n, n+16, n+32, n+48}, in the vector ALU: the gfx950 permlane
// swaps trade rows (16 lanes) and halves (32 lanes) between two registers, so with both operands
// the same value the two results hold v[lane] and v[lane ^ 16] (resp. ^ 32) in some order -
// enough for a symmetric reduction, and without the LDS round trip of a bpermute
__device__ __forceinline__ float quad_rows_max(float v) {
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
// max / sum over the two lanes {n, n ^ 32}
__device__ __forceinline__ float halves_max(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float quad_rows_sum(float v) {
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// One rotary pair: (x1, x2) turned by the angle whose cosine and sine are c and s.  The two products and
// the sum or difference of each result are separately rounded fp32 operations.  hipcc would otherwise fuse
// a product into the addition (and, for fp16 results, the conversion as well), which rounds differently on
// rare inputs; rotated rows are defined to be bit-identical to the unfused evaluation on a CPU.
__device__ __forceinline__ void rotate_pair(float x1, float x2, float c, float s, float &r1, float &r2) {
#pragma clang fp contract(off)
    const float a = x1 * c, b = x2 * s;
    const float e = x1 * s, f = x2 * c;
    r1 = a - b;
    r2 = e + f;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Window normalisation of the reference host (csrc/ascend910/flash_attn_npu/flash_api.cpp:483-505):
// a side >= M is unbounded, causal forces right = 0; if what remains is a true window (not plain
// causal), an unbounded side becomes M.  On return -1 still means unbounded.
__device__ __forceinline__ void normalize_window(int &wl, int &wr, int causal, int M) {
    if (M > 0 && wl >= M) wl = -1;
    if (M > 0 && wr >= M) wr = -1;
    if (causal) wr = 0;
    const bool is_causal = wl < 0 && wr == 0;
    const bool is_local = (wl >= 0 || wr >= 0) && !is_causal;
    if (is_local) {
        if (wl < 0) wl = M;
        if (wr < 0) wr = M;
    }
}

// Largest key count of the batch, max_b(seqlens[b] + add): the M of the window normalisation, which
// the reference obtains by copying the lengths to the host (flash_api.cpp:459,477-481).  Every
// thread of the workgroup must call; the result is the same in all of them.
__device__ __forceinline__ int block_max_keys(const int32_t *seqlens, int batch, int add) {
    __shared__ int s_max[16];
    int m = 0;
    for (int b = threadIdx.x; b < batch; b += blockDim.x) m = max(m, seqlens[b] + add);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) m = max(m, __shfl_xor(m, d, 64));
    const int nw = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = m;
    __syncthreads();
    m = s_max[0];
    for (int w = 1; w < nw; ++w) m = max(m, s_max[w]);
    __syncthreads();
    return m;
}

// Keys per split when a launch cuts every unit into at most `nsplits` ranges and the cut is sized on
// the device from the longest sequence of the batch (a multiple of 256 keys).  The kernel that
// writes the partial results and the one that merges them must agree on it.
__device__ __forceinline__ int adaptive_split_keys(int max_keys, int nsplits) {
    const int per = (max(max_keys, 1) + nsplits - 1) / nsplits;
    return (per + 255) / 256 * 256;
}

// 16-byte global load / store through plain vector types
// Cut of the keys a query block of Sq rows over Sk keys can see (window already normalised) into ranges of
// `split_keys` keys, counted from the 32-aligned first visible key; at most `nsplits` ranges, the last one
// takes the rest.  A block that sees nothing has one (empty) range.  The kernel that writes the partial
// results and the one that merges them derive the cut from this one function.
struct KeyRanges {
    int lo, hi;      // visible keys of the block: [lo, hi)
    int count;       // ranges the block is cut into (>= 1)
    int first;       // 32-aligned start of range 0
    __device__ __forceinline__ int begin(int r, int split_keys) const { return max(lo, first + r * split_keys); }
    __device__ __forceinline__ int end(int r, int split_keys) const {
        return (r == count - 1) ? hi : min(hi, first + (r + 1) * split_keys);
    }
};
__device__ __forceinline__ KeyRanges key_ranges(int Sq, int Sk, int wl, int wr, int split_keys, int nsplits) {
    KeyRanges kr;
    const int off = Sk - Sq;
    kr.lo = 0;
    kr.hi = Sk;
    if (wr >= 0) kr.hi = min(Sk, Sq - 1 + off + wr + 1);
    if (wl >= 0) kr.lo = max(0, off - wl);
    const bool empty = Sk <= 0 || kr.hi <= kr.lo;
    kr.first = kr.lo / 32 * 32;
    kr.count = empty ? 1 : min(nsplits, (kr.hi - kr.first + split_keys - 1) / split_keys);
    if (empty) kr.hi = kr.lo;
    return kr;
}

__device__ __forceinline__ u32x4_t load16(const void *p) { return *reinterpret_cast<const u32x4_t *>(p); }
// the same load marked non-temporal: data that is read once (the KV stream) need not stay in the caches
__device__ __forceinline__ u32x4_t load16_stream(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
}
__device__ __forceinline__ void store16(void *p, const u32x4_t &v) { *reinterpret_cast<u32x4_t *>(p) = v; }

}  // namespace fa
