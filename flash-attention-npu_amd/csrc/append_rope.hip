// In-place paged append of new K/V rows, rotary applied to K.
//
// Semantics are those the reference documents for flash_attn_with_kvcache
// (flash_attn_npu/flash_attn_npu_interface.py:1460-1474,1508-1513,1527-1530) and its host code
// accepts but drops (csrc/ascend910/flash_attn_npu/flash_api.cpp:422-427):
//   p = cache_seqlens[b] + t;  k_cache[block_table[b][p / page]][p % page][h] = rope(k_new[b][t][h], p)
//   v_cache[...] = v_new[b][t][h].
// Rotary arithmetic: operands widened to fp32, two separately rounded products and one separately
// rounded add/sub (never a fused multiply-add), result rounded to nearest-even in the cache dtype,
// so the written bytes can be compared bit-for-bit with a host computation.
#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {

// grid: (Hk, Snew, B); block: 64 threads striding over the element pairs of one head row
template <typename T>
__global__ void __launch_bounds__(64) append_kv_kernel(const AppendParams p) {
    // one-dimensional grid (the y and z extents stop at 65535): block = (b * seqlen_new + t) * nheads_k + h
    const int h = blockIdx.x % p.nheads_k;
    const int t = (blockIdx.x / p.nheads_k) % p.seqlen_new;
    const int b = blockIdx.x / (p.nheads_k * p.seqlen_new);
    const int pos = p.cache_seqlens[b] + t;
    if (pos < 0) return;
    const int page = pos / p.page_size;
    if (page >= p.max_blocks) return;   // no capacity: nothing is written
    const int blk = p.block_table[(int64_t)b * p.bt_stride_b + page];
    if (blk < 0 || blk >= p.num_blocks) return;
    const int inpage = pos - page * p.page_size;

    uint16_t *kdst = reinterpret_cast<uint16_t *>(p.k_cache) + (int64_t)blk * p.k_stride_block +
                     (int64_t)inpage * p.k_stride_row + (int64_t)h * p.k_stride_h;
    uint16_t *vdst = reinterpret_cast<uint16_t *>(p.v_cache) + (int64_t)blk * p.v_stride_block +
                     (int64_t)inpage * p.v_stride_row + (int64_t)h * p.v_stride_h;
    const uint16_t *ksrc = reinterpret_cast<const uint16_t *>(p.k_new) + (int64_t)b * p.kn_stride_b +
                           (int64_t)t * p.kn_stride_s + (int64_t)h * p.kn_stride_h;
    const uint16_t *vsrc = reinterpret_cast<const uint16_t *>(p.v_new) + (int64_t)b * p.vn_stride_b +
                           (int64_t)t * p.vn_stride_s + (int64_t)h * p.vn_stride_h;

    const uint16_t *cosT = reinterpret_cast<const uint16_t *>(p.rotary_cos);
    const uint16_t *sinT = reinterpret_cast<const uint16_t *>(p.rotary_sin);
    const int rot = (cosT != nullptr) ? p.rotary_dim : 0;
    const int half = rot >> 1;
    const int rpos = min(pos, p.seqlen_ro - 1);

    for (int c = threadIdx.x; c < p.headdim_qk / 2; c += 64) {
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
    if ((p.headdim_qk & 1) && threadIdx.x == 0) kdst[p.headdim_qk - 1] = ksrc[p.headdim_qk - 1];
    for (int d = threadIdx.x; d < p.headdim_v; d += 64) vdst[d] = vsrc[d];
}

// Quantising append into the int8 latent cache: one wave per new token.
//   scale = absmax / 127 (fp32, correctly rounded division); code = clamp(rne(x / scale), -127, 127);
//   an all-zero token gets scale 0 and codes 0.
// The codes go to k_cache (v_cache is a view of it), the scale to k_scale (and to v_scale when that
// is a separate tensor).  Every operation is a single correctly rounded fp32 operation, so codes
// and scales can be compared bit-for-bit with a host computation.
template <typename T>
__global__ void __launch_bounds__(64) append_quant_i8_kernel(const AppendParams p) {
    const int t = blockIdx.x % p.seqlen_new;     // one-dimensional grid: block = b * seqlen_new + t
    const int b = blockIdx.x / p.seqlen_new;
    const int lane = threadIdx.x;
    const int pos = p.cache_seqlens[b] + t;
    if (pos < 0) return;
    const int page = pos / p.page_size;
    if (page >= p.max_blocks) return;   // no capacity: nothing is written
    const int blk = p.block_table[(int64_t)b * p.bt_stride_b + page];
    if (blk < 0 || blk >= p.num_blocks) return;
    const int inpage = pos - page * p.page_size;
    const int d = p.headdim_qk;

    const uint16_t *src = reinterpret_cast<const uint16_t *>(p.k_new) + (int64_t)b * p.kn_stride_b + (int64_t)t * p.kn_stride_s;
    int8_t *dst = reinterpret_cast<int8_t *>(p.k_cache) + (int64_t)blk * p.k_stride_block + (int64_t)inpage * p.k_stride_row;

    float absmax = 0.f;
    for (int e = lane; e < d; e += 64) absmax = fmaxf(absmax, fabsf(to_float<T>(src[e])));
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) absmax = fmaxf(absmax, __shfl_xor(absmax, m, 64));
    const float scale = __fdiv_rn(absmax, 127.0f);
    for (int e = lane; e < d; e += 64) {
        float c = 0.f;
        if (scale > 0.f) c = fminf(fmaxf(rintf(__fdiv_rn(to_float<T>(src[e]), scale)), -127.f), 127.f);
        dst[e] = (int8_t)(int)c;
    }
    if (lane == 0) {
        const int64_t so = (int64_t)blk * p.ks_stride_block + (int64_t)inpage * p.ks_stride_row;
        p.k_scale[so] = scale;
        if (p.v_scale && p.v_scale != p.k_scale) p.v_scale[so] = scale;
    }
}

hipError_t launch_append_quant_i8(const AppendParams &p, int dtype, hipStream_t stream) {
    if ((int64_t)p.seqlen_new * p.batch > INT32_MAX) return hipErrorInvalidValue;
    dim3 grid((unsigned)(p.seqlen_new * p.batch));
    if (dtype == 0)
        hipLaunchKernelGGL(append_quant_i8_kernel<BF16>, grid, dim3(64), 0, stream, p);
    else
        hipLaunchKernelGGL(append_quant_i8_kernel<FP16>, grid, dim3(64), 0, stream, p);
    return hipGetLastError();
}

// q rotated at position cache_seqlens[b] + i (per-token) or cache_seqlens[b] (all tokens alike),
// same arithmetic as the append (flash_attn_npu_interface.py:1469-1474).  grid: (Hq, Sq, B)
template <typename T>
__global__ void __launch_bounds__(64) rotate_q_kernel(const RotateQParams p) {
    const int h = blockIdx.x % p.nheads;         // one-dimensional grid: block = (b * seqlen_q + i) * nheads + h
    const int i = (blockIdx.x / p.nheads) % p.seqlen_q;
    const int b = blockIdx.x / (p.nheads * p.seqlen_q);
    const int pos = p.cache_seqlens[b] + (p.rotary_per_token ? i : 0);
    const int rpos = min(max(pos, 0), p.seqlen_ro - 1);
    const uint16_t *src = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_stride_b + (int64_t)i * p.q_stride_s +
                          (int64_t)h * p.q_stride_h;
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (((int64_t)b * p.seqlen_q + i) * p.nheads + h) * p.headdim;
    const uint16_t *cosT = reinterpret_cast<const uint16_t *>(p.rotary_cos);
    const uint16_t *sinT = reinterpret_cast<const uint16_t *>(p.rotary_sin);
    const int rot = p.rotary_dim;
    const int half = rot >> 1;
    for (int c = threadIdx.x; c < p.headdim / 2; c += 64) {
        int d1, d2;
        if (c < half) {
            d1 = p.rotary_interleaved ? 2 * c : c;
            d2 = p.rotary_interleaved ? 2 * c + 1 : c + half;
        } else {
            d1 = rot + 2 * (c - half);
            d2 = d1 + 1;
        }
        uint16_t o1 = src[d1], o2 = src[d2];
        if (c < half) {
            const float cs = to_float<T>(cosT[(int64_t)rpos * half + c]);
            const float sn = to_float<T>(sinT[(int64_t)rpos * half + c]);
            const float x1 = to_float<T>(o1), x2 = to_float<T>(o2);
            float r1, r2;
            rotate_pair(x1, x2, cs, sn, r1, r2);
            o1 = from_float<T>(r1);
            o2 = from_float<T>(r2);
        }
        dst[d1] = o1;
        dst[d2] = o2;
    }
}

hipError_t launch_rotate_q(const RotateQParams &p, int dtype, hipStream_t stream) {
    if ((int64_t)p.nheads * p.seqlen_q * p.batch > INT32_MAX) return hipErrorInvalidValue;
    dim3 grid((unsigned)(p.nheads * p.seqlen_q * p.batch));
    if (dtype == 0)
        hipLaunchKernelGGL(rotate_q_kernel<BF16>, grid, dim3(64), 0, stream, p);
    else
        hipLaunchKernelGGL(rotate_q_kernel<FP16>, grid, dim3(64), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_append_kv(const AppendParams &p, int dtype, hipStream_t stream) {
    if ((int64_t)p.nheads_k * p.seqlen_new * p.batch > INT32_MAX) return hipErrorInvalidValue;
    dim3 grid((unsigned)(p.nheads_k * p.seqlen_new * p.batch));
    if (dtype == 0)
        hipLaunchKernelGGL(append_kv_kernel<BF16>, grid, dim3(64), 0, stream, p);
    else
        hipLaunchKernelGGL(append_kv_kernel<FP16>, grid, dim3(64), 0, stream, p);
    return hipGetLastError();
}

}  // namespace fa
