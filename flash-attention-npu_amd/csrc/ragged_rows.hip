// Short query blocks of a token-major batch, moved to and from the batch-major layout of the decode
// kernels.  A batch of prompt chunks and decode rows over a paged cache (the third-generation call
// surface, flash_attn_npu_3/flash_attn_npu_interface.py:965-996, takes such batches in one call) is
// served by two kernels: the decode kernels stream the keys of the short blocks, the tiled forward
// computes the others.  Which block is which is decided here, on the device, from cu_seqlens_q.
//
// A short block has 1 .. slots query tokens.  In the batch-major copy every sequence owns `slots` query
// positions and a block of n tokens fills the LAST n of them: position slots - n + t of a block aligned
// to the end of Lk keys sees the keys up to Lk - slots + (slots - n + t) = Lk - n + t, which is what
// token t of an n-token block sees on its own (the same holds for both window sides).  The positions in
// front are zero rows whose results nobody reads.
#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {

// grid: batch; block: 256.  Sequence b with 1 .. slots query tokens: its q rows go to the tail of block b
// of q_rows and lens_rows[b] = seqused_k[b]; every other sequence gets lens_rows[b] = 0, so that the decode
// launch over (q_rows, lens_rows) finds nothing to read for it.
__global__ void __launch_bounds__(256) gather_short_blocks_kernel(const ShortBlocksParams p) {
    const int b = blockIdx.x;
    const int q0 = p.cu_seqlens_q[b];
    const int n = p.cu_seqlens_q[b + 1] - q0;
    const bool is_short = n >= 1 && n <= p.slots;
    if (threadIdx.x == 0) {
        p.lens_rows[b] = is_short ? p.seqused_k[b] : 0;
        p.live_rows[b] = is_short ? n : 0;
    }
    if (b == 0 && p.long_ids) {
        // the sequences left to the tiled kernel, in batch order: flags counted wave by wave, 256 sequences a pass
        __shared__ int s_wave[4];
        int done = 0;
        for (int base = 0; base < p.batch; base += 256) {
            const int i = base + threadIdx.x;
            const bool is_long = i < p.batch && p.cu_seqlens_q[i + 1] - p.cu_seqlens_q[i] > p.slots;
            const uint64_t mask = __ballot(is_long);
            const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
            if (lane == 0) s_wave[wave] = __popcll(mask);
            __syncthreads();
            int before = done;
            for (int w = 0; w < wave; ++w) before += s_wave[w];
            if (is_long) p.long_ids[before + __popcll(mask & ((1ull << lane) - 1))] = i;
            done += s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
            __syncthreads();
        }
        if (threadIdx.x == 0) p.list_state[0] = done;
        if (threadIdx.x >= 1 && threadIdx.x <= 8) p.list_state[threadIdx.x] = 0;
    }
    const int pieces_per_head = p.headdim / 8;
    const int pieces_per_token = p.nheads * pieces_per_head;
    const int pad = is_short ? p.slots - n : p.slots;
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.q_rows) + (int64_t)b * p.slots * p.nheads * p.headdim;
    for (int i = threadIdx.x; i < p.slots * pieces_per_token; i += blockDim.x) {
        const int s = i / pieces_per_token, r = i - s * pieces_per_token;
        const int h = r / pieces_per_head, c = r - h * pieces_per_head;
        u32x4_t v = u32x4_t{0, 0, 0, 0};
        if (s >= pad)
            v = load16(reinterpret_cast<const uint16_t *>(p.q) + (int64_t)(q0 + s - pad) * p.q_stride_t + (int64_t)h * p.q_stride_h + c * 8);
        store16(dst + ((int64_t)s * p.nheads + h) * p.headdim + c * 8, v);
    }
}

// grid: batch; block: 256.  The tail of the decode launch's block b (outputs, and log-sum-exps laid out
// (batch, head, slot)) goes back to the tokens of sequence b when that sequence is a short block.
__global__ void __launch_bounds__(256) scatter_short_blocks_kernel(const ShortBlocksParams p) {
    const int b = blockIdx.x;
    const int q0 = p.cu_seqlens_q[b];
    const int n = p.cu_seqlens_q[b + 1] - q0;
    if (n < 1 || n > p.slots) return;
    const int pad = p.slots - n;
    const int pieces_per_head = p.headdim / 8;
    const int pieces_per_token = p.nheads * pieces_per_head;
    const uint16_t *src = reinterpret_cast<const uint16_t *>(p.out_rows) + (int64_t)b * p.slots * p.nheads * p.headdim;
    for (int i = threadIdx.x; i < n * pieces_per_token; i += blockDim.x) {
        const int t = i / pieces_per_token, r = i - t * pieces_per_token;
        const int h = r / pieces_per_head, c = r - h * pieces_per_head;
        store16(reinterpret_cast<uint16_t *>(p.out) + (int64_t)(q0 + t) * p.o_stride_t + (int64_t)h * p.o_stride_h + c * 8,
                load16(src + ((int64_t)(pad + t) * p.nheads + h) * p.headdim + c * 8));
    }
    for (int i = threadIdx.x; i < n * p.nheads; i += blockDim.x) {
        const int t = i / p.nheads, h = i - t * p.nheads;
        p.lse[(int64_t)h * p.total_q + q0 + t] = p.lse_rows[((int64_t)b * p.nheads + h) * p.slots + pad + t];
    }
}

hipError_t launch_gather_short_blocks(const ShortBlocksParams &p, hipStream_t stream) {
    if (p.batch <= 0 || p.slots <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gather_short_blocks_kernel, dim3(p.batch), dim3(256), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_scatter_short_blocks(const ShortBlocksParams &p, hipStream_t stream) {
    if (p.batch <= 0 || p.slots <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(scatter_short_blocks_kernel, dim3(p.batch), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace fa
