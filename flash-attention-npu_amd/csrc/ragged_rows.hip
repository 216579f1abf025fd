// One-token query blocks of a token-major batch, moved to and from the batch-major layout of the decode
// kernels.  A batch of prompt chunks and decode rows over a paged cache (the third-generation call
// surface, flash_attn_npu_3/flash_attn_npu_interface.py:965-996, takes such batches in one call) is
// served by two kernels: the decode kernels stream the keys of the one-token blocks, the tiled forward
// computes the others.  Which block is which is decided here, on the device, from cu_seqlens_q.
#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {

// grid: batch; block: 256.  Sequence b with exactly one query token: its q row (nheads x headdim) goes to
// row b of q_rows and lens_rows[b] = seqused_k[b]; every other sequence gets lens_rows[b] = 0, so that the
// decode launch over (q_rows, lens_rows) finds nothing to read for it.
__global__ void __launch_bounds__(256) gather_single_rows_kernel(const SingleRowsParams p) {
    const int b = blockIdx.x;
    const int q0 = p.cu_seqlens_q[b];
    const bool single = p.cu_seqlens_q[b + 1] - q0 == 1;
    if (threadIdx.x == 0) p.lens_rows[b] = single ? p.seqused_k[b] : 0;
    if (!single) return;
    const int pieces_per_head = p.headdim / 8;
    const uint16_t *src = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)q0 * p.q_stride_t;
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.q_rows) + (int64_t)b * p.nheads * p.headdim;
    for (int i = threadIdx.x; i < p.nheads * pieces_per_head; i += blockDim.x) {
        const int h = i / pieces_per_head, c = i - h * pieces_per_head;
        store16(dst + (int64_t)h * p.headdim + c * 8, load16(src + (int64_t)h * p.q_stride_h + c * 8));
    }
}

// grid: batch; block: 256.  The decode launch's row b (output and log-sum-exp) goes back to the token of
// sequence b when that sequence has exactly one query token.
__global__ void __launch_bounds__(256) scatter_single_rows_kernel(const SingleRowsParams p) {
    const int b = blockIdx.x;
    const int q0 = p.cu_seqlens_q[b];
    if (p.cu_seqlens_q[b + 1] - q0 != 1) return;
    const int pieces_per_head = p.headdim / 8;
    const uint16_t *src = reinterpret_cast<const uint16_t *>(p.out_rows) + (int64_t)b * p.nheads * p.headdim;
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)q0 * p.o_stride_t;
    for (int i = threadIdx.x; i < p.nheads * pieces_per_head; i += blockDim.x) {
        const int h = i / pieces_per_head, c = i - h * pieces_per_head;
        store16(dst + (int64_t)h * p.o_stride_h + c * 8, load16(src + (int64_t)h * p.headdim + c * 8));
    }
    for (int h = threadIdx.x; h < p.nheads; h += blockDim.x)
        p.lse[(int64_t)h * p.total_q + q0] = p.lse_rows[(int64_t)b * p.nheads + h];
}

hipError_t launch_gather_single_rows(const SingleRowsParams &p, hipStream_t stream) {
    if (p.batch <= 0) return hipSuccess;
    hipLaunchKernelGGL(gather_single_rows_kernel, dim3(p.batch), dim3(256), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_scatter_single_rows(const SingleRowsParams &p, hipStream_t stream) {
    if (p.batch <= 0) return hipSuccess;
    hipLaunchKernelGGL(scatter_single_rows_kernel, dim3(p.batch), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace fa
