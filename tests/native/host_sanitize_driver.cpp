// Host-only exerciser of the library's validators and planners, meant to be built with AddressSanitizer and
// UndefinedBehaviorSanitizer on the HOST pass only (tests/test_host_sanitizers.py holds the command) and run without a GPU.
// It links the real fa_rocm_api.cpp; the kernel launchers are replaced by stubs that are never reached, because no
// entry point that enqueues work is called.  Every integer field of both argument records is swept over edge values
// (negative, zero, odd, the 16-bit grid limits, INT_MAX) on top of several valid base calls, so that an overflow, a
// division by zero or an out-of-range shift in the size arithmetic trips a sanitizer; any report makes the run fail.
#include <climits>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../flash-attention-npu_amd/csrc/fa_kernels.h"
#include "../../include/fa_rocm.h"

namespace fa {
hipError_t launch_append_kv(const AppendParams &, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_append_quant_i8(const AppendParams &, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_rotate_q(const RotateQParams &, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_decode_paged(const DecodeParams &, int, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_decode_wave(const DecodeParams &, int, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_splitkv_combine(const DecodeParams &, int, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_decode_mla_i8(const DecodeParams &, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_prefill(const PrefillParams &, int, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_prefill_combine(const PrefillParams &, int, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_gather_short_blocks(const ShortBlocksParams &, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_scatter_short_blocks(const ShortBlocksParams &, hipStream_t) { return hipErrorNotSupported; }
}  // namespace fa

namespace {

// never dereferenced by the functions under test: any non-null value stands for a device pointer
void *const kPtr = reinterpret_cast<void *>(0x1000);

const int32_t kEdges[] = {INT_MIN, -65536, -2, -1, 0, 1, 2, 3, 15, 16, 17, 31, 32, 33, 64, 127, 128, 129, 255, 256, 257,
                          512, 576, 4095, 4096, 65535, 65536, 1 << 20, INT_MAX - 1, INT_MAX};

fa_kvcache_args kv_base(int batch, int seqlen_q, int hq, int hk, int d, int dv, int page, int blocks_per_seq, int dtype, int kv_dtype,
                        int seqlen_new, int num_splits) {
    fa_kvcache_args a;
    std::memset(&a, 0, sizeof(a));
    a.q = a.out = a.k_cache = a.v_cache = kPtr;
    a.softmax_lse = static_cast<float *>(kPtr);
    a.cache_seqlens = a.block_table = static_cast<const int32_t *>(kPtr);
    if (kv_dtype == FA_INT8) a.k_scale_cache = a.v_scale_cache = static_cast<float *>(kPtr);
    if (seqlen_new) a.k_new = a.v_new = kPtr;
    a.batch = batch, a.seqlen_q = seqlen_q, a.nheads = hq, a.nheads_k = hk, a.headdim_qk = d, a.headdim_v = dv;
    a.seqlen_new = seqlen_new;
    a.page_size = page, a.max_blocks_per_seq = blocks_per_seq, a.num_blocks = batch * blocks_per_seq;
    a.q_stride_h = d, a.q_stride_s = (int64_t)hq * d, a.q_stride_b = a.q_stride_s * seqlen_q;
    a.o_stride_h = dv, a.o_stride_s = (int64_t)hq * dv, a.o_stride_b = a.o_stride_s * seqlen_q;
    a.k_stride_h = d, a.k_stride_row = (int64_t)hk * d, a.k_stride_block = a.k_stride_row * page;
    a.v_stride_h = kv_dtype == FA_INT8 ? d : dv, a.v_stride_row = (int64_t)hk * a.v_stride_h, a.v_stride_block = a.v_stride_row * page;
    a.ks_stride_row = hk, a.ks_stride_block = (int64_t)hk * page;
    a.kn_stride_h = d, a.kn_stride_s = (int64_t)hk * d, a.kn_stride_b = a.kn_stride_s * (seqlen_new ? seqlen_new : 1);
    a.vn_stride_h = a.kn_stride_h, a.vn_stride_s = a.kn_stride_s, a.vn_stride_b = a.kn_stride_b;
    a.bt_stride_b = blocks_per_seq;
    a.io_dtype = dtype, a.kv_dtype = kv_dtype;
    a.softmax_scale = 0.1f;
    a.window_left = a.window_right = -1;
    a.num_splits = num_splits;
    return a;
}

fa_varlen_args vl_base(int batch, int total_q, int hq, int hk, int d, int max_q, int max_k, bool paged, int num_splits) {
    fa_varlen_args a;
    std::memset(&a, 0, sizeof(a));
    a.q = a.k = a.v = a.out = kPtr;
    a.softmax_lse = static_cast<float *>(kPtr);
    a.cu_seqlens_q = a.cu_seqlens_k = static_cast<const int32_t *>(kPtr);
    a.batch = batch, a.total_q = total_q, a.nheads = hq, a.nheads_k = hk, a.headdim = d;
    a.max_seqlen_q = max_q, a.max_seqlen_k = max_k;
    a.q_stride_h = d, a.q_stride_t = (int64_t)hq * d, a.o_stride_h = d, a.o_stride_t = a.q_stride_t;
    a.k_stride_h = a.v_stride_h = d, a.k_stride_t = a.v_stride_t = (int64_t)hk * d;
    if (paged) {
        a.seqused_k = a.block_table = static_cast<const int32_t *>(kPtr);
        a.page_size = 128, a.max_blocks_per_seq = (max_k + 127) / 128, a.num_blocks = batch * a.max_blocks_per_seq;
        a.k_stride_block = a.v_stride_block = a.k_stride_t * 128;
        a.bt_stride_b = a.max_blocks_per_seq;
    }
    a.io_dtype = FA_BF16;
    a.softmax_scale = 0.1f;
    a.window_left = a.window_right = -1;
    a.num_splits = num_splits;
    return a;
}

long g_calls = 0, g_ok = 0;

void probe(const fa_kvcache_args &a) {
    for (int cus : {0, 1, 256, 304}) {
        fa_split_plan plan;
        const int rv = fa_rocm_kvcache_validate(&a);
        const int rp = fa_rocm_plan_kvcache(&a, cus, &plan);
        const size_t ws = fa_rocm_kvcache_workspace_bytes(&a, cus);
        ++g_calls;
        if (rv == FA_OK && rp == FA_OK) {
            ++g_ok;
            if (ws != plan.workspace_bytes) {
                std::printf("workspace_bytes %zu differs from the plan's %zu\n", ws, plan.workspace_bytes);
                std::exit(2);
            }
        }
        if (rv != FA_OK && fa_rocm_last_error()[0] == 0) {
            std::printf("validate failed with code %d and no message\n", rv);
            std::exit(2);
        }
    }
}

void probe(const fa_varlen_args &a) {
    for (int cus : {0, 1, 256}) {
        const int rv = fa_rocm_varlen_validate(&a);
        const int ns = fa_rocm_varlen_num_splits(&a, cus);
        const size_t ws = fa_rocm_varlen_workspace_bytes(&a, cus);
        ++g_calls;
        if (rv == FA_OK) ++g_ok;
        (void)ns;
        (void)ws;
    }
}

template <class Args>
void sweep_i32(const Args &base, std::initializer_list<int32_t Args::*> fields) {
    probe(base);
    for (auto f : fields)
        for (int32_t e : kEdges) {
            Args a = base;
            a.*f = e;
            probe(a);
        }
    // pairs of fields at their largest accepted-looking values: products of two dimensions are where sizes overflow
    for (auto f : fields)
        for (auto g : fields) {
            if (f == g) continue;
            for (int32_t e : {65535, 1 << 20, INT_MAX}) {
                Args a = base;
                a.*f = e;
                a.*g = e;
                probe(a);
            }
        }
}

}  // namespace

int main() {
    std::vector<fa_kvcache_args> kv = {
        kv_base(128, 1, 32, 8, 128, 128, 128, 32, FA_BF16, FA_BF16, 1, 0),    // decode, balanced partition, append
        kv_base(4, 1, 32, 8, 128, 128, 128, 64, FA_FP16, FA_FP16, 0, 8),      // explicit split count
        kv_base(2, 64, 32, 8, 128, 128, 128, 64, FA_BF16, FA_BF16, 64, 0),    // tall query block: tiled kernel
        kv_base(64, 1, 128, 1, 576, 512, 64, 64, FA_BF16, FA_INT8, 1, 0),     // int8 latent cache
        kv_base(3, 2, 14, 2, 64, 64, 16, 9, FA_BF16, FA_BF16, 2, 1),          // odd group, small pages, no split
    };
    for (const auto &b : kv)
        sweep_i32<fa_kvcache_args>(b, {&fa_kvcache_args::batch, &fa_kvcache_args::seqlen_q, &fa_kvcache_args::nheads, &fa_kvcache_args::nheads_k,
                                       &fa_kvcache_args::headdim_qk, &fa_kvcache_args::headdim_v, &fa_kvcache_args::seqlen_new,
                                       &fa_kvcache_args::num_blocks, &fa_kvcache_args::page_size, &fa_kvcache_args::max_blocks_per_seq,
                                       &fa_kvcache_args::rotary_dim, &fa_kvcache_args::seqlen_ro, &fa_kvcache_args::io_dtype,
                                       &fa_kvcache_args::kv_dtype, &fa_kvcache_args::causal, &fa_kvcache_args::window_left,
                                       &fa_kvcache_args::window_right, &fa_kvcache_args::num_splits});
    std::vector<fa_varlen_args> vl = {
        vl_base(8, 32768, 32, 8, 128, 4096, 4096, false, 0),   // packed prefill
        vl_base(4, 2048, 32, 8, 128, 512, 16384, true, 0),     // paged, chunked prefill
        vl_base(64, 70, 32, 8, 128, 4, 8192, true, 0),         // paged, decode rows with a few tokens each
        vl_base(16, 16 + 4095, 16, 16, 64, 4096, 8192, true, 4),   // one prompt among decode rows
    };
    for (const auto &b : vl)
        sweep_i32<fa_varlen_args>(b, {&fa_varlen_args::batch, &fa_varlen_args::total_q, &fa_varlen_args::nheads, &fa_varlen_args::nheads_k,
                                      &fa_varlen_args::headdim, &fa_varlen_args::max_seqlen_q, &fa_varlen_args::max_seqlen_k,
                                      &fa_varlen_args::page_size, &fa_varlen_args::max_blocks_per_seq, &fa_varlen_args::num_blocks,
                                      &fa_varlen_args::io_dtype, &fa_varlen_args::causal, &fa_varlen_args::window_left,
                                      &fa_varlen_args::window_right, &fa_varlen_args::num_splits});
    // null pointers, one at a time
    for (const auto &b : kv) {
        for (const void *fa_kvcache_args::*f : {&fa_kvcache_args::q, &fa_kvcache_args::k_new, &fa_kvcache_args::v_new, &fa_kvcache_args::rotary_cos}) {
            fa_kvcache_args a = b;
            a.*f = nullptr;
            probe(a);
        }
        fa_kvcache_args a = b;
        a.block_table = nullptr;
        probe(a);
        a = b;
        a.cache_seqlens = nullptr;
        probe(a);
    }
    std::printf("host sanitizer sweep: %ld calls, %ld accepted\n", g_calls, g_ok);
    if (g_ok == 0) return 3;   // the base records must be valid, or the sweep only exercises the first check
    return 0;
}
