// C ABI of the library: argument validation, split planning, workspace sizing and kernel
// sequencing for one flash_attn_with_kvcache / flash_attn_varlen_func forward call.
//
// Host-side counterpart of the reference's mha_fwd_kvcache and mha_varlen_fwd
// (csrc/ascend910/flash_attn_npu/flash_api.cpp:356-637 and :848-1089).  Unlike those it never
// copies cache_seqlens to the host, uploads no mask and no tiling block: every decision made here
// depends on shapes only, per-row lengths are read by the kernels.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <climits>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/fa_rocm.h"
#include "fa_kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

constexpr float kLog2e = 1.4426950408889634f;

int device_cus() {
    // cached per host thread and device; a property query, not an allocation
    thread_local int cached_dev = -1;
    thread_local int cached_cus = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return -1;
    if (dev != cached_dev) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -1;
        cached_dev = dev;
        cached_cus = cus;
    }
    return cached_cus;
}

bool is_mla_i8(const fa_kvcache_args *a) { return a->kv_dtype == FA_INT8; }
bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// columns of a row of fp32 partials: the width the kernels are compiled for
int partial_width(const fa_kvcache_args *a) { return is_mla_i8(a) ? a->headdim_v : fa::tile_headdim(a->headdim_v); }
// bytes of one partial row in the workspace: its columns (fp16 for the 512-column latent kernel, fp32 otherwise) and
// its fp32 log-sum-exp
size_t partial_row_bytes(const fa_kvcache_args *a) {
    const int w = partial_width(a);
    return (size_t)w * (fa::partials_are_half(w) ? sizeof(uint16_t) : sizeof(float)) + sizeof(float);
}

// Experiment knobs and the validation switch, from the environment.  They are read ONCE, on the first call that
// needs them (or again when fa_rocm_reload_env() is called): nothing on the call path touches the environment.
struct EnvKnobs {
    int decode_max_rows = 0;       // FA_ROCM_DECODE_MAX_ROWS: 16 or 32, else the built-in rule
    int wave_max_rows = 0;         // FA_ROCM_WAVE_MAX_ROWS: 16, 32, 48 or 64: tallest block cut into 16-row tiles for the wave-level kernel
    int wave_two_tiles = 0;        // FA_ROCM_WAVE_TWO_TILES=1: 17-32-row blocks as two tiles in one wave whatever the number of units
    int decode_wgs = 0;            // FA_ROCM_DECODE_WGS: workgroups of the balanced partition
    bool block_workers = false;    // FA_ROCM_DECODE_BLOCK_WORKERS
    int min_share = 0;             // FA_ROCM_MIN_SHARE
    int piece_cost = -1;           // FA_ROCM_PIECE_COST
    bool no_head_interleave = false, separate_append = false, no_short_blocks = false;
    bool validate = false;         // FA_ROCM_VALIDATE: check tables, capacities and positions on the device (slow)
};
EnvKnobs g_env;
std::once_flag g_env_once;

void load_env() {
    EnvKnobs e;
    auto num = [](const char *name, int dflt) {
        const char *v = std::getenv(name);
        return v ? std::atoi(v) : dflt;
    };
    auto flag = [](const char *name) {
        const char *v = std::getenv(name);
        return v != nullptr && std::strcmp(v, "0") != 0;
    };
    e.decode_max_rows = num("FA_ROCM_DECODE_MAX_ROWS", 0);
    e.wave_max_rows = num("FA_ROCM_WAVE_MAX_ROWS", 0);
    e.wave_two_tiles = num("FA_ROCM_WAVE_TWO_TILES", 0);
    e.decode_wgs = num("FA_ROCM_DECODE_WGS", 0);
    e.block_workers = flag("FA_ROCM_DECODE_BLOCK_WORKERS");
    e.min_share = num("FA_ROCM_MIN_SHARE", 0);
    e.piece_cost = std::getenv("FA_ROCM_PIECE_COST") ? std::max(0, num("FA_ROCM_PIECE_COST", 0)) : -1;
    e.no_head_interleave = flag("FA_ROCM_NO_HEAD_INTERLEAVE");
    e.separate_append = flag("FA_ROCM_SEPARATE_APPEND");
    e.no_short_blocks = flag("FA_ROCM_NO_SHORT_BLOCKS");
    e.validate = flag("FA_ROCM_VALIDATE");
    g_env = e;
}
const EnvKnobs &env() {
    std::call_once(g_env_once, load_env);
    return g_env;
}

// ---- FA_ROCM_VALIDATE: the checks that need the device's own data (lengths and page ids live there) ----
// One thread per batch row; the first violation found is recorded as {kind, row, value, limit}.
enum { kBadNone = 0, kBadLength = 1, kBadCapacity = 2, kBadPage = 3, kBadRotary = 4 };
static __device__ int g_check_result[4];

__global__ void check_paged_rows_kernel(const int32_t *__restrict__ lens, const int32_t *__restrict__ block_table, int64_t bt_stride_b,
                                        int batch, int add, int page_size, int max_blocks, int num_blocks, int seqlen_ro, int *result) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= batch) return;
    auto report = [&](int kind, int value, int limit) {
        if (atomicCAS(&result[0], kBadNone, kind) == kBadNone) {
            result[1] = b;
            result[2] = value;
            result[3] = limit;
        }
    };
    const int len = lens[b];
    if (len < 0) return report(kBadLength, len, 0);
    const int64_t total = (int64_t)len + add;
    const int64_t capacity = (int64_t)max_blocks * page_size;
    if (total > capacity) return report(kBadCapacity, (int)(total < INT32_MAX ? total : INT32_MAX), (int)(capacity < INT32_MAX ? capacity : INT32_MAX));
    if (seqlen_ro > 0 && total > seqlen_ro) return report(kBadRotary, (int)total, seqlen_ro);
    const int used = (int)((total + page_size - 1) / page_size);
    for (int i = 0; i < used; ++i) {
        const int id = block_table[b * bt_stride_b + i];
        if (id < 0 || id >= num_blocks) return report(kBadPage, id, num_blocks);
    }
}

// Runs the check and WAITS for it (the only place where the library synchronises with the host): a debugging mode,
// unusable while `stream` is being captured.  `what` names the length array in the message.
int check_paged_rows(const char *what, const int32_t *lens, const int32_t *block_table, int64_t bt_stride_b, int batch, int add,
                     int page_size, int max_blocks, int num_blocks, int seqlen_ro, hipStream_t stream) {
    if (batch <= 0) return FA_OK;
    // one set of result words per process: calls that validate (a debugging mode) take their turn, whatever their
    // threads and streams; each waits for its own check before it returns, so the lock is held for one round trip
    static std::mutex validate_mutex;
    std::lock_guard<std::mutex> validate_lock(validate_mutex);
    int *result = nullptr;
    if (hipGetSymbolAddress((void **)&result, HIP_SYMBOL(g_check_result)) != hipSuccess || !result)
        return fail(FA_ERR_LAUNCH, "FA_ROCM_VALIDATE: the result words of the check kernel have no device address");
    int host[4] = {0, 0, 0, 0};
    hipError_t e = hipMemcpyAsync(result, host, sizeof(host), hipMemcpyHostToDevice, stream);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(check_paged_rows_kernel, dim3((batch + 255) / 256), dim3(256), 0, stream, lens, block_table, bt_stride_b, batch, add,
                           page_size, max_blocks, num_blocks, seqlen_ro, result);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(host, result, sizeof(host), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return fail(FA_ERR_LAUNCH, "FA_ROCM_VALIDATE: %s", hipGetErrorString(e));
    switch (host[0]) {
        case kBadLength:
            return fail(FA_ERR_SHAPE, "%s[%d] = %d is negative", what, host[1], host[2]);
        case kBadCapacity:
            return fail(FA_ERR_SHAPE, "batch row %d holds %d keys (%s + new tokens) but its block_table row addresses only %d", host[1], host[2],
                        what, host[3]);
        case kBadRotary:
            return fail(FA_ERR_SHAPE, "batch row %d needs %d rotary positions but rotary_cos / rotary_sin have seqlen_ro = %d rows", host[1], host[2],
                        host[3]);
        case kBadPage:
            return fail(FA_ERR_SHAPE, "block_table row %d names page %d; the cache has num_blocks = %d", host[1], host[2], host[3]);
        default:
            return FA_OK;
    }
}

// bytes of the rotated copy of q that a tall query block with rotary embedding keeps at the start of
// the workspace (a multiple of 256 so that the partials behind it stay aligned)
size_t tall_q_bytes(const fa_kvcache_args *a) {
    if (!a->rotary_cos) return 0;
    const size_t n = (size_t)a->batch * a->seqlen_q * a->nheads * a->headdim_qk * sizeof(uint16_t);
    return (n + 255) / 256 * 256;
}

// Tallest query block (rows = seqlen_q * group) that the wave-level kernel takes.  Blocks of 17-32 rows run there as
// two 16-row tiles in one wave (fa::wave_rows_per_unit) when the call has at least as many units (batch rows x kv
// heads) as the device has compute units: then a unit is cut into few pieces and the stream is bounded by the bytes
// in flight, which that kernel keeps highest; with fewer units the fixed costs of the many pieces and their merge
// weigh more than that, and the tiled kernel (or, at d = 64, the workgroup-level decode kernel) is ahead (measured at
// 64 sequences x 8 K keys, d = 128, whole call, wave-level / tiled: 8 kv heads 364 / 392 us, 4 heads 204 / 217,
// 2 heads 127 / 113, 1 head 87 / 66).  FA_ROCM_WAVE_MAX_ROWS = 16, 32, 48 or 64 overrides the rule for experiments: the
// block is then cut into 16-row tiles that are units of their own; FA_ROCM_WAVE_TWO_TILES = 1 drops the unit count from
// the rule (tests).
int wave_max_rows(const fa_kvcache_args *a, int num_cus) {
    const int v = env().wave_max_rows;
    if (v == 16 || v == 32 || v == 48 || v == 64) return v;
    const int per_unit = fa::wave_rows_per_unit(fa::tile_headdim(a->headdim_qk));
    return (per_unit > 16 && ((int64_t)a->batch * a->nheads_k >= num_cus || env().wave_two_tiles > 0)) ? per_unit : 16;
}

// Tallest query block (rows = seqlen_q * group) that runs on the decode kernels: the workgroup-level ones up to
// fa::block_decode_max_rows (FA_ROCM_DECODE_MAX_ROWS = 16 or 32 overrides it), the wave-level one, which runs the
// balanced partition only, up to wave_max_rows().
int decode_max_rows(const fa_kvcache_args *a, int num_cus) {
    const int v = env().decode_max_rows;
    const int block_level = (v == 16 || v == 32) ? v : fa::block_decode_max_rows(fa::tile_headdim(a->headdim_qk));
    const bool wave_level = a->num_splits == 0 && !is_mla_i8(a) && !env().block_workers;
    return wave_level ? std::max(block_level, wave_max_rows(a, num_cus)) : block_level;
}

// Units that a query block is cut into for the wave-level kernel (1: the block is one unit, of one or two 16-row tiles
// that one wave carries; more: 16-row tiles that are units of their own; 0: not that kernel's)
int wave_row_tiles(const fa_kvcache_args *a, size_t rows, int num_cus) {
    if (is_mla_i8(a) || env().block_workers || rows > (size_t)wave_max_rows(a, num_cus)) return 0;
    if (rows <= (size_t)fa::wave_rows_per_unit(fa::tile_headdim(a->headdim_qk)) && env().wave_max_rows == 0) return 1;
    return (int)((rows + 15) / 16);
}

int64_t live_keys_bound(const fa_kvcache_args *a) {
    int64_t cap = (int64_t)a->max_blocks_per_seq * a->page_size;
    const int wr = a->causal ? 0 : a->window_right;
    if (a->window_left >= 0) {
        // keys in [off - wl, Sq-1 + off + max(wr, 0)] plus alignment slack of one 32-key chunk
        int64_t span = (int64_t)a->window_left + a->seqlen_q + (wr > 0 ? wr : 0) + 32;
        if (span < cap) cap = span;
    }
    return cap > 0 ? cap : 1;
}

}  // namespace

extern "C" {

int fa_rocm_abi_version(void) { return FA_ROCM_ABI_VERSION; }

const char *fa_rocm_last_error(void) { return g_err; }

size_t fa_rocm_sizeof_kvcache_args(void) { return sizeof(fa_kvcache_args); }

size_t fa_rocm_sizeof_varlen_args(void) { return sizeof(fa_varlen_args); }

size_t fa_rocm_sizeof_split_plan(void) { return sizeof(fa_split_plan); }

int fa_rocm_num_cus(void) { return device_cus(); }

void fa_rocm_reload_env(void) {
    (void)env();
    load_env();
}

int fa_rocm_kvcache_validate(const fa_kvcache_args *a) {
    if (!a) return fail(FA_ERR_NULL, "args is NULL");
    if (a->io_dtype != FA_BF16 && a->io_dtype != FA_FP16)
        return fail(FA_ERR_DTYPE, "FlashAttention only supports FP16 and BF16 data types");
    if (a->kv_dtype != a->io_dtype && a->kv_dtype != FA_INT8)
        return fail(FA_ERR_DTYPE, "query and key_cache must have the same dtype");
    if (!a->q || !a->out || !a->softmax_lse || !a->k_cache || !a->v_cache)
        return fail(FA_ERR_NULL, "q, out, softmax_lse, k_cache and v_cache must be non-NULL");
    if (!a->block_table) return fail(FA_ERR_UNSUPPORTED, "only the paged KV cache (block_table) is supported");
    if (!a->cache_seqlens) return fail(FA_ERR_NULL, "cache_seqlens must be given with a paged KV cache");
    if (a->batch <= 0) return fail(FA_ERR_SHAPE, "batch size must be positive");
    if (a->seqlen_q <= 0 || a->nheads <= 0 || a->nheads_k <= 0) return fail(FA_ERR_SHAPE, "empty query");
    if (a->nheads % a->nheads_k != 0)
        return fail(FA_ERR_SHAPE, "Number of heads in key/value must divide number of heads in query");
    // 32-key chunks must not straddle pages; a table one page wide (a dense cache) cannot straddle
    if (a->page_size <= 0 || (a->page_size % 32 != 0 && a->max_blocks_per_seq != 1))
        return fail(FA_ERR_SHAPE, "page_block_size must be a positive multiple of 32");
    if (a->num_blocks <= 0 || a->max_blocks_per_seq <= 0) return fail(FA_ERR_SHAPE, "empty block_table or cache");
    if (a->softcap < 0.f) return fail(FA_ERR_SHAPE, "softcap must be non-negative (0.0 disables softcap)");
    if (a->num_splits < 0) return fail(FA_ERR_SHAPE, "num_splits must be non-negative");
    if (is_mla_i8(a)) {
        if (!a->k_scale_cache) return fail(FA_ERR_NULL, "int8 KV cache needs k_scale_cache");
        if (a->headdim_qk != 576 || a->headdim_v != 512 || a->nheads_k != 1)
            return fail(FA_ERR_SHAPE, "int8 KV cache supports the latent layout only (1 kv head, 576/512 dims)");
        if (a->k_new) {
            // quantising append: new latent rows in the I/O dtype; v is the view k[..., :512] like the cache
            if (a->v_new != a->k_new || a->vn_stride_b != a->kn_stride_b || a->vn_stride_s != a->kn_stride_s)
                return fail(FA_ERR_UNSUPPORTED, "int8 KV cache: v must be the view k[..., :512] of the new latent rows");
            if (a->rotary_cos) return fail(FA_ERR_UNSUPPORTED, "rotary embedding is not supported with an int8 KV cache");
        }
        if (a->v_cache != a->k_cache || a->v_stride_block != a->k_stride_block || a->v_stride_row != a->k_stride_row)
            return fail(FA_ERR_UNSUPPORTED, "int8 KV cache: v_cache must be the view k_cache[..., :512] of the latent cache");
        if (a->k_stride_row % 16 || a->k_stride_block % 16)
            return fail(FA_ERR_SHAPE, "int8 cache strides must be multiples of 16 bytes");
    } else {
        if (a->headdim_qk > 256) return fail(FA_ERR_SHAPE, "FlashAttention only supports head dimension at most 256");
        if (a->headdim_qk != a->headdim_v) return fail(FA_ERR_SHAPE, "k and v head dimensions must match");
        if (a->headdim_qk < 8 || a->headdim_qk % 8 != 0)
            return fail(FA_ERR_SHAPE, "head dimension must be a positive multiple of 8");
    }
    // the combine and the explicit-split kernels put the batch and the units of a row (kv heads; for the latent cache
    // query tokens x 128-head groups) in the grid's y / z extents
    if (a->batch > 65535) return fail(FA_ERR_SHAPE, "batch size must be at most 65535");
    if ((int64_t)a->nheads_k > 65535 || (is_mla_i8(a) && (int64_t)a->seqlen_q * (((int64_t)a->nheads + 127) / 128) > 65535))
        return fail(FA_ERR_SHAPE, "too many units per batch row (kv heads, or query tokens x head groups): at most 65535");
    if ((a->k_new == nullptr) != (a->v_new == nullptr)) return fail(FA_ERR_NULL, "k and v must be passed together");
    if (a->k_new && a->seqlen_new <= 0) return fail(FA_ERR_SHAPE, "seqlen_new must be positive when k is given");
    if (!a->k_new && a->seqlen_new != 0) return fail(FA_ERR_SHAPE, "seqlen_new must be 0 without k");
    if ((a->rotary_cos == nullptr) != (a->rotary_sin == nullptr))
        return fail(FA_ERR_NULL, "rotary_cos and rotary_sin must be passed together");
    if (a->rotary_cos) {
        if (!a->k_new) return fail(FA_ERR_UNSUPPORTED, "rotary embedding is only applied when k and v are passed");
        if (a->rotary_dim <= 0 || a->rotary_dim > a->headdim_qk || a->rotary_dim % 16 != 0)
            return fail(FA_ERR_SHAPE, "rotary_dim must be divisible by 16 and at most headdim");
        if (a->seqlen_ro <= 0) return fail(FA_ERR_SHAPE, "rotary tables are empty");
    }
    // strides the kernels turn into 32-bit byte offsets inside a page / 16-byte accesses
    if (a->k_stride_row % 8 || a->k_stride_h % 8 || a->k_stride_block % 8 || a->v_stride_row % 8 ||
        a->v_stride_h % 8 || a->v_stride_block % 8 || a->q_stride_h % 8 || a->q_stride_s % 8 || a->q_stride_b % 8 ||
        a->o_stride_h % 8 || a->o_stride_s % 8 || a->o_stride_b % 8)
        if (!is_mla_i8(a)) return fail(FA_ERR_SHAPE, "tensor strides must be multiples of 8 elements (16 bytes)");
    if ((int64_t)a->page_size * a->k_stride_row * 2 >= (1ll << 31) || (int64_t)a->page_size * a->v_stride_row * 2 >= (1ll << 31))
        return fail(FA_ERR_SHAPE, "a cache page must span less than 2 GiB");
    // every row is moved 16 bytes at a time (K/V rows straight into LDS)
    if (!aligned16(a->q) || !aligned16(a->out) || !aligned16(a->k_cache) || !aligned16(a->v_cache) || !aligned16(a->k_new) ||
        !aligned16(a->v_new))
        return fail(FA_ERR_SHAPE, "tensor data must be 16-byte aligned");
    return FA_OK;
}

int fa_rocm_plan_kvcache(const fa_kvcache_args *a, int num_cus, fa_split_plan *plan) {
    if (!a || !plan) return fail(FA_ERR_NULL, "args or plan is NULL");
    if (num_cus <= 0) num_cus = 256;
    std::memset(plan, 0, sizeof(*plan));
    {
        // The plan is defined for exactly the shapes the call accepts.  A caller that only plans may leave the tensor
        // pointers NULL: they are stood in for here, so that the dimension checks of the validator decide alone.
        fa_kvcache_args c = *a;
        alignas(16) static char placeholder[16];
        void *const some = placeholder;
        if (!c.q) c.q = some;
        if (!c.out) c.out = some;
        if (!c.softmax_lse) c.softmax_lse = static_cast<float *>(some);
        if (!c.k_cache && !c.v_cache) c.k_cache = c.v_cache = some;
        if (!c.block_table) c.block_table = static_cast<const int32_t *>(some);
        if (!c.cache_seqlens) c.cache_seqlens = static_cast<const int32_t *>(some);
        if (is_mla_i8(&c) && !c.k_scale_cache) c.k_scale_cache = static_cast<float *>(some);
        if (c.seqlen_new > 0 && !c.k_new && !c.v_new) c.k_new = c.v_new = some;
        const int rc = fa_rocm_kvcache_validate(&c);
        if (rc != FA_OK) return rc;
    }
    const int group = a->nheads / a->nheads_k;
    // the int8 latent kernel works on units of 128 query heads and always uses the balanced partition
    const size_t rows = is_mla_i8(a) ? 128 : (size_t)a->seqlen_q * group;
    size_t slot_bytes = rows * partial_row_bytes(a);
    if (!is_mla_i8(a) && rows > (size_t)decode_max_rows(a, num_cus)) {
        // Query block too tall for the decode kernels: the tiled forward.  When its tiles alone
        // cannot fill the device (few sequences, short blocks) the keys of every unit are cut into
        // ranges as well; the range length is sized on the device from the longest sequence, so only
        // the number of ranges is planned here.  With rotary embedding the workspace starts with the
        // rotated copy of q.
        plan->mode = FA_SPLIT_GRID;
        const int64_t bound = live_keys_bound(a);
        int64_t n = 1;
        if (a->num_splits > 1) {
            n = a->num_splits;
        } else if (a->num_splits == 0) {
            const int64_t tiles = (int64_t)a->batch * fa::prefill_tiles(a->nheads, a->nheads_k, a->seqlen_q);
            const int64_t slots = (int64_t)num_cus * (a->headdim_qk <= 128 ? 2 : 1);
            if (tiles * 2 <= slots) n = (slots + tiles - 1) / tiles;
        }
        const int64_t most = (bound + 255) / 256;   // at least 256 keys (four tiles) per range
        if (n > most) n = most;
        if (n > 64) n = 64;
        if (n < 1) n = 1;
        plan->nsplits = (int32_t)n;
        plan->split_keys = 0;
        plan->workspace_bytes = tall_q_bytes(a) + (n > 1 ? (size_t)a->batch * a->nheads_k * n * slot_bytes : 0);
        return FA_OK;
    }
    if (a->num_splits == 0 || is_mla_i8(a)) {
        plan->mode = FA_SPLIT_BALANCED;
        plan->nsplits = 1;
        // Query blocks of up to wave_max_rows() rows: every wave is a worker with its own contiguous share (no
        // workgroup barrier anywhere in the stream), blocks of more than 16 rows as 16-row tiles that are units of
        // their own; taller blocks and the latent kernel: the workgroup is the worker.
        const int tiles = wave_row_tiles(a, rows, num_cus);
        const bool wave_workers = tiles >= 1;
        if (tiles > 1) slot_bytes = 16 * partial_row_bytes(a);
        const int per_cu = is_mla_i8(a) ? 1 : fa::decode_wgs_per_cu(a->headdim_qk, wave_workers ? 16 : (int)rows);
        plan->num_wgs = num_cus * per_cu;
        // latent kernel: a piece costs ~15 us of pipeline fill and a 131 KB partial, so tiny launches are
        // not cut below 4 chunks per workgroup (1 sequence x 8 K tokens: 46 -> 37 us)
        plan->min_share = is_mla_i8(a) ? 4 : 1;
        // tuning aid: FA_ROCM_DECODE_WGS overrides the workgroup count of the balanced partition
        if (env().decode_wgs > 0) plan->num_wgs = env().decode_wgs;
        plan->num_workers = wave_workers ? plan->num_wgs * 4 : plan->num_wgs;
        if (wave_workers) plan->min_share = 2;   // short shares: the pipeline fill dominates tiny contexts otherwise
        if (env().min_share > 0) plan->min_share = env().min_share;
        // every worker writes at most two partials (the units cut at the two ends of its share)
        // ... and workgroup 0 leaves the partition behind them for the merge kernel
        plan->workspace_bytes = (size_t)plan->num_workers * 2 * slot_bytes + fa::kPartitionHeaderBytes;
        return FA_OK;
    }
    const int64_t bound = live_keys_bound(a);
    const int64_t granule = 256;
    int64_t sk;
    if (a->num_splits == 1) {
        sk = (bound + granule - 1) / granule * granule;
    } else {
        // forced mode (flash_attn_npu_3/fa_split.h:345-350): blocks per split = ceil(nblk / num_splits)
        const int64_t nblk = (bound + granule - 1) / granule;
        const int64_t per = (nblk + a->num_splits - 1) / a->num_splits;
        sk = per * granule;
    }
    if (sk > (1 << 30)) sk = 1 << 30;
    int64_t n = (bound + sk - 1) / sk;
    if (n < 1) n = 1;
    plan->mode = FA_SPLIT_GRID;
    plan->nsplits = (int32_t)n;
    plan->split_keys = (int32_t)sk;
    plan->workspace_bytes = n > 1 ? (size_t)a->batch * a->nheads_k * n * slot_bytes : 0;
    return FA_OK;
}

size_t fa_rocm_kvcache_workspace_bytes(const fa_kvcache_args *a, int num_cus) {
    fa_split_plan plan;
    if (fa_rocm_plan_kvcache(a, num_cus, &plan) != FA_OK) return 0;
    return plan.workspace_bytes;
}

static void fill_append(const fa_kvcache_args *a, fa::AppendParams &p) {
    std::memset(&p, 0, sizeof(p));
    p.k_cache = a->k_cache;
    p.v_cache = a->v_cache;
    p.k_new = a->k_new;
    p.v_new = a->v_new;
    p.rotary_cos = a->rotary_cos;
    p.rotary_sin = a->rotary_sin;
    p.cache_seqlens = a->cache_seqlens;
    p.block_table = a->block_table;
    p.batch = a->batch;
    p.seqlen_new = a->seqlen_new;
    p.nheads_k = a->nheads_k;
    p.headdim_qk = a->headdim_qk;
    p.headdim_v = a->headdim_v;
    p.num_blocks = a->num_blocks;
    p.page_size = a->page_size;
    p.max_blocks = a->max_blocks_per_seq;
    p.rotary_dim = a->rotary_dim;
    p.seqlen_ro = a->seqlen_ro;
    p.rotary_interleaved = a->rotary_interleaved;
    p.k_stride_block = a->k_stride_block;
    p.k_stride_row = a->k_stride_row;
    p.k_stride_h = a->k_stride_h;
    p.v_stride_block = a->v_stride_block;
    p.v_stride_row = a->v_stride_row;
    p.v_stride_h = a->v_stride_h;
    p.kn_stride_b = a->kn_stride_b;
    p.kn_stride_s = a->kn_stride_s;
    p.kn_stride_h = a->kn_stride_h;
    p.vn_stride_b = a->vn_stride_b;
    p.vn_stride_s = a->vn_stride_s;
    p.vn_stride_h = a->vn_stride_h;
    p.bt_stride_b = a->bt_stride_b;
    // the scale tensors are inputs of attention and outputs of the quantising append
    p.k_scale = a->k_scale_cache;
    p.v_scale = a->v_scale_cache;
    p.ks_stride_block = a->ks_stride_block;
    p.ks_stride_row = a->ks_stride_row;
}

int fa_rocm_append_kv(const fa_kvcache_args *a, void *stream) {
    const int rc = fa_rocm_kvcache_validate(a);
    if (rc != FA_OK) return rc;
    if (!a->k_new) return FA_OK;
    fa::AppendParams p;
    fill_append(a, p);
    const hipError_t e = is_mla_i8(a) ? fa::launch_append_quant_i8(p, a->io_dtype, static_cast<hipStream_t>(stream))
                                      : fa::launch_append_kv(p, a->io_dtype, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(FA_ERR_LAUNCH, "append_kv launch failed: %s", hipGetErrorString(e));
    return FA_OK;
}

static int fwd_kvcache_impl(const fa_kvcache_args *a, void *stream_, void *const *events, const int32_t *q_live = nullptr);

int fa_rocm_fwd_kvcache(const fa_kvcache_args *a, void *stream_) { return fwd_kvcache_impl(a, stream_, nullptr); }

int fa_rocm_fwd_kvcache_profiled(const fa_kvcache_args *a, void *stream_, void *const events[4]) {
    if (!events) return fail(FA_ERR_NULL, "events is NULL");
    return fwd_kvcache_impl(a, stream_, events);
}

static int fwd_kvcache_impl(const fa_kvcache_args *a, void *stream_, void *const *events, const int32_t *q_live) {
    int rc = fa_rocm_kvcache_validate(a);
    if (rc != FA_OK) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (env().validate && q_live == nullptr) {
        rc = check_paged_rows("cache_seqlens", a->cache_seqlens, a->block_table, a->bt_stride_b, a->batch, a->seqlen_new, a->page_size,
                              a->max_blocks_per_seq, a->num_blocks, a->rotary_cos ? a->seqlen_ro : 0, stream);
        if (rc != FA_OK) return rc;
    }
    auto mark = [&](int i) {
        if (events) (void)hipEventRecord(static_cast<hipEvent_t>(events[i]), stream);
    };
    mark(0);
    const int group = a->nheads / a->nheads_k;
    const int rows = a->seqlen_q * group;

    const bool local = a->window_left >= 0 || a->window_right >= 0;

    int cus_t = device_cus();
    if (cus_t <= 0) cus_t = 256;
    if (!is_mla_i8(a) && rows > decode_max_rows(a, cus_t)) {
        // query block too tall for the decode kernel: tiled forward over the paged cache
        fa_split_plan tplan;
        rc = fa_rocm_plan_kvcache(a, cus_t, &tplan);
        if (rc != FA_OK) return rc;
        if (tplan.workspace_bytes > 0 && (!a->workspace || a->workspace_bytes < tplan.workspace_bytes))   // before anything is written
            return fail(FA_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", tplan.workspace_bytes,
                        a->workspace ? a->workspace_bytes : (size_t)0);
        if (a->k_new) {
            rc = fa_rocm_append_kv(a, stream_);
            if (rc != FA_OK) return rc;
        }
        mark(1);
        fa::PrefillParams pp;
        std::memset(&pp, 0, sizeof(pp));
        pp.q = a->q;
        pp.k = a->k_cache;
        pp.v = a->v_cache;
        pp.out = a->out;
        pp.lse = a->softmax_lse;
        pp.seqused_k = a->cache_seqlens;
        pp.block_table = a->block_table;
        pp.batch = a->batch;
        pp.nheads = a->nheads;
        pp.nheads_k = a->nheads_k;
        pp.group = group;
        pp.seqlen_q_fixed = a->seqlen_q;
        pp.seqlen_k_add = a->seqlen_new;
        pp.max_seqlen_q = a->seqlen_q;
        pp.total_q = a->batch * a->seqlen_q;
        pp.page_size = a->page_size;
        pp.max_blocks = a->max_blocks_per_seq;
        pp.num_blocks = a->num_blocks;
        pp.q_stride_b = a->q_stride_b;
        pp.q_stride_t = a->q_stride_s;
        pp.q_stride_h = a->q_stride_h;
        pp.o_stride_b = a->o_stride_b;
        pp.o_stride_t = a->o_stride_s;
        pp.o_stride_h = a->o_stride_h;
        pp.k_stride_t = a->k_stride_row;
        pp.k_stride_h = a->k_stride_h;
        pp.k_stride_block = a->k_stride_block;
        pp.v_stride_t = a->v_stride_row;
        pp.v_stride_h = a->v_stride_h;
        pp.v_stride_block = a->v_stride_block;
        pp.bt_stride_b = a->bt_stride_b;
        pp.lse_stride_b = (int64_t)a->nheads * a->seqlen_q;
        pp.lse_stride_h = a->seqlen_q;
        pp.scale_log2 = a->softmax_scale * kLog2e;
        if (a->softcap > 0.f) {
            pp.softcap_pre = a->softmax_scale / a->softcap;
            pp.softcap_post = a->softcap * kLog2e;
        }
        pp.causal = a->causal;
        pp.window_left = a->window_left;
        pp.window_right = a->window_right;
        pp.window_norm_m = 0;
        if (a->rotary_cos) {
            fa::RotateQParams rq;
            std::memset(&rq, 0, sizeof(rq));
            rq.q = a->q;
            rq.out = a->workspace;
            rq.rotary_cos = a->rotary_cos;
            rq.rotary_sin = a->rotary_sin;
            rq.cache_seqlens = a->cache_seqlens;
            rq.batch = a->batch;
            rq.seqlen_q = a->seqlen_q;
            rq.nheads = a->nheads;
            rq.headdim = a->headdim_qk;
            rq.rotary_dim = a->rotary_dim;
            rq.seqlen_ro = a->seqlen_ro;
            rq.rotary_interleaved = a->rotary_interleaved;
            rq.rotary_per_token = (a->causal || local) ? 1 : 0;
            rq.q_stride_b = a->q_stride_b;
            rq.q_stride_s = a->q_stride_s;
            rq.q_stride_h = a->q_stride_h;
            const hipError_t er = fa::launch_rotate_q(rq, a->io_dtype, stream);
            if (er != hipSuccess) return fail(FA_ERR_LAUNCH, "rotate_q launch failed: %s", hipGetErrorString(er));
            pp.q = a->workspace;
            pp.q_stride_h = a->headdim_qk;
            pp.q_stride_t = (int64_t)a->nheads * a->headdim_qk;
            pp.q_stride_b = (int64_t)a->seqlen_q * pp.q_stride_t;
        }
        float *partials = reinterpret_cast<float *>(static_cast<char *>(a->workspace) + tall_q_bytes(a));
        const size_t slot_rows = (size_t)a->batch * a->nheads_k * tplan.nsplits * rows;
        if (tplan.nsplits > 1) {
            pp.nsplits = tplan.nsplits;
            pp.rows = rows;
            pp.o_partial = partials;
            pp.lse_partial = partials + slot_rows * partial_width(a);
        }
        pp.headdim = a->headdim_qk;
        const hipError_t e = fa::launch_prefill(pp, a->io_dtype, fa::tile_headdim(a->headdim_qk), stream);
        if (e != hipSuccess) return fail(FA_ERR_LAUNCH, "prefill launch failed: %s", hipGetErrorString(e));
        mark(2);
        if (tplan.nsplits > 1) {
            // the decode kernels' grid-mode combine merges the ranges: same slots, same row order
            fa::DecodeParams cp;
            std::memset(&cp, 0, sizeof(cp));
            cp.out = a->out;
            cp.lse = a->softmax_lse;
            cp.cache_seqlens = a->cache_seqlens;
            cp.batch = a->batch;
            cp.seqlen_q = a->seqlen_q;
            cp.nheads = a->nheads;
            cp.nheads_k = a->nheads_k;
            cp.group = group;
            cp.rows = rows;
            cp.seqlen_new = a->seqlen_new;
            cp.page_size = a->page_size;
            cp.max_blocks = a->max_blocks_per_seq;
            cp.o_stride_b = a->o_stride_b;
            cp.o_stride_s = a->o_stride_s;
            cp.o_stride_h = a->o_stride_h;
            cp.causal = a->causal;
            cp.window_left = a->window_left;
            cp.window_right = a->window_right;
            cp.nsplits = tplan.nsplits;
            cp.split_keys = 256;
            cp.split_adaptive = 1;
            cp.o_partial = pp.o_partial;
            cp.lse_partial = pp.lse_partial;
            cp.headdim = a->headdim_v;
            const hipError_t ec = fa::launch_splitkv_combine(cp, a->io_dtype, partial_width(a), stream);
            if (ec != hipSuccess) return fail(FA_ERR_LAUNCH, "combine launch failed: %s", hipGetErrorString(ec));
        }
        mark(3);
        return FA_OK;
    }

    int cus = device_cus();
    if (cus <= 0) cus = 256;
    fa_split_plan plan;
    rc = fa_rocm_plan_kvcache(a, cus, &plan);
    if (rc != FA_OK) return rc;
    const size_t need = plan.workspace_bytes;
    if (need > 0 && (!a->workspace || a->workspace_bytes < need))
        return fail(FA_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, a->workspace ? a->workspace_bytes : (size_t)0);

    fa::DecodeParams p;
    std::memset(&p, 0, sizeof(p));
    p.q = a->q;
    p.out = a->out;
    p.lse = a->softmax_lse;
    p.k_cache = a->k_cache;
    p.v_cache = a->v_cache;
    p.k_scale = a->k_scale_cache;
    p.v_scale = a->v_scale_cache ? a->v_scale_cache : a->k_scale_cache;
    p.rotary_cos = a->k_new ? a->rotary_cos : nullptr;
    p.rotary_sin = a->k_new ? a->rotary_sin : nullptr;
    p.cache_seqlens = a->cache_seqlens;
    p.block_table = a->block_table;
    p.q_live = q_live;
    p.batch = a->batch;
    p.seqlen_q = a->seqlen_q;
    p.nheads = a->nheads;
    p.nheads_k = a->nheads_k;
    p.group = group;
    p.rows = rows;
    p.headdim = a->headdim_v;
    p.seqlen_new = a->seqlen_new;
    p.num_blocks = a->num_blocks;
    p.page_size = a->page_size;
    p.max_blocks = a->max_blocks_per_seq;
    p.rotary_dim = a->rotary_dim;
    p.seqlen_ro = a->seqlen_ro;
    p.rotary_interleaved = a->rotary_interleaved;
    p.rotary_per_token = (a->causal || local) ? 1 : 0;
    p.q_stride_b = a->q_stride_b;
    p.q_stride_s = a->q_stride_s;
    p.q_stride_h = a->q_stride_h;
    p.o_stride_b = a->o_stride_b;
    p.o_stride_s = a->o_stride_s;
    p.o_stride_h = a->o_stride_h;
    p.k_stride_block = a->k_stride_block;
    p.k_stride_row = a->k_stride_row;
    p.k_stride_h = a->k_stride_h;
    p.v_stride_block = a->v_stride_block;
    p.v_stride_row = a->v_stride_row;
    p.v_stride_h = a->v_stride_h;
    p.ks_stride_block = a->ks_stride_block;
    p.ks_stride_row = a->ks_stride_row;
    p.bt_stride_b = a->bt_stride_b;
    p.scale_log2 = a->softmax_scale * kLog2e;
    if (a->softcap > 0.f) {
        p.softcap_pre = a->softmax_scale / a->softcap;
        p.softcap_post = a->softcap * kLog2e;
    }
    p.causal = a->causal;
    p.window_left = a->window_left;
    p.window_right = a->window_right;
    p.nsplits = plan.nsplits;
    p.split_keys = plan.split_keys > 0 ? plan.split_keys : 256;
    p.balanced = plan.mode == FA_SPLIT_BALANCED;
    p.num_wgs = plan.num_wgs;
    p.num_workers = plan.num_workers;
    p.min_share = plan.min_share;
    p.wave_workers = plan.num_workers != plan.num_wgs;
    p.min_share_long = (p.wave_workers && env().min_share <= 0) ? 4 : 0;
    // wave workers of neighbouring kv heads walk the same token range together
    // Fixed cost of starting on a unit, in chunk times.  Latent kernel: ~15 us of q staging and pipeline
    // fill against ~2 us per chunk; charging 7 chunks takes the workgroups that start a second unit off
    // the critical path (c4 kernel 150 -> 145 us).  Wave-level kernel: ~6 us against ~5 us per chunk;
    // charging 1-3 chunks measured within +-1 %, so it is not charged.
    p.piece_cost = is_mla_i8(a) ? 7 : 0;
    if (env().piece_cost >= 0) p.piece_cost = env().piece_cost;
    const int row_tiles = p.wave_workers ? wave_row_tiles(a, rows, cus) : 0;
    if (row_tiles > 1) {
        // (kv head, 16-row tile) units: the tiles of a kv head are neighbouring units
        p.row_tiles = row_tiles;
        p.rows_total = (int32_t)rows;
        p.rows = 16;
        p.nheads_k = a->nheads_k * row_tiles;
    }
    p.head_interleave = p.wave_workers && p.nheads_k > 1 && plan.num_workers % p.nheads_k == 0 &&
                        !env().no_head_interleave;
    const bool needs_combine = need > 0;
    if (needs_combine) {
        const size_t hdr = p.balanced ? fa::kPartitionHeaderBytes : 0;
        const size_t slot_rows = (need - hdr) / partial_row_bytes(a);
        if (p.balanced) p.part_hdr = reinterpret_cast<int32_t *>(static_cast<char *>(a->workspace) + need - hdr);
        p.o_partial = static_cast<float *>(a->workspace);
        p.lse_partial = reinterpret_cast<float *>(static_cast<char *>(a->workspace) + slot_rows * (partial_row_bytes(a) - sizeof(float)));
    }

    // The wave-level kernel appends on the fly when every new position is certain to be visible
    // (and so owned by exactly one wave): causal or no right bound, and no left bound that could
    // exclude the oldest new key.  Otherwise the rows are written by their own kernel first.
    // With row tiles several waves read every chunk and only one of them would write the row: no fusion.
    const bool fuse_append = a->k_new && p.balanced && p.wave_workers && row_tiles <= 1 && (a->causal || a->window_right < 0) &&
                             (a->window_left < 0 || (int64_t)a->seqlen_q + a->window_left >= a->seqlen_new) &&
                             !env().separate_append;
    if (fuse_append) {
        p.k_new = a->k_new;
        p.v_new = a->v_new;
        p.kn_stride_b = a->kn_stride_b;
        p.kn_stride_s = a->kn_stride_s;
        p.kn_stride_h = a->kn_stride_h;
        p.vn_stride_b = a->vn_stride_b;
        p.vn_stride_s = a->vn_stride_s;
        p.vn_stride_h = a->vn_stride_h;
    } else if (a->k_new) {
        rc = fa_rocm_append_kv(a, stream_);
        if (rc != FA_OK) return rc;
    }
    mark(1);

    hipError_t e;
    if (is_mla_i8(a)) {
        p.units_per_token = (a->nheads + 127) / 128;      // 128-head groups (the last one may be partly empty)
        p.nheads_k = a->seqlen_q * p.units_per_token;     // units per batch row
        p.group = 128;
        p.rows = 128;
        e = fa::launch_decode_mla_i8(p, a->io_dtype, stream);
    }
    else {
        e = fa::launch_decode_paged(p, a->io_dtype, fa::tile_headdim(a->headdim_qk), stream);
    }
    if (e != hipSuccess) return fail(FA_ERR_LAUNCH, "decode launch failed: %s", hipGetErrorString(e));
    mark(2);
    if (needs_combine) {
        e = fa::launch_splitkv_combine(p, a->io_dtype, partial_width(a), stream);
        if (e != hipSuccess) return fail(FA_ERR_LAUNCH, "combine launch failed: %s", hipGetErrorString(e));
    }
    mark(3);
    return FA_OK;
}

// ---- the kvcache call for callers that cannot allocate: the split workspace is a static device array.
// Every GPU the library runs on holds its own copy of the array, at its own address, until the process
// ends; the name below is only a host-side handle, the address comes from hipGetSymbolAddress.
}  // extern "C"

namespace {
static __device__ __align__(256) unsigned char scratch[FA_ROCM_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];   // device address of `scratch`, per device

// Device address of the current device's copy of `scratch`; looked up on the first call on that device
// (a symbol query: it allocates nothing, but it must not run while a stream is being captured).
int static_scratch(void **ptr_out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(FA_ERR_LAUNCH, "no current HIP device (or a device index beyond %d)", kMaxDevices - 1);
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(FA_ERR_LAUNCH, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // two racing threads store the same address
    }
    *ptr_out = ptr;
    return FA_OK;
}
}  // namespace

extern "C" {

int fa_rocm_fwd_kvcache_static(const fa_kvcache_args *args, void *stream) {
    const int rc = fa_rocm_kvcache_validate(args);
    if (rc != FA_OK) return rc;
    int cus = device_cus();
    if (cus <= 0) cus = 256;
    fa_split_plan plan;
    const int rp = fa_rocm_plan_kvcache(args, cus, &plan);
    if (rp != FA_OK) return rp;
    if (plan.workspace_bytes > (size_t)FA_ROCM_STATIC_SCRATCH_BYTES)
        return fail(FA_ERR_WORKSPACE,
                    "the call needs a workspace of %zu bytes, the static scratch of fa_rocm_fwd_kvcache_static holds %zu: "
                    "use fa_rocm_fwd_kvcache with a caller-owned workspace",
                    plan.workspace_bytes, (size_t)FA_ROCM_STATIC_SCRATCH_BYTES);
    fa_kvcache_args a = *args;
    a.workspace = nullptr;
    a.workspace_bytes = 0;
    if (plan.workspace_bytes > 0) {
        void *ptr = nullptr;
        const int rs = static_scratch(&ptr);
        if (rs != FA_OK) return rs;
        // Nothing in the scratch has to start at zero: every partial slot a launch merges was written by
        // that launch (the kernels and the combine derive the same partition), so the contents the last
        // call left are never read.
        a.workspace = ptr;
        a.workspace_bytes = FA_ROCM_STATIC_SCRATCH_BYTES;
    }
    return fwd_kvcache_impl(&a, stream, nullptr);
}

int fa_rocm_varlen_validate(const fa_varlen_args *a) {
    if (!a) return fail(FA_ERR_NULL, "args is NULL");
    if (a->io_dtype != FA_BF16 && a->io_dtype != FA_FP16)
        return fail(FA_ERR_DTYPE, "FlashAttention only supports FP16 and BF16 data types");
    if (!a->q || !a->k || !a->v || !a->out || !a->softmax_lse) return fail(FA_ERR_NULL, "q, k, v, out and softmax_lse must be non-NULL");
    if (!a->cu_seqlens_q) return fail(FA_ERR_NULL, "cu_seqlens_q must be non-NULL");
    if (!a->block_table && !a->cu_seqlens_k) return fail(FA_ERR_NULL, "cu_seqlens_k must be non-NULL");
    if (a->block_table && !a->seqused_k) return fail(FA_ERR_NULL, "paged K/V needs seqused_k");
    if (a->batch <= 0) return fail(FA_ERR_SHAPE, "batch size must be positive");
    if (a->nheads <= 0 || a->nheads_k <= 0 || a->nheads % a->nheads_k != 0)
        return fail(FA_ERR_SHAPE, "Number of heads in key/value must divide number of heads in query");
    if (a->headdim > 256) return fail(FA_ERR_SHAPE, "FlashAttention only supports head dimension at most 256");
    if (a->headdim < 8 || a->headdim % 8 != 0) return fail(FA_ERR_SHAPE, "head dimension must be a positive multiple of 8");
    if (a->softcap < 0.f) return fail(FA_ERR_SHAPE, "softcap must be non-negative (0.0 disables softcap)");
    if (a->max_seqlen_q <= 0) return fail(FA_ERR_SHAPE, "max_seqlen_q must be positive");
    if (a->num_splits < 0) return fail(FA_ERR_SHAPE, "num_splits must be non-negative");
    if (a->block_table && (a->page_size <= 0 || a->page_size % 32 != 0))
        return fail(FA_ERR_SHAPE, "page_block_size must be a positive multiple of 32");
    if (a->block_table && (a->num_blocks <= 0 || a->max_blocks_per_seq <= 0))
        return fail(FA_ERR_SHAPE, "empty block_table or cache");
    if (a->q_stride_t % 8 || a->q_stride_h % 8 || a->k_stride_t % 8 || a->k_stride_h % 8 || a->v_stride_t % 8 ||
        a->v_stride_h % 8 || a->o_stride_t % 8 || a->o_stride_h % 8)
        return fail(FA_ERR_SHAPE, "tensor strides must be multiples of 8 elements (16 bytes)");
    if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->out))
        return fail(FA_ERR_SHAPE, "tensor data must be 16-byte aligned");
    return FA_OK;
}

}  // extern "C"

namespace {

size_t align256(size_t n) { return (n + 255) / 256 * 256; }

// Where the pieces of a varlen call's workspace lie: the partials of the key ranges first, then the
// batch-major rows of the one-token query blocks and the workspace of the decode launch over them.
struct VarlenWorkspace {
    int nsplits;
    bool short_blocks;
    int slots;           // query positions per sequence in the decode launch over the short blocks
    bool decode_only;    // no block is longer than `slots`: the tiled kernel has nothing to do
    size_t partials, q_rows, out_rows, lse_rows, lens_rows, live_rows, long_ids, list_state, decode_ws, decode_ws_bytes, total;
};

// The decode launch over the one-token blocks of a token-major batch: batch row b is sequence b, with
// lens_rows[b] keys (0 for the sequences the tiled kernel computes).  `base` may be NULL for planning.
fa_kvcache_args short_blocks_call(const fa_varlen_args *a, char *base, const VarlenWorkspace &w) {
    fa_kvcache_args k;
    std::memset(&k, 0, sizeof(k));
    char *b = base ? base : reinterpret_cast<char *>(uintptr_t(256));   // never followed when planning
    k.q = b + w.q_rows;
    k.out = b + w.out_rows;
    k.softmax_lse = reinterpret_cast<float *>(b + w.lse_rows);
    k.cache_seqlens = reinterpret_cast<const int32_t *>(b + w.lens_rows);
    k.k_cache = const_cast<void *>(a->k);
    k.v_cache = const_cast<void *>(a->v);
    k.block_table = a->block_table;
    k.workspace = w.decode_ws_bytes ? b + w.decode_ws : nullptr;
    k.workspace_bytes = w.decode_ws_bytes;
    k.batch = a->batch;
    k.seqlen_q = w.slots;
    k.nheads = a->nheads;
    k.nheads_k = a->nheads_k;
    k.headdim_qk = k.headdim_v = a->headdim;
    k.num_blocks = a->num_blocks;
    k.page_size = a->page_size;
    k.max_blocks_per_seq = a->max_blocks_per_seq;
    k.q_stride_h = k.o_stride_h = a->headdim;
    k.q_stride_s = k.o_stride_s = (int64_t)a->nheads * a->headdim;
    k.q_stride_b = k.o_stride_b = (int64_t)w.slots * a->nheads * a->headdim;
    k.k_stride_block = a->k_stride_block;
    k.k_stride_row = a->k_stride_t;
    k.k_stride_h = a->k_stride_h;
    k.v_stride_block = a->v_stride_block;
    k.v_stride_row = a->v_stride_t;
    k.v_stride_h = a->v_stride_h;
    k.bt_stride_b = a->bt_stride_b;
    k.io_dtype = k.kv_dtype = a->io_dtype;
    k.softmax_scale = a->softmax_scale;
    k.softcap = a->softcap;
    k.causal = a->causal;
    k.window_left = a->window_left;
    k.window_right = a->window_right;
    return k;
}

// Query positions per sequence of the decode launch over the short blocks: as many tokens as fit the 16 rows
// (tokens x q heads per kv head) of the wave-level decode kernel's one tile, so the launch costs the same
// whether the blocks hold one token or several (decode rows, or speculative decoding's few tokens).
// The query blocks other than the longest one are, on average, at most a quarter of it: a prompt chunk (or a
// few) among decode rows.  From shapes alone; the block lengths themselves stay on the device.
bool uneven_blocks(const fa_varlen_args *a) {
    return a->batch >= 2 && ((int64_t)a->total_q - a->max_seqlen_q) * 4 <= (int64_t)(a->batch - 1) * a->max_seqlen_q;
}

int short_block_slots(const fa_varlen_args *a) {
    const int group = a->nheads / a->nheads_k;
    return std::max(1, std::min(16 / std::max(group, 1), 8));
}

// A token-major batch over a paged cache whose query blocks are far shorter than the longest one on average
// is taken for prompt chunks among decode rows: its short blocks go to the decode kernels (which stream
// their keys at memory speed), the tiled forward computes the rest.  Decided from shapes; which block is
// short is decided on the device.  When no block can be longer than the slots, the decode kernels do it all.
bool routes_short_blocks(const fa_varlen_args *a) {
    if (!a->block_table || a->total_q <= 0) return false;
    if (a->nheads / a->nheads_k > fa::kDecodeMaxRows) return false;
    if (a->max_seqlen_q > short_block_slots(a) && !uneven_blocks(a)) return false;
    return !env().no_short_blocks;
}

VarlenWorkspace varlen_workspace(const fa_varlen_args *a, int num_cus) {
    VarlenWorkspace w;
    std::memset(&w, 0, sizeof(w));
    w.short_blocks = routes_short_blocks(a);
    w.slots = std::min(short_block_slots(a), std::max(a->max_seqlen_q, 1));
    if (w.short_blocks) {
        const fa_kvcache_args probe = short_blocks_call(a, nullptr, w);
        if (fa_rocm_kvcache_validate(&probe) != FA_OK) w.short_blocks = false;   // a cache the decode kernels do not take
    }
    w.decode_only = w.short_blocks && a->max_seqlen_q <= w.slots;
    w.nsplits = w.decode_only ? 1 : fa_rocm_varlen_num_splits(a, num_cus);
    size_t off = 0;
    if (w.nsplits > 1) off = align256((size_t)a->total_q * a->nheads * w.nsplits * ((size_t)fa::tile_headdim(a->headdim) + 1) * sizeof(float));
    if (w.short_blocks) {
        const size_t rows = (size_t)a->batch * w.slots * a->nheads;
        w.q_rows = off;
        off += align256(rows * a->headdim * 2);
        w.out_rows = off;
        off += align256(rows * a->headdim * 2);
        w.lse_rows = off;
        off += align256(rows * sizeof(float));
        w.lens_rows = off;
        off += align256((size_t)a->batch * sizeof(int32_t));
        w.live_rows = off;
        off += align256((size_t)a->batch * sizeof(int32_t));
        w.long_ids = off;
        off += align256((size_t)a->batch * sizeof(int32_t));
        w.list_state = off;
        off += 256;
        const fa_kvcache_args k = short_blocks_call(a, nullptr, w);
        fa_split_plan plan;
        if (fa_rocm_plan_kvcache(&k, num_cus, &plan) != FA_OK) plan.workspace_bytes = 0;   // cannot fail after the check above
        w.decode_ws = off;
        w.decode_ws_bytes = plan.workspace_bytes;
        off += align256(plan.workspace_bytes);
    }
    w.total = off;
    return w;
}

}  // namespace

extern "C" {

int fa_rocm_varlen_num_splits(const fa_varlen_args *a, int num_cus) {
    if (fa_rocm_varlen_validate(a) != FA_OK) return 1;
    if (!a->block_table || a->num_splits == 1 || a->total_q <= 0) return 1;
    if (num_cus <= 0) num_cus = 256;
    const int group = a->nheads / a->nheads_k;
    const bool pack_short = fa::prefill_pack_short(group, a->max_seqlen_q, a->total_q, a->batch) != 0;
    const int pack = pack_short ? group : fa::prefill_pack(group, a->max_seqlen_q);
    // the lengths of the query blocks stay on the device: sum_b ceil(rows_b / 128) <= rows / 128 + batch
    const int64_t blocks = ((int64_t)a->total_q * pack + 127) / 128 + a->batch;
    const int64_t tiles = blocks * (pack > 1 ? a->nheads_k : a->nheads);
    int64_t n = 1;
    if (a->num_splits > 1) {
        n = a->num_splits;
    } else {
        const int64_t slots = (int64_t)num_cus * (a->headdim <= 128 ? 2 : 1);
        // query blocks far shorter than the longest one on average (a prompt chunk among decode rows): the
        // longest block is the critical path long before the tiles fill the device, so it is cut earlier
        const bool uneven = uneven_blocks(a);
        if (uneven) {
            if (tiles < 2 * slots) n = (2 * slots + tiles - 1) / tiles;
        } else if (tiles * 2 <= slots) {
            n = (slots + tiles - 1) / tiles;
        }
    }
    const int64_t bound = std::min<int64_t>(a->max_seqlen_k > 0 ? a->max_seqlen_k : INT32_MAX,
                                            (int64_t)a->max_blocks_per_seq * a->page_size);
    const int64_t most = (bound + 255) / 256;   // at least 256 keys (four tiles) per range
    n = std::min<int64_t>(std::min<int64_t>(n, most), 64);
    return (int)std::max<int64_t>(n, 1);
}

size_t fa_rocm_varlen_workspace_bytes(const fa_varlen_args *a, int num_cus) {
    if (fa_rocm_varlen_validate(a) != FA_OK) return 0;
    return varlen_workspace(a, num_cus <= 0 ? 256 : num_cus).total;
}

int fa_rocm_varlen_fwd(const fa_varlen_args *a, void *stream_) {
    const int rc = fa_rocm_varlen_validate(a);
    if (rc != FA_OK) return rc;
    int cus = device_cus();
    if (cus <= 0) cus = 256;
    const VarlenWorkspace w = varlen_workspace(a, cus);
    const int nsplits = w.nsplits;
    if (w.total > 0 && (!a->workspace || a->workspace_bytes < w.total))
        return fail(FA_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", w.total, a->workspace ? a->workspace_bytes : (size_t)0);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (env().validate && a->block_table) {
        const int rv = check_paged_rows("seqused_k", a->seqused_k, a->block_table, a->bt_stride_b, a->batch, 0, a->page_size,
                                        a->max_blocks_per_seq, a->num_blocks, 0, stream);
        if (rv != FA_OK) return rv;
    }
    fa::ShortBlocksParams sr;
    std::memset(&sr, 0, sizeof(sr));
    if (w.short_blocks) {
        // the short blocks: gathered into batch-major blocks of `slots` query positions, computed by the decode kernels
        // with every other sequence's key count set to 0, scattered back after the tiled kernel (which skips them) has
        // been queued
        char *base = static_cast<char *>(a->workspace);
        sr.q = a->q;
        sr.out = a->out;
        sr.lse = a->softmax_lse;
        sr.cu_seqlens_q = a->cu_seqlens_q;
        sr.seqused_k = a->seqused_k;
        sr.q_rows = base + w.q_rows;
        sr.out_rows = base + w.out_rows;
        sr.lse_rows = reinterpret_cast<float *>(base + w.lse_rows);
        sr.lens_rows = reinterpret_cast<int32_t *>(base + w.lens_rows);
        sr.live_rows = reinterpret_cast<int32_t *>(base + w.live_rows);
        if (!w.decode_only) {
            sr.long_ids = reinterpret_cast<int32_t *>(base + w.long_ids);
            sr.list_state = reinterpret_cast<int32_t *>(base + w.list_state);
        }
        sr.batch = a->batch;
        sr.total_q = a->total_q;
        sr.nheads = a->nheads;
        sr.headdim = a->headdim;
        sr.slots = w.slots;
        sr.q_stride_t = a->q_stride_t;
        sr.q_stride_h = a->q_stride_h;
        sr.o_stride_t = a->o_stride_t;
        sr.o_stride_h = a->o_stride_h;
        const hipError_t eg = fa::launch_gather_short_blocks(sr, stream);
        if (eg != hipSuccess) return fail(FA_ERR_LAUNCH, "gather launch failed: %s", hipGetErrorString(eg));
        const fa_kvcache_args k = short_blocks_call(a, base, w);
        // the padded query positions in front of a block's tokens are computed with them but neither stored nor merged
        const int rk = fwd_kvcache_impl(&k, stream_, nullptr, w.slots > 1 ? sr.live_rows : nullptr);
        if (rk != FA_OK) return rk;
    }
    fa::PrefillParams pp;
    std::memset(&pp, 0, sizeof(pp));
    pp.q = a->q;
    pp.k = a->k;
    pp.v = a->v;
    pp.out = a->out;
    pp.lse = a->softmax_lse;
    pp.cu_seqlens_q = a->cu_seqlens_q;
    pp.cu_seqlens_k = a->cu_seqlens_k;
    pp.seqused_k = a->seqused_k;
    pp.block_table = a->block_table;
    pp.batch = a->batch;
    pp.nheads = a->nheads;
    pp.nheads_k = a->nheads_k;
    pp.group = a->nheads / a->nheads_k;
    pp.max_seqlen_q = a->max_seqlen_q;
    pp.total_q = a->total_q;
    pp.page_size = a->page_size;
    pp.max_blocks = a->max_blocks_per_seq;
    pp.num_blocks = a->num_blocks;
    pp.q_stride_t = a->q_stride_t;
    pp.q_stride_h = a->q_stride_h;
    pp.o_stride_t = a->o_stride_t;
    pp.o_stride_h = a->o_stride_h;
    pp.k_stride_t = a->k_stride_t;
    pp.k_stride_h = a->k_stride_h;
    pp.k_stride_block = a->k_stride_block;
    pp.v_stride_t = a->v_stride_t;
    pp.v_stride_h = a->v_stride_h;
    pp.v_stride_block = a->v_stride_block;
    pp.bt_stride_b = a->bt_stride_b;
    pp.headdim = a->headdim;
    pp.lse_stride_b = 0;
    pp.lse_stride_h = a->total_q;
    pp.scale_log2 = a->softmax_scale * kLog2e;
    if (a->softcap > 0.f) {
        pp.softcap_pre = a->softmax_scale / a->softcap;
        pp.softcap_post = a->softcap * kLog2e;
    }
    // window normalisation with max_seqlen_k, as mha_varlen_fwd does (flash_api.cpp:938-943)
    pp.causal = a->causal;
    pp.window_left = a->window_left;
    pp.window_right = a->window_right;
    pp.window_norm_m = a->max_seqlen_k;
    if (nsplits > 1) {
        pp.nsplits = nsplits;
        pp.o_partial = static_cast<float *>(a->workspace);
        pp.lse_partial = pp.o_partial + (size_t)a->total_q * a->nheads * nsplits * fa::tile_headdim(a->headdim);
    }
    pp.skip_short = w.short_blocks ? w.slots : 0;
    if (w.short_blocks && !w.decode_only) {
        // the sequences left to the tiled kernel are listed on the device by the gather kernel
        pp.long_ids = sr.long_ids;
        pp.list_state = sr.list_state;
        pp.list_wgs = cus * (a->headdim <= 128 ? 2 : 1);
    }
    if (!w.decode_only) {
        const hipError_t e = fa::launch_prefill(pp, a->io_dtype, fa::tile_headdim(a->headdim), stream);
        if (e != hipSuccess) return fail(FA_ERR_LAUNCH, "prefill launch failed: %s", hipGetErrorString(e));
        const hipError_t ec = fa::launch_prefill_combine(pp, a->io_dtype, fa::tile_headdim(a->headdim), stream);
        if (ec != hipSuccess) return fail(FA_ERR_LAUNCH, "combine launch failed: %s", hipGetErrorString(ec));
    }
    if (w.short_blocks) {
        const hipError_t es = fa::launch_scatter_short_blocks(sr, stream);
        if (es != hipSuccess) return fail(FA_ERR_LAUNCH, "scatter launch failed: %s", hipGetErrorString(es));
    }
    return FA_OK;
}

}  // extern "C"
