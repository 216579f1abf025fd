/*
 * fa_rocm.h - C ABI of the MI355X (gfx950) paged KV-cache attention library.
 *
 * Plain C: pointers, sizes, PODs.  No torch, no HIP types in the signatures (a
 * stream is passed as void* and must be a hipStream_t or NULL for the default
 * stream).  Every entry point enqueues work on the given stream and returns;
 * nothing here synchronises with the host or allocates device memory, and the
 * only process-wide state is read-only after the first call (the device's
 * compute-unit count and the FA_ROCM_* environment settings, see
 * fa_rocm_reload_env), so calls from several host threads on different
 * streams are safe.  The caller owns every buffer, including the workspace.
 * Two exceptions, each described at its declaration: FA_ROCM_VALIDATE=1 makes
 * the calls wait for a check kernel, and fa_rocm_fwd_kvcache_static keeps its
 * partials in a device array of the library's own.
 *
 * Return value: 0 on success; a negative FA_ERR_* code otherwise, with a
 * human-readable message retrievable (per host thread) via fa_rocm_last_error().
 *
 * Each entry point names the reference interface it stands in for
 * (paths relative to the MinghuasLab/flash-attention-npu checkout).
 */
#ifndef FA_ROCM_H_
#define FA_ROCM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA_ROCM_ABI_VERSION 2

enum fa_dtype { FA_BF16 = 0, FA_FP16 = 1, FA_INT8 = 2 };

enum fa_error {
    FA_OK = 0,
    FA_ERR_NULL = -1,        /* a required pointer is NULL                         */
    FA_ERR_DTYPE = -2,       /* unsupported dtype combination                      */
    FA_ERR_SHAPE = -3,       /* dimension out of the supported range               */
    FA_ERR_UNSUPPORTED = -4, /* feature the reference rejects too (alibi, leftpad) */
    FA_ERR_WORKSPACE = -5,   /* workspace missing or too small                     */
    FA_ERR_LAUNCH = -6       /* HIP reported a launch error                        */
};

/*
 * Arguments of one flash_attn_with_kvcache call on a paged cache.
 * Strides are in ELEMENTS of the tensor's dtype; the last dimension of every
 * tensor is contiguous.  Mirrors the reference's kernel-launch record
 * FwdLaunchArgs (csrc/ascend910/flash_attn_npu/fwd_dispatch.hpp:29-50) plus the
 * parts of FAInferTilingData (tilingdata.h:34-62) the host fills from shapes.
 */
typedef struct fa_kvcache_args {
    /* tensors (device pointers) */
    const void *q;               /* (B, Sq, Hq, Dqk)            io dtype                         */
    void *out;                   /* (B, Sq, Hq, Dv)             io dtype                         */
    float *softmax_lse;          /* (B, Hq, Sq) fp32, natural log; +inf for rows with no key     */
    void *k_cache;               /* (num_blocks, page, Hk, Dqk) kv dtype; written when k_new set */
    void *v_cache;               /* (num_blocks, page, Hk, Dv)  kv dtype; may alias k_cache      */
    float *k_scale_cache;        /* (num_blocks, page, Hk) fp32 per-token scale; int8 cache only;
                                    written for the appended tokens when k_new is given         */
    float *v_scale_cache;        /* same for V; NULL = use k_scale_cache.  Value range of the int8 latent
                                    path: a unit whose keys are cut over several workgroups passes its
                                    normalised partial outputs on as fp16 for either io dtype, so outputs of
                                    magnitude 6e-5 .. 65504 keep 11 significant bits; smaller ones lose bits
                                    and flush to zero below 6e-8, larger ones saturate at 65504           */
    const void *k_new;           /* (B, Snew, Hk, Dqk) io dtype or NULL                          */
    const void *v_new;           /* (B, Snew, Hk, Dv)  io dtype or NULL                          */
    const void *rotary_cos;      /* (seqlen_ro, rotary_dim/2) io dtype or NULL                   */
    const void *rotary_sin;      /* same.  The caller provides seqlen_ro >= cache_seqlens + Snew; the
                                    lengths live on the device, so the call cannot check: a position
                                    past the table uses its last row (no out-of-bounds read)        */
    const int32_t *cache_seqlens;/* (B,) keys already in the cache, per row                      */
    const int32_t *block_table;  /* (B, max_blocks_per_seq) page ids                             */
    void *workspace;             /* >= fa_rocm_kvcache_workspace_bytes(); may be NULL if that is 0 */
    size_t workspace_bytes;

    /* dimensions */
    int32_t batch, seqlen_q, nheads, nheads_k;
    int32_t headdim_qk, headdim_v;   /* equal, a multiple of 8, at most 256 (int8 latent cache: 576 / 512) */
    int32_t seqlen_new;          /* 0 when k_new == NULL */
    int32_t num_blocks, page_size, max_blocks_per_seq;
    int32_t rotary_dim, seqlen_ro;

    /* strides, elements */
    int64_t q_stride_b, q_stride_s, q_stride_h;
    int64_t o_stride_b, o_stride_s, o_stride_h;
    int64_t k_stride_block, k_stride_row, k_stride_h;   /* k_cache */
    int64_t v_stride_block, v_stride_row, v_stride_h;   /* v_cache */
    int64_t ks_stride_block, ks_stride_row;              /* scale caches (head stride 1) */
    int64_t kn_stride_b, kn_stride_s, kn_stride_h;      /* k_new */
    int64_t vn_stride_b, vn_stride_s, vn_stride_h;      /* v_new */
    int64_t bt_stride_b;                                 /* block_table row stride */

    /* scalars */
    int32_t io_dtype;            /* FA_BF16 or FA_FP16                                  */
    int32_t kv_dtype;            /* same as io_dtype, or FA_INT8 (needs *_scale_cache)  */
    float softmax_scale;
    float softcap;               /* 0 = off                                             */
    int32_t causal;              /* bottom-right aligned                                */
    int32_t window_left, window_right;  /* -1 = unbounded                              */
    int32_t rotary_interleaved;
    int32_t num_splits;          /* 0 = heuristic, 1 = no split, >1 = at most that many */
} fa_kvcache_args;

/*
 * Arguments of one flash_attn_varlen_func forward (token-major "TND" layout).
 * K/V are either dense (total_k, Hk, D) addressed through cu_seqlens_k, or paged
 * (block_table != NULL) with per-sequence lengths in seqused_k.  With dense K/V seqused_k is
 * optional: when given, sequence b uses only its first seqused_k[b] keys (the argument of that name of
 * the reference's third-generation host, csrc/ascend910/flash_attn_npu_3/flash_api.cpp:72,143-147).
 */
typedef struct fa_varlen_args {
    const void *q;               /* (total_q, Hq, D) */
    const void *k;               /* (total_k, Hk, D) or paged (num_blocks, page, Hk, D) */
    const void *v;
    void *out;                   /* (total_q, Hq, D) */
    float *softmax_lse;          /* (Hq, total_q) fp32 */
    const int32_t *cu_seqlens_q; /* (B+1,) */
    const int32_t *cu_seqlens_k; /* (B+1,) ; ignored when paged */
    const int32_t *seqused_k;    /* (B,) ; paged: the lengths ; dense: NULL or the keys used per sequence */
    const int32_t *block_table;  /* (B, max_blocks_per_seq) or NULL */
    int32_t batch, total_q, nheads, nheads_k, headdim;
    int32_t max_seqlen_q, max_seqlen_k;
    int32_t page_size, max_blocks_per_seq, num_blocks;   /* paged only */
    int64_t q_stride_t, q_stride_h;
    int64_t k_stride_t, k_stride_h;   /* dense: token stride ; paged: row stride */
    int64_t v_stride_t, v_stride_h;
    int64_t k_stride_block, v_stride_block;
    int64_t o_stride_t, o_stride_h;
    int64_t bt_stride_b;
    int32_t io_dtype;
    float softmax_scale;
    float softcap;
    int32_t causal;
    int32_t window_left, window_right;
    /* Paged K/V only: cut of every sequence's keys into ranges when the query tiles alone cannot fill the
     * device (few sequences, short query blocks, long contexts: chunked prefill, mixed prefill / decode
     * batches).  0 = as many ranges as it takes, 1 = never, n = at most n.  The ranges leave fp32
     * partials in `workspace` (fa_rocm_varlen_workspace_bytes), merged by a second kernel.  The
     * reference's third-generation surface takes num_splits for token-major q the same way
     * (flash_attn_npu_3/flash_attn_npu_interface.py:965-996).
     * When the query blocks are far shorter than the longest one on average
     * (4 * (total_q - max_seqlen_q) <= (batch - 1) * max_seqlen_q: prompt chunks among decode rows), the short blocks - as many
     * tokens as fit 16 rows of tokens x q heads per kv head, at most 8 - are computed by the decode kernels
     * of fa_rocm_fwd_kvcache instead, and so is a whole call whose max_seqlen_q is that short; their
     * batch-major copies and that launch's own workspace are part of `workspace` too.  Which blocks are
     * short is decided on the device, so the call records into a graph like every other. */
    int32_t num_splits;
    void *workspace;
    size_t workspace_bytes;
} fa_varlen_args;

/* Library / device facts. */
int fa_rocm_abi_version(void);
const char *fa_rocm_last_error(void);
/* sizeof the two argument records as this library was compiled (binding self-check). */
size_t fa_rocm_sizeof_kvcache_args(void);
size_t fa_rocm_sizeof_varlen_args(void);
size_t fa_rocm_sizeof_split_plan(void);
/* Compute units of the current HIP device (256 on MI355X); < 0 on error. */
int fa_rocm_num_cus(void);

/*
 * The FA_ROCM_* environment variables are read once, by the first call that needs them; this reads them again
 * (for tests and tuning scripts that change them inside a process; not safe beside calls running on other threads).
 *   FA_ROCM_VALIDATE=1   debugging mode: before any work is queued, fa_rocm_fwd_kvcache* and fa_rocm_varlen_fwd (paged)
 *                        run a check kernel over the data only the device holds and WAIT for it: negative lengths,
 *                        cache_seqlens + seqlen_new beyond the pages of a block_table row (an append past the end),
 *                        page ids outside [0, num_blocks), positions beyond seqlen_ro.  A violation returns
 *                        FA_ERR_SHAPE naming the row; nothing is written.  Not usable under stream capture.
 *                        Calls that validate share one set of result words and take turns on a process-wide lock
 *                        (each holds it for its own check's round trip), whatever their threads and streams.
 *                        Without it these cases are the caller's contract, as in the reference, whose host
 *                        never reads the table either (csrc/ascend910/flash_attn_npu/flash_api.cpp:386-420).
 *   FA_ROCM_DECODE_MAX_ROWS, FA_ROCM_DECODE_WGS, FA_ROCM_DECODE_BLOCK_WORKERS, FA_ROCM_MIN_SHARE, FA_ROCM_PIECE_COST,
 *   FA_ROCM_NO_HEAD_INTERLEAVE, FA_ROCM_SEPARATE_APPEND, FA_ROCM_NO_SHORT_BLOCKS: experiment switches of the decode
 *   partition and the kernel choice; results do not depend on them beyond rounding.
 */
void fa_rocm_reload_env(void);

/*
 * Split-KV plan of a kvcache call, decided from shapes alone (per-row lengths stay on the device).
 * Stands in for the reference's flash-decode heuristic and partition
 * (csrc/ascend910/flash_attn_npu/flash_api.cpp:525-550, splitBN2S1GS2 :343-354; forced mode
 * csrc/ascend910/flash_attn_npu_3/fa_split.h:345-350).
 *   mode FA_SPLIT_BALANCED (num_splits == 0): `num_workers` workers (workgroups, or single waves
 *     when the query block is one 16-row tile) share the list of all 32-key chunks of all
 *     (batch row, kv head) units equally, cutting inside a unit where a share ends; the shares
 *     are computed on the device from cache_seqlens.
 *   mode FA_SPLIT_GRID (num_splits >= 1): every unit is cut into at most `nsplits` ranges of
 *     `split_keys` keys (a multiple of 256); num_splits == 1 gives nsplits == 1 (no split).
 *     Query blocks of more than 32 rows (seqlen_q * nheads / nheads_k) run on the tiled kernel and
 *     always get this mode: num_splits == 0 then picks as many ranges as it takes to fill the device
 *     when the tiles alone cannot (at most 64, at least 256 addressable keys each), and
 *     `split_keys` is 0: the range length is set on the device from the longest sequence.
 * Pure host integer code: needs no GPU.  `num_cus` <= 0 means 256.
 */
enum fa_split_mode { FA_SPLIT_GRID = 0, FA_SPLIT_BALANCED = 1 };
typedef struct fa_split_plan {
    int32_t mode;
    int32_t nsplits;          /* grid mode: split slots per unit (>= 1)          */
    int32_t split_keys;       /* grid mode: keys per split                       */
    int32_t num_wgs;          /* balanced mode: workgroups launched              */
    int32_t num_workers;      /* balanced mode: workers sharing the chunk list (a workgroup, or each of its 4 waves) */
    int32_t min_share;        /* balanced mode: least 32-key chunks per share    */
    size_t workspace_bytes;   /* partial outputs + LSEs the call needs           */
} fa_split_plan;
int fa_rocm_plan_kvcache(const fa_kvcache_args *args, int num_cus, fa_split_plan *plan);

/* Bytes of workspace the kvcache call needs (plan.workspace_bytes; 0 when nothing is split). */
size_t fa_rocm_kvcache_workspace_bytes(const fa_kvcache_args *args, int num_cus);

/*
 * Argument validation only (no GPU work): same checks and messages as the reference host
 * function mha_fwd_kvcache (csrc/ascend910/flash_attn_npu/flash_api.cpp:386-420,455-457).
 */
int fa_rocm_kvcache_validate(const fa_kvcache_args *args);
int fa_rocm_varlen_validate(const fa_varlen_args *args);

/*
 * flash_attn_with_kvcache on a paged cache: optional in-place append of k_new/v_new
 * (with rotary), attention of q over cache_seqlens+seqlen_new keys, split-KV combine.
 * Replaces mha_fwd_kvcache (csrc/ascend910/flash_attn_npu/flash_api.cpp:356-637) and the
 * launch behind it (fwd_dispatch.hpp:60-67, mha_fwd_kvcache.cpp:1025-1106).
 */
int fa_rocm_fwd_kvcache(const fa_kvcache_args *args, void *stream);

/*
 * Same call with phase timing for benchmarks: `events` holds four hipEvent_t handles that the
 * library records on `stream` before the append, after it (before the attention kernel), after
 * the attention kernel and after the combine.  hipEventElapsedTime(events[1], events[2]) is the
 * attention kernel alone.  No counterpart in the reference (its unused host timers are at
 * csrc/ascend910/flash_attn_npu_3/flash_api.cpp:99).
 */
int fa_rocm_fwd_kvcache_profiled(const fa_kvcache_args *args, void *stream, void *const events[4]);

/*
 * flash_attn_varlen_func forward.  Replaces mha_varlen_fwd
 * (csrc/ascend910/flash_attn_npu/flash_api.cpp:848-1089).
 */
int fa_rocm_varlen_fwd(const fa_varlen_args *args, void *stream);

/* Ranges the varlen call cuts every sequence's keys into (1 = no cut), from shapes alone, and the bytes
 * of workspace it then needs (0 when nothing is cut).  Pure host integer code: needs no GPU.
 * `num_cus` <= 0 means 256. */
int fa_rocm_varlen_num_splits(const fa_varlen_args *args, int num_cus);
size_t fa_rocm_varlen_workspace_bytes(const fa_varlen_args *args, int num_cus);

/*
 * The in-place append on its own (k_new/v_new -> pages, rotary on k_new).  The reference
 * documents it (flash_attn_npu/flash_attn_npu_interface.py:1460-1467) but its host drops the
 * tensors (flash_api.cpp:422-427); exposed separately so cache writers can be tested bit-exactly.
 */
int fa_rocm_append_kv(const fa_kvcache_args *args, void *stream);

/*
 * fa_rocm_fwd_kvcache for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose
 * host allocates its workspace on every call (csrc/ascend910/flash_attn_npu/flash_api.cpp:552-567).
 * Same arguments and results as fa_rocm_fwd_kvcache, except that args->workspace / workspace_bytes are
 * ignored: the fp32 split partials go to a static device array of FA_ROCM_STATIC_SCRATCH_BYTES that the
 * library holds on every GPU it runs on until the process ends.  The call allocates and frees nothing.
 * A call whose plan (fa_rocm_plan_kvcache) needs more than that returns FA_ERR_WORKSPACE and enqueues
 * nothing (36 MiB holds the partials of every bf16 / fp16 decode launch, i.e. any query block of up to 32
 * rows = seqlen_q * nheads / nheads_k; the int8 latent kernel's partials at 128 query heads do not fit, and a
 * taller block over few long sequences may not).
 * All calls on one GPU share that GPU's array: two such calls that overlap in time on one device (two
 * streams, two host threads) race on it; calls ordered on one stream do not.  The first call on a
 * device looks the array's address up (a symbol query) and must not be made while a stream is being
 * captured; later calls may.
 */
#define FA_ROCM_STATIC_SCRATCH_BYTES (36u << 20)
int fa_rocm_fwd_kvcache_static(const fa_kvcache_args *args, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FA_ROCM_H_ */
