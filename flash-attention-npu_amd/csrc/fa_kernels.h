// Kernel parameter blocks and host-side launchers of the gfx950 attention kernels.
// The C ABI (fa_rocm_api.cpp) fills these from fa_kvcache_args / fa_varlen_args.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fa {

// Parameters of the paged decode kernel and of the split-KV combine kernel.  Passed by value
// (the counterpart of FAInferTilingData, csrc/ascend910/flash_attn_npu/tilingdata.h:34-62,
// which the reference uploads with a host-to-device copy on every call).
struct DecodeParams {
    const void *q;
    void *out;
    float *lse;
    const void *k_cache;
    const void *v_cache;
    const float *k_scale;
    const float *v_scale;
    const void *k_new;      // fused append (wave-level kernel): rows written by the wave that owns their chunk
    const void *v_new;
    const void *rotary_cos;
    const void *rotary_sin;
    const int32_t *cache_seqlens;
    const int32_t *block_table;
    const int32_t *q_live;   // per batch row: how many query tokens, at the END of the block, are real; the rows of the
                             // others are computed but neither written nor merged.  NULL: all (balanced wave-level launch only)
    float *o_partial;    // (B, Hk, nsplits, rows, Dv) fp32 (fp16 where partials_are_half(Dv)), each normalised by its own sum
    float *lse_partial;  // (B, Hk, nsplits, rows)     fp32, base-2 log-sum-exp, -inf when empty
    int32_t *part_hdr;   // balanced mode, batches of at most 256 rows: kPartitionHeaderBytes in which the decode kernel leaves
                         // its partition for the merge kernel (NULL: the merge kernel recomputes it)
    int32_t batch, seqlen_q, nheads, nheads_k, group, rows;  // rows = seqlen_q * group
    int32_t headdim;     // columns of an output row (and of a q / k / v row, except for the latent cache): a multiple of 8;
                         // the kernels' compile-time width is tile_headdim() of it and the partials are that wide
    int32_t seqlen_new, num_blocks, page_size, max_blocks;
    int32_t rotary_dim, seqlen_ro, rotary_interleaved, rotary_per_token;
    int64_t q_stride_b, q_stride_s, q_stride_h;
    int64_t o_stride_b, o_stride_s, o_stride_h;
    int64_t k_stride_block, k_stride_row, k_stride_h;
    int64_t v_stride_block, v_stride_row, v_stride_h;
    int64_t ks_stride_block, ks_stride_row;
    int64_t kn_stride_b, kn_stride_s, kn_stride_h;
    int64_t vn_stride_b, vn_stride_s, vn_stride_h;
    int64_t bt_stride_b;
    float scale_log2;      // softmax_scale * log2(e)            (softcap off)
    float softcap_pre;     // softmax_scale / softcap            (softcap on)
    float softcap_post;    // softcap * log2(e)
    int32_t causal, window_left, window_right;
    int32_t nsplits, split_keys;   // grid mode: split slots per unit, keys per split
    int32_t balanced, num_wgs;     // balanced mode: workgroups launched
    int32_t num_workers, min_share;  // workers sharing the chunk list (workgroups, or waves), least chunks per share
    int32_t min_share_long;          // > 0: the least share when the units are long (kLongUnitChunks chunks on average)
    int32_t wave_workers;          // 1: every wave is a worker (num_workers = 4 * num_wgs)
    int32_t head_interleave;       // 1: worker w streams share w / Hk of the per-head list for kv head w % Hk
    int32_t piece_cost;            // balanced mode: list length charged for starting on a unit, in chunks (decode_common.h)
    int32_t split_adaptive;        // grid mode: keys per split = adaptive_split_keys(longest sequence, nsplits), not split_keys
    int32_t units_per_token;       // latent int8 cache: 64-head groups per query token (nheads_k = seqlen_q * this); else 0
    int32_t row_tiles;             // > 1: a query block of 17 .. 16 * row_tiles rows is cut into 16-row tiles, each a unit of
                                   // its own for the wave-level kernel: nheads_k = kv heads * row_tiles units per batch row (unit =
                                   // kv head * row_tiles + tile), rows = 16 per unit, rows_total = seqlen_q * group; else 0 or 1
    int32_t rows_total;            // seqlen_q * group when row_tiles > 1
};

struct AppendParams {
    void *k_cache;
    void *v_cache;
    const void *k_new;
    const void *v_new;
    const void *rotary_cos;
    const void *rotary_sin;
    float *k_scale;      // int8 latent cache: per-token scales written by the quantising append
    float *v_scale;
    const int32_t *cache_seqlens;
    const int32_t *block_table;
    int32_t batch, seqlen_new, nheads_k, headdim_qk, headdim_v;
    int32_t num_blocks, page_size, max_blocks;
    int32_t rotary_dim, seqlen_ro, rotary_interleaved;
    int64_t k_stride_block, k_stride_row, k_stride_h;
    int64_t v_stride_block, v_stride_row, v_stride_h;
    int64_t kn_stride_b, kn_stride_s, kn_stride_h;
    int64_t vn_stride_b, vn_stride_s, vn_stride_h;
    int64_t ks_stride_block, ks_stride_row;
    int64_t bt_stride_b;
};

// Rotation of the query block of a kvcache call into a contiguous (B, Sq, Hq, D) copy, for the
// query blocks that go to the tiled forward (the decode kernels rotate q while they stage it).
struct RotateQParams {
    const void *q;
    void *out;
    const void *rotary_cos;
    const void *rotary_sin;
    const int32_t *cache_seqlens;
    int32_t batch, seqlen_q, nheads, headdim;
    int32_t rotary_dim, seqlen_ro, rotary_interleaved, rotary_per_token;
    int64_t q_stride_b, q_stride_s, q_stride_h;
};

// Short query blocks (1 .. slots tokens) of a token-major batch between the token-major tensors of the call
// and the batch-major blocks (B, slots, Hq, D) / (B, Hq, slots) that the decode kernels work on; a block of n
// tokens occupies the last n slots.
struct ShortBlocksParams {
    const void *q;                 // (total_q, Hq, D)
    void *out;                     // (total_q, Hq, D)
    float *lse;                    // (Hq, total_q)
    const int32_t *cu_seqlens_q;   // (B + 1,)
    const int32_t *seqused_k;      // (B,)
    void *q_rows;                  // (B, slots, Hq, D) contiguous
    const void *out_rows;          // (B, slots, Hq, D) contiguous
    const float *lse_rows;         // (B, Hq, slots)
    int32_t *lens_rows;            // (B,): seqused_k of the short blocks' sequences, 0 for the others
    int32_t *live_rows;            // (B,): tokens of the short blocks (their real query positions), 0 for the others
    int32_t *long_ids;             // (B,): the sequences with more than `slots` tokens, in batch order
    int32_t *list_state;           // [0] = how many, [1..8] = 0 (block counters of the tiled launch that follows)
    int32_t batch, total_q, nheads, headdim, slots;
    int64_t q_stride_t, q_stride_h, o_stride_t, o_stride_h;
};

// Parameters of the tiled (MFMA) forward used for varlen prefill and for kvcache calls whose
// query block does not fit the decode kernel.
struct PrefillParams {
    const void *q;
    const void *k;
    const void *v;
    void *out;
    float *lse;
    const int32_t *cu_seqlens_q;   // NULL: fixed seqlen_q per batch row (kvcache layout)
    const int32_t *cu_seqlens_k;   // dense K/V only
    const int32_t *seqused_k;      // paged: keys per row (cache_seqlens); dense: optional, the keys used of each sequence
    const int32_t *block_table;    // NULL: dense K/V
    int32_t batch, nheads, nheads_k, group;
    int32_t headdim;               // columns of a q / k / v / out row, a multiple of 8; the kernel is compiled for tile_headdim() of it
    int32_t pack;                  // set by the launcher: 1, or group when tile rows are (query, head) pairs
    int32_t pack_short;            // set by the launcher: pack == 1, but a short query block packs its heads on its own
    int32_t skip_short;            // token-major q: sequences with 1 .. skip_short query tokens are computed elsewhere (0 = none)
    // token-major q whose live sequences are listed on the device (with skip_short): the sequences with more than
    // skip_short tokens, list_state[0] of them; list_state[1..8] are the per-XCD block counters of the launch, zero
    // when it starts; list_wgs workgroups are launched (as many as the device holds)
    const int32_t *long_ids;
    int32_t *list_state;
    int32_t list_wgs;
    int32_t num_mb, units8;        // set by the launcher: 128-row blocks per unit, units rounded up to 8
    int32_t seqlen_q_fixed, seqlen_k_add;   // kvcache layout: Sq per row, keys appended this call
    int32_t max_seqlen_q, total_q;
    int32_t page_size, max_blocks, num_blocks;
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t o_stride_b, o_stride_t, o_stride_h;
    int64_t k_stride_t, k_stride_h, k_stride_block;
    int64_t v_stride_t, v_stride_h, v_stride_block;
    int64_t bt_stride_b;
    int64_t lse_stride_b, lse_stride_h;     // lse index = b*stride_b + h*stride_h + token
    float scale_log2, softcap_pre, softcap_post;
    int32_t causal, window_left, window_right;
    int32_t window_norm_m;                  // key count the window is normalised with; 0 = each row's own
    // split of the keys (paged K/V): ranges of adaptive_split_keys() keys; a query block cut into several
    // ranges leaves fp32 partials and base-2 LSEs, in slot (batch row * nheads_k + kv head) * nsplits + split
    // of `rows` rows each for the split-KV combine kernel (kvcache layout), or at
    // (token * nheads + head) * nsplits + split for prefill_combine_kernel (token-major q)
    int32_t nsplits, rows;                  // rows = seqlen_q_fixed * group
    float *o_partial;
    float *lse_partial;
};

// The partial rows of the 512-column kernel (the int8 latent cache: 128 heads x 512 columns per piece) are kept as
// fp16: they are normalised outputs, i.e. averages of dequantised cache rows (11 significant bits against the 8 or 11
// of the final rounding), and halving them halves what the split costs in writes and in the merge's reads.  Their
// writer clamps to the fp16 range: outputs of magnitude 6e-5 .. 65504 are independent of the partition up to the
// rounding of the I/O type, smaller ones lose bits (zero below 6e-8) and larger ones saturate, for bf16 I/O as well.
// Every other width keeps fp32 partials.
constexpr bool partials_are_half(int dv) { return dv == 512; }

// Balanced mode: the partition of a launch (share size, list length, prefix of the rows' chunk counts) as the decode
// kernel computed it, left behind the partials for the merge kernel.
// Few long units (a handful of sequences with a long window) are cut into shares of at least min_share_long chunks:
// 32 units x 128 chunks over 2048 waves ran 26.4 us with 2-chunk shares and 25.5 us with 4-chunk shares, while many
// short units (64 x 8 heads x 8 chunks) go the other way (28.8 against 33.4 us).  The lengths live on the device, so
// the choice is made there.
constexpr int kLongUnitChunks = 64;
constexpr int kPartitionHeaderInts = 8;                 // M, cost, W (2), S (2), 2 spare; then prefix[0 .. batch]
constexpr size_t kPartitionHeaderBytes = 2048;          // 8 + 257 ints, rounded up


// Width the kernels are compiled for, for a head dimension of d columns.
inline int tile_headdim(int d) { return d <= 64 ? 64 : d <= 128 ? 128 : 256; }

// ---- planning rules shared by the host API and the launchers (host integer code; 64-bit inside so that no
// combination of 32-bit dimensions overflows) ----
constexpr int kPrefillTileRows = 128;   // query rows of one tile of the tiled forward

// GQA group packed into the tile rows of the tiled forward for query blocks of max_seqlen_q rows
// (1 = one q head per tile): the heads of a group share a tile when that saves at least a quarter of the tiles.
inline int prefill_pack(int group, int max_seqlen_q) {
    if (group <= 1 || max_seqlen_q <= 0) return 1;
    const int64_t tiles_plain = (int64_t)group * (((int64_t)max_seqlen_q + kPrefillTileRows - 1) / kPrefillTileRows);
    const int64_t tiles_packed = ((int64_t)max_seqlen_q * group + kPrefillTileRows - 1) / kPrefillTileRows;
    return tiles_packed * 4 <= tiles_plain * 3 ? group : 1;
}
// 1 when the blocks of a token-major launch that does not pack (prefill_pack == 1) pack on their own where they are
// short: blocks that differ in length and whose average would pack (mixed prefill / decode batches).
inline int prefill_pack_short(int group, int max_seqlen_q, int total_q, int batch) {
    if (group <= 1 || batch <= 0 || total_q <= 0 || prefill_pack(group, max_seqlen_q) > 1) return 0;
    return prefill_pack(group, (int)(((int64_t)total_q + batch - 1) / batch)) > 1 ? 1 : 0;
}
// Tiles (workgroups) of the tiled forward per batch row.
inline int64_t prefill_tiles(int nheads, int nheads_k, int max_seqlen_q) {
    const int pack = prefill_pack(nheads / nheads_k, max_seqlen_q);
    return (int64_t)(pack > 1 ? nheads_k : nheads) * (((int64_t)max_seqlen_q * pack + kPrefillTileRows - 1) / kPrefillTileRows);
}

// dtype: 0 = bf16, 1 = fp16 (enum fa_dtype).  All return hipError_t of the launch.
hipError_t launch_append_kv(const AppendParams &p, int dtype, hipStream_t stream);
hipError_t launch_append_quant_i8(const AppendParams &p, int dtype, hipStream_t stream);
hipError_t launch_rotate_q(const RotateQParams &p, int dtype, hipStream_t stream);
hipError_t launch_decode_paged(const DecodeParams &p, int dtype, int headdim, hipStream_t stream);
hipError_t launch_decode_wave(const DecodeParams &p, int dtype, int headdim, hipStream_t stream);
hipError_t launch_splitkv_combine(const DecodeParams &p, int dtype, int headdim_v, hipStream_t stream);
hipError_t launch_decode_mla_i8(const DecodeParams &p, int dtype, hipStream_t stream);
hipError_t launch_prefill(const PrefillParams &p, int dtype, int headdim, hipStream_t stream);
// merge of the key ranges of token-major query blocks (cu_seqlens_q set, nsplits > 1) after launch_prefill
hipError_t launch_prefill_combine(const PrefillParams &p, int dtype, int headdim, hipStream_t stream);

hipError_t launch_gather_short_blocks(const ShortBlocksParams &p, hipStream_t stream);
hipError_t launch_scatter_short_blocks(const ShortBlocksParams &p, hipStream_t stream);

// Resident decode workgroups per compute unit for a head dimension / query-block height.
inline int decode_wgs_per_cu(int headdim, int rows) { return (headdim <= 128 && rows <= 32) ? 2 : 1; }

// Which kernel takes a query block of rows = seqlen_q * group rows (balanced partition), by measurement with a cold
// cache (the pools of a step rotated past the 256 MB last-level cache; 64 sequences x 8 K keys, one query token, 32 q
// heads per kv head; whole call in us: wave-level kernel / tiled kernel, both filling their LDS tiles straight from
// global memory):
//   D = 128: 8 kv heads (2.1 GB) 364 (5.9 TB/s) / 392; 4 kv heads 204 / 217; 2 kv heads 127 / 113; 1 kv head 87 / 66
//   D = 64:  8 kv heads (1.1 GB) 193 (5.6 TB/s) / workgroup-level decode kernel 212; 1 kv head (134 MB) 50 / 44
//   D = 256: 8 kv heads (4.3 GB), the block as two 16-row units of the wave-level kernel 1050 / tiled 830 (5.2 TB/s)
// A stream like this is bounded by the bytes it keeps in flight, and the wave-level kernel keeps every wave's chunk in
// flight for all the rows of a block: with two 16-row tiles in one wave (D <= 128, where the registers that used to
// stage K hold the second set of accumulators) one pass over the keys serves 32 rows.  That pays when the units are
// cut into few pieces (at least as many units as compute units: the host's rule, wave_max_rows() in fa_rocm_api.cpp);
// cut 16 or 32 ways, the fixed costs of the pieces and their merge outweigh it.  At D = 256 the accumulators of two
// tiles do not fit a wave, and tiles as units of their own read the keys twice (1.7 x the traffic).  Up to 16 rows the
// wave-level kernel is far ahead everywhere; from 33 rows on the tiled kernel runs (64 rows x 8 kv heads: 418 us,
// 5.2 TB/s).
// Tallest block for the workgroup-level decode kernels (decode_balanced_kernel; decode_paged_kernel for explicit
// num_splits); kDecodeMaxRows is what those kernels can take at all (two 16-row tiles).
constexpr int kDecodeMaxRows = 32;
inline int block_decode_max_rows(int tile_headdim) { return tile_headdim == 64 ? 32 : 16; }
// Rows of a unit of the wave-level kernel: one 16-row tile per wave, or two where the registers of a wave that shares
// its SIMD with another hold two sets of accumulators (D <= 128).
constexpr int wave_rows_per_unit(int tile_headdim) { return tile_headdim <= 128 ? 32 : 16; }


}  // namespace fa
