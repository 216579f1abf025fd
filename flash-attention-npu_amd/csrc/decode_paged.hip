// Paged GQA/MQA decode for gfx950: one workgroup per (batch row, kv head, KV split) that packs
// every query row of the group (seqlen_q * group <= 64) and streams the row's K/V pages once.
//
// It takes the place of the reference's FAInfer task loop for decode-shaped calls
// (csrc/ascend910/flash_attn_npu/mha_fwd_kvcache.cpp:436-970: paged addressing :496,527, key-range
// clipping :556-595, 512-key online-softmax loop :632-969) and of its flash-decode epilogue
// (CombineScale.hpp:76-357), with these differences of design:
//   * each of the NW wavefronts walks its own 32-key chunks with a private running (max, sum, O);
//     there is no workgroup barrier in the stream loop, waves merge once at the end through LDS;
//   * K rows are fetched as whole 16-byte-per-lane coalesced rows, staged through a swizzled LDS
//     tile and read back in MFMA operand order; V rows are fetched straight into the operand
//     order (lanes 16q..16q+15 read one whole row) and transposed in registers with v_perm;
//   * S^T = K Q^T and O^T = V^T P^T run on the 16x16x32 MFMA so the softmax state of a query row
//     lives in one lane column for both products (no cross-lane traffic for the rescale);
//   * lengths are read on the device; no host copy of cache_seqlens, no mask tensor.
#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {

constexpr int kChunk = 32;  // keys per wave step

template <int D> struct DecodeCfg {
    static constexpr int kLanesPerRow = D / 8;            // 16-byte pieces in one K row
    static constexpr int kRowsPerLoad = 64 / kLanesPerRow;
    static constexpr int kKLoads = kChunk / kRowsPerLoad;  // K load instructions per chunk
    static constexpr int kKSteps = D / 32;                 // MFMA k-steps of QK^T
    static constexpr int kVW = (D >= 128) ? 8 : D / 16;    // V columns one lane holds per key and pass
    static constexpr int kVH = D / (16 * kVW);             // column passes (128 columns each)
    static constexpr int kColTiles = D / 16;               // 16-column tiles of O^T
    static constexpr int kSwzMask = (kLanesPerRow >= 16) ? 15 : kLanesPerRow - 1;
};

// byte offset of 16-byte piece `ch` of row `row` in a wave's swizzled K tile
template <int D> __device__ __forceinline__ int k_tile_offset(int row, int ch) {
    return row * (D * 2) + ((ch ^ (row & DecodeCfg<D>::kSwzMask)) << 4);
}

template <typename T, int D, int RT, int NW, bool SOFTCAP>
__global__ void __launch_bounds__(NW * 64, (D <= 128 && RT <= 2) ? 2 : 1)
decode_paged_kernel(const DecodeParams p) {
    using Cfg = DecodeCfg<D>;
    constexpr int ROWS = 16 * RT;
    constexpr int K_TILE_BYTES = kChunk * D * 2;
    constexpr int O_STAGE_BYTES = ROWS * D * 4;
    constexpr int MAIN_BYTES = (NW * K_TILE_BYTES > O_STAGE_BYTES) ? NW * K_TILE_BYTES : O_STAGE_BYTES;

    __shared__ __attribute__((aligned(16))) uint8_t s_main[MAIN_BYTES];  // K tiles, later the O merge buffer
    __shared__ __attribute__((aligned(16))) uint16_t s_q[ROWS * D];
    __shared__ float s_m[NW][ROWS];
    __shared__ float s_l[NW][ROWS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lq = lane >> 4;   // lane group: MFMA k-slot / key sub-block
    const int ln = lane & 15;   // MFMA row or column index

    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    const int b = blockIdx.z;

    const int len_cache = p.cache_seqlens[b];
    const int Lk = len_cache + p.seqlen_new;
    const int Sq = p.seqlen_q;
    const int off = Lk - Sq;
    const int wr_eff = p.causal ? 0 : p.window_right;
    const int wl = p.window_left;

    // live key range of the whole query block
    int lo = 0, hi = Lk;
    if (wr_eff >= 0) hi = min(Lk, Sq - 1 + off + wr_eff + 1);
    if (wl >= 0) lo = max(0, off - wl);
    const bool empty = (Lk <= 0) || (hi <= lo);
    const int lo_al = lo & ~(kChunk - 1);
    // splits this row really has; the grid was sized from shapes, so clamp and let the last split
    // run to the end of the range if the caller's lengths exceed what the shapes promised
    const int nsplits_row = empty ? 1 : min(p.nsplits, (hi - lo_al + p.split_keys - 1) / p.split_keys);
    if (split >= nsplits_row) return;
    const bool write_final = (nsplits_row == 1);

    int range_lo = lo, range_hi = hi;
    if (!empty) {
        range_lo = max(lo, lo_al + split * p.split_keys);
        range_hi = (split == nsplits_row - 1) ? hi : min(hi, lo_al + (split + 1) * p.split_keys);
    } else {
        range_lo = 0;
        range_hi = 0;
    }

    // ---- stage Q (with rotary) into LDS as 16-bit rows -------------------------------------
    {
        const uint16_t *qbase = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_stride_b;
        const uint16_t *cosT = reinterpret_cast<const uint16_t *>(p.rotary_cos);
        const uint16_t *sinT = reinterpret_cast<const uint16_t *>(p.rotary_sin);
        const int rot = (cosT != nullptr) ? p.rotary_dim : 0;
        const int half = rot >> 1;
        for (int idx = tid; idx < ROWS * (D / 2); idx += NW * 64) {
            const int row = idx / (D / 2);
            const int c = idx - row * (D / 2);
            int d1, d2;
            if (c < half) {
                d1 = p.rotary_interleaved ? 2 * c : c;
                d2 = p.rotary_interleaved ? 2 * c + 1 : c + half;
            } else {
                d1 = rot + 2 * (c - half);
                d2 = d1 + 1;
            }
            uint16_t o1 = 0, o2 = 0;
            if (row < p.rows) {
                const int qi = row / p.group;
                const int g = row - qi * p.group;
                const uint16_t *src = qbase + (int64_t)qi * p.q_stride_s + (int64_t)(kvh * p.group + g) * p.q_stride_h;
                o1 = src[d1];
                o2 = src[d2];
                if (c < half) {
                    int pos = len_cache + (p.rotary_per_token ? qi : 0);
                    pos = min(max(pos, 0), p.seqlen_ro - 1);
                    const float cs = to_float<T>(cosT[(int64_t)pos * half + c]);
                    const float sn = to_float<T>(sinT[(int64_t)pos * half + c]);
                    const float x1 = to_float<T>(o1), x2 = to_float<T>(o2);
                    const float r1 = __fsub_rn(__fmul_rn(x1, cs), __fmul_rn(x2, sn));
                    const float r2 = __fadd_rn(__fmul_rn(x1, sn), __fmul_rn(x2, cs));
                    o1 = from_float<T>(r1);
                    o2 = from_float<T>(r2);
                }
            }
            s_q[row * D + d1] = o1;
            s_q[row * D + d2] = o2;
        }
    }
    __syncthreads();

    // Q^T as MFMA B operand: lane (lq, ln) holds row ln, elements t*32 + lq*8 .. +7
    u32x4_t qreg[RT][Cfg::kKSteps];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < Cfg::kKSteps; ++t)
            qreg[r][t] = *reinterpret_cast<const u32x4_t *>(&s_q[(r * 16 + ln) * D + t * 32 + lq * 8]);

    // per-lane visible key interval of query row (r*16 + ln), clipped to this split
    int row_lo[RT], row_hi[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int row = r * 16 + ln;
        const int qi = row / p.group;
        int klo = range_lo, khi = range_hi - 1;
        if (wl >= 0) klo = max(klo, qi + off - wl);
        if (wr_eff >= 0) khi = min(khi, qi + off + wr_eff);
        if (row >= p.rows) khi = -1;
        row_lo[r] = klo;
        row_hi[r] = khi;
    }

    float m_run[RT], l_run[RT];
    float4_t o_acc[RT][Cfg::kColTiles];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        m_run[r] = -INFINITY;
        l_run[r] = 0.f;
#pragma unroll
        for (int t = 0; t < Cfg::kColTiles; ++t) o_acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    uint8_t *ktile = s_main + wave * K_TILE_BYTES;
    const uint8_t *kc_base = reinterpret_cast<const uint8_t *>(p.k_cache) + (int64_t)kvh * p.k_stride_h * 2;
    const uint8_t *vc_base = reinterpret_cast<const uint8_t *>(p.v_cache) + (int64_t)kvh * p.v_stride_h * 2;
    const int32_t *bt_row = p.block_table + (int64_t)b * p.bt_stride_b;

    const int c_begin = range_lo / kChunk;
    const int c_end = (range_hi + kChunk - 1) / kChunk;

    u32x4_t kreg[Cfg::kKLoads];
    uint32_t vreg[8][Cfg::kVH][Cfg::kVW / 2];

    // per-lane byte offsets inside a page that do not change from chunk to chunk
    const uint32_t k_row_bytes = (uint32_t)p.k_stride_row * 2u;
    const uint32_t v_row_bytes = (uint32_t)p.v_stride_row * 2u;
    const int k_lane_row = lane / Cfg::kLanesPerRow;
    const uint32_t k_lane_col = (uint32_t)(lane % Cfg::kLanesPerRow) * 16u;
    const uint32_t v_lane_col = (uint32_t)(ln * Cfg::kVW) * 2u;
    uint32_t koff[Cfg::kKLoads], voff[8];
#pragma unroll
    for (int j = 0; j < Cfg::kKLoads; ++j) koff[j] = (uint32_t)(j * Cfg::kRowsPerLoad + k_lane_row) * k_row_bytes + k_lane_col;
#pragma unroll
    for (int e = 0; e < 8; ++e) voff[e] = (uint32_t)((e >> 2) * 16 + lq * 4 + (e & 3)) * v_row_bytes + v_lane_col;

    // page id of chunk c (clamped into the pool so a corrupt table cannot fault)
    auto fetch_blk = [&](int c) -> int {
        if (c >= c_end) return 0;
        int page = (c * kChunk) / p.page_size;
        page = min(page, p.max_blocks - 1);
        const int blk = __builtin_amdgcn_readfirstlane(bt_row[page]);
        return min(max(blk, 0), p.num_blocks - 1);
    };

    auto load_v = [&](const uint8_t *s2, int e, int hh) {
        if constexpr (Cfg::kVW == 8) {
            const u32x4_t t4 = load16(s2);
            vreg[e][hh][0] = t4[0];
            vreg[e][hh][1] = t4[1];
            vreg[e][hh][2] = t4[2];
            vreg[e][hh][3] = t4[3];
        } else if constexpr (Cfg::kVW == 4) {
            const uint2 t2 = *reinterpret_cast<const uint2 *>(s2);
            vreg[e][hh][0] = t2.x;
            vreg[e][hh][1] = t2.y;
        } else {
            vreg[e][hh][0] = *reinterpret_cast<const uint32_t *>(s2);
        }
    };

    auto issue_loads = [&](int c, int blk) {
        const int key0 = c * kChunk;
        const int inpage0 = key0 % p.page_size;
        const int last = Lk - 1 - key0;  // last initialised key, relative to the chunk (>= 0)
        const uint8_t *kb = kc_base + (int64_t)blk * p.k_stride_block * 2 + (int64_t)inpage0 * k_row_bytes;
        const uint8_t *vb = vc_base + (int64_t)blk * p.v_stride_block * 2 + (int64_t)inpage0 * v_row_bytes;
        if (last >= kChunk - 1) {
#pragma unroll
            for (int j = 0; j < Cfg::kKLoads; ++j) kreg[j] = load16(kb + koff[j]);
#pragma unroll
            for (int e = 0; e < 8; ++e)
#pragma unroll
                for (int hh = 0; hh < Cfg::kVH; ++hh) load_v(vb + voff[e] + hh * 256, e, hh);
        } else {
            // tail chunk: rows past the last written key re-read that key (their scores are masked)
#pragma unroll
            for (int j = 0; j < Cfg::kKLoads; ++j) {
                const int row = min(j * Cfg::kRowsPerLoad + k_lane_row, last);
                kreg[j] = load16(kb + (uint32_t)row * k_row_bytes + k_lane_col);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int row = min((e >> 2) * 16 + lq * 4 + (e & 3), last);
#pragma unroll
                for (int hh = 0; hh < Cfg::kVH; ++hh) load_v(vb + (uint32_t)row * v_row_bytes + v_lane_col + hh * 256, e, hh);
            }
        }
    };

    int c = c_begin + wave;
    int blk_next = fetch_blk(c);
    if (c < c_end) issue_loads(c, blk_next);
    blk_next = fetch_blk(c + NW);

    while (c < c_end) {
        // ---- move the staged chunk: K -> swizzled LDS tile, V -> transposed operand registers
#pragma unroll
        for (int j = 0; j < Cfg::kKLoads; ++j) {
            const int row = j * Cfg::kRowsPerLoad + lane / Cfg::kLanesPerRow;
            const int ch = lane % Cfg::kLanesPerRow;
            *reinterpret_cast<u32x4_t *>(ktile + k_tile_offset<D>(row, ch)) = kreg[j];
        }
        // vt[T]: 8 keys of column tile T for this lane's column; dword u = keys (2u, 2u+1)
        u32x4_t vt[Cfg::kColTiles];
#pragma unroll
        for (int hh = 0; hh < Cfg::kVH; ++hh)
#pragma unroll
            for (int w2 = 0; w2 < Cfg::kVW / 2; ++w2)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t a = vreg[2 * u][hh][w2];
                    const uint32_t bb = vreg[2 * u + 1][hh][w2];
                    vt[hh * Cfg::kVW + 2 * w2][u] = __builtin_amdgcn_perm(bb, a, 0x05040100u);
                    vt[hh * Cfg::kVW + 2 * w2 + 1][u] = __builtin_amdgcn_perm(bb, a, 0x07060302u);
                }
        __builtin_amdgcn_wave_barrier();

        const int cn = c + NW;
        if (cn < c_end) issue_loads(cn, blk_next);
        blk_next = fetch_blk(cn + NW);
        __builtin_amdgcn_sched_barrier(0);

        // ---- S^T = K Q^T : two 16-key tiles x RT row tiles
        float4_t s[2][RT];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < RT; ++r) s[tt][r] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < Cfg::kKSteps; ++t)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const u32x4_t a =
                    *reinterpret_cast<const u32x4_t *>(ktile + k_tile_offset<D>(tt * 16 + ln, t * 4 + lq));
#pragma unroll
                for (int r = 0; r < RT; ++r) s[tt][r] = mfma16<T>(a, qreg[r][t], s[tt][r]);
            }

        // ---- online softmax per query row (lane column ln of tile r)
        const int key_base = c * kChunk + lq * 4;
        u32x4_t pk[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            float x[8];
            float mloc = -INFINITY;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = key_base + (e >> 2) * 16 + (e & 3);
                float v = s[e >> 2][r][e & 3];
                if constexpr (SOFTCAP) {
                    // cap * tanh(s*scale/cap), then to base 2
                    const float y = v * p.softcap_pre;
                    const float e2 = __expf(2.f * y);
                    v = p.softcap_post * (1.f - 2.f / (e2 + 1.f));
                } else {
                    v *= p.scale_log2;
                }
                const bool vis = (key >= row_lo[r]) && (key <= row_hi[r]);
                v = vis ? v : -INFINITY;
                x[e] = v;
                mloc = fmaxf(mloc, v);
            }
            mloc = quad_rows_max(mloc);
            const float m_new = fmaxf(m_run[r], mloc);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run[r] - m_use);
            m_run[r] = m_new;
            float psum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[e] = fast_exp2(x[e] - m_use);
                psum += x[e];
            }
            l_run[r] = l_run[r] * alpha + psum;
            pk[r][0] = pack2<T>(x[0], x[1]);
            pk[r][1] = pack2<T>(x[2], x[3]);
            pk[r][2] = pack2<T>(x[4], x[5]);
            pk[r][3] = pack2<T>(x[6], x[7]);
#pragma unroll
            for (int t = 0; t < Cfg::kColTiles; ++t) {
                o_acc[r][t][0] *= alpha;
                o_acc[r][t][1] *= alpha;
                o_acc[r][t][2] *= alpha;
                o_acc[r][t][3] *= alpha;
            }
        }

        // ---- O^T += V^T P^T
#pragma unroll
        for (int t = 0; t < Cfg::kColTiles; ++t)
#pragma unroll
            for (int r = 0; r < RT; ++r) o_acc[r][t] = mfma16<T>(vt[t], pk[r], o_acc[r][t]);

        c = cn;
    }

    // ---- merge the waves --------------------------------------------------------------------
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        l_run[r] = quad_rows_sum(l_run[r]);
        if (lq == 0) {
            s_m[wave][r * 16 + ln] = m_run[r];
            s_l[wave][r * 16 + ln] = l_run[r];
        }
    }
    __syncthreads();  // also: every wave is done with its K tile

    float fac[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        float mg = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) mg = fmaxf(mg, s_m[w][r * 16 + ln]);
        const float mg_use = (mg == -INFINITY) ? 0.f : mg;
        fac[r] = fast_exp2(m_run[r] - mg_use);
    }

    float *o_stage = reinterpret_cast<float *>(s_main);  // [ROWS][D]
    for (int w = 0; w < NW; ++w) {
        if (wave == w) {
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int t = 0; t < Cfg::kColTiles; ++t) {
                    const int hh = t / Cfg::kVW, w2 = t % Cfg::kVW;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int col = hh * 128 + (lq * 4 + i) * Cfg::kVW + w2;
                        float *dst = &o_stage[(r * 16 + ln) * D + col];
                        const float v = o_acc[r][t][i] * fac[r];
                        if (w == 0) *dst = v; else *dst += v;
                    }
                }
        }
        __syncthreads();
    }

    // ---- write: final output or split partial ------------------------------------------------
    constexpr int PIECES = D / 8;  // 8-column pieces per row
    for (int idx = tid; idx < p.rows * PIECES; idx += NW * 64) {
        const int row = idx / PIECES;
        const int piece = idx - row * PIECES;
        float mg = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) mg = fmaxf(mg, s_m[w][row]);
        const float mg_use = (mg == -INFINITY) ? 0.f : mg;
        float lg = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) lg += s_l[w][row] * fast_exp2(s_m[w][row] - mg_use);
        const float inv = (lg > 0.f) ? 1.f / lg : 0.f;
        const float *src = &o_stage[row * D + piece * 8];
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = src[e] * inv;
        const int qi = row / p.group;
        const int g = row - qi * p.group;
        const int head = kvh * p.group + g;
        if (write_final) {
            u32x4_t o4;
            o4[0] = pack2<T>(v[0], v[1]);
            o4[1] = pack2<T>(v[2], v[3]);
            o4[2] = pack2<T>(v[4], v[5]);
            o4[3] = pack2<T>(v[6], v[7]);
            uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                            (int64_t)head * p.o_stride_h + piece * 8;
            store16(dst, o4);
            if (piece == 0)
                p.lse[((int64_t)b * p.nheads + head) * Sq + qi] = (lg > 0.f) ? (mg + fast_log2(lg)) * kLn2 : INFINITY;
        } else {
            const int64_t slot = (((int64_t)b * p.nheads_k + kvh) * p.nsplits + split) * p.rows + row;
            float *dst = p.o_partial + slot * D + piece * 8;
            *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4 *>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
            if (piece == 0) p.lse_partial[slot] = (lg > 0.f) ? mg + fast_log2(lg) : -INFINITY;
        }
    }
}

// Split-KV combine (CombineScale.hpp:166-194,249-316): LSE = M + log sum exp(lse_s - M),
// out = sum exp(lse_s - LSE) * O_s.  One workgroup per (batch row, kv head, query row).
template <typename T, int D>
__global__ void __launch_bounds__(D / 4) splitkv_combine_kernel(const DecodeParams p) {
    const int row = blockIdx.x;
    const int kvh = blockIdx.y;
    const int b = blockIdx.z;
    const int tid = threadIdx.x;  // owns 4 columns

    const int Lk = p.cache_seqlens[b] + p.seqlen_new;
    const int Sq = p.seqlen_q;
    const int off = Lk - Sq;
    const int wr_eff = p.causal ? 0 : p.window_right;
    int lo = 0, hi = Lk;
    if (wr_eff >= 0) hi = min(Lk, Sq - 1 + off + wr_eff + 1);
    if (p.window_left >= 0) lo = max(0, off - p.window_left);
    const bool empty = (Lk <= 0) || (hi <= lo);
    const int lo_al = lo & ~(kChunk - 1);
    const int ns = empty ? 1 : min(p.nsplits, (hi - lo_al + p.split_keys - 1) / p.split_keys);
    if (ns == 1) return;  // the decode kernel already wrote this row

    const int64_t slot0 = (((int64_t)b * p.nheads_k + kvh) * p.nsplits) * p.rows + row;
    float mx = -INFINITY;
    for (int s = 0; s < ns; ++s) mx = fmaxf(mx, p.lse_partial[slot0 + (int64_t)s * p.rows]);
    const float mx_use = (mx == -INFINITY) ? 0.f : mx;
    float tot = 0.f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < ns; ++s) {
        const int64_t slot = slot0 + (int64_t)s * p.rows;
        const float w = fast_exp2(p.lse_partial[slot] - mx_use);
        tot += w;
        const float4 o = *reinterpret_cast<const float4 *>(p.o_partial + slot * D + tid * 4);
        acc[0] += w * o.x;
        acc[1] += w * o.y;
        acc[2] += w * o.z;
        acc[3] += w * o.w;
    }
    const float inv = (tot > 0.f) ? 1.f / tot : 0.f;
    const int qi = row / p.group;
    const int g = row - qi * p.group;
    const int head = kvh * p.group + g;
    uint2 o2;
    o2.x = pack2<T>(acc[0] * inv, acc[1] * inv);
    o2.y = pack2<T>(acc[2] * inv, acc[3] * inv);
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                    (int64_t)head * p.o_stride_h + tid * 4;
    *reinterpret_cast<uint2 *>(dst) = o2;
    if (tid == 0)
        p.lse[((int64_t)b * p.nheads + head) * Sq + qi] = (tot > 0.f) ? (mx + fast_log2(tot)) * kLn2 : INFINITY;
}

template <typename T, int D, int RT>
static hipError_t launch_decode_rt(const DecodeParams &p, hipStream_t stream) {
    constexpr int NW = 4;
    dim3 grid(p.nsplits, p.nheads_k, p.batch);
    dim3 block(NW * 64);
    const bool softcap = p.softcap_post != 0.f;
    if (softcap)
        hipLaunchKernelGGL((decode_paged_kernel<T, D, RT, NW, true>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((decode_paged_kernel<T, D, RT, NW, false>), grid, block, 0, stream, p);
    return hipGetLastError();
}

template <typename T, int D> static hipError_t launch_decode_d(const DecodeParams &p, hipStream_t stream) {
    const int rt = (p.rows + 15) / 16;
    if (rt <= 1) return launch_decode_rt<T, D, 1>(p, stream);
    if (rt <= 2) return launch_decode_rt<T, D, 2>(p, stream);
    return launch_decode_rt<T, D, 4>(p, stream);
}

template <typename T> static hipError_t launch_decode_t(const DecodeParams &p, int headdim, hipStream_t stream) {
    switch (headdim) {
        case 64: return launch_decode_d<T, 64>(p, stream);
        case 128: return launch_decode_d<T, 128>(p, stream);
        case 256: return launch_decode_d<T, 256>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_decode_paged(const DecodeParams &p, int dtype, int headdim, hipStream_t stream) {
    return dtype == 0 ? launch_decode_t<BF16>(p, headdim, stream) : launch_decode_t<FP16>(p, headdim, stream);
}

template <typename T> static hipError_t launch_combine_t(const DecodeParams &p, int headdim_v, hipStream_t stream) {
    dim3 grid(p.rows, p.nheads_k, p.batch);
    switch (headdim_v) {
        case 64: hipLaunchKernelGGL((splitkv_combine_kernel<T, 64>), grid, dim3(16), 0, stream, p); break;
        case 128: hipLaunchKernelGGL((splitkv_combine_kernel<T, 128>), grid, dim3(32), 0, stream, p); break;
        case 256: hipLaunchKernelGGL((splitkv_combine_kernel<T, 256>), grid, dim3(64), 0, stream, p); break;
        case 512: hipLaunchKernelGGL((splitkv_combine_kernel<T, 512>), grid, dim3(128), 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_splitkv_combine(const DecodeParams &p, int dtype, int headdim_v, hipStream_t stream) {
    return dtype == 0 ? launch_combine_t<BF16>(p, headdim_v, stream) : launch_combine_t<FP16>(p, headdim_v, stream);
}

}  // namespace fa
