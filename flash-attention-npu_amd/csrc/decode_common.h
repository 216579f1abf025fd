// Pieces shared by the decode kernels: the live key range of a (batch row) unit and the balanced
// partition of all units' 32-key chunks over the workgroups of a launch.
//
// The chunks of all (batch row, kv head) units, in (b, kvh) order, form one list of W chunks that
// is cut into gridDim.x equal contiguous shares, one per workgroup, cutting inside a unit where a
// share ends - the reference's flash-decode partition (csrc/ascend910/flash_attn_npu/
// flash_api.cpp:97-354, splitBN2S1GS2) computed by every workgroup for itself from the
// device-resident lengths.  A workgroup writes the final output of every unit that lies wholly
// inside its share and at most two partials.
#pragma once
#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {

constexpr int kChunk = 32;  // keys per wave step

// Live key range [lo, hi) of the query block of batch row b, and its 32-key chunk span.
// M of the window normalisation for a decode launch: the batch maximum of the key counts when a
// window was requested, else irrelevant (1).  Every thread of the workgroup must call.
__device__ __forceinline__ int window_norm_m(const DecodeParams &p) {
    if (p.window_left < 0 && p.window_right < 0) return 1;
    return block_max_keys(p.cache_seqlens, p.batch, p.seqlen_new);
}

// Rows of batch row b's query block that nobody reads (padding in front of the real query tokens): the
// kernels compute them with the others but skip their stores and their merge.
__device__ __forceinline__ int dead_rows(const DecodeParams &p, int b) {
    return (p.q_live && p.row_tiles <= 1) ? max(p.seqlen_q - p.q_live[b], 0) * p.group : 0;
}

struct UnitRange {
    int len_cache, Lk, lo, hi;
    int wl, wr;       // window after normalisation (-1 = unbounded); causal gives wr = 0
    int c0, nchunks;  // first chunk index (absolute) and number of chunks; nchunks == 0: nothing visible
};

__device__ __forceinline__ UnitRange unit_range(const DecodeParams &p, int b, int M) {
    UnitRange u;
    u.len_cache = p.cache_seqlens[b];
    u.Lk = u.len_cache + p.seqlen_new;
    const int off = u.Lk - p.seqlen_q;
    u.wl = p.window_left;
    u.wr = p.window_right;
    normalize_window(u.wl, u.wr, p.causal, M);
    u.lo = 0;
    u.hi = u.Lk;
    if (u.wr >= 0) u.hi = min(u.Lk, p.seqlen_q - 1 + off + u.wr + 1);
    if (u.wl >= 0) u.lo = max(0, off - u.wl);
    // keys the block table cannot address are not read
    u.hi = min(u.hi, p.max_blocks * p.page_size);
    if (u.Lk <= 0 || u.hi <= u.lo) {
        u.lo = u.hi = 0;
        u.c0 = u.nchunks = 0;
    } else {
        u.c0 = u.lo / kChunk;
        u.nchunks = (u.hi + kChunk - 1) / kChunk - u.c0;
    }
    return u;
}

// Length of a unit in the list that the partition cuts: its chunks plus `cost`, the fixed cost of
// starting on a unit (lengths -> table -> keys, q staging, pipeline fill, the stores) in units of one
// chunk's streaming time.  The cost sits at the beginning of the unit's interval, so a worker whose
// share holds the start of a further unit gets that many fewer chunks.  Partition::cost is
// p.piece_cost when the shares are long against it and 0 otherwise: every worker pays for its first
// piece anyway, and with shares of a few chunks charging the unit starts would unbalance them.
__device__ __forceinline__ int unit_cost(int nchunks, int cost) { return nchunks > 0 ? nchunks + cost : 0; }

// exclusive prefixes over 256 equal segments of the batch: s_pref[t] = chunks of rows [0, t*seg),
// s_cnt[t] = rows among them with a visible key; [256] = totals.  All threads of the block must call
// (256 or more threads; the first 256 do the work).  Returns whether some batch row has no visible key.
__device__ __forceinline__ bool batch_chunk_prefix(const DecodeParams &p, int *s_pref, int *s_cnt, int seg, int M) {
    __shared__ int s_wave[4], s_wave_cnt[4];
    const int tid = threadIdx.x;
    int sum = 0, cnt = 0;
    for (int b = tid * seg; b < min(p.batch, (tid + 1) * seg); ++b) {
        const int n = unit_range(p, b, M).nchunks;
        sum += n;
        cnt += (n > 0);
    }
    const bool empty_row = tid * seg < p.batch && cnt < min(p.batch, (tid + 1) * seg) - tid * seg;
    int inc = sum, inc_cnt = cnt;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int v = __shfl_up(inc, d, 64);
        const int vc = __shfl_up(inc_cnt, d, 64);
        if ((tid & 63) >= d) {
            inc += v;
            inc_cnt += vc;
        }
    }
    if ((tid & 63) == 63 && tid < 256) {
        s_wave[tid >> 6] = inc;
        s_wave_cnt[tid >> 6] = inc_cnt;
    }
    const bool any_empty = __syncthreads_or(empty_row ? 1 : 0) != 0;
    if (tid < 256) {
        int base = 0, base_cnt = 0;
        for (int w = 0; w < (tid >> 6); ++w) {
            base += s_wave[w];
            base_cnt += s_wave_cnt[w];
        }
        s_pref[tid + 1] = base + inc;
        s_cnt[tid + 1] = base_cnt + inc_cnt;
    }
    if (tid == 0) s_pref[0] = s_cnt[0] = 0;
    __syncthreads();
    return any_empty;
}

// Query token and query head of row `row` of unit `kvh` of a batch row.  Ordinary caches: the unit
// is a kv head, its rows are (query token, head of the group).  Latent int8 cache
// (p.units_per_token > 0): the unit is (query token, 64-head group) and its rows are heads.  Query blocks cut
// into 16-row tiles (p.row_tiles > 1): the unit is (kv head, tile) and its rows are rows 16 * tile .. of the block;
// rows behind the block's last get head = p.nheads, which every caller treats as "no such row".
struct RowId { int qi, head; };
__device__ __forceinline__ RowId row_id(const DecodeParams &p, int kvh, int row) {
    RowId r;
    if (p.units_per_token > 0) {
        r.qi = kvh / p.units_per_token;
        r.head = (kvh - r.qi * p.units_per_token) * p.group + row;
    } else if (p.row_tiles > 1) {
        const int kv = kvh / p.row_tiles;
        const int full = (kvh - kv * p.row_tiles) * 16 + row;
        r.qi = full / p.group;
        r.head = full < p.rows_total ? kv * p.group + (full - r.qi * p.group) : p.nheads;
        if (full >= p.rows_total) r.qi = 0;
    } else {
        r.qi = row / p.group;
        r.head = kvh * p.group + (row - r.qi * p.group);
    }
    return r;
}

struct UnitPos {
    int b;          // batch row
    int pref;       // list length of the rows before b (one kv head's worth)
};

// batch row whose units contain list position `pos` (0 <= pos < Hk * total)
__device__ __forceinline__ UnitPos locate_row(const DecodeParams &p, const int *s_pref, int seg, int64_t pos, int M,
                                              int list_heads, int cost) {
    const int target = (int)(pos / list_heads);  // rows with pref <= target < pref + n
    int lo = 0, hi = 256;                        // segment t with s_pref[t] <= target < s_pref[t+1]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_pref[mid] <= target) lo = mid; else hi = mid;
    }
    UnitPos u;
    u.b = lo * seg;
    u.pref = s_pref[lo];
    for (;;) {
        const int n = unit_cost(unit_range(p, u.b, M).nchunks, cost);
        if (target < u.pref + n || u.b + 1 >= p.batch) break;
        u.pref += n;
        ++u.b;
    }
    return u;
}


// Where a unit's pieces live: it is cut over shares g_first .. g_first + ns - 1; piece s sits in
// slot 2*worker of its share's worker, except that piece 0 sits in the odd slot when its worker's
// share started in an earlier unit.
struct UnitPieces {
    int ns;
    int64_t g_first;
    bool first_is_late;
    int stride, offset;   // worker of share g: g * stride + offset
    __device__ __forceinline__ int64_t slot(int s) const {
        return ((g_first + s) * stride + offset) * 2 + ((s == 0 && first_is_late) ? 1 : 0);
    }
};

// Split-KV merge of one query row by one wave (CombineScale.hpp:166-194,249-316):
// LSE = M + log sum exp(lse_s - M), out = sum exp(lse_s - LSE) * O_s.  Lanes own DV/64 columns.
template <typename T, int DV, typename SlotFn>
__device__ __forceinline__ void combine_row_wave(const DecodeParams &p, int b, int kvh, int row, int ns, SlotFn slot_of) {
    constexpr int CPL = DV / 64;   // columns per lane (2, 4 or 8)
    static_assert(CPL == 1 || CPL == 2 || CPL == 4 || CPL == 8, "column split");
    if (row_id(p, kvh, row).head >= p.nheads) return;   // a row of the latent kernel's last, partly empty head group
    const int lane = threadIdx.x & 63;
    constexpr bool HALF = partials_are_half(DV);
    constexpr int PB = (CPL >= 8 && !HALF) ? 4 : 8;   // pieces whose rows are in flight together
    float mx = -INFINITY;
    float tot = 0.f;
    float acc[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) acc[c] = 0.f;
    // The pieces of a unit were written by other compute units: every dependent load is a trip to memory.  Rows and
    // log-sum-exps of PB pieces are therefore requested together and only then used; a unit of at most PB pieces (the
    // common case) is merged with a single trip, the maximum taken from the values every lane then holds.
    auto fetch = [&](int s0, float (&lw)[PB], float (&v)[PB][CPL]) {
#pragma unroll
        for (int i = 0; i < PB; ++i) {
            const int64_t srow = slot_of(min(s0 + i, ns - 1)) * p.rows + row;
            lw[i] = (s0 + i < ns) ? p.lse_partial[srow] : -INFINITY;
            const float *src = p.o_partial + srow * DV + lane * CPL;
            if constexpr (HALF) {
                static_assert(!HALF || CPL == 8, "16-bit partial rows are read 16 bytes per lane");
                const u32x4_t t = *reinterpret_cast<const u32x4_t *>(reinterpret_cast<const uint16_t *>(p.o_partial) + srow * DV + lane * CPL);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    v[i][2 * c] = to_float<FP16>((uint16_t)(t[c] & 0xffffu));
                    v[i][2 * c + 1] = to_float<FP16>((uint16_t)(t[c] >> 16));
                }
            } else if constexpr (CPL == 1) {
                v[i][0] = src[0];
            } else if constexpr (CPL == 2) {
                const float2 t = *reinterpret_cast<const float2 *>(src);
                v[i][0] = t.x, v[i][1] = t.y;
            } else {
#pragma unroll
                for (int c = 0; c < CPL; c += 4) {
                    const float4 t = *reinterpret_cast<const float4 *>(src + c);
                    v[i][c] = t.x, v[i][c + 1] = t.y, v[i][c + 2] = t.z, v[i][c + 3] = t.w;
                }
            }
        }
    };
    auto add = [&](const float (&lw)[PB], const float (&v)[PB][CPL], float mx_use) {
#pragma unroll
        for (int i = 0; i < PB; ++i) {
            const float w = fast_exp2(lw[i] - mx_use);   // 0 behind the last piece (-inf)
            tot += w;
#pragma unroll
            for (int c = 0; c < CPL; ++c) acc[c] += w * v[i][c];
        }
    };
    if (ns <= PB) {
        float lw[PB];
        float v[PB][CPL];
        fetch(0, lw, v);
#pragma unroll
        for (int i = 0; i < PB; ++i) mx = fmaxf(mx, lw[i]);
        add(lw, v, (mx == -INFINITY) ? 0.f : mx);
    } else {
        for (int s = lane; s < ns; s += 64) mx = fmaxf(mx, p.lse_partial[slot_of(s) * p.rows + row]);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
        const float mx_use = (mx == -INFINITY) ? 0.f : mx;
        for (int s0 = 0; s0 < ns; s0 += PB) {
            float lw[PB];
            float v[PB][CPL];
            fetch(s0, lw, v);
            add(lw, v, mx_use);
        }
    }
    const float inv = (tot > 0.f) ? 1.f / tot : 0.f;
    const RowId rid = row_id(p, kvh, row);
    const int qi = rid.qi, head = rid.head;
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                    (int64_t)head * p.o_stride_h + lane * CPL;
    if (lane * CPL < p.headdim) {   // the partials are DV wide; the output row ends at the head dimension
        if constexpr (CPL == 1) {
            dst[0] = from_float<T>(acc[0] * inv);
        } else {
#pragma unroll
            for (int c = 0; c < CPL; c += 2) *reinterpret_cast<uint32_t *>(dst + c) = pack2<T>(acc[c] * inv, acc[c + 1] * inv);
        }
    }
    if (lane == 0)
        p.lse[((int64_t)b * p.nheads + head) * p.seqlen_q + qi] = (tot > 0.f) ? (mx + fast_log2(tot)) * kLn2 : INFINITY;
}

// out = 0, lse = +inf for every row of a unit that has no visible key (init_outputs.hpp:58-102)
template <int DV> __device__ __forceinline__ void init_empty_unit(const DecodeParams &p, int b, int kvh) {
    for (int idx = threadIdx.x; idx < p.rows * (DV / 8); idx += blockDim.x) {
        const int row = idx / (DV / 8);
        const int piece = idx - row * (DV / 8);
        const RowId rid = row_id(p, kvh, row);
        const int qi = rid.qi, head = rid.head;
        if (head >= p.nheads || piece * 8 >= p.headdim) continue;
        uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_stride_b + (int64_t)qi * p.o_stride_s +
                        (int64_t)head * p.o_stride_h + piece * 8;
        store16(dst, u32x4_t{0, 0, 0, 0});
        if (piece == 0) p.lse[((int64_t)b * p.nheads + head) * p.seqlen_q + qi] = INFINITY;
    }
}

// The balanced partition of a launch: W chunks in the list, S chunks per worker share.
// Two list orders.  Plain: units (b, kvh) with kvh inner, a share is any contiguous run of the
// whole list.  Head-interleaved (p.head_interleave): the list holds the chunks of ONE kv head
// (they are the same for every head); worker w streams share w / Hk of it for kv head w % Hk, so
// Hk neighbouring workers read the same token range of all heads at the same time - adjacent
// 256-byte pieces of the same cache rows.
struct Partition {
    int M;          // window normalisation key count
    int seg;        // batch rows per prefix segment
    int list_heads; // kv heads inside the list: nheads_k (plain) or 1 (head-interleaved)
    int cost;       // list length charged per unit on top of its chunks (unit_cost)
    int64_t W, S;
    bool any_empty; // some batch row has no visible key
    __device__ __forceinline__ int64_t worker_of(int64_t share, int kvh, int hk) const {
        return list_heads == 1 ? share * hk + kvh : share;
    }
};

// Block-level (256 threads, contains barriers): prefix sums into s_pref[257], share size for
// p.num_workers workers (never below p.min_share chunks).
__device__ __forceinline__ Partition make_partition(const DecodeParams &p, int *s_pref) {
    Partition pt;
    pt.seg = (p.batch + 255) / 256;
    pt.M = window_norm_m(p);
    __shared__ int s_cnt[257];
    pt.any_empty = batch_chunk_prefix(p, s_pref, s_cnt, pt.seg, pt.M);
    pt.list_heads = p.head_interleave ? 1 : p.nheads_k;
    const int64_t shares = p.head_interleave ? max(p.num_workers / p.nheads_k, 1) : p.num_workers;
    const int64_t chunks = (int64_t)s_pref[256] * pt.list_heads;
    pt.cost = (p.piece_cost > 0 && chunks >= 4 * (int64_t)p.piece_cost * shares) ? p.piece_cost : 0;
    if (pt.cost > 0) {   // block-uniform: the prefix becomes one of list lengths
        __syncthreads();
        for (int t = threadIdx.x; t < 257; t += blockDim.x) s_pref[t] += pt.cost * s_cnt[t];
        __syncthreads();
    }
    pt.W = (int64_t)s_pref[256] * pt.list_heads;
    const bool long_units = p.min_share_long > 0 && (int64_t)s_pref[256] >= (int64_t)kLongUnitChunks * max(s_cnt[256], 1) + (int64_t)pt.cost * s_cnt[256];
    pt.S = max((pt.W + shares - 1) / shares, (int64_t)max(long_units ? p.min_share_long : p.min_share, 1));
    return pt;
}

// Workgroup 0 of a decode launch leaves the partition in the workspace: the merge kernel that follows then finds a
// unit's pieces from a handful of values it reads in one trip, instead of loading every length and redoing the
// block-wide prefix pass with its barriers.  Only for batches of one row per prefix segment.
__device__ __forceinline__ void publish_partition(const DecodeParams &p, const Partition &pt, const int *s_pref) {
    if (!p.part_hdr || blockIdx.x != 0 || pt.seg != 1) return;
    for (int t = threadIdx.x; t <= p.batch; t += blockDim.x) p.part_hdr[kPartitionHeaderInts + t] = s_pref[t];
    if (threadIdx.x == 0) {
        p.part_hdr[0] = pt.M;
        p.part_hdr[1] = pt.cost;
        p.part_hdr[2] = (int32_t)(uint32_t)pt.W;
        p.part_hdr[3] = (int32_t)((uint64_t)pt.W >> 32);
        p.part_hdr[4] = (int32_t)(uint32_t)pt.S;
        p.part_hdr[5] = (int32_t)((uint64_t)pt.S >> 32);
    }
}
__device__ __forceinline__ bool partition_published(const DecodeParams &p) { return p.part_hdr && p.batch <= 256; }
// the published partition; *pref_b: chunks of the batch rows before b
__device__ __forceinline__ Partition read_partition(const DecodeParams &p, int b, int *pref_b) {
    const int32_t *h = p.part_hdr;
    Partition pt;
    pt.seg = 1;
    pt.M = h[0];
    pt.cost = h[1];
    pt.W = (int64_t)(((uint64_t)(uint32_t)h[3] << 32) | (uint32_t)h[2]);
    pt.S = (int64_t)(((uint64_t)(uint32_t)h[5] << 32) | (uint32_t)h[4]);
    pt.list_heads = p.head_interleave ? 1 : p.nheads_k;
    pt.any_empty = false;   // not kept: the merge has no use for it
    *pref_b = h[kPartitionHeaderInts + b];
    return pt;
}

// chunks of batch rows before b (one kv head's worth)
__device__ __forceinline__ int chunks_before(const DecodeParams &p, const Partition &pt, const int *s_pref, int b) {
    const int t = b / pt.seg;
    int pref = s_pref[t];
    for (int bb = t * pt.seg; bb < b; ++bb) pref += unit_cost(unit_range(p, bb, pt.M).nchunks, pt.cost);
    return pref;
}

// unit_start: list position of the unit's interval (its piece cost first, then its chunks)
__device__ __forceinline__ UnitPieces unit_pieces(const Partition &pt, int64_t unit_start, int nchunks, int kvh, int hk,
                                                  int piece_cost) {
    UnitPieces pcs;
    const int64_t first_chunk = unit_start + piece_cost;
    pcs.g_first = first_chunk / pt.S;
    pcs.ns = (int)((first_chunk + nchunks - 1) / pt.S - pcs.g_first + 1);
    // the worker of piece 0 had a piece of an earlier unit before it iff its share begins before this unit
    pcs.first_is_late = (pcs.g_first * pt.S < unit_start);
    pcs.stride = (pt.list_heads == 1) ? hk : 1;
    pcs.offset = (pt.list_heads == 1) ? kvh : 0;
    return pcs;
}

// Walks the share of `worker` and calls piece(b, kvh, unit, range_lo, range_hi, whole, slot) for
// every piece in it.  `whole`: the piece is a complete unit (write the final output); otherwise
// the partial goes to slot 2*worker (piece starts the share) or 2*worker + 1.  No barriers inside:
// a worker may be a workgroup or a single wave.
template <typename PieceFn>
__device__ __forceinline__ void walk_share(const DecodeParams &p, const Partition &pt, const int *s_pref, int64_t worker,
                                           PieceFn piece) {
    const bool inter = pt.list_heads == 1;
    const int64_t share = inter ? worker / p.nheads_k : worker;
    const int fixed_kvh = inter ? (int)(worker - share * p.nheads_k) : 0;
    int64_t pos = share * pt.S;
    const int64_t end = min(pt.W, pos + pt.S);
    if (pos >= end) return;
    UnitPos up = locate_row(p, s_pref, pt.seg, pos, pt.M, pt.list_heads, pt.cost);
    UnitRange ur = unit_range(p, up.b, pt.M);
    const int64_t row_start = (int64_t)up.pref * pt.list_heads;   // list position of unit (b, 0)
    int ucost = unit_cost(ur.nchunks, pt.cost);
    int kvh = (int)((pos - row_start) / ucost);
    int cost_off = (int)((pos - row_start) - (int64_t)kvh * ucost);  // offset into the unit's interval
    bool first = true;
    while (pos < end) {
        const int take_cost = (int)min((int64_t)(ucost - cost_off), end - pos);
        // the chunks of the unit that this stretch of its interval holds
        const int off_lo = max(0, cost_off - pt.cost);
        const int off_hi = max(0, cost_off + take_cost - pt.cost);
        if (off_hi > off_lo) {
            const bool whole = (off_lo == 0) && (off_hi == ur.nchunks);
            const int c_lo = ur.c0 + off_lo;
            const int range_lo = max(ur.lo, c_lo * kChunk);
            const int range_hi = min(ur.hi, (ur.c0 + off_hi) * kChunk);
            piece(up.b, inter ? fixed_kvh : kvh, ur, range_lo, range_hi, whole, worker * 2 + (first ? 0 : 1));
            first = false;
        }
        pos += take_cost;
        cost_off = 0;
        if (++kvh == pt.list_heads) {
            kvh = 0;
            do {
                ++up.b;
                if (up.b < p.batch) ur = unit_range(p, up.b, pt.M);
            } while (up.b < p.batch && ur.nchunks == 0);
            if (up.b >= p.batch) break;
            ucost = unit_cost(ur.nchunks, pt.cost);
        }
    }
}

// Units without a visible key belong to no share: workgroup g initialises units g, g + G, ...
template <int DV> __device__ __forceinline__ void init_empty_units(const DecodeParams &p, const Partition &pt) {
    if (!pt.any_empty) return;
    const int units = p.batch * p.nheads_k;
    for (int u = blockIdx.x; u < units; u += gridDim.x) {
        const int b = u / p.nheads_k;
        if (unit_range(p, b, pt.M).nchunks == 0) init_empty_unit<DV>(p, b, u - b * p.nheads_k);
    }
}

// Workgroup-level worker: the share `worker` (a permutation of the workgroup numbers), then the empty-unit duty.
template <int DV, typename PieceFn>
__device__ __forceinline__ void balanced_driver(const DecodeParams &p, int worker, PieceFn piece) {
    __shared__ int s_pref[257];
    const Partition pt = make_partition(p, s_pref);
    publish_partition(p, pt, s_pref);
    walk_share(p, pt, s_pref, worker, piece);
    init_empty_units<DV>(p, pt);
}

}  // namespace fa
