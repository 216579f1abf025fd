// PyTorch extension module `flash_attn_npu._C`: the operator layer in C++.
//
// Takes the place of the reference's pybind module (csrc/ascend910/flash_attn_npu/flash_api.cpp:1330-1338):
// `fwd_kvcache` and `varlen_fwd` with the reference's argument order (:356-377, :848-869) and TORCH_CHECK texts.
// Everything device-side happens behind the C ABI of libfa_rocm.so (include/fa_rocm.h), which this module links:
// here tensors are checked, the plain-C argument record is filled, outputs and the split workspace are taken from
// PyTorch's caching allocator, and the call is enqueued on PyTorch's current stream.  There is no fallback path.
// PyTorch-ROCm names its device type "cuda": the guard and the stream are the ROCm build's own classes for that
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "../../include/fa_rocm.h"

namespace {

using OptTensor = std::optional<at::Tensor>;

int dtype_code(const at::Tensor &t) {
    switch (t.scalar_type()) {
        case at::kBFloat16: return FA_BF16;
        case at::kHalf: return FA_FP16;
        case at::kChar: return FA_INT8;
        default: return -1;
    }
}

// Every tensor of a call lives on one ROCm device: the kernels dereference all of them from the same launch.
void require_device(std::initializer_list<const at::Tensor *> tensors) {
    const at::Tensor *first = nullptr;
    for (const at::Tensor *t : tensors) {
        if (t == nullptr || !t->defined()) continue;
        TORCH_CHECK(t->is_cuda(), "flash_attn_npu (MI355X build) needs tensors on a ROCm device; there is no CPU path");
        if (first == nullptr) first = t;
        TORCH_CHECK(t->device() == first->device(), "all tensors of a call must be on the same device");
    }
}

const at::Tensor *ptr_of(const OptTensor &t) { return t.has_value() ? &t.value() : nullptr; }

void check_rc(int rc) { TORCH_CHECK(rc == FA_OK, fa_rocm_last_error()); }

// Small constant tensors for dense caches called without a table or lengths, one per (kind, device, shape).  The
// first kCachedTables distinct shapes are kept for the life of the process, so a captured HIP graph may hold their
// addresses; past that bound a call gets a fresh tensor of its own, which lives as long as the caller's results do
// (callers that capture such calls pass cache_seqlens / block_table themselves).
constexpr size_t kCachedTables = 256;
at::Tensor cached_table(int kind, const at::Device &dev, int64_t batch, int64_t value) {
    static std::mutex mu;
    static std::map<std::tuple<int, int, int64_t, int64_t>, at::Tensor> cache;
    const auto opts = at::TensorOptions().dtype(at::kInt).device(dev);
    const auto make = [&]() {
        return kind == 0 ? at::arange(batch, opts).view({batch, 1})   // identity block table of a dense cache
                         : at::full({batch}, value, opts);            // every row holds `value` keys
    };
    std::lock_guard<std::mutex> lock(mu);
    const auto key = std::make_tuple(kind, (int)dev.index(), batch, value);
    auto it = cache.find(key);
    if (it != cache.end()) return it->second;
    if (cache.size() >= kCachedTables) return make();
    return cache.emplace(key, make()).first->second;
}

// mha_fwd_kvcache (flash_api.cpp:356-637).  Returns {out, softmax_lse}.
std::vector<at::Tensor> fwd_kvcache(const at::Tensor &q, const at::Tensor &kcache, const at::Tensor &vcache, const OptTensor &k_,
                                    const OptTensor &v_, const OptTensor &seqlens_k_, const OptTensor &rotary_cos_,
                                    const OptTensor &rotary_sin_, const OptTensor &cache_batch_idx_, const OptTensor &leftpad_k_,
                                    const OptTensor &block_table_, const OptTensor &alibi_slopes_, const OptTensor &out_,
                                    double softmax_scale, bool is_causal, int64_t window_size_left, int64_t window_size_right,
                                    double softcap, bool is_rotary_interleaved, int64_t num_splits, const OptTensor &k_scale_cache_,
                                    const OptTensor &v_scale_cache_) {
    const bool is_i8 = kcache.scalar_type() == at::kChar;
    TORCH_CHECK(q.scalar_type() == at::kBFloat16 || q.scalar_type() == at::kHalf,
                "FlashAttention only supports FP16 and BF16 data types");
    if (!is_i8) {
        TORCH_CHECK(kcache.scalar_type() == q.scalar_type(), "query and key_cache must have the same dtype");
        TORCH_CHECK(vcache.scalar_type() == q.scalar_type(), "query and value_cache must have the same dtype");
    } else {
        TORCH_CHECK(vcache.scalar_type() == at::kChar, "key_cache and value_cache must have the same dtype");
        TORCH_CHECK(k_scale_cache_.has_value(), "int8 KV cache needs k_scale_cache");
    }
    TORCH_CHECK(q.dim() == 4 && kcache.dim() == 4 && vcache.dim() == 4, "q, kcache and vcache must be 4-D");
    TORCH_CHECK(q.stride(-1) == 1, "Input tensor q must have contiguous last dimension");
    TORCH_CHECK(kcache.stride(-1) == 1, "Input tensor kcache must have contiguous last dimension");
    TORCH_CHECK(vcache.stride(-1) == 1, "Input tensor vcache must have contiguous last dimension");
    // A dense cache (batch_cache, seqlen_cache, nheads_k, headdim) is a paged one with a single page per row: the
    // table is the identity, or cache_batch_idx (flash_attn_npu_interface.py:1516-1519).
    at::Tensor block_table, seqlens_k;
    if (!block_table_.has_value()) {
        if (cache_batch_idx_.has_value()) {
            const at::Tensor &idx = cache_batch_idx_.value();
            TORCH_CHECK(idx.scalar_type() == at::kInt && idx.dim() == 1 && idx.size(0) == q.size(0),
                        "cache_batch_idx must be (batch_size,) int32");
            block_table = idx.contiguous().view({-1, 1});
        } else {
            TORCH_CHECK(kcache.size(0) >= q.size(0), "batch size of the cache must be at least that of q");
            require_device({&q});
            block_table = cached_table(0, q.device(), q.size(0), 0);
        }
        if (!seqlens_k_.has_value()) {
            TORCH_CHECK(!k_.has_value(), "cache_seqlens must be given to append k / v");
            require_device({&q});
            seqlens_k = cached_table(1, q.device(), q.size(0), kcache.size(1));
        }
    } else {
        TORCH_CHECK(!cache_batch_idx_.has_value(), "Paged KVcache does not support cache_batch_idx");
        block_table = block_table_.value();
    }
    TORCH_CHECK(block_table.scalar_type() == at::kInt, "block_table must have dtype int32");
    TORCH_CHECK(block_table.dim() == 2, "block_table must be (batch_size, max_num_blocks_per_seq)");
    TORCH_CHECK(block_table.stride(-1) == 1, "block_table must have contiguous last dimension");
    if (!seqlens_k.defined()) {
        TORCH_CHECK(seqlens_k_.has_value(), "cache_seqlens must be given with a paged KV cache");
        seqlens_k = seqlens_k_.value();
    }
    TORCH_CHECK(seqlens_k.scalar_type() == at::kInt, "seqlens_k must have dtype int32");
    TORCH_CHECK(seqlens_k.dim() == 1, "seqlens_k must be (batch_size,)");
    TORCH_CHECK(!alibi_slopes_.has_value(), "NPU FlashAttention does not support alibi_slopes");
    TORCH_CHECK(!leftpad_k_.has_value(), "NPU FlashAttention does not support leftpad_k");
    TORCH_CHECK(softcap >= 0.0, "softcap must be non-negative (0.0 disables softcap)");
    // the rotation is part of the append (positions cache_seqlens .. + seqlen_new of q and k); without new tokens the
    // tables would be silently unused
    TORCH_CHECK(k_.has_value() || v_.has_value() || (!rotary_cos_.has_value() && !rotary_sin_.has_value()),
                "rotary_cos / rotary_sin are only applied together with new k / v");

    const int64_t B = q.size(0), sq = q.size(1), hq = q.size(2), d = q.size(3);
    const int64_t num_blocks = kcache.size(0), page = kcache.size(1), hk = kcache.size(2), dk = kcache.size(3);
    const int64_t dv = vcache.size(3);
    TORCH_CHECK(B > 0, "batch size must be positive");
    TORCH_CHECK(d == dk, "q and kcache must have the same head dimension");
    // the kernels index both caches (and the scale caches) with the page ids, rows and heads of kcache
    TORCH_CHECK(vcache.size(0) == num_blocks && vcache.size(1) == page && vcache.size(2) == hk,
                "vcache must have the num_blocks, page_block_size and nheads_k of kcache");
    TORCH_CHECK(hq % hk == 0, "Number of heads in key/value must divide number of heads in query");
    TORCH_CHECK(block_table.size(0) == B && seqlens_k.size(0) == B, "block_table / cache_seqlens batch mismatch");
    if (k_scale_cache_.has_value()) {
        const at::Tensor &ks = k_scale_cache_.value();
        TORCH_CHECK(ks.scalar_type() == at::kFloat && ks.dim() == 3 && ks.stride(-1) == 1 && ks.size(0) == num_blocks &&
                        ks.size(1) == page && ks.size(2) == hk,
                    "k_scale_cache must be fp32 (num_blocks, page_block_size, nheads_k)");
        if (v_scale_cache_.has_value()) {
            const at::Tensor &vs = v_scale_cache_.value();
            TORCH_CHECK(vs.scalar_type() == at::kFloat && vs.sizes() == ks.sizes() && vs.strides() == ks.strides(),
                        "v_scale_cache must match k_scale_cache's layout");
        }
    }
    require_device({&q, &kcache, &vcache, ptr_of(k_), ptr_of(v_), &seqlens_k, &block_table, ptr_of(rotary_cos_), ptr_of(rotary_sin_),
                    ptr_of(out_), ptr_of(k_scale_cache_), ptr_of(v_scale_cache_)});
    seqlens_k = seqlens_k.contiguous();

    const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    at::Tensor out;
    if (out_.has_value()) {
        out = out_.value();
        TORCH_CHECK(out.scalar_type() == q.scalar_type() && out.dim() == 4 && out.size(0) == B && out.size(1) == sq && out.size(2) == hq &&
                        out.size(3) == dv && out.stride(-1) == 1,
                    "out must have shape (batch_size, seqlen_q, num_heads, head_size_v) and the dtype of q");
    } else {
        out = at::empty({B, sq, hq, dv}, q.options());
    }
    at::Tensor lse = at::empty({B, hq, sq}, q.options().dtype(at::kFloat));

    fa_kvcache_args a = {};
    a.q = q.data_ptr();
    a.out = out.data_ptr();
    a.softmax_lse = lse.data_ptr<float>();
    a.k_cache = kcache.data_ptr();
    a.v_cache = vcache.data_ptr();
    a.cache_seqlens = seqlens_k.data_ptr<int32_t>();
    a.block_table = block_table.data_ptr<int32_t>();
    a.batch = (int32_t)B, a.seqlen_q = (int32_t)sq, a.nheads = (int32_t)hq, a.nheads_k = (int32_t)hk;
    a.headdim_qk = (int32_t)d, a.headdim_v = (int32_t)dv;
    a.num_blocks = (int32_t)num_blocks, a.page_size = (int32_t)page, a.max_blocks_per_seq = (int32_t)block_table.size(1);
    a.q_stride_b = q.stride(0), a.q_stride_s = q.stride(1), a.q_stride_h = q.stride(2);
    a.o_stride_b = out.stride(0), a.o_stride_s = out.stride(1), a.o_stride_h = out.stride(2);
    a.k_stride_block = kcache.stride(0), a.k_stride_row = kcache.stride(1), a.k_stride_h = kcache.stride(2);
    a.v_stride_block = vcache.stride(0), a.v_stride_row = vcache.stride(1), a.v_stride_h = vcache.stride(2);
    a.bt_stride_b = block_table.stride(0);
    if (k_scale_cache_.has_value()) {
        const at::Tensor &ks = k_scale_cache_.value();
        a.k_scale_cache = ks.data_ptr<float>();
        a.ks_stride_block = ks.stride(0), a.ks_stride_row = ks.stride(1);
        if (v_scale_cache_.has_value()) a.v_scale_cache = v_scale_cache_->data_ptr<float>();
    }
    at::Tensor k, v, rc, rs;   // kept alive until the call is enqueued
    if (k_.has_value() || v_.has_value()) {
        TORCH_CHECK(k_.has_value() && v_.has_value(), "k and v must be passed together");
        k = k_.value(), v = v_.value();
        TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "Key and value must have the same dtype as query");
        TORCH_CHECK(k.dim() == 4 && k.size(0) == B && k.size(2) == hk && k.size(3) == d && v.dim() == 4 && v.size(0) == B &&
                        v.size(1) == k.size(1) && v.size(2) == hk && v.size(3) == dv,
                    "k / v must be (batch_size, seqlen_new, nheads_k, headdim)");
        if (is_i8) {
            // quantising append: the new latent rows come in the I/O dtype, v aliased like the cache
            TORCH_CHECK(k.stride(-1) == 1 && v.data_ptr() == k.data_ptr() && v.strides() == k.strides(),
                        "int8 KV cache: v must be the view k[..., :512] of the new latent rows");
            TORCH_CHECK(!rotary_cos_.has_value() && !rotary_sin_.has_value(), "rotary embedding is not supported with an int8 KV cache");
        }
        if (k.stride(-1) != 1) k = k.contiguous();
        if (v.stride(-1) != 1) v = v.contiguous();
        a.k_new = k.data_ptr(), a.v_new = v.data_ptr(), a.seqlen_new = (int32_t)k.size(1);
        a.kn_stride_b = k.stride(0), a.kn_stride_s = k.stride(1), a.kn_stride_h = k.stride(2);
        a.vn_stride_b = v.stride(0), a.vn_stride_s = v.stride(1), a.vn_stride_h = v.stride(2);
        if (rotary_cos_.has_value() || rotary_sin_.has_value()) {
            TORCH_CHECK(rotary_cos_.has_value() && rotary_sin_.has_value(), "rotary_cos and rotary_sin must be passed together");
            TORCH_CHECK(rotary_cos_->scalar_type() == q.scalar_type() && rotary_sin_->scalar_type() == q.scalar_type(),
                        "rotary_cos / rotary_sin must have the same dtype as query");
            TORCH_CHECK(rotary_cos_->dim() == 2 && rotary_cos_->sizes() == rotary_sin_->sizes(),
                        "rotary_cos / rotary_sin must be (seqlen_ro, rotary_dim / 2)");
            rc = rotary_cos_->contiguous(), rs = rotary_sin_->contiguous();
            a.rotary_cos = rc.data_ptr(), a.rotary_sin = rs.data_ptr();
            a.seqlen_ro = (int32_t)rc.size(0), a.rotary_dim = (int32_t)(2 * rc.size(1));
            TORCH_CHECK(a.rotary_dim <= d, "rotary_dim must be <= headdim");
            TORCH_CHECK(a.rotary_dim % 16 == 0, "Only rotary dimensions divisible by 16 are currently supported");
        }
    }
    a.io_dtype = dtype_code(q);
    a.kv_dtype = dtype_code(kcache);
    a.softmax_scale = (float)softmax_scale, a.softcap = (float)softcap;
    a.causal = is_causal ? 1 : 0;
    a.window_left = (int32_t)window_size_left, a.window_right = (int32_t)window_size_right;
    a.rotary_interleaved = is_rotary_interleaved ? 1 : 0;
    a.num_splits = (int32_t)num_splits;

    fa_split_plan plan;
    check_rc(fa_rocm_plan_kvcache(&a, fa_rocm_num_cus(), &plan));   // validates as well
    at::Tensor ws;
    if (plan.workspace_bytes > 0) {
        ws = at::empty({(int64_t)((plan.workspace_bytes + 3) / 4)}, q.options().dtype(at::kFloat));
        a.workspace = ws.data_ptr(), a.workspace_bytes = (size_t)ws.numel() * 4;
    }
    // the caching allocator reuses ws only for work enqueued later on this same stream, so it may go out of scope here
    check_rc(fa_rocm_fwd_kvcache(&a, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream()));
    return {out, lse};
}

// mha_varlen_fwd (flash_api.cpp:848-1089), its 21 arguments in its order: the last of them is the random generator
// (flash_api.cpp:868; unused without dropout, callers pass None).  Returns {out, softmax_lse (Hq, total_q), p,
// rng_state}.  num_splits is a trailing extra with a default (paged K/V only; not an argument of the reference's
// function): 0 cuts every sequence's keys into as many ranges as it takes to fill the device when the query tiles
// alone cannot, 1 never, n at most n.
std::vector<at::Tensor> varlen_fwd(const at::Tensor &q, const at::Tensor &k, const at::Tensor &v, const OptTensor &out_,
                                   const at::Tensor &cu_seqlens_q, const OptTensor &cu_seqlens_k, const OptTensor &seqused_k_,
                                   const OptTensor &leftpad_k_, const OptTensor &block_table_, const OptTensor &alibi_slopes_,
                                   int64_t max_seqlen_q, int64_t max_seqlen_k, double p_dropout, double softmax_scale, bool zero_tensors,
                                   bool is_causal, int64_t window_size_left, int64_t window_size_right, double softcap,
                                   bool return_softmax, const std::optional<at::Generator> &gen_, int64_t num_splits) {
    (void)gen_;
    TORCH_CHECK(q.scalar_type() == at::kBFloat16 || q.scalar_type() == at::kHalf,
                "FlashAttention only supports FP16 and BF16 data types");
    TORCH_CHECK(k.scalar_type() == q.scalar_type(), "query and key must have the same dtype");
    TORCH_CHECK(v.scalar_type() == q.scalar_type(), "query and value must have the same dtype");
    TORCH_CHECK(cu_seqlens_q.scalar_type() == at::kInt, "cu_seqlens_q must have dtype int32");
    TORCH_CHECK(q.dim() == 3, "q must be (total_q, nheads, headdim)");
    TORCH_CHECK(q.stride(-1) == 1 && k.stride(-1) == 1 && v.stride(-1) == 1, "Input tensor must have contiguous last dimension");
    TORCH_CHECK(!leftpad_k_.has_value(), "NPU FlashAttention does not support leftpad_k");
    TORCH_CHECK(!alibi_slopes_.has_value(), "NPU FlashAttention does not support alibi_slopes");
    TORCH_CHECK(p_dropout == 0.0, "NPU FlashAttention does not support dropout");
    TORCH_CHECK(!return_softmax, "NPU FlashAttention does not support return_softmax");
    TORCH_CHECK(softcap >= 0.0, "softcap must be non-negative (0.0 disables softcap)");
    // flash_api.cpp:890 (the outputs are written in full either way, nothing is left to clear)
    TORCH_CHECK(!zero_tensors, "NPU FlashAttention does not support zero_tensors.");
    const bool paged = block_table_.has_value();
    // flash_api.cpp:886 rejects seqused_k always (the Python layer of that generation keeps doing so for packed keys);
    // here it is the length array of paged K/V, and with packed keys the number of keys used of each sequence
    // (flash_attn_npu_3/flash_api.cpp:143-147)
    const int64_t total_q = q.size(0), hq = q.size(1), d = q.size(2);
    const int64_t B = cu_seqlens_q.numel() - 1;
    TORCH_CHECK(B > 0, "batch size must be positive");

    fa_varlen_args a = {};
    at::Tensor seqused_k, cu_k;
    int64_t hk;
    if (paged) {
        const at::Tensor &bt = block_table_.value();
        TORCH_CHECK(bt.scalar_type() == at::kInt, "block_table must have dtype int32");
        TORCH_CHECK(bt.dim() == 2 && bt.size(0) == B, "block_table must be (batch_size, max_num_blocks_per_seq)");
        TORCH_CHECK(bt.stride(-1) == 1, "block_table must have contiguous last dimension");
        TORCH_CHECK(k.dim() == 4 && v.dim() == 4, "paged k / v must be (num_blocks, page_block_size, nheads_k, headdim)");
        TORCH_CHECK(v.size(0) == k.size(0) && v.size(1) == k.size(1) && v.size(2) == k.size(2),
                    "paged v must have the num_blocks, page_block_size and nheads_k of k");
        if (seqused_k_.has_value()) {
            seqused_k = seqused_k_.value();
        } else {
            TORCH_CHECK(cu_seqlens_k.has_value(), "paged K/V needs seqused_k or cu_seqlens_k");
            seqused_k = (cu_seqlens_k->slice(0, 1) - cu_seqlens_k->slice(0, 0, -1)).to(at::kInt);
        }
        TORCH_CHECK(seqused_k.scalar_type() == at::kInt, "seqused_k must have dtype int32");
        TORCH_CHECK(seqused_k.dim() == 1 && seqused_k.size(0) == B, "seqused_k must be (batch_size,)");
        seqused_k = seqused_k.contiguous();
        hk = k.size(2);
        a.page_size = (int32_t)k.size(1), a.max_blocks_per_seq = (int32_t)bt.size(1), a.num_blocks = (int32_t)k.size(0);
        a.k_stride_block = k.stride(0), a.k_stride_t = k.stride(1), a.k_stride_h = k.stride(2);
        a.v_stride_block = v.stride(0), a.v_stride_t = v.stride(1), a.v_stride_h = v.stride(2);
        a.block_table = bt.data_ptr<int32_t>(), a.seqused_k = seqused_k.data_ptr<int32_t>(), a.bt_stride_b = bt.stride(0);
    } else {
        TORCH_CHECK(cu_seqlens_k.has_value() && cu_seqlens_k->scalar_type() == at::kInt, "cu_seqlens_k must have dtype int32");
        TORCH_CHECK(k.dim() == 3 && v.dim() == 3, "k / v must be (total_k, nheads_k, headdim)");
        TORCH_CHECK(v.size(0) == k.size(0) && v.size(1) == k.size(1), "v must have the total_k and nheads_k of k");
        TORCH_CHECK(cu_seqlens_k->numel() == B + 1, "cu_seqlens_k must have batch_size + 1 entries");
        if (seqused_k_.has_value()) {
            seqused_k = seqused_k_.value();
            TORCH_CHECK(seqused_k.scalar_type() == at::kInt, "seqused_k must have dtype int32");
            TORCH_CHECK(seqused_k.dim() == 1 && seqused_k.size(0) == B, "seqused_k must be (batch_size,)");
            seqused_k = seqused_k.contiguous();
            a.seqused_k = seqused_k.data_ptr<int32_t>();
        }
        hk = k.size(1);
        a.k_stride_t = k.stride(0), a.k_stride_h = k.stride(1);
        a.v_stride_t = v.stride(0), a.v_stride_h = v.stride(1);
    }
    TORCH_CHECK(k.size(-1) == d && v.size(-1) == d, "q, k and v must have the same head dimension");
    TORCH_CHECK(d <= 256, "FlashAttention only supports head dimension at most 256");
    TORCH_CHECK(hq % hk == 0, "Number of heads in key/value must divide number of heads in query");
    require_device({&q, &k, &v, &cu_seqlens_q, ptr_of(cu_seqlens_k), ptr_of(seqused_k_), ptr_of(block_table_), ptr_of(out_)});
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    const at::Tensor cu_q = cu_seqlens_q.contiguous();
    if (cu_seqlens_k.has_value()) cu_k = cu_seqlens_k->contiguous();
    at::Tensor out;
    if (out_.has_value()) {
        out = out_.value();
        TORCH_CHECK(out.scalar_type() == q.scalar_type() && out.sizes() == q.sizes() && out.stride(-1) == 1, "out must match q");
    } else {
        out = at::empty({total_q, hq, d}, q.options());
    }
    at::Tensor lse = at::empty({hq, total_q}, q.options().dtype(at::kFloat));
    a.q = q.data_ptr(), a.k = k.data_ptr(), a.v = v.data_ptr(), a.out = out.data_ptr(), a.softmax_lse = lse.data_ptr<float>();
    a.cu_seqlens_q = cu_q.data_ptr<int32_t>();
    a.cu_seqlens_k = cu_k.defined() ? cu_k.data_ptr<int32_t>() : nullptr;
    a.batch = (int32_t)B, a.total_q = (int32_t)total_q, a.nheads = (int32_t)hq, a.nheads_k = (int32_t)hk, a.headdim = (int32_t)d;
    a.max_seqlen_q = (int32_t)max_seqlen_q, a.max_seqlen_k = (int32_t)max_seqlen_k;
    a.q_stride_t = q.stride(0), a.q_stride_h = q.stride(1);
    a.o_stride_t = out.stride(0), a.o_stride_h = out.stride(1);
    a.io_dtype = dtype_code(q);
    a.softmax_scale = (float)softmax_scale, a.softcap = (float)softcap;
    a.causal = is_causal ? 1 : 0;
    a.window_left = (int32_t)window_size_left, a.window_right = (int32_t)window_size_right;
    TORCH_CHECK(num_splits >= 0, "num_splits must be non-negative");
    a.num_splits = (int32_t)num_splits;
    if (total_q > 0) {
        const size_t need = fa_rocm_varlen_workspace_bytes(&a, fa_rocm_num_cus());
        at::Tensor ws;
        if (need > 0) {
            ws = at::empty({(int64_t)((need + 3) / 4)}, q.options().dtype(at::kFloat));
            a.workspace = ws.data_ptr(), a.workspace_bytes = (size_t)ws.numel() * 4;
        }
        check_rc(fa_rocm_varlen_fwd(&a, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream()));
    }   // no query tokens: nothing to compute (and empty tensors have no address to validate)
    at::Tensor p = at::empty({0}, q.options());
    at::Tensor rng_state = at::empty({2}, q.options().dtype(at::kLong));
    return {out, lse, p, rng_state};
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "flash_attn_npu on MI355X: operator layer over libfa_rocm.so";
    namespace py = pybind11;
    // the reference's 20 arguments (flash_api.cpp:356-377), then the scale caches of an int8 cache as optional extras
    m.def("fwd_kvcache", &fwd_kvcache, "Forward pass, with KV-cache (paged, optional in-place append)", py::arg("q"), py::arg("kcache"),
          py::arg("vcache"), py::arg("k"), py::arg("v"), py::arg("seqlens_k"), py::arg("rotary_cos"), py::arg("rotary_sin"),
          py::arg("cache_batch_idx"), py::arg("leftpad_k"), py::arg("block_table"), py::arg("alibi_slopes"), py::arg("out"),
          py::arg("softmax_scale"), py::arg("is_causal"), py::arg("window_size_left"), py::arg("window_size_right"), py::arg("softcap"),
          py::arg("is_rotary_interleaved"), py::arg("num_splits"), py::arg("k_scale_cache") = py::none(),
          py::arg("v_scale_cache") = py::none());
    m.def("varlen_fwd", &varlen_fwd, "Forward pass (variable length)", py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out"),
          py::arg("cu_seqlens_q"), py::arg("cu_seqlens_k"), py::arg("seqused_k"), py::arg("leftpad_k"), py::arg("block_table"),
          py::arg("alibi_slopes"), py::arg("max_seqlen_q"), py::arg("max_seqlen_k"), py::arg("p_dropout"), py::arg("softmax_scale"),
          py::arg("zero_tensors"), py::arg("is_causal"), py::arg("window_size_left"), py::arg("window_size_right"), py::arg("softcap"),
          py::arg("return_softmax"), py::arg("gen") = py::none(), py::arg("num_splits") = 0);
    m.def("abi_version", []() { return fa_rocm_abi_version(); });
}
