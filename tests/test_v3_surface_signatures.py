"""The flash_attn_npu_3 surface keeps the reference's parameter names, order and defaults
(flash_attn_npu_3/flash_attn_npu_interface.py:828-846, :911-934, :965-996, :1129-1146), so call sites
written against the reference run unchanged.  No GPU needed."""
import inspect

import torch


def names(fn):
    return list(inspect.signature(fn).parameters)


def test_exports_and_signatures():
    import flash_attn_npu_3 as v3
    assert set(v3.__all__) == {"flash_attn_func", "flash_attn_varlen_func", "flash_attn_with_kvcache",
                               "get_scheduler_metadata"}
    assert names(v3.flash_attn_with_kvcache) == [
        "q", "k_cache", "v_cache", "k", "v", "qv", "rotary_cos", "rotary_sin", "cache_seqlens", "cache_batch_idx",
        "cache_leftpad", "page_table", "cu_seqlens_q", "cu_seqlens_k_new", "max_seqlen_q", "rotary_seqlens", "q_descale",
        "k_descale", "v_descale", "softmax_scale", "causal", "window_size", "attention_chunk", "softcap",
        "rotary_interleaved", "scheduler_metadata", "num_splits", "pack_gqa", "sm_margin", "return_softmax_lse"]
    assert names(v3.get_scheduler_metadata) == [
        "batch_size", "max_seqlen_q", "max_seqlen_k", "num_heads_q", "num_heads_kv", "headdim", "cache_seqlens", "qkv_dtype",
        "headdim_v", "cu_seqlens_q", "cu_seqlens_k_new", "cache_leftpad", "page_size", "max_seqlen_k_new", "causal",
        "window_size", "attention_chunk", "has_softcap", "num_splits", "pack_gqa", "sm_margin"]
    assert names(v3.flash_attn_func) == [
        "q", "k", "v", "softmax_scale", "causal", "qv", "q_descale", "k_descale", "v_descale", "window_size",
        "attention_chunk", "softcap", "num_splits", "pack_gqa", "deterministic", "sm_margin", "return_attn_probs",
        "scheduler_metadata"]
    assert names(v3.flash_attn_varlen_func) == [
        "q", "k", "v", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "seqused_q", "seqused_k",
        "softmax_scale", "causal", "qv", "q_descale", "k_descale", "v_descale", "window_size", "attention_chunk", "softcap",
        "num_splits", "pack_gqa", "deterministic", "sm_margin", "return_attn_probs", "scheduler_metadata"]
    d = {k: p.default for k, p in inspect.signature(v3.flash_attn_with_kvcache).parameters.items()}
    assert d["rotary_interleaved"] is True and d["num_splits"] == 0 and d["window_size"] == (-1, -1) and d["softcap"] == 0.0
    d = {k: p.default for k, p in inspect.signature(v3.flash_attn_func).parameters.items()}
    assert d["num_splits"] == 1 and d["causal"] is False
    d = {k: p.default for k, p in inspect.signature(v3.get_scheduler_metadata).parameters.items()}
    assert d["qkv_dtype"] == torch.bfloat16 and d["page_size"] is None and d["num_splits"] == 0


def test_host_checks_need_no_gpu():
    # argument checks that come before any device work raise the reference's messages on any host
    import pytest
    import flash_attn_npu_3 as v3
    q = torch.zeros(1, 1, 4, 128, dtype=torch.bfloat16)
    kc = torch.zeros(1, 128, 2, 128, dtype=torch.bfloat16)
    lens = torch.zeros(1, dtype=torch.int32)
    for kw, msg in [(dict(cache_leftpad=lens), "does not support leftpad_k"), (dict(attention_chunk=2), "attention_chunk"),
                    (dict(pack_gqa=True), "pack_gqa"), (dict(qv=q), "does not support qv"),
                    (dict(softcap=-0.5), "softcap must be non-negative")]:
        with pytest.raises(RuntimeError, match=msg):
            v3.flash_attn_with_kvcache(q, kc, kc, cache_seqlens=lens, **kw)
    with pytest.raises(RuntimeError, match="there is no CPU path"):
        v3.flash_attn_with_kvcache(q, kc, kc, cache_seqlens=lens)
    with pytest.raises(RuntimeError, match="cache_seqlens must have dtype int32"):
        v3.get_scheduler_metadata(1, 1, 128, 4, 2, 128, lens.long())
