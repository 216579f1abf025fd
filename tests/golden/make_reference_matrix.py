"""Writes the parameter rows of the reference's own forward tests as fixtures, read from the test files' text:

  reference_matrix.json     tests/test_flash_attn_npu_v2.py: kvcache (:145-286), dense forward (:436-459), varlen (:522-560)
  reference_matrix_v3.json  tests/test_flash_attn_npu_v3.py: kvcache (:148-303), dense forward (:545-567), varlen (:622-660)
  reference_matrix_v4.json  tests/test_flash_attn_npu_v4.py: the paged / packed / dense varlen matrix (:220-397)

    python tests/golden/make_reference_matrix.py [/root/reference]

Nothing of the reference is imported or run: the `test_cases = [...]` lists are cut out of the source text and their
tuples parsed as literals (dtype names become strings; rows the reference itself has commented out stay out).  The
rows are data - shapes, layouts, flags and window sizes - and the fixtures hold nothing else."""
import ast
import json
import os
import re
import sys


def rows(text: str, start: int):
    i = text.index("test_cases = [", start)
    j = text.index("\n]", i)
    body = text[i + len("test_cases = "):j + 2]
    body = re.sub(r"torch\.(bfloat16|float16)", r'"\1"', body)
    return [list(t) for t in ast.literal_eval(body)], j


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    text = open(os.path.join(ref, "tests", "test_flash_attn_npu_v2.py")).read()
    kv, end = rows(text, 0)
    dn, end = rows(text, end)
    vl, _ = rows(text, end)
    assert all(len(r) == 13 for r in kv) and all(len(r) == 10 for r in dn) and all(len(r) == 11 for r in vl)
    out = {
        "source": "tests/test_flash_attn_npu_v2.py of MinghuasLab/flash-attention-npu v0.3.0",
        "kvcache_columns": ["dtype", "batch", "heads", "kv_heads", "q_seqlen", "kv_seqlen", "head_size", "paged", "block",
                            "causal", "window_left", "window_right", "softcap"],
        "kvcache": kv,
        "dense_columns": ["dtype", "batch", "heads", "kv_heads", "q_seqlen", "kv_seqlen", "head_size", "return_attn_probs",
                          "causal", "softcap"],
        "dense": dn,
        "varlen_columns": ["dtype", "batch", "heads", "kv_heads", "q_seqlen", "kv_seqlen", "head_size", "causal",
                           "window_left", "window_right", "softcap"],
        "varlen": vl,
    }
    here = os.path.dirname(os.path.abspath(__file__))
    path = os.path.join(here, "reference_matrix.json")
    with open(path, "w") as f:
        f.write("{\n")
        for k in ("source", "kvcache_columns", "dense_columns", "varlen_columns"):
            f.write(f'  "{k}": {json.dumps(out[k])},\n')
        for k in ("kvcache", "dense", "varlen"):
            f.write(f'  "{k}": [\n' + ",\n".join("    " + json.dumps(r) for r in out[k]) + "\n  ]" + (",\n" if k != "varlen" else "\n"))
        f.write("}\n")
    print(path, len(kv), "kvcache rows,", len(dn), "dense rows,", len(vl), "varlen rows")

    text = open(os.path.join(ref, "tests", "test_flash_attn_npu_v3.py")).read()
    kv, end = rows(text, 0)
    dn, end = rows(text, end)
    vl, _ = rows(text, end)
    assert all(len(r) == 14 for r in kv) and all(len(r) == 10 for r in dn) and all(len(r) == 11 for r in vl)
    write(os.path.join(here, "reference_matrix_v3.json"), {
        "source": "tests/test_flash_attn_npu_v3.py of MinghuasLab/flash-attention-npu v0.3.0; every kvcache row runs with "
                  "cache_mode 0 (dense / packed keys) and 1 (pages of 128) and num_splits 0 and 2 (2 only paged + TND), :305-316",
        "kvcache_columns": ["dtype", "batch", "heads", "kv_heads", "q_seqlen", "kv_seqlen", "head_size", "block", "causal",
                            "layout", "is_varied", "window_left", "window_right", "softcap"],
        "dense_columns": ["dtype", "batch", "heads", "kv_heads", "q_seqlen", "kv_seqlen", "head_size", "return_attn_probs",
                          "causal", "softcap"],
        "varlen_columns": ["dtype", "batch", "heads", "kv_heads", "q_seqlen", "kv_seqlen", "head_size", "causal",
                           "window_left", "window_right", "softcap"],
        "kvcache": kv, "dense": dn, "varlen": vl}, ("kvcache", "dense", "varlen"))

    text = open(os.path.join(ref, "tests", "test_flash_attn_npu_v4.py")).read()
    vl, _ = rows(text, 0)
    assert all(len(r) == 14 for r in vl)
    write(os.path.join(here, "reference_matrix_v4.json"), {
        "source": "tests/test_flash_attn_npu_v4.py of MinghuasLab/flash-attention-npu v0.3.0; every row runs with "
                  "num_splits 0, 1 and 2 (2 only paged + TND), :399-406",
        "varlen_columns": ["dtype", "batch", "heads", "kv_heads", "q_seqlen", "kv_seqlen", "head_size", "cache_mode", "block",
                           "causal", "layout", "is_varied", "window_left", "window_right"],
        "varlen": vl}, ("varlen",))


def write(path, out, lists):
    with open(path, "w") as f:
        f.write("{\n")
        for k in out:
            if k not in lists:
                f.write(f'  "{k}": {json.dumps(out[k])},\n')
        for k in lists:
            f.write(f'  "{k}": [\n' + ",\n".join("    " + json.dumps(r) for r in out[k]) + "\n  ]" + (",\n" if k != lists[-1] else "\n"))
        f.write("}\n")
    print(path, ", ".join(f"{len(out[k])} {k} rows" for k in lists))


if __name__ == "__main__":
    main()
