"""Writes tests/golden/reference_matrix.json: the parameter rows of the reference's own kvcache and varlen
forward tests and of its dense forward test (tests/test_flash_attn_npu_v2.py:145-286, :522-560 and :436-459), read
from the file's text.

    python tests/golden/make_reference_matrix.py [/root/reference]

Nothing of the reference is imported or run: the three `test_cases = [...]` lists are cut out of the source text
and their tuples parsed as literals (dtype names become strings).  The rows are data - shapes, flags and window
sizes - and the fixture holds nothing else."""
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
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_matrix.json")
    with open(path, "w") as f:
        f.write("{\n")
        for k in ("source", "kvcache_columns", "dense_columns", "varlen_columns"):
            f.write(f'  "{k}": {json.dumps(out[k])},\n')
        for k in ("kvcache", "dense", "varlen"):
            f.write(f'  "{k}": [\n' + ",\n".join("    " + json.dumps(r) for r in out[k]) + "\n  ]" + (",\n" if k != "varlen" else "\n"))
        f.write("}\n")
    print(path, len(kv), "kvcache rows,", len(dn), "dense rows,", len(vl), "varlen rows")


if __name__ == "__main__":
    main()
