"""Writes tests/golden/tiny-llama-random/golden_ids.json.

The prompt ids come from tokenising "Hello" with the tokenizer.json data file that sits
beside the tiny random Llama checkpoint in the reference tree (a 3.5 MB data file that is not
copied here); encode(prompt, add_special_tokens=False) as crates/llm/src/session.rs:341-345.
The expected new ids are the constants of crates/llm/tests/tinyllama_random.rs:20-24.
Run once in the build container:  python tests/golden/make_prompt_ids.py
"""
import json
import os
import sys

from tokenizers import Tokenizer

src = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/models/hf/tiny-llama-random/tokenizer.json"
tok = Tokenizer.from_file(src)
prompt = "Hello"
ids = tok.encode(prompt, add_special_tokens=False).ids
out = {
    "prompt": prompt,
    "prompt_ids": ids,
    "expected_new_ids": [3038, 25190, 6074, 6566, 21376, 8002, 12090, 28535],
    "stream_sink": 4,
    "stream_window": 28,
}
dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tiny-llama-random", "golden_ids.json")
with open(dst, "w") as f:
    json.dump(out, f, indent=1)
print(out)
