"""Writes tokenizer_expected.json: ids and vocabulary strings for the reference's two test prompts, computed by
the ORACLE's restatement of Tokenizer::bpe_encode (oracle/oracle.c), never by the product's encoder."""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle import oracle_lib  # noqa: E402

PROMPTS = [  # tests/test_tokenizer.py:14-16 of the reference
    "The climate change need to be properly addressed through the",
    "Please give me 200 words about deep learning.",
]
oracle_lib.build()
t = oracle_lib.Tokenizer.from_file(os.path.join(HERE, "tokenizer.bin"))
out = []
for p in PROMPTS:
    ids = t.bpe_encode(" " + p.strip())
    out.append({"prompt": p, "ids": ids, "pieces": [t.vocab[i].decode("utf-8") for i in ids]})
with open(os.path.join(HERE, "tokenizer_expected.json"), "w") as f:
    json.dump(out, f, indent=1, ensure_ascii=False)
print(json.dumps(out, ensure_ascii=False))
