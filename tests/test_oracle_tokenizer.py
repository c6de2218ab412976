"""Pins the oracle's tokenizer (or_str_lookup, or_bpe_encode: src/util.rs:29-37, src/tokenizer.rs:46-108) and
then holds the product's l2_tokenizer_encode to it.  No GPU needed: the tokenizer is host code on both sides.

What pins the oracle:
  * a toy vocabulary whose merge order is worked out by hand (best score first, leftmost on equal scores, the
    merged pair's own score decides and not the parts'), and the ids-from-260-first lookup rule on a vocabulary
    that holds one string twice;
  * the SentencePiece library's BPE encoder over the same vocabulary: the reference's own test
    (tests/test_tokenizer.py:8-23) asserts that bpe_encode(" " + prompt) equals the Hugging Face Llama tokenizer's
    ids, which is SentencePiece BPE over this vocabulary.  The model is built here from tokenizer.bin itself
    (pieces and scores as they stand, spaces written as U+2581, byte pieces named <0xNN>, dummy prefix on), so
    nothing is fetched.  Compared on the reference's two prompts and on seeded ordinary text (words drawn from
    the vocabulary's own pieces, digits, punctuation, accented and CJK characters, single spaces).
"""
import json
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(ROOT, "tests", "golden")
PROMPTS = [  # tests/test_tokenizer.py:14-16 of the reference
    "The climate change need to be properly addressed through the",
    "Please give me 200 words about deep learning.",
]


@pytest.fixture(scope="module")
def otok(oracle):
    return oracle.Tokenizer.from_file(os.path.join(GOLD, "tokenizer.bin"))


def sentencepiece_model(vocab, scores):
    spm = pytest.importorskip("sentencepiece")
    from sentencepiece import sentencepiece_model_pb2 as pb
    m = pb.ModelProto()
    for i, (v, s) in enumerate(zip(vocab, scores)):
        p = m.pieces.add()
        p.score = float(s)
        if i == 0:
            p.piece, p.type = "<unk>", pb.ModelProto.SentencePiece.UNKNOWN
        elif i in (1, 2):
            p.piece, p.type = ("<s>", "</s>")[i - 1], pb.ModelProto.SentencePiece.CONTROL
        elif i < 259:
            p.piece, p.type = "<0x%02X>" % (i - 3), pb.ModelProto.SentencePiece.BYTE
        else:
            p.piece, p.type = v.decode("utf-8").replace(" ", "▁"), pb.ModelProto.SentencePiece.NORMAL
    m.trainer_spec.model_type = pb.TrainerSpec.BPE
    m.trainer_spec.byte_fallback = True
    m.trainer_spec.unk_id, m.trainer_spec.bos_id, m.trainer_spec.eos_id, m.trainer_spec.pad_id = 0, 1, 2, -1
    m.normalizer_spec.name = "identity"
    m.normalizer_spec.add_dummy_prefix = True
    m.normalizer_spec.remove_extra_whitespaces = False
    m.normalizer_spec.escape_whitespaces = True
    return spm.SentencePieceProcessor(model_proto=m.SerializeToString())


def seeded_texts(vocab, n, seed):
    """Ordinary text: words are vocabulary pieces that start with a space and hold letters only (any script),
    mixed with numbers and punctuation, joined without doubling spaces."""
    rng = np.random.default_rng(seed)
    words = [v.decode("utf-8") for v in vocab[260:] if v[:1] == b" " and len(v) > 1 and v[1:].decode("utf-8").isalpha()]
    tails = [v.decode("utf-8") for v in vocab[260:] if v[:1] != b" " and v.decode("utf-8").isalpha()]
    punct = [",", ".", "!", "?", ";", ":", "-", "'", "(", ")", '"']
    out = []
    for _ in range(n):
        parts = []
        for _ in range(int(rng.integers(2, 9))):
            r = rng.random()
            if r < 0.6:
                parts.append(words[int(rng.integers(len(words)))])
            elif r < 0.75:
                parts.append(words[int(rng.integers(len(words)))] + tails[int(rng.integers(len(tails)))])
            elif r < 0.9:
                parts.append(" " + str(int(rng.integers(0, 100000))))
            else:
                parts.append(punct[int(rng.integers(len(punct)))])
        text = "".join(parts).strip()
        if text:
            out.append(text)
    return out


def test_toy_vocabulary_merge_order_by_hand(oracle):
    # ids 0..259 are fillers that never match (the lookup prefers ids from 260 on)
    vocab = [b"\xff%d" % i for i in range(260)]
    scores = [0.0] * 260
    toy = [(b"a", -1.0), (b"b", -1.0), (b"c", -1.0), (b"ab", -5.0), (b"bc", -3.0), (b"abc", -2.0), (b"ca", -3.0),
           (b"d", -1.0), (b"dd", -4.0), (b"bca", -9.0), (b"cab", -1.5), (b"e", 0.0)]
    for v, s in toy:
        vocab.append(v)
        scores.append(s)
    t = oracle.Tokenizer(vocab, scores)
    ID = {v: 260 + i for i, (v, _) in enumerate(toy)}
    # "abc": pairs ab (-5) and bc (-3): bc wins; then a+bc = abc (-2) merges.
    assert t.bpe_encode("abc") == [ID[b"abc"]]
    # "abca": ab -5, bc -3, ca -3 -> bc (leftmost of the two -3, strict '>'); then a+bc=abc -2, bc+a=bca -9 -> abc;
    # then abc+a: not in the vocabulary.
    assert t.bpe_encode("abca") == [ID[b"abc"], ID[b"a"]]
    # "cab": ca -3, ab -5 -> ca; ca+b = cab -1.5 merges.
    assert t.bpe_encode("cab") == [ID[b"cab"]]
    # "ddd": dd at 0 and at 1 score alike: the leftmost merges; dd+d is no entry.
    assert t.bpe_encode("ddd") == [ID[b"dd"], ID[b"d"]]
    # "ae": no pair in the vocabulary
    assert t.bpe_encode("ae") == [ID[b"a"], ID[b"e"]]
    # a character outside the vocabulary is the reference's expect("not good")
    with pytest.raises(ValueError):
        t.bpe_encode("az")
    with pytest.raises(ValueError):
        t.bpe_encode("")


def test_lookup_prefers_ids_from_260(oracle):
    vocab = [b"x%d" % i for i in range(300)]
    vocab[7] = b"dup"
    vocab[100] = b"low"
    vocab[270] = b"dup"
    vocab[280] = b"dup"
    t = oracle.Tokenizer(vocab, np.zeros(300, np.float32))
    assert t.str_lookup("dup") == 270      # first match at or after 260, not 7, not 280
    assert t.str_lookup("low") == 100      # only below 260: found by the second scan
    assert t.str_lookup("nope") == -1
    short = oracle.Tokenizer([b"a", b"b", b"a"], [0.0, 0.0, 0.0])   # fewer than 260 entries: skip(260) is empty
    assert short.str_lookup("a") == 0


def test_oracle_equals_sentencepiece_on_the_reference_prompts_and_seeded_text(oracle, otok):
    vocab, scores, max_len = oracle.read_tokenizer_file(os.path.join(GOLD, "tokenizer.bin"), 32000)
    assert max_len == 27 and len(vocab) == 32000
    sp = sentencepiece_model(vocab, scores)
    for p in PROMPTS:   # as the reference's test calls it: " " + prompt.strip() against ids[1:] (BOS dropped)
        assert otok.bpe_encode(" " + p.strip()) == sp.encode(p)
    texts = seeded_texts(vocab, 150, seed=3) + ["héllo wörld", "naïve café 42", "你好 世界", "x = y + 1;", "a" * 40]
    for text in texts:
        assert otok.bpe_encode(" " + text) == sp.encode(text), text


def test_golden_ids_come_from_the_oracle(otok):
    for case in json.load(open(os.path.join(GOLD, "tokenizer_expected.json"))):
        assert otok.bpe_encode(" " + case["prompt"].strip()) == case["ids"]


def test_product_encoder_equals_the_oracle(oracle, otok):
    import llama2_rs
    t = llama2_rs.Tokenizer(os.path.join(GOLD, "tokenizer.bin"))
    vocab, _, _ = oracle.read_tokenizer_file(os.path.join(GOLD, "tokenizer.bin"), 32000)
    texts = [" " + p for p in PROMPTS] + [" " + s for s in seeded_texts(vocab, 120, seed=11)]
    # strings outside ordinary text: repeated spaces, leading and trailing spaces, newlines and tabs (byte
    # tokens below 260), digits runs, multi-byte UTF-8
    texts += ["  two  spaces", " trailing ", "   ", "\n", "a\nb\tc", " 1234567890", "日本語のテキスト", " çà et là", "\r\n",
              " ...", "''", " a", "a"]
    for text in texts:
        assert t.bpe_encode(text) == otok.bpe_encode(text), repr(text)
    with pytest.raises(Exception):
        t.bpe_encode("")
