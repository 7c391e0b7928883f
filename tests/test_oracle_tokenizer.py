"""Pins the Python tokenizer checker (oracle/tokenizer_ref.py).  CPU only."""
import os

import pytest

from oracle import tokenizer_ref as T


def _byte_vocab():
    # ids 0..2 specials, 3..258 the raw bytes as <0xHH>, as in the reference's sentencepiece exports
    vocab = [b"<unk>", b"<s>", b"</s>"] + [("<0x%02X>" % b).encode() for b in range(256)]
    scores = [0.0] * len(vocab)
    return vocab, scores


def test_hand_worked_merges_and_tie_rule():
    vocab, scores = _byte_vocab()
    extra = {b" ": -1.0, b"a": -2.0, b"b": -3.0, b"c": -4.0, b"ab": -0.5, b"bc": -0.5, b" a": -0.7, b"abc": -0.1, b" ab": -9.0}
    for k, v in extra.items():
        vocab.append(k)
        scores.append(v)
    tok = T.Tokenizer(vocab, scores)
    idx = {k: tok.lookup(k) for k in extra}
    # " abc": start [" ", a, b, c].  Candidates: " a" (-0.7), "ab" (-0.5), "bc" (-0.5): the tie between "ab" and "bc"
    # goes to the leftmost (strict >), giving [" ", ab, c]; then " ab" (-9.0) vs "abc" (-0.1): "abc" -> [" ", abc];
    # " abc" is not in the vocabulary, so that is the result.
    assert tok.encode("abc", bos=True, eos=True) == [1, idx[b" "], idx[b"abc"], 2]
    # empty text: no dummy prefix
    assert tok.encode("", bos=True, eos=False) == [1]
    assert tok.encode("", bos=False, eos=False) == []


def test_byte_fallback_utf8_and_decode():
    vocab, scores = _byte_vocab()
    for k in (b" ", "é".encode(), b"x"):
        vocab.append(k)
        scores.append(-1.0)
    tok = T.Tokenizer(vocab, scores)
    e = "é".encode()
    snow = "☃".encode()          # three bytes, not in the vocabulary -> three byte tokens (+3)
    ids = tok.encode("xé☃", bos=False)
    assert ids == [tok.lookup(b" "), tok.lookup(b"x"), tok.lookup(e)] + [b + 3 for b in snow]
    assert b"".join(tok.decode(0, i) for i in ids) == b" x" + e + snow
    # leading space is dropped only right after BOS
    assert tok.decode(1, tok.lookup(b" ")) == b"" and tok.decode(5, tok.lookup(b" ")) == b" "
    assert tok.decode(0, 3) == b""          # <0x00> is the empty C string
    assert tok.decode(0, 3 + 0x41) == b"A"


def test_file_round_trip(tmp_path):
    vocab, scores = _byte_vocab()
    vocab += [b" ", b"hello", b" world"]
    scores += [-1.0, -2.5, -3.25]
    p = str(tmp_path / "tok.bin")
    T.write_tokenizer(p, vocab, scores)
    v2, s2, mx = T.read_tokenizer(p, len(vocab))
    assert v2 == vocab and s2 == scores and mx == max(len(v) for v in vocab)


def test_encode_matches_sentencepiece_bpe(tmp_path):
    """Independent implementation: a BPE model trained here by sentencepiece, exported the way the reference's
    tokenizer files are made (pieces with U+2581 turned into spaces, scores as they are)."""
    spm = pytest.importorskip("sentencepiece")
    corpus = str(tmp_path / "corpus.txt")
    words = ("the quick brown fox jumps over the lazy dog while seven wizards quietly boxed jam and a cat sat on the mat "
             "because matrices multiply faster when tiles stay in registers and caches remember what lanes forget").split()
    import random
    rnd = random.Random(3)
    with open(corpus, "w") as f:
        for _ in range(400):
            f.write(" ".join(rnd.choice(words) for _ in range(rnd.randint(3, 12))) + "\n")
    prefix = str(tmp_path / "m")
    spm.SentencePieceTrainer.train(input=corpus, model_prefix=prefix, vocab_size=400, model_type="bpe", byte_fallback=True,
                                   character_coverage=1.0, normalization_rule_name="identity", unk_id=0, bos_id=1, eos_id=2,
                                   minloglevel=2)
    sp = spm.SentencePieceProcessor(model_file=prefix + ".model")
    vocab = [sp.id_to_piece(i).replace("▁", " ").encode("utf-8") for i in range(sp.get_piece_size())]
    scores = [sp.get_score(i) for i in range(sp.get_piece_size())]
    tok = T.Tokenizer(vocab, scores)
    for _ in range(60):
        text = " ".join(rnd.choice(words) for _ in range(rnd.randint(1, 9)))
        assert tok.encode(text, bos=False, eos=False) == sp.encode(text), text
    # round trip through decode
    ids = tok.encode("the lazy cat", bos=True)
    assert ids[0] == 1
    prev, out = 1, b""
    for i in ids[1:]:          # the piece after BOS loses its leading space
        out += tok.decode(prev, i)
        prev = i
    assert out == b"the lazy cat"
