"""Python restatement of the reference's BPE tokenizer and of its text-generation loop.

TEST INFRASTRUCTURE ONLY (parity checker for the tokenizer and the text entry of the llama2 extension).
Follows CudaExtension.llm32.llama2/Files/llama2_tokenizer.cpp (build_tokenizer :28-52, decode :66-78,
encode :101-220) and LLMData::Generate (llm.cpp:193-263).

Pins (tests/test_oracle_tokenizer.py): a hand-worked merge example whose result is fixed by the merge rule
(highest score first, leftmost on ties); byte fallback and <0xHH> decoding on constructed vocabularies; and an
independent implementation: a sentencepiece BPE model trained in the test on a small corpus, exported to this
file format, whose own ``encode`` must give the same ids on plain ASCII sentences.
"""
import re
import struct


def write_tokenizer(path, vocab, scores, max_token_length=None):
    """vocab: list of bytes; the layout build_tokenizer reads (llama2_tokenizer.cpp:28-52)."""
    if max_token_length is None:
        max_token_length = max(len(v) for v in vocab)
    with open(path, "wb") as f:
        f.write(struct.pack("<i", max_token_length))
        for v, s in zip(vocab, scores):
            f.write(struct.pack("<fi", float(s), len(v)))
            f.write(v)


def read_tokenizer(path, vocab_size):
    vocab, scores = [], []
    with open(path, "rb") as f:
        (max_len,) = struct.unpack("<i", f.read(4))
        for _ in range(vocab_size):
            s, n = struct.unpack("<fi", f.read(8))
            v = f.read(n)
            vocab.append(v.split(b"\0")[0])      # C strings
            scores.append(s)
    return vocab, scores, max_len


class Tokenizer:
    def __init__(self, vocab, scores):
        self.vocab = [bytes(v) for v in vocab]
        self.scores = [float(s) for s in scores]
        self.index = {}
        for i in range(len(self.vocab) - 1, -1, -1):   # lowest id wins among duplicates
            self.index[self.vocab[i]] = i

    def lookup(self, s):
        return self.index.get(bytes(s), -1)

    def encode(self, text, bos=True, eos=False):
        """llama2_tokenizer.cpp:101-220; ``text`` is bytes (UTF-8) or str."""
        if isinstance(text, str):
            text = text.encode("utf-8")
        text = text.split(b"\0")[0]
        tokens = []
        if bos:
            tokens.append(1)
        if text:
            tokens.append(self.lookup(b" "))
        cp = bytearray()
        for i, c in enumerate(text):
            if (c & 0xC0) != 0x80:
                cp = bytearray()
            cp.append(c)
            nx = text[i + 1] if i + 1 < len(text) else 0
            if (nx & 0xC0) == 0x80 and len(cp) < 4:
                continue
            tid = self.lookup(cp)
            if tid != -1:
                tokens.append(tid)
            else:
                tokens.extend(b + 3 for b in cp)
            cp = bytearray()
        while True:
            best, best_id, best_idx = -1e10, -1, -1
            for i in range(len(tokens) - 1):
                tid = self.lookup(self._piece(tokens[i]) + self._piece(tokens[i + 1]))
                if tid != -1 and self.scores[tid] > best:
                    best, best_id, best_idx = self.scores[tid], tid, i
            if best_idx == -1:
                break
            tokens[best_idx:best_idx + 2] = [best_id]
        if eos:
            tokens.append(2)
        return tokens

    def _piece(self, tid):
        return self.vocab[tid] if 0 <= tid < len(self.vocab) else b""

    def decode(self, prev_token, token):
        """llama2_tokenizer.cpp:66-78."""
        p = self.vocab[token]
        if prev_token == 1 and p[:1] == b" ":
            p = p[1:]
        m = re.match(rb"<0x([0-9A-Fa-f]{1,2})", p)     # sscanf("<0x%02hhX>") stops checking after the digits
        if m:
            b = int(m.group(1), 16)
            return bytes([b]) if b else b""
        return p


def generate_text(model, tok, prompt, steps):
    """LLMData::Generate (llm.cpp:193-263) with greedy sampling; ``model`` has forward-free access through
    ``generate_greedy(prompt_ids, n)`` returning the id chosen after every position.  Returns the response bytes."""
    toks = tok.encode(prompt, True, False)
    n = len(toks)
    out = model.generate_greedy(toks, steps)
    resp = b""
    for pos in range(steps):
        token = toks[pos] if pos < n else int(out[pos - 1])
        nxt = int(out[pos])
        if pos + 1 >= n and nxt != 2:
            resp += tok.decode(token, nxt)
        if token == 2 or nxt == 2:
            break
    return resp


def generate_text_sampled(model, tok, prompt, steps, sampler):
    """LLMData::Generate (llm.cpp:193-263) with the engine's sampler: ``model.forward(token, pos)`` gives the logits,
    ``sampler.sample(logits)`` is called at every position (the prompt's included), and the loop ends on the step that
    feeds or draws the end-of-text id, so the sampler's random state carries over to the next call as in the reference.
    Returns the response bytes."""
    toks = tok.encode(prompt, True, False)
    n = len(toks)
    resp = b""
    nxt = 0
    for pos in range(steps):
        token = toks[pos] if pos < n else nxt
        nxt = sampler.sample(model.forward(token, pos))
        if pos + 1 >= n and nxt != 2:
            resp += tok.decode(token, nxt)
        if token == 2 or nxt == 2:
            break
    return resp
