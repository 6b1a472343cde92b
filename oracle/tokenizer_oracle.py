"""CPU restatement of the reference's byte-level BPE tokenizer -- TEST INFRASTRUCTURE ONLY.

Only tests/ may import this file.  It follows engine/tokenizer.cpp line by line, including its cost
(one pass over the text per merge), so it is for short texts and small merge tables:

  load              engine/tokenizer.cpp:161-208  (vocab.bin, merges.bin, byte_encoder.bin)
  bpe_encode        engine/tokenizer.cpp:295-326
  tokenize          engine/tokenizer.cpp:366-431  (special-token splitting, BOS in front)
  detokenize        engine/tokenizer.cpp:433-449
  detokenize_one    engine/tokenizer.cpp:451-506

Pinned by tests/test_tokenizer.py: on merge tables trained by the `tokenizers` library the encoder
equals that library's BPE model (no pre-tokenizer); the byte table of `bytes_to_unicode`
(engine/extract_tokenizer.py:12-22) equals the one `transformers` ships for GPT-2.  The reference's
sentencepiece backend (engine/tokenizer.cpp:12-29) is a call into the sentencepiece library and is not
restated here: tests/test_tokenizer_sp.py checks the product against that library (its Python package).
"""
import os
import struct


def bytes_to_unicode():
    """GPT-2 byte -> printable character table (engine/extract_tokenizer.py:12-22)."""
    bs = list(range(ord("!"), ord("~") + 1)) + list(range(0xA1, 0xAC + 1)) + list(range(0xAE, 0xFF + 1))
    cs = bs[:]
    n = 0
    for b in range(256):
        if b not in bs:
            bs.append(b)
            cs.append(256 + n)
            n += 1
    return {b: chr(c) for b, c in zip(bs, cs)}


class RefTokenizer:
    def __init__(self, model_dir):
        with open(os.path.join(model_dir, "vocab.bin"), "rb") as f:
            n_vocab, self.bos_id, self.eos_id = struct.unpack("<iii", f.read(12))
            self.id_to_token, self.token_to_id = {}, {}
            for i in range(n_vocab):
                (ln,) = struct.unpack("<H", f.read(2))
                t = f.read(ln)
                self.token_to_id[t] = i
                self.id_to_token[i] = t
        self.vocab_size = n_vocab
        with open(os.path.join(model_dir, "merges.bin"), "rb") as f:
            (n_merges,) = struct.unpack("<i", f.read(4))
            self.merges = []
            for _ in range(n_merges):
                la, lb = struct.unpack("<HH", f.read(4))
                a = f.read(la)
                b = f.read(lb)
                self.merges.append((a, b))
        be = os.path.join(model_dir, "byte_encoder.bin")
        if os.path.exists(be):
            self.byte_encoder = []
            with open(be, "rb") as f:
                for _ in range(256):
                    (ln,) = struct.unpack("<B", f.read(1))
                    self.byte_encoder.append(f.read(ln))
        else:
            self.byte_encoder = [bytes([i]) for i in range(256)]
        self.byte_decoder = {}
        for i in range(256):
            if self.byte_encoder[i]:
                self.byte_decoder[self.byte_encoder[i]] = i
        self.special_tokens = []          # (text bytes, id), longest first

    def add_special(self, text: bytes, tid: int):
        self.special_tokens.append((text, tid))
        self.special_tokens.sort(key=lambda s: -len(s[0]))      # stable, longest first (:136-140)

    def bpe_encode(self, text: bytes):
        tokens = [self.byte_encoder[c] for c in text]
        for left, right in self.merges:
            i = 0
            while i + 1 < len(tokens):
                if tokens[i] == left and tokens[i + 1] == right:
                    tokens[i] = left + right
                    del tokens[i + 1]
                else:
                    i += 1
        return [self.token_to_id.get(t, 0) for t in tokens]

    def tokenize(self, text: bytes):
        if not self.special_tokens:
            return [self.bos_id] + self.bpe_encode(text)
        ids, pos = [], 0
        while pos < len(text):
            hit = next(((s, i) for s, i in self.special_tokens if text.startswith(s, pos)), None)
            if hit:
                ids.append(hit[1])
                pos += len(hit[0])
                continue
            stop = len(text)
            for s, _ in self.special_tokens:
                at = text.find(s, pos)
                if at != -1 and at < stop:
                    stop = at
            if stop > pos:
                ids += self.bpe_encode(text[pos:stop])
            pos = stop
        return [self.bos_id] + ids

    def detokenize(self, ids):
        return b"".join(self.id_to_token[i] for i in ids if i in self.id_to_token)

    def detokenize_one(self, tid):
        for s, i in self.special_tokens:
            if i == tid:
                return s
        if tid not in self.id_to_token:
            return b""
        t = self.id_to_token[tid]
        out, i = bytearray(), 0
        while i < len(t):
            for ln in (4, 3, 2, 1):
                if i + ln <= len(t) and t[i:i + ln] in self.byte_decoder:
                    out.append(self.byte_decoder[t[i:i + ln]])
                    i += ln
                    break
            else:
                out.append(t[i])
                i += 1
        return bytes(out)
