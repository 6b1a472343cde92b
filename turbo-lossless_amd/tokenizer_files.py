"""tokenizer.json (Hugging Face byte-level BPE) -> the three binary files the engine's tokenizer reads.

    extract(tokenizer_json_path, out_dir)

Counterpart of the reference's engine/extract_tokenizer.py:24-105, same formats:

    vocab.bin         <iii n_vocab, bos_id, eos_id>, then per id <H length> + UTF-8 bytes
    merges.bin        <i n_merges>, then per merge <HH len_a, len_b> + bytes_a + bytes_b
    byte_encoder.bin  256 x (<B length> + UTF-8 bytes), the GPT-2 byte -> character table

`n_vocab` is the number of entries of model.vocab; an id in [0, n_vocab) that the vocabulary does not
use is written as the empty string (:69-73).  BOS / EOS come from added_tokens: <|begin_of_text|> /
<|end_of_text|>, or special <s> / </s>; defaults 128000 / 128001 (:51-62).
"""
from __future__ import annotations

import json
import os
import struct


def bytes_to_unicode() -> dict:
    """byte -> printable character: printable Latin-1 bytes map to themselves, the other 68 to U+0100...
    in byte order (engine/extract_tokenizer.py:12-22)."""
    keep = list(range(0x21, 0x7F)) + list(range(0xA1, 0xAD)) + list(range(0xAE, 0x100))
    table, spare = {}, 0
    for b in range(256):
        if b in keep:
            table[b] = chr(b)
        else:
            table[b] = chr(256 + spare)
            spare += 1
    return table


def write_files(out_dir: str, tokens_by_id, merges, bos_id: int, eos_id: int, byte_table=None) -> None:
    """tokens_by_id: list of str or bytes (index = id); merges: list of (a, b) in rank order;
    byte_table: {byte: str} or None for no byte_encoder.bin (the engine then maps bytes to themselves)."""
    def raw(s):
        return s if isinstance(s, (bytes, bytearray)) else s.encode("utf-8")

    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "vocab.bin"), "wb") as f:
        f.write(struct.pack("<iii", len(tokens_by_id), bos_id, eos_id))
        for t in tokens_by_id:
            b = raw(t)
            f.write(struct.pack("<H", len(b)))
            f.write(b)
    with open(os.path.join(out_dir, "merges.bin"), "wb") as f:
        f.write(struct.pack("<i", len(merges)))
        for a, b in merges:
            a, b = raw(a), raw(b)
            f.write(struct.pack("<HH", len(a), len(b)))
            f.write(a)
            f.write(b)
    if byte_table is not None:
        with open(os.path.join(out_dir, "byte_encoder.bin"), "wb") as f:
            for i in range(256):
                b = raw(byte_table[i])
                f.write(struct.pack("<B", len(b)))
                f.write(b)


def extract(tokenizer_json: str, out_dir: str) -> dict:
    with open(tokenizer_json, encoding="utf-8") as f:
        tok = json.load(f)
    model = tok.get("model", {})
    vocab = model.get("vocab", {})
    by_id = {v: k for k, v in vocab.items()}
    bos_id, eos_id = 128000, 128001
    for at in tok.get("added_tokens", []):
        content, tid = at.get("content", ""), at.get("id", -1)
        if content == "<|begin_of_text|>":
            bos_id = tid
        elif content == "<|end_of_text|>":
            eos_id = tid
        if at.get("special", False):
            if content == "<s>":
                bos_id = tid
            if content == "</s>":
                eos_id = tid
    merges = []
    for m in model.get("merges", []):
        a, b = m.split(" ", 1) if isinstance(m, str) else (m[0], m[1])
        merges.append((a, b))
    write_files(out_dir, [by_id.get(i, "") for i in range(len(vocab))], merges, bos_id, eos_id, bytes_to_unicode())
    return {"n_vocab": len(vocab), "n_merges": len(merges), "bos_id": bos_id, "eos_id": eos_id}
