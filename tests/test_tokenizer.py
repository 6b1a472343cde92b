"""CPU: the engine's byte-level BPE tokenizer (host code of the C-ABI library) against the oracle restatement of
engine/tokenizer.cpp, and the oracle against independent implementations:

* `tokenizers` (Hugging Face, Rust): a BPE model trained by that library, encoded by it without any
  pre-tokenizer, must give the ids the reference rule gives (rank-ordered passes == lowest-rank-first BPE on
  a consistent merge table);
* `transformers`: the GPT-2 byte table.

Where the reference's rule differs from textbook BPE (a pair listed twice, a merge listed before the merges
that build its parts) only the oracle, which restates the reference's loops literally, is the checker.
"""
import json
import os
import random
import struct

import pytest

from oracle.tokenizer_oracle import RefTokenizer, bytes_to_unicode as oracle_b2u


@pytest.fixture(scope="module")
def tf(t12):
    from importlib import import_module
    return import_module(t12.__name__ + ".tokenizer_files")


def random_text(rng, n, alphabet):
    return bytes(rng.choice(alphabet) for _ in range(n))


def random_table(rng, n_merges, alphabet, consistent=True):
    """A merge table over single-byte symbols (identity byte encoder).  consistent: every merge joins two symbols
    that exist by then, no pair twice (what a trainer emits); else parts are drawn from all symbols the table
    will ever hold and pairs repeat."""
    syms = [bytes([a]) for a in alphabet]
    merges, seen = [], set()
    if consistent:
        while len(merges) < n_merges:
            a, b = rng.choice(syms), rng.choice(syms)
            if (a, b) in seen or len(a + b) > 12:
                continue
            seen.add((a, b))
            merges.append((a, b))
            if a + b not in syms:
                syms.append(a + b)
    else:
        pool = list(syms)
        for _ in range(n_merges):
            a, b = rng.choice(pool), rng.choice(pool)
            if len(a + b) <= 10:
                pool.append(a + b)
        while len(merges) < n_merges:
            a, b = rng.choice(pool), rng.choice(pool)
            merges.append((a, b))
            if rng.random() < 0.15 and merges:
                merges.append(rng.choice(merges))
    return merges


def vocab_for(rng, merges, alphabet, drop=0.1):
    """ids for most symbols; some left out (-> id 0), one string listed twice (last id wins for encoding)."""
    toks = [b"<unk>", b"<s>", b"</s>"] + [bytes([a]) for a in alphabet]
    for a, b in merges:
        if a + b not in toks and rng.random() > drop:
            toks.append(a + b)
    if len(toks) > 6:
        toks.append(toks[5])
    return toks


def both(t12, tf, tmp_path, toks, merges, byte_table=None, bos=1, eos=2):
    d = str(tmp_path)
    tf.write_files(d, toks, merges, bos, eos, byte_table)
    return t12.Tokenizer(d), RefTokenizer(d)


@pytest.mark.parametrize("seed,consistent", [(1, True), (2, True), (3, False), (4, False), (5, False)])
def test_encode_equals_reference_rule(t12, tf, tmp_path, seed, consistent):
    rng = random.Random(seed)
    alphabet = list(b"abcdef \n")
    merges = random_table(rng, 60, alphabet, consistent)
    toks = vocab_for(rng, merges, alphabet)
    ours, ref = both(t12, tf, tmp_path, toks, merges)
    assert (ours.bos_id, ours.eos_id, ours.vocab_size) == (ref.bos_id, ref.eos_id, ref.vocab_size) == (1, 2, len(toks))
    for n in [0, 1, 2, 3, 7, 40, 200, 600]:
        for _ in range(6):
            text = random_text(rng, n, alphabet)
            assert ours.tokenize(text) == ref.tokenize(text), (text, merges)
    ours.close()


def test_repeated_symbols_merge_left_to_right(t12, tf, tmp_path):
    merges = [(b"a", b"a"), (b"aa", b"a"), (b"aa", b"aa")]
    toks = [b"?", b"<s>", b"</s>", b"a", b"aa", b"aaa", b"aaaa"]
    ours, ref = both(t12, tf, tmp_path, toks, merges)
    for n in range(0, 12):
        assert ours.tokenize(b"a" * n) == ref.tokenize(b"a" * n)
    assert ours.tokenize(b"aaa") == [1, 5]                 # (a a) a -> (aa a)
    assert ours.tokenize(b"aaaa") == [1, 6]                # (a a)(a a) -> (aa aa): (aa, a) finds nothing in between
    assert ours.tokenize(b"aaaaa") == [1, 4, 5]            # (aa)(aa)(a) -> (aa)(aa a): passes go left to right, once
    ours.close()


def test_merge_listed_before_its_parts_exist_is_never_applied(t12, tf, tmp_path):
    """(ab, c) at rank 0, (a, b) at rank 1: when "ab" appears, the pass of rank 0 is over -- the reference's loop
    (engine/tokenizer.cpp:305-314) does not come back, textbook lowest-rank-first BPE would."""
    merges = [(b"ab", b"c"), (b"a", b"b"), (b"ab", b"c")]
    toks = [b"?", b"<s>", b"</s>", b"a", b"b", b"c", b"ab", b"abc"]
    ours, ref = both(t12, tf, tmp_path, toks, merges)
    assert ref.tokenize(b"abc") == [1, 7]                  # the second listing, rank 2, does apply
    assert ours.tokenize(b"abc") == [1, 7]
    ours.close()
    merges = merges[:2]
    sub = tmp_path / "once"
    sub.mkdir()
    ours, ref = both(t12, tf, sub, toks, merges)
    assert ref.tokenize(b"abc") == [1, 6, 5]
    assert ours.tokenize(b"abc") == [1, 6, 5]
    ours.close()


def test_unknown_symbol_is_id_zero_and_duplicate_string_takes_last_id(t12, tf, tmp_path):
    toks = [b"?", b"<s>", b"</s>", b"a", b"b", b"a"]       # "a" twice: id 5 encodes, both decode
    merges = [(b"a", b"b")]                                # "ab" is not in the vocabulary
    ours, ref = both(t12, tf, tmp_path, toks, merges)
    assert ours.tokenize(b"aab") == ref.tokenize(b"aab") == [1, 5, 0]
    assert ours.detokenize([3, 5, 4, 99, -1]) == ref.detokenize([3, 5, 4, 99, -1]) == b"aab"
    ours.close()


def test_special_tokens_are_cut_out_longest_first(t12, tf, tmp_path):
    rng = random.Random(9)
    alphabet = list(b"abIN[]/ ")
    merges = random_table(rng, 30, alphabet)
    toks = vocab_for(rng, merges, alphabet, drop=0.0)
    ours, ref = both(t12, tf, tmp_path, toks, merges)
    for text, tid in [(b"[INST]", 900), (b"[/INST]", 901), (b"[IN", 902), (b"]", 903)]:
        ours.add_special(text, tid)
        ref.add_special(text, tid)
    cases = [b"[INST] ab [/INST]", b"[INST][INST]", b"ab[IN", b"[INS", b"a]b]", b"", b"[/INST", b"[INST] a [/INST] b [INST] a"]
    cases += [random_text(rng, 50, alphabet) for _ in range(30)]
    for text in cases:
        assert ours.tokenize(text) == ref.tokenize(text), text
    assert ours.detokenize_one(901) == ref.detokenize_one(901) == b"[/INST]"
    ours.close()


def test_byte_table_round_trip_and_display_text(t12, tf, tmp_path):
    table = tf.bytes_to_unicode()
    rng = random.Random(11)
    toks = [b"<unk>", b"<s>", b"</s>"] + [table[b].encode() for b in range(256)]
    merges = []
    for _ in range(300):
        a, b = rng.choice(toks[3:]), rng.choice(toks[3:])
        if (a, b) not in merges and len(a + b) < 40:
            merges.append((a, b))
            if a + b not in toks:
                toks.append(a + b)
    ours, ref = both(t12, tf, tmp_path, toks, merges, table)
    for text in [bytes(range(256)), "héllo wörld ▁ \U0001F600\n\t".encode(), random_text(rng, 500, list(range(256)))]:
        ids = ours.tokenize(text)
        assert ids == ref.tokenize(text)
        assert ours.detokenize(ids[1:]) == ref.detokenize(ids[1:])
        shown = b"".join(ours.detokenize_one(i) for i in ids[1:])
        assert shown == b"".join(ref.detokenize_one(i) for i in ids[1:]) == text       # every symbol is in the vocabulary
    assert ours.detokenize_one(10 ** 6) == ref.detokenize_one(10 ** 6) == b""
    assert ours.detokenize_one(0) == ref.detokenize_one(0) == b"<unk>"                 # not byte-encoder text: passes through
    ours.close()


def test_identity_byte_table_when_file_is_absent(t12, tf, tmp_path):
    toks = [b"?", b"<s>", b"</s>", b"\xc3", b"\xa9", b"\xc3\xa9"]
    ours, ref = both(t12, tf, tmp_path, toks, [(b"\xc3", b"\xa9")], byte_table=None)
    assert not os.path.exists(tmp_path / "byte_encoder.bin")
    assert ours.tokenize("é".encode()) == ref.tokenize("é".encode()) == [1, 5]
    assert ours.detokenize_one(5) == ref.detokenize_one(5) == "é".encode()
    ours.close()


def test_missing_and_malformed_files(t12, tf, tmp_path):
    with pytest.raises(t12.T12Error):
        t12.Tokenizer(str(tmp_path))                        # nothing there
    (tmp_path / "tokenizer.model").write_bytes(b"\x0a\x00")
    with pytest.raises(t12.T12Error):
        t12.Tokenizer(str(tmp_path))                        # sentencepiece model only: not read by this build
    tf.write_files(str(tmp_path), [b"a", b"b"], [(b"a", b"b")], 0, 1)
    t12.Tokenizer(str(tmp_path)).close()
    data = (tmp_path / "merges.bin").read_bytes()
    (tmp_path / "merges.bin").write_bytes(data[:-1])
    with pytest.raises(t12.T12Error):
        t12.Tokenizer(str(tmp_path))                        # truncated
    (tmp_path / "merges.bin").write_bytes(struct.pack("<iHH", 1, 1, 0) + b"a")
    with pytest.raises(t12.T12Error):
        t12.Tokenizer(str(tmp_path))                        # empty merge part


# ---- the oracle against independent implementations --------------------------------------------------------------

def test_oracle_byte_table_is_the_gpt2_table(tf):
    from tokenizers import pre_tokenizers
    from transformers.convert_slow_tokenizer import bytes_to_unicode as hf_b2u
    assert oracle_b2u() == hf_b2u() == tf.bytes_to_unicode()
    assert set(oracle_b2u().values()) == set(pre_tokenizers.ByteLevel.alphabet())


def trained_tokenizer_json(tmp_path, seed):
    """A byte-level BPE trained by the `tokenizers` library on seeded text; returns (tokenizer.json path, library
    encoder without pre-tokenisation)."""
    import tokenizers
    from tokenizers import decoders, models, pre_tokenizers, trainers

    rng = random.Random(seed)
    words = ["".join(rng.choice("abcdefgh") for _ in range(rng.randint(1, 7))) for _ in range(60)]
    words += ["é", "ß", "日本", "\n", "  "]
    corpus = [" ".join(rng.choice(words) for _ in range(30)) for _ in range(200)]
    tk = tokenizers.Tokenizer(models.BPE())
    tk.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)
    tk.decoder = decoders.ByteLevel()
    trainer = trainers.BpeTrainer(vocab_size=600, special_tokens=["<s>", "</s>"], show_progress=False,
                                  initial_alphabet=pre_tokenizers.ByteLevel.alphabet())
    tk.train_from_iterator(corpus, trainer)
    path = os.path.join(str(tmp_path), "tokenizer.json")
    tk.save(path)
    return path, tk, words


@pytest.mark.parametrize("seed", [21, 22])
def test_oracle_and_engine_equal_the_tokenizers_library_on_a_trained_table(t12, tf, tmp_path, seed):
    path, tk, words = trained_tokenizer_json(tmp_path, seed)
    out = tmp_path / "bin"
    info = tf.extract(path, str(out))
    spec = json.load(open(path))
    assert info["n_vocab"] == len(spec["model"]["vocab"]) and info["n_merges"] == len(spec["model"]["merges"]) > 100
    assert (info["bos_id"], info["eos_id"]) == (0, 1)       # special <s>, </s> (engine/extract_tokenizer.py:60-62)
    ours, ref = t12.Tokenizer(str(out)), RefTokenizer(str(out))
    rng = random.Random(seed + 100)
    for _ in range(40):
        text = " ".join(rng.choice(words) for _ in range(rng.randint(1, 25)))
        want = tk.encode(text, add_special_tokens=False).ids          # whole text as one word: no regex split
        assert ref.tokenize(text.encode())[1:] == want, text
        assert ours.tokenize(text.encode())[1:] == want, text
        shown = b"".join(ours.detokenize_one(i) for i in want)
        assert shown == text.encode() == tk.decode(want).encode()
    ours.close()


def test_long_text_on_a_larger_trained_table_equals_the_tokenizers_library(t12, tf, tmp_path):
    """20 kB of text through a 3000-entry table: too long for the literal restatement (one pass per merge), so the
    checker here is the `tokenizers` library alone."""
    import tokenizers
    from tokenizers import models, pre_tokenizers, trainers

    rng = random.Random(77)
    words = ["".join(rng.choice("abcdefghijklmnop") for _ in range(rng.randint(1, 9))) for _ in range(800)] + ["\n", "é", "€"]
    corpus = [" ".join(rng.choice(words) for _ in range(40)) for _ in range(600)]
    tk = tokenizers.Tokenizer(models.BPE())
    tk.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)
    tk.train_from_iterator(corpus, trainers.BpeTrainer(vocab_size=3000, special_tokens=["<s>", "</s>"], show_progress=False,
                                                       initial_alphabet=pre_tokenizers.ByteLevel.alphabet()))
    path = os.path.join(str(tmp_path), "tokenizer.json")
    tk.save(path)
    tf.extract(path, str(tmp_path))
    ours = t12.Tokenizer(str(tmp_path))
    text = " ".join(rng.choice(words) for _ in range(4000))
    assert len(text) > 20000
    assert ours.tokenize(text)[1:] == tk.encode(text, add_special_tokens=False).ids
    ours.close()


def test_extract_writes_the_reference_file_formats(tf, tmp_path):
    """Bytes of the three files for a hand-written tokenizer.json (formats: engine/extract_tokenizer.py:66-104)."""
    spec = {"added_tokens": [{"id": 7, "content": "<|begin_of_text|>", "special": True},
                             {"id": 8, "content": "<|end_of_text|>", "special": True},
                             {"id": 9, "content": "</s>", "special": False}],
            "model": {"vocab": {"a": 0, "Ġb": 2, "aĠb": 3}, "merges": ["a Ġb", ["Ġ", "b"]]}}
    p = tmp_path / "tokenizer.json"
    p.write_text(json.dumps(spec), encoding="utf-8")
    info = tf.extract(str(p), str(tmp_path))
    assert info == {"n_vocab": 3, "n_merges": 2, "bos_id": 7, "eos_id": 8}
    g = "Ġ".encode()
    want = struct.pack("<iii", 3, 7, 8) + struct.pack("<H", 1) + b"a" + struct.pack("<H", 0) + struct.pack("<H", 3) + g + b"b"
    assert (tmp_path / "vocab.bin").read_bytes() == want      # id 1 unused -> empty string; id 3 is beyond n_vocab = len(vocab)
    want = struct.pack("<i", 2) + struct.pack("<HH", 1, 3) + b"a" + g + b"b" + struct.pack("<HH", 2, 1) + g + b"b"
    assert (tmp_path / "merges.bin").read_bytes() == want
    be = (tmp_path / "byte_encoder.bin").read_bytes()
    # byte 0 -> U+0100; 94 printable ASCII bytes keep 1 UTF-8 byte, the other 162 characters take 2
    assert be[:3] == b"\x02\xc4\x80" and len(be) == 256 + 94 + 2 * 162


def test_encode_equals_reference_rule_on_generated_tables(t12, tf, tmp_path):
    """Property test (hypothesis): any merge table over a three-letter alphabet -- pairs repeated, merges listed
    before their parts exist, results missing from the vocabulary -- and any text: same ids as the literal rule."""
    hyp = pytest.importorskip("hypothesis")
    st = pytest.importorskip("hypothesis.strategies")
    sym = st.text(alphabet="abc", min_size=1, max_size=4).map(str.encode)
    tables = st.lists(st.tuples(sym, sym), min_size=0, max_size=12)
    texts_ = st.lists(st.text(alphabet="abc", min_size=0, max_size=40).map(str.encode), min_size=1, max_size=6)
    counter = [0]

    @hyp.settings(max_examples=150, deadline=None, suppress_health_check=list(hyp.HealthCheck))
    @hyp.given(merges=tables, texts=texts_, drop=st.integers(0, 3))
    def check(merges, texts, drop):
        counter[0] += 1
        d = tmp_path / ("t%d" % counter[0])
        d.mkdir()
        toks = [b"?", b"<s>", b"</s>", b"a", b"b", b"c"]
        for i, (x, y) in enumerate(merges):
            if x + y not in toks and i % 4 != drop:
                toks.append(x + y)
        tf.write_files(str(d), toks, merges, 1, 2, None)
        ours, ref = t12.Tokenizer(str(d)), RefTokenizer(str(d))
        try:
            for text in texts:
                assert ours.tokenize(text) == ref.tokenize(text), (merges, text)
        finally:
            ours.close()

    check()
