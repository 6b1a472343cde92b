"""CPU: the engine's reader / encoder of sentencepiece BPE models (the reference's first tokenizer backend,
engine/tokenizer.cpp:12-29,366-506, which calls the sentencepiece library) against that library itself: the
`sentencepiece` Python package wraps the same C++ code.  Models are trained here, by the library, on seeded text."""
import io
import json
import random

import pytest

spm = pytest.importorskip("sentencepiece")

SPACE = "▁"


def train(seed, **kw):
    rng = random.Random(seed)
    words = ["".join(rng.choice("abcdefghij") for _ in range(rng.randint(1, 7))) for _ in range(150)] + ["é", "ß", "naïve"]
    corpus = [" ".join(rng.choice(words) for _ in range(20)) for _ in range(400)]
    out = io.BytesIO()
    args = dict(sentence_iterator=iter(corpus), model_writer=out, vocab_size=kw.pop("vocab_size", 330), model_type="bpe",
                normalization_rule_name="identity", character_coverage=1.0, bos_id=1, eos_id=2, unk_id=0, pad_id=-1,
                minloglevel=2)
    args.update(kw)
    spm.SentencePieceTrainer.train(**args)
    return out.getvalue(), words


def texts(rng, words):
    odd = ["日本語", "🙂", "x", "Q", "\t", "\n", "  ", "   ", "<0x41>", "<s>", "</s>", "<unk>", SPACE, "a" * 40]
    out = ["", " ", "  ", "a", " a", "a ", "  a  b   c  ", "\n", "é", "日本", "ab\tcd", "<s>ab</s>"]
    for _ in range(120):
        n = rng.randint(1, 14)
        parts = [rng.choice(words) if rng.random() < 0.8 else rng.choice(odd) for _ in range(n)]
        out.append(rng.choice(["", " ", "  "]) + rng.choice([" ", "  ", ""]).join(parts) + rng.choice(["", " ", "\n"]))
    return out


def load_both(t12, tmp_path, proto):
    (tmp_path / "tokenizer.model").write_bytes(proto)
    return t12.Tokenizer(str(tmp_path)), spm.SentencePieceProcessor(model_proto=proto)


CONFIGS = {
    "llama_like": dict(byte_fallback=True, remove_extra_whitespaces=False),
    "defaults": dict(byte_fallback=True),
    "no_byte_fallback": dict(byte_fallback=False, vocab_size=80),
    "no_dummy_prefix": dict(byte_fallback=True, add_dummy_prefix=False, remove_extra_whitespaces=False),
    "larger_vocab": dict(byte_fallback=True, remove_extra_whitespaces=False, vocab_size=560),
    "user_defined": dict(byte_fallback=True, remove_extra_whitespaces=False, user_defined_symbols=["[INST]", "[/INST]", "<sep>"]),
}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_encode_and_decode_equal_the_sentencepiece_library(t12, tmp_path, name):
    proto, words = train(7 + len(name), **CONFIGS[name])
    ours, sp = load_both(t12, tmp_path, proto)
    assert ours.type == 0
    assert (ours.bos_id, ours.eos_id, ours.vocab_size) == (sp.bos_id(), sp.eos_id(), sp.get_piece_size())
    rng = random.Random(99)
    cases = texts(rng, words)
    if name == "user_defined":
        cases += ["[INST] ab [/INST]", "a[INST]b", "[INS", "<sep><sep>", " [INST]", "x<sep> y"]
    for text in cases:
        want = sp.encode(text)
        got = ours.tokenize(text)
        assert got[0] == sp.bos_id() and got[1:] == want, (name, text, sp.encode(text, out_type=str))
        assert ours.detokenize(want) == sp.decode(want).encode(), (name, text)
    # decoding of id sequences no encoder produces: control ids inside, byte runs cut mid-character, the unknown id
    n = sp.get_piece_size()
    for _ in range(200):
        ids = [rng.randrange(n) for _ in range(rng.randint(0, 12))]
        assert ours.detokenize(ids) == sp.decode(ids).encode(), (name, ids, [sp.id_to_piece(i) for i in ids])
    ours.close()


def test_bytes_that_are_not_utf8_become_the_replacement_character(t12, tmp_path):
    proto, _ = train(3, byte_fallback=True, remove_extra_whitespaces=False)
    ours, sp = load_both(t12, tmp_path, proto)
    for raw in [b"\xff", b"ab\xc3", b"\xc3\x28", b"\xe2\x82", b"a\xf0\x9f\x99\x82b", b"\xed\xa0\x80", b"\xc0\xaf"]:
        assert ours.tokenize(raw)[1:] == sp.encode(raw), raw
    ours.close()


def test_display_text_of_single_ids(t12, tmp_path):
    """detokenize_one is the reference's own conversion of IdToPiece (engine/tokenizer.cpp:484-506): escaped blanks
    become spaces, <0xXX> the byte, everything else passes through (control pieces included)."""
    proto, _ = train(4, byte_fallback=True)
    ours, sp = load_both(t12, tmp_path, proto)
    for i in list(range(0, 270)) + [sp.get_piece_size() - 1]:
        piece = sp.id_to_piece(i)
        if piece.startswith("<0x") and piece.endswith(">") and len(piece) == 6:
            want = bytes([int(piece[3:5], 16)])
        else:
            want = piece.replace(SPACE, " ").encode()
        assert ours.detokenize_one(i) == want, (i, piece)
    assert ours.detokenize_one(10 ** 6) == b"" and ours.detokenize_one(-1) == b""
    ours.close()


def test_special_tokens_are_read_from_tokenizer_json_like_the_reference_does(t12, tmp_path):
    proto, _ = train(5, byte_fallback=True, remove_extra_whitespaces=False)
    spec = {"added_tokens": [
        {"id": 0, "content": "<unk>", "special": True},                       # id <= 2: left out
        {"id": 2, "content": "</s>", "special": True},
        {"id": 300, "content": "[INST]", "special": True},
        {"id": 301, "content": "[/INST]", "normalized": False, "special": True},
        {"id": 302, "content": "<tool>", "normalized": True, "special": False},   # "special" and a true: counted (:113-114)
        {"id": 303, "content": "x", "special": True},                         # one character: left out
        {"id": 304, "content": "<plain>", "normalized": False, "special": False}],
        "model": {"vocab": {}}}
    (tmp_path / "tokenizer.json").write_text(json.dumps(spec))
    ours, sp = load_both(t12, tmp_path, proto)
    assert ours.special_tokens() == [(b"[/INST]", 301), (b"[INST]", 300), (b"<tool>", 302)]
    assert ours.eos_id == 2
    got = ours.tokenize("[INST] ab [/INST]cd<tool>")
    assert got == [sp.bos_id(), 300] + sp.encode(" ab ") + [301] + sp.encode("cd") + [302]     # stretches are encoded on their own
    assert ours.detokenize_one(301) == b"[/INST]"
    ours.close()
    spec["added_tokens"].append({"id": 7, "content": "</s>", "special": True})
    (tmp_path / "tokenizer.json").write_text(json.dumps(spec))
    ours, _ = load_both(t12, tmp_path, proto)
    assert ours.eos_id == 7                                                    # a special </s> moves eos_id (:125-126)
    ours.close()


def test_models_this_build_does_not_read_fall_through_to_the_bpe_tables(t12, tmp_path):
    rng = random.Random(1)
    corpus = [" ".join("".join(rng.choice("abcdef") for _ in range(rng.randint(1, 6))) for _ in range(20)) for _ in range(300)]
    out = io.BytesIO()
    spm.SentencePieceTrainer.train(sentence_iterator=iter(corpus), model_writer=out, vocab_size=60, model_type="unigram",
                                   normalization_rule_name="identity", minloglevel=2)
    (tmp_path / "tokenizer.model").write_bytes(out.getvalue())
    with pytest.raises(t12.T12Error):
        t12.Tokenizer(str(tmp_path))                        # unigram model, no vocab.bin: nothing to load
    out = io.BytesIO()
    spm.SentencePieceTrainer.train(sentence_iterator=iter(corpus), model_writer=out, vocab_size=60, model_type="bpe",
                                   minloglevel=2)           # default normalisation: a character map
    (tmp_path / "tokenizer.model").write_bytes(out.getvalue())
    with pytest.raises(t12.T12Error):
        t12.Tokenizer(str(tmp_path))
    tf = __import__("importlib").import_module(t12.__name__ + ".tokenizer_files")
    tf.write_files(str(tmp_path), [b"a", b"b"], [], 0, 1)
    tok = t12.Tokenizer(str(tmp_path))                      # like the reference: the second backend gets its turn
    assert tok.type == 1
    tok.close()


@pytest.mark.parametrize("name", ["llama_like", "defaults"])
def test_arbitrary_unicode_text_equals_the_library(t12, tmp_path, name):
    """Property test (hypothesis): any Unicode text -- blanks of every kind, control characters, astral code points,
    the escaped-blank character itself -- encodes to the library's ids and decodes to the library's text."""
    hyp = pytest.importorskip("hypothesis")
    st = pytest.importorskip("hypothesis.strategies")
    proto, words = train(11, **CONFIGS[name])
    ours, sp = load_both(t12, tmp_path, proto)
    alphabet = st.one_of(st.sampled_from(list("abcdefghij éß \t\n" + SPACE + "<>0x/")), st.characters(blacklist_categories=("Cs",)))

    @hyp.settings(max_examples=300, deadline=None, suppress_health_check=list(hyp.HealthCheck))
    @hyp.given(text=st.text(alphabet=alphabet, max_size=60))
    def check(text):
        want = sp.encode(text)
        assert ours.tokenize(text)[1:] == want, (text, sp.encode(text, out_type=str))
        assert ours.detokenize(want) == sp.decode(want).encode(), text

    try:
        check()
    finally:
        ours.close()
