"""GPU parity of the interactive-loop extensions of the engine -- shift_context and chat_turn, the reference's
engine/main.cpp:139-213 as functions -- against the CPU decode step driven through the same turn logic."""
import importlib
import os

import numpy as np
import pytest

from test_gpu_engine import SMALL, build_small

pytestmark = pytest.mark.gpu
V = SMALL["n_vocab"]
CTX = 160
BOS, EOS = 1, 2


@pytest.fixture(scope="module")
def model(t12, oracle, tmp_path_factory):
    os.environ["TURBO_CTX"] = str(CTX)
    synth = importlib.import_module("turbo_lossless_amd.synth")
    modelio = importlib.import_module("turbo_lossless_amd.modelio")
    parts = build_small(oracle, synth, SMALL)
    path = str(tmp_path_factory.mktemp("chat_model"))
    modelio.write_model_dir(path, SMALL, *parts)
    return path, (SMALL,) + tuple(parts)


def load(t12, path, **kw):
    os.environ["TURBO_CTX"] = str(CTX)          # read by load_model (cache positions of the model's region)
    return t12.Engine.load(path, **kw)


def rel(a, b):
    return float(np.abs(a - b).max() / np.abs(b).max())


def shift_ref(ref, current_pos, discard):
    keep = current_pos - discard
    for arr in (ref.kc, ref.vc, ref.ks, ref.vs):
        arr[:, :keep] = arr[:, discard:current_pos].copy()


class RefChat:
    """engine/main.cpp:139-213 over the oracle's decode step."""

    def __init__(self, ref, max_seq):
        self.ref, self.max_seq, self.pos, self.logits = ref, max_seq, 0, None

    def turn(self, tokens, max_tokens, oracle):
        tokens = list(tokens)
        if self.pos > 0 and tokens and tokens[0] == BOS:
            tokens = tokens[1:]
        discard = 0
        if self.pos + len(tokens) + max_tokens + 64 > self.max_seq or self.pos > 1024:
            discard = self.pos // 2
            shift_ref(self.ref, self.pos, discard)
            self.pos -= discard
        for t in tokens:
            self.logits = self.ref.step(int(t), self.pos)
            self.pos += 1
        out = []
        for _ in range(max_tokens):
            nxt = oracle.argmax_first(self.logits)
            if nxt in (EOS, BOS):
                break
            out.append(nxt)
            self.logits = self.ref.step(nxt, self.pos)
            self.pos += 1
        self.logits = self.ref.step(EOS if EOS > 0 else 2, self.pos)
        self.pos += 1
        return out, discard


def test_shift_context_moves_rows_like_the_reference_loop(t12, oracle, model):
    """After the shift the next token attends to the kept rows at their new places: logits equal the CPU step on
    arrays shifted the same way.  Odd and even row counts (an odd count makes source and destination of a single
    copy overlap), discard 1, discard = everything but one row, discard 0."""
    path, parts = model
    rng = np.random.default_rng(31)
    for n_ctx, discard in [(21, 10), (20, 10), (9, 1), (9, 8), (7, 0), (33, 5)]:
        eng = load(t12, path, batch=1)
        try:
            ref = oracle.RefModel(*parts, max_seq=CTX)
            toks = [int(x) for x in rng.integers(3, V, size=n_ctx)]
            for pos, t in enumerate(toks):
                eng.forward([t])
                ref.step(t, pos)
            eng.shift_context(n_ctx, discard)
            shift_ref(ref, n_ctx, discard)
            pos = n_ctx - discard
            eng.set_positions([pos])
            for t in [int(x) for x in rng.integers(3, V, size=3)]:
                eng.forward([t])
                want = ref.step(t, pos)
                pos += 1
                assert rel(eng.logits(V).cpu().numpy()[0], want) < 2e-2, (n_ctx, discard)
            assert eng.positions() == [pos]
        finally:
            eng.close()


def test_shift_context_of_one_sequence_leaves_the_others(t12, oracle, model):
    path, parts = model
    rng = np.random.default_rng(32)
    B, T = 3, 11
    streams = rng.integers(3, V, size=(B, T))
    eng = load(t12, path, batch=B, per_sequence=48)
    try:
        refs = [oracle.RefModel(*parts, max_seq=48) for _ in range(B)]
        for t in range(T):
            eng.forward(streams[:, t])
            for b in range(B):
                refs[b].step(int(streams[b, t]), t)
        eng.shift_context(T, 4, seq=1)
        shift_ref(refs[1], T, 4)
        pos = [T, T - 4, T]
        eng.set_positions(pos)
        nxt = rng.integers(3, V, size=B)
        eng.forward(nxt)
        got = eng.logits(V).cpu().numpy()
        for b in range(B):
            assert rel(got[b], refs[b].step(int(nxt[b]), pos[b])) < 2e-2, b
    finally:
        eng.close()


def test_chat_turns_with_context_shifts_equal_the_reference_loop(t12, oracle, model):
    """Sixteen turns on a 160-position cache: BOS only opens the first turn, every turn's end-of-turn id enters the
    context, and from the fifth turn on the older half of the context is discarded first (odd and even counts)."""
    path, parts = model
    rng = np.random.default_rng(33)
    eng = load(t12, path, batch=1)
    try:
        chat = RefChat(oracle.RefModel(*parts, max_seq=CTX), CTX)
        pos, shifts = 0, 0
        for turn in range(16):
            tokens = [BOS] + [int(x) for x in rng.integers(3, V, size=4 + turn % 3)]
            max_tokens = 9 + turn % 2
            want, want_discard = chat.turn(tokens, max_tokens, oracle)
            got, pos, discarded = eng.chat_turn(pos, tokens, max_tokens, BOS, EOS)
            assert got == want, turn
            assert (pos, discarded) == (chat.pos, want_discard), turn
            assert eng.positions() == [pos]
            shifts += discarded > 0
        assert shifts >= 2
    finally:
        eng.close()


def test_batched_prompt_pass_of_a_batch_one_state(t12, oracle, model):
    """prefill_rows: 37 prompt tokens, 16 per pass (16 + 16 + 5), into the batch-1 state's own cache region through a helper
    state; the logits equal the CPU step token by token to rounding, the cache serves the decode that follows, and
    a second prompt continues from the new position."""
    path, parts = model
    rng = np.random.default_rng(34)
    eng = load(t12, path, batch=1)
    try:
        ref = oracle.RefModel(*parts, max_seq=CTX)
        pos = 0
        for n, rows in [(37, 16), (1, 16), (9, 4), (5, 1)]:
            toks = [int(x) for x in rng.integers(3, V, size=n)]
            for t in toks:
                want = ref.step(t, pos)
                pos += 1
            eng.prefill_rows(toks, rows)
            assert eng.positions() == [pos]
            assert rel(eng.logits(V).cpu().numpy()[0], want) < 2e-2, (n, rows)
            got = eng.decode(3)
            for g in got:
                assert g == oracle.argmax_first(want)
                want = ref.step(g, pos)
                pos += 1
            assert eng.positions() == [pos]
    finally:
        eng.close()


def test_chat_turns_with_batched_prompts(t12, oracle, model):
    path, parts = model
    rng = np.random.default_rng(35)
    eng = load(t12, path, batch=1)
    try:
        chat = RefChat(oracle.RefModel(*parts, max_seq=CTX), CTX)
        pos = 0
        for turn in range(7):
            tokens = [BOS] + [int(x) for x in rng.integers(3, V, size=6 + 3 * (turn % 3))]
            want, want_discard = chat.turn(tokens, 8, oracle)
            got, pos, discarded = eng.chat_turn(pos, tokens, 8, BOS, EOS, prompt_rows=8)
            assert got == want, turn
            assert (pos, discarded) == (chat.pos, want_discard), turn
    finally:
        eng.close()


def test_text_in_text_out(t12, oracle, model, tmp_path):
    """tokenize -> chat_turn -> detokenize_one over a tokenizer whose ids fit the model's vocabulary."""
    tf = importlib.import_module("turbo_lossless_amd.tokenizer_files")
    path, parts = model
    table = tf.bytes_to_unicode()
    toks = [b"<unk>", b"<s>", b"</s>"] + [table[b].encode() for b in range(256)]
    merges = [(table[ord("h")], table[ord("i")]), (table[ord(" ")], table[ord("t")])]
    toks += [(a + b).encode() for a, b in merges]
    toks += [b"w%d" % i for i in range(len(toks), V)]          # every id the model can emit has a text
    tf.write_files(str(tmp_path), toks, merges, BOS, EOS, table)
    tok = t12.Tokenizer(str(tmp_path))
    eng = load(t12, path, batch=1)
    try:
        ids = tok.tokenize("hi there")
        assert ids[0] == BOS and len(ids) == 1 + 1 + 1 + 4      # <s>, "hi", " t", h e r e
        chat = RefChat(oracle.RefModel(*parts, max_seq=CTX), CTX)
        want, _ = chat.turn(ids, 12, oracle)
        got, pos, _ = eng.chat_turn(0, ids, 12, tok.bos_id, tok.eos_id)
        assert got == want and pos == chat.pos
        from oracle.tokenizer_oracle import RefTokenizer
        rt = RefTokenizer(str(tmp_path))
        text = b"".join(tok.detokenize_one(i) for i in got)
        assert text == b"".join(rt.detokenize_one(i) for i in got) and len(text) >= len(got)
    finally:
        eng.close()
        tok.close()
