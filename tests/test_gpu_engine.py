"""GPU parity: the engine API (load_model / create_inference_state / forward / generate / sample)
against the CPU oracle's decode step on small random-init models."""
import importlib
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SMALL = dict(n_vocab=1024, n_embd=256, n_head=8, n_head_kv=2, n_layer=2, n_ff=512, n_ctx=256,
             rope_theta=500000.0, rms_norm_eps=1e-5)


@pytest.fixture(scope="module")
def synth(t12):
    return importlib.import_module("turbo_lossless_amd.synth")


@pytest.fixture(scope="module")
def modelio(t12):
    return importlib.import_module("turbo_lossless_amd.modelio")


def build_small(oracle, synth, cfg, seed=4000):
    """numpy model: N(0,.02) weights with outliers, norms near 1, embeddings N(0,.02)."""
    n, ff, hd = cfg["n_embd"], cfg["n_ff"], cfg["n_embd"] // cfg["n_head"]
    kv = cfg["n_head_kv"] * hd
    rng = np.random.default_rng(seed)
    s = [seed]

    def mk(M, K):
        s[0] += 1
        return oracle.pack(synth.weights_llm(M, K, s[0], p_outlier=2e-3))

    layers = []
    for _ in range(cfg["n_layer"]):
        layers.append(dict(attn_norm=(1 + 0.05 * rng.standard_normal(n)).astype(np.float32),
                           ffn_norm=(1 + 0.05 * rng.standard_normal(n)).astype(np.float32),
                           wq=mk(n, n), wk=mk(kv, n), wv=mk(kv, n), wo=mk(n, n),
                           w_gate=mk(ff, n), w_up=mk(ff, n), w_down=mk(n, ff)))
    embd = synth.weights_llm(cfg["n_vocab"], n, seed + 999, sigma=1.0, p_outlier=0)
    onorm = (1 + 0.05 * rng.standard_normal(n)).astype(np.float32)
    head = mk(cfg["n_vocab"], n)
    return embd, onorm, head, layers


@pytest.fixture(scope="module")
def small_model(t12, oracle, synth, modelio, tmp_path_factory):
    os.environ["TURBO_CTX"] = "256"
    embd, onorm, head, layers = build_small(oracle, synth, SMALL)
    path = str(tmp_path_factory.mktemp("model"))
    modelio.write_model_dir(path, SMALL, embd, onorm, head, layers)
    ref = oracle.RefModel(SMALL, embd, onorm, head, layers, max_seq=256)
    return path, ref


def test_forward_logits_match_oracle(t12, oracle, small_model):
    path, ref = small_model
    eng = t12.Engine.load(path, batch=1)
    try:
        toks = [5, 900, 17, 3, 1023, 44]
        for pos, tok in enumerate(toks):
            eng.forward([tok])
            got = eng.logits(SMALL["n_vocab"]).cpu().numpy()[0]
            want = ref.step(tok, pos)
            err = np.abs(got - want).max() / np.abs(want).max()
            assert err < 2e-2, (pos, err)        # bf16 activations between layers: ~1e-3 typical
            assert eng.positions() == [pos + 1]
    finally:
        eng.close()


def test_greedy_stream_identical_64_tokens(t12, oracle, small_model):
    """North star: greedy token streams identical for the first 64 tokens (fused GPU path vs the
    decode-then-fp32 CPU restatement)."""
    path, _ = small_model
    embd, onorm, head, layers = build_small(oracle, importlib.import_module("turbo_lossless_amd.synth"), SMALL)
    ref = oracle.RefModel(SMALL, embd, onorm, head, layers, max_seq=256)
    rng = np.random.default_rng(1)
    prompt = [int(t) for t in rng.integers(3, SMALL["n_vocab"], size=16)]
    want = ref.generate(prompt, 64)
    eng = t12.Engine.load(path, batch=1)
    try:
        got = eng.generate(prompt, 64)
    finally:
        eng.close()
    assert len(want) >= 32
    assert got == want


def test_batched_forward_equals_b1(t12, small_model):
    """B identical streams (the reference's batched mode) give B identical rows equal to the B = 1 logits
    up to the GEMV/GEMM summation order."""
    path, _ = small_model
    e1 = t12.Engine.load(path, batch=1)
    try:
        outs = []
        for tok in [9, 200, 31]:
            e1.forward([tok])
            outs.append(e1.logits(SMALL["n_vocab"]).clone())
    finally:
        e1.close()
    for B in (2, 5, 40):
        eb = t12.Engine.load(path, batch=B)
        try:
            for i, tok in enumerate([9, 200, 31]):
                eb.forward([tok] * B)
                lg = eb.logits(SMALL["n_vocab"])
                assert torch.equal(lg[0], lg[B - 1])
                err = (lg[0] - outs[i][0]).abs().max() / outs[i][0].abs().max()
                assert err < 5e-3, (B, i, float(err))
            assert eb.sample() == [int(lg[0].argmax())] * B
        finally:
            eb.close()


def test_fused_and_unfused_b1_paths_agree(t12, small_model):
    """TURBO_NO_FUSE=1 runs one launch per reference kernel; the default B = 1 path fuses norms, SiLU*mul,
    RoPE and the KV store into the linears / attention.  Same logits up to bf16 rounding flips."""
    path, _ = small_model
    outs = {}
    for flag in ("1", "0"):
        os.environ["TURBO_NO_FUSE"] = flag
        e = t12.Engine.load(path, batch=1)
        try:
            seq = []
            for tok in [9, 200, 31, 7]:
                e.forward([tok])
                seq.append(e.logits(SMALL["n_vocab"]).clone())
            outs[flag] = seq
        finally:
            e.close()
    os.environ.pop("TURBO_NO_FUSE")
    for a, b in zip(outs["0"], outs["1"]):
        assert float((a - b).abs().max() / b.abs().max()) < 1e-2
        assert int(a.argmax()) == int(b.argmax())


def test_loader_reads_files_bit_exact(t12, oracle, small_model, modelio):
    path, _ = small_model
    eng = t12.Engine.load(path, batch=1)
    try:
        for layer, which, name in [(0, 0, "layer.0.wq"), (1, 6, "layer.1.w_down"), (-1, 0, "output_proj")]:
            seg, K, P = eng.weight(layer, which)
            f = modelio.read_tensor(path, name)
            assert (seg.M, K, P, seg.base_exp) == (f.M, f.K, len(f.cols), f.base_exp)
            out = torch.empty((f.M, f.K), dtype=torch.int16, device="cuda")
            t12.check(t12.lib.t12_decompress(seg.sm, seg.gr, seg.base_exp, seg.row_off, seg.cols, seg.correct,
                                             out.data_ptr(), f.M, f.K, 1, t12.current_stream()))
            torch.cuda.synchronize()
            want = oracle.decode(oracle.Packed(f.M, f.K, f.base_exp, f.sm, f.gr, f.row_off, f.cols, f.correct, f.wrong))
            assert np.array_equal(out.cpu().numpy().view(np.uint16), want)
    finally:
        eng.close()


def test_load_errors(t12, small_model, tmp_path, modelio):
    assert not t12.lib.t12_engine_load(os.fsencode(str(tmp_path)), 0)          # no config.bin -> nullptr
    modelio.write_config(str(tmp_path), SMALL)
    assert not t12.lib.t12_engine_load(os.fsencode(str(tmp_path)), 0)          # no tok_embd.bin -> nullptr


def test_synthetic_model_save_load_roundtrip(t12, tmp_path):
    cfg = dict(SMALL, n_layer=1)
    a = t12.Engine.synthetic(cfg, seed=77, max_seq=128, p_outlier=2e-3)
    try:
        with pytest.raises(t12.T12Error, match="directory must exist"):
            a.save(str(tmp_path / "not" / "there"))
        a.save(str(tmp_path))
        toks = [4, 8, 15]
        la = []
        for t in toks:
            a.forward([t]); la.append(a.logits(cfg["n_vocab"]).clone())
        seg, K, P = a.weight(0, 4)
        assert P > 0
    finally:
        a.close()
    os.environ["TURBO_CTX"] = "128"
    b = t12.Engine.load(str(tmp_path), batch=1)
    try:
        for t, ref in zip(toks, la):
            b.forward([t])
            assert torch.equal(b.logits(cfg["n_vocab"]), ref)
    finally:
        b.close()


def _state_with_order(base, B, sequential):
    """A state on base's model whose greedy loop runs pipelined, or in the reference's sample-wait-forward order
    (TURBO_NO_PIPELINE, read when the state is created)."""
    if sequential:
        os.environ["TURBO_NO_PIPELINE"] = "1"
    try:
        return base.new_state(B)
    finally:
        os.environ.pop("TURBO_NO_PIPELINE", None)


@pytest.mark.parametrize("B", [1, 3])
def test_pipelined_decode_equals_step_by_step(t12, small_model, B):
    """decode_greedy enqueues step t + 1 on the device-resident ids before the host has read token t;
    the stream, the stop at id 2 and the positions left behind must equal the reference's order
    (sample, wait, forward), which TURBO_NO_PIPELINE=1 runs."""
    path, _ = small_model
    rng = np.random.default_rng(11)
    prompts = [[int(t) for t in rng.integers(3, SMALL["n_vocab"], size=5)] for _ in range(12)]
    base = t12.Engine.load(path, batch=1)
    engs = [_state_with_order(base, B, True), _state_with_order(base, B, False)]     # (they share the model's cache region)
    try:
        saw_eos = False
        for prompt in prompts:
            runs = []
            for eng in engs:
                toks = eng.generate(prompt, 40)
                runs.append((toks, eng.positions()))
            assert runs[0] == runs[1]
            saw_eos = saw_eos or len(runs[0][0]) < 40
            assert runs[0][1] == [len(prompt) + len(runs[0][0])] * B
        # decode() continues from the logits left behind, without the stop rule
        a = engs[0].generate(prompts[0], 8) + engs[0].decode(8)
        b = engs[1].generate(prompts[0], 8) + engs[1].decode(8)
        assert a == b and (len(a) == 16 or 2 in a or saw_eos)
    finally:
        for e in engs:
            e.close()
        base.close()


@pytest.mark.parametrize("B", [1, 2])
def test_stop_leaves_the_state_as_the_sequential_order_does(t12, small_model, B):
    """When a stop id ends the stream, the pipelined loop has already enqueued the forward on that id: positions are
    stepped back AND state->logits are the logits the stop id was sampled from (the loop alternates two logits
    buffers), so whatever the caller does next -- look at the logits, decode again -- matches the reference's order."""
    path, _ = small_model
    rng = np.random.default_rng(12)
    prompt = [int(t) for t in rng.integers(3, SMALL["n_vocab"], size=6)]
    base = t12.Engine.load(path, batch=1)
    seq, pipe = _state_with_order(base, B, True), _state_with_order(base, B, False)
    try:
        def prompt_in(e):
            for i, t in enumerate(prompt):
                e.set_positions([i] * B)
                e.forward([t] * B)
        prompt_in(seq)
        free_run = seq.decode(12)
        assert len(free_run) == 12
        stop = free_run[7]                                   # the stream must stop before its 8th token
        k = free_run.index(stop)
        results = []
        for e in (seq, pipe):
            prompt_in(e)
            got = e.decode_until(12, stop)
            lg = e.logits(SMALL["n_vocab"]).clone()
            again = e.decode_until(5, stop)                  # the same logits: the stop id comes first again
            results.append((got, e.positions(), lg, again, e.decode_until(3, -1)))
        assert results[0][0] == free_run[:k] and results[0][3] == []
        assert int(results[0][2][0].argmax()) == stop
        for a, b in zip(results[0], results[1]):
            assert torch.equal(a, b) if torch.is_tensor(a) else a == b
    finally:
        seq.close()
        pipe.close()
        base.close()


def test_stop_id_with_the_cache_exactly_full(t12, small_model):
    """The last cache row is written, the next sampled id is the stop id: the loop ends cleanly in both orders (the
    pipelined one must not enqueue a forward past the cache before it has looked at the id)."""
    path, _ = small_model
    rng = np.random.default_rng(13)
    base = t12.Engine.load(path, batch=1)
    seq, pipe = _state_with_order(base, 1, True), _state_with_order(base, 1, False)
    try:
        max_seq = t12.lib.t12_engine_max_seq(base.model)
        start = max_seq - 6
        tok0 = int(rng.integers(3, SMALL["n_vocab"]))
        seq.set_positions([start]); seq.forward([tok0])
        stream = seq.decode(5)                               # fills positions start+1 .. max_seq-1
        assert seq.positions() == [max_seq]
        stop = seq.sample()[0]                               # what comes next with the cache full
        outs = []
        for e in (seq, pipe):
            e.set_positions([start]); e.forward([tok0])
            outs.append((e.decode_until(8, stop), e.positions()))
        assert outs[0] == outs[1]
        assert outs[0][0] == stream[:stream.index(stop)] if stop in stream else outs[0] == (stream, [max_seq])
    finally:
        seq.close()
        pipe.close()
        base.close()


def test_two_states_on_their_own_streams_do_not_share_scratch(t12, small_model):
    """Two states of one model (own cache regions, own streams) decode past 256 positions -- where a B = 1 launch
    splits the context across workgroups and keeps partial results and arrival counters in library-owned scratch --
    with their forwards and argmax launches enqueued alternately and no synchronisation in between.  The scratch is
    per (device, stream), so each state's logits and tokens equal those of the same steps run alone."""
    path, _ = small_model
    rng = np.random.default_rng(21)
    n_prompt, n_steps = 300, 24
    prompts = [[int(t) for t in rng.integers(3, SMALL["n_vocab"], size=n_prompt)] for _ in range(2)]
    base = t12.Engine.load(path, batch=1)
    states = [base.new_state(1, per_sequence=400) for _ in range(2)]
    try:
        # alone: prompt, then greedy steps one state after the other
        alone_tokens, alone_logits = [], []
        for st, prompt in zip(states, prompts):
            st.set_positions([0])
            st.prefill_rows(prompt, 64)
            toks = []
            for _ in range(n_steps):
                t = st.sample()[0]
                toks.append(t)
                st.forward([t])
            alone_tokens.append(toks)
            alone_logits.append(st.logits(SMALL["n_vocab"]).clone())
        # together: the same steps, enqueued alternately
        for st, prompt in zip(states, prompts):
            st.set_positions([0])
            st.prefill_rows(prompt, 64)
        both = [[], []]
        for _ in range(n_steps):
            toks = [st.sample()[0] for st in states]        # (sample synchronises its own stream only)
            for i, st in enumerate(states):
                both[i].append(toks[i])
                st.forward([toks[i]])
        for i, st in enumerate(states):
            assert both[i] == alone_tokens[i]
            assert torch.equal(st.logits(SMALL["n_vocab"]), alone_logits[i])
    finally:
        for st in states:
            st.close()
        base.close()


def test_errors_come_back_as_codes_not_as_a_dead_process(t12, small_model):
    """Where the reference ends the process (a position past the cache: engine/inference.cpp:73,223,306 and its
    GPU_CHECK), the C face returns T12_EENGINE with the text in t12_last_error(), and the Python wrapper raises.
    Every condition here is found on the host before any kernel is launched."""
    path, _ = small_model
    base = t12.Engine.load(path, batch=1)
    two = base.new_state(2)
    try:
        max_seq = t12.lib.t12_engine_max_seq(base.model)
        base.set_positions([max_seq])
        arr = (t12.C.c_int * 1)(5)
        assert t12.lib.t12_engine_forward(base.state, arr) == -3
        assert b"exceeds the KV cache" in t12.lib.t12_last_error()
        with pytest.raises(t12.T12Error, match="exceeds the KV cache"):
            base.forward([5])
        base.set_positions([0])
        with pytest.raises(t12.T12Error, match="outside the cache"):
            base.shift_context(current_pos=4, discard=9)
        with pytest.raises(t12.T12Error, match="outside the batch"):
            two.prefill(2, [3, 4, 5])
        with pytest.raises(t12.T12Error, match="batch size 1"):
            two.prefill_rows([3, 4, 5], 4)
        with pytest.raises(t12.T12Error, match="batch size 1"):
            two.chat_turn(0, [3, 4], 4, 1, 2)
        with pytest.raises(t12.T12Error, match="exceeds the KV cache"):
            base.prefill_rows(list(range(3, 3 + max_seq + 1)), 8)
        # the refusals above launched nothing: the state still decodes
        base.set_positions([0])
        base.forward([7])
        assert len(base.decode(4)) == 4
    finally:
        two.close()
        base.close()


def test_states_give_their_stream_buffers_back(t12, small_model):
    """A state's stream carries library buffers (K-split sums, argmax partials, context-split scratch, sampler ids);
    free_inference_state hands them back (t12_release_stream), so states that come and go leave device memory where it
    was.  After a release the stream works as before (new buffers on first use)."""
    path, _ = small_model
    base = t12.Engine.load(path, batch=1)
    try:
        def cycle():
            for B in (1, 8, 64):
                e = base.new_state(B)
                e.set_positions([0] * B)
                e.forward([5] * B)
                e.decode_all(3)
                e.sample()
                e.close()
        cycle()
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        for _ in range(6):
            cycle()
        torch.cuda.synchronize()
        assert free0 - torch.cuda.mem_get_info()[0] < (4 << 20)
        base.set_positions([0])
        base.forward([9])
        want = base.decode(4)
        t12.check(t12.lib.t12_release_stream(t12.lib.t12_engine_stream(base.state)), "release")
        base.set_positions([0])
        base.forward([9])
        assert base.decode(4) == want
    finally:
        base.close()
