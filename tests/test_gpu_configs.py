"""GPU parity at the FULL sizes the benchmark configurations name, through the C ABI vs the CPU oracle:

  * escape-heavy 2560 x 10240 (decode-only bit-exact, decode-GEMV, decode+GEMM at B = 64);
  * the Llama-3.1-8B layer shapes at B in {16, 64, 256}: down 4096 x 14336, the three-segment
    q|k|v launch (4096 + 1024 + 1024 rows x 4096), gate|up (2 x 14336 rows x 4096);
  * a decoder at the full widths (hidden 4096, FFN 14336, 32 / 8 heads of 128, vocabulary 128256), two layers:
    logits against the CPU decode step, the greedy stream against the CPU decode loop, B = 256 rows against
    B = 1, fused launches against one launch per reference kernel.

The GPU computes every output; the oracle checks all rows of the smaller products and, for the big ones, the rows
of four 128-row blocks per tensor (first, last, and two across tile boundaries in between) to bound host time --
the GPU result of ALL rows is additionally checked for finiteness and against a checksum identity
(sum over rows of out[b, :] = (sum of the weight rows) . x[b], computed from the decoded tensor in float64).
"""
import importlib
import os

import numpy as np
import pytest
import torch

from gpu_util import dev, rel_err, to_dev_bits

pytestmark = pytest.mark.gpu
TOL = 1e-4           # target 1e-2 relative; fp32 accumulation on both sides gives ~1e-6


@pytest.fixture(scope="module")
def synth(t12):
    return importlib.import_module("turbo_lossless_amd.synth")


def sub_rows(oracle, p, r0, r1):
    """Rows [r0, r1) of a packed tensor as a packed tensor of its own (K even: rows start on nibble-byte
    boundaries; the CSR slice is rebased)."""
    assert p.K % 2 == 0
    K = p.K
    a, b = int(p.row_off[r0]), int(p.row_off[r1])
    return oracle.Packed(r1 - r0, K, p.base_exp, p.sm[r0 * K:r1 * K], p.gr[r0 * K // 2:r1 * K // 2],
                         (p.row_off[r0:r1 + 1] - a).astype(np.int32), p.cols[a:b], p.correct[a:b], p.wrong[a:b])


def row_blocks(M):
    if M <= 1024:
        return [(0, M)]
    mid = (M // 2 // 128) * 128
    return [(0, 128), (mid - 64, mid + 64), (mid + 192 - 3, mid + 192 + 125), (M - 128, M)]


_COLSUM = {}


def check_rows(oracle, p, X, got):
    """got [B, M] (GPU) against the oracle on the row blocks, plus the all-rows column-sum identity."""
    assert np.isfinite(got).all()
    for r0, r1 in row_blocks(p.M):
        ref = oracle.gemm(sub_rows(oracle, p, r0, r1), X)
        assert rel_err(got[:, r0:r1], ref) < TOL, (r0, r1)
    if id(p) not in _COLSUM:
        _COLSUM[id(p)] = (p, oracle.bf16_bits_to_f32(oracle.decode(p)).sum(axis=0, dtype=np.float64))   # [K]
    colsum = _COLSUM[id(p)][1]
    want = oracle.bf16_bits_to_f32(X).astype(np.float64) @ colsum
    have = got.astype(np.float64).sum(axis=1)
    scale = np.abs(got).astype(np.float64).sum(axis=1)
    assert np.all(np.abs(have - want) <= 1e-5 * scale + 1e-6)


# ------------------------------------------------------------------------------ escape-heavy 2560 x 10240
@pytest.fixture(scope="module")
def c3_tensor(oracle, synth):
    w = synth.weights_diffusion(2560, 10240, seed=3003)
    p = oracle.pack(w)
    assert 0.0015 < p.P / w.size < 0.01 and np.all(np.diff(p.row_off) > 0)      # every row holds escapes
    return w, p


def test_c3_2560x10240_decode_bit_exact(t12, oracle, c3_tensor):
    w, p = c3_tensor
    dt = t12.DeviceTensor12.from_packed(p, dev())
    pat = t12.decompress(dt, patched=True)
    un = t12.decompress(dt, patched=False)
    torch.cuda.synchronize()
    assert np.array_equal(pat.cpu().numpy().view(np.uint16), w)
    assert np.array_equal(un.cpu().numpy().view(np.uint16), oracle.decode(p, patched=False))


def test_c3_2560x10240_gemv_and_gemm_b64(t12, oracle, synth, c3_tensor):
    _, p = c3_tensor
    dt = t12.DeviceTensor12.from_packed(p, dev())
    x = synth.activations(1, p.K, seed=3004)
    (g1,) = t12.gemv(dt, to_dev_bits(x[0]))
    X = synth.activations(64, p.K, seed=3005)
    (g64,) = t12.gemm(dt, to_dev_bits(X).reshape(X.shape))
    torch.cuda.synchronize()
    assert rel_err(g1.cpu().numpy(), oracle.gemv(p, x[0])) < TOL
    assert rel_err(g64.cpu().numpy(), oracle.gemm(p, X)) < TOL


# ----------------------------------------------------------------------------- Llama-3.1-8B layer shapes
@pytest.fixture(scope="module")
def llama_layer(oracle, synth):
    shapes = dict(wq=(4096, 4096), wk=(1024, 4096), wv=(1024, 4096), gate=(14336, 4096), up=(14336, 4096),
                  down=(4096, 14336))
    out = {}
    for i, (name, (M, K)) in enumerate(shapes.items()):
        out[name] = oracle.pack(synth.weights_llm(M, K, seed=2000 + i))
        assert out[name].P > 0
    return out


@pytest.fixture(scope="module")
def llama_layer_dev(t12, llama_layer):
    return {k: t12.DeviceTensor12.from_packed(p, dev()) for k, p in llama_layer.items()}


@pytest.mark.parametrize("B", [16, 64, 256])
def test_c2_down_full_size(t12, oracle, synth, llama_layer, llama_layer_dev, B):
    X = synth.activations(B, 14336, seed=2100 + B)
    (got,) = t12.gemm(llama_layer_dev["down"], to_dev_bits(X).reshape(X.shape))
    torch.cuda.synchronize()
    check_rows(oracle, llama_layer["down"], X, got.cpu().numpy())


@pytest.mark.parametrize("B", [16, 64, 256])
def test_c2_qkv_three_segments_full_size(t12, oracle, synth, llama_layer, llama_layer_dev, B):
    """One launch, three tensors, outputs in column slices of one [B, 6144] buffer."""
    X = synth.activations(B, 4096, seed=2200 + B)
    big = torch.full((B, 6144), float("nan"), device=dev())
    names = ["wq", "wk", "wv"]
    outs = [big[:, 0:4096], big[:, 4096:5120], big[:, 5120:6144]]
    t12.gemm([llama_layer_dev[n] for n in names], to_dev_bits(X).reshape(X.shape), outs=outs)
    torch.cuda.synchronize()
    h = big.cpu().numpy()
    for n, (c0, c1) in zip(names, [(0, 4096), (4096, 5120), (5120, 6144)]):
        check_rows(oracle, llama_layer[n], X, h[:, c0:c1])


@pytest.mark.parametrize("B", [16, 64, 256])
def test_c2_gate_up_full_size(t12, oracle, synth, llama_layer, llama_layer_dev, B):
    X = synth.activations(B, 4096, seed=2300 + B)
    g, u = t12.gemm([llama_layer_dev["gate"], llama_layer_dev["up"]], to_dev_bits(X).reshape(X.shape))
    torch.cuda.synchronize()
    check_rows(oracle, llama_layer["gate"], X, g.cpu().numpy())
    check_rows(oracle, llama_layer["up"], X, u.cpu().numpy())


@pytest.mark.parametrize("B", [64, 256])
def test_c2_o_alone_full_size(t12, oracle, synth, llama_layer, llama_layer_dev, B):
    """O 4096 x 4096 as a launch of its own: 32 row tiles, the launch with the most K splits of the four layer shapes."""
    import ctypes as C
    X = synth.activations(B, 4096, seed=2500 + B)
    Xd = to_dev_bits(X).reshape(X.shape)
    (got,) = t12.gemm(llama_layer_dev["wq"], Xd)
    torch.cuda.synchronize()
    check_rows(oracle, llama_layer["wq"], X, got.cpu().numpy())
    # the split the library chose for this launch, and its partial sums added up on the host
    out = torch.full((B, 4096), float("nan"), device=dev())
    part = t12.GemmPartials()
    segs = t12._seg_array([llama_layer_dev["wq"].segment(out)])
    t12.check(t12.lib.t12_gemm_deferred(segs, 1, Xd.data_ptr(), 4096, 4096, 4096, B, C.byref(part), t12.current_stream()))
    torch.cuda.synchronize()
    assert part.nsplit >= 4
    ws = torch.empty(part.nsplit * part.split_stride, dtype=torch.float32, device=dev())
    assert t12._hip_memcpy_d2d(ws.data_ptr(), part.ws, ws.numel() * 4) == 0
    tot = ws.view(part.nsplit, B, part.ld)[:, :, :4096].sum(dim=0)
    assert rel_err(tot.cpu().numpy(), got.cpu().numpy()) < 1e-6


def test_c2_b1_full_size_segments(t12, oracle, synth, llama_layer, llama_layer_dev):
    """B = 1 of the same launches through the decode-GEMV: q|k|v, gate|up, down."""
    x = synth.activations(1, 4096, seed=2400)[0]
    xf = synth.activations(1, 14336, seed=2401)[0]
    q, k, v = t12.gemv([llama_layer_dev[n] for n in ("wq", "wk", "wv")], to_dev_bits(x))
    g, u = t12.gemv([llama_layer_dev["gate"], llama_layer_dev["up"]], to_dev_bits(x))
    (d,) = t12.gemv(llama_layer_dev["down"], to_dev_bits(xf))
    torch.cuda.synchronize()
    for got, n, xx in [(q, "wq", x), (k, "wk", x), (v, "wv", x), (g, "gate", x), (u, "up", x), (d, "down", xf)]:
        assert rel_err(got.cpu().numpy(), oracle.gemv(llama_layer[n], xx)) < TOL, n


# -------------------------------------------------------------- decoder at the full Llama-3.1-8B widths
FULL = dict(n_vocab=128256, n_embd=4096, n_head=32, n_head_kv=8, n_layer=2, n_ff=14336, n_ctx=256,
            rope_theta=500000.0, rms_norm_eps=1e-5)


@pytest.fixture(scope="module")
def full_width_model(t12, oracle, tmp_path_factory):
    """Two layers at full width, generated and packed on the GPU, written in the converter's layout and read back
    for the CPU decode step (so the loader, the GPU packer and the engine see the same bytes)."""
    modelio = importlib.import_module("turbo_lossless_amd.modelio")
    path = str(tmp_path_factory.mktemp("full_width"))
    eng = t12.Engine.synthetic(FULL, seed=4100, max_seq=256)
    try:
        eng.save(path)
    finally:
        eng.close()
    assert t12.check_model_dir(path) == ""

    def tensor(prefix):
        t = modelio.read_tensor(path, prefix)
        return oracle.Packed(t.M, t.K, t.base_exp, t.sm, t.gr, t.row_off, t.cols, t.correct, t.wrong)

    layers = []
    for i in range(FULL["n_layer"]):
        L = {k: tensor("layer.%d.%s" % (i, k)) for k in modelio.TENSORS}
        L["attn_norm"] = np.fromfile(os.path.join(path, "layer.%d.attn_norm.bin" % i), np.float32)
        L["ffn_norm"] = np.fromfile(os.path.join(path, "layer.%d.ffn_norm.bin" % i), np.float32)
        layers.append(L)
    embd = np.fromfile(os.path.join(path, "tok_embd.bin"), np.uint16).reshape(FULL["n_vocab"], FULL["n_embd"])
    onorm = np.fromfile(os.path.join(path, "output_norm.bin"), np.float32)
    head = tensor("output_proj")
    os.environ["TURBO_CTX"] = "256"
    return path, (embd, onorm, head, layers)


def test_c4_full_width_logits_and_greedy_stream(t12, oracle, full_width_model):
    """B = 1 at full widths: logits of the prompt positions against the CPU decode step, then the greedy stream
    of 64 tokens identical to the CPU decode loop's."""
    path, parts = full_width_model
    ref = oracle.RefModel(FULL, *parts, max_seq=256)
    rng = np.random.default_rng(4101)
    prompt = [int(t) for t in rng.integers(3, FULL["n_vocab"], size=6)]
    eng = t12.Engine.load(path, batch=1)
    try:
        want_logits = None
        for pos, tok in enumerate(prompt):
            eng.forward([tok])
            got = eng.logits(FULL["n_vocab"]).cpu().numpy()[0]
            want_logits = ref.step(tok, pos)
            assert rel_err(got, want_logits) < 2e-2, pos           # bf16 activations between layers
        got_stream = eng.decode(64, stop_on_eos=True)
    finally:
        eng.close()
    want_stream, logits, pos = [], want_logits, len(prompt)
    for _ in range(64):
        nxt = oracle.argmax_first(logits)
        if nxt == 2:
            break
        want_stream.append(nxt)
        logits = ref.step(nxt, pos)
        pos += 1
    assert len(want_stream) >= 32
    assert got_stream == want_stream


@pytest.mark.parametrize("batch,variant", [(1, ""), (8, ""), (64, "_nv")])
def test_c4_full_width_reference_host_engine_on_this_builds_launchers(t12, full_width_model, batch, variant, capsys):
    """The reference's host engine (engine/model.cpp + inference.cpp + sampler.cpp compiled unchanged by oracle/Makefile,
    target ref_engine) linked with libturbo12.so, on the full-width model directory: its loader reads what this build's
    save_model wrote, its forward_b1 / forward_b8 issue this build's launchers, and its greedy stream of 48 tokens is
    this engine's (which the test above ties to the CPU decode step).  Prints both decode rates.
    variant "_nv": the build of the same files with their other branch selected (oracle/Makefile); at 64 rows its
    forward_batch_tiled calls nv_launch_split12_fused_gemm_async for the tensors of 4096 rows and more,
    nv_launch_split12_cublas_batch_async for wk / wv, and the corrections as nv_launch_patches_batch_async."""
    import subprocess
    import time
    driver = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref",
                          "reference_engine_driver" + variant)
    if not os.path.exists(driver):
        pytest.skip("oracle/_ref/reference_engine_driver%s not built (needs the reference tree at build time)" % variant)
    path, _ = full_width_model
    rng = np.random.default_rng(4102)
    prompt = [int(t) for t in rng.integers(3, FULL["n_vocab"], size=6)]
    n_new = 48
    env = dict(os.environ, TURBO_CTX="256", REF_DRIVER_TIMED="1")
    env.pop("TURBO_FAST", None)
    r = subprocess.run([driver, path, str(batch), str(n_new)] + [str(t) for t in prompt], capture_output=True,
                       timeout=170, env=env)
    assert r.returncode == 0, (r.returncode, r.stdout[-1500:], r.stderr[-1500:])
    lines = r.stdout.split(b"\n")
    got = [int(t) for t in [l for l in lines if l.startswith(b"tokens:")][0].split()[1:]]
    sec, calls = [l for l in lines if l.startswith(b"timed:")][0].split()[1:]
    eng = t12.Engine.load(path, batch=batch)
    try:
        want = eng.generate(prompt, n_new)
        t0 = time.perf_counter()
        again = eng.generate(prompt, n_new)
        own_sec = time.perf_counter() - t0
    finally:
        eng.close()
    assert again == want and len(want) >= 16
    assert got == want
    with capsys.disabled():
        print("\n[2 layers at Llama-3.1-8B widths, B=%d%s] reference host code over this build's launchers: %.2f ms per "
              "forward; this build's engine: %.2f ms per forward" % (batch, variant, float(sec) / int(calls) * 1e3,
                                                                    own_sec / (len(prompt) + len(want)) * 1e3), flush=True)



def test_c4_full_width_b256_rows_equal_b1(t12, full_width_model):
    """256 lock-step copies through the decode+GEMM kernels give 256 identical rows that agree with the B = 1
    decode-GEMV logits up to the summation order."""
    path, _ = full_width_model
    toks = [9, 70000, 31, 128255]
    e1 = t12.Engine.load(path, batch=1)
    try:
        outs = []
        for tok in toks:
            e1.forward([tok])
            outs.append(e1.logits(FULL["n_vocab"]).clone())
    finally:
        e1.close()
    for B in (16, 256):
        eb = t12.Engine.load(path, batch=B)
        try:
            for i, tok in enumerate(toks):
                eb.forward([tok] * B)
                lg = eb.logits(FULL["n_vocab"])
                assert torch.equal(lg, lg[0:1].expand_as(lg)), (B, i)
                err = (lg[0] - outs[i][0]).abs().max() / outs[i][0].abs().max()
                assert float(err) < 2e-2, (B, i, float(err))
                assert int(lg[0].argmax()) == int(outs[i][0].argmax())
        finally:
            eb.close()


def test_c4_full_width_fused_equals_unfused_stream(t12, full_width_model):
    """The 5-launch-per-layer decode step against one launch per reference kernel (TURBO_NO_FUSE=1): the same
    64 greedy tokens."""
    path, _ = full_width_model
    rng = np.random.default_rng(4102)
    prompt = [int(t) for t in rng.integers(3, FULL["n_vocab"], size=8)]
    streams = []
    for nofuse in ("0", "1"):
        os.environ["TURBO_NO_FUSE"] = nofuse
        try:
            eng = t12.Engine.load(path, batch=1)
        finally:
            del os.environ["TURBO_NO_FUSE"]
        try:
            for i, t in enumerate(prompt):
                eng.forward([t])
            streams.append(eng.decode(64, stop_on_eos=False))
        finally:
            eng.close()
    assert len(streams[0]) == 64 and streams[0] == streams[1]


def test_loader_escape_tables_match_oracle(t12, oracle, full_width_model):
    """escape_row_base / escape_vals / patch_nonempty_rows built by load_compressed (engine/model.cpp:86-160) read
    back from the device and compared with the oracle's brute-force tables, for every tensor of layer 0 and
    the output projection."""
    path, (embd, onorm, head, layers) = full_width_model
    eng = t12.Engine.load(path, batch=1)
    try:
        cases = [(0, i, layers[0][n]) for i, n in enumerate(("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"))]
        cases.append((-1, 0, head))
        for layer, which, p in cases:
            rb, vals, ne, n_ne = eng.weight_tables(layer, which)
            want_rb, _, want_vals, want_ne = oracle.escape_tables(p)
            assert p.P > 0 and rb and vals and ne

            def pull(ptr, n, dt):
                out = torch.empty(n, dtype=dt, device=dev())
                assert t12._hip_memcpy_d2d(out.data_ptr(), ptr, n * out.element_size()) == 0
                return out.cpu().numpy()
            assert np.array_equal(pull(rb, p.M, torch.int32), want_rb), (layer, which)
            assert np.array_equal(pull(vals, p.P, torch.int16), want_vals), (layer, which)
            assert n_ne == len(want_ne)
            assert np.array_equal(pull(ne, n_ne, torch.int32), want_ne), (layer, which)
    finally:
        eng.close()


# ------------------------------------------------------- decoder at full depth: 32 layers, 128-id prompt, 256 tokens
def test_c4_full_depth_streams(t12):
    """BASELINE config 4 as bench.py builds it: 32 layers at full widths, a prompt of 128 random ids, 256 greedy
    tokens, a 2048-token cache.  No CPU decode loop is fast enough for this size, so the checks are properties.

    What can be asked of two correct implementations here: this random-init network (N(0, 0.02) weights with 3e-4
    outliers of N(0, 8)) amplifies rounding noise.  Measured between the B = 1 step and the B = 256 step on the same
    token stream, median relative logit difference by depth: 2e-4 (1 layer), 6e-4 (2), 2.5e-3 (4), 9e-3 (8),
    1.5e-2 (16), 2.3e-2 (32), with single steps far above the median (one step of 64 reaches 0.5 of the logit
    scale after four layers, where the 17-row decode+GEMM path agrees with the CPU decode step to 4e-3 and the
    decode-GEMV path does not; every attention output of that run, in every kernel form, is within bf16 rounding of
    a float64 evaluation of the same cache).  So free-running streams of two summation orders part at the first
    near-tie, and the comparison is made on ONE stream, statistically:
      * B = 1 fused: the pipelined decode loop returns exactly the ids of forward + argmax step by step (same kernels);
      * B = 1 TURBO_NO_FUSE and B = 256 (lock-step rows through the decode+GEMM kernels) are fed the fused stream:
        logits finite; cosine similarity with the fused logits >= 0.99 on at least 90 % of the steps with a median
        >= 0.997 (measured: B = 1 unfused 0.99973, B = 256 0.99899); the same argmax on at least 90 % of the steps;
      * B = 256: all 256 rows identical (checked every 32 steps); its free-running stream equals the fused stream up to
        the first step where its replay's argmax differs."""
    cfg = dict(FULL, n_layer=32, n_ctx=2048)
    V = cfg["n_vocab"]
    rng = np.random.default_rng(4001)
    prompt = [int(t) for t in rng.integers(3, V, size=128)]
    n_gen = 256
    eng = t12.Engine.synthetic(cfg, seed=4000, max_seq=2048, batch=1)
    try:
        def prefill(e, B):
            for i, t in enumerate(prompt):
                e.set_positions([i] * B)
                e.forward([t] * B)

        # fused, step by step: the stream and its logits
        prefill(eng, 1)
        fused, LF = [], torch.empty((n_gen, V), dtype=torch.float32, device=dev())
        for s_ in range(n_gen):
            row = eng.logits(V)[0]
            LF[s_] = row
            tok = int(row.argmax())
            fused.append(tok)
            eng.set_positions([len(prompt) + s_])
            eng.forward([tok])
        assert bool(torch.isfinite(LF).all())
        prefill(eng, 1)
        assert eng.decode(n_gen, stop_on_eos=False) == fused          # the pipelined loop

        def replay(e, B, rows_every):
            """Feeds the fused stream; returns the step of the first argmax disagreement (n_gen if none)."""
            prefill(e, B)
            same, first, cos = 0, n_gen, []
            for s_, tok in enumerate(fused):
                lg = e.logits(V)
                if s_ % rows_every == 0 or s_ == n_gen - 1:
                    assert torch.equal(lg, lg[0:1].expand_as(lg)), s_
                row = lg[0]
                assert bool(torch.isfinite(row).all()), s_
                cos.append(float(torch.dot(row, LF[s_]) / (row.norm() * LF[s_].norm())))
                if int(row.argmax()) == tok:
                    same += 1
                else:
                    first = min(first, s_)
                e.set_positions([len(prompt) + s_] * B)
                e.forward([tok] * B)
            cos = np.array(cos)
            print("replay B=%d: cos >= 0.99 on %.3f of the steps, median %.5f, min %.3f, same argmax %d / %d, first miss at %d"
                  % (B, (cos >= 0.99).mean(), np.median(cos), cos.min(), same, n_gen, first), flush=True)
            assert (cos >= 0.99).mean() >= 0.9 and np.median(cos) >= 0.997, (B, float(np.median(cos)), float(cos.min()))
            assert same >= n_gen * 9 // 10, (B, same)
            return first

        os.environ["TURBO_NO_FUSE"] = "1"
        try:
            e2 = eng.new_state(1)
        finally:
            del os.environ["TURBO_NO_FUSE"]
        try:
            replay(e2, 1, 1)
        finally:
            e2.close()

        e256 = eng.new_state(256)
        try:
            first = replay(e256, 256, 32)
            prefill(e256, 256)
            s256 = e256.decode(n_gen, stop_on_eos=False)
            assert len(s256) == n_gen and s256[:first] == fused[:first]
        finally:
            e256.close()
    finally:
        eng.close()
