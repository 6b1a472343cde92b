"""The reference's own command-line front end driving this engine on the GPU.

oracle/_ref/reference_cli is the reference's engine/main.cpp, compiled unchanged (oracle/Makefile, target ref_cli)
against include/turbo/*.h and linked with libturbo12.so: every call it makes -- load_model, load_tokenizer, tokenize,
create_inference_state, generate, forward, sample_greedy, detokenize_one, the fields it reads and writes
(state->positions, state->logits, state->stream, model->kv_cache_*, model->max_seq_len, tok->bos_id / eos_id) -- lands
in this build.  Its output on a small synthetic model is compared with the same model driven through the Python face
of the engine and with the CPU decode step (engine/main.cpp:22-58 single shot, :118-218 interactive loop).
The binary is built where the reference tree is mounted and travels with the tree; without it the tests skip."""
import importlib
import os
import subprocess

import numpy as np
import pytest

from test_gpu_chat import RefChat
from test_gpu_engine import SMALL, build_small

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "oracle", "_ref", "reference_cli")
CTX = 160
BOS, EOS = 1, 2


def vocabulary(n):
    """id 0 unknown, 1 <s>, 2 </s>, 3..258 the single bytes, then distinct two-letter words: every id of the model's
    vocabulary prints as something recognisable, and a prompt tokenises to its bytes."""
    toks = [b"<unk>", b"<s>", b"</s>"] + [bytes([b]) for b in range(256)]
    i = 0
    while len(toks) < n:
        toks.append(b"[" + bytes([97 + i // 26 % 26, 97 + i % 26]) + (b"%d" % (i // 676)) + b"]")
        i += 1
    return toks


@pytest.fixture(scope="module")
def model_dir(t12, oracle, tmp_path_factory):
    if not os.path.exists(CLI):
        pytest.skip("oracle/_ref/reference_cli not built (needs the reference tree at build time)")
    synth = importlib.import_module("turbo_lossless_amd.synth")
    modelio = importlib.import_module("turbo_lossless_amd.modelio")
    tf = importlib.import_module("turbo_lossless_amd.tokenizer_files")
    parts = build_small(oracle, synth, SMALL)
    path = str(tmp_path_factory.mktemp("cli_model"))
    modelio.write_model_dir(path, SMALL, *parts)
    tf.write_files(path, vocabulary(SMALL["n_vocab"]), [], BOS, EOS, None)
    return path, parts


def run_cli(args, stdin=None):
    env = dict(os.environ, TURBO_CTX=str(CTX))
    r = subprocess.run([CLI] + args, input=stdin, capture_output=True, timeout=120, env=env)
    assert r.returncode == 0, (r.returncode, r.stdout[-2000:], r.stderr[-2000:])
    return r.stdout


def field(out, name):
    for line in out.split(b"\n"):
        if line.startswith(name + b":"):
            return line[len(name) + 1:].strip()
    raise AssertionError((name, out[-1500:]))


@pytest.mark.parametrize("batch", [1, 4])
def test_single_shot_prints_the_engines_greedy_stream(t12, oracle, model_dir, batch):
    path, parts = model_dir
    prompt, max_tokens = "split twelve", 24
    out = run_cli([path, prompt, str(max_tokens), str(batch)])
    os.environ["TURBO_CTX"] = str(CTX)
    tok = t12.Tokenizer(path)
    ids = tok.tokenize(prompt)
    assert ids[0] == BOS and len(ids) == 1 + len(prompt)
    ref = oracle.RefModel(SMALL, *parts, max_seq=CTX)
    want = ref.generate(ids, max_tokens, eos=EOS)
    eng = t12.Engine.load(path, batch=batch)
    try:
        assert eng.generate(ids, max_tokens) == want
    finally:
        eng.close()
    text = b"".join(tok.detokenize_one(t) for t in want)
    tok.close()
    assert len(want) >= 8                                    # (the stream does not stop at once on this model)
    assert int(field(out, b"Prompt tokens")) == len(ids)
    assert int(field(out, b"Generated tokens")) == len(want)
    body = out.split(b"Generating...\n\n", 1)[1].split(b"\n\n--- Stats ---", 1)[0]
    assert body == text, (body, text)
    if batch > 1:
        assert b"Total throughput" in out


def test_interactive_turns_keep_the_context(t12, oracle, model_dir):
    """Three turns through the reference's interactive loop (engine/main.cpp:118-218): the cache persists between
    turns, BOS is kept on the first turn only, EOS is fed after every answer."""
    path, parts = model_dir
    lines, max_tokens = ["first turn", "and a second one", "third"], 12
    out = run_cli([path, "--interactive", str(max_tokens)], stdin=("\n".join(lines) + "\nquit\n").encode())
    os.environ["TURBO_CTX"] = str(CTX)
    tok = t12.Tokenizer(path)
    chat = RefChat(oracle.RefModel(SMALL, *parts, max_seq=CTX), CTX)
    turns = out.split(b"Generating...\n\n")[1:]
    assert len(turns) == len(lines)
    for line, got in zip(lines, turns):
        ids = tok.tokenize(line)
        want, discard = chat.turn(ids, max_tokens, oracle)
        assert discard == 0
        text = b"".join(tok.detokenize_one(t) for t in want)
        assert got.split(b"\n\n--- Stats ---", 1)[0] == text, (line, got[:200], text)
        assert int(field(got, b"Generated tokens")) == len(want)
        assert field(got, b"Context").split(b" / ")[0] == b"%d" % chat.pos
    tok.close()


# ---- the reference's HOST ENGINE over this build's kernel launchers ------------------------------------------------
DRIVER = os.path.join(ROOT, "oracle", "_ref", "reference_engine_driver")


@pytest.mark.parametrize("fast_tables", [False, True])
@pytest.mark.parametrize("batch", [1, 4, 8, 16])
def test_reference_host_engine_runs_on_this_builds_launchers(oracle, model_dir, batch, fast_tables):
    """oracle/_ref/reference_engine_driver = the reference's engine/model.cpp + inference.cpp + sampler.cpp, compiled
    unchanged with their own headers, plus a thin driver, linked with libturbo12.so: the reference's loader builds the
    derived escape tables (TURBO_FAST=1: with the per-lane count table), its forward_b1 / forward_b4 / forward_b8 /
    chunks-of-8 dispatch issues the launches (inference.cpp:198-712), and every one of the 18 launchers it declares
    (inference.cpp:7-41, sampler.cpp:4-5) is this build's.  The greedy stream must be the CPU decode step's."""
    if not os.path.exists(DRIVER):
        pytest.skip("oracle/_ref/reference_engine_driver not built (needs the reference tree at build time)")
    path, parts = model_dir
    rng = np.random.default_rng(7)
    prompt = [BOS] + [int(t) for t in rng.integers(3, SMALL["n_vocab"], 9)]
    max_tokens = 24
    env = dict(os.environ, TURBO_CTX=str(CTX))
    env.pop("TURBO_FAST", None)
    if fast_tables:
        env["TURBO_FAST"] = "1"
    r = subprocess.run([DRIVER, path, str(batch), str(max_tokens)] + [str(t) for t in prompt], capture_output=True,
                       timeout=120, env=env)
    assert r.returncode == 0, (r.returncode, r.stdout[-1500:], r.stderr[-1500:])
    line = [l for l in r.stdout.split(b"\n") if l.startswith(b"tokens:")]
    assert len(line) == 1, r.stdout[-1500:]
    got = [int(t) for t in line[0].split()[1:]]
    want = oracle.RefModel(SMALL, *parts, max_seq=CTX).generate(prompt, max_tokens, eos=EOS)
    assert len(want) >= 8
    assert got == want


DRIVER_NV = os.path.join(ROOT, "oracle", "_ref", "reference_engine_driver_nv")


@pytest.mark.parametrize("batch", [1, 8, 12, 64, 256])
def test_reference_host_engine_other_branch_runs_on_this_builds_launchers(oracle, model_dir, batch):
    """The same three reference files compiled with the macro that selects their other branch (inference.cpp:32-41,
    227-330, 537-677): batch 1 goes through nv_launch_split12_v2(_dual)_async and the batched patch launcher, batch 8
    through launch_split12_batch8_async, larger batches through forward_batch_tiled -- nv_launch_split12_cublas_batch_async
    for this model's tensors (all under 4096 rows), the corrections as nv_launch_patches_batch_async on the state's second
    stream, the batch forms of the RoPE / store / attention launchers.  Greedy stream = the CPU decode step's."""
    if not os.path.exists(DRIVER_NV):
        pytest.skip("oracle/_ref/reference_engine_driver_nv not built (needs the reference tree at build time)")
    path, parts = model_dir
    rng = np.random.default_rng(8)
    prompt = [BOS] + [int(t) for t in rng.integers(3, SMALL["n_vocab"], 7)]
    max_tokens = 20
    env = dict(os.environ, TURBO_CTX=str(CTX))
    env.pop("TURBO_FAST", None)
    env.pop("TURBO_CUBLAS", None)
    r = subprocess.run([DRIVER_NV, path, str(batch), str(max_tokens)] + [str(t) for t in prompt], capture_output=True,
                       timeout=120, env=env)
    assert r.returncode == 0, (r.returncode, r.stdout[-1500:], r.stderr[-1500:])
    line = [l for l in r.stdout.split(b"\n") if l.startswith(b"tokens:")]
    assert len(line) == 1, r.stdout[-1500:]
    got = [int(t) for t in line[0].split()[1:]]
    want = oracle.RefModel(SMALL, *parts, max_seq=CTX).generate(prompt, max_tokens, eos=EOS)
    assert len(want) >= 8
    assert got == want
