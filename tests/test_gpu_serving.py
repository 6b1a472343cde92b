"""GPU parity of the serving extensions of the engine: independent sequences with their own KV-cache regions
(create_inference_state_per_sequence) and the batched prompt pass (prefill), against the CPU decode step run
once per sequence, token by token."""
import importlib
import os

import numpy as np
import pytest
import torch

from test_gpu_engine import SMALL, build_small

pytestmark = pytest.mark.gpu
V = SMALL["n_vocab"]
# head_dim 128 with four query heads per KV head: the shape that has the specialised attention kernels
HD128 = dict(SMALL, n_embd=512, n_head=4, n_head_kv=1, n_ff=1024)
CFGS = {"hd32": SMALL, "hd128": HD128}


@pytest.fixture(scope="module", params=["hd32", "hd128"])
def model(request, t12, oracle, tmp_path_factory):
    os.environ["TURBO_CTX"] = "256"
    synth = importlib.import_module("turbo_lossless_amd.synth")
    modelio = importlib.import_module("turbo_lossless_amd.modelio")
    cfg = CFGS[request.param]
    parts = build_small(oracle, synth, cfg)
    path = str(tmp_path_factory.mktemp("serving_model"))
    modelio.write_model_dir(path, cfg, *parts)
    return path, (cfg,) + tuple(parts)


def ref_model(oracle, parts):
    return oracle.RefModel(*parts, max_seq=256)


def rel(a, b):
    return float(np.abs(a - b).max() / np.abs(b).max())


def test_independent_sequences_match_single_sequence_runs(t12, oracle, model):
    path, parts = model
    rng = np.random.default_rng(5)
    B, T = 3, 6
    streams = rng.integers(3, V, size=(B, T))
    eng = t12.Engine.load(path, batch=B, per_sequence=64)
    try:
        refs = [ref_model(oracle, parts) for _ in range(B)]
        for t in range(T):
            eng.forward(streams[:, t])
            got = eng.logits(V).cpu().numpy()
            for b in range(B):
                want = refs[b].step(int(streams[b, t]), t)
                assert rel(got[b], want) < 2e-2, (t, b)
            assert eng.positions() == [t + 1] * B
        # the rows are really independent: different streams give different logits
        assert rel(got[0], got[1]) > 0.1
    finally:
        eng.close()


def test_batched_prefill_then_joint_decode(t12, oracle, model):
    """Prompts of different lengths (chunks of 4, 4, 2; 4, 1; 3; 4, 4, 4, 1), then all sequences decode together
    from their own positions."""
    path, parts = model
    rng = np.random.default_rng(6)
    B = 4
    lens = [10, 5, 3, 13]
    prompts = [[int(x) for x in rng.integers(3, V, size=n)] for n in lens]
    eng = t12.Engine.load(path, batch=B, per_sequence=64)
    try:
        refs = [ref_model(oracle, parts) for _ in range(B)]
        want = []
        for b in range(B):
            for pos, tok in enumerate(prompts[b]):
                lg = refs[b].step(tok, pos)
            want.append(lg)
        for b in (2, 0, 3, 1):                          # any order: the regions are separate
            eng.prefill(b, prompts[b])
        assert eng.positions() == lens
        got = eng.logits(V).cpu().numpy()
        for b in range(B):
            assert rel(got[b], want[b]) < 2e-2, b
            assert int(got[b].argmax()) == int(want[b].argmax())
        # joint greedy decode from staggered positions
        steps = 6
        toks = eng.decode_all(steps)
        assert len(toks) == steps and eng.positions() == [n + steps for n in lens]
        for b in range(B):
            cur = int(want[b].argmax())
            for t in range(steps):
                assert toks[t][b] == cur, (b, t)
                cur = int(refs[b].step(cur, lens[b] + t).argmax())
    finally:
        eng.close()


def test_prefill_equals_token_by_token_prompt_on_the_gpu(t12, model):
    """Same engine, same sequence: the batched prompt pass against forward() one token at a time (GEMM vs GEMV
    summation order and bf16 roundings only)."""
    path, _ = model
    rng = np.random.default_rng(7)
    prompt = [int(x) for x in rng.integers(3, V, size=21)]
    e1 = t12.Engine.load(path, batch=1)
    try:
        for tok in prompt:
            e1.forward([tok])
        want = e1.logits(V).clone()
    finally:
        e1.close()
    eb = t12.Engine.load(path, batch=8, per_sequence=32)
    try:
        eb.prefill(5, prompt)
        got = eb.logits(V)[5]
        assert float((got - want[0]).abs().max() / want[0].abs().max()) < 1e-2
        assert eb.positions() == [0, 0, 0, 0, 0, 21, 0, 0]
    finally:
        eb.close()


def test_prefill_on_a_shared_region_state(t12, oracle, model):
    """Lock-step copies on the model's one region: prefill advances every row and hands every row the logits."""
    path, parts = model
    rng = np.random.default_rng(8)
    prompt = [int(x) for x in rng.integers(3, V, size=11)]
    ref = ref_model(oracle, parts)
    for pos, tok in enumerate(prompt):
        want = ref.step(tok, pos)
    eng = t12.Engine.load(path, batch=4)
    try:
        eng.prefill(0, prompt)
        got = eng.logits(V)
        assert eng.positions() == [11] * 4
        assert torch.equal(got[0], got[3]) and torch.equal(got[0], got[1])
        assert rel(got[0].cpu().numpy(), want) < 2e-2
        nxt = int(want.argmax())
        eng.forward([nxt] * 4)
        assert rel(eng.logits(V)[2].cpu().numpy(), ref.step(nxt, 11)) < 2e-2
    finally:
        eng.close()


def test_per_sequence_batch_one_and_cache_bounds(t12, oracle, model):
    path, parts = model
    ref = ref_model(oracle, parts)
    eng = t12.Engine.load(path, batch=1, per_sequence=16)       # B = 1: the fused decode path on the state's own cache
    try:
        eng.prefill(0, [7, 8, 9])                                  # batch 1: token by token
        eng.forward([10])
        for pos, tok in enumerate([7, 8, 9, 10]):
            want = ref.step(tok, pos)
        assert rel(eng.logits(V).cpu().numpy()[0], want) < 2e-2
        assert eng.positions() == [4]
    finally:
        eng.close()
