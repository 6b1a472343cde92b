"""GPU: safetensors checkpoint -> split-12 model directory (packed on the GPU) -> engine.

The converted files are compared byte for byte with what the CPU restatement of the reference packer
(split12_pack.c) writes for the same bf16 tensors, cast by torch as the reference converter casts them
(engine/convert_model.py:159,190); the engine then runs the converted directory against the CPU decode step."""
import importlib
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

CFG = dict(hidden_size=256, num_attention_heads=8, num_key_value_heads=2, num_hidden_layers=2, intermediate_size=512,
           vocab_size=1024, max_position_embeddings=4096, rope_theta=10000.0, rms_norm_eps=1e-5,
           rope_scaling=dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=8.0,
                             original_max_position_embeddings=64))


def hf_checkpoint(path, tied, seed=11):
    """A two-shard Llama-named checkpoint with bf16, fp16 and fp32 tensors; returns {name: torch tensor}."""
    st = importlib.import_module("safetensors.torch")
    g = torch.Generator().manual_seed(seed)
    n, ff, V = CFG["hidden_size"], CFG["intermediate_size"], CFG["vocab_size"]
    kv = n // CFG["num_attention_heads"] * CFG["num_key_value_heads"]

    def w(M, K, dtype):
        t = torch.randn((M, K), generator=g) * 0.02
        m = torch.rand((M, K), generator=g) < 2e-3
        return torch.where(m, torch.randn((M, K), generator=g) * 4.0, t).to(dtype)

    a = {"model.embed_tokens.weight": torch.randn((V, n), generator=g).to(torch.bfloat16),
         "model.norm.weight": (1 + 0.05 * torch.randn(n, generator=g)).to(torch.bfloat16)}
    b = {}
    if not tied:
        b["lm_head.weight"] = w(V, n, torch.float32)
    for i in range(CFG["num_hidden_layers"]):
        d = a if i == 0 else b
        p = "model.layers.%d." % i
        d[p + "input_layernorm.weight"] = 1 + 0.05 * torch.randn(n, generator=g)
        d[p + "post_attention_layernorm.weight"] = (1 + 0.05 * torch.randn(n, generator=g)).to(torch.float16)
        d[p + "self_attn.q_proj.weight"] = w(n, n, torch.bfloat16)
        d[p + "self_attn.k_proj.weight"] = w(kv, n, torch.float16)
        d[p + "self_attn.v_proj.weight"] = w(kv, n, torch.float32)
        d[p + "self_attn.o_proj.weight"] = w(n, n, torch.bfloat16)
        d[p + "mlp.gate_proj.weight"] = w(ff, n, torch.float32)
        d[p + "mlp.up_proj.weight"] = w(ff, n, torch.bfloat16)
        d[p + "mlp.down_proj.weight"] = w(n, ff, torch.float16)
    os.makedirs(path, exist_ok=True)
    st.save_file(a, os.path.join(path, "model-00001-of-00002.safetensors"))
    st.save_file(b, os.path.join(path, "model-00002-of-00002.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(dict(CFG, tie_word_embeddings=tied), f)
    return {**a, **b}


def bits(t):
    return t.to(torch.bfloat16).contiguous().view(torch.int16).numpy().view(np.uint16)


NAMES = dict(wq="self_attn.q_proj", wk="self_attn.k_proj", wv="self_attn.v_proj", wo="self_attn.o_proj",
             w_gate="mlp.gate_proj", w_up="mlp.up_proj", w_down="mlp.down_proj")


@pytest.mark.parametrize("tied", [False, True])
def test_converted_directory_equals_cpu_packer_and_runs(t12, oracle, tmp_path, tied):
    pytest.importorskip("safetensors.torch")
    cv = importlib.import_module("turbo_lossless_amd.convert")
    modelio = importlib.import_module("turbo_lossless_amd.modelio")
    src, out, want_dir = str(tmp_path / "hf"), str(tmp_path / "t12"), str(tmp_path / "want")
    tensors = hf_checkpoint(src, tied)
    stats = cv.convert(src, out)
    assert len(stats) == 1 + 7 * CFG["num_hidden_layers"]

    # the same directory through the CPU packer
    cfg = cv.read_config(src)
    assert cfg["rope_scaling"] == (4.0, 1.0, 8.0, 64.0)
    layers = []
    for i in range(cfg["n_layer"]):
        p = "model.layers.%d." % i
        L = dict(attn_norm=tensors[p + "input_layernorm.weight"].float().numpy(),
                 ffn_norm=tensors[p + "post_attention_layernorm.weight"].float().numpy())
        for ours, hf in NAMES.items():
            L[ours] = oracle.pack(bits(tensors[p + hf + ".weight"]))
        layers.append(L)
    embd = bits(tensors["model.embed_tokens.weight"])
    head = oracle.pack(bits(tensors["model.embed_tokens.weight" if tied else "lm_head.weight"]))
    onorm = tensors["model.norm.weight"].float().numpy()
    modelio.write_model_dir(want_dir, cfg, embd, onorm, head, layers)
    files = sorted(os.listdir(want_dir))
    assert sorted(os.listdir(out)) == files and "rope_scaling.bin" in files and len(files) == 4 + 7 + 2 * (2 + 49)
    for f in files:
        assert open(os.path.join(out, f), "rb").read() == open(os.path.join(want_dir, f), "rb").read(), f
    assert sum(s[2] for s in stats.values()) > 0                                   # escapes were exercised

    # the engine on the converted directory, positions far enough for all three bands of the scaling rule
    os.environ["TURBO_CTX"] = "256"
    ref = oracle.RefModel(cfg, embd, onorm, head, layers, max_seq=256)
    plain = oracle.RefModel({k: v for k, v in cfg.items() if k != "rope_scaling"}, embd, onorm, head, layers, max_seq=256)
    eng = t12.Engine.load(out, batch=1)
    try:
        toks = [5, 900, 17, 3, 1023, 44, 7, 300]
        differs = 0.0
        for pos, tok in enumerate(toks):
            eng.forward([tok])
            got = eng.logits(cfg["n_vocab"]).cpu().numpy()[0]
            want = ref.step(tok, pos)
            err = np.abs(got - want).max() / np.abs(want).max()
            assert err < 2e-2, (pos, err)
            differs = max(differs, np.abs(plain.step(tok, pos) - want).max() / np.abs(want).max())
        assert differs > 5e-2, differs              # the scaling is not a no-op on this model
        # save_model keeps the scaling
        saved = str(tmp_path / "saved")
        os.makedirs(saved)
        eng.save(saved)
        assert open(os.path.join(saved, "rope_scaling.bin"), "rb").read() == open(os.path.join(out, "rope_scaling.bin"), "rb").read()
    finally:
        eng.close()


def test_missing_tensor_is_an_error(t12, tmp_path):
    st = pytest.importorskip("safetensors.torch")
    cv = importlib.import_module("turbo_lossless_amd.convert")
    src = str(tmp_path / "hf")
    tensors = hf_checkpoint(src, tied=False)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    for f in os.listdir(src):
        if f.endswith(".safetensors"):
            os.remove(os.path.join(src, f))
    st.save_file(tensors, os.path.join(src, "model.safetensors"))
    with pytest.raises(KeyError):
        cv.convert(src, str(tmp_path / "out"))
