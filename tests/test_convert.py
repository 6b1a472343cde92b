"""CPU: the checkpoint side of the converter (safetensors container, bf16 rounding, config keys, tensor naming)
and the RoPE frequency table with the "llama3" scaling rule.

Checkers: the safetensors package for the container, torch's own float -> bfloat16 cast for the rounding (the
reference converter casts with Tensor.to(torch.bfloat16), engine/convert_model.py:159,190), transformers'
implementation of the published llama3 rule for the frequency table (the reference has no such rule)."""
import ctypes
import importlib
import json
import os

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def cv(t12):
    return importlib.import_module("turbo_lossless_amd.convert")


def test_reader_matches_safetensors_package(cv, tmp_path):
    st = pytest.importorskip("safetensors.torch")
    g = torch.Generator().manual_seed(1)
    tensors = {
        "a.bf16": torch.randn((7, 33), generator=g).to(torch.bfloat16),
        "b.f16": torch.randn((5, 64), generator=g).to(torch.float16),
        "c.f32": torch.randn((3, 10), generator=g),
        "d.vec": torch.randn((129,), generator=g),
        "e.empty": torch.zeros((0, 8)),
    }
    path = str(tmp_path / "x.safetensors")
    st.save_file(tensors, path, metadata={"format": "pt"})
    f = cv.SafetensorsFile(path)
    assert sorted(f.keys()) == sorted(tensors)
    for name, t in tensors.items():
        dt, shape = f.info(name)
        assert shape == tuple(t.shape)
        got = f.get(name)
        if t.dtype == torch.bfloat16:
            assert dt == "BF16" and np.array_equal(got, t.view(torch.int16).numpy().view(np.uint16))
        else:
            assert np.array_equal(got, t.numpy())
    f.close()


def test_reader_rejects_truncated_and_inconsistent_files(cv, tmp_path):
    p = tmp_path / "short.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(ValueError):
        cv.SafetensorsFile(str(p))
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4, 4], "data_offsets": [0, 64]}}).encode()
    p = tmp_path / "trunc.safetensors"
    p.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0" * 32)          # 32 of 64 bytes present
    with pytest.raises(ValueError):
        cv.SafetensorsFile(str(p))
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4, 4], "data_offsets": [0, 60]}}).encode()
    p = tmp_path / "size.safetensors"
    p.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0" * 64)
    with pytest.raises(ValueError):
        cv.SafetensorsFile(str(p))
    p = tmp_path / "hdr.safetensors"
    p.write_bytes((1 << 40).to_bytes(8, "little") + b"{}")
    with pytest.raises(ValueError):
        cv.SafetensorsFile(str(p))


def _torch_bf16_bits(t):
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_bf16_rounding_equals_torch_cast(cv):
    rng = np.random.default_rng(7)
    u = rng.integers(0, 1 << 32, size=400000, dtype=np.uint64).astype(np.uint32)      # every kind of fp32 pattern
    special = np.array([0x00000000, 0x80000000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x7F800001, 0xFFFFFFFF, 0x7FBFFFFF,
                        0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF, 0x7F7F8000, 0x00000001, 0x00008000,
                        0x00018000, 0x807FFFFF], dtype=np.uint32)                        # ties, overflow to Inf, NaNs, subnormals
    u = np.concatenate([u, special])
    f = u.view(np.float32)
    got = cv.to_bf16_bits(f, "F32")
    want = _torch_bf16_bits(torch.from_numpy(f.copy()))
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], want[~nan])
    # NaN: torch keeps a NaN; so do we (quiet NaN 0x7FC0), whatever the payload
    assert np.all((got[nan] & 0x7FFF) > 0x7F80) and np.all((want[nan] & 0x7FFF) > 0x7F80)


def test_fp16_to_bf16_equals_torch_cast_on_every_pattern(cv):
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    got = cv.to_bf16_bits(h, "F16")
    want = _torch_bf16_bits(torch.from_numpy(h.copy()))
    nan = np.isnan(h)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7FFF) > 0x7F80)


def test_bf16_passes_through_untouched(cv):
    b = np.arange(65536, dtype=np.uint16)
    assert np.array_equal(cv.to_bf16_bits(b, "BF16"), b)


def test_config_keys_and_fallbacks(cv, tmp_path):
    d = tmp_path / "hf"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(dict(
        hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, num_hidden_layers=32, intermediate_size=14336,
        vocab_size=128256, max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5,
        rope_scaling=dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192,
                          rope_type="llama3"))))
    c = cv.read_config(str(d))
    assert (c["n_vocab"], c["n_embd"], c["n_head"], c["n_head_kv"], c["n_layer"], c["n_ff"], c["n_ctx"]) == \
        (128256, 4096, 32, 8, 32, 14336, 131072)
    assert c["rope_theta"] == 500000.0 and c["rms_norm_eps"] == 1e-5
    assert c["rope_scaling"] == (8.0, 1.0, 4.0, 8192.0)
    # Meta-style keys and the defaults of engine/convert_model.py:46-54
    (d / "config.json").write_text(json.dumps(dict(dim=512, n_heads=8, n_layers=4)))
    c = cv.read_config(str(d))
    assert (c["n_vocab"], c["n_embd"], c["n_head"], c["n_head_kv"], c["n_layer"], c["n_ff"], c["n_ctx"]) == \
        (32000, 512, 8, 8, 4, 2048, 32768)
    assert c["rope_theta"] == 10000.0 and c["rms_norm_eps"] == 1e-5 and "rope_scaling" not in c
    # other kinds of scaling are not applied
    (d / "config.json").write_text(json.dumps(dict(dim=512, rope_scaling=dict(type="linear", factor=2.0))))
    assert "rope_scaling" not in cv.read_config(str(d))


def test_tensor_lookup_prefers_exact_names(cv, tmp_path):
    st = pytest.importorskip("safetensors.torch")
    d = tmp_path / "hf"
    d.mkdir()
    z = torch.zeros((2, 2))
    st.save_file({"model.layers.10.self_attn.q_proj.weight": z + 10, "model.layers.1.self_attn.q_proj.weight": z + 1,
                  "model.norm.weight": z[0], "model.layers.1.input_layernorm.weight": z[0] + 5}, str(d / "m-00001.safetensors"))
    st.save_file({"model.embed_tokens.weight": z, "lm_head.weight": z + 3}, str(d / "m-00002.safetensors"))
    ck = cv.Checkpoint(str(d))
    assert ck.find("layers.1.self_attn.q_proj") == "model.layers.1.self_attn.q_proj.weight"
    assert ck.find("layers.10.self_attn.q_proj") == "model.layers.10.self_attn.q_proj.weight"
    assert ck.find("layers.1.input_layernorm") == "model.layers.1.input_layernorm.weight"
    assert ck.find("embed_tokens") == "model.embed_tokens.weight" and ck.find("lm_head") == "lm_head.weight"
    assert ck.find("layers.2.self_attn.q_proj") is None
    assert float(ck.f32("model.layers.10.self_attn.q_proj.weight")[0, 0]) == 10.0
    ck.close()


LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "turbo-lossless_amd", "libturbo12.so")


def _c_freqs(head_dim, theta, scaling):
    lib = ctypes.CDLL(LIB)
    lib.t12_rope_freqs.argtypes = [ctypes.c_int] + [ctypes.c_float] * 5 + [ctypes.c_void_p]
    lib.t12_rope_freqs.restype = None
    out = np.zeros(head_dim // 2, np.float32)
    lib.t12_rope_freqs(head_dim, theta, *(scaling or (0.0, 0.0, 0.0, 0.0)), out.ctypes.data)
    return out


@pytest.mark.parametrize("head_dim,theta,scaling", [
    (128, 500000.0, (8.0, 1.0, 4.0, 8192.0)),      # Llama-3.1
    (64, 500000.0, (32.0, 1.0, 4.0, 8192.0)),      # Llama-3.2 1B
    (128, 10000.0, (4.0, 1.0, 8.0, 256.0)),        # a band that cuts through the middle of the table
])
def test_llama3_frequency_table_matches_transformers(oracle, head_dim, theta, scaling):
    ru = pytest.importorskip("transformers.modeling_rope_utils")
    from transformers import LlamaConfig
    cfg = LlamaConfig(hidden_size=head_dim * 4, num_attention_heads=4, rope_theta=theta, max_position_embeddings=131072,
                      rope_scaling={"rope_type": "llama3", "factor": scaling[0], "low_freq_factor": scaling[1],
                                    "high_freq_factor": scaling[2], "original_max_position_embeddings": int(scaling[3])})
    want, att = ru.ROPE_INIT_FUNCTIONS["llama3"](cfg, "cpu")
    want = want.numpy()
    assert att == 1.0
    got = _c_freqs(head_dim, theta, scaling)
    np.testing.assert_allclose(got, want, rtol=2e-6)                    # fp32 pow differs by an ulp between libraries
    np.testing.assert_allclose(oracle.rope_freqs(head_dim, theta, scaling), want, rtol=2e-6)
    # the three bands are all present, so a wrong comparison or a swapped factor shows
    plain = _c_freqs(head_dim, theta, None)
    ratio = got / plain
    assert np.isclose(ratio[0], 1.0) and np.isclose(ratio[-1], 1.0 / scaling[0])
    assert np.all(np.diff(ratio) <= 1e-6)


def test_plain_frequency_table(oracle):
    for hd, theta in ((128, 500000.0), (64, 10000.0), (96, 1e6)):
        want = (1.0 / np.float64(theta) ** (np.arange(0, hd, 2, dtype=np.float64) / hd))
        np.testing.assert_allclose(_c_freqs(hd, theta, None), want, rtol=1e-5)
        np.testing.assert_allclose(_c_freqs(hd, theta, None), oracle.rope_freqs(hd, theta), rtol=3e-7)   # powf vs numpy: 1 ulp
