"""Pins for the oracle's glue formulas and decode step (CPU only).

Every function of oracle/oracle.py that restates engine/kernels.hip or engine/inference.cpp is checked here
against something that is NOT the same formula retyped: torch's own operators in float64, the `transformers`
Llama implementation (rotate-half RoPE, attention with grouped KV heads, the decoder wiring), complex
multiplication, or invariants the mathematics fixes.  Each test also shows that a plausible mistake (the
"mutant") would fail it on the very inputs it uses, so a green run is evidence and not coincidence.
"""
import importlib

import numpy as np
import pytest
import torch
import torch.nn.functional as F


def _ulp_bf16(x):
    """Spacing of bf16 at |x| (8 significant bits)."""
    x = np.maximum(np.abs(np.asarray(x, np.float64)), 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(x)) - 7)


def _assert_bf16_close(bits, want64, what, exact_share=0.97):
    """bf16 result within one unit of the float64 value rounded to bf16, and equal to it almost everywhere
    (the restated formula works in fp32, so a value next to a rounding boundary may land one step away)."""
    from oracle import oracle as o
    got = o.bf16_bits_to_f32(bits).astype(np.float64)
    want_bits = torch.from_numpy(np.asarray(want64, np.float64)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    want = o.bf16_bits_to_f32(want_bits).astype(np.float64)
    assert np.all(np.abs(got - want) <= _ulp_bf16(want) * 1.0001), what
    share = float((np.asarray(bits).ravel() == want_bits.ravel()).mean())
    assert share >= exact_share, (what, share)


# ------------------------------------------------------------------------------------------------ bf16
def test_bf16_rounding_equals_torch_cast(oracle):
    """kernels.hip:21-27 is round-to-nearest-even: equal to torch's float32 -> bfloat16 cast on every finite value
    tried, including exact ties, the largest finite float (rounds to Inf) and subnormals."""
    rng = np.random.default_rng(0)
    u = rng.integers(0, 2 ** 32, size=400_000, dtype=np.uint64).astype(np.uint32)
    ties = (rng.integers(0, 2 ** 16, size=4096, dtype=np.uint64).astype(np.uint32) << 16) | np.uint32(0x8000)
    special = np.array([0x00000000, 0x80000000, 0x7F7FFFFF, 0x00000001, 0x807FFFFF, 0x3F808000, 0x3F818000,
                        0x7F800000, 0xFF800000], np.uint32)
    u = np.concatenate([u, ties, special])
    f = u.view(np.float32)
    f = f[~np.isnan(f)]
    want = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16_bits(f), want)
    # truncation (the plausible mistake) differs on about half of the random values
    assert (((f.view(np.uint32) >> 16).astype(np.uint16)) != want).mean() > 0.3
    # the inverse is the exact widening
    b = rng.integers(0, 2 ** 16, size=10000, dtype=np.uint64).astype(np.uint16)
    back = torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(oracle.bf16_bits_to_f32(b).view(np.uint32), back.view(np.uint32))


def test_embed_lookup(oracle):
    rng = np.random.default_rng(1)
    embd = rng.integers(0, 2 ** 16, size=(50, 16), dtype=np.uint64).astype(np.uint16)
    embd[(embd & 0x7F80) == 0x7F80] = 0          # keep it finite
    ids = [0, 49, 7, 50, -1]
    got = oracle.embed_lookup(embd, ids, 50)
    table = torch.from_numpy(embd.view(np.int16).copy()).view(torch.bfloat16).to(torch.float32)
    want = F.embedding(torch.tensor([0, 49, 7]), table).numpy()
    assert np.array_equal(got[:3], want)
    assert not got[3:].any()                      # ids outside the vocabulary give zero rows (kernels.hip:57-73)


# --------------------------------------------------------------------------------------------- RMSNorm
@pytest.mark.parametrize("n,scale", [(64, 1.0), (4096, 1.0), (256, 2e-3), (1000, 30.0)])
def test_rms_norm_vs_torch(oracle, n, scale):
    """kernels.hip:355-392 against torch.nn.functional.rms_norm in float64.  scale = 2e-3 makes mean(x^2) ~ 4e-6,
    smaller than eps = 1e-5: eps placed outside the square root, or dropped, fails there."""
    rng = np.random.default_rng(n)
    x = (rng.standard_normal((5, n)) * scale).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32)
    eps = 1e-5
    got = oracle.rms_norm_bf16(x, w, eps)
    want = F.rms_norm(torch.from_numpy(x).double(), (n,), torch.from_numpy(w).double(), eps).numpy()
    _assert_bf16_close(got, want, "rms_norm")
    if scale < 1e-2:
        x64 = x.astype(np.float64)
        wrong = x64 / (np.sqrt((x64 ** 2).mean(-1, keepdims=True)) + eps) * w      # eps outside the root
        g = oracle.bf16_bits_to_f32(got).astype(np.float64)
        assert np.abs(g - wrong).max() > 20 * _ulp_bf16(want).max()
        noeps = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True)) * w
        assert np.abs(g - noeps).max() > 20 * _ulp_bf16(want).max()


def test_add_rms_norm_vs_torch(oracle):
    """kernels.hip:399-442: the sum is written back in fp32 and the norm is taken of the SUM."""
    rng = np.random.default_rng(5)
    n = 512
    x = rng.standard_normal((3, n)).astype(np.float32)
    r = (3 * rng.standard_normal((3, n))).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32)
    s, y = oracle.add_rms_norm_bf16(x, r, w, 1e-5)
    assert s.dtype == np.float32
    assert np.array_equal(s, (torch.from_numpy(x) + torch.from_numpy(r)).numpy())
    want = F.rms_norm((torch.from_numpy(x).double() + torch.from_numpy(r).double()), (n,), torch.from_numpy(w).double(), 1e-5)
    _assert_bf16_close(y, want.numpy(), "add_rms_norm")
    # norm of x alone (residual forgotten) is far away
    alone = F.rms_norm(torch.from_numpy(x).double(), (n,), torch.from_numpy(w).double(), 1e-5).numpy()
    assert np.abs(oracle.bf16_bits_to_f32(y) - alone).max() > 0.5


def test_silu_mul_vs_torch(oracle):
    """kernels.hip:447-459 against torch's silu in float64, over the whole range incl. large |g|."""
    rng = np.random.default_rng(6)
    g = np.concatenate([rng.standard_normal(5000) * 3, np.array([0.0, -0.0, 20.0, -20.0, 88.0, -88.0, -100.0, 100.0])]).astype(np.float32)
    u = np.concatenate([rng.standard_normal(5000) * 2, np.ones(8)]).astype(np.float32)
    got = oracle.silu_mul_bf16(g, u)
    want = (F.silu(torch.from_numpy(g).double()) * torch.from_numpy(u).double()).numpy()
    _assert_bf16_close(got, want, "silu_mul")
    # silu(up) * gate, or sigmoid(g) * up without the factor g: both far away
    gg = oracle.bf16_bits_to_f32(got).astype(np.float64)
    swapped = (F.silu(torch.from_numpy(u).double()) * torch.from_numpy(g).double()).numpy()
    assert np.abs(gg - swapped).max() > 0.5
    sig = (torch.sigmoid(torch.from_numpy(g).double()) * torch.from_numpy(u).double()).numpy()
    assert np.abs(gg - sig).max() > 0.5


# ------------------------------------------------------------------------------------------------ RoPE
def _hf_rope(x, pos, n_head, hd, theta):
    """transformers' Llama rotary embedding (rotate_half form) applied to one token's heads, float64."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding, apply_rotary_pos_emb
    cfg = LlamaConfig(hidden_size=n_head * hd, num_attention_heads=n_head, num_key_value_heads=n_head,
                      rope_theta=theta, max_position_embeddings=1 << 16, head_dim=hd)
    rot = LlamaRotaryEmbedding(cfg)
    rot.inv_freq = rot.inv_freq.double()
    t = torch.from_numpy(np.asarray(x, np.float64)).reshape(1, 1, n_head, hd).transpose(1, 2)   # [b, heads, seq, hd]
    cos, sin = rot(t, torch.tensor([[pos]]))
    q, _ = apply_rotary_pos_emb(t, t, cos.double(), sin.double())
    return q.transpose(1, 2).reshape(-1).numpy()


@pytest.mark.parametrize("hd,n_head,theta", [(128, 4, 500000.0), (64, 3, 10000.0), (32, 8, 500000.0)])
def test_rope_vs_transformers_and_complex(oracle, hd, n_head, theta):
    """kernels.hip:174-213.  Checked against (i) transformers' rotate-half implementation, (ii) complex
    multiplication (x[d] + i x[d + hd/2]) * exp(i pos freq[d]), (iii) norm preservation per pair and pos = 0."""
    rng = np.random.default_rng(hd)
    x = rng.standard_normal(n_head * hd).astype(np.float32)
    h = hd // 2
    freq = theta ** (-2.0 * np.arange(h) / hd)
    assert np.allclose(oracle.rope_freqs(hd, theta), freq, rtol=3e-6, atol=0)
    for pos in (0, 1, 7, 300, 2047):
        got = oracle.rope(x, pos, n_head, hd, theta).astype(np.float64)
        # fp32 frequencies times pos: the angle is off by up to pos * 3e-6, the values (|x| < 6) by that times |x|
        v = x.astype(np.float64).reshape(n_head, hd)
        z = (v[:, :h] + 1j * v[:, h:]) * np.exp(1j * pos * freq)
        want = np.concatenate([z.real, z.imag], axis=1).reshape(-1)
        assert np.abs(got - want).max() < (1e-6 if pos == 0 else pos * 4e-6 * 6 + 1e-6), pos
        hf = _hf_rope(x, pos, n_head, hd, theta)
        assert np.abs(got - hf).max() < pos * 4e-6 * 6 + 1e-5, pos
        g = got.reshape(n_head, hd)
        assert np.allclose(g[:, :h] ** 2 + g[:, h:] ** 2, v[:, :h] ** 2 + v[:, h:] ** 2, rtol=1e-5, atol=1e-6)
        if pos == 0:
            assert np.array_equal(got.astype(np.float32), x)
    # the interleaved pairing (2d, 2d+1) and the opposite rotation sense are both far from the result
    got = oracle.rope(x, 7, n_head, hd, theta).astype(np.float64)
    v = x.astype(np.float64).reshape(n_head, h, 2)
    zi = (v[..., 0] + 1j * v[..., 1]) * np.exp(1j * 7 * freq)
    inter = np.stack([zi.real, zi.imag], axis=-1).reshape(-1)
    assert np.abs(got - inter).max() > 0.3
    v = x.astype(np.float64).reshape(n_head, hd)
    zc = (v[:, :h] + 1j * v[:, h:]) * np.exp(-1j * 7 * freq)
    assert np.abs(got - np.concatenate([zc.real, zc.imag], axis=1).reshape(-1)).max() > 0.3


# ------------------------------------------------------------------------------------- INT8 KV store
def test_quant_kv_int8_invariants(oracle):
    """kernels.hip:220-304: symmetric per-(position, KV head) INT8.  Fixed by the definition: |q| <= 127, the
    element of largest magnitude maps to +-127, q * scale is within scale / 2 of the value (rint, not truncation),
    ties to even, an all-zero head gives scale 0 and q 0, heads are independent."""
    rng = np.random.default_rng(9)
    nkv, hd = 4, 64
    v = rng.standard_normal(nkv * hd).astype(np.float32) * np.repeat([0.01, 1.0, 50.0, 1.0], hd).astype(np.float32)
    v[3 * hd:] = 0
    q, s = oracle.quant_kv_int8(v, nkv, hd)
    assert q.dtype == np.int8 and q.shape == (nkv, hd) and s.dtype == np.float32
    vv = v.reshape(nkv, hd)
    assert np.abs(q.astype(int)).max() <= 127
    for hh in range(3):
        am = np.abs(vv[hh]).argmax()
        assert abs(int(q[hh, am])) == 127 and np.sign(q[hh, am]) == np.sign(vv[hh, am])
        assert np.isclose(s[hh], np.abs(vv[hh]).max() / 127.0, rtol=1e-6)
        assert np.abs(q[hh] * np.float64(s[hh]) - vv[hh]).max() <= s[hh] / 2 * (1 + 1e-4)
        # truncation toward zero would leave errors up to a whole step
        trunc = np.trunc(vv[hh].astype(np.float64) / s[hh])
        assert np.abs(trunc * s[hh] - vv[hh]).max() > s[hh] * 0.9
    assert s[3] == 0 and not q[3].any()
    # same as torch's symmetric quantisation written with its own primitives
    t = torch.from_numpy(vv[:3]).double()
    tq = torch.clamp(torch.round(t * (127.0 / t.abs().amax(dim=1, keepdim=True))), -127, 127)
    assert (np.abs(q[:3].astype(np.float64) - tq.numpy()) <= 1).all() and (q[:3] == tq.numpy()).mean() > 0.99
    # exact ties go to even (rintf): absmax 127 -> step exactly 1
    tie = np.zeros(hd, np.float32)
    tie[:6] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5]
    qt, st = oracle.quant_kv_int8(tie, 1, hd)
    assert st[0] == 1.0 and list(qt[0, :6]) == [127, 0, 2, 2, 0, -2]


# ------------------------------------------------------------------------------------------ attention
@pytest.mark.parametrize("nh,nkv,hd,seq", [(8, 2, 32, 37), (4, 4, 64, 5), (32, 8, 128, 130), (6, 1, 16, 1)])
def test_attention_int8_vs_torch_sdpa(oracle, nh, nkv, hd, seq):
    """kernels.hip:499-586 against torch's scaled_dot_product_attention (float64) on the dequantised cache with
    the KV heads expanded by repeat_interleave (query head h reads KV head h // ratio)."""
    rng = np.random.default_rng(nh * 100 + seq)
    max_seq = seq + 3
    q = rng.standard_normal(nh * hd).astype(np.float32) * 2
    kc = rng.integers(-127, 128, size=(max_seq, nkv, hd)).astype(np.int8)
    vc = rng.integers(-127, 128, size=(max_seq, nkv, hd)).astype(np.int8)
    ks = (rng.random((max_seq, nkv)) * 0.02 + 0.001).astype(np.float32)
    vs = (rng.random((max_seq, nkv)) * 0.02 + 0.001).astype(np.float32)
    got = oracle.attention_int8(q, kc, vc, ks, vs, seq, nh, nkv, hd)
    Kd = torch.from_numpy(kc[:seq].astype(np.float64) * ks[:seq, :, None].astype(np.float64))     # [seq, nkv, hd]
    Vd = torch.from_numpy(vc[:seq].astype(np.float64) * vs[:seq, :, None].astype(np.float64))
    ratio = nh // nkv
    Ke = Kd.permute(1, 0, 2).repeat_interleave(ratio, dim=0).unsqueeze(0)                          # [1, nh, seq, hd]
    Ve = Vd.permute(1, 0, 2).repeat_interleave(ratio, dim=0).unsqueeze(0)
    Q = torch.from_numpy(q.astype(np.float64)).reshape(1, nh, 1, hd)
    want = F.scaled_dot_product_attention(Q, Ke, Ve).reshape(-1).numpy()                           # scale 1/sqrt(hd)
    _assert_bf16_close(got, want, "attention", exact_share=0.95)
    if nkv > 1 and ratio > 1:
        # the other head map (h % nkv) is far away; so are positions past seq_len if they were read
        Kw = Kd.permute(1, 0, 2).repeat(ratio, 1, 1).unsqueeze(0)
        Vw = Vd.permute(1, 0, 2).repeat(ratio, 1, 1).unsqueeze(0)
        wrong = F.scaled_dot_product_attention(Q, Kw, Vw).reshape(-1).numpy()
        assert np.abs(oracle.bf16_bits_to_f32(got) - wrong).max() > 0.05


def test_argmax_first(oracle):
    rng = np.random.default_rng(3)
    for _ in range(20):
        x = rng.integers(-5, 6, size=200).astype(np.float32)          # many exact ties
        best, arg = -np.inf, -1
        for i, v in enumerate(x):                                       # brute force: first maximum
            if v > best:
                best, arg = v, i
        assert oracle.argmax_first(x) == arg
    assert oracle.argmax_first(np.array([1.0, 3.0, 3.0, -2.0], np.float32)) == 1


# ---------------------------------------------------------------------------------------- decode step
CFG = dict(n_vocab=320, n_embd=128, n_head=8, n_head_kv=2, n_layer=2, n_ff=192, n_ctx=64,
           rope_theta=500000.0, rms_norm_eps=1e-5)


def _build(oracle, cfg, seed=77):
    synth = importlib.import_module("turbo_lossless_amd.synth")
    n, ff, hd = cfg["n_embd"], cfg["n_ff"], cfg["n_embd"] // cfg["n_head"]
    kv = cfg["n_head_kv"] * hd
    rng = np.random.default_rng(seed)
    s = [seed]

    def mk(M, K):
        s[0] += 1
        return oracle.pack(synth.weights_llm(M, K, s[0], sigma=0.08, p_outlier=2e-3, sigma_outlier=2.0))

    layers = []
    for _ in range(cfg["n_layer"]):
        layers.append(dict(attn_norm=(1 + 0.1 * rng.standard_normal(n)).astype(np.float32),
                           ffn_norm=(1 + 0.1 * rng.standard_normal(n)).astype(np.float32),
                           wq=mk(n, n), wk=mk(kv, n), wv=mk(kv, n), wo=mk(n, n),
                           w_gate=mk(ff, n), w_up=mk(ff, n), w_down=mk(n, ff)))
    embd = synth.weights_llm(cfg["n_vocab"], n, seed + 999, sigma=1.0, p_outlier=0)
    onorm = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    head = mk(cfg["n_vocab"], n)
    return embd, onorm, head, layers


def _hf_model(oracle, cfg, embd, onorm, head, layers):
    """The same weights (decoded, exact) in transformers' LlamaForCausalLM, float64, eager attention."""
    from transformers import LlamaConfig, LlamaForCausalLM
    hc = LlamaConfig(vocab_size=cfg["n_vocab"], hidden_size=cfg["n_embd"], intermediate_size=cfg["n_ff"],
                     num_hidden_layers=cfg["n_layer"], num_attention_heads=cfg["n_head"],
                     num_key_value_heads=cfg["n_head_kv"], rms_norm_eps=cfg["rms_norm_eps"],
                     rope_theta=cfg["rope_theta"], max_position_embeddings=cfg["n_ctx"],
                     tie_word_embeddings=False, attention_bias=False, mlp_bias=False)
    hc._attn_implementation = "eager"
    m = LlamaForCausalLM(hc).double().eval()

    def W(p):
        return torch.from_numpy(oracle.bf16_bits_to_f32(oracle.decode(p)).astype(np.float64))

    sd = {"model.embed_tokens.weight": torch.from_numpy(oracle.bf16_bits_to_f32(embd).astype(np.float64)),
          "model.norm.weight": torch.from_numpy(onorm.astype(np.float64)), "lm_head.weight": W(head)}
    names = dict(wq="self_attn.q_proj", wk="self_attn.k_proj", wv="self_attn.v_proj", wo="self_attn.o_proj",
                 w_gate="mlp.gate_proj", w_up="mlp.up_proj", w_down="mlp.down_proj")
    for i, L in enumerate(layers):
        for k, hn in names.items():
            sd["model.layers.%d.%s.weight" % (i, hn)] = W(L[k])
        sd["model.layers.%d.input_layernorm.weight" % i] = torch.from_numpy(L["attn_norm"].astype(np.float64))
        sd["model.layers.%d.post_attention_layernorm.weight" % i] = torch.from_numpy(L["ffn_norm"].astype(np.float64))
    missing, unexpected = m.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in k or "inv_freq" in k for k in missing), (missing, unexpected)
    return m


def test_refmodel_step_vs_transformers_llama(oracle, t12):
    """RefModel.step (engine/inference.cpp:198-366 restated) against transformers' Llama decoder in float64 on the
    decoded weights, six positions of one sequence.  The restatement rounds the matvec inputs to bf16 and keeps
    K/V as INT8 (as the reference does), so the logits agree to ~1e-2 of their scale and not to the last bit;
    every wiring mistake tried below is an order of magnitude further away."""
    embd, onorm, head, layers = _build(oracle, CFG)
    toks = [5, 311, 17, 3, 200, 44]
    with torch.no_grad():
        want = _hf_model(oracle, CFG, embd, onorm, head, layers)(torch.tensor([toks])).logits[0].numpy()

    def run(ref):
        return np.stack([ref.step(t, i) for i, t in enumerate(toks)])

    got = run(oracle.RefModel(CFG, embd, onorm, head, layers, max_seq=64))
    scale = np.abs(want).max(axis=1, keepdims=True)
    err = (np.abs(got - want) / scale).max(axis=1)
    assert err.max() < 2e-2, err
    assert all(int(np.argmax(g)) == int(np.argmax(w)) for g, w in zip(got, want))

    # mutants: each one must be clearly worse than the bound above
    def mutant(**swap):
        saved = {k: getattr(oracle, k) for k in swap}
        try:
            for k, fn in swap.items():
                setattr(oracle, k, fn)
            g = run(oracle.RefModel(CFG, embd, onorm, head, layers, max_seq=64))
        finally:
            for k, fn in saved.items():
                setattr(oracle, k, fn)
        return (np.abs(g - want) / scale).max(axis=1)

    real_rope, real_attn, real_add = oracle.rope, oracle.attention_int8, oracle.add_rms_norm_bf16

    def rope_interleaved(x, pos, n_head, hd, theta, scaling=None):
        v = x.astype(np.float64).reshape(n_head, hd // 2, 2)
        f = theta ** (-2.0 * np.arange(hd // 2) / hd)
        z = (v[..., 0] + 1j * v[..., 1]) * np.exp(1j * pos * f)
        return np.stack([z.real, z.imag], -1).reshape(-1).astype(np.float32)

    def rope_off_by_one(x, pos, *a, **k):
        return real_rope(x, pos + 1, *a, **k) if x.size == CFG["n_embd"] else real_rope(x, pos, *a, **k)   # Q only

    def attn_wrong_heads(q, kc, vc, ks, vs, seq, nh, nkv, hd):
        perm = np.arange(nh).reshape(nh // nkv, nkv).T.reshape(-1)       # h -> h % nkv
        out = real_attn(q.reshape(nh, hd)[perm].reshape(-1), kc, vc, ks, vs, seq, nh, nkv, hd)
        return out.reshape(nh, hd)[np.argsort(perm)].reshape(-1)

    def attn_short(q, kc, vc, ks, vs, seq, nh, nkv, hd):                 # forgets the newest position
        return real_attn(q, kc, vc, ks, vs, max(seq - 1, 1), nh, nkv, hd)

    def add_no_residual(x, r, w, eps):
        return x.astype(np.float32), oracle.rms_norm_bf16(x, w, eps)

    assert mutant(rope=rope_interleaved)[1:].max() > 5e-2
    assert mutant(rope=rope_off_by_one)[1:].max() > 5e-2
    assert mutant(attention_int8=attn_wrong_heads)[1:].max() > 5e-2
    assert mutant(attention_int8=attn_short)[1:].max() > 5e-2
    assert mutant(add_rms_norm_bf16=add_no_residual).max() > 5e-2
    assert real_add is oracle.add_rms_norm_bf16 and real_rope is oracle.rope


def test_refmodel_generate_is_greedy_loop(oracle, t12):
    """generate() (engine/inference.cpp:716-730): prompt token by token, then argmax -> step, stopping before id 2.
    Checked against the same loop driven by transformers' Llama on the decoded weights with the oracle's own
    logits deciding ties of rounding: the two streams agree while the float64 top-2 margin exceeds the oracle's
    error bound, which is asserted for the tokens compared."""
    embd, onorm, head, layers = _build(oracle, CFG, seed=91)
    m = _hf_model(oracle, CFG, embd, onorm, head, layers)
    prompt = [9, 100, 33]
    ref = oracle.RefModel(CFG, embd, onorm, head, layers, max_seq=64)
    out = ref.generate(prompt, 12)
    assert 2 not in out and len(out) <= 12
    seq = list(prompt)
    checked = 0
    for t in out:
        with torch.no_grad():
            lg = m(torch.tensor([seq])).logits[0, -1].numpy()
        top = np.sort(lg)[-2:]
        if (top[1] - top[0]) > 4e-2 * np.abs(lg).max():
            assert int(np.argmax(lg)) == t
            checked += 1
        seq.append(t)
    assert checked >= 6
    # a stop id in the stream ends it without emitting it
    first = out[0]
    assert ref.__class__(CFG, embd, onorm, head, layers, max_seq=64).generate(prompt, 12, eos=first) == []
