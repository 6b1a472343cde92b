"""CPU oracle for the split-12 path -- TEST INFRASTRUCTURE ONLY.

Python face of ``t12_oracle.c`` (ctypes) plus numpy restatements of the engine
glue formulas.  Only tests, the smoke check and the benchmark's ``cpu_baseline``
leg may import this module; the shipped library never does.

Reference citations are relative to the upstream tree:
  split12_pack.c:18-37,47-128        packer (find_base_exp, pack)
  decompress_v2.hip:148-227,78-99    matvec / patch semantics
  nvidia_kernels.cu:533-548          standalone (unpatched) decode
  engine/model.cpp:86-160            derived escape tables
  engine/kernels.hip                 glue formulas (lines cited per function)
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libt12_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libsplit12_ref.so")


def build(force: bool = False) -> None:
    """Compile the C oracle (and the reference packer when its tree is mounted)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])


def _ptr(a, ctype):
    if a is None:
        return None
    return a.ctypes.data_as(C.POINTER(ctype))


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        u8p, u16p, i16p, i32p, f32p = (C.POINTER(t) for t in (C.c_uint8, C.c_uint16, C.c_int16, C.c_int32, C.c_float))
        L.t12o_find_base_exp.argtypes = [u16p, C.c_int64]
        L.t12o_find_base_exp.restype = C.c_int
        L.t12o_count_escapes.argtypes = [u16p, C.c_int64, C.c_int]
        L.t12o_count_escapes.restype = C.c_int64
        L.t12o_pack.argtypes = [u16p, C.c_int, C.c_int, C.c_int, u8p, u8p, i32p, i32p, i16p, i16p]
        L.t12o_pack.restype = C.c_int64
        L.t12o_decode.argtypes = [u8p, u8p, C.c_int, C.c_int, C.c_int, i32p, i32p, i16p, C.c_int, u16p]
        L.t12o_decode.restype = None
        L.t12o_escape_tables.argtypes = [C.c_int, i32p, i32p, i16p, i32p, u8p, i16p, i32p]
        L.t12o_escape_tables.restype = C.c_int
        L.t12o_gemm.argtypes = [u8p, u8p, C.c_int, C.c_int, C.c_int, i32p, i32p, i16p, u16p, C.c_int, C.c_int, f32p, C.c_int]
        L.t12o_gemm.restype = None
        L.t12o_apply_patches.argtypes = [i32p, i32p, i16p, i16p, u16p, f32p, C.c_int]
        L.t12o_apply_patches.restype = None
        L.t12o_num_threads.restype = C.c_int
        L.t12o_set_num_threads.argtypes = [C.c_int]
        L.t12o_set_num_threads.restype = None
        _lib = L
    return _lib


def ref_lib():
    """The reference's own packer built from split12_pack.c (None when absent)."""
    if not os.path.exists(_REF_PATH):
        return None
    L = C.CDLL(_REF_PATH)
    L.split12_find_base_exp.argtypes = [C.POINTER(C.c_uint16), C.c_int]
    L.split12_find_base_exp.restype = C.c_int
    L.pack_split12.argtypes = [C.POINTER(C.c_uint16), C.c_int, C.c_int, C.c_int,
                               C.POINTER(C.c_uint8), C.POINTER(C.c_uint8), C.POINTER(C.c_int32),
                               C.POINTER(C.c_int32), C.POINTER(C.c_int16), C.POINTER(C.c_int16)]
    L.pack_split12.restype = C.c_int
    return L


# ----------------------------------------------------------------- bf16 helpers
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even, no NaN special case (engine/kernels.hip:21-27)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b).view(np.uint16).astype(np.uint32) << 16).view(np.float32)


# ------------------------------------------------------------------- pack/decode
class Packed:
    """One tensor in split-12 form: the arrays pack_split12 emits."""

    def __init__(self, M, K, base_exp, sm, gr, row_off, cols, correct, wrong):
        self.M, self.K, self.base_exp = int(M), int(K), int(base_exp)
        self.sm, self.gr, self.row_off = sm, gr, row_off
        self.cols, self.correct, self.wrong = cols, correct, wrong

    @property
    def P(self):
        return int(self.row_off[-1])


def find_base_exp(w_bits: np.ndarray) -> int:
    w = np.ascontiguousarray(w_bits, dtype=np.uint16).ravel()
    return int(lib().t12o_find_base_exp(_ptr(w, C.c_uint16), w.size))


def pack(w_bits: np.ndarray, base_exp: int | None = None) -> Packed:
    w = np.ascontiguousarray(w_bits, dtype=np.uint16)
    M, K = w.shape
    if base_exp is None:
        base_exp = find_base_exp(w)
    n = M * K
    P = int(lib().t12o_count_escapes(_ptr(w, C.c_uint16), n, base_exp))
    sm = np.empty(n, np.uint8)
    gr = np.empty((n + 1) // 2, np.uint8)
    row_off = np.empty(M + 1, np.int32)
    cols = np.empty(P, np.int32)
    correct = np.empty(P, np.int16)
    wrong = np.empty(P, np.int16)
    got = lib().t12o_pack(_ptr(w, C.c_uint16), M, K, base_exp, _ptr(sm, C.c_uint8), _ptr(gr, C.c_uint8),
                          _ptr(row_off, C.c_int32), _ptr(cols, C.c_int32), _ptr(correct, C.c_int16),
                          _ptr(wrong, C.c_int16))
    assert got == P
    return Packed(M, K, base_exp, sm, gr, row_off, cols, correct, wrong)


def decode(p: Packed, patched: bool = True) -> np.ndarray:
    out = np.empty((p.M, p.K), np.uint16)
    lib().t12o_decode(_ptr(p.sm, C.c_uint8), _ptr(p.gr, C.c_uint8), p.base_exp, p.M, p.K,
                      _ptr(p.row_off, C.c_int32), _ptr(p.cols, C.c_int32), _ptr(p.correct, C.c_int16),
                      int(patched), _ptr(out, C.c_uint16))
    return out


def escape_tables(p: Packed):
    """(row_base[M], counts_u8[M*256], esc_vals[P], nonempty_rows) -- model.cpp:86-160."""
    row_base = np.empty(p.M, np.int32)
    counts = np.empty(p.M * 256, np.uint8)
    esc_vals = np.empty(max(p.P, 1), np.int16)
    nonempty = np.empty(p.M, np.int32)
    nne = lib().t12o_escape_tables(p.M, _ptr(p.row_off, C.c_int32), _ptr(p.cols, C.c_int32),
                                   _ptr(p.correct, C.c_int16), _ptr(row_base, C.c_int32),
                                   _ptr(counts, C.c_uint8), _ptr(esc_vals, C.c_int16), _ptr(nonempty, C.c_int32))
    return row_base, counts, esc_vals[:p.P], nonempty[:nne]


def gemm(p: Packed, x_bits: np.ndarray, patched: bool = True) -> np.ndarray:
    """out[b, m] fp32 = decode-then-fp32-accumulate W.x over the rows of x_bits [B, K]."""
    x = np.ascontiguousarray(x_bits, dtype=np.uint16).reshape(-1, p.K)
    B = x.shape[0]
    out = np.empty((B, p.M), np.float32)
    ro = _ptr(p.row_off, C.c_int32) if patched else None
    lib().t12o_gemm(_ptr(p.sm, C.c_uint8), _ptr(p.gr, C.c_uint8), p.base_exp, p.M, p.K, ro,
                    _ptr(p.cols, C.c_int32), _ptr(p.correct, C.c_int16), _ptr(x, C.c_uint16), p.K, B,
                    _ptr(out, C.c_float), p.M)
    return out


def gemv(p: Packed, x_bits: np.ndarray, patched: bool = True) -> np.ndarray:
    return gemm(p, np.asarray(x_bits).reshape(1, -1), patched)[0]


def apply_patches(p: Packed, x_bits: np.ndarray, out: np.ndarray) -> None:
    x = np.ascontiguousarray(x_bits, dtype=np.uint16)
    assert out.dtype == np.float32 and out.flags.c_contiguous
    lib().t12o_apply_patches(_ptr(p.row_off, C.c_int32), _ptr(p.cols, C.c_int32), _ptr(p.correct, C.c_int16),
                             _ptr(p.wrong, C.c_int16), _ptr(x, C.c_uint16), _ptr(out, C.c_float), p.M)


def num_threads() -> int:
    return int(lib().t12o_num_threads())


def set_num_threads(n: int) -> None:
    """Threads of the C oracle's parallel loops from now on (n < 1: the OpenMP default)."""
    lib().t12o_set_num_threads(int(n))


# ------------------------------------------------------------------ engine glue
def embed_lookup(embd_bits: np.ndarray, token_ids, n_vocab: int) -> np.ndarray:
    """hidden[b] = f32(embd[token_b]); out-of-range id -> zeros (kernels.hip:57-73)."""
    n_embd = embd_bits.shape[1]
    out = np.zeros((len(token_ids), n_embd), np.float32)
    for b, t in enumerate(token_ids):
        if 0 <= t < n_vocab:
            out[b] = bf16_bits_to_f32(embd_bits[t])
    return out


def rms_norm_bf16(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """bf16_rne(x * rsqrt(mean(x^2) + eps) * w), row-wise (kernels.hip:355-392)."""
    x = x.astype(np.float32)
    ms = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)
    r = (1.0 / np.sqrt(ms + eps)).astype(np.float32)
    return f32_to_bf16_bits((x * r) * weight.astype(np.float32))


def add_rms_norm_bf16(x: np.ndarray, residual: np.ndarray, weight: np.ndarray, eps: float):
    """x += residual (fp32), then RMSNorm -> bf16 (kernels.hip:399-442). Returns (x_new, y_bits)."""
    s = (x.astype(np.float32) + residual.astype(np.float32)).astype(np.float32)
    return s, rms_norm_bf16(s, weight, eps)


def silu_mul_bf16(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """bf16_rne(g / (1 + exp(-g)) * up) (kernels.hip:447-459)."""
    g = gate.astype(np.float32)
    with np.errstate(over="ignore"):          # exp(-g) = inf for g < -88: g / inf = -0, what expf gives on the GPU too
        s = g / (np.float32(1.0) + np.exp(-g, dtype=np.float32))
    return f32_to_bf16_bits(s * up.astype(np.float32))


def rope_freqs(head_dim: int, theta: float, scaling=None) -> np.ndarray:
    """freq[d] = 1 / theta^(2d/head_dim), fp32 powf on the host (kernels.hip:129-140).

    scaling = (factor, low_freq_factor, high_freq_factor, original_ctx): the "llama3" rule of a checkpoint's
    rope_scaling entry, which the reference drops (engine/convert_model.py:54).  Not reference behaviour; pinned
    against transformers' implementation of the published rule in tests/test_convert.py."""
    d = np.arange(head_dim // 2, dtype=np.float32)
    f = (np.float32(1.0) / np.power(np.float32(theta), (2 * d) / np.float32(head_dim), dtype=np.float32)).astype(np.float32)
    if scaling:
        factor, low, high, orig = (np.float32(x) for x in scaling)
        wavelen = np.float32(2 * np.pi) / f
        smooth = (orig / wavelen - low) / (high - low)
        mid = (np.float32(1) - smooth) * f / factor + smooth * f
        f = np.where(wavelen > orig / low, f / factor, np.where(wavelen < orig / high, f, mid)).astype(np.float32)
    return f


def rope(x: np.ndarray, pos: int, n_head: int, head_dim: int, theta: float, scaling=None) -> np.ndarray:
    """Rotate-half RoPE: pairs (d, d+hd/2), angle = pos*freq[d] (kernels.hip:174-213)."""
    h = head_dim // 2
    f = rope_freqs(head_dim, theta, scaling).astype(np.float64)
    ang = pos * f
    c, s = np.cos(ang), np.sin(ang)
    v = x.astype(np.float64).reshape(n_head, head_dim).copy()
    x0, x1 = v[:, :h].copy(), v[:, h:].copy()
    v[:, :h] = x0 * c - x1 * s
    v[:, h:] = x0 * s + x1 * c
    return v.reshape(-1).astype(np.float32)


def quant_kv_int8(v: np.ndarray, n_head_kv: int, head_dim: int):
    """Per-(position, kv_head) symmetric int8: scale = absmax/127,
    q = clamp(rint(v * (127/absmax)), +-127) (kernels.hip:220-304). Returns (int8[nkv,hd], scale[nkv])."""
    v = v.astype(np.float32).reshape(n_head_kv, head_dim)
    amax = np.abs(v).max(axis=1)
    scale = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(amax > 0, np.float32(127.0) / np.where(amax > 0, amax, 1), 0).astype(np.float32)
    q = np.clip(np.rint(v * inv[:, None]), -127, 127).astype(np.int8)
    return q, scale


def attention_int8(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray, scale_k: np.ndarray,
                   scale_v: np.ndarray, seq_len: int, n_head: int, n_head_kv: int, head_dim: int) -> np.ndarray:
    """softmax(q . (int8 K * sk) / sqrt(hd)) . (int8 V * sv) -> bf16 bits, GQA by head // ratio
    (kernels.hip:499-586; the tiled variant :883-993 computes the same function)."""
    ratio = n_head // n_head_kv
    out = np.empty(n_head * head_dim, np.float32)
    qh = q.astype(np.float64).reshape(n_head, head_dim)
    for h in range(n_head):
        kv = h // ratio
        Kd = k_cache[:seq_len, kv, :].astype(np.float64) * scale_k[:seq_len, kv].astype(np.float64)[:, None]
        Vd = v_cache[:seq_len, kv, :].astype(np.float64) * scale_v[:seq_len, kv].astype(np.float64)[:, None]
        s = (Kd @ qh[h]) / np.sqrt(head_dim)
        s = np.exp(s - s.max())
        s /= s.sum()
        out[h * head_dim:(h + 1) * head_dim] = (s @ Vd).astype(np.float32)
    return f32_to_bf16_bits(out)


def argmax_first(logits: np.ndarray) -> int:
    """Index of the maximum logit; lowest index among exact ties (kernels.hip:90-122
    resolves ties by thread id; the rewrite fixes the rule to lowest index)."""
    return int(np.argmax(logits))


# ------------------------------------------------------------ whole decode step
class RefModel:
    """CPU restatement of one decode step at B = 1: the layer wiring of the reference's forward_b1
    (engine/inference.cpp:198-366) over the oracle's decode-then-fp32 GEMV and glue formulas.
    For small models only (pure numpy between the C GEMVs)."""

    def __init__(self, cfg, embd_bits, output_norm, output_proj, layers, max_seq):
        self.cfg = dict(cfg)
        self.embd = np.asarray(embd_bits, np.uint16).reshape(cfg["n_vocab"], cfg["n_embd"])
        self.output_norm = np.asarray(output_norm, np.float32)
        self.output_proj = output_proj
        self.layers = layers
        self.hd = cfg["n_embd"] // cfg["n_head"]
        nl, nkv = cfg["n_layer"], cfg["n_head_kv"]
        self.kc = np.zeros((nl, max_seq, nkv, self.hd), np.int8)
        self.vc = np.zeros((nl, max_seq, nkv, self.hd), np.int8)
        self.ks = np.zeros((nl, max_seq, nkv), np.float32)
        self.vs = np.zeros((nl, max_seq, nkv), np.float32)

    def step(self, token: int, pos: int) -> np.ndarray:
        c = self.cfg
        nh, nkv, hd, eps, theta = c["n_head"], c["n_head_kv"], self.hd, c["rms_norm_eps"], c["rope_theta"]
        cur = embed_lookup(self.embd, [token], c["n_vocab"])[0]
        a = None
        for li, L in enumerate(self.layers):
            if li == 0:
                a = rms_norm_bf16(cur, L["attn_norm"], eps)
            q = gemv(L["wq"], a)
            k = gemv(L["wk"], a)
            v = gemv(L["wv"], a)
            q = rope(q, pos, nh, hd, theta, c.get("rope_scaling"))
            k = rope(k, pos, nkv, hd, theta, c.get("rope_scaling"))
            self.kc[li, pos], self.ks[li, pos] = quant_kv_int8(k, nkv, hd)
            self.vc[li, pos], self.vs[li, pos] = quant_kv_int8(v, nkv, hd)
            att = attention_int8(q, self.kc[li], self.vc[li], self.ks[li], self.vs[li], pos + 1, nh, nkv, hd)
            res = gemv(L["wo"], att)
            res, a = add_rms_norm_bf16(res, cur, L["ffn_norm"], eps)
            b = silu_mul_bf16(gemv(L["w_gate"], a), gemv(L["w_up"], a))
            cur = gemv(L["w_down"], b)
            nxt = self.layers[li + 1]["attn_norm"] if li + 1 < len(self.layers) else self.output_norm
            cur, a = add_rms_norm_bf16(cur, res, nxt, eps)
        if not self.layers:
            a = rms_norm_bf16(cur, self.output_norm, eps)
        return gemv(self.output_proj, a)

    def generate(self, prompt, max_tokens, eos=2):
        """generate() of engine/inference.cpp:716-730 (greedy, stops at token id 2)."""
        logits = None
        for i, t in enumerate(prompt):
            logits = self.step(int(t), i)
        pos = len(prompt)
        out = []
        for _ in range(max_tokens):
            nxt = argmax_first(logits)
            if nxt == eos:
                break
            out.append(nxt)
            logits = self.step(nxt, pos)
            pos += 1
        return out
