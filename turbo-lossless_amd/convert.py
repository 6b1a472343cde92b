"""safetensors checkpoint (Hugging Face Llama / Mistral naming) -> split-12 model directory.

    convert(hf_model_dir, output_dir)

Counterpart of the reference converter (engine/convert_model.py:40-197): same config keys and
fallbacks (:46-54), same `config.bin` struct (:57-60), same tensor naming (:144-183), same
per-tensor file set (:127-134).  What differs:

* the packing runs on the GPU (`t12_pack_*`: histogram -> base_exp -> planes -> CSR escapes)
  instead of the C packer on the host, with byte-identical output;
* the safetensors container is read here (8-byte little-endian header length, JSON header,
  raw little-endian tensors), memory-mapped, without torch or the safetensors package;
* fp16 / fp32 sources are rounded to bf16 with round-to-nearest-even, NaN -> 0x7FC0, which is
  what `Tensor.to(torch.bfloat16)` does (:159,190);
* a checkpoint without `lm_head` (tied embeddings) gets `output_proj` packed from the
  embedding matrix; the reference writes no `output_proj` there and its loader then reads
  uninitialised memory (engine/model.cpp:209-211);
* a `rope_scaling` entry of type "llama3" is kept (`rope_scaling.bin`, four little-endian
  floats: factor, low_freq_factor, high_freq_factor, original_max_position_embeddings); the
  reference drops it (:54).
"""
from __future__ import annotations

import glob
import json
import mmap
import os
import struct
import time

import numpy as np

from . import modelio

_DTYPES = {"BF16": (np.uint16, 2), "F16": (np.float16, 2), "F32": (np.float32, 4), "F64": (np.float64, 8)}


class SafetensorsFile:
    """Read-only view of one .safetensors file."""

    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise ValueError("%s: too short for a safetensors header" % path)
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8 or n > (100 << 20):
            raise ValueError("%s: header length %d does not fit the file" % (path, n))
        header = json.loads(self._f.read(n).decode("utf-8"))
        header.pop("__metadata__", None)
        self._base = 8 + n
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self.entries = {}
        for name, e in header.items():
            b, end = e["data_offsets"]
            shape = tuple(int(d) for d in e["shape"])
            dt = e["dtype"]
            if dt in _DTYPES:
                want = int(np.prod(shape, dtype=np.int64)) * _DTYPES[dt][1]
                if end - b != want or self._base + end > size:
                    raise ValueError("%s: tensor %s has %d bytes, shape %s %s needs %d" %
                                     (path, name, end - b, shape, dt, want))
            self.entries[name] = (dt, shape, b, end)

    def keys(self):
        return list(self.entries)

    def info(self, name):
        dt, shape, _, _ = self.entries[name]
        return dt, shape

    def get(self, name) -> np.ndarray:
        """The tensor as a numpy view of the mapping; bf16 comes back as its uint16 bit patterns."""
        dt, shape, b, e = self.entries[name]
        if dt not in _DTYPES:
            raise TypeError("%s: dtype %s of %s is not a floating-point weight type" % (self.path, dt, name))
        return np.frombuffer(self._mm, dtype=np.dtype(_DTYPES[dt][0]).newbyteorder("<"), count=(e - b) // _DTYPES[dt][1],
                             offset=self._base + b).reshape(shape)

    def close(self):
        # numpy views of the mapping may still be alive: leave the unmapping to the collector
        self._f.close()


def to_bf16_bits(a: np.ndarray, dtype: str) -> np.ndarray:
    """Weight values -> bf16 bit patterns (uint16), rounding as Tensor.to(torch.bfloat16) does."""
    if dtype == "BF16":
        return np.ascontiguousarray(a, dtype=np.uint16)
    f = np.ascontiguousarray(a, dtype=np.float32)      # fp16 -> fp32 is exact; fp64 -> fp32 rounds to nearest even first
    u = f.view(np.uint32)
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    if nan.any():
        r[nan] = 0x7FC0
    return r


def read_config(model_dir: str) -> dict:
    """config.json -> the nine values of config.bin, with the reference's key fallbacks
    (engine/convert_model.py:46-54), plus `rope_scaling` when it is of the llama3 kind."""
    with open(os.path.join(model_dir, "config.json")) as f:
        c = json.load(f)
    n_embd = c.get("hidden_size", c.get("dim", 4096))
    n_head = c.get("num_attention_heads", c.get("n_heads", 32))
    cfg = dict(
        n_vocab=c.get("vocab_size", 32000), n_embd=n_embd, n_head=n_head,
        n_head_kv=c.get("num_key_value_heads", c.get("n_kv_heads", n_head)),
        n_layer=c.get("num_hidden_layers", c.get("n_layers", 32)),
        n_ff=c.get("intermediate_size", c.get("hidden_dim", n_embd * 4)),
        n_ctx=c.get("max_position_embeddings", c.get("max_seq_len", 32768)),
        rope_theta=float(c.get("rope_theta", 10000.0)), rms_norm_eps=float(c.get("rms_norm_eps", 1e-5)))
    rs = c.get("rope_scaling")
    if isinstance(rs, dict) and rs.get("rope_type", rs.get("type")) == "llama3":
        cfg["rope_scaling"] = (float(rs["factor"]), float(rs.get("low_freq_factor", 1.0)),
                               float(rs.get("high_freq_factor", 4.0)),
                               float(rs.get("original_max_position_embeddings", 8192)))
    return cfg


class Checkpoint:
    """All *.safetensors shards of a directory under one name space."""

    def __init__(self, model_dir: str):
        self.files = [SafetensorsFile(p) for p in sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))]
        if not self.files:
            raise FileNotFoundError("no *.safetensors in %s" % model_dir)
        self.where = {}
        for f in self.files:
            for k in f.keys():
                self.where.setdefault(k, f)

    def find(self, pattern: str):
        """`model.<pattern>.weight` or `<pattern>.weight` when present, else the first tensor name
        that contains the pattern (the reference's rule, engine/convert_model.py:75-79)."""
        for cand in ("model.%s.weight" % pattern, "%s.weight" % pattern, pattern):
            if cand in self.where:
                return cand
        for name in self.where:
            if pattern in name:
                return name
        return None

    def bf16(self, name):
        """(bits uint16 ndarray, source dtype) of a tensor."""
        f = self.where[name]
        dt, _ = f.info(name)
        return to_bf16_bits(f.get(name), dt), dt

    def f32(self, name):
        f = self.where[name]
        dt, _ = f.info(name)
        a = f.get(name)
        if dt == "BF16":
            return (a.astype(np.uint32) << 16).view(np.float32)
        return np.ascontiguousarray(a, dtype=np.float32)

    def close(self):
        for f in self.files:
            f.close()


LAYER_TENSORS = (("wq", "self_attn.q_proj"), ("wk", "self_attn.k_proj"), ("wv", "self_attn.v_proj"),
                 ("wo", "self_attn.o_proj"), ("w_gate", "mlp.gate_proj"), ("w_up", "mlp.up_proj"),
                 ("w_down", "mlp.down_proj"))


class _HostPacked:
    pass


def pack_bits_on_gpu(t12, bits: np.ndarray, device):
    """bf16 bit patterns [M, K] -> packed planes and CSR list as host arrays (packed on the GPU)."""
    import torch

    w = torch.from_numpy(np.array(bits, dtype=np.uint16, order="C", copy=True).view(np.int16)).to(device)
    d = t12.pack_device(w)
    p = _HostPacked()
    p.M, p.K, p.base_exp = d.M, d.K, d.base_exp
    p.sm, p.gr = d.sm.cpu().numpy(), d.gr.cpu().numpy()
    p.row_off = d.row_off.cpu().numpy()
    p.cols, p.correct, p.wrong = d.cols.cpu().numpy(), d.correct.cpu().numpy(), d.wrong.cpu().numpy()
    return p


def convert(model_dir: str, output_dir: str, device="cuda:0", log=None) -> dict:
    """Writes the engine's model directory for the checkpoint in `model_dir`; returns
    {tensor prefix: (M, K, escapes, base_exp)}."""
    import importlib

    t12 = importlib.import_module(__package__)      # raises when the HIP library is missing: no CPU packer here

    log = log or (lambda *a: None)
    cfg = read_config(model_dir)
    ck = Checkpoint(model_dir)
    os.makedirs(output_dir, exist_ok=True)
    modelio.write_config(output_dir, cfg)
    stats = {}
    t0 = time.time()

    def compressed(prefix, name):
        bits, dt = ck.bf16(name)
        if bits.ndim != 2:
            raise ValueError("%s: expected a matrix, got shape %s" % (name, bits.shape))
        p = pack_bits_on_gpu(t12, bits, device)
        modelio.write_tensor(output_dir, prefix, p)
        stats[prefix] = (p.M, p.K, len(p.cols), p.base_exp)
        log("  %s <- %s %s %dx%d escapes=%d base_exp=%d" % (prefix, name, dt, p.M, p.K, len(p.cols), p.base_exp))

    embd = ck.find("embed_tokens")
    if embd is None:
        raise KeyError("no embed_tokens tensor in %s" % model_dir)
    bits, _ = ck.bf16(embd)
    if bits.shape != (cfg["n_vocab"], cfg["n_embd"]):
        raise ValueError("embed_tokens is %s, config.json says %s" % (bits.shape, (cfg["n_vocab"], cfg["n_embd"])))
    bits.tofile(os.path.join(output_dir, "tok_embd.bin"))
    norm = next((n for n in ("model.norm.weight", "norm.weight") if n in ck.where), None) or ck.find("model.norm.weight")
    if norm is None:
        raise KeyError("no model.norm.weight tensor in %s" % model_dir)
    ck.f32(norm).tofile(os.path.join(output_dir, "output_norm.bin"))
    head = ck.find("lm_head")
    compressed("output_proj", head if head is not None else embd)       # tied embeddings: head = embedding matrix
    for i in range(cfg["n_layer"]):
        for hf, ours in (("input_layernorm", "attn_norm"), ("post_attention_layernorm", "ffn_norm")):
            name = ck.find("layers.%d.%s" % (i, hf))
            if name is None:
                raise KeyError("layer %d: no %s" % (i, hf))
            ck.f32(name).tofile(os.path.join(output_dir, "layer.%d.%s.bin" % (i, ours)))
        for ours, hf in LAYER_TENSORS:
            name = ck.find("layers.%d.%s" % (i, hf))
            if name is None:
                raise KeyError("layer %d: no %s" % (i, hf))
            compressed("layer.%d.%s" % (i, ours), name)
    ck.close()
    log("converted %d tensors in %.1f s -> %s" % (len(stats), time.time() - t0, output_dir))
    return stats

