"""Writer of the model directory layout the engine's load_model reads -- the files
the reference's converter emits (engine/convert_model.py:57-62,127-152):
config.bin, tok_embd.bin, *_norm.bin and seven files per tensor."""
from __future__ import annotations

import os
import struct

import numpy as np

TENSORS = ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")


def write_config(path, cfg):
    """config.bin, and rope_scaling.bin (factor, low_freq_factor, high_freq_factor, original context: four
    float32; an addition to the reference's layout) when cfg carries a "rope_scaling" tuple."""
    with open(os.path.join(path, "config.bin"), "wb") as f:
        f.write(struct.pack("<iiiiiiiff", cfg["n_vocab"], cfg["n_embd"], cfg["n_head"], cfg["n_head_kv"],
                            cfg["n_layer"], cfg["n_ff"], cfg["n_ctx"], cfg["rope_theta"], cfg["rms_norm_eps"]))
    if cfg.get("rope_scaling"):
        with open(os.path.join(path, "rope_scaling.bin"), "wb") as f:
            f.write(struct.pack("<ffff", *cfg["rope_scaling"]))


def write_tensor(path, prefix, p):
    """p: anything with M, K, base_exp, sm, gr, row_off, cols, correct, wrong (numpy arrays)."""
    base = os.path.join(path, prefix)
    np.ascontiguousarray(p.sm, np.uint8).tofile(base + ".sm.bin")
    np.ascontiguousarray(p.gr, np.uint8).tofile(base + ".gr.bin")
    np.ascontiguousarray(p.row_off, np.int32).tofile(base + ".row_off.bin")
    np.ascontiguousarray(p.cols, np.int32).tofile(base + ".patch_cols.bin")
    np.ascontiguousarray(p.correct, np.int16).tofile(base + ".patch_correct.bin")
    np.ascontiguousarray(p.wrong, np.int16).tofile(base + ".patch_wrong.bin")
    with open(base + ".dims", "w") as f:
        f.write("%d %d %d %d" % (p.M, p.K, len(p.cols), p.base_exp))


def write_model_dir(path, cfg, embd_bits, output_norm, output_proj, layers):
    """layers: list of dicts with attn_norm, ffn_norm (fp32 arrays) and the seven packed tensors."""
    os.makedirs(path, exist_ok=True)
    write_config(path, cfg)
    np.ascontiguousarray(embd_bits, np.uint16).tofile(os.path.join(path, "tok_embd.bin"))
    np.ascontiguousarray(output_norm, np.float32).tofile(os.path.join(path, "output_norm.bin"))
    write_tensor(path, "output_proj", output_proj)
    for i, L in enumerate(layers):
        np.ascontiguousarray(L["attn_norm"], np.float32).tofile(os.path.join(path, "layer.%d.attn_norm.bin" % i))
        np.ascontiguousarray(L["ffn_norm"], np.float32).tofile(os.path.join(path, "layer.%d.ffn_norm.bin" % i))
        for t in TENSORS:
            write_tensor(path, "layer.%d.%s" % (i, t), L[t])


def read_tensor(path, prefix):
    """Inverse of write_tensor: a plain object holding the arrays of one tensor."""
    base = os.path.join(path, prefix)
    M, K, P, be = (int(x) for x in open(base + ".dims").read().split())

    class T:
        pass

    t = T()
    t.M, t.K, t.base_exp = M, K, be
    t.sm = np.fromfile(base + ".sm.bin", np.uint8)
    t.gr = np.fromfile(base + ".gr.bin", np.uint8)
    t.row_off = np.fromfile(base + ".row_off.bin", np.int32)
    t.cols = np.fromfile(base + ".patch_cols.bin", np.int32)
    t.correct = np.fromfile(base + ".patch_correct.bin", np.int16)
    t.wrong = np.fromfile(base + ".patch_wrong.bin", np.int16)
    assert len(t.cols) == P
    return t
