"""Writes tests/golden/pack_cases.npz: inputs and the arrays the REFERENCE C packer
(oracle/_ref/libsplit12_ref.so, compiled from /root/reference/split12_pack.c by
oracle/Makefile) emits for them.  Run in the build container, where the reference
tree is mounted:   python tests/golden/make_golden.py

The fixture holds data only: bf16 inputs, base_exp, sm, gr, row_off, cols, correct,
wrong per case.
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle  # noqa: E402


def bf16(x):
    return oracle.f32_to_bf16_bits(np.asarray(x, np.float32))


def cases():
    rng = np.random.default_rng(20240611)
    out = {}
    out["normal_8x64"] = bf16(rng.standard_normal((8, 64)) * 0.02)
    w = rng.standard_normal((16, 256)) * 0.02
    w[rng.random((16, 256)) < 0.01] = 7.5
    w[3, 17] = -300.0
    out["outliers_16x256"] = bf16(w)
    out["tiny_3x6"] = bf16(rng.standard_normal((3, 6)))
    # odd K: the nibble of the last element of a row shares a byte with the next row
    out["oddK_3x5"] = bf16(rng.standard_normal((3, 5)) * 0.1)
    out["oddcount_1x7"] = bf16(rng.standard_normal((1, 7)) * 4)
    out["zeros_4x32"] = np.zeros((4, 32), np.uint16)
    sp = bf16(rng.standard_normal((4, 64)) * 0.02)
    sp[0, 0] = 0x7F80   # +Inf
    sp[0, 1] = 0xFF80   # -Inf
    sp[1, 5] = 0x7FC1   # NaN
    sp[2, 9] = 0x0001   # smallest subnormal
    sp[2, 10] = 0x807F  # negative subnormal
    sp[3, 63] = 0x8000  # -0
    out["special_4x64"] = sp
    # two windows with equal population: the earliest must win
    tie = np.empty((2, 30), np.uint16)
    tie[0] = (np.arange(30) % 15 + 40).astype(np.uint16) << 7
    tie[1] = (np.arange(30) % 15 + 120).astype(np.uint16) << 7
    out["tie_2x30"] = tie
    # exponents at the top of the range (window 241..255 -> base_exp 240)
    hi = ((np.arange(64) % 20 + 236).clip(0, 255).astype(np.uint16) << 7) | (np.arange(64) % 128).astype(np.uint16)
    hi[::3] |= 0x8000
    out["high_exp_2x32"] = hi.reshape(2, 32)
    top = ((np.arange(60) % 15 + 241).astype(np.uint16) << 7) | (np.arange(60) % 128).astype(np.uint16)
    out["top_window_2x30"] = top.reshape(2, 30)
    # exponents at the bottom (subnormals + tiny): base_exp -1 or 0
    lo = ((np.arange(96) % 18).astype(np.uint16) << 7) | (np.arange(96) * 7 % 128).astype(np.uint16)
    out["low_exp_3x32"] = lo.reshape(3, 32)
    w = rng.standard_normal((64, 512)) * 0.02
    m = rng.random((64, 512)) < 3e-3
    w[m] = rng.standard_normal(int(m.sum())) * 8
    out["llm_64x512"] = bf16(w)
    w = rng.standard_normal((32, 1280)) * 0.05
    m = rng.random((32, 1280)) < 0.02
    w[m] = rng.standard_normal(int(m.sum()))
    out["diffusion_32x1280"] = bf16(w)
    # a forced (not optimal) base_exp: pack must honour whatever it is given
    out["forced_be_8x64"] = bf16(rng.standard_normal((8, 64)) * 0.5)
    return out


FORCED = {"forced_be_8x64": 100}


def main():
    ref = oracle.ref_lib()
    if ref is None:
        raise SystemExit("oracle/_ref/libsplit12_ref.so missing: run `make -C oracle` with the reference mounted")
    blob = {}
    for name, w in cases().items():
        w = np.ascontiguousarray(w, np.uint16)
        M, K = w.shape
        n = M * K
        p16 = w.ctypes.data_as(C.POINTER(C.c_uint16))
        be = ref.split12_find_base_exp(p16, n)
        blob[name + ".found_base_exp"] = np.int32(be)
        be = FORCED.get(name, be)
        sm = np.zeros(n, np.uint8)
        gr = np.zeros((n + 1) // 2, np.uint8)
        ro = np.zeros(M + 1, np.int32)
        cols = np.zeros(n, np.int32)
        cor = np.zeros(n, np.int16)
        wr = np.zeros(n, np.int16)
        P = ref.pack_split12(p16, M, K, be, sm.ctypes.data_as(C.POINTER(C.c_uint8)),
                             gr.ctypes.data_as(C.POINTER(C.c_uint8)), ro.ctypes.data_as(C.POINTER(C.c_int32)),
                             cols.ctypes.data_as(C.POINTER(C.c_int32)), cor.ctypes.data_as(C.POINTER(C.c_int16)),
                             wr.ctypes.data_as(C.POINTER(C.c_int16)))
        blob[name + ".w"] = w
        blob[name + ".base_exp"] = np.int32(be)
        blob[name + ".sm"] = sm
        blob[name + ".gr"] = gr
        blob[name + ".row_off"] = ro
        blob[name + ".cols"] = cols[:P].copy()
        blob[name + ".correct"] = cor[:P].copy()
        blob[name + ".wrong"] = wr[:P].copy()
        print(f"{name:22s} {M}x{K} base_exp={be} P={P}")
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pack_cases.npz")
    np.savez_compressed(path, **blob)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
