"""CPU: pins the oracle's packer/decoder (no GPU, no product code).

Three independent anchors:
  1. byte equality with the arrays the REFERENCE C packer produced (golden fixture,
     written by tests/golden/make_golden.py from split12_pack.c);
  2. live equality with oracle/_ref when that library is present;
  3. what the format fixes by itself: lossless round trip, wrong == unpatched decode,
     brute-force window search.
"""
import ctypes as C

import numpy as np
import pytest

FIELDS = ["sm", "gr", "row_off", "cols", "correct", "wrong"]


def _check_against(o, w, be_expected, arrays, forced=None):
    be = o.find_base_exp(w)
    assert be == int(be_expected)
    p = o.pack(w, forced if forced is not None else be)
    for f in FIELDS:
        got = getattr(p, f)
        assert got.dtype == arrays[f].dtype, f
        assert np.array_equal(got, arrays[f]), f
    return p


def test_golden_cases_byte_exact(oracle, golden):
    assert len(golden) >= 13
    for name, g in golden.items():
        forced = int(g["base_exp"]) if int(g["base_exp"]) != int(g["found_base_exp"]) else None
        _check_against(oracle, g["w"], g["found_base_exp"], g, forced)


def test_golden_round_trip_and_wrong(oracle, golden):
    for name, g in golden.items():
        w = g["w"]
        p = oracle.pack(w, int(g["base_exp"]))
        assert np.array_equal(oracle.decode(p, patched=True), w), name
        un = oracle.decode(p, patched=False)
        rows = np.repeat(np.arange(p.M), np.diff(p.row_off))
        assert np.array_equal(un[rows, p.cols].view(np.int16), p.wrong), name
        # everything that is not an escape already decodes right without patches
        mask = np.ones_like(w, bool)
        mask[rows, p.cols] = False
        assert np.array_equal(un[mask], w[mask]), name


def test_live_reference_packer_matches(oracle):
    ref = oracle.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(7)
    for (M, K, sig, pout) in [(5, 12, 0.02, 0.0), (33, 130, 0.02, 0.01), (64, 1024, 0.05, 0.02), (1, 2, 1.0, 0.0),
                              (128, 4096, 0.02, 3e-4)]:
        w = rng.standard_normal((M, K)).astype(np.float32) * sig
        m = rng.random((M, K)) < pout
        w[m] = rng.standard_normal(int(m.sum())) * 8
        wb = oracle.f32_to_bf16_bits(w).reshape(M, K)
        n = M * K
        p16 = wb.ctypes.data_as(C.POINTER(C.c_uint16))
        be = ref.split12_find_base_exp(p16, n)
        sm = np.zeros(n, np.uint8); gr = np.zeros((n + 1) // 2, np.uint8); ro = np.zeros(M + 1, np.int32)
        cols = np.zeros(n, np.int32); cor = np.zeros(n, np.int16); wr = np.zeros(n, np.int16)
        P = ref.pack_split12(p16, M, K, be, sm.ctypes.data_as(C.POINTER(C.c_uint8)),
                             gr.ctypes.data_as(C.POINTER(C.c_uint8)), ro.ctypes.data_as(C.POINTER(C.c_int32)),
                             cols.ctypes.data_as(C.POINTER(C.c_int32)), cor.ctypes.data_as(C.POINTER(C.c_int16)),
                             wr.ctypes.data_as(C.POINTER(C.c_int16)))
        _check_against(oracle, wb, be, dict(sm=sm, gr=gr, row_off=ro, cols=cols[:P], correct=cor[:P], wrong=wr[:P]))


def test_find_base_exp_brute_force(oracle):
    rng = np.random.default_rng(11)
    for trial in range(40):
        n = int(rng.integers(1, 200))
        centre = int(rng.integers(0, 256))
        e = np.clip(centre + rng.integers(-12, 13, size=n), 0, 255).astype(np.uint16)
        w = (e << 7) | rng.integers(0, 128, size=n).astype(np.uint16) | (rng.integers(0, 2, size=n).astype(np.uint16) << 15)
        hist = np.bincount(e, minlength=256)
        sums = [hist[s:s + 15].sum() for s in range(242)]
        expect = int(np.argmax(sums)) - 1   # argmax returns the earliest maximum
        assert oracle.find_base_exp(w) == expect
    assert oracle.find_base_exp(np.zeros(0, np.uint16)) == -1
    assert oracle.find_base_exp(np.zeros(9, np.uint16)) == -1


def test_escape_tables_brute_force(oracle, golden):
    for name in ["outliers_16x256", "llm_64x512", "diffusion_32x1280", "forced_be_8x64", "zeros_4x32"]:
        g = golden[name]
        p = oracle.pack(g["w"], int(g["base_exp"]))
        row_base, counts, vals, nonempty = oracle.escape_tables(p)
        assert np.array_equal(row_base, p.row_off[:-1])
        cnt = counts.reshape(p.M, 256).astype(np.int64)
        assert np.array_equal(cnt.sum(axis=1), np.diff(p.row_off))
        exp_vals = []
        for r in range(p.M):
            sl = slice(p.row_off[r], p.row_off[r + 1])
            c, v = p.cols[sl], p.correct[sl]
            order = np.lexsort((c, c % 256))
            exp_vals.append(v[order])
            assert np.array_equal(np.bincount(c % 256, minlength=256), cnt[r])
        exp_vals = np.concatenate(exp_vals) if exp_vals else np.zeros(0, np.int16)
        assert np.array_equal(vals, exp_vals)
        assert np.array_equal(nonempty, np.nonzero(np.diff(p.row_off))[0])


def test_gemm_matches_float64_matmul(oracle):
    import importlib.util, os
    rng = np.random.default_rng(3)
    M, K, B = 96, 512, 5
    w = rng.standard_normal((M, K)).astype(np.float32) * 0.02
    m = rng.random((M, K)) < 0.01
    w[m] = rng.standard_normal(int(m.sum())) * 8
    wb = oracle.f32_to_bf16_bits(w).reshape(M, K)
    xb = oracle.f32_to_bf16_bits(rng.standard_normal((B, K)).astype(np.float32)).reshape(B, K)
    p = oracle.pack(wb)
    assert p.P > 0
    W = oracle.bf16_bits_to_f32(wb).reshape(M, K).astype(np.float64)
    X = oracle.bf16_bits_to_f32(xb).reshape(B, K).astype(np.float64)
    truth = X @ W.T
    got = oracle.gemm(p, xb)
    assert got.shape == (B, M)
    assert np.allclose(got, truth, rtol=1e-4, atol=1e-4)
    # unpatched + patch correction == patched, to fp32 rounding (the B=1 reference recipe)
    un = oracle.gemv(p, xb[0], patched=False).copy()
    assert not np.allclose(un, truth[0], rtol=1e-3, atol=1e-3)   # escapes matter
    oracle.apply_patches(p, xb[0], un)
    assert np.allclose(un, truth[0], rtol=1e-4, atol=1e-4)


def test_bf16_rounding_rule(oracle):
    x = np.array([1.0, 1.00390625, 1.01171875, -3.0e-40, 65504.0, 3.3895314e38], np.float32)
    b = oracle.f32_to_bf16_bits(x)
    # 1.00390625 = 0x3F808000 is a tie -> even (0x3F80); 1.01171875 = 0x3F818000 tie -> 0x3F82
    assert list(b[:3]) == [0x3F80, 0x3F80, 0x3F82]
    assert np.array_equal(oracle.bf16_bits_to_f32(b).view(np.uint32) >> 16, b)
