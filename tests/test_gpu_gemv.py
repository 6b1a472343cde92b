"""GPU parity: split-12 decode-GEMV (B = 1) through the C ABI vs the CPU oracle.

Tolerance: the target is outputs within 1e-2 relative of the
decode-then-fp32-accumulate reference.  The kernels accumulate in fp32 like the
oracle, so the observed error is ~1e-6; the assertions use 1e-4 to catch a wrong
pairing / dropped tile, which would show at 1e-2..1.
"""
import importlib

import numpy as np
import pytest
import torch

from gpu_util import dev, rel_err, to_dev_bits

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def synth(t12):
    return importlib.import_module("turbo_lossless_amd.synth")


def run_gemv(t12, packs, x, patched=True):
    dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in packs]
    outs = t12.gemv(dts, to_dev_bits(x), patched=patched)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs]


@pytest.mark.parametrize("M,K", [(4096, 4096), (1024, 4096), (256, 14336), (300, 1280), (77, 5120),
                                 (1, 1024), (9, 16), (64, 1040), (5, 2064), (16, 20480), (8, 28672), (3, 16400)])
def test_gemv_llm_law(t12, oracle, synth, M, K):
    """(Rows wider than 16384 columns stage the rest of the activations in a loop behind the pieces requested up front.)"""
    w = synth.weights_llm(M, K, seed=1001 + M + K, p_outlier=3e-4 if M * K > 1e5 else 2e-2)
    x = synth.activations(1, K, seed=1002)[0]
    p = oracle.pack(w)
    (got,) = run_gemv(t12, [p], x)
    assert rel_err(got, oracle.gemv(p, x)) < TOL


def test_gemv_config1_escape_statistics(t12, oracle, synth):
    """Single-tensor case: 4096x4096 N(0,.02) + 0.03 % N(0,8) outliers."""
    w = synth.weights_llm(4096, 4096, seed=1001)
    x = synth.activations(1, 4096, seed=1002)[0]
    p = oracle.pack(w)
    assert p.base_exp == 108 and 0.0003 < p.P / w.size < 0.0007
    (got,) = run_gemv(t12, [p], x)
    ref = oracle.gemv(p, x)
    assert rel_err(got, ref) < TOL
    # escapes matter: dropping the patch list must be visible
    (un,) = run_gemv(t12, [p], x, patched=False)
    assert rel_err(un, oracle.gemv(p, x, patched=False)) < TOL
    assert rel_err(un, ref) > 1e-2


def test_gemv_escape_heavy(t12, oracle, synth):
    """Diffusion-UNet-like weight law: every row holds several escapes."""
    for (M, K) in [(1280, 5120), (640, 1280)]:
        w = synth.weights_diffusion(M, K, seed=3000 + M)
        x = synth.activations(1, K, seed=3001)[0]
        p = oracle.pack(w)
        assert p.P > 2 * M and (K < 5120 or np.all(np.diff(p.row_off) > 0))
        (got,) = run_gemv(t12, [p], x)
        assert rel_err(got, oracle.gemv(p, x)) < TOL


def test_gemv_fused_segments(t12, oracle, synth):
    """wq|wk|wv in one launch: three tensors, three base_exp, one activation vector."""
    K = 2048
    ws = [synth.weights_llm(512, K, seed=1, sigma=0.02), synth.weights_llm(130, K, seed=2, sigma=0.3),
          synth.weights_llm(128, K, seed=3, sigma=0.002)]
    x = synth.activations(1, K, seed=4)[0]
    ps = [oracle.pack(w) for w in ws]
    assert len({p.base_exp for p in ps}) == 3
    gots = run_gemv(t12, ps, x)
    for g, p in zip(gots, ps):
        assert rel_err(g, oracle.gemv(p, x)) < TOL


def test_gemv_eight_segments(t12, oracle, synth):
    K = 1024
    ps = [oracle.pack(synth.weights_llm(8 + 3 * i, K, seed=10 + i, sigma=0.01 * (i + 1))) for i in range(8)]
    x = synth.activations(1, K, seed=5)[0]
    for g, p in zip(run_gemv(t12, ps, x), ps):
        assert rel_err(g, oracle.gemv(p, x)) < TOL


def test_gemv_general_path(t12, oracle, synth, golden):
    """Odd K, K % 16 != 0, base_exp = -1 and the reference-packed golden cases."""
    rng = np.random.default_rng(5)
    for name, g in golden.items():
        w = g["w"]
        M, K = w.shape
        p = oracle.pack(w, int(g["base_exp"]))
        x = oracle.f32_to_bf16_bits(rng.standard_normal(K).astype(np.float32))
        if name in ("special_4x64", "high_exp_2x32", "top_window_2x30"):
            # weights up to 2^127 and Inf / NaN patterns (all of them escapes): activations of magnitude ~2^-100
            # keep every finite product finite; rows that hold an Inf or NaN weight must come out as the same
            # kind of non-finite value, the others within the tolerance.  high_exp_2x32 (K = 32, base_exp 235)
            # takes the fast kernel, the other two the general one.
            x = oracle.f32_to_bf16_bits((rng.uniform(0.5, 1.0, K) * rng.choice([-1.0, 1.0], K) * 2.0 ** -100).astype(np.float32))
            (got,) = run_gemv(t12, [p], x)
            ref = oracle.gemv(p, x)
            assert np.array_equal(np.isnan(got), np.isnan(ref)), name
            assert np.array_equal(np.isposinf(got), np.isposinf(ref)) and np.array_equal(np.isneginf(got), np.isneginf(ref)), name
            fin = np.isfinite(ref)
            if fin.any():
                assert rel_err(got[fin], ref[fin]) < TOL, name
            continue
        (got,) = run_gemv(t12, [p], x)
        ref = oracle.gemv(p, x)
        assert rel_err(got, ref) < TOL, name
    w = synth.weights_llm(33, 1001, seed=9, p_outlier=0.01)
    x = synth.activations(1, 1001, seed=9)[0]
    p = oracle.pack(w)
    (got,) = run_gemv(t12, [p], x)
    assert rel_err(got, oracle.gemv(p, x)) < TOL


def test_gemv_nonfinite(t12, oracle, synth):
    """An Inf weight (always an escape here) must surface as Inf in exactly its row."""
    w = synth.weights_llm(32, 1024, seed=21, p_outlier=0)
    w[5, 100] = 0x7F80
    x = synth.activations(1, 1024, seed=22)[0]
    x[100] = 0x3F80  # 1.0
    p = oracle.pack(w)
    (got,) = run_gemv(t12, [p], x)
    ref = oracle.gemv(p, x)
    assert np.isinf(got[5]) and np.isinf(ref[5])
    mask = np.ones(32, bool); mask[5] = False
    assert rel_err(got[mask], ref[mask]) < TOL


def test_reference_named_launchers(t12, oracle, synth):
    """launch_split12_v2_async (+dual) give the UNPATCHED product; the patch launchers add
    (correct - wrong) * x -- the call sequence of the reference's forward_b1."""
    M, K = 256, 2048
    pa = oracle.pack(synth.weights_llm(M, K, seed=41, p_outlier=2e-3))
    pb = oracle.pack(synth.weights_llm(M, K, seed=42, sigma=0.2, p_outlier=2e-3))
    x = synth.activations(1, K, seed=43)[0]
    xd = to_dev_bits(x)
    st = t12.current_stream()
    da, db = (t12.DeviceTensor12.from_packed(p, dev()) for p in (pa, pb))
    oa = torch.zeros(M, device=dev()); ob = torch.zeros(M, device=dev())
    t12.check(t12.lib.launch_split12_v2_async(da.sm.data_ptr(), da.gr.data_ptr(), da.base_exp, xd.data_ptr(),
                                              oa.data_ptr(), M, K, st))
    torch.cuda.synchronize()
    assert rel_err(oa.cpu().numpy(), oracle.gemv(pa, x, patched=False)) < TOL
    t12.check(t12.lib.launch_patches_v2_async(da.row_off.data_ptr(), da.cols.data_ptr(), da.correct.data_ptr(),
                                              da.wrong.data_ptr(), xd.data_ptr(), oa.data_ptr(), M, st))
    torch.cuda.synchronize()
    assert rel_err(oa.cpu().numpy(), oracle.gemv(pa, x)) < TOL
    # dual + batched patches
    oa.zero_()
    t12.check(t12.lib.launch_split12_v2_dual_async(da.sm.data_ptr(), da.gr.data_ptr(), da.base_exp,
                                                   db.sm.data_ptr(), db.gr.data_ptr(), db.base_exp, xd.data_ptr(),
                                                   oa.data_ptr(), ob.data_ptr(), M, K, st))
    descs = (t12.PatchBatchDesc * 2)(
        t12.PatchBatchDesc(da.row_off.data_ptr(), da.cols.data_ptr(), da.correct.data_ptr(), da.wrong.data_ptr(),
                           xd.data_ptr(), oa.data_ptr(), M),
        t12.PatchBatchDesc(db.row_off.data_ptr(), db.cols.data_ptr(), db.correct.data_ptr(), db.wrong.data_ptr(),
                           xd.data_ptr(), ob.data_ptr(), M))
    scratch = torch.zeros(8 * 56, dtype=torch.uint8, device=dev())
    t12.check(t12.lib.launch_patches_b1_batched_async(scratch.data_ptr(), descs, 2, M, st))
    torch.cuda.synchronize()
    assert rel_err(oa.cpu().numpy(), oracle.gemv(pa, x)) < TOL
    assert rel_err(ob.cpu().numpy(), oracle.gemv(pb, x)) < TOL


def test_patch_launchers_ragged_rows_and_heavy_rows(t12, oracle, synth):
    """The patch launchers alone, on a zeroed output: a row count that is no multiple of the rows a workgroup takes,
    rows with 0, 1, 9, 70 and 300 entries, two descriptors of different M in one call; the sum of a row's entries
    against float64."""
    K = 4096
    shapes = [(77, 51), (1000, 52)]
    rng = np.random.default_rng(53)
    x = synth.activations(1, K, seed=54)[0]
    xd = to_dev_bits(x)
    xf = oracle.bf16_bits_to_f32(x).astype(np.float64)
    packs, devs, outs = [], [], []
    for M, seed in shapes:
        w = synth.weights_llm(M, K, seed=seed, p_outlier=3e-4).copy()
        for r, n in ((0, 1), (M // 2, 9), (M - 2, 70), (M - 1, 300)):
            w[r, rng.choice(K, n, replace=False)] = oracle.f32_to_bf16_bits(rng.uniform(3.0, 60.0, n).astype(np.float32))
        p = oracle.pack(w)
        packs.append(p)
        devs.append(t12.DeviceTensor12.from_packed(p, dev()))
        outs.append(torch.zeros(M, device=dev()))
    descs = (t12.PatchBatchDesc * 2)(*[
        t12.PatchBatchDesc(d.row_off.data_ptr(), d.cols.data_ptr(), d.correct.data_ptr(), d.wrong.data_ptr(),
                           xd.data_ptr(), o.data_ptr(), d.M) for d, o in zip(devs, outs)])
    scratch = torch.zeros(8 * 56, dtype=torch.uint8, device=dev())
    t12.check(t12.lib.launch_patches_b1_batched_async(scratch.data_ptr(), descs, 2, 1000, t12.current_stream()))
    torch.cuda.synchronize()
    for p, o in zip(packs, outs):
        delta = oracle.bf16_bits_to_f32(p.correct.view(np.uint16)).astype(np.float64) - \
                oracle.bf16_bits_to_f32(p.wrong.view(np.uint16)).astype(np.float64)
        want = np.zeros(p.M)
        np.add.at(want, np.repeat(np.arange(p.M), np.diff(p.row_off)), delta * xf[p.cols])
        got = o.cpu().numpy()
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
        assert (got[np.diff(p.row_off) == 0] == 0).all()


def test_gemv_rejects_bad_operands(t12):
    segs = (t12.Segment * 1)(t12.Segment(None, None, None, None, None, None, None, 4, 100, 0, 0))
    x = torch.zeros(16, dtype=torch.int16, device=dev())
    assert t12.lib.t12_gemv(segs, 1, x.data_ptr(), 16, None) == -1
    assert b"null" in t12.lib.t12_last_error()
    assert t12.lib.t12_gemv(segs, 0, x.data_ptr(), 16, None) == -1
    assert t12.lib.t12_gemv(segs, 9, x.data_ptr(), 16, None) == -1


def test_full_size_linearity(t12, oracle, synth):
    """Size-independent property at a full Llama layer shape (down: 4096 x 14336):
    W.(x1 + x2) == W.x1 + W.x2 when x1, x2 have disjoint support (so the bf16 sum is exact)."""
    M, K = 4096, 14336
    w = synth.weights_llm(M, K, seed=2003)
    p = oracle.pack(w)
    x = synth.activations(1, K, seed=2004)[0]
    x1 = x.copy(); x1[K // 2:] = 0
    x2 = x.copy(); x2[:K // 2] = 0
    dt = t12.DeviceTensor12.from_packed(p, dev())
    o, o1, o2 = (t12.gemv(dt, to_dev_bits(v))[0].clone() for v in (x, x1, x2))
    torch.cuda.synchronize()
    assert rel_err((o1 + o2).cpu().numpy(), o.cpu().numpy()) < 1e-5
    ref = oracle.gemv(p, x)
    assert rel_err(o.cpu().numpy(), ref) < TOL


def _run_batch_launcher(t12, NB, d, acts, tables, M, K):
    """launch_split12_batch{NB}_async on device tensor d; tables = (row_base, counts or None, vals) or None."""
    fn = t12.lib.launch_split12_batch4_async if NB == 4 else t12.lib.launch_split12_batch8_async
    outs = [torch.zeros(M, device=dev()) for _ in range(NB)]
    tb = [None, None, None] if tables is None else [None if a is None else a.data_ptr() for a in tables]
    args = [d.sm.data_ptr(), d.gr.data_ptr(), d.base_exp] + [a.data_ptr() for a in acts] + tb + \
           [o.data_ptr() for o in outs] + [M, K, t12.current_stream()]
    t12.check(fn(*args))
    torch.cuda.synchronize()
    return np.stack([o.cpu().numpy() for o in outs])


# (M, K, p_outlier): K % 128 == 0 runs the streaming form, the others the reference's column ownership;
# 77 and 5 rows: a last group of 16 that is part empty; 4096 columns: every col % 256 class 16 columns deep
@pytest.mark.parametrize("NB", [4, 8])
@pytest.mark.parametrize("M,K,p_out", [(96, 2304, 5e-3), (77, 4096, 2e-3), (5, 128, 2e-2), (64, 2320, 5e-3),
                                       (33, 1000, 5e-3), (300, 8192, 3e-4)])
def test_reference_named_batch_launchers(t12, oracle, synth, NB, M, K, p_out):
    """launch_split12_batch4/8_async take the derived escape tables of the reference's loader
    (esc_row_base / esc_counts / esc_vals, engine/model.cpp:86-160); esc_counts may be NULL here, and without
    tables the product is the unpatched one (decompress_v2.hip:573-701 with esc_vals == NULL)."""
    p = oracle.pack(synth.weights_llm(M, K, seed=50 + NB + M, p_outlier=p_out))
    assert p.P > 0
    row_base, counts, vals, _ = oracle.escape_tables(p)
    X = synth.activations(NB, K, seed=60)
    ref = oracle.gemm(p, X)
    d = t12.DeviceTensor12.from_packed(p, dev())
    acts = [to_dev_bits(X[j]) for j in range(NB)]
    rb, cn, vl = (torch.from_numpy(a).to(dev()) for a in (row_base, counts, vals))
    for tables in ((rb, cn, vl), (rb, None, vl)):
        got = _run_batch_launcher(t12, NB, d, acts, tables, M, K)
        for j in range(NB):
            assert rel_err(got[j], ref[j]) < TOL, (tables[1] is None, j)
    got = _run_batch_launcher(t12, NB, d, acts, None, M, K)
    assert rel_err(got, oracle.gemm(p, X, patched=False)) < TOL


def test_reference_named_batch_launchers_escape_order_and_overflow(t12, oracle, synth):
    """The slot of an escape in esc_vals is its rank by (col % 256, col) within its row: rows whose escapes share
    col % 256 classes in both orders, distinct values everywhere (a wrong rank picks a wrong value), and one row
    with more escapes than the streaming form keeps per row (it then recomputes its 16 rows the reference's way)."""
    M, K, NB = 40, 4096, 8
    w = synth.weights_llm(M, K, seed=91, p_outlier=0.0).copy()
    rng = np.random.default_rng(92)
    big = lambda n: oracle.f32_to_bf16_bits((rng.uniform(3.0, 60.0, n) * rng.choice([-1.0, 1.0], n)).astype(np.float32))
    w[3, [5, 261, 517, 4, 260, 1029, 2, 4095, 3839]] = big(9)          # classes 5, 4, 2, 255 in mixed column order
    w[17, np.arange(0, 4096, 256)] = big(16)                           # one class, sixteen deep
    w[18, np.arange(255, 0, -5)] = big(51)                             # one per class
    heavy = rng.choice(K, 300, replace=False)
    w[37, heavy] = big(300)                                            # above the per-row list of the streaming form
    p = oracle.pack(w)
    row_base, counts, vals, _ = oracle.escape_tables(p)
    slot3 = vals[row_base[3]:row_base[4]].tolist()
    assert len(slot3) >= 9 and len(set(slot3)) == len(slot3)
    X = synth.activations(NB, K, seed=93)
    ref = oracle.gemm(p, X)
    d = t12.DeviceTensor12.from_packed(p, dev())
    acts = [to_dev_bits(X[j]) for j in range(NB)]
    rb, cn, vl = (torch.from_numpy(a).to(dev()) for a in (row_base, counts, vals))
    for tables in ((rb, cn, vl), (rb, None, vl)):
        got = _run_batch_launcher(t12, NB, d, acts, tables, M, K)
        # per row: an escape taken from the wrong slot moves its row by the size of an outlier
        for r in range(M):
            assert np.abs(got[:, r] - ref[:, r]).max() <= 1e-4 * max(np.abs(ref[:, r]).max(), 1.0), r


def test_gemv_batch_entry_point(t12, oracle, synth):
    M, K = 200, 2048
    p = oracle.pack(synth.weights_llm(M, K, seed=70, p_outlier=2e-3))
    d = t12.DeviceTensor12.from_packed(p, dev())
    for B in (1, 3, 8):
        X = synth.activations(B, K, seed=71 + B)
        Xd = to_dev_bits(X).reshape(B, K)
        out = torch.zeros((B, M), device=dev())
        segs = t12._seg_array([d.segment(out)])
        t12.check(t12.lib.t12_gemv_batch(segs, 1, Xd.data_ptr(), K, M, K, B, t12.current_stream()))
        torch.cuda.synchronize()
        assert rel_err(out.cpu().numpy(), oracle.gemm(p, X)) < TOL
    assert t12.lib.t12_gemv_batch(segs, 1, Xd.data_ptr(), K, M, K, 9, None) == -1


@pytest.mark.parametrize("M,K", [(14336, 4096), (520, 2048), (77, 1040), (9, 16)])
def test_gemv_swiglu_fused_is_bit_identical_to_unfused(t12, oracle, synth, M, K):
    """t12_gemv_swiglu == t12_gemv(gate|up) followed by launch_silu_mul_bf16_batch, bit for bit,
    and both match the oracle's closed form."""
    pg = oracle.pack(synth.weights_llm(M, K, seed=81, sigma=0.05, p_outlier=2e-3))
    pu = oracle.pack(synth.weights_llm(M, K, seed=82, sigma=0.2, p_outlier=2e-3))
    x = synth.activations(1, K, seed=83)[0]
    dg, du = (t12.DeviceTensor12.from_packed(p, dev()) for p in (pg, pu))
    xd = to_dev_bits(x)
    og, ou = t12.gemv([dg, du], xd)
    unfused = torch.zeros(M, dtype=torch.int16, device=dev())
    st = t12.current_stream()
    t12.lib.launch_silu_mul_bf16_batch(og.data_ptr(), ou.data_ptr(), unfused.data_ptr(), M, 1, st)
    fused = torch.zeros(M, dtype=torch.int16, device=dev())
    sg, su = dg.segment(None), du.segment(None)
    import ctypes
    t12.check(t12.lib.t12_gemv_swiglu(ctypes.byref(sg), ctypes.byref(su), xd.data_ptr(), K, fused.data_ptr(), st))
    torch.cuda.synchronize()
    assert torch.equal(fused, unfused)
    ref = oracle.silu_mul_bf16(oracle.gemv(pg, x), oracle.gemv(pu, x))
    got = fused.cpu().numpy().view(np.uint16)
    gf, rf = oracle.bf16_bits_to_f32(got), oracle.bf16_bits_to_f32(ref)
    assert np.abs(gf - rf).max() <= 2e-2 * np.abs(rf).max()
    assert (got == ref).mean() > 0.97


@pytest.mark.parametrize("K,with_res", [(4096, True), (4096, False), (1040, True), (8192, True), (16, False)])
def test_gemv_norm_prologue(t12, oracle, synth, K, with_res):
    """t12_gemv_norm / t12_gemv_swiglu_norm: RMSNorm (+ residual add) folded into the GEMV prologue."""
    import ctypes
    rng = np.random.default_rng(K)
    M = 264
    pa = oracle.pack(synth.weights_llm(M, K, seed=91, p_outlier=2e-3))
    pb = oracle.pack(synth.weights_llm(M, K, seed=92, sigma=0.1, p_outlier=2e-3))
    x = rng.standard_normal(K).astype(np.float32) * 2
    r = rng.standard_normal(K).astype(np.float32) if with_res else None
    w = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    s = x + r if with_res else x
    a_bits = oracle.rms_norm_bf16(s, w, 1e-5)
    da, db = (t12.DeviceTensor12.from_packed(p, dev()) for p in (pa, pb))
    xd, wd = torch.from_numpy(x).to(dev()), torch.from_numpy(w).to(dev())
    rd = torch.from_numpy(r).to(dev()) if with_res else None
    hid = torch.zeros(K, device=dev())
    oa, ob = torch.zeros(M, device=dev()), torch.zeros(M, device=dev())
    segs = t12._seg_array([da.segment(oa), db.segment(ob)])
    st = t12.current_stream()
    t12.check(t12.lib.t12_gemv_norm(segs, 2, xd.data_ptr(), rd.data_ptr() if with_res else None, wd.data_ptr(), 1e-5,
                                    hid.data_ptr() if with_res else None, K, st))
    torch.cuda.synchronize()
    for o, p in ((oa, pa), (ob, pb)):
        assert rel_err(o.cpu().numpy(), oracle.gemv(p, a_bits)) < 2e-3     # a 1-ulp bf16 flip in the prologue is allowed
    if with_res:
        assert np.array_equal(hid.cpu().numpy(), s)
    fused = torch.zeros(M, dtype=torch.int16, device=dev())
    sg, su = da.segment(None), db.segment(None)
    t12.check(t12.lib.t12_gemv_swiglu_norm(ctypes.byref(sg), ctypes.byref(su), xd.data_ptr(),
                                           rd.data_ptr() if with_res else None, wd.data_ptr(), 1e-5, None, K,
                                           fused.data_ptr(), st))
    torch.cuda.synchronize()
    ref = oracle.bf16_bits_to_f32(oracle.silu_mul_bf16(oracle.gemv(pa, a_bits), oracle.gemv(pb, a_bits)))
    got = oracle.bf16_bits_to_f32(fused.cpu().numpy().view(np.uint16))
    assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
    # aliasing is rejected
    if with_res:
        assert t12.lib.t12_gemv_norm(segs, 2, xd.data_ptr(), rd.data_ptr(), wd.data_ptr(), 1e-5, xd.data_ptr(), K, st) == -1


@pytest.mark.parametrize("M,K", [(4096, 4096), (300, 14336), (77, 1040), (9, 15)])
def test_gemv_add_is_bit_identical_to_gemv_plus_add(t12, oracle, synth, M, K):
    """t12_gemv_add folds the residual add into the store: out = residual + W.x with the same single fp32 add
    the separate kernel does (the odd-K case runs the general kernel)."""
    p = oracle.pack(synth.weights_llm(M, K, seed=M * 3 + K, p_outlier=2e-3))
    dt = t12.DeviceTensor12.from_packed(p, dev())
    x = to_dev_bits(synth.activations(1, K, seed=9)[0])
    g = torch.Generator(device=dev()); g.manual_seed(M)
    res = torch.randn(M, generator=g, device=dev())
    (plain,) = t12.gemv([dt], x)
    want = plain + res
    out = torch.full((M,), float("nan"), dtype=torch.float32, device=dev())
    segs = t12._seg_array([dt.segment(out)])
    t12.check(t12.lib.t12_gemv_add(segs, x.data_ptr(), K, res.data_ptr(), t12.current_stream()), "t12_gemv_add")
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    assert t12.lib.t12_gemv_add(segs, x.data_ptr(), K, None, t12.current_stream()) == -1
