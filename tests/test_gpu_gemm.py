"""GPU parity: split-12 decode+GEMM (bf16 MFMA, fp32 accumulate) through the C ABI vs the
CPU oracle's decode-then-fp32-accumulate GEMM.

Tolerance: the target is 1e-2 relative; both sides multiply bf16 x bf16 exactly and accumulate
in fp32, so the observed error is ~1e-6 and the assertions use 1e-4.
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


def run_gemm(t12, packs, X, patched=True):
    dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in packs]
    Xd = to_dev_bits(X).reshape(X.shape)
    outs = t12.gemm(dts, Xd, patched=patched)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs]


@pytest.mark.parametrize("B", [1, 7, 16, 32, 33, 64, 100, 128, 129, 200, 256, 300, 512])
def test_gemm_batches(t12, oracle, synth, B):
    M, K = 300, 1024
    p = oracle.pack(synth.weights_llm(M, K, seed=B, p_outlier=2e-3))
    X = synth.activations(B, K, seed=100 + B)
    (got,) = run_gemm(t12, [p], X)
    assert got.shape == (B, M)
    assert rel_err(got, oracle.gemm(p, X)) < TOL


@pytest.mark.parametrize("M,K,B", [(4096, 4096, 16), (1024, 4096, 64), (512, 14336, 256), (1280, 5120, 64),
                                   (5120, 1280, 64), (129, 64, 5), (1, 128, 256)])
def test_gemm_shapes(t12, oracle, synth, M, K, B):
    gen = synth.weights_diffusion if K in (5120, 1280) else synth.weights_llm
    p = oracle.pack(gen(M, K, seed=M + K))
    X = synth.activations(B, K, seed=B)
    (got,) = run_gemm(t12, [p], X)
    assert rel_err(got, oracle.gemm(p, X)) < TOL
    (un,) = run_gemm(t12, [p], X, patched=False)
    assert rel_err(un, oracle.gemm(p, X, patched=False)) < TOL


def test_gemm_every_k_split(t12, oracle, synth):
    """One row tile (M = 128): the launch splits K across workgroups as far as its rule allows, so the length of K
    picks the number of splits.  The number the library chose is read back through t12_gemm_deferred; every count from
    1 to 16 that is a power of two must occur among the cases, and chunks that are not a power of two (K = 1088,
    6272).  The summed result is checked against the oracle both through t12_gemm (its own reduction launch) and
    through the deferred partial sums added up on the host."""
    import ctypes as C
    M = 128
    seen = set()
    for K, B in [(256, 96), (512, 96), (1024, 96), (2048, 96), (4096, 96), (8192, 96), (16384, 96), (4096, 200),
                 (8192, 200), (16384, 40), (1088, 40), (6272, 96), (64, 33)]:
        p = oracle.pack(synth.weights_llm(M, K, seed=K + B, p_outlier=1e-3))
        X = synth.activations(B, K, seed=6)
        ref = oracle.gemm(p, X)
        (got,) = run_gemm(t12, [p], X)
        assert rel_err(got, ref) < TOL, (K, B)
        dt = t12.DeviceTensor12.from_packed(p, dev())
        Xd = to_dev_bits(X).reshape(X.shape)
        out = torch.full((B, M), float("nan"), device=dev())
        part = t12.GemmPartials()
        segs = t12._seg_array([dt.segment(out)])
        t12.check(t12.lib.t12_gemm_deferred(segs, 1, Xd.data_ptr(), K, M, K, B, C.byref(part), t12.current_stream()))
        torch.cuda.synchronize()
        seen.add(part.nsplit)
        if part.nsplit > 1:
            ws = torch.empty(part.nsplit * part.split_stride, dtype=torch.float32, device=dev())
            assert t12._hip_memcpy_d2d(ws.data_ptr(), part.ws, ws.numel() * 4) == 0
            tot = ws.view(part.nsplit, B, part.ld)[:, :, :M].sum(dim=0)
            assert rel_err(tot.cpu().numpy(), ref) < TOL, (K, B, part.nsplit)
        else:
            assert rel_err(out.cpu().numpy(), ref) < TOL, (K, B)
    assert {1, 2, 4, 8, 16} <= seen, seen


def test_gemm_fused_segments_and_strides(t12, oracle, synth):
    """Three tensors with three base_exp in one launch; activations with a padded row stride;
    outputs written into column slices of one [B, sum M] buffer (out_stride > M)."""
    K, B = 2048, 48
    ps = [oracle.pack(synth.weights_llm(512, K, seed=1, sigma=0.02)),
          oracle.pack(synth.weights_llm(130, K, seed=2, sigma=0.3)),
          oracle.pack(synth.weights_llm(128, K, seed=3, sigma=0.002))]
    X = synth.activations(B, K, seed=4)
    Xpad = torch.zeros((B, K + 64), dtype=torch.int16, device=dev())
    Xpad[:, :K] = to_dev_bits(X).reshape(B, K)
    dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in ps]
    total = sum(p.M for p in ps)
    big = torch.full((B, total), float("nan"), device=dev())
    outs, c = [], 0
    for p in ps:
        outs.append(big[:, c:c + p.M]); c += p.M
    t12.gemm(dts, Xpad[:, :K], outs=outs)
    torch.cuda.synchronize()
    c = 0
    for p in ps:
        assert rel_err(big[:, c:c + p.M].cpu().numpy(), oracle.gemm(p, X)) < TOL
        c += p.M


def test_gemm_general_path(t12, oracle, synth, golden):
    rng = np.random.default_rng(8)
    for name in ("oddK_3x5", "zeros_4x32", "low_exp_3x32", "tie_2x30", "outliers_16x256", "llm_64x512"):
        g = golden[name]
        p = oracle.pack(g["w"], int(g["base_exp"]))
        X = oracle.f32_to_bf16_bits(rng.standard_normal((11, p.K)).astype(np.float32)).reshape(11, p.K)
        (got,) = run_gemm(t12, [p], X)
        assert rel_err(got, oracle.gemm(p, X)) < TOL, name


def test_gemm_matches_gemv_at_b1(t12, oracle, synth):
    M, K = 700, 4096
    p = oracle.pack(synth.weights_llm(M, K, seed=77))
    x = synth.activations(1, K, seed=78)
    (g,) = run_gemm(t12, [p], x)
    dt = t12.DeviceTensor12.from_packed(p, dev())
    (v,) = t12.gemv(dt, to_dev_bits(x[0]))
    torch.cuda.synchronize()
    assert rel_err(g[0], v.cpu().numpy()) < 1e-5


def test_full_size_linearity_b256(t12, oracle, synth):
    """Full Llama O-projection shape at B=256: rows of X that are copies of one another must give
    identical output rows, and X with disjoint halves must add up (size-independent properties)."""
    M, K, B = 4096, 4096, 256
    w = synth.weights_llm(M, K, seed=2003)
    p = oracle.pack(w)
    x = synth.activations(2, K, seed=9)
    X = np.repeat(x, B // 2, axis=0)
    (got,) = run_gemm(t12, [p], X)
    assert np.array_equal(got[0], got[B // 2 - 1]) and np.array_equal(got[B // 2], got[B - 1])
    ref = oracle.gemm(p, x)
    assert rel_err(got[[0, B - 1]], ref) < TOL


def test_gemm_rejects_bad_operands(t12):
    segs = (t12.Segment * 1)(t12.Segment(None, None, None, None, None, None, None, 4, 100, 0, 0))
    x = torch.zeros(64, dtype=torch.int16, device=dev())
    assert t12.lib.t12_gemm(segs, 1, x.data_ptr(), 64, 4, 64, 1, None) == -1
    assert t12.lib.t12_gemm(segs, 1, x.data_ptr(), 32, 4, 64, 1, None) == -1


@pytest.mark.parametrize("M,K,B", [(512, 4096, 256), (256, 14336, 96), (300, 1024, 40), (4096, 4096, 16)])
def test_deferred_reduction_into_add_rms_norm(t12, oracle, synth, M, K, B):
    """t12_gemm_deferred leaves the K-split partial sums for launch_sum_add_rms_norm_bf16_batch; the pair must
    give what t12_gemm + launch_add_rms_norm_bf16_batch give: identical sums (same summation order), normalised
    output equal to the last bf16 place."""
    p = oracle.pack(synth.weights_llm(M, K, seed=M + B, p_outlier=1e-3))
    dt = t12.DeviceTensor12.from_packed(p, dev())
    X = to_dev_bits(synth.activations(B, K, seed=3)).reshape(B, K)
    g = torch.Generator(device=dev()); g.manual_seed(4)
    res = torch.randn((B, M), generator=g, device=dev())
    w = 1 + 0.1 * torch.randn(M, generator=g, device=dev())
    st = t12.current_stream()
    # reference pair
    out_a = torch.empty((B, M), dtype=torch.float32, device=dev())
    t12.gemm([dt], X, outs=[out_a])
    y_a = torch.empty((B, M), dtype=torch.int16, device=dev())
    t12.lib.launch_add_rms_norm_bf16_batch(out_a.data_ptr(), res.data_ptr(), w.data_ptr(), y_a.data_ptr(), M, 1e-5, B, st)
    # deferred pair
    out_b = torch.full((B, M), float("nan"), dtype=torch.float32, device=dev())
    y_b = torch.empty((B, M), dtype=torch.int16, device=dev())
    part = t12.GemmPartials()
    segs = t12._seg_array([dt.segment(out_b)])
    t12.check(t12.lib.t12_gemm_deferred(segs, 1, X.data_ptr(), K, M, K, B, part, st), "t12_gemm_deferred")
    if part.nsplit > 1:
        t12.lib.launch_sum_add_rms_norm_bf16_batch(out_b.data_ptr(), part.ws, part.nsplit, part.split_stride, part.ld,
                                                   res.data_ptr(), w.data_ptr(), y_b.data_ptr(), M, 1e-5, B, st)
    else:
        t12.lib.launch_add_rms_norm_bf16_batch(out_b.data_ptr(), res.data_ptr(), w.data_ptr(), y_b.data_ptr(), M, 1e-5, B, st)
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b)                      # sums: the same additions in the same order
    # the normalised bf16 output may differ in the last place: the two kernels cut the row into
    # different per-thread pieces for the sum of squares
    fa = (y_a.view(torch.bfloat16).float(), y_b.view(torch.bfloat16).float())
    assert float(((fa[0] - fa[1]).abs() / fa[0].abs().clamp_min(1e-30)).max()) <= 2.0 ** -7
    if (M, K, B) == (512, 4096, 256):
        assert part.nsplit > 1          # this shape does split K: the fused path is the one compared


@pytest.mark.parametrize("B", [16, 64, 128, 256])
def test_gemm_more_escapes_than_the_lds_list_holds(t12, oracle, synth, B):
    """A 128-row tile with ~10 k escapes overflows the in-LDS escape list (1536 / 2048 entries): the kernel then
    multiplies the unpatched values and adds (correct - wrong) * x per entry in its epilogue -- still exact to
    fp32 rounding, with a K split (few row tiles) and without one (many)."""
    M, K = 256, 4096
    p = oracle.pack(synth.weights_llm(M, K, seed=77, p_outlier=3e-2))
    assert p.P > 2 * 4096                       # > 2048 entries in every 128-row tile
    X = synth.activations(B, K, seed=B + 1)
    ref = oracle.gemm(p, X)
    (got,) = run_gemm(t12, [p], X)                      # two row tiles: K is split 4 ways (B <= 128: 8)
    assert rel_err(got, ref) < TOL
    # without a K split: the same rows as the first 256 of a tensor with enough row tiles to fill the chip
    M2 = 128 * 200
    w2 = np.tile(oracle.decode(p), (M2 // M, 1))
    p2 = oracle.pack(w2, p.base_exp)
    (got2,) = run_gemm(t12, [p2], X)
    assert rel_err(got2[:, :M], ref) < TOL and rel_err(got2[:, M2 - M:], ref) < TOL


@pytest.mark.parametrize("M,K,B,p_out", [(14336, 4096, 256, 3e-4), (12300, 512, 129, 2e-3), (12352, 256, 300, 5e-2),
                                          (12288, 64, 512, 0.0), (14336, 4096, 128, 3e-4), (12300, 512, 65, 2e-3),
                                          (12352, 256, 100, 5e-2)])
def test_gemm_swiglu_epilogue_is_bit_identical_to_unfused(t12, synth, M, K, B, p_out):
    """t12_gemm_swiglu == t12_gemm on (gate, up) + launch_silu_mul_bf16_batch, bit for bit (ragged last tile,
    escape lists that fit the LDS staging and ones that overflow it, tensors without escapes; batch tiles of 256
    rows and, for 65 .. 128 rows, of 128)."""
    g = torch.Generator(device=dev())

    def mk(seed):
        g.manual_seed(seed)
        w = torch.randn((M, K), generator=g, device=dev()) * 0.02
        if p_out > 0:
            m = torch.rand((M, K), generator=g, device=dev()) < p_out
            w = torch.where(m, torch.randn((M, K), generator=g, device=dev()) * 8, w)
        return t12.pack_device(w.to(torch.bfloat16))

    gate, up = mk(1), mk(2)
    g.manual_seed(3)
    X = torch.randn((B, K), generator=g, device=dev()).to(torch.bfloat16).view(torch.int16)
    st = t12.current_stream()
    og, ou = t12.gemm([gate, up], X)
    want = torch.empty((B, M), dtype=torch.int16, device=dev())
    t12.lib.launch_silu_mul_bf16_batch(og.data_ptr(), ou.data_ptr(), want.data_ptr(), M, B, st)
    got = torch.full((B, M), -1, dtype=torch.int16, device=dev())
    sg = t12._seg_array([gate.segment(None)])
    su = t12._seg_array([up.segment(None)])
    rc = t12.lib.t12_gemm_swiglu(sg, su, X.data_ptr(), K, K, B, got.data_ptr(), M, st)
    torch.cuda.synchronize()
    assert rc == 0, t12.lib.t12_last_error()
    assert torch.equal(got, want)


@pytest.mark.parametrize("M,K,B,p_out", [(14336, 4096, 8, 3e-4), (14336, 4096, 5, 3e-4), (1000, 512, 5, 2e-3), (37, 128, 7, 5e-2),
                                          (4096, 1280, 6, 2e-2), (2001, 256, 8, 0.0), (520, 2048, 7, 0.2)])
def test_gemm_swiglu_small_batches_bit_identical_to_unfused(t12, synth, M, K, B, p_out):
    """5 .. 8 batch rows: t12_gemm_swiglu runs the whole-row sweep with gate rows and the same rows of up in one
    workgroup and must give t12_gemm on (gate, up) + launch_silu_mul_bf16_batch bit for bit: ragged row counts, one
    128-column block per row, rows with more escapes than waves, unlike base_exp of gate and up (unlike sigma)."""
    g = torch.Generator(device=dev())

    def mk(seed, sigma):
        g.manual_seed(seed)
        w = torch.randn((M, K), generator=g, device=dev()) * sigma
        if p_out > 0:
            m = torch.rand((M, K), generator=g, device=dev()) < p_out
            w = torch.where(m, torch.randn((M, K), generator=g, device=dev()) * 8, w)
        return t12.pack_device(w.to(torch.bfloat16))

    gate, up = mk(1, 0.02), mk(2, 0.3)
    if p_out < 1e-2:                                          # (many outliers pull both windows to the same place)
        assert gate.segment(None).base_exp != up.segment(None).base_exp
    g.manual_seed(3)
    X = torch.randn((B, K), generator=g, device=dev()).to(torch.bfloat16).view(torch.int16)
    st = t12.current_stream()
    og, ou = t12.gemm([gate, up], X)
    want = torch.empty((B, M), dtype=torch.int16, device=dev())
    t12.lib.launch_silu_mul_bf16_batch(og.data_ptr(), ou.data_ptr(), want.data_ptr(), M, B, st)
    got = torch.full((B, M + 8), -1, dtype=torch.int16, device=dev())
    sg = t12._seg_array([gate.segment(None)])
    su = t12._seg_array([up.segment(None)])
    rc = t12.lib.t12_gemm_swiglu(sg, su, X.data_ptr(), K, K, B, got.data_ptr(), M + 8, st)
    torch.cuda.synchronize()
    assert rc == 0, t12.lib.t12_last_error()
    assert torch.equal(got[:, :M], want)
    assert bool((got[:, M:] == -1).all())                     # nothing written past the last row


def test_gemm_swiglu_declines_shapes_without_a_fused_kernel(t12, oracle, synth):
    p = oracle.pack(synth.weights_llm(512, 256, seed=1))
    dt = t12.DeviceTensor12.from_packed(p, dev())
    X = to_dev_bits(synth.activations(256, 256, seed=2)).reshape(256, 256)
    out = torch.empty((256, 512), dtype=torch.int16, device=dev())
    s1 = t12._seg_array([dt.segment(None)])
    st = t12.current_stream()
    assert t12.lib.t12_gemm_swiglu(s1, s1, X.data_ptr(), 256, 256, 256, out.data_ptr(), 512, st) == 1      # few rows
    assert t12.lib.t12_gemm_swiglu(s1, s1, X.data_ptr(), 256, 256, 64, out.data_ptr(), 512, st) == 1       # 9 .. 64 rows
    assert t12.lib.t12_gemm_swiglu(s1, s1, X.data_ptr(), 256, 256, 16, out.data_ptr(), 512, st) == 1
    assert t12.lib.t12_gemm_swiglu(s1, s1, X.data_ptr(), 256, 256, 4, out.data_ptr(), 512, st) == 1        # up to 4 rows
    assert t12.lib.t12_gemm_swiglu(s1, s1, X.data_ptr(), 256, 256, 256, out.data_ptr(), 100, st) == -1     # out_stride < M


@pytest.mark.parametrize("M,K,B", [(300, 1024, 48), (1024, 4096, 256), (77, 320, 9)])
def test_reference_named_batch_entry_points(t12, oracle, synth, M, K, B):
    """nv_launch_split12_fused_gemm_async with and without the escape lists, the separate correction launch
    nv_launch_patches_batch_async on top of the unpatched product, and nv_launch_split12_cublas_batch_async
    (nvidia_kernels.cu:426-584), called with the reference's argument lists."""
    p = oracle.pack(synth.weights_llm(M, K, seed=M + B, p_outlier=3e-3))
    X = synth.activations(B, K, seed=K + B)
    ref, ref_un = oracle.gemm(p, X), oracle.gemm(p, X, patched=False)
    d = t12.DeviceTensor12.from_packed(p, dev())
    Xd = to_dev_bits(X).reshape(X.shape)
    st = t12.current_stream()
    ptr = lambda t: t.data_ptr()

    out = torch.full((B, M + 3), float("nan"), device=dev())                 # out_stride > M
    rc = t12.lib.nv_launch_split12_fused_gemm_async(ptr(d.sm), ptr(d.gr), d.base_exp, ptr(Xd), K, ptr(out), M + 3, M, K, B, st,
                                                    ptr(d.row_off), ptr(d.cols), ptr(d.correct), ptr(d.wrong))
    assert rc == 0
    torch.cuda.synchronize()
    assert rel_err(out[:, :M].cpu().numpy(), ref) < TOL

    un = torch.zeros((B, M), device=dev())
    assert t12.lib.nv_launch_split12_fused_gemm_async(ptr(d.sm), ptr(d.gr), d.base_exp, ptr(Xd), K, ptr(un), M, M, K, B, st,
                                                      None, None, None, None) == 0
    via_buf = torch.zeros((B, M), device=dev())
    scratch = torch.zeros(8, dtype=torch.int16, device=dev())                # not touched by this build
    assert t12.lib.nv_launch_split12_cublas_batch_async(ptr(d.sm), ptr(d.gr), d.base_exp, ptr(Xd), K, ptr(via_buf), M,
                                                        ptr(scratch), 4, M, K, B, st) == 0
    torch.cuda.synchronize()
    assert rel_err(un.cpu().numpy(), ref_un) < TOL
    assert torch.equal(un, via_buf) and int(scratch.abs().sum()) == 0

    # the reference's two-launch form: unpatched product, then the correction over the rows that have escapes
    ro = p.row_off
    rows = np.nonzero(ro[1:] > ro[:-1])[0].astype(np.int32)
    assert 0 < len(rows)
    rows_d = torch.from_numpy(rows).to(dev())
    assert t12.lib.nv_launch_patches_batch_async(ptr(d.row_off), ptr(d.cols), ptr(d.correct), ptr(d.wrong), ptr(rows_d), len(rows),
                                                 ptr(Xd), K, ptr(un), M, B, st) == 0
    torch.cuda.synchronize()
    assert rel_err(un.cpu().numpy(), ref) < TOL
    assert t12.lib.nv_launch_patches_batch_async(None, None, None, None, None, 0, None, K, None, M, B, st) == 0   # nothing to do


@pytest.mark.parametrize("B", [2, 4, 5, 8, 9, 16])
@pytest.mark.parametrize("M,K,law", [(4096, 4096, "llm"), (1000, 1280, "diffusion"), (37, 128, "llm"), (2560, 10240, "diffusion"),
                                     (28672, 256, "llm"), (16, 14336, "llm")])
def test_gemm_small_batches_dense_sweep(t12, oracle, synth, M, K, law, B):
    """B <= 16 with K % 128 == 0 takes the kernel that sweeps whole rows (16 rows per workgroup, the waves of a
    workgroup interleaved over the 128-column blocks, activations straight from memory): ragged row counts, one
    block per row, rows with far more escapes than waves (the diffusion law: ~50-100 per row at K = 10240), row
    counts that make it share activation loads across two and four row groups, padded batches."""
    w = synth.weights_diffusion(M, K, seed=M + K) if law == "diffusion" else synth.weights_llm(M, K, seed=M + K, p_outlier=1e-3)
    p = oracle.pack(w)
    X = synth.activations(B, K, seed=B)
    (got,) = run_gemm(t12, [p], X)
    assert rel_err(got, oracle.gemm(p, X)) < TOL
    (un,) = run_gemm(t12, [p], X, patched=False)
    assert rel_err(un, oracle.gemm(p, X, patched=False)) < TOL


def test_gemm_small_batch_segments_and_strides(t12, oracle, synth):
    """Three tensors with three base_exp in one small-batch launch; activation rows with a padded stride; outputs in
    column slices of one buffer; enough rows (2 x 14336 + 100) that the launch shares activation loads across row
    groups and a segment ends inside a shared group."""
    K, B = 512, 12
    ps = [oracle.pack(synth.weights_llm(14336, K, seed=1, sigma=0.02)), oracle.pack(synth.weights_llm(100, K, seed=2, sigma=0.3)),
          oracle.pack(synth.weights_llm(14336, K, seed=3, sigma=0.002))]
    X = synth.activations(B, K, seed=4)
    Xpad = torch.zeros((B, K + 64), dtype=torch.int16, device=dev())
    Xpad[:, :K] = to_dev_bits(X).reshape(B, K)
    dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in ps]
    total = sum(p.M for p in ps)
    big = torch.full((B, total), float("nan"), device=dev())
    outs, off = [], 0
    for p in ps:
        outs.append(big[:, off:off + p.M])
        off += p.M
    t12.gemm(dts, Xpad[:, :K], outs=outs)
    torch.cuda.synchronize()
    h = big.cpu().numpy()
    off = 0
    for p in ps:
        assert rel_err(h[:, off:off + p.M], oracle.gemm(p, X)) < TOL
        off += p.M


@pytest.mark.parametrize("B,K", [(7, 256), (16, 128), (11, 384)])
def test_gemm_small_batch_ragged_segments_head_and_tail_workgroups(t12, oracle, synth, B, K):
    """Six tensors of unlike, ragged row counts (one of a single row group, one that is no multiple of 16) in one
    small-batch launch of ~29 000 rows: more workgroups than one round of the chip and a last round that would be
    partly empty, so the launch cuts every tensor into a head and a tail with fewer row groups per workgroup (the
    16-row tensor has no head at all).  Every output row must be written once and equal the oracle's."""
    Ms = [9001, 16, 5000, 1234, 7777, 6000]
    ps = [oracle.pack(synth.weights_llm(M, K, seed=50 + i, sigma=0.02 * (i + 1), p_outlier=2e-3)) for i, M in enumerate(Ms)]
    X = synth.activations(B, K, seed=B + K)
    dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in ps]
    total = sum(Ms)
    big = torch.full((B, total + 8), float("nan"), device=dev())
    outs, off = [], 0
    for M in Ms:
        outs.append(big[:, off:off + M])
        off += M
    t12.gemm(dts, to_dev_bits(X).reshape(B, K), outs=outs)
    torch.cuda.synchronize()
    h = big.cpu().numpy()
    assert np.isnan(h[:, total:]).all()                      # nothing written past the last tensor
    off = 0
    for p, M in zip(ps, Ms):
        assert rel_err(h[:, off:off + M], oracle.gemm(p, X)) < TOL
        off += M


@pytest.mark.parametrize("B", [17, 24, 31, 32])
@pytest.mark.parametrize("M,K,law", [(4096, 4096, "llm"), (37, 128, "llm"), (1280, 5120, "diffusion"), (8000, 1280, "diffusion"),
                                     (5000, 4096, "llm"), (2048, 8192, "llm")])
def test_gemm_17_to_32_rows_two_batch_tiles(t12, oracle, synth, M, K, law, B):
    """17 .. 32 batch rows on tensors of at most one round of workgroups take the whole-row sweep with two batch tiles
    per weight load (16 or 32 weight rows per workgroup by row count; long rows fall back to the tile kernel by
    K x B, so both sides of that rule are among the cases): ragged row counts, a second batch tile with a single row
    (B = 17), rows with many escapes (the diffusion law), patched and unpatched."""
    w = synth.weights_diffusion(M, K, seed=M + K) if law == "diffusion" else synth.weights_llm(M, K, seed=M + K, p_outlier=1e-3)
    p = oracle.pack(w)
    X = synth.activations(B, K, seed=B)
    (got,) = run_gemm(t12, [p], X)
    assert rel_err(got, oracle.gemm(p, X)) < TOL
    (un,) = run_gemm(t12, [p], X, patched=False)
    assert rel_err(un, oracle.gemm(p, X, patched=False)) < TOL


def test_gemm_17_to_32_rows_segments_and_strides(t12, oracle, synth):
    """q|k|v-like: three tensors (4096 + 1000 + 1024 rows, three base_exp) in one launch at B = 20, padded activation
    stride, outputs in column slices of one buffer whose other columns must stay untouched."""
    K, B = 2048, 20
    ps = [oracle.pack(synth.weights_llm(4096, K, seed=1, sigma=0.02)), oracle.pack(synth.weights_llm(1000, K, seed=2, sigma=0.3)),
          oracle.pack(synth.weights_llm(1024, K, seed=3, sigma=0.002, p_outlier=5e-3))]
    X = synth.activations(B, K, seed=4)
    Xpad = torch.zeros((B, K + 64), dtype=torch.int16, device=dev())
    Xpad[:, :K] = to_dev_bits(X).reshape(B, K)
    dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in ps]
    total = sum(p.M for p in ps)
    big = torch.full((B, total + 8), float("nan"), device=dev())
    outs, off = [], 0
    for p in ps:
        outs.append(big[:, off:off + p.M])
        off += p.M
    t12.gemm(dts, Xpad[:, :K], outs=outs)
    torch.cuda.synchronize()
    h = big.cpu().numpy()
    assert np.isnan(h[:, total:]).all()
    off = 0
    for p in ps:
        assert rel_err(h[:, off:off + p.M], oracle.gemm(p, X)) < TOL
        off += p.M


@pytest.mark.parametrize("B", [2, 3, 4])
@pytest.mark.parametrize("M,K,law", [(4096, 4096, "llm"), (101, 2048, "diffusion"), (8, 1024, "llm"), (300, 8192, "diffusion")])
def test_gemm_two_to_four_rows_whole_row_kernel(t12, oracle, synth, M, K, law, B):
    """B = 2 with K a multiple of 1024 (up to 8192) takes the kernel whose waves read whole rows, like the B = 1
    kernel, with one accumulator per batch row (B = 3, 4 on the same shapes: the 16-row MFMA kernel): ragged row
    counts, the largest K its LDS holds, escape-heavy rows (more entries than lanes), unpatched mode; and three
    tensors with three base_exp in one launch."""
    w = synth.weights_diffusion(M, K, seed=M + K) if law == "diffusion" else synth.weights_llm(M, K, seed=M + K, p_outlier=1e-3)
    p = oracle.pack(w)
    X = synth.activations(B, K, seed=B)
    (got,) = run_gemm(t12, [p], X)
    assert rel_err(got, oracle.gemm(p, X)) < TOL
    (un,) = run_gemm(t12, [p], X, patched=False)
    assert rel_err(un, oracle.gemm(p, X, patched=False)) < TOL
    if M == 101:
        ps = [p, oracle.pack(synth.weights_llm(9, K, seed=2, sigma=0.3)), oracle.pack(synth.weights_llm(64, K, seed=3, sigma=0.002))]
        outs = run_gemm(t12, ps, X)
        for q, o in zip(ps, outs):
            assert rel_err(o, oracle.gemm(q, X)) < TOL
