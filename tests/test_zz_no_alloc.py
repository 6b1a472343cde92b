"""GPU: t12_gemm_noalloc (the entry point that never allocates: K-split partial sums in a fixed array of the
library's device image) against t12_gemm through the C ABI -- bit for bit, on two calls in a row, the second with
a smaller input, then a shape that needs no split, and the refusal of a shape beyond the fixed workspace."""
import importlib

import numpy as np
import pytest
import torch

from gpu_util import dev, rel_err, to_dev_bits

pytestmark = pytest.mark.gpu


def _call(t12, fn, dts, X, outs):
    B, K = X.shape
    segs = t12._seg_array([t.segment(o) for t, o in zip(dts, outs)])
    rc = fn(segs, len(dts), X.data_ptr(), X.stride(0), outs[0].stride(0), K, B, t12.current_stream())
    return rc


def _free_device_bytes():
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_noalloc_allocates_nothing_on_a_fresh_stream(t12, oracle):
    """The property the entry point exists for: a K-split launch on a stream the library has never seen changes the
    free device memory by nothing (t12_gemm on the same fresh stream grows a workspace with hipMalloc: the control
    that shows the measurement sees such a thing)."""
    synth = importlib.import_module("turbo_lossless_amd.synth")
    lib = t12.lib
    M, K, B = 1024, 4096, 200                                     # 8 row tiles: K is split, partial sums are needed
    p = oracle.pack(synth.weights_llm(M, K, seed=61, p_outlier=2e-3))
    dt = t12.DeviceTensor12.from_packed(p, dev())
    X = synth.activations(B, K, seed=62)
    Xd = to_dev_bits(X).reshape(X.shape)
    o = torch.full((B, M), float("nan"), device=dev())
    o2 = torch.full((B, M), float("nan"), device=dev())
    segs = t12._seg_array([dt.segment(o)])
    segs2 = t12._seg_array([dt.segment(o2)])
    fresh = torch.cuda.Stream()                                   # default priority
    fresh.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    # on the caller's own stream first: the library takes the array's device address once per device
    assert lib.t12_gemm_noalloc(segs, 1, Xd.data_ptr(), K, M, K, B, t12.current_stream()) == 0
    torch.cuda.synchronize()
    o.fill_(float("nan"))
    torch.cuda.synchronize()
    before = _free_device_bytes()
    assert lib.t12_gemm_noalloc(segs, 1, Xd.data_ptr(), K, M, K, B, fresh.cuda_stream) == 0, lib.t12_last_error()
    torch.cuda.synchronize()
    assert _free_device_bytes() == before
    assert rel_err(o.cpu().numpy(), oracle.gemm(p, X)) < 1e-4
    # control: the allocating entry point on the same fresh stream takes memory for its partial sums
    assert lib.t12_gemm(segs2, 1, Xd.data_ptr(), K, M, K, B, fresh.cuda_stream) == 0
    torch.cuda.synchronize()
    taken = before - _free_device_bytes()
    assert taken >= 8 * B * M * 4 // 2                            # at least the partial sums of a few splits
    assert torch.equal(o, o2)
    assert lib.t12_release_stream(fresh.cuda_stream) == 0


def test_noalloc_equals_gemm_two_calls_in_a_row(t12, oracle):
    synth = importlib.import_module("turbo_lossless_amd.synth")
    lib = t12.lib
    # (M, K, B): both split K (few row tiles); the second call is smaller in every dimension and so reads a
    # workspace region that still holds the first call's partial sums
    cases = [(1024, 4096, 200), (384, 2048, 48)]
    packs = [oracle.pack(synth.weights_llm(M, K, seed=70 + i, p_outlier=2e-3)) for i, (M, K, B) in enumerate(cases)]
    dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in packs]
    Xs = [synth.activations(B, K, seed=80 + i) for i, (M, K, B) in enumerate(cases)]
    Xd = [to_dev_bits(X).reshape(X.shape) for X in Xs]
    got, want = [], []
    for dt, X, (M, K, B) in zip(dts, Xd, cases):                # the two calls back to back, nothing in between
        o = torch.full((B, M), float("nan"), device=dev())
        assert _call(t12, lib.t12_gemm_noalloc, [dt], X, [o]) == 0, lib.t12_last_error()
        got.append(o)
    torch.cuda.synchronize()
    for dt, X, (M, K, B) in zip(dts, Xd, cases):
        o = torch.full((B, M), float("nan"), device=dev())
        assert _call(t12, lib.t12_gemm, [dt], X, [o]) == 0, lib.t12_last_error()
        want.append(o)
    torch.cuda.synchronize()
    for g, w, p, X in zip(got, want, packs, Xs):
        assert torch.equal(g, w)                                 # same kernels, same split: the same bits
        assert rel_err(g.cpu().numpy(), oracle.gemm(p, X)) < 1e-4
    # once more in the other order: the big call after the small one
    for i in (1, 0):
        M, K, B = cases[i]
        o = torch.full((B, M), float("nan"), device=dev())
        assert _call(t12, lib.t12_gemm_noalloc, [dts[i]], Xd[i], [o]) == 0
        torch.cuda.synchronize()
        assert torch.equal(o, want[i])


def test_noalloc_segments_without_split_and_general_path(t12, oracle):
    """Three segments in one launch (q|k|v shape at a reduced width), a launch with enough row tiles to need no
    split (no workspace at all), and a shape that takes the general kernel (K not a multiple of 64)."""
    synth = importlib.import_module("turbo_lossless_amd.synth")
    lib = t12.lib
    K, B = 1024, 96
    packs = [oracle.pack(synth.weights_llm(M, K, seed=90 + i, p_outlier=1e-3)) for i, M in enumerate((512, 128, 128))]
    dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in packs]
    X = synth.activations(B, K, seed=95)
    Xd = to_dev_bits(X).reshape(X.shape)
    outs_a = [torch.full((B, p.M), float("nan"), device=dev()) for p in packs]
    outs_b = [torch.full((B, p.M), float("nan"), device=dev()) for p in packs]
    assert _call(t12, lib.t12_gemm_noalloc, dts, Xd, outs_a) == 0, lib.t12_last_error()
    assert _call(t12, lib.t12_gemm, dts, Xd, outs_b) == 0
    torch.cuda.synchronize()
    for a, b, p in zip(outs_a, outs_b, packs):
        assert torch.equal(a, b)
        assert rel_err(a.cpu().numpy(), oracle.gemm(p, X)) < 1e-4
    for (M, K, B) in [(28672 // 2, 512, 64), (40, 200, 9)]:
        p = oracle.pack(synth.weights_llm(M, K, seed=M + K, p_outlier=1e-3))
        dt = t12.DeviceTensor12.from_packed(p, dev())
        X = synth.activations(B, K, seed=3)
        Xd = to_dev_bits(X).reshape(X.shape)
        a = torch.full((B, M), float("nan"), device=dev())
        b = torch.full((B, M), float("nan"), device=dev())
        assert _call(t12, lib.t12_gemm_noalloc, [dt], Xd, [a]) == 0, lib.t12_last_error()
        assert _call(t12, lib.t12_gemm, [dt], Xd, [b]) == 0
        torch.cuda.synchronize()
        assert torch.equal(a, b)


def test_noalloc_refuses_what_does_not_fit(t12, oracle):
    """8320 x 4096 at B = 256 splits K four ways and would need 4 x 256 x 8320 floats = 32.5 MiB of partial sums:
    refused on the host with a message that names the limit; nothing is launched (the output keeps its fill).
    8192 rows need exactly 32 MiB and pass."""
    synth = importlib.import_module("turbo_lossless_amd.synth")
    M, K, B = 8320, 4096, 256
    w = torch.from_numpy(synth.weights_llm(M, K, seed=5).view(np.int16)).to(dev())
    dt = t12.pack_device(w)
    X = torch.zeros((B, K), dtype=torch.int16, device=dev())
    o = torch.full((B, M), 7.0, device=dev())
    rc = _call(t12, t12.lib.t12_gemm_noalloc, [dt], X, [o])
    assert rc == -1
    msg = t12.lib.t12_last_error().decode()
    assert "t12_gemm_noalloc" in msg and "fixed" in msg and str(32 << 20) in msg
    torch.cuda.synchronize()
    assert float(o.min()) == 7.0 and float(o.max()) == 7.0
    dt2 = t12.DeviceTensor12(8192, K, dt.base_exp, dt.sm, dt.gr, dt.row_off, dt.cols, dt.correct, dt.wrong)
    a, b = torch.full((B, 8192), 7.0, device=dev()), torch.full((B, 8192), 7.0, device=dev())
    assert _call(t12, t12.lib.t12_gemm_noalloc, [dt2], X, [a]) == 0, t12.lib.t12_last_error()
    assert _call(t12, t12.lib.t12_gemm, [dt2], X, [b]) == 0
    torch.cuda.synchronize()
    assert torch.equal(a, b) and float(a.abs().max()) == 0.0
