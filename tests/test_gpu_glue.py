"""GPU parity: engine glue launchers (reference names/signatures) vs the oracle's closed forms.

bf16 outputs: the kernels round fp32 results to bf16; the oracle computes the same formulas in
float64/float32, so an output may differ by one bf16 ulp where the fp32 value sits next to a rounding
boundary.  Assertions: every element within 1 bf16 ulp and >= 99 % bit-identical."""
import numpy as np
import pytest
import torch

from gpu_util import dev

pytestmark = pytest.mark.gpu


def st(t12):
    return t12.current_stream()


def bf16_close(got_bits, ref_bits, frac=0.99):
    g = got_bits.astype(np.uint16).view(np.int16).astype(np.int32)
    r = ref_bits.astype(np.uint16).view(np.int16).astype(np.int32)
    # bf16 bit patterns are monotone in magnitude per sign; compare as sign-magnitude integers
    gi = np.where(g < 0, -(g & 0x7FFF), g)
    ri = np.where(r < 0, -(r & 0x7FFF), r)
    assert np.abs(gi - ri).max() <= 1
    assert (g == r).mean() >= frac


def test_embed_lookup(t12, oracle):
    rng = np.random.default_rng(0)
    V, n = 50, 96
    embd = oracle.f32_to_bf16_bits(rng.standard_normal((V, n)).astype(np.float32)).reshape(V, n)
    toks = [3, 49, 0, -1, 50]
    e = torch.from_numpy(embd.view(np.int16)).to(dev())
    t = torch.tensor(toks, dtype=torch.int32, device=dev())
    out = torch.full((len(toks), n), 7.0, device=dev())
    t12.lib.launch_embed_lookup(e.data_ptr(), t.data_ptr(), out.data_ptr(), n, len(toks), V, st(t12))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.embed_lookup(embd, toks, V))


@pytest.mark.parametrize("n,B", [(4096, 1), (4096, 5), (256, 3), (14336, 2), (100, 1), (8192, 2), (4100, 2), (6, 3), (1022, 2)])
def test_rms_norm_and_add(t12, oracle, n, B):
    """Rows of a multiple of 4 values up to 8192 take the 128-bit form of the kernel (one or two pieces per thread),
    the others the scalar form."""
    rng = np.random.default_rng(n + B)
    x = rng.standard_normal((B, n)).astype(np.float32) * 3
    r = rng.standard_normal((B, n)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    xd, rd, wd = (torch.from_numpy(a).to(dev()) for a in (x, r, w))
    y = torch.zeros((B, n), dtype=torch.int16, device=dev())
    t12.lib.launch_rms_norm_bf16_batch(xd.data_ptr(), wd.data_ptr(), y.data_ptr(), n, 1e-5, B, st(t12))
    torch.cuda.synchronize()
    bf16_close(y.cpu().numpy().view(np.uint16), oracle.rms_norm_bf16(x, w, 1e-5).reshape(B, n))
    assert np.array_equal(xd.cpu().numpy(), x)
    t12.lib.launch_add_rms_norm_bf16_batch(xd.data_ptr(), rd.data_ptr(), wd.data_ptr(), y.data_ptr(), n, 1e-5, B, st(t12))
    torch.cuda.synchronize()
    s, yb = oracle.add_rms_norm_bf16(x, r, w, 1e-5)
    assert np.array_equal(xd.cpu().numpy(), s)          # x += residual, exact in fp32
    bf16_close(y.cpu().numpy().view(np.uint16), yb.reshape(B, n))


def test_rms_norm_unaligned_rows_take_the_scalar_form(t12, oracle):
    """Operands that are not 16-byte aligned (a view one float into a buffer) still give the same result."""
    rng = np.random.default_rng(5)
    n, B = 512, 3
    x = rng.standard_normal((B, n)).astype(np.float32) * 3
    r = rng.standard_normal((B, n)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)

    def off(a):                                         # a device copy that starts 4 bytes past a 16-byte boundary
        buf = torch.zeros(a.size + 1, dtype=torch.float32, device=dev())
        buf[1:] = torch.from_numpy(a.reshape(-1)).to(dev())
        return buf[1:]
    xd, rd, wd = off(x), off(r), off(w)
    assert xd.data_ptr() % 16 == 4
    y = torch.zeros((B, n), dtype=torch.int16, device=dev())
    t12.lib.launch_add_rms_norm_bf16_batch(xd.data_ptr(), rd.data_ptr(), wd.data_ptr(), y.data_ptr(), n, 1e-5, B, st(t12))
    torch.cuda.synchronize()
    s_, yb = oracle.add_rms_norm_bf16(x, r, w, 1e-5)
    assert np.array_equal(xd.cpu().numpy().reshape(B, n), s_)
    bf16_close(y.cpu().numpy().view(np.uint16), yb.reshape(B, n))


def test_silu_mul_and_add(t12, oracle):
    rng = np.random.default_rng(2)
    for (n, B) in [(14336, 2), (1001, 3)]:
        g = rng.standard_normal((B, n)).astype(np.float32) * 4
        u = rng.standard_normal((B, n)).astype(np.float32)
        gd, ud = torch.from_numpy(g).to(dev()), torch.from_numpy(u).to(dev())
        o = torch.zeros((B, n), dtype=torch.int16, device=dev())
        t12.lib.launch_silu_mul_bf16_batch(gd.data_ptr(), ud.data_ptr(), o.data_ptr(), n, B, st(t12))
        t12.lib.launch_add_batch(gd.data_ptr(), ud.data_ptr(), n, B, st(t12))
        torch.cuda.synchronize()
        bf16_close(o.cpu().numpy().view(np.uint16), oracle.silu_mul_bf16(g, u).reshape(B, n), frac=0.98)
        assert np.array_equal(gd.cpu().numpy(), g + u)


def make_qkv(rng, B, nh, nkv, hd):
    q = rng.standard_normal((B, nh * hd)).astype(np.float32)
    k = rng.standard_normal((B, nkv * hd)).astype(np.float32)
    v = rng.standard_normal((B, nkv * hd)).astype(np.float32) * 2
    return q, k, v


@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 128), (4, 4, 64), (8, 2, 32)])
def test_rope_store_kv_b1(t12, oracle, nh, nkv, hd):
    rng = np.random.default_rng(nh)
    theta, pos, max_seq = 500000.0, 37, 64
    q, k, v = make_qkv(rng, 1, nh, nkv, hd)
    qd, kd, vd = (torch.from_numpy(a.copy()).to(dev()) for a in (q, k, v))
    ck = torch.zeros((max_seq, nkv, hd), dtype=torch.int8, device=dev()); cv = torch.zeros_like(ck)
    sk = torch.zeros((max_seq, nkv), device=dev()); sv = torch.zeros_like(sk)
    t12.lib.launch_rope_store_kv(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), ck.data_ptr(), cv.data_ptr(),
                                 sk.data_ptr(), sv.data_ptr(), hd, nh, nkv, pos, max_seq, theta, st(t12))
    torch.cuda.synchronize()
    qr = oracle.rope(q[0], pos, nh, hd, theta); kr = oracle.rope(k[0], pos, nkv, hd, theta)
    assert np.allclose(qd.cpu().numpy()[0], qr, rtol=1e-5, atol=1e-5)
    assert np.allclose(kd.cpu().numpy()[0], kr, rtol=1e-5, atol=1e-5)
    # quantisation is checked on the GPU's own rotated K (rounding boundaries are discontinuous)
    k8, ks = oracle.quant_kv_int8(kd.cpu().numpy()[0], nkv, hd)
    v8, vs = oracle.quant_kv_int8(v[0], nkv, hd)
    assert np.array_equal(ck.cpu().numpy()[pos], k8) and np.array_equal(cv.cpu().numpy()[pos], v8)
    assert np.allclose(sk.cpu().numpy()[pos], ks, rtol=1e-6) and np.allclose(sv.cpu().numpy()[pos], vs, rtol=1e-6)
    assert not ck.cpu().numpy()[:pos].any() and not ck.cpu().numpy()[pos + 1:].any()


def test_rope_and_store_batch_launchers(t12, oracle):
    rng = np.random.default_rng(5)
    nh, nkv, hd, B, theta, max_seq = 8, 2, 64, 3, 10000.0, 40
    q, k, v = make_qkv(rng, B, nh, nkv, hd)
    positions = [0, 7, 39]
    pd = torch.tensor(positions, dtype=torch.int32, device=dev())
    qd, kd, vd = (torch.from_numpy(a.copy()).to(dev()) for a in (q, k, v))
    t12.lib.launch_rope_batch(qd.data_ptr(), kd.data_ptr(), pd.data_ptr(), hd, nh, nkv, nh * hd, nkv * hd, theta, B, st(t12))
    ck = torch.zeros((max_seq, nkv, hd), dtype=torch.int8, device=dev()); cv = torch.zeros_like(ck)
    sk = torch.zeros((max_seq, nkv), device=dev()); sv = torch.zeros_like(sk)
    t12.lib.launch_store_kv_batch(kd.data_ptr(), vd.data_ptr(), ck.data_ptr(), cv.data_ptr(), sk.data_ptr(), sv.data_ptr(),
                                  pd.data_ptr(), nkv * hd, max_seq, nkv, hd, B, st(t12))
    torch.cuda.synchronize()
    for b, pos in enumerate(positions):
        assert np.allclose(qd.cpu().numpy()[b], oracle.rope(q[b], pos, nh, hd, theta), rtol=1e-5, atol=1e-5)
        k8, ks = oracle.quant_kv_int8(kd.cpu().numpy()[b], nkv, hd)
        v8, vs = oracle.quant_kv_int8(v[b], nkv, hd)
        assert np.array_equal(ck.cpu().numpy()[pos], k8) and np.array_equal(cv.cpu().numpy()[pos], v8)
        assert np.allclose(sv.cpu().numpy()[pos], vs, rtol=1e-6)
    # the fused batch launcher gives the same cache
    q2, k2, v2 = (torch.from_numpy(a.copy()).to(dev()) for a in (q, k, v))
    ck2 = torch.zeros_like(ck); cv2 = torch.zeros_like(cv); sk2 = torch.zeros_like(sk); sv2 = torch.zeros_like(sv)
    t12.lib.launch_rope_store_kv_batch(q2.data_ptr(), k2.data_ptr(), v2.data_ptr(), ck2.data_ptr(), cv2.data_ptr(),
                                       sk2.data_ptr(), sv2.data_ptr(), pd.data_ptr(), hd, nh, nkv, nh * hd, nkv * hd,
                                       theta, B, st(t12))
    torch.cuda.synchronize()
    assert torch.equal(ck, ck2) and torch.equal(cv, cv2) and torch.equal(sk, sk2) and torch.equal(q2, qd)


@pytest.fixture(params=[1, 3, 4, 0], ids=["fast", "fast-wave-per-head", "fast-wave-per-64-positions", "general"])
def attn_mode(request, t12):
    t12.lib.t12_tune_attention(request.param)
    yield request.param
    t12.lib.t12_tune_attention(1)


@pytest.mark.parametrize("nh,nkv,hd,seq", [(32, 8, 128, 1), (32, 8, 128, 300), (32, 8, 128, 1500), (4, 4, 64, 77),
                                            (16, 1, 32, 513), (8, 8, 128, 130), (16, 2, 128, 65), (16, 4, 64, 257)])
def test_attention_b1_both_names(t12, oracle, attn_mode, nh, nkv, hd, seq):
    rng = np.random.default_rng(seq)
    max_seq = seq + 3
    q = rng.standard_normal(nh * hd).astype(np.float32)
    kc = rng.integers(-127, 128, size=(max_seq, nkv, hd)).astype(np.int8)
    vc = rng.integers(-127, 128, size=(max_seq, nkv, hd)).astype(np.int8)
    ks = (rng.random((max_seq, nkv)).astype(np.float32) + 0.5) / 127
    vs = (rng.random((max_seq, nkv)).astype(np.float32) + 0.5) / 127
    if seq % 2:      # odd lengths: a few outlier dims per head, 60x the rest (the INT8 limbs of Q scale with the head's maximum)
        q = q.reshape(nh, hd)
        q[:, [1, hd // 2, hd - 3]] *= 60.0
        q = q.reshape(-1)
        ks = ks * np.float32(0.02)        # keep the scores in a range where the softmax is not one-hot
    ref = oracle.attention_int8(q, kc, vc, ks, vs, seq, nh, nkv, hd)
    d = [torch.from_numpy(a).to(dev()) for a in (q, kc, vc, ks, vs)]
    for fn in (t12.lib.launch_attention_all_heads, t12.lib.launch_flash_attention):
        out = torch.zeros(nh * hd, dtype=torch.int16, device=dev())
        fn(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), d[4].data_ptr(), out.data_ptr(),
           nh, nkv, hd, seq, max_seq, 1.0 / np.sqrt(hd), st(t12))
        torch.cuda.synchronize()
        got = oracle.bf16_bits_to_f32(out.cpu().numpy().view(np.uint16))
        want = oracle.bf16_bits_to_f32(ref)
        assert np.abs(got - want).max() <= 2e-2 * np.abs(want).max()   # bf16 output: 2^-8 relative steps


def test_attention_batch_shared_and_strided_cache(t12, oracle, attn_mode):
    rng = np.random.default_rng(9)
    nh, nkv, hd, B, max_seq = 8, 2, 64, 3, 50
    positions = [4, 30, 49]
    q = rng.standard_normal((B, nh * hd)).astype(np.float32)
    kc = rng.integers(-127, 128, size=(B, max_seq, nkv, hd)).astype(np.int8)
    vc = rng.integers(-127, 128, size=(B, max_seq, nkv, hd)).astype(np.int8)
    ks = (rng.random((B, max_seq, nkv)).astype(np.float32) + 0.5) / 127
    vs = (rng.random((B, max_seq, nkv)).astype(np.float32) + 0.5) / 127
    d = [torch.from_numpy(a).to(dev()) for a in (q, kc, vc, ks, vs)]
    pd = torch.tensor(positions, dtype=torch.int32, device=dev())
    for stride, sel in ((0, lambda b: 0), (max_seq * nkv * hd, lambda b: b)):
        out = torch.zeros((B, nh * hd), dtype=torch.int16, device=dev())
        t12.lib.launch_attention_all_heads_batch(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                                 d[4].data_ptr(), out.data_ptr(), pd.data_ptr(), nh, nkv, hd,
                                                 max(positions) + 1, 1.0 / np.sqrt(hd), B, stride, st(t12))
        torch.cuda.synchronize()
        for b in range(B):
            s = sel(b)
            ref = oracle.attention_int8(q[b], kc[s], vc[s], ks[s], vs[s], positions[b] + 1, nh, nkv, hd)
            got = oracle.bf16_bits_to_f32(out.cpu().numpy()[b].view(np.uint16))
            want = oracle.bf16_bits_to_f32(ref)
            assert np.abs(got - want).max() <= 2e-2 * np.abs(want).max()


def test_argmax(t12, oracle):
    rng = np.random.default_rng(4)
    for (B, n) in [(1, 128256), (7, 1000), (256, 4099), (1, 5)]:
        x = rng.standard_normal((B, n)).astype(np.float32)
        x[0, n // 2] = x[0, n - 1] = 50.0        # exact tie: lowest index wins
        xd = torch.from_numpy(x).to(dev())
        r = torch.full((B,), -1, dtype=torch.int32, device=dev())
        if B == 1:
            t12.lib.launch_argmax(xd.data_ptr(), r.data_ptr(), n, st(t12))
        else:
            t12.lib.launch_argmax_batch(xd.data_ptr(), r.data_ptr(), n, B, st(t12))
        torch.cuda.synchronize()
        assert r.cpu().tolist() == [oracle.argmax_first(row) for row in x]
    nanrow = np.full((1, 300), np.nan, np.float32); nanrow[0, 17] = -3.0
    xd = torch.from_numpy(nanrow).to(dev()); r = torch.zeros(1, dtype=torch.int32, device=dev())
    t12.lib.launch_argmax(xd.data_ptr(), r.data_ptr(), 300, st(t12)); torch.cuda.synchronize()
    assert r.item() == 17


@pytest.mark.parametrize("nh,nkv,hd,B", [(32, 8, 128, 1), (32, 8, 128, 5), (4, 4, 64, 2), (8, 2, 32, 3)])
def test_fused_rope_store_attention_equals_separate_launches(t12, oracle, attn_mode, nh, nkv, hd, B):
    """launch_rope_store_attention == launch_rope_store_kv_batch + launch_attention_all_heads_batch:
    same caches, same scales, same bf16 output (the fused kernel leaves q unrotated)."""
    rng = np.random.default_rng(B)
    theta, max_seq, pos = 500000.0, 300, 277
    q, k, v = make_qkv(rng, B, nh, nkv, hd)
    q[1:], k[1:], v[1:] = q[0], k[0], v[0]          # lock-step copies: all sequences share one cache slot
    kc = rng.integers(-127, 128, size=(max_seq, nkv, hd)).astype(np.int8)
    vc = rng.integers(-127, 128, size=(max_seq, nkv, hd)).astype(np.int8)
    ks = (rng.random((max_seq, nkv)).astype(np.float32) + 0.5) / 127
    vs = (rng.random((max_seq, nkv)).astype(np.float32) + 0.5) / 127
    pd = torch.full((B,), pos, dtype=torch.int32, device=dev())
    sc = 1.0 / np.sqrt(hd)

    def fresh():
        return [torch.from_numpy(a.copy()).to(dev()) for a in (q, k, v, kc, vc, ks, vs)]

    a = fresh(); oa = torch.zeros((B, nh * hd), dtype=torch.int16, device=dev())
    t12.lib.launch_rope_store_kv_batch(a[0].data_ptr(), a[1].data_ptr(), a[2].data_ptr(), a[3].data_ptr(), a[4].data_ptr(),
                                       a[5].data_ptr(), a[6].data_ptr(), pd.data_ptr(), hd, nh, nkv, nh * hd, nkv * hd,
                                       theta, B, st(t12))
    t12.lib.launch_attention_all_heads_batch(a[0].data_ptr(), a[3].data_ptr(), a[4].data_ptr(), a[5].data_ptr(),
                                             a[6].data_ptr(), oa.data_ptr(), pd.data_ptr(), nh, nkv, hd, pos + 1, sc, B, 0,
                                             st(t12))
    for positions in ([pd.data_ptr()] if B > 1 else [pd.data_ptr(), None]):
        f = fresh(); of = torch.zeros_like(oa)
        t12.lib.launch_rope_store_attention(f[0].data_ptr(), f[1].data_ptr(), f[2].data_ptr(), f[3].data_ptr(),
                                            f[4].data_ptr(), f[5].data_ptr(), f[6].data_ptr(), of.data_ptr(), positions,
                                            pos, nh, nkv, hd, theta, sc, B, 0, st(t12))
        torch.cuda.synchronize()
        assert torch.equal(f[3], a[3]) and torch.equal(f[4], a[4])      # caches
        assert torch.equal(f[5], a[5]) and torch.equal(f[6], a[6])      # scales
        if positions is not None:
            assert torch.equal(of, oa)
        else:
            # without a position array the launch may be split along the context: other tile boundaries, other
            # rounding of the partial sums (and of the INT8 weight limbs of the long-context form)
            got = oracle.bf16_bits_to_f32(of.cpu().numpy().view(np.uint16))
            want = oracle.bf16_bits_to_f32(oa.cpu().numpy().view(np.uint16))
            assert np.abs(got - want).max() <= 2.0 ** -7 * np.abs(want).max()


@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 128), (8, 2, 32), (4, 4, 64)])
def test_per_sequence_caches_fused_and_from_partial_sums(t12, oracle, attn_mode, nh, nkv, hd):
    """Independent sequences, each with its own cache region (kv_stride != 0) and its own position: the fused
    launch and the launch that first adds up K-split partial sums of q | k | v both equal one separate
    RoPE/store + attention launch per sequence on that sequence's region."""
    rng = np.random.default_rng(hd)
    B, theta, max_seq = 3, 500000.0, 96
    pos = [70, 5, 33]
    q, k, v = make_qkv(rng, B, nh, nkv, hd)
    kc = rng.integers(-127, 128, size=(B, max_seq, nkv, hd)).astype(np.int8)
    vc = rng.integers(-127, 128, size=(B, max_seq, nkv, hd)).astype(np.int8)
    ks = (rng.random((B, max_seq, nkv)).astype(np.float32) + 0.5) / 127
    vs = (rng.random((B, max_seq, nkv)).astype(np.float32) + 0.5) / 127
    pd = torch.tensor(pos, dtype=torch.int32, device=dev())
    sc = 1.0 / np.sqrt(hd)
    kv_stride = max_seq * nkv * hd
    # partial sums of the fused [q | k | v] row: two splits whose fp32 sum is the value itself
    row = np.concatenate([q.reshape(B, -1), k.reshape(B, -1), v.reshape(B, -1)], axis=1).astype(np.float32)
    p0 = (rng.standard_normal(row.shape) * 0.5).astype(np.float32)
    p1 = (row - p0).astype(np.float32)
    row = (p0 + p1).astype(np.float32)
    nq, nk = nh * hd, nkv * hd
    q, k, v = row[:, :nq].copy(), row[:, nq:nq + nk].copy(), row[:, nq + nk:].copy()

    def fresh():
        return [torch.from_numpy(a.copy()).to(dev()) for a in (q, k, v, kc, vc, ks, vs)]

    a = fresh(); oa = torch.zeros((B, nq), dtype=torch.int16, device=dev())
    for b in range(B):                      # one sequence at a time on its own region
        t12.lib.launch_rope_store_kv_batch(a[0][b].data_ptr(), a[1][b].data_ptr(), a[2][b].data_ptr(), a[3][b].data_ptr(),
                                           a[4][b].data_ptr(), a[5][b].data_ptr(), a[6][b].data_ptr(), pd[b:].data_ptr(),
                                           hd, nh, nkv, nq, nk, theta, 1, st(t12))
        t12.lib.launch_attention_all_heads_batch(a[0][b].data_ptr(), a[3][b].data_ptr(), a[4][b].data_ptr(),
                                                 a[5][b].data_ptr(), a[6][b].data_ptr(), oa[b].data_ptr(), pd[b:].data_ptr(),
                                                 nh, nkv, hd, max_seq, sc, 1, 0, st(t12))
    f = fresh(); of = torch.zeros_like(oa)
    t12.lib.launch_rope_store_attention(f[0].data_ptr(), f[1].data_ptr(), f[2].data_ptr(), f[3].data_ptr(), f[4].data_ptr(),
                                        f[5].data_ptr(), f[6].data_ptr(), of.data_ptr(), pd.data_ptr(), 0, nh, nkv, hd,
                                        theta, sc, B, kv_stride, st(t12))
    g = fresh(); og = torch.zeros_like(oa)
    g[0].zero_(); g[1].zero_(); g[2].zero_()                  # the values come from the partial sums only
    ws = torch.from_numpy(np.stack([p0, p1])).to(dev())
    t12.lib.launch_rope_store_attention_partials(g[0].data_ptr(), g[1].data_ptr(), g[2].data_ptr(), g[3].data_ptr(),
                                                 g[4].data_ptr(), g[5].data_ptr(), g[6].data_ptr(), og.data_ptr(),
                                                 pd.data_ptr(), 0, nh, nkv, hd, theta, sc, B, ws.data_ptr(), 2,
                                                 B * row.shape[1], row.shape[1], kv_stride, st(t12))
    torch.cuda.synchronize()
    assert not torch.equal(a[3], torch.from_numpy(kc).to(dev()))         # the stores happened
    for x in (f, g):
        assert torch.equal(x[3], a[3]) and torch.equal(x[4], a[4])      # caches: only each sequence's own slot changed
        assert torch.equal(x[5], a[5]) and torch.equal(x[6], a[6])      # scales
    assert torch.equal(of, oa) and torch.equal(og, oa)
    assert not torch.equal(oa[0], oa[1])


@pytest.mark.parametrize("nh,nkv,hd,B,pos", [(32, 8, 128, 3, [70, 5, 33]), (32, 8, 128, 40, None), (8, 2, 32, 3, [1, 90, 64]),
                                             (4, 4, 64, 2, [300, 17]), (32, 8, 128, 1, [1290]), (32, 8, 128, 2, [700, 700])])
def test_head_major_regions_equal_the_reference_layout(t12, oracle, attn_mode, nh, nkv, hd, B, pos):
    """launch_rope_store_attention_regions / _partials_regions work on regions laid out [kv head][position][dim]
    (scales [kv head][position]).  On the transposed data they give bit-identical outputs, rotated q / k, and --
    transposed back -- bit-identical caches and scales, for per-sequence regions with a position array (fused form at
    small batches, separate launches at B = 40), for the launch fed by K-split partial sums, and for one region without a
    position array (the context-split form at long contexts, lock-step rows)."""
    rng = np.random.default_rng(hd + B)
    theta = 500000.0
    shared = B <= 2 and pos[0] == pos[-1] and pos[0] >= 700          # one region, no position array
    if pos is None:
        pos = [int(x) for x in rng.integers(0, 280, size=B)]
    max_seq = max(pos) + 9
    R = 1 if shared else B                                          # regions
    q, k, v = make_qkv(rng, B, nh, nkv, hd)
    if shared:
        q[1:], k[1:], v[1:] = q[0], k[0], v[0]
    kc = rng.integers(-127, 128, size=(R, max_seq, nkv, hd)).astype(np.int8)
    vc = rng.integers(-127, 128, size=(R, max_seq, nkv, hd)).astype(np.int8)
    ks = (rng.random((R, max_seq, nkv)).astype(np.float32) + 0.5) / 127
    vs = (rng.random((R, max_seq, nkv)).astype(np.float32) + 0.5) / 127
    hm = lambda a: np.ascontiguousarray(np.swapaxes(a, 1, 2))       # [R, pos, head, ...] <-> [R, head, pos, ...]
    pd = torch.tensor(pos, dtype=torch.int32, device=dev())
    sc = 1.0 / np.sqrt(hd)
    kv_stride = 0 if shared else max_seq * nkv * hd
    pptr = None if shared else pd.data_ptr()
    nq, nk = nh * hd, nkv * hd
    row = np.concatenate([q.reshape(B, -1), k.reshape(B, -1), v.reshape(B, -1)], axis=1).astype(np.float32)
    p0 = (rng.standard_normal(row.shape) * 0.5).astype(np.float32)
    if shared:
        p0[1:] = p0[0]                                              # lock-step rows store one slot: bit-identical rows
    p1 = (row - p0).astype(np.float32)
    row = (p0 + p1).astype(np.float32)
    q, k, v = row[:, :nq].copy(), row[:, nq:nq + nk].copy(), row[:, nq + nk:].copy()
    ws = torch.from_numpy(np.stack([p0, p1])).to(dev())

    def run(head_major, partials):
        arrs = (q, k, v, hm(kc), hm(vc), hm(ks), hm(vs)) if head_major else (q, k, v, kc, vc, ks, vs)
        f = [torch.from_numpy(a.copy()).to(dev()) for a in arrs]
        o = torch.zeros((B, nq), dtype=torch.int16, device=dev())
        head = [f[i].data_ptr() for i in range(7)] + [o.data_ptr(), pptr, max(pos), nh, nkv, hd, theta, sc, B]
        if partials:
            f[0].zero_(); f[1].zero_(); f[2].zero_()
            tail = [ws.data_ptr(), 2, B * row.shape[1], row.shape[1], kv_stride]
            if head_major:
                t12.lib.launch_rope_store_attention_partials_regions(*head, *tail, max_seq, st(t12))
            else:
                t12.lib.launch_rope_store_attention_partials(*head, *tail, st(t12))
        elif head_major:
            t12.lib.launch_rope_store_attention_regions(*head, kv_stride, max_seq, st(t12))
        else:
            t12.lib.launch_rope_store_attention(*head, kv_stride, st(t12))
        torch.cuda.synchronize()
        if head_major:
            for i in (3, 4, 5, 6):
                f[i] = f[i].transpose(1, 2).contiguous()
        return f, o

    for partials in (False, True):
        if partials and shared and B == 1:
            continue                                                # (the K-split launch is a batch path)
        a, oa = run(False, partials)
        b, ob = run(True, partials)
        assert not torch.equal(a[3], torch.from_numpy(kc).to(dev()))
        for i in range(7):
            assert torch.equal(a[i], b[i]), (partials, i)
        assert torch.equal(oa, ob), partials


@pytest.mark.parametrize("nh,nkv,hd,B,pos", [(32, 8, 128, 1, 1290), (32, 8, 128, 2, 700), (16, 4, 64, 3, 333)])
def test_context_split_equals_single_pass(t12, oracle, nh, nkv, hd, B, pos):
    """A launch without a position array at a long context is split along the context (partial softmax per
    chunk, folded by the workgroup that finishes last).  Same result as the single pass up to the order of the
    fp32 sums, on repeated launches (the arrival counters reset themselves), for the fused and the plain launch."""
    rng = np.random.default_rng(pos)
    theta, max_seq = 500000.0, pos + 9
    q, k, v = make_qkv(rng, B, nh, nkv, hd)
    q[1:], k[1:], v[1:] = q[0], k[0], v[0]                     # lock-step copies on one cache region
    kc = rng.integers(-127, 128, size=(max_seq, nkv, hd)).astype(np.int8)
    vc = rng.integers(-127, 128, size=(max_seq, nkv, hd)).astype(np.int8)
    ks = (rng.random((max_seq, nkv)).astype(np.float32) + 0.5) / 127
    vs = (rng.random((max_seq, nkv)).astype(np.float32) + 0.5) / 127
    sc = 1.0 / np.sqrt(hd)

    def run(mode):
        t12.lib.t12_tune_attention(mode)
        f = [torch.from_numpy(a.copy()).to(dev()) for a in (q, k, v, kc, vc, ks, vs)]
        of = torch.zeros((B, nh * hd), dtype=torch.int16, device=dev())
        t12.lib.launch_rope_store_attention(f[0].data_ptr(), f[1].data_ptr(), f[2].data_ptr(), f[3].data_ptr(),
                                            f[4].data_ptr(), f[5].data_ptr(), f[6].data_ptr(), of.data_ptr(), None, pos,
                                            nh, nkv, hd, theta, sc, B, 0, st(t12))
        torch.cuda.synchronize()
        return f, of

    try:
        base, ob = run(2)                                       # never split
        want = oracle.bf16_bits_to_f32(ob.cpu().numpy().view(np.uint16))
        for mode in (1, 64, 1):                                 # default, many small chunks, default again
            f, of = run(mode)
            assert torch.equal(f[3], base[3]) and torch.equal(f[4], base[4])
            assert torch.equal(f[5], base[5]) and torch.equal(f[6], base[6])
            got = oracle.bf16_bits_to_f32(of.cpu().numpy().view(np.uint16))
            assert np.abs(got - want).max() <= 2.0 ** -7 * np.abs(want).max(), mode     # a bf16 step at most
            assert torch.equal(of[0], of[B - 1])
        # against the CPU restatement, through the plain launcher (sequence 0)
        # q in `base` was left unrotated by the fused launch: rotate on the CPU for the reference
        qr = oracle.rope(q[0], pos, nh, hd, theta)
        ref = oracle.attention_int8(qr, base[3].cpu().numpy(), base[4].cpu().numpy(), base[5].cpu().numpy(),
                                    base[6].cpu().numpy(), pos + 1, nh, nkv, hd)
        wantr = oracle.bf16_bits_to_f32(ref)
        assert np.abs(want[0] - wantr).max() <= 2e-2 * np.abs(wantr).max()
    finally:
        t12.lib.t12_tune_attention(1)


def test_measurement_aids_return_plausible_figures(t12):
    """t12_probe_clock and t12_probe_launch_gap (no counterpart in the reference): they run, return T12_OK and figures
    a gfx950 can have; bad operands are refused on the host."""
    import ctypes as C
    ghz, tf, us = C.c_double(), C.c_double(), C.c_double()
    assert t12.lib.t12_probe_clock(64, 200, 0, C.byref(ghz), C.byref(tf), st(t12)) == 0
    assert 0.5 < ghz.value < 3.0 and 10.0 < tf.value < 2500.0, (ghz.value, tf.value)
    assert t12.lib.t12_probe_clock(64, 200, 1, C.byref(ghz), C.byref(tf), st(t12)) == 0
    assert 0.5 < ghz.value < 3.0 and 1.0 < tf.value < 2500.0, (ghz.value, tf.value)
    for any_order in (0, 1):
        assert t12.lib.t12_probe_launch_gap(200, any_order, C.byref(us), st(t12)) == 0
        assert 0.2 < us.value < 50.0, us.value
    assert t12.lib.t12_probe_launch_gap(0, 0, C.byref(us), st(t12)) < 0
    assert t12.lib.t12_probe_clock(0, 1, 0, C.byref(ghz), C.byref(tf), st(t12)) < 0
