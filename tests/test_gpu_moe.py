"""GPU parity: Mixtral-shaped MoE FFN (top-2 of 8 split-12 experts, tokens grouped per expert
through the decode+GEMM) -- small layer against the CPU oracle, full-size layer against a
decode-then-fp32 matmul of the same (bit-exact, separately tested) decoded weights.

Tolerance: 1e-2 relative (the target); observed ~1e-5 (fp32 accumulation order only; the
SwiGLU activation is rounded to bf16 on both sides, as the engine does between the two GEMMs).
"""
import importlib

import numpy as np
import pytest
import torch

from gpu_util import dev, rel_err, to_dev_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def synth(t12):
    return importlib.import_module("turbo_lossless_amd.synth")


@pytest.fixture(scope="module")
def moe(t12):
    return importlib.import_module("turbo_lossless_amd.moe")


def bf16_to_f32(bits):
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def test_moe_small_vs_oracle(t12, oracle, synth, moe):
    E, n, n_ff, T = 8, 512, 1024, 64
    packs = [[oracle.pack(synth.weights_llm(m, k, seed=5000 + 3 * e + j, p_outlier=5e-4))
              for j, (m, k) in enumerate([(n_ff, n), (n_ff, n), (n, n_ff)])] for e in range(E)]
    experts = [moe.Expert(*[t12.DeviceTensor12.from_packed(p, dev()) for p in ps]) for ps in packs]
    X = synth.activations(T, n, seed=77)
    rng = np.random.default_rng(5)
    logits = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).to(dev())
    ids, w = moe.route_top_k(logits, 2)
    got = moe.moe_ffn(experts, to_dev_bits(X).reshape(T, n), ids, w).cpu().numpy()
    ids_h, w_h = ids.cpu().numpy(), w.cpu().numpy()
    assert sorted(np.bincount(ids_h.reshape(-1), minlength=E).tolist())[0] >= 0      # ragged groups, some may be empty
    ref = np.zeros((T, n), np.float64)
    for e in range(E):
        rows, slots = np.nonzero(ids_h == e)
        if len(rows) == 0:
            continue
        xe = X[rows]
        g = oracle.gemm(packs[e][0], xe)
        u = oracle.gemm(packs[e][1], xe)
        a = oracle.silu_mul_bf16(g, u)
        y = oracle.gemm(packs[e][2], a)
        ref[rows] += w_h[rows, slots][:, None].astype(np.float64) * y
    assert rel_err(got, ref) < 1e-4


def test_moe_single_expert_gets_every_token(t12, oracle, synth, moe):
    # all tokens routed to one expert (the other seven groups are empty): equals a plain FFN
    E, n, n_ff, T = 4, 256, 512, 33
    packs = [[oracle.pack(synth.weights_llm(m, k, seed=60 + 3 * e + j)) for j, (m, k) in
              enumerate([(n_ff, n), (n_ff, n), (n, n_ff)])] for e in range(E)]
    experts = [moe.Expert(*[t12.DeviceTensor12.from_packed(p, dev()) for p in ps]) for ps in packs]
    X = synth.activations(T, n, seed=78)
    ids = torch.full((T, 1), 2, dtype=torch.int64, device=dev())
    w = torch.ones((T, 1), dtype=torch.float32, device=dev())
    got = moe.moe_ffn(experts, to_dev_bits(X).reshape(T, n), ids, w).cpu().numpy()
    a = oracle.silu_mul_bf16(oracle.gemm(packs[2][0], X), oracle.gemm(packs[2][1], X))
    assert rel_err(got, oracle.gemm(packs[2][2], a)) < 1e-4


def test_moe_mixtral_shape_b256(t12, synth, moe):
    # full size: 8 experts x (4096 -> 14336 -> 4096), 256 tokens, top-2; weights N(0, 0.02) + 5e-4 outliers
    E, n, n_ff, T = 8, 4096, 14336, 256
    g = torch.Generator(device=dev())

    def mk(M, K, seed):
        g.manual_seed(seed)
        wt = torch.randn((M, K), generator=g, device=dev()) * 0.02
        m = torch.rand((M, K), generator=g, device=dev()) < 5e-4
        wt = torch.where(m, torch.randn((M, K), generator=g, device=dev()) * 8, wt).to(torch.bfloat16)
        return t12.pack_device(wt)

    experts = [moe.Expert(mk(n_ff, n, 5000 + 3 * e), mk(n_ff, n, 5001 + 3 * e), mk(n, n_ff, 5002 + 3 * e))
               for e in range(E)]
    g.manual_seed(9)
    Xf = torch.randn((T, n), generator=g, device=dev()).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g, device=dev())
    ids, w = moe.route_top_k(logits, 2)
    got = moe.moe_ffn(experts, Xf.view(torch.int16), ids, w)
    torch.cuda.synchronize()
    ref = torch.zeros((T, n), dtype=torch.float32, device=dev())
    for e in range(E):
        rows, slots = torch.nonzero(ids == e, as_tuple=True)
        if rows.numel() == 0:
            continue
        dec = [t12.decompress(t).view(torch.bfloat16).float() for t in (experts[e].w1, experts[e].w3, experts[e].w2)]
        xe = Xf[rows].float()
        gate, up = xe @ dec[0].t(), xe @ dec[1].t()
        a = (torch.nn.functional.silu(gate) * up).to(torch.bfloat16).float()
        ref[rows] += w[rows, slots][:, None] * (a @ dec[2].t())
        del dec
    err = float((got - ref).abs().max() / ref.abs().max())
    assert err < 1e-2, err


@pytest.mark.parametrize("batches", [[40, 0, 64, 7, 1, 33], [130, 64, 65, 3], [300, 20], [16, 9, 2, 5]])
@pytest.mark.parametrize("M,K", [(384, 1024), (1000, 4096), (128, 14336), (100, 192)])
def test_grouped_gemm_vs_oracle(t12, oracle, synth, moe, M, K, batches):
    """t12_gemm_grouped: every group its own tensor (own base_exp), activations and batch in one launch -- batch
    tiles of 64 / 128 / 256 rows by the largest group, empty groups, K splits (few row tiles) with the per-group
    workspace layout, K = 192 (three stages: an odd window), M not a multiple of the row tile."""
    rng = np.random.default_rng(M + K + len(batches))
    packs, Xs, items, outs = [], [], [], []
    for i, B in enumerate(batches):
        p = oracle.pack(synth.weights_llm(M, K, seed=300 + i, sigma=float(rng.choice([0.002, 0.02, 0.3])), p_outlier=1e-3))
        X = synth.activations(max(B, 1), K, seed=400 + i)[:B]
        out = torch.full((B, M), float("nan"), device=dev())
        packs.append(p); Xs.append(X); outs.append(out)
        xd = to_dev_bits(X).reshape(B, K) if B else torch.empty((0, K), dtype=torch.int16, device=dev())
        items.append((t12.DeviceTensor12.from_packed(p, dev()), xd, out))
    moe.gemm_grouped(items, K)
    torch.cuda.synchronize()
    for p, X, out in zip(packs, Xs, outs):
        if X.shape[0]:
            assert rel_err(out.cpu().numpy(), oracle.gemm(p, X)) < 1e-4


def test_grouped_gemm_general_path_and_errors(t12, oracle, synth, moe):
    """K not a multiple of 64 and a tensor of subnormals (base_exp -1): the groups run one by one through t12_gemm's
    general kernel; more than 16 groups and a short activation stride are refused."""
    K = 100
    ps = [oracle.pack(synth.weights_llm(50, K, seed=1)), oracle.pack(np.full((20, K), 0x0001, np.uint16))]
    Xs = [synth.activations(5, K, seed=2), synth.activations(70, K, seed=3)]
    outs = [torch.full((X.shape[0], p.M), float("nan"), device=dev()) for p, X in zip(ps, Xs)]
    items = [(t12.DeviceTensor12.from_packed(p, dev()), to_dev_bits(X).reshape(-1, K), o) for p, X, o in zip(ps, Xs, outs)]
    moe.gemm_grouped(items, K)
    torch.cuda.synchronize()
    for p, X, o in zip(ps, Xs, outs):
        ref = oracle.gemm(p, X)
        assert np.abs(o.cpu().numpy() - ref).max() <= 1e-4 * max(np.abs(ref).max(), 1e-30)
    with pytest.raises(t12.T12Error, match="groups"):
        moe.gemm_grouped([items[0]] * 17, K)
    with pytest.raises(t12.T12Error, match="act_stride"):
        moe.gemm_grouped([items[0]], K + 8)


def test_moe_route_tables_and_refusals(t12, oracle, synth, moe):
    """Ragged routing incl. an expert nobody chose, int32 ids, a strided activation matrix, k = 3: against the
    oracle's per-expert products; an id outside the experts is left out and reported by status()."""
    E, n, n_ff, T, k = 5, 256, 512, 77, 3
    packs = [[oracle.pack(synth.weights_llm(m, kk, seed=900 + 3 * e + j, p_outlier=1e-3))
              for j, (m, kk) in enumerate([(n_ff, n), (n_ff, n), (n, n_ff)])] for e in range(E)]
    layer = moe.MoeLayer([moe.Expert(*[t12.DeviceTensor12.from_packed(p, dev()) for p in ps]) for ps in packs])
    X = synth.activations(T, n, seed=79)
    rng = np.random.default_rng(8)
    ids_h = np.stack([rng.choice([0, 1, 2, 4], size=k, replace=False) for _ in range(T)]).astype(np.int32)   # expert 3 unused
    w_h = rng.random((T, k)).astype(np.float32)
    Xd = torch.zeros((T, n + 24), dtype=torch.int16, device=dev())
    Xd[:, :n] = to_dev_bits(X).reshape(T, n)
    for _ in range(2):                                      # the second call reuses the workspace
        got = layer(Xd[:, :n], torch.from_numpy(ids_h).to(dev()), torch.from_numpy(w_h).to(dev())).cpu().numpy()
    ref = np.zeros((T, n), np.float64)
    for e in range(E):
        rows, slots = np.nonzero(ids_h == e)
        if len(rows) == 0:
            continue
        a = oracle.silu_mul_bf16(oracle.gemm(packs[e][0], X[rows]), oracle.gemm(packs[e][1], X[rows]))
        ref[rows] += w_h[rows, slots][:, None].astype(np.float64) * oracle.gemm(packs[e][2], a)
    assert rel_err(got, ref) < 1e-4
    layer.status()                                          # nothing to report
    # an id outside the experts: its pair is left out of the sum, and status() says so
    bad = ids_h.copy()
    bad[5, 1] = E
    got_bad = layer(Xd[:, :n], torch.from_numpy(bad).to(dev()), torch.from_numpy(w_h).to(dev())).cpu().numpy()
    with pytest.raises(t12.T12Error, match="outside"):
        layer.status()
    e5 = int(ids_h[5, 1])
    a = oracle.silu_mul_bf16(oracle.gemm(packs[e5][0], X[5:6]), oracle.gemm(packs[e5][1], X[5:6]))
    ref_bad = ref.copy()
    ref_bad[5] -= float(w_h[5, 1]) * oracle.gemm(packs[e5][2], a)[0].astype(np.float64)
    assert rel_err(got_bad, ref_bad) < 1e-4
    # tokens that name one expert twice: an expert then receives more rows than there are tokens (and more than one
    # batch tile); both slots count
    twice = ids_h.copy()
    twice[:, 1] = twice[:, 0]
    twice[:, 2] = twice[:, 0]
    twice[:, 0] = 0                                          # expert 0 receives every token at least once
    got2 = layer(Xd[:, :n], torch.from_numpy(twice).to(dev()), torch.from_numpy(w_h).to(dev())).cpu().numpy()
    layer.status()
    ref2 = np.zeros((T, n), np.float64)
    for e in range(E):
        rows, slots = np.nonzero(twice == e)
        if len(rows) == 0:
            continue
        a = oracle.silu_mul_bf16(oracle.gemm(packs[e][0], X[rows]), oracle.gemm(packs[e][1], X[rows]))
        np.add.at(ref2, rows, w_h[rows, slots][:, None].astype(np.float64) * oracle.gemm(packs[e][2], a))
    assert np.bincount(twice.ravel(), minlength=E).max() > T
    assert rel_err(got2, ref2) < 1e-4


def test_moe_twenty_experts_in_several_grouped_launches(t12, oracle, synth, moe):
    """More experts than one grouped launch holds (16 groups): gate|up go out eight experts at a time, down sixteen."""
    E, n, n_ff, T, k = 20, 128, 256, 90, 2
    packs = [[oracle.pack(synth.weights_llm(m, kk, seed=1300 + 3 * e + j, p_outlier=1e-3))
              for j, (m, kk) in enumerate([(n_ff, n), (n_ff, n), (n, n_ff)])] for e in range(E)]
    layer = moe.MoeLayer([moe.Expert(*[t12.DeviceTensor12.from_packed(p, dev()) for p in ps]) for ps in packs])
    X = synth.activations(T, n, seed=80)
    rng = np.random.default_rng(9)
    ids_h = np.stack([rng.choice(E, size=k, replace=False) for _ in range(T)]).astype(np.int64)
    w_h = rng.random((T, k)).astype(np.float32)
    got = layer(to_dev_bits(X).reshape(T, n), torch.from_numpy(ids_h).to(dev()), torch.from_numpy(w_h).to(dev())).cpu().numpy()
    ref = np.zeros((T, n), np.float64)
    for e in range(E):
        rows, slots = np.nonzero(ids_h == e)
        if len(rows) == 0:
            continue
        a = oracle.silu_mul_bf16(oracle.gemm(packs[e][0], X[rows]), oracle.gemm(packs[e][1], X[rows]))
        ref[rows] += w_h[rows, slots][:, None].astype(np.float64) * oracle.gemm(packs[e][2], a)
    assert rel_err(got, ref) < 1e-4
    with pytest.raises(t12.T12Error, match="experts"):
        moe.MoeLayer([layer.experts[0]] * 129)(to_dev_bits(X).reshape(T, n), torch.from_numpy(ids_h).to(dev()),
                                               torch.from_numpy(w_h).to(dev()))


def test_moe_sixty_four_experts_and_a_shape_sized_on_the_host(t12, oracle, synth, moe):
    """64 experts (the routing sort's count rows take more than 48 KB of LDS), top-4; 128 experts, the most the call takes
    (131 KB of count rows), top-3; and a layer whose widths are not
    multiples of 64, which the tile kernel does not take: its launches are sized from a host copy of the counts."""
    for E, n, n_ff, T, k, seed in [(64, 128, 128, 150, 4, 1500), (128, 64, 64, 90, 3, 1600), (3, 96, 160, 40, 2, 1700)]:
        packs = [[oracle.pack(synth.weights_llm(m, kk, seed=seed + 3 * e + j, p_outlier=1e-3))
                  for j, (m, kk) in enumerate([(n_ff, n), (n_ff, n), (n, n_ff)])] for e in range(E)]
        layer = moe.MoeLayer([moe.Expert(*[t12.DeviceTensor12.from_packed(p, dev()) for p in ps]) for ps in packs])
        X = synth.activations(T, n, seed=seed + 1)
        rng = np.random.default_rng(seed)
        ids_h = np.stack([rng.choice(E, size=k, replace=False) for _ in range(T)]).astype(np.int32)
        w_h = rng.random((T, k)).astype(np.float32)
        got = layer(to_dev_bits(X).reshape(T, n), torch.from_numpy(ids_h).to(dev()), torch.from_numpy(w_h).to(dev())).cpu().numpy()
        layer.status()
        ref = np.zeros((T, n), np.float64)
        for e in range(E):
            rows, slots = np.nonzero(ids_h == e)
            if len(rows) == 0:
                continue
            a = oracle.silu_mul_bf16(oracle.gemm(packs[e][0], X[rows]), oracle.gemm(packs[e][1], X[rows]))
            ref[rows] += w_h[rows, slots][:, None].astype(np.float64) * oracle.gemm(packs[e][2], a)
        assert rel_err(got, ref) < 1e-4, (E, n)


def test_moe_few_rows_per_expert_and_one_expert_above_sixteen(t12, oracle, synth, moe):
    """Few (token, expert) pairs per expert on average: the layer takes the kernel that sweeps whole rows and reads each
    expert's row count on the device; experts nobody names cost nothing, and an expert that, against the odds, gets
    more than 16 rows (every token names expert 3 here) is swept once per 16 rows."""
    E, n, n_ff, seed = 16, 128, 256, 2300
    packs = [[oracle.pack(synth.weights_llm(m, kk, seed=seed + 3 * e + j, p_outlier=1e-3))
              for j, (m, kk) in enumerate([(n_ff, n), (n_ff, n), (n, n_ff)])] for e in range(E)]
    layer = moe.MoeLayer([moe.Expert(*[t12.DeviceTensor12.from_packed(p, dev()) for p in ps]) for ps in packs])
    rng = np.random.default_rng(seed)
    cases = []
    T = 24
    cases.append((T, np.full((T, 1), 3, np.int32)))                                   # one expert, 24 rows
    ids = np.stack([np.array([3, 1 + rng.integers(0, 2) * 8]) for _ in range(17)]).astype(np.int32)
    cases.append((17, ids))                                                            # 17 rows on expert 3, the rest on 1 / 9
    cases.append((1, np.array([[5, 11]], np.int32)))                                   # a single token, top-2
    cases.append((3, np.stack([rng.choice(E, size=2, replace=False) for _ in range(3)]).astype(np.int32)))
    for T, ids_h in cases:
        k = ids_h.shape[1]
        X = synth.activations(T, n, seed=seed + T)
        w_h = rng.random((T, k)).astype(np.float32)
        got = layer(to_dev_bits(X).reshape(T, n), torch.from_numpy(ids_h).to(dev()), torch.from_numpy(w_h).to(dev())).cpu().numpy()
        layer.status()
        ref = np.zeros((T, n), np.float64)
        for e in range(E):
            rows, slots = np.nonzero(ids_h == e)
            if len(rows) == 0:
                continue
            a = oracle.silu_mul_bf16(oracle.gemm(packs[e][0], X[rows]), oracle.gemm(packs[e][1], X[rows]))
            ref[rows] += w_h[rows, slots][:, None].astype(np.float64) * oracle.gemm(packs[e][2], a)
        assert rel_err(got, ref) < 1e-4, (T, k)


def test_moe_handful_of_pairs_runs_matrix_vector_products(t12, oracle, synth, moe):
    """Up to eight (token, expert) pairs on at most eight experts of 2048 columns and more: each slot is one
    matrix-vector product with the tensors of its expert, picked on the device (gate|up with the SwiGLU in the
    epilogue, then down).  One token with top-2 and top-1, four tokens that share experts, a pair list that names one
    expert in every slot, an id out of range (left out, flagged), rows of 2048 and 2560 columns with escapes."""
    E, n, n_ff, seed = 8, 2048, 2560, 2400
    packs = [[oracle.pack(synth.weights_llm(m, kk, seed=seed + 3 * e + j, p_outlier=1e-3))
              for j, (m, kk) in enumerate([(n_ff, n), (n_ff, n), (n, n_ff)])] for e in range(E)]
    layer = moe.MoeLayer([moe.Expert(*[t12.DeviceTensor12.from_packed(p, dev()) for p in ps]) for ps in packs])
    rng = np.random.default_rng(seed)
    cases = [np.array([[5, 2]], np.int32), np.array([[7]], np.int32),
             np.array([[0, 3], [3, 1], [6, 0], [3, 7]], np.int32), np.full((8, 1), 4, np.int32),
             np.array([[1, 9], [2, 1]], np.int32)]
    for ids_h in cases:
        T, k = ids_h.shape
        X = synth.activations(T, n, seed=seed + 11 * T + k)
        w_h = rng.random((T, k)).astype(np.float32)
        got = layer(to_dev_bits(X).reshape(T, n), torch.from_numpy(ids_h).to(dev()), torch.from_numpy(w_h).to(dev())).cpu().numpy()
        if (ids_h >= E).any():
            with pytest.raises(t12.T12Error):
                layer.status()
        else:
            layer.status()
        ref = np.zeros((T, n), np.float64)
        for e in range(E):
            rows, slots = np.nonzero(ids_h == e)
            if len(rows) == 0:
                continue
            a = oracle.silu_mul_bf16(oracle.gemm(packs[e][0], X[rows]), oracle.gemm(packs[e][1], X[rows]))
            ref[rows] += w_h[rows, slots][:, None].astype(np.float64) * oracle.gemm(packs[e][2], a)
        assert rel_err(got, ref) < 1e-4, ids_h.tolist()
