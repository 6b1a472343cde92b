"""GPU parity: seeded random sweeps over shapes, batch sizes, escape densities, forced base exponents, routings and model
configurations -- the cases nobody thought of listing.  Each sweep is bounded (a few seconds) and reproducible.

Error measures: a GEMV / GEMM output is compared with the oracle's against sum_k |w||x| of that output, the quantity fp32
rounding scales with (a single output whose terms cancel has no meaningful error relative to itself); the bound 3e-5
leaves room for K up to 5120 and is a thousand times below what a wrong element or a dropped term gives."""
import importlib
import os
import shutil
import tempfile

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
    return importlib.import_module(t12.__name__ + ".moe")


def test_random_gemm_and_gemv(t12, oracle, synth):
    rng = np.random.default_rng(20241)
    done = 0
    while done < 160:
        nseg = int(rng.choice([1, 1, 2, 3]))
        kind = int(rng.integers(0, 6))
        K = [int(rng.integers(1, 40)) * 64, int(rng.integers(1, 12)) * 128, int(rng.integers(1, 5)) * 1024,
             int(rng.integers(1, 700)), int(rng.integers(1, 20)) * 16, int(rng.choice([4096, 5120, 1280, 2048]))][kind]
        Ms = [int(rng.choice([1, 7, 16, 17, 31, 64, 100, 127, 128, 129, 200, 255, 256, 300, 513])) for _ in range(nseg)]
        B = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300]))
        if K * max(Ms) * B > 1e8:
            continue
        p_out = float(rng.choice([0.0, 3e-4, 2e-3, 2e-2, 0.2]))
        seed = int(rng.integers(0, 1 << 30))
        packs = []
        for i, M in enumerate(Ms):
            W = synth.weights_llm(M, K, seed=seed + i, p_outlier=p_out)
            packs.append(oracle.pack(W, int(rng.integers(100, 126))) if rng.random() < 0.15 else oracle.pack(W))
        X = synth.activations(B, K, seed=seed + 77)
        case = (Ms, K, B, p_out, seed)
        dts = [t12.DeviceTensor12.from_packed(p, dev()) for p in packs]
        Xf = np.abs(oracle.bf16_bits_to_f32(X).astype(np.float64))
        absw = [np.abs(np.nan_to_num(oracle.bf16_bits_to_f32(oracle.decode(p)).astype(np.float64))) for p in packs]
        outs = t12.gemm(dts, to_dev_bits(X).reshape(X.shape))
        torch.cuda.synchronize()
        for p, o, aw in zip(packs, outs, absw):
            err = np.abs(o.cpu().numpy().astype(np.float64) - oracle.gemm(p, X)) / (Xf @ aw.T + 1e-30)
            assert err.max() < 3e-5, ("gemm", case, float(err.max()))
        if B == 1 or rng.random() < 0.3:
            outs = t12.gemv(dts, to_dev_bits(X[:1]).reshape(-1))
            torch.cuda.synchronize()
            for p, o, aw in zip(packs, outs, absw):
                err = np.abs(o.cpu().numpy().astype(np.float64) - oracle.gemm(p, X[:1])[0]) / ((Xf[:1] @ aw.T)[0] + 1e-30)
                assert err.max() < 3e-5, ("gemv", case, float(err.max()))
        done += 1


def test_random_pack_and_decompress(t12, oracle, synth):
    """GPU packer == oracle packer byte for byte; patched decode == the original bits; unpatched decode == the oracle's."""
    rng = np.random.default_rng(20242)
    for _ in range(400):
        M = int(rng.choice([1, 2, 3, 7, 16, 33, 100, 128, 255, 600]))
        K = int(rng.choice([1, 2, 3, 15, 16, 17, 63, 64, 65, 127, 128, 1000, 1024, 1025, 3000]))
        law = int(rng.integers(0, 5))
        seed = int(rng.integers(0, 1 << 30))
        if law == 0:
            w = synth.weights_llm(M, K, seed=seed, p_outlier=float(rng.choice([0, 3e-4, 0.05, 0.5])))
        elif law == 1:
            w = synth.weights_diffusion(M, K, seed=seed)
        elif law == 2:
            w = rng.integers(0, 65536, size=(M, K)).astype(np.uint16)          # every pattern, NaN / Inf included
        elif law == 3:
            w = np.zeros((M, K), np.uint16)
        else:
            w = synth.weights_llm(M, K, seed=seed, sigma=float(rng.choice([1e-30, 1e-3, 1.0, 1e30])))
        be = None if rng.random() < 0.6 else int(rng.choice([-1, 0, 1, 50, 100, 110, 127, 200, 239, 240]))
        case = (M, K, law, seed, be)
        wd = to_dev_bits(w).reshape(w.shape)
        if be is None:
            assert t12.find_base_exp_device(wd) == oracle.find_base_exp(w), case
        d = t12.pack_device(wd, be)
        p = oracle.pack(w, be)
        torch.cuda.synchronize()
        assert d.base_exp == p.base_exp, case
        for f in ("sm", "gr", "row_off", "cols", "correct", "wrong"):
            assert np.array_equal(getattr(d, f).cpu().numpy(), getattr(p, f)), (case, f)
        out = t12.decompress(d, patched=True)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint16).reshape(M, K), w), case
        out = t12.decompress(d, patched=False)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint16).reshape(-1), oracle.decode(p, patched=False).reshape(-1)), case


def test_random_moe_layers(t12, oracle, synth, moe):
    """Expert counts 1..64, widths that take the tile kernel, the few-row kernel or the host-counted path, even and skewed
    routings, int32 and int64 ids.  Mild outliers (0.3 against sigma 0.02) and 2e-3: the activation between the two
    projections is rounded to bf16, and where the GPU's fp32 sum falls on the other side of a rounding boundary than the
    oracle's, one of 48..320 terms moves by a bf16 step."""
    rng = np.random.default_rng(20243)
    for _ in range(120):
        E = int(rng.choice([1, 2, 3, 4, 8, 9, 16, 17, 33, 64]))
        n = int(rng.choice([64, 128, 192, 256, 96, 80]))
        n_ff = int(rng.choice([64, 128, 256, 320, 160, 48]))
        k = int(rng.integers(1, min(E, 4) + 1))
        T = int(rng.choice([1, 2, 3, 4, 5, 8, 16, 17, 40, 70, 130, 200, 300]))
        skew = rng.random() < 0.4
        seed = int(rng.integers(0, 1 << 30))
        case = (E, n, n_ff, T, k, skew, seed)
        packs = [[oracle.pack(synth.weights_llm(m, kk, seed=seed + 3 * e + j, p_outlier=float(rng.choice([0, 1e-3, 2e-2])),
                                                sigma_outlier=0.3))
                  for j, (m, kk) in enumerate([(n_ff, n), (n_ff, n), (n, n_ff)])] for e in range(E)]
        layer = moe.MoeLayer([moe.Expert(*[t12.DeviceTensor12.from_packed(p, dev()) for p in ps]) for ps in packs])
        pw = None
        if skew:
            pw = rng.random(E) ** 4 + 1e-3
            pw /= pw.sum()
        ids_h = np.stack([rng.choice(E, size=k, replace=False, p=pw) for _ in range(T)]).astype(np.int32)
        ids_t = torch.from_numpy(ids_h.astype(np.int64) if rng.random() < 0.5 else ids_h).to(dev())
        X = synth.activations(T, n, seed=seed + 1)
        w_h = rng.random((T, k)).astype(np.float32)
        got = layer(to_dev_bits(X).reshape(T, n), ids_t, torch.from_numpy(w_h).to(dev())).cpu().numpy()
        layer.status()
        ref = np.zeros((T, n), np.float64)
        for e in range(E):
            rows, slots = np.nonzero(ids_h == e)
            if len(rows) == 0:
                continue
            a = oracle.silu_mul_bf16(oracle.gemm(packs[e][0], X[rows]), oracle.gemm(packs[e][1], X[rows]))
            ref[rows] += w_h[rows, slots][:, None].astype(np.float64) * oracle.gemm(packs[e][2], a)
        assert rel_err(got, ref) < 2e-3, case


def test_random_model_configurations(t12, oracle, synth):
    """Engine logits against the CPU decode step over head_dim 32 / 64 / 128, GQA ratios 1 / 2 / 4 / 8, 1-3 layers, batches of
    2 / 5 / 17 lock-step rows, fused and TURBO_NO_FUSE.  Weights without the heavy outliers of the other tests (3e-4 at 0.3):
    with them a 3-layer model of these widths turns one bf16 step of an attention output into tens of percent of a logit,
    and the INT8 form of the attention is allowed such a step."""
    modelio = importlib.import_module(t12.__name__ + ".modelio")
    rng = np.random.default_rng(20244)
    old_ctx = os.environ.get("TURBO_CTX")
    os.environ["TURBO_CTX"] = "64"
    done = 0
    try:
        while done < 24:
            hd = int(rng.choice([32, 64, 128]))
            nkv = int(rng.choice([1, 2, 4]))
            nh = nkv * int(rng.choice([1, 2, 4, 8]))
            if nh * hd > 1024:
                continue
            cfg = dict(n_vocab=int(rng.choice([64, 300, 1024])), n_embd=nh * hd, n_head=nh, n_head_kv=nkv,
                       n_layer=int(rng.integers(1, 4)), n_ff=int(rng.choice([192, 512, 1024])), n_ctx=64,
                       rope_theta=float(rng.choice([10000.0, 500000.0])), rms_norm_eps=1e-5)
            seed = int(rng.integers(0, 1 << 20))
            B = int(rng.choice([1, 2, 5, 17]))
            nofuse = rng.random() < 0.3
            n, ff, kv = cfg["n_embd"], cfg["n_ff"], nkv * hd
            wr = np.random.default_rng(seed)
            cnt = [seed]

            def mk(M, K):
                cnt[0] += 1
                return oracle.pack(synth.weights_llm(M, K, cnt[0], p_outlier=3e-4, sigma_outlier=0.3))
            layers = [dict(attn_norm=(1 + 0.05 * wr.standard_normal(n)).astype(np.float32),
                           ffn_norm=(1 + 0.05 * wr.standard_normal(n)).astype(np.float32),
                           wq=mk(n, n), wk=mk(kv, n), wv=mk(kv, n), wo=mk(n, n), w_gate=mk(ff, n), w_up=mk(ff, n),
                           w_down=mk(n, ff)) for _ in range(cfg["n_layer"])]
            embd = synth.weights_llm(cfg["n_vocab"], n, seed + 999, sigma=1.0, p_outlier=0)
            onorm = (1 + 0.05 * wr.standard_normal(n)).astype(np.float32)
            head = mk(cfg["n_vocab"], n)
            path = tempfile.mkdtemp()
            try:
                modelio.write_model_dir(path, cfg, embd, onorm, head, layers)
                ref = oracle.RefModel(cfg, embd, onorm, head, layers, max_seq=64)
                if nofuse:
                    os.environ["TURBO_NO_FUSE"] = "1"
                try:
                    eng = t12.Engine.load(path, batch=B)
                finally:
                    os.environ.pop("TURBO_NO_FUSE", None)
                try:
                    toks = [int(t) for t in np.random.default_rng(seed + 5).integers(3, cfg["n_vocab"], size=6)]
                    for pos, tok in enumerate(toks):
                        eng.forward([tok] * B)
                        got = eng.logits(cfg["n_vocab"]).cpu().numpy()
                        want = ref.step(tok, pos)
                        assert np.array_equal(got, np.broadcast_to(got[0], got.shape)), (cfg, seed, B, pos)
                        err = np.abs(got[0] - want).max() / np.abs(want).max()
                        assert err < 2e-2, (cfg, seed, B, nofuse, pos, float(err))
                finally:
                    eng.close()
            finally:
                shutil.rmtree(path, ignore_errors=True)
            done += 1
    finally:
        if old_ctx is None:
            os.environ.pop("TURBO_CTX", None)
        else:
            os.environ["TURBO_CTX"] = old_ctx
