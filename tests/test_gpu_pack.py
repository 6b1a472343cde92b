"""GPU parity: the GPU-side packer emits byte-identical arrays to the oracle's
(reference-pinned) packer."""
import importlib

import numpy as np
import pytest
import torch

from gpu_util import to_dev_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def synth(t12):
    return importlib.import_module("turbo_lossless_amd.synth")


def check_same(t12, oracle, w, base_exp=None):
    wd = to_dev_bits(w).reshape(w.shape)
    if base_exp is None:
        assert t12.find_base_exp_device(wd) == oracle.find_base_exp(w)
    d = t12.pack_device(wd, base_exp)
    p = oracle.pack(w, base_exp)
    torch.cuda.synchronize()
    assert d.base_exp == p.base_exp
    for f in ("sm", "gr", "row_off", "cols", "correct", "wrong"):
        assert np.array_equal(getattr(d, f).cpu().numpy(), getattr(p, f)), f
    return d, p


def test_golden_cases(t12, oracle, golden):
    for name, g in golden.items():
        forced = int(g["base_exp"]) if int(g["base_exp"]) != int(g["found_base_exp"]) else None
        check_same(t12, oracle, g["w"], forced)


@pytest.mark.parametrize("M,K", [(4096, 4096), (1280, 5120), (333, 1001), (1, 15), (7, 17), (128256 // 8, 4096)])
def test_shapes(t12, oracle, synth, M, K):
    gen = synth.weights_diffusion if K == 5120 else synth.weights_llm
    d, p = check_same(t12, oracle, gen(M, K, seed=M * 7 + K))
    # and the packed tensor decodes back on the GPU
    out = t12.decompress(d, patched=True)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), oracle.decode(p))


def test_all_patterns_and_forced_base(t12, oracle):
    w = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    for be in (None, -1, 0, 100, 127, 240):
        check_same(t12, oracle, w, be)
