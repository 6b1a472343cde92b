"""GPU parity: standalone decompress through the C ABI -- bit-exact."""
import importlib

import numpy as np
import pytest
import torch

from gpu_util import dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def synth(t12):
    return importlib.import_module("turbo_lossless_amd.synth")


def roundtrip(t12, oracle, w, base_exp=None):
    p = oracle.pack(w, base_exp)
    dt = t12.DeviceTensor12.from_packed(p, dev())
    pat = t12.decompress(dt, patched=True)
    un = t12.decompress(dt, patched=False)
    torch.cuda.synchronize()
    assert np.array_equal(pat.cpu().numpy().view(np.uint16), w), "patched decode must equal the packed tensor"
    assert np.array_equal(un.cpu().numpy().view(np.uint16), oracle.decode(p, patched=False))
    return p


def test_golden_cases_bit_exact(t12, oracle, golden):
    for name, g in golden.items():
        roundtrip(t12, oracle, g["w"], int(g["base_exp"]))


@pytest.mark.parametrize("M,K", [(4096, 4096), (1280, 5120), (5120, 1280), (333, 1001), (1, 15), (7, 17)])
def test_shapes_bit_exact(t12, oracle, synth, M, K):
    gen = synth.weights_diffusion if K in (5120, 1280) else synth.weights_llm
    p = roundtrip(t12, oracle, gen(M, K, seed=M + K))
    if M * K > 1e6:
        assert p.P > 0


def test_all_bf16_patterns(t12, oracle):
    """Every one of the 65536 bf16 bit patterns survives pack -> GPU decompress."""
    w = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    roundtrip(t12, oracle, w)
    roundtrip(t12, oracle, w, base_exp=-1)
    roundtrip(t12, oracle, w, base_exp=240)


def test_full_size_idempotent_checksum(t12, oracle, synth):
    """Llama gate shape 14336 x 4096: decode on GPU, compare whole tensor on the host."""
    w = synth.weights_llm(14336, 4096, seed=2001)
    roundtrip(t12, oracle, w)


def test_empty_and_errors(t12):
    z = torch.zeros(16, dtype=torch.uint8, device=dev())
    assert t12.lib.t12_decompress(z.data_ptr(), z.data_ptr(), 100, None, None, None, z.data_ptr(), 0, 16, 0, None) == 0
    assert t12.lib.t12_decompress(None, z.data_ptr(), 100, None, None, None, z.data_ptr(), 1, 16, 0, None) == -1
    assert t12.lib.t12_decompress(z.data_ptr(), z.data_ptr(), 300, None, None, None, z.data_ptr(), 1, 16, 0, None) == -1
