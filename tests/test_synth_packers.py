"""The torch packers that make synthetic weights for the benchmark produce valid GGUF blocks: the oracle
dequantizes them back to within one quantization step of the source (CPU tensors here; same code runs on GPU)."""
import importlib

import numpy as np
import pytest
import torch

from helpers import oracle_lib as O

synth = importlib.import_module("neural-api_amd.synth")


@pytest.mark.parametrize("qt,packer", [(O.Q8_0, "pack_q8_0"), (O.Q4_0, "pack_q4_0"), (O.Q4_K, "pack_q4_k"), (O.Q6_K, "pack_q6_k")])
def test_torch_packer_roundtrip(qt, packer):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(16, 1024, generator=g) * 0.02
    raw = getattr(synth, packer)(x).reshape(-1).numpy()
    assert raw.size == 16 * O.row_bytes(qt, 1024)
    y = O.dequant(qt, raw, x.numel()).reshape(16, 1024)
    grp = 16 if qt == O.Q6_K else 32
    xb = x.numpy().reshape(-1, grp)
    step = {O.Q8_0: np.abs(xb).max(1) / 127, O.Q4_0: np.abs(xb).max(1) / 8, O.Q4_K: (xb.max(1) - np.minimum(xb.min(1), 0)) / 15,
            O.Q6_K: np.abs(xb).max(1) / 31}[qt]
    err = np.abs(x.numpy() - y).reshape(-1, grp).max(1)
    assert np.all(err <= 1.3 * step + 1e-6)
    if qt == O.Q8_0:  # same recipe as the reference writer -> identical bytes to the C packer
        assert np.array_equal(raw, O.quantize(O.Q8_0, x.numpy()))
