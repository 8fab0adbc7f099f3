"""The torch synthetic-weight encoders produce valid GGUF blocks (checked with the CPU oracle)."""
import numpy as np
import pytest
import torch

from magnitude_amd import synth

Q8_0, Q4_K, Q6_K = 8, 12, 14


@pytest.mark.parametrize("qtype,tol", [(Q8_0, 0.01), (Q4_K, 0.09), (Q6_K, 0.025)])
def test_synth_blocks_dequantize_close_to_input(orc, qtype, tol):
    g = torch.Generator().manual_seed(3)
    w = torch.randn((16, 1024), generator=g) * 0.02
    w[2, 256:512] = 0.0
    blocks = synth.quantize(qtype, w).numpy()
    assert blocks.shape == (16, orc.row_bytes(qtype, 1024))
    y = orc.dequantize(qtype, blocks, 1024)
    rel = np.linalg.norm(y - w.numpy()) / np.linalg.norm(w.numpy())
    assert rel < tol, rel
    assert not y[2, 256:512].any()


def test_synth_q8_0_is_the_spec_quantizer(orc):
    g = torch.Generator().manual_seed(4)
    w = torch.randn((8, 4096), generator=g) * 0.02
    assert np.array_equal(synth.quantize_q8_0(w).numpy(), orc.quantize(Q8_0, w.numpy()))


def test_random_weight_is_deterministic():
    a = synth.random_weight(Q4_K, 8, 512, seed=5, device="cpu")
    b = synth.random_weight(Q4_K, 8, 512, seed=5, device="cpu")
    assert torch.equal(a, b) and a.shape == (8, 2 * 144)
