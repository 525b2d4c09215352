"""The PyTorch-CPU baseline (oracle/torch_cpu.py, what bench.py's cpu_baseline leg times) computes
the same values as the C oracle's fp32 recurrence, which is itself held to vectors recorded from
the reference's own module (tests/test_golden_fp32_reference.py)."""
import os

import numpy as np
import pytest
import torch

from oracle import torch_cpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "fp32_reference.npz")


@pytest.mark.parametrize("bits,B,T,C", [(4, 2, 70, 96), (2, 1, 33, 64), (8, 3, 40, 32)])
def test_torch_cpu_recurrence_equals_c_oracle(oracle, bits, B, T, C):
    g = torch.Generator().manual_seed(bits * 100 + T)
    x = torch.randn(B, T, C, generator=g) * 1.5
    x[:, :, 0] += 6.0 * torch.sin(0.05 * torch.arange(T))[None]
    zp0 = 0.1 * torch.randn(C, generator=g)
    sc0 = 0.5 + torch.rand(C, generator=g)
    alpha = 0.9 + 0.099 * torch.rand(C, generator=g)
    beta = 0.05 * torch.rand(C, generator=g)
    tgt = torch.full((C,), (2 ** (bits - 1) - 1) / 2.0)
    out, zp, sc, codes = torch_cpu.quant_stream_f32(x, zp0, sc0, alpha, beta, tgt, bits=bits, want_codes=True)
    want = oracle.quant_f32(x.numpy(), zp0.numpy(), sc0.numpy(), alpha.numpy(), beta.numpy(), tgt.numpy(),
                            bits=bits)
    assert np.array_equal(codes.numpy(), want["codes"])
    assert np.array_equal(out.numpy().view(np.int32), want["xhat"].view(np.int32))
    assert np.array_equal(zp.numpy().view(np.int32), want["zp"].view(np.int32))
    assert np.array_equal(sc.numpy().view(np.int32), want["sc"].view(np.int32))


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_torch_cpu_recurrence_reproduces_reference_vectors(tag):
    """The vectors recorded from the reference's ADKVTrainModel (inputs, dequantised outputs)."""
    z = np.load(GOLDEN)
    g = lambda k: torch.from_numpy(np.ascontiguousarray(z[f"{tag}_{k}"]))
    out, _, _, _ = torch_cpu.quant_stream_f32(g("x"), g("zp0"), g("sc0"), g("alpha"), g("beta"), g("tgt"),
                                              bits=int(z[f"{tag}_bits"]), sc_min=float(z[f"{tag}_sc_min"]),
                                              sc_max=float(z[f"{tag}_sc_max"]))
    assert np.array_equal(out.numpy().view(np.int32), z[f"{tag}_xhat"].view(np.int32))


def test_torch_cpu_attention_matches_f64(oracle):
    B, H, T, D = 2, 3, 50, 16
    g = torch.Generator().manual_seed(4)
    q = torch.randn(B, H * D, generator=g)
    k = torch.randn(B, T, H * D, generator=g)
    v = torch.randn(B, T, H * D, generator=g)
    got = torch_cpu.single_query_attention(q, k, v, H, D ** -0.5).view(B, H, D).numpy()
    K = k.view(B, T, H, D).transpose(1, 2).contiguous().numpy()
    V = v.view(B, T, H, D).transpose(1, 2).contiguous().numpy()
    want, _ = oracle.attention_f64(q.view(B, H, D).numpy(), K, V, D ** -0.5)
    assert np.max(np.abs(got - want)) < 1e-5
