"""The oracle's fp32 recurrence against vectors recorded from the reference's own module.

tests/golden/fp32_reference.npz holds inputs and outputs of the reference's ``ADKVTrainModel``
(src/adkv/train/train_model.py:89-213, i.e. its ``torch.compile``d ``_adkv_chunk_forward`` on the
CPU) for three seeded cases (4-, 2- and 8-bit ranges), written by
tests/golden/make_fp32_reference_vectors.py.  Bit-for-bit agreement pins the one thing the
closed-form checks cannot: that the compiled function evaluates the recurrence operation by
operation in fp32, as ``adkv_o_quant_f32`` and the GPU kernel do."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp32_reference.npz")
CASES = ("a", "b", "c")


def _case(z, tag):
    g = lambda k: z[f"{tag}_{k}"]
    return dict(bits=int(g("bits")), x=g("x"), zp0=g("zp0"), sc0=g("sc0"), alpha=g("alpha"), beta=g("beta"),
                tgt=g("tgt"), sc_min=float(g("sc_min")), sc_max=float(g("sc_max")),
                xhat=g("xhat"), zp_seq=g("zp_seq"), sc_seq=g("sc_seq"))


def _same_bits(a, b):
    return np.array_equal(np.ascontiguousarray(a, np.float32).view(np.int32),
                          np.ascontiguousarray(b, np.float32).view(np.int32))


@pytest.mark.parametrize("tag", CASES)
def test_oracle_matches_reference_vectors(oracle, tag):
    c = _case(np.load(GOLDEN), tag)
    got = oracle.quant_f32(c["x"], c["zp0"], c["sc0"], c["alpha"], c["beta"], c["tgt"], bits=c["bits"],
                           sc_min=c["sc_min"], sc_max=c["sc_max"], want_seq=True)
    assert _same_bits(got["xhat"], c["xhat"])
    assert _same_bits(got["zp_seq"], c["zp_seq"])
    assert _same_bits(got["sc_seq"], c["sc_seq"])


@pytest.mark.gpu
@pytest.mark.parametrize("tag", CASES)
def test_gpu_matches_reference_vectors(gpu, tag):
    import torch
    from adkv_amd.train import quant_f32
    c = _case(np.load(GOLDEN), tag)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)
    lo, hi = -2 ** (c["bits"] - 1), 2 ** (c["bits"] - 1) - 1
    xhat, _, zs, ss = quant_f32(t(c["x"]), t(c["alpha"]), t(c["beta"]), t(c["tgt"]), lo, hi,
                                c["sc_min"], c["sc_max"], zp_init=t(c["zp0"]), sc_init=t(c["sc0"]),
                                output_states=True)
    torch.cuda.synchronize()
    assert _same_bits(xhat.cpu().numpy(), c["xhat"])
    assert _same_bits(zs.cpu().numpy(), c["zp_seq"])
    assert _same_bits(ss.cpu().numpy(), c["sc_seq"])
