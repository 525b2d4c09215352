"""Writes input/output vectors of the reference's fp32 quantiser for tests/golden/fp32_reference.npz.

Runs ONLY in the development container, where the reference checkout exists: it imports the
reference's own ``ADKVTrainModel`` (src/adkv/train/train_model.py, pure torch) and records what its
``forward(..., output_states=True)`` returns on seeded inputs, i.e. the outputs of the
``torch.compile``d ``_adkv_chunk_forward`` on the CPU.  The one property nothing else can pin is
whether that compiled function is bit-identical to an operation-by-operation fp32 evaluation; the
vectors settle it.  The tests only read the .npz.

    python tests/golden/make_fp32_reference_vectors.py [/root/reference]
"""
import os
import sys

import numpy as np
import torch


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sys.path.insert(0, os.path.join(ref, "src"))
    from adkv.train.train_model import ADKVTrainModel  # the reference's module

    out = {}
    cases = [("a", 4, 2, 70, 96, 11), ("b", 2, 1, 257, 64, 12), ("c", 8, 1, 40, 32, 13)]
    for tag, bits, B, T, C, seed in cases:
        torch.manual_seed(seed)
        m = ADKVTrainModel(C, truncation=32, bits=bits)
        with torch.no_grad():
            m.init_zp.normal_(0.0, 0.3)
            m.init_log_sc.normal_(0.0, 0.3)
            m.alpha.normal_(2.0, 1.0)
            m.beta.normal_(0.0, 1.5)
            m.target.fill_(m.upper_limit / 2)
        x = torch.randn(B, T, C) * 2.0
        x[:, :, ::9] += 5.0 * torch.sin(0.05 * torch.arange(T, dtype=torch.float32))[None, :, None]
        with torch.no_grad():
            xhat, zp_seq, sc_seq = m(x, output_states=True)
        out.update({
            f"{tag}_bits": np.int32(bits), f"{tag}_x": x.numpy(),
            f"{tag}_zp0": m.init_zp.detach().numpy(), f"{tag}_sc0": m.get_sc().detach().numpy(),
            f"{tag}_alpha": m.get_alpha().detach().numpy(), f"{tag}_beta": m.get_beta().detach().numpy(),
            f"{tag}_tgt": m.target.detach().numpy(),
            f"{tag}_sc_min": np.float32(m.sc_min), f"{tag}_sc_max": np.float32(m.sc_max),
            f"{tag}_xhat": xhat.numpy(), f"{tag}_zp_seq": zp_seq.numpy(), f"{tag}_sc_seq": sc_seq.numpy(),
        })
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fp32_reference.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes; torch", torch.__version__)


if __name__ == "__main__":
    main()
