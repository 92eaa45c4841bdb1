"""Writes tests/golden/hotpath_small.npz: small, fixed inputs of the hot path and the oracle's outputs.

The reference's own tests hold no golden vectors for this path (they are input recipes), and the
reference cannot run here, so these vectors come from the NumPy oracle (oracle/decdec_oracle.py).  They
freeze its behaviour: the CPU suite checks that the NumPy and the independent C restatement both still
reproduce them, the GPU suite checks the HIP library against them.  Regenerate with
    python tests/golden/make_fixtures.py
only when the oracle is deliberately changed.
"""
from __future__ import annotations

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from decdec_amd import formats as F          # noqa: E402
from oracle import decdec_oracle as O        # noqa: E402


def main(path):
    g = torch.Generator().manual_seed(20240607)
    out = {}
    # --- DEC: ragged K (2 full chunks + a 512-channel tail), k_chunk 16
    K, N, kc = 2560, 64, 16
    W = (torch.randn(N, K, generator=g) * 0.02).half()
    idx, lut = F.quantize_uniform_rows(W, 3)
    q, s = F.quantize_residual((W.float() - F.dequant_lut(idx, lut).float()).half())
    cheat, scales = F.pack_residual(q, s)
    x = F.make_activation(K, g)
    th = F.calibrate_thresholds(K, g, draws=16)
    xn, thn = x.numpy().reshape(-1), th.numpy()
    k = kc * K // 1024
    rows, acts, filled = O.select_channels(xn, thn, kc, "fp16")
    out.update(dec_K=K, dec_N=N, dec_k_chunk=kc, dec_x=xn, dec_thresholds=thn,
               dec_floors=O.bucket_floors(float(thn[0]), float(thn[k - 1]), "fp16"),
               dec_rows=rows, dec_acts=acts, dec_filled=filled,
               dec_cheat=cheat.numpy(), dec_scales=scales.half().numpy(),
               dec_out=O.dec_apply(xn, cheat.numpy(), scales.half().numpy(), rows[filled]))
    # --- any-precision 3-bit and 5-bit GEMV on the same activations (first 1024 + tail mapping)
    qw3 = F.pack_anyprec(idx, 3).numpy()
    out.update(ap3_qweight=qw3, ap3_lut=lut.numpy(), ap3_out=O.anyprec_gemv(xn, qw3, lut.numpy(), 3))
    idx5 = torch.randint(0, 32, (32, K), generator=g, dtype=torch.int64)
    lut5 = (torch.randn(32, 32, generator=g) * 0.02).half()
    qw5 = F.pack_anyprec(idx5, 5).numpy()
    out.update(ap5_qweight=qw5, ap5_lut=lut5.numpy(), ap5_out=O.anyprec_gemv(xn, qw5, lut5.numpy(), 5))
    # --- LUT-GEMM 3-bit, group 128
    Kl, Nl = 1024, 66
    Wl = (torch.randn(Nl, Kl, generator=g) * 0.02).half()
    ql, sl, zl = F.awq_pseudo_quantize(Wl, 3, 128)
    qwl, alpha, qbias = F.pack_bcq(ql, sl, zl, 3, torch.float16)
    xl = F.make_activation(Kl, g).numpy().reshape(-1)
    out.update(lg_x=xl, lg_qweight=qwl.numpy(), lg_alpha=alpha.numpy(), lg_qbias=qbias.numpy(),
               lg_out=O.lutgemm_gemv(xl, qwl.numpy(), alpha.numpy(), qbias.numpy(), 128))
    # --- SqueezeLLM 4-bit and 3-bit
    for bits in (4, 3):
        idxs = torch.randint(0, 1 << bits, (Nl, Kl), generator=g, dtype=torch.int64)
        luts = (torch.randn(Nl, 1 << bits, generator=g) * 0.02).half()
        mat = F.pack_sqllm(idxs, bits).numpy()
        out.update({f"sq{bits}_mat": mat, f"sq{bits}_lut": luts.numpy(),
                    f"sq{bits}_out": O.sqllm_gemv(xl, mat, luts.numpy(), bits)})
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main(os.path.join(os.path.dirname(os.path.abspath(__file__)), "hotpath_small.npz"))
