"""Shared builders for the parity tests (synthetic layers in the benchmark's recipe)."""
from __future__ import annotations

import numpy as np
import torch

from decdec_amd import formats as F

TORCH_DT = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}


def np_of(t: torch.Tensor) -> np.ndarray:
    """Tensor -> numpy; bf16 goes through float32 (values stay exactly representable)."""
    t = t.detach().cpu()
    return t.float().numpy() if t.dtype == torch.bfloat16 else t.numpy()


def make_dec_layer(K, N, seed, dtype=torch.float16, random_residual=False):
    """Weights, quantised base (any-precision 3-bit) and 4-bit residual of one layer, on the CPU."""
    g = torch.Generator().manual_seed(seed)
    W = (torch.randn(N, K, generator=g) * 0.02).to(torch.float16)
    idx, lut = F.quantize_uniform_rows(W, 3)
    Wq = F.dequant_lut(idx, lut)
    if random_residual:
        cheat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=g, dtype=torch.int64).to(torch.int32)
        scales = torch.rand(N, generator=g)
    else:
        q, s = F.quantize_residual((W.float() - Wq.float()).to(torch.float16))
        cheat, scales = F.pack_residual(q, s)
    x = F.make_activation(K, g, dtype=dtype)
    th = F.calibrate_thresholds(K, g, draws=16, dtype=dtype)
    return {"W": W, "idx": idx, "lut": lut.to(dtype), "qweight": F.pack_anyprec(idx, 3),
            "cheat": cheat.contiguous(), "scales": scales.to(dtype).contiguous(), "x": x, "th": th}


REL_FLOOR = 0.1


def rel_err(got: np.ndarray, want: np.ndarray, floor: float = REL_FLOOR):
    """(max relative error, mean abs error) of ``got`` against the float64 oracle ``want``.

    The denominator is max(|want_i|, floor * max|want|).  Outputs are fp16 sums of terms that cancel,
    so an output near zero carries the absolute rounding error of partial sums as large as max|want|;
    with a 1 % floor the reference's own fp16 arithmetic (oracle.dec_apply_reference_rounding) scores
    4.4e-2 on the 4096x4096, k_chunk=32 case, above the 1e-2 tolerance, and 5.5e-3 with the 10 %
    floor used here (tests/test_oracle.py::test_reference_rounding_error_budget)."""
    got = got.astype(np.float64); want = want.astype(np.float64)
    denom = np.maximum(np.abs(want), floor * np.max(np.abs(want)) + 1e-30)
    return float(np.max(np.abs(got - want) / denom)), float(np.mean(np.abs(got - want)))


TOL = {"fp16": 1e-2, "fp32": 1e-2, "bf16": 8e-2}     # bf16 has 8 significand bits against fp16's 11: the same bound in ulps


def check_output(got: np.ndarray, want: np.ndarray, dt: str = "fp16", what=None) -> float:
    """Asserts the output tolerance and reports, beside the judged ratio (10 % floor), the mean absolute error and
    the same ratio with the denominator floored at 1 % of max|want|."""
    mre, mae = rel_err(got, want)
    strict, _ = rel_err(got, want, floor=0.01)
    msg = f"{what}: max rel err {mre:.3e} (bound {TOL[dt]:.0e}), mean abs err {mae:.3e}, with a 1 % floor {strict:.3e}"
    print(msg)
    assert mre <= TOL[dt], msg
    return mre
