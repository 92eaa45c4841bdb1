"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Bar: selected channel indices bit-exact; outputs within max relative error 1e-2 of the float64
oracle (denominator floored at 1 % of max|y| so near-zero outputs do not dominate).
"""
import numpy as np
import pytest
import torch

from decdec_amd import ext, formats as F
from oracle import decdec_oracle as O
from tests.helpers import TORCH_DT, make_dec_layer, np_of, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _ctx(n_tb, K, dtype):
    rows = torch.full((K,), -7, dtype=torch.int32, device="cuda")
    acts = torch.zeros(K, dtype=dtype, device="cuda")
    return ext.create_dec_context(n_tb, rows, acts), rows, acts


@pytest.mark.parametrize("K,N,k_chunk,n_tb", [
    (4096, 4096, 32, 8), (4096, 1024, 32, 8), (14336, 4096, 20, 24), (4096, 14336, 8, 16),
    (5120, 5120, 64, 32), (17920, 5120, 32, 8), (1024, 256, 16, 1), (2048 + 512, 64, 32, 4),
])
@pytest.mark.parametrize("dt", ["fp16"])
def test_dec_selection_and_output(K, N, k_chunk, n_tb, dt, c_oracle):
    dtype = TORCH_DT[dt]
    L = make_dec_layer(K, N, seed=K + N + k_chunk, dtype=dtype)
    ctx, rows, acts = _ctx(n_tb, K, dtype)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=dtype, device="cuda")
    ext.dec(cfg, x, out)
    torch.cuda.synchronize()
    want_rows, want_acts, filled = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk, dt)
    k = k_chunk * K // 1024
    got_rows = rows.cpu().numpy()
    assert np.array_equal(got_rows[:k], want_rows[:k]), "selected channel indices differ from the oracle"
    assert np.array_equal(np_of(acts)[:k], want_acts[:k].astype(np_of(acts).dtype))
    assert (got_rows[k:] == -7).all(), "wrote past the k selected entries"
    want = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows, dt)
    mre, mae = rel_err(np_of(out).reshape(-1), want)
    assert mre <= TOL, (mre, mae)
    ext.destroy_dec_config(cfg)
    ext.destroy_dec_context(ctx)


@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 1024), (14336, 4096), (5120, 7680), (17920, 5120), (1024, 64)])
def test_anyprec_gemv_3bit(K, N, c_oracle):
    L = make_dec_layer(K, N, seed=K * 3 + N)
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.anyprec_gemv(x, out, L["qweight"].cuda(), L["lut"].cuda(), 3)
    torch.cuda.synchronize()
    want = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
    mre, mae = rel_err(np_of(out).reshape(-1), want)
    assert mre <= TOL, (mre, mae)


def test_dec_anyprec_fused_matches_sum(c_oracle):
    K, N, k_chunk = 4096, 4096, 32
    L = make_dec_layer(K, N, seed=11)
    ctx, rows, acts = _ctx(8, K, torch.float16)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dec_anyprec(cfg, x, out, L["qweight"].cuda(), L["lut"].cuda(), 3)
    torch.cuda.synchronize()
    want_rows, _, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk)
    assert np.array_equal(rows.cpu().numpy()[:128], want_rows[:128])
    want = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3) + \
        c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    mre, mae = rel_err(np_of(out).reshape(-1), want)
    assert mre <= TOL, (mre, mae)
    # the DEC-compensated output must be closer to the unquantised layer than the base GEMV alone
    exact = L["W"].double().numpy() @ np_of(L["x"]).astype(np.float64).reshape(-1)
    base = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
    assert np.abs(np_of(out).reshape(-1) - exact).mean() < np.abs(base - exact).mean()
