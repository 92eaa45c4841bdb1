"""Committed vectors (tests/golden/hotpath_small.npz, written by tests/golden/make_fixtures.py).

CPU: the NumPy oracle and the independent C restatement both reproduce them.  GPU: the HIP library does."""
import os

import numpy as np
import pytest
import torch

from oracle import decdec_oracle as O
from tests.helpers import rel_err

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hotpath_small.npz")
TOL = 1e-2


@pytest.fixture(scope="module")
def gold():
    return dict(np.load(PATH, allow_pickle=False))


def test_numpy_oracle_reproduces_fixtures(gold):
    g = gold
    kc, K = int(g["dec_k_chunk"]), int(g["dec_K"])
    k = kc * K // 1024
    assert np.array_equal(O.bucket_floors(g["dec_thresholds"][0], g["dec_thresholds"][k - 1], "fp16"), g["dec_floors"])
    rows, acts, filled = O.select_channels(g["dec_x"], g["dec_thresholds"], kc, "fp16")
    assert np.array_equal(rows, g["dec_rows"]) and np.array_equal(filled, g["dec_filled"])
    assert np.array_equal(acts, g["dec_acts"])
    np.testing.assert_allclose(O.dec_apply(g["dec_x"], g["dec_cheat"], g["dec_scales"], rows[filled]), g["dec_out"], rtol=1e-12)
    np.testing.assert_allclose(O.anyprec_gemv(g["dec_x"], g["ap3_qweight"], g["ap3_lut"], 3), g["ap3_out"], rtol=1e-12)
    np.testing.assert_allclose(O.anyprec_gemv(g["dec_x"], g["ap5_qweight"], g["ap5_lut"], 5), g["ap5_out"], rtol=1e-12)
    np.testing.assert_allclose(O.lutgemm_gemv(g["lg_x"], g["lg_qweight"], g["lg_alpha"], g["lg_qbias"], 128), g["lg_out"], rtol=1e-12)
    for bits in (4, 3):
        np.testing.assert_allclose(O.sqllm_gemv(g["lg_x"], g[f"sq{bits}_mat"], g[f"sq{bits}_lut"], bits), g[f"sq{bits}_out"], rtol=1e-12)


def test_c_oracle_reproduces_fixtures(gold, c_oracle):
    g = gold
    kc, K = int(g["dec_k_chunk"]), int(g["dec_K"])
    k = kc * K // 1024
    assert np.array_equal(c_oracle.bucket_floors(g["dec_thresholds"][0], g["dec_thresholds"][k - 1], "fp16"), g["dec_floors"])
    rows, acts = c_oracle.select(g["dec_x"], g["dec_thresholds"], kc, "fp16")
    assert np.array_equal(rows, g["dec_rows"])
    filled = g["dec_filled"]
    assert np.array_equal(acts.view(np.float16)[filled].astype(np.float32), g["dec_acts"][filled])
    # the C restatement accumulates in double in its own order: equal up to float64 rounding
    np.testing.assert_allclose(c_oracle.dec_apply(g["dec_x"], g["dec_cheat"], g["dec_scales"], rows[filled]), g["dec_out"], rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(c_oracle.anyprec_gemv(g["dec_x"], g["ap3_qweight"], g["ap3_lut"], 3), g["ap3_out"], rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(c_oracle.anyprec_gemv(g["dec_x"], g["ap5_qweight"], g["ap5_lut"], 5), g["ap5_out"], rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(c_oracle.lutgemm_gemv(g["lg_x"], g["lg_qweight"], g["lg_alpha"], g["lg_qbias"], 3, 128), g["lg_out"], rtol=1e-9, atol=1e-12)
    for bits in (4, 3):
        np.testing.assert_allclose(c_oracle.sqllm_gemv(g["lg_x"], g[f"sq{bits}_mat"], g[f"sq{bits}_lut"], bits), g[f"sq{bits}_out"], rtol=1e-9, atol=1e-12)


@pytest.mark.gpu
def test_hip_library_reproduces_fixtures(gold):
    from decdec_amd import ext
    g = gold
    dev = "cuda"
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    kc, K, N = int(g["dec_k_chunk"]), int(g["dec_K"]), int(g["dec_N"])
    x = t(g["dec_x"]).view(1, 1, K).to(dev)
    rows = torch.full((K,), -1, dtype=torch.int32, device=dev)
    acts = torch.zeros(K, dtype=torch.float16, device=dev)
    th = t(g["dec_thresholds"])
    ctx = ext.create_dec_context(8, rows, acts)
    cfg = ext.create_dec_config(ctx, kc, t(g["dec_cheat"]), t(g["dec_scales"]), th)
    out = torch.zeros(1, 1, N, dtype=torch.float16, device=dev)
    ext.dec(cfg, x, out)
    torch.cuda.synchronize()
    n = g["dec_rows"].shape[0]
    filled = g["dec_filled"]
    assert np.array_equal(rows[:n].cpu().numpy()[filled], g["dec_rows"][filled]), "selected rows must be bit-exact"
    assert np.array_equal(acts[:n].cpu().numpy()[filled].astype(np.float32), g["dec_acts"][filled])
    assert rel_err(out.cpu().numpy().reshape(-1), g["dec_out"])[0] <= TOL
    ext.destroy_dec_config(cfg)
    ext.destroy_dec_context(ctx)

    def gemv(fn, n_out, want):
        o = torch.zeros(1, 1, n_out, dtype=torch.float16, device=dev)
        fn(o)
        torch.cuda.synchronize()
        mre, mae = rel_err(o.cpu().numpy().reshape(-1), want)
        assert mre <= TOL, (mre, mae)

    gemv(lambda o: ext.anyprec_gemv(x, o, t(g["ap3_qweight"]).to(dev), t(g["ap3_lut"]).to(dev), 3), N, g["ap3_out"])
    gemv(lambda o: ext.anyprec_gemv(x, o, t(g["ap5_qweight"]).to(dev), t(g["ap5_lut"]).to(dev), 5), 32, g["ap5_out"])
    xl = t(g["lg_x"]).view(1, 1, -1).to(dev)
    gemv(lambda o: ext.lutgemm_gemv(xl, o, t(g["lg_qweight"]).to(dev), t(g["lg_alpha"]).to(dev), t(g["lg_qbias"]).to(dev), 3, 128),
         g["lg_out"].shape[0], g["lg_out"])
    for bits in (4, 3):
        gemv(lambda o: ext.sqllm_gemv(xl, o, t(g[f"sq{bits}_mat"]).to(dev), t(g[f"sq{bits}_lut"]).to(dev), bits),
             g[f"sq{bits}_out"].shape[0], g[f"sq{bits}_out"])
