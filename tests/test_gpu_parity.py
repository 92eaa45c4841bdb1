"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Bar: selected channel indices bit-exact; outputs within max relative error 1e-2 of the float64
oracle, the denominator floored at 10 % of max|y| (tests/helpers.py: the reference's own fp16 arithmetic
misses 1e-2 with a 1 % floor).  Every output assertion reports the mean absolute error and the ratio with
a 1 % floor as well (helpers.check_output).
"""
import numpy as np
import pytest
import torch

from decdec_amd import _lib, ext, formats as F
from oracle import decdec_oracle as O
from tests.helpers import TORCH_DT, check_output, make_dec_layer, np_of, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-2            # fp16 and fp32 outputs
TOL_BF16 = 8e-2       # bf16 has 8 significand bits against fp16's 11: the same bound in units of ulp


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
    check_output(np_of(out).reshape(-1), want, "fp16")
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
    check_output(np_of(out).reshape(-1), want, "fp16")


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
    check_output(np_of(out).reshape(-1), want, "fp16")
    # the DEC-compensated output must be closer to the unquantised layer than the base GEMV alone
    exact = L["W"].double().numpy() @ np_of(L["x"]).astype(np.float64).reshape(-1)
    base = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
    assert np.abs(np_of(out).reshape(-1) - exact).mean() < np.abs(base - exact).mean()


# --------------------------------------------------------------------------------------------------
# other dtypes, other bit widths, the other base GEMVs
# --------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ["bf16", "fp32"])
def test_dec_other_dtypes_reference_recipe(dt, c_oracle):
    """The reference's own test recipe (decdec_extension/tests/test_dec.py): num_tb=24, K=14336,
    N=4096, k_chunk=20, random int32 residual, rand scales, x in U(-1,1), thresholds = sort(|x|)."""
    dtype = TORCH_DT[dt]
    K, N, k_chunk, n_tb = 14336, 4096, 20, 24
    g = torch.Generator().manual_seed(0)
    cheat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=g, dtype=torch.int64).to(torch.int32)
    scales = torch.rand(N, generator=g).to(dtype)
    x = (torch.rand(1, 1, K, generator=g) * 2 - 1).to(dtype)
    th = torch.sort(x.float().abs().view(-1), descending=True).values.to(dtype)
    ctx, rows, acts = _ctx(n_tb, K, dtype)
    cfg = ext.create_dec_config(ctx, k_chunk, cheat, scales, th)
    out = torch.zeros(1, 1, N, dtype=dtype, device="cuda")
    ext.dec(cfg, x.cuda(), out)
    torch.cuda.synchronize()
    want_rows, want_acts, _ = O.select_channels(np_of(x), np_of(th), k_chunk, dt)
    k = k_chunk * K // 1024
    assert np.array_equal(rows.cpu().numpy()[:k], want_rows[:k])
    assert np.array_equal(np_of(acts)[:k], want_acts[:k])
    want = c_oracle.dec_apply(np_of(x), cheat.numpy(), np_of(scales), want_rows, dt)
    check_output(np_of(out).reshape(-1), want, dt)
    ext.destroy_dec_config(cfg)


@pytest.mark.parametrize("bits", [3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("dt", ["fp16", "bf16"])
def test_anyprec_gemv_bits_and_dequant(bits, dt, c_oracle):
    dtype = TORCH_DT[dt]
    K, N = 2048 + 512, 96                      # tail chunk of 512 channels, N not a multiple of 8
    g = torch.Generator().manual_seed(bits)
    idx = torch.randint(0, 1 << bits, (N, K), generator=g, dtype=torch.int64)
    lut = torch.randn(N, 1 << bits, generator=g).to(dtype)
    qweight = F.pack_anyprec(idx, bits)
    x = F.make_activation(K, g, dtype=dtype)
    out = torch.zeros(1, 1, N, dtype=dtype, device="cuda")
    ext.anyprec_gemv(x.cuda(), out, qweight.cuda(), lut.cuda(), bits)
    w = ext.anyprec_dequant(qweight.cuda(), lut.cuda(), bits)
    torch.cuda.synchronize()
    want_w = O.anyprec_dequant(qweight.numpy(), np_of(lut), bits)
    assert np.array_equal(np_of(w), want_w), "dequantised weights must be bit-exact LUT entries"
    want = c_oracle.anyprec_gemv(np_of(x), qweight.numpy(), np_of(lut), bits, dt)
    check_output(np_of(out).reshape(-1), want, dt)


@pytest.mark.parametrize("cs", [2, 4, 8])
@pytest.mark.parametrize("K,N,dt", [(4096, 4096, "fp16"), (2048, 130, "fp16"), (1024, 64, "bf16"), (14336, 257, "fp16")])
def test_anyprec3_tile_decoder(K, N, dt, cs, c_oracle):
    """The optional 3-bit tile decoder (lane = row, LDS-transposed tiles, activations in SGPRs) gives the
    same result as the oracle; N not a multiple of 64 exercises the clamped rows and the odd tail."""
    dtype = TORCH_DT[dt]
    g = torch.Generator().manual_seed(K * 7 + N)
    idx = torch.randint(0, 8, (N, K), generator=g, dtype=torch.int64)
    lut = (torch.randn(N, 8, generator=g) * 0.02).to(dtype)
    qweight = F.pack_anyprec(idx, 3)
    x = F.make_activation(K, g, dtype=dtype)
    out = torch.zeros(1, 1, N, dtype=dtype, device="cuda")
    _lib.set_option("anyprec_tile", cs)
    try:
        ext.anyprec_gemv(x.cuda(), out, qweight.cuda(), lut.cuda(), 3)
        torch.cuda.synchronize()
    finally:
        _lib.set_option("anyprec_tile", 0)
    want = c_oracle.anyprec_gemv(np_of(x), qweight.numpy(), np_of(lut), 3, dt)
    check_output(np_of(out).reshape(-1), want, dt)


def test_anyprec_extra_planes_are_ignored(c_oracle):
    """qweight may hold more planes than `bitwidth` (any-precision storage); only the first are read."""
    K, N = 1024, 64
    g = torch.Generator().manual_seed(5)
    idx8 = torch.randint(0, 256, (N, K), generator=g, dtype=torch.int64)
    q8 = F.pack_anyprec(idx8, 8)
    lut3 = torch.randn(N, 8, generator=g).half()
    x = F.make_activation(K, g)
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.anyprec_gemv(x.cuda(), out, q8.cuda(), lut3.cuda(), 3)
    torch.cuda.synchronize()
    want = c_oracle.anyprec_gemv(np_of(x), q8.numpy()[:3].copy(), np_of(lut3), 3)
    check_output(np_of(out).reshape(-1), want, "fp16")


@pytest.mark.parametrize("K,N,bits,group", [(5120, 5120, 3, 128), (4096, 1024, 4, 128), (1024, 258, 2, 64)])
@pytest.mark.parametrize("dt", ["fp16", "fp32", "bf16"])
def test_lutgemm_gemv(K, N, bits, group, dt, c_oracle):
    dtype = TORCH_DT[dt]
    g = torch.Generator().manual_seed(K + N)
    W = (torch.randn(N, K, generator=g) * 0.02).half()
    q, s, z = F.awq_pseudo_quantize(W, bits, group)
    qw, alpha, q_bias = F.pack_bcq(q, s, z, bits, dtype)
    x = F.make_activation(K, g, dtype=dtype)
    out = torch.zeros(1, 1, N, dtype=dtype, device="cuda")
    ext.lutgemm_gemv(x.cuda(), out, qw.cuda(), alpha.cuda(), q_bias.cuda(), bits, group)
    torch.cuda.synchronize()
    want = c_oracle.lutgemm_gemv(np_of(x), qw.numpy(), np_of(alpha), np_of(q_bias), bits, group, dt)
    check_output(np_of(out).reshape(-1), want, dt)


@pytest.mark.parametrize("K,N,bits", [(4096, 4096, 4), (4096, 1024, 3), (1024, 130, 4), (2048, 66, 3)])
@pytest.mark.parametrize("dt", ["fp16", "fp32", "bf16"])
def test_sqllm_gemv(K, N, bits, dt, c_oracle):
    dtype = TORCH_DT[dt]
    g = torch.Generator().manual_seed(K + N + bits)
    idx = torch.randint(0, 1 << bits, (N, K), generator=g, dtype=torch.int64)
    lut = (torch.randn(N, 1 << bits, generator=g) * 0.02).to(dtype)
    mat = F.pack_sqllm(idx, bits)
    x = F.make_activation(K, g, dtype=dtype)
    out = torch.zeros(1, 1, N, dtype=dtype, device="cuda")
    ext.sqllm_gemv(x.cuda(), out, mat.cuda(), lut.cuda(), bits)
    torch.cuda.synchronize()
    want = c_oracle.sqllm_gemv(np_of(x), mat.numpy(), np_of(lut), bits, dt)
    check_output(np_of(out).reshape(-1), want, dt)


# --------------------------------------------------------------------------------------------------
# fused DEC + GEMV (both fusion modes), unfused DEC, config updates, edge cases
# --------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("fusion", [1, 0])
@pytest.mark.parametrize("kind", ["anyprec", "lutgemm", "sqllm"])
def test_dec_plus_gemv(kind, fusion, c_oracle):
    from decdec_amd import _lib
    K, N, k_chunk = 5120, 5120, 32
    L = make_dec_layer(K, N, seed=77)
    g = torch.Generator().manual_seed(78)
    ctx, rows, acts = _ctx(16, K, torch.float16)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    _lib.set_option("fusion", fusion)
    try:
        if kind == "anyprec":
            ext.dec_anyprec(cfg, x, out, L["qweight"].cuda(), L["lut"].cuda(), 3)
            base = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
        elif kind == "lutgemm":
            q, s, z = F.awq_pseudo_quantize(L["W"], 3, 128)
            qw, alpha, q_bias = F.pack_bcq(q, s, z, 3)
            ext.dec_lutgemm(cfg, x, out, qw.cuda(), alpha.cuda(), q_bias.cuda(), 3, 128)
            base = c_oracle.lutgemm_gemv(np_of(L["x"]), qw.numpy(), np_of(alpha), np_of(q_bias), 3, 128)
        else:
            idx, lut = F.quantize_uniform_rows(L["W"], 4)
            mat = F.pack_sqllm(idx, 4)
            ext.dec_sqllm(cfg, x, out, mat.cuda(), lut.cuda(), 4)
            base = c_oracle.sqllm_gemv(np_of(L["x"]), mat.numpy(), np_of(lut), 4)
        torch.cuda.synchronize()
    finally:
        _lib.set_option("fusion", 1)
    want_rows, _, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk)
    k = k_chunk * K // 1024
    assert np.array_equal(rows.cpu().numpy()[:k], want_rows[:k])
    want = base + c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    check_output(np_of(out).reshape(-1), want, "fp16")
    ext.destroy_dec_config(cfg)


@pytest.mark.parametrize("kind", ["anyprec", "sqllm"])
@pytest.mark.parametrize("K,N,k_chunk", [(4096, 4096, 4), (14336, 1032, 2), (1536, 2056, 8)])
def test_fused_launch_with_two_workgroups_per_cu(kind, K, N, k_chunk, c_oracle):
    """The register-budgeted instances of the fused kernels (any-precision: every wave walks over its own
    units) against the oracle, forced on whatever the estimate would choose."""
    from decdec_amd import _lib
    L = make_dec_layer(K, N, seed=K + N)
    ctx, rows, acts = _ctx(16, K, torch.float16)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    _lib.set_option("fused_two_per_cu", 1)
    try:
        if kind == "anyprec":
            ext.dec_anyprec(cfg, x, out, L["qweight"].cuda(), L["lut"].cuda(), 3)
            base = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
        else:
            idx, lut = F.quantize_uniform_rows(L["W"], 4)
            mat = F.pack_sqllm(idx, 4)
            ext.dec_sqllm(cfg, x, out, mat.cuda(), lut.cuda(), 4)
            base = c_oracle.sqllm_gemv(np_of(L["x"]), mat.numpy(), np_of(lut), 4)
        torch.cuda.synchronize()
    finally:
        _lib.set_option("fused_two_per_cu", -1)
    want_rows, _, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk)
    want = base + c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    check_output(np_of(out).reshape(-1), want, "fp16")
    ext.destroy_dec_config(cfg)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("K,N,k_chunk,n_tb", [(4096, 4096, 4, 16), (14336, 1032, 2, 8), (11008, 4096, 40, 32),
                                               (1536, 2056, 8, 4), (8192, 1024, 100, 16), (5120, 7680, 1, 32)])
def test_fused_anyprec_in_small_workgroups(dtype, K, N, k_chunk, n_tb, c_oracle):
    """3-bit any-precision + DEC in one launch of 4- or 8-wave workgroups (the GEMV's standalone size, the DEC
    role with the launch plan for that size), forced on for every shape that allows it: selection bit-exact,
    output against the oracle."""
    from decdec_amd import _lib
    L = make_dec_layer(K, N, seed=K + N + k_chunk, dtype=dtype)
    ctx, rows, acts = _ctx(n_tb, K, dtype)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=dtype, device="cuda")
    _lib.set_option("fused_small", 1)
    try:
        ext.dec_anyprec(cfg, x, out, L["qweight"].cuda(), L["lut"].cuda(), 3)
        torch.cuda.synchronize()
    finally:
        _lib.set_option("fused_small", -1)
    want_rows, _, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk,
                                        "fp16" if dtype == torch.float16 else "bf16")
    k = k_chunk * K // 1024
    assert np.array_equal(rows.cpu().numpy()[:k], want_rows[:k])
    base = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
    want = base + c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    check_output(np_of(out).reshape(-1), want, "fp16" if dtype == torch.float16 else "bf16")
    ext.destroy_dec_config(cfg)


def test_unfused_dec_uses_caller_indices(c_oracle):
    """evaluation/evaltools.py:327-343: exact top-k indices are written into the context's row
    buffer and unfused_dec fetches those rows."""
    K, N, k_chunk = 4096, 1024, 16
    L = make_dec_layer(K, N, seed=31)
    ctx, rows, acts = _ctx(8, K, torch.float16)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    x = L["x"].cuda()
    k = k_chunk * K // 1024
    topk = torch.topk(x[0, 0].abs().float(), k, largest=True).indices.to(torch.int32)
    rows[:k] = topk
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.unfused_dec(cfg, x, out)
    torch.cuda.synchronize()
    want = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), topk.cpu().numpy())
    check_output(np_of(out).reshape(-1), want, "fp16")
    # duplicates count twice, out-of-range indices are ignored
    rows[:k] = topk
    rows[0] = rows[1]
    rows[2] = K + 5
    out.zero_()
    ext.unfused_dec(cfg, x, out)
    torch.cuda.synchronize()
    r = rows[:k].cpu().numpy().copy()
    want = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), r)
    check_output(np_of(out).reshape(-1), want, "fp16")
    ext.destroy_dec_config(cfg)


def test_select_all_channels_reduces_to_dense_gemv():
    """k_chunk = 1024 selects every channel: DEC becomes the dense GEMV x @ R_hat (textbook check)."""
    K, N = 2048, 512
    L = make_dec_layer(K, N, seed=3)
    ctx, rows, acts = _ctx(8, K, torch.float16)
    cfg = ext.create_dec_config(ctx, 1024, L["cheat"], L["scales"], L["th"])
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dec(cfg, L["x"].cuda(), out)
    torch.cuda.synchronize()
    R = F.unpack_residual(L["cheat"], L["scales"]).double()
    want = (L["x"].double().reshape(1, -1) @ R).reshape(-1).numpy()
    check_output(np_of(out).reshape(-1), want, "fp16")
    assert sorted(rows.cpu().numpy()[:K].tolist()) == list(range(K))
    ext.destroy_dec_config(cfg)


def test_k_chunk_zero_is_a_noop_and_update_config(c_oracle):
    K, N = 4096, 4096
    L = make_dec_layer(K, N, seed=9)
    ctx, rows, acts = _ctx(8, K, torch.float16)
    cfg = ext.create_dec_config(ctx, 0, L["cheat"], L["scales"], L["th"])
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dec(cfg, x, out)
    ext.dec_anyprec(cfg, x, out, L["qweight"].cuda(), L["lut"].cuda(), 3)
    torch.cuda.synchronize()
    base = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
    check_output(np_of(out).reshape(-1), base, "fp16")
    assert (rows.cpu().numpy() == -7).all()
    # retune: new context (other n_tb) and k_chunk, residual not copied again
    ctx2 = ext.create_dec_context(32, rows, acts)
    ext.update_dec_config(cfg, ctx2, 8)
    assert ext.read_dec_config(cfg)["k_chunk"] == 8
    out.zero_()
    ext.dec(cfg, x, out)
    torch.cuda.synchronize()
    want_rows, _, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), 8)
    assert np.array_equal(rows.cpu().numpy()[:32], want_rows[:32])
    want = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    check_output(np_of(out).reshape(-1), want, "fp16")
    # a context whose buffers are too small is rejected (dec_config.cu:180-181)
    small = ext.create_dec_context(8, rows[:16], acts[:16])
    with pytest.raises(RuntimeError, match="buffer size is too small"):
        ext.update_dec_config(cfg, small, 32)
    assert ext.read_dec_config(cfg)["k_chunk"] == 8
    ext.destroy_dec_config(cfg)


def test_selector_edge_cases_general_path(c_oracle):
    """Non-monotone thresholds (a < b), ties, inf / NaN activations and fewer members than k_chunk:
    the kernel's general path must still reproduce the oracle bit for bit."""
    K, N, k_chunk = 3072, 256, 32
    L = make_dec_layer(K, N, seed=21)
    x = L["x"].clone()
    x[0, 0, 5] = float("inf"); x[0, 0, 1030] = float("nan"); x[0, 0, 2050:2200] = 3.0   # ties in one bucket
    cases = {
        "reversed": torch.flip(L["th"], dims=[0]),
        "constant": torch.full_like(L["th"], 2.0),
        "zeros": torch.zeros_like(L["th"]),
        "calibrated": L["th"],
    }
    for name, th in cases.items():
        th = th.contiguous()
        ctx, rows, acts = _ctx(4, K, torch.float16)
        cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], th)
        out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
        xs = torch.nan_to_num(x, nan=0.0, posinf=0.0) if name == "never" else x
        ext.dec(cfg, xs.cuda(), out)
        torch.cuda.synchronize()
        want_rows, _, filled = O.select_channels(np_of(xs), np_of(th), k_chunk)
        got = rows.cpu().numpy()[: want_rows.shape[0]]
        assert np.array_equal(got[filled], want_rows[filled]), name
        assert (got[~filled] == -7).all(), name          # slots the reference leaves untouched stay untouched
        ext.destroy_dec_config(cfg)


@pytest.mark.parametrize("waves", [4, 8])
def test_dec_in_smaller_workgroups(waves, c_oracle):
    """The DEC role in workgroups of 4 and 8 waves: fast selection with few and with many candidates, the
    general path (non-monotone floors, select-all), caller-supplied indices, short last chunk."""
    from decdec_amd import _lib
    _lib.set_option("dec_block_waves", waves)
    try:
        for K, N, k_chunk, n_tb in [(4096, 4096, 8, 16), (4096, 1024, 64, 8), (14336, 4096, 20, 24),
                                    (2048 + 512, 64, 32, 4), (5120, 7680, 32, 32)]:
            L = make_dec_layer(K, N, seed=K + N + k_chunk)
            ctx, rows, acts = _ctx(n_tb, K, torch.float16)
            cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
            out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
            ext.dec(cfg, L["x"].cuda(), out)
            torch.cuda.synchronize()
            want_rows, want_acts, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk)
            k = k_chunk * K // 1024
            assert np.array_equal(rows.cpu().numpy()[:k], want_rows[:k]), (K, N, k_chunk)
            assert (rows.cpu().numpy()[k:] == -7).all()
            want = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
            check_output(np_of(out).reshape(-1), want, "fp16", (K, N, k_chunk))
            # caller-supplied indices
            topk = torch.topk(L["x"][0, 0].abs().float(), k).indices.to(torch.int32).cuda()
            rows[:k] = topk
            out.zero_()
            ext.unfused_dec(cfg, L["x"].cuda(), out)
            torch.cuda.synchronize()
            want = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), topk.cpu().numpy())
            check_output(np_of(out).reshape(-1), want, "fp16")
            ext.destroy_dec_config(cfg)
        # general path: reversed thresholds, ties, inf / NaN
        K, N, k_chunk = 3072, 256, 32
        L = make_dec_layer(K, N, seed=21)
        x = L["x"].clone()
        x[0, 0, 5] = float("inf"); x[0, 0, 1030] = float("nan"); x[0, 0, 2050:2200] = 3.0
        for th in (torch.flip(L["th"], dims=[0]).contiguous(), torch.full_like(L["th"], 2.0), L["th"]):
            ctx, rows, acts = _ctx(4, K, torch.float16)
            cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], th)
            out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
            ext.dec(cfg, x.cuda(), out)
            torch.cuda.synchronize()
            want_rows, _, filled = O.select_channels(np_of(x), np_of(th), k_chunk)
            got = rows.cpu().numpy()[: want_rows.shape[0]]
            assert np.array_equal(got[filled], want_rows[filled])
            assert (got[~filled] == -7).all()
            ext.destroy_dec_config(cfg)
        # select-all
        K, N = 2048, 512
        L = make_dec_layer(K, N, seed=3)
        ctx, rows, acts = _ctx(8, K, torch.float16)
        cfg = ext.create_dec_config(ctx, 1024, L["cheat"], L["scales"], L["th"])
        out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
        ext.dec(cfg, L["x"].cuda(), out)
        torch.cuda.synchronize()
        R = F.unpack_residual(L["cheat"], L["scales"]).double()
        want = (L["x"].double().reshape(1, -1) @ R).reshape(-1).numpy()
        check_output(np_of(out).reshape(-1), want, "fp16")
        assert sorted(rows.cpu().numpy()[:K].tolist()) == list(range(K))
        ext.destroy_dec_config(cfg)
    finally:
        _lib.set_option("dec_block_waves", 16)


@pytest.mark.parametrize("rows_per_round", [0, 2, 4, 8])
def test_residual_fetch_with_every_request_width(rows_per_round, c_oracle):
    """The fetch loop requests 2, 4 or 8 residual rows per wave and round (chosen per launch; option
    dec_rows_in_flight fixes it): the same outputs whichever it is, with row counts per wave that are not multiples of
    the width (k_chunk 3, 20, 33), a short last chunk, DEC alone and fused, 16- and 8-wave workgroups."""
    from decdec_amd import _lib
    _lib.set_option("dec_rows_in_flight", rows_per_round)
    try:
        for K, N, k_chunk, n_tb in [(4096, 4096, 3, 16), (4096, 1024, 33, 8), (14336, 4096, 20, 24), (2048 + 512, 64, 32, 4),
                                    (4096, 14336, 32, 32)]:
            L = make_dec_layer(K, N, seed=K + N + k_chunk + 1)
            ctx, rows, acts = _ctx(n_tb, K, torch.float16)
            cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
            want_rows, _, filled = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk)
            dec = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows[filled])
            base = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
            for mode in ("dec", "dec8", "fused"):
                _lib.set_option("dec_block_waves", 8 if mode == "dec8" else 16)
                rows.fill_(-7)
                out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
                if mode == "fused":
                    ext.dec_anyprec(cfg, L["x"].cuda(), out, L["qweight"].cuda(), L["lut"].cuda(), 3)
                else:
                    ext.dec(cfg, L["x"].cuda(), out)
                torch.cuda.synchronize()
                got = rows.cpu().numpy()[: want_rows.shape[0]]
                assert np.array_equal(got[filled], want_rows[filled]), (K, N, k_chunk, mode)
                check_output(np_of(out).reshape(-1), dec + (base if mode == "fused" else 0.0), "fp16", (K, N, k_chunk, mode, rows_per_round))
            ext.destroy_dec_config(cfg)
    finally:
        _lib.set_option("dec_rows_in_flight", 0)
        _lib.set_option("dec_block_waves", 16)


@pytest.mark.parametrize("waves", [4, 8, 16])
def test_selection_with_crowded_windows(waves, c_oracle):
    """Activations far weaker than the calibration set: the cut falls among the crowded low buckets, where a bucket
    holds more channels than one wave can rank (two waves rank up to 128; beyond, the selection splits the window at a
    bucket boundary and the cut bucket's members take their slots in channel order), down to the last bucket, ties
    included.  Indices and
    activations bit for bit against the oracle, outputs within tolerance, at every workgroup size."""
    from decdec_amd import _lib
    _lib.set_option("dec_block_waves", waves)
    seen = {"two ranking waves": 0, "split window": 0}
    try:
        for K, N, scale, k_chunk in [(4096, 512, 0.1, 32), (4096, 512, 0.18, 64), (4096, 512, 0.08, 64),
                                     (4096 + 512, 256, 0.1, 32), (14336, 512, 0.04, 8), (4096, 512, 0.02, 2)]:
            L = make_dec_layer(K, N, seed=K + k_chunk)
            gen = torch.Generator().manual_seed(K + k_chunk)
            x = (torch.randn(1, 1, K, generator=gen) * scale * float(L["th"][k_chunk * K // 1024 - 1])).to(torch.float16)
            x[0, 0, 700:900] = x[0, 0, 700]                                  # a run of ties inside one bucket
            ctx, rows, acts = _ctx(16, K, torch.float16)
            cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
            out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
            ext.dec(cfg, x.cuda(), out)
            torch.cuda.synchronize()
            want_rows, want_acts, filled = O.select_channels(np_of(x), np_of(L["th"]), k_chunk)
            # the case is what it claims to be: some chunk's winning two-bucket window holds more than 64 channels
            floors = O.bucket_floors(float(L["th"][0]), float(L["th"][k_chunk * K // 1024 - 1]), "fp16")
            a = np.abs(np_of(x).reshape(-1).astype(np.float32))
            for c0 in range(0, K, 1024):
                kc = k_chunk * min(1024, K - c0) // 1024
                counts = [(a[c0:c0 + 1024] >= floors[b]).sum() for b in range(15, 32, 2)]
                window = next(n for n in counts if n >= kc)
                seen["two ranking waves"] += 64 < window <= 128
                seen["split window"] += window > 128
            k = want_rows.shape[0]
            assert np.array_equal(rows.cpu().numpy()[:k][filled], want_rows[filled]), (K, scale, k_chunk)
            assert (rows.cpu().numpy()[:k][~filled] == -7).all()
            assert np.array_equal(acts.cpu().float().numpy()[:k][filled], want_acts[filled])
            want = c_oracle.dec_apply(np_of(x), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
            check_output(np_of(out).reshape(-1), want, "fp16", (K, N, k_chunk, "crowded"))
            ext.destroy_dec_config(cfg)
        assert min(seen.values()) > 0, seen
    finally:
        _lib.set_option("dec_block_waves", 16)


def test_residual_on_device_is_used_in_place(c_oracle, capfd):
    K, N, k_chunk = 4096, 1024, 32
    L = make_dec_layer(K, N, seed=13)
    ctx, rows, acts = _ctx(8, K, torch.float16)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"].cuda(), L["scales"].cuda(), L["th"])
    assert ext.read_dec_config(cfg, native=True)["hip_residual_on_host"] == 0
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dec(cfg, L["x"].cuda(), out)
    torch.cuda.synchronize()
    want_rows, _, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk)
    want = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    check_output(np_of(out).reshape(-1), want, "fp16")
    ext.destroy_dec_config(cfg)


def test_dummy_ops_run_the_base_gemv(c_oracle):
    K, N = 4096, 1024
    L = make_dec_layer(K, N, seed=17)
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dummy_anyprec(L["x"].cuda(), out, L["qweight"].cuda(), L["lut"].cuda(), 3, 4, 1000)
    torch.cuda.synchronize()
    want = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
    check_output(np_of(out).reshape(-1), want, "fp16")


def test_linear_modules_decode_and_prefill(c_oracle):
    from decdec_amd.linear import APLinear
    K, N, k_chunk = 4096, 1024, 16
    L = make_dec_layer(K, N, seed=23)
    lin = APLinear(K, N, 3)
    lin.qweight.copy_(L["qweight"]); lin.lut.copy_(L["lut"])
    lin.load_dec_data(L["cheat"], L["scales"], L["th"])
    rows = torch.zeros(K, dtype=torch.int32, device="cuda"); acts = torch.zeros(K, dtype=torch.float16, device="cuda")
    ctx = ext.create_dec_context(8, rows, acts)
    lin.create_dec_config(ctx, k_chunk)
    y = lin(L["x"].cuda())
    torch.cuda.synchronize()
    want_rows, _, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), k_chunk)
    want = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3) + \
        c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    check_output(np_of(y).reshape(-1), want, "fp16")
    xs = torch.randn(1, 5, K, dtype=torch.float16, device="cuda")
    yp = lin(xs)                                  # prefill: dequantise + matmul
    wd = F.dequant_lut(L["idx"], L["lut"]).cuda()
    assert torch.allclose(yp, xs @ wd.T, rtol=1e-2, atol=1e-2)


def test_full_size_layer_properties():
    """BASELINE shapes too large for the oracle in seconds: size-independent properties.
    (i) linearity in x of the base GEMV; (ii) dec(x) with k_chunk selecting everything equals the dense
    residual GEMV computed by torch on the GPU; (iii) selection returns distinct in-range channels."""
    K, N = 8192, 28672
    g = torch.Generator().manual_seed(1)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (3, N, K // 32), generator=g, dtype=torch.int64).to(torch.int32).cuda()
    lut = torch.randn(N, 8, generator=g).half().cuda()
    x1 = F.make_activation(K, g).cuda(); x2 = F.make_activation(K, g).cuda()
    o1 = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda"); o2 = torch.zeros_like(o1); o12 = torch.zeros_like(o1)
    ext.anyprec_gemv(x1, o1, qw, lut, 3); ext.anyprec_gemv(x2, o2, qw, lut, 3)
    ext.anyprec_gemv((x1.float() * 0.5 + x2.float() * 0.25).half(), o12, qw, lut, 3)
    torch.cuda.synchronize()
    lin = o1.float() * 0.5 + o2.float() * 0.25
    scale = lin.abs().max()
    assert ((o12.float() - lin).abs().max() / scale) < 2e-2
    w = ext.anyprec_dequant(qw, lut, 3)
    ref = (x1.float().reshape(1, -1) @ w.float().T).reshape(-1)
    assert ((o1.float().reshape(-1) - ref).abs().max() / ref.abs().max()) < 1e-2
    # selection at the 70B 'down' input width
    K2, N2, k_chunk = 28672, 1024, 32
    cheat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K2, N2 // 8), generator=g, dtype=torch.int64).to(torch.int32)
    th = F.calibrate_thresholds(K2, g, draws=4)
    ctx, rows, acts = _ctx(32, K2, torch.float16)
    cfg = ext.create_dec_config(ctx, k_chunk, cheat, torch.rand(N2, generator=g).half(), th)
    x = F.make_activation(K2, g).cuda()
    out = torch.zeros(1, 1, N2, dtype=torch.float16, device="cuda")
    ext.dec(cfg, x, out)
    torch.cuda.synchronize()
    k = k_chunk * K2 // 1024
    r = rows.cpu().numpy()[:k]
    assert len(set(r.tolist())) == k and r.min() >= 0 and r.max() < K2
    assert ((r // 1024) == np.repeat(np.arange(K2 // 1024), k_chunk)).all()
    assert torch.equal(acts[:k], x[0, 0][torch.from_numpy(r).long().cuda()])
    ext.destroy_dec_config(cfg)


def test_full_size_lutgemm_and_sqllm_against_dense_torch():
    """Phi-3-medium gate_up (5120 -> 35840, LUT-GEMM 3-bit, group 128) and Llama-3-8B gate (4096 -> 14336,
    SqueezeLLM 4-bit) at full size: the packed operands are expanded to a dense fp32 matrix with plain torch
    ops on the GPU (bit extraction, gather) and multiplied; the HIP result must agree to the output tolerance."""
    g = torch.Generator().manual_seed(3)
    dev = "cuda"
    # LUT-GEMM: w[c, n] = q_bias[g, n] + sum_b alpha[g, b, n] * (2 bit - 1)
    K, N, bits, grp = 5120, 35840, 3, 128
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, bits, N), generator=g, dtype=torch.int64).to(torch.int32).to(dev)
    alpha = (torch.rand(K // grp, bits, N, generator=g) * 0.01).half().to(dev)
    qb = ((torch.rand(K // grp, N, generator=g) - 0.5) * 0.01).half().to(dev)
    x = F.make_activation(K, g).to(dev)
    out = torch.zeros(1, 1, N, dtype=torch.float16, device=dev)
    ext.lutgemm_gemv(x, out, qw, alpha, qb, bits, grp)
    ref = torch.zeros(N, dtype=torch.float32, device=dev)
    xf = x.float().reshape(-1)
    shifts = torch.arange(32, device=dev, dtype=torch.int32).view(1, 32, 1)
    for t0 in range(0, K // 32, 16):                      # 16 tiles (512 channels) at a time
        tiles = qw[t0:t0 + 16]                            # [16, bits, N]
        w = torch.zeros(16, 32, N, dtype=torch.float32, device=dev)
        gi = (torch.arange(t0, t0 + 16, device=dev) * 32) // grp
        for b in range(bits):
            sign = ((tiles[:, b, :].unsqueeze(1) >> shifts) & 1).float() * 2 - 1          # [16, 32, N]
            w += alpha[gi, b, :].float().unsqueeze(1) * sign
        w += qb[gi].float().unsqueeze(1)
        ref += (xf[t0 * 32:(t0 + 16) * 32].view(16, 32, 1) * w).sum(dim=(0, 1))
    torch.cuda.synchronize()
    assert ((out.float().reshape(-1) - ref).abs().max() / ref.abs().max()) < 1e-2
    del qw, alpha, qb, w
    # SqueezeLLM 4-bit: channel c of column n = nibble c % 8 of mat[c // 8, n]
    K, N = 4096, 14336
    mat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), generator=g, dtype=torch.int64).to(torch.int32).to(dev)
    lut = (torch.randn(N, 16, generator=g) * 0.02).half().to(dev)
    x = F.make_activation(K, g).to(dev)
    out = torch.zeros(1, 1, N, dtype=torch.float16, device=dev)
    ext.sqllm_gemv(x, out, mat, lut, 4)
    xf = x.float().reshape(-1)
    ref = torch.zeros(N, dtype=torch.float32, device=dev)
    lutT = lut.float().T.contiguous()                     # [16, N]
    for j in range(8):
        idx = ((mat >> (4 * j)) & 15).long()              # [K/8, N]
        ref += (torch.gather(lutT, 0, idx) * xf[j::8].view(-1, 1)).sum(0)
    torch.cuda.synchronize()
    assert ((out.float().reshape(-1) - ref).abs().max() / ref.abs().max()) < 1e-2
