"""Pins of the CPU oracle (no GPU): each oracle function is checked against something other than its
own formula -- an independent second implementation, a closed form, a brute force, or a special case
that reduces to a library routine -- chosen so that a dropped term, a wrong index or a transposed
operand fails."""
import numpy as np
import pytest
import torch

from oracle import decdec_oracle as O


# ---------------------------------------------------------------- bucket floors (dec.cu:117-137)
@pytest.mark.parametrize("dt", ["fp16", "bf16", "fp32"])
def test_floors_invariants(dt):
    T = O._rounder(dt)
    rng = np.random.default_rng(0)
    for _ in range(300):
        a = float(T(np.float32(abs(rng.standard_normal()) * 10.0 ** rng.integers(-2, 3))))
        b = float(T(np.float32(a * rng.random())))
        fl = O.bucket_floors(a, b, dt)
        assert fl[0] == np.float32(a)                     # a + T(0) = a
        assert fl[31] == 0.0                              # b * 0 / 16
        assert fl[16] == T(np.float32(np.float32(b) * np.float32(15)) / np.float32(16))
        assert fl[23] == T(np.float32(b) / np.float32(2))  # power-of-two scaling is exact before rounding
        assert np.all(np.diff(fl[16:]) <= 0)              # the lower half is monotone whatever the rounding
        assert abs(float(fl[15]) - b) <= 2 * np.spacing(np.float32(a)) * (1 if dt == "fp32" else 2 ** (13 if dt == "fp16" else 16))


def test_floors_c_and_numpy_restatements_agree_bitwise(c_oracle):
    rng = np.random.default_rng(1)
    for _ in range(1500):
        a = np.float16(abs(rng.standard_normal()) * 10.0 ** rng.integers(-3, 3))
        b = np.float16(float(a) * rng.random())
        for dt in ("fp16", "bf16", "fp32"):
            aa, bb = O._rounder(dt)(a), O._rounder(dt)(b)
            f1 = O.bucket_floors(aa, bb, dt)
            f2 = c_oracle.bucket_floors(float(aa), float(bb), dt)
            assert np.array_equal(f1.view(np.uint32), f2.view(np.uint32))


def _round_to_format(v, p, emin):
    """Exact rational `v` rounded to nearest, ties to even, in a binary format with `p` significand bits and minimum
    normal exponent `emin` (subnormals included; no overflow handling: the cases below stay finite)."""
    from fractions import Fraction
    if v == 0:
        return Fraction(0)
    sign = -1 if v < 0 else 1
    v = abs(v)
    e = v.numerator.bit_length() - v.denominator.bit_length()        # floor(log2 v) or one above
    if Fraction(2) ** e > v:
        e -= 1
    e = max(e, emin)
    ulp = Fraction(2) ** (e - p + 1)
    q, rem = divmod(v, ulp)
    if rem * 2 > ulp or (rem * 2 == ulp and q % 2 == 1):
        q += 1
    return sign * q * ulp


@pytest.mark.parametrize("dt,p,emin", [("fp16", 11, -14), ("bf16", 8, -126), ("fp32", 24, -126)])
def test_floors_against_exact_rational_arithmetic(dt, p, emin, c_oracle):
    """dec.cu:117-130 evaluated with exact fractions and one explicit round-to-nearest-even per operation (the
    subtraction and the final addition in the activation type, the multiply and the divide in float32, the cast
    back in the activation type).  Shares no machinery with the NumPy or the C restatement: a dropped intermediate
    rounding, a multiply done in the 16-bit type or a divide fused into the multiply changes some of these cases."""
    from fractions import Fraction
    T = lambda v: _round_to_format(v, p, emin)
    F32 = lambda v: _round_to_format(v, 24, -126)
    rng = np.random.default_rng(20241)
    pairs = [(1.0, 0.5), (3.0, 1.0), (0.333251953125, 0.111083984375), (6.1e-5, 3.0e-5), (60000.0, 1.5), (0.5, 1.0),
             (1.0, 1.0), (2.0 ** -20, 2.0 ** -24), (7.0, 0.0)]
    for _ in range(300):
        a = float(np.exp(rng.uniform(-9, 5))); b = a * float(rng.uniform(0.02, 1.0))
        pairs.append((a, b))
    tdt = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}[dt]
    differing = 0
    for a, b in pairs:
        a = float(torch.tensor(a).to(tdt).float()); b = float(torch.tensor(b).to(tdt).float())   # representable inputs
        fa, fb = Fraction(a), Fraction(b)
        want = []
        for idx in range(32):
            if idx < 16:
                d = T(fb - fa)
                step = F32(F32(d * idx) / 15)
                want.append(T(fa + T(step)))
            else:
                want.append(T(F32(F32(fb * (31 - idx)) / 16)))
        want = np.array([float(w) for w in want], dtype=np.float32)
        got = O.bucket_floors(a, b, dt)
        assert np.array_equal(got, want), (dt, a, b, got, want)
        assert np.array_equal(c_oracle.bucket_floors(a, b, dt), want), (dt, a, b)
        # the pin bites: without the cast of the step back to the activation type (one rounding of a + step instead
        # of two) some inputs give other floors
        lazy = np.array([float(T(fa + F32(F32(T(fb - fa) * idx) / 15))) for idx in range(16)], dtype=np.float32)
        differing += int(not np.array_equal(lazy, want[:16]))
    assert differing > 0 or dt == "fp32"


def test_soft_float_conversion_matches_numpy(c_oracle):
    rng = np.random.default_rng(2)
    L = c_oracle.lib()
    vals = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 4000).astype(np.float32),
                           np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 6e-8, 2.98e-8, 2.99e-8, 5.96e-8, 1e-10], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    for v, w in zip(vals, want):
        assert L.dd_f32_to_half(float(v)) == int(w)
    for bits in rng.integers(0, 0x7C00, 2000):
        assert L.dd_half_to_f32(int(bits)) == float(np.uint16(bits).view(np.float16))


# ---------------------------------------------------------------- selection (dec.cu:78-182)
@pytest.mark.parametrize("K,k_chunk", [(1024, 32), (2048 + 512, 16), (3072, 64), (512, 32)])
def test_select_vectorised_bruteforce_and_c_agree(K, k_chunk, c_oracle):
    rng = np.random.default_rng(K + k_chunk)
    x = O.make_activation(K, rng)
    th = O.calibrate_thresholds(K, rng, 8)
    r1, a1, f1 = O.select_channels(x, th, k_chunk)
    r2 = O.select_channels_bruteforce(x, th, k_chunk)
    r3, a3 = c_oracle.select(x, th, k_chunk)
    assert np.array_equal(r1, r2) and np.array_equal(r1, r3)
    assert f1.sum() == k_chunk * K // 1024
    assert np.array_equal(a1[f1].astype(np.float16).view(np.uint16), a3[f1])


def test_select_partition_invariants():
    rng = np.random.default_rng(5)
    K, k_chunk = 4096, 32
    x = O.make_activation(K, rng)
    th = O.calibrate_thresholds(K, rng, 8)
    rows, acts, filled = O.select_channels(x, th, k_chunk)
    k = k_chunk * K // 1024
    floors = O.bucket_floors(th[0], th[k - 1]); ceils = O.bucket_ceils(floors)
    ax = np.abs(x.astype(np.float32))
    bucket = np.array([next((i for i in range(32) if floors[i] <= v < ceils[i]), 99) for v in ax])
    for c in range(4):
        sel = rows[c * k_chunk:(c + 1) * k_chunk]
        assert len(set(sel.tolist())) == k_chunk and sel.min() >= c * 1024 and sel.max() < (c + 1) * 1024
        bsel = bucket[sel]
        assert np.all(np.diff(bsel) >= 0)                                   # bucket-major order
        cut = bsel.max()
        chunk = np.arange(c * 1024, (c + 1) * 1024)
        assert set(chunk[bucket[chunk] < cut]).issubset(set(sel.tolist()))   # everything above the cut bucket
        assert not (set(chunk[bucket[chunk] > cut]) & set(sel.tolist()))     # nothing below it
        for b in np.unique(bsel):                                           # ascending channel inside a bucket
            assert np.all(np.diff(sel[bsel == b]) > 0)
        assert np.array_equal(acts[c * k_chunk:(c + 1) * k_chunk].astype(np.float16), x[sel])


def test_select_equals_topk_when_thresholds_are_the_sorted_activations():
    """Recipe of decdec_extension/tests/test_dec.py:21 on one chunk with distinct |x|: b is the k-th
    largest |x|, so the bucket walk must return exactly torch.topk's set."""
    rng = np.random.default_rng(7)
    for trial in range(20):
        x = rng.permutation(np.linspace(0.01, 4.0, 1024)).astype(np.float16) * rng.choice([-1, 1], 1024).astype(np.float16)
        assert len(np.unique(np.abs(x))) == 1024
        th = np.sort(np.abs(x.astype(np.float32)))[::-1].astype(np.float16)
        rows, _, filled = O.select_channels(x, th, 32)
        top = torch.topk(torch.from_numpy(np.abs(x.astype(np.float32))), 32).indices.numpy()
        assert set(rows[:32].tolist()) == set(top.tolist())


def test_select_degenerate_inputs():
    x = np.zeros(1024, dtype=np.float16); x[3] = np.inf; x[7] = np.nan
    th = np.full(1024, 1.0, dtype=np.float16)
    rows, _, filled = O.select_channels(x, th, 8)
    assert filled.sum() == 8 and 3 not in rows[:8] and 7 not in rows[:8]      # inf and NaN are in no bucket
    assert np.array_equal(rows[:8], np.array([0, 1, 2, 4, 5, 6, 8, 9]))      # all zeros share bucket 31
    assert not O.select_channels(x, th, 0)[2].any()                           # k_chunk 0: nothing


# ---------------------------------------------------------------- launch geometry (dec_config.cu:34-115)
@pytest.mark.parametrize("K,N,n_tb,want", [
    (4096, 4096, 8, dict(channels_per_tb=64, block_dim_x=64, block_dim_y=16, n_tb=8, shared_memory_size=18176)),
    (4096, 4096, 16, dict(channels_per_tb=32, block_dim_x=32, block_dim_y=32, n_tb=16, shared_memory_size=17664)),
    (4096, 1024, 64, dict(channels_per_tb=32, block_dim_x=32, block_dim_y=32, n_tb=4, shared_memory_size=17664)),
    (4096, 14336, 8, dict(channels_per_tb=224, block_dim_x=224, block_dim_y=4, n_tb=8, shared_memory_size=18688)),
    (4096, 14336, 16, dict(channels_per_tb=128, block_dim_x=128, block_dim_y=8, n_tb=14, shared_memory_size=19200)),
    (14336, 4096, 8, dict(channels_per_tb=64, block_dim_x=64, block_dim_y=16, n_tb=8, shared_memory_size=20096)),
    (5120, 35840, 8, dict(channels_per_tb=576, block_dim_x=192, block_dim_y=5, n_tb=8, shared_memory_size=19392)),
    (17920, 5120, 16, dict(channels_per_tb=64, block_dim_x=64, block_dim_y=16, n_tb=16, shared_memory_size=20864)),
    (28672, 8192, 32, dict(channels_per_tb=32, block_dim_x=32, block_dim_y=32, n_tb=32, shared_memory_size=22272)),
])
def test_dec_geometry_hand_evaluated_table(K, N, n_tb, want):
    got = O.dec_geometry(K, N, n_tb, 32, itemsize=2, max_shared_memory=49152)
    for key, v in want.items():
        assert got[key] == v, (key, got)
    assert got["reduced_shared_memory"] == 0


# ---------------------------------------------------------------- residual format and DEC math
def test_residual_pack_unpack_roundtrip_and_dense_special_case(c_oracle):
    rng = np.random.default_rng(11)
    N, K = 64, 2048
    q = rng.integers(-7, 8, (N, K)).astype(np.int8)
    scales = (rng.random(N) * 0.01 + 1e-3).astype(np.float16)
    cheat, reord = O.pack_residual(q, scales)
    assert cheat.shape == (K, N // 8) and cheat.dtype == np.int32
    R = O.unpack_residual(cheat, reord)                                    # [K, N]
    assert np.array_equal(R, (q.astype(np.float64) * scales.astype(np.float64)[:, None]).T)
    # nibble j of word m is output 8m+j: one hand-built word
    q1 = np.zeros((8, 1), dtype=np.int8); q1[:, 0] = [-7, -3, 0, 1, 2, 5, 7, -1]
    c1, r1 = O.pack_residual(q1, np.arange(1, 9, dtype=np.float16))
    assert int(c1.view(np.uint32)[0, 0]) == sum(((int(v) + 8) & 0xF) << (4 * j) for j, v in enumerate(q1[:, 0]))
    assert np.array_equal(r1, np.arange(1, 9, dtype=np.float16))            # N/8 == 1: reorder is the identity
    # selecting every channel turns DEC into the dense GEMV x @ R (numpy matmul)
    x = O.make_activation(K, rng)
    dense = x.astype(np.float64) @ R
    assert np.allclose(O.dec_apply(x, cheat, reord, np.arange(K)), dense, rtol=1e-12, atol=1e-12)
    assert np.allclose(c_oracle.dec_apply(x, cheat, reord, np.arange(K)), dense, rtol=1e-12, atol=1e-12)
    # duplicates count twice; -1 entries are skipped
    rows = np.array([5, 5, -1, 9], dtype=np.int32)
    want = 2 * x[5].astype(np.float64) * R[5] + x[9].astype(np.float64) * R[9]
    assert np.allclose(O.dec_apply(x, cheat, reord, rows), want) and np.allclose(c_oracle.dec_apply(x, cheat, reord, rows), want)


def test_quantize_residual_properties():
    rng = np.random.default_rng(13)
    E = (rng.standard_normal((16, 512)) * 0.003).astype(np.float16)
    q, s = O.quantize_residual(E)
    assert q.min() >= -7 and q.max() <= 7
    e32, s32 = E.astype(np.float32), s.astype(np.float32)[:, None]
    unclamped = np.abs(q) < 7
    assert np.all(np.abs(e32 - q * s32)[unclamped] <= s32.repeat(512, 1)[unclamped] * 0.5 * 1.01)
    # the chosen scale is the float32-MSE minimiser of the 32-point grid (brute force, row 0)
    ms = np.float32(np.float16(np.float16(np.abs(E[0]).max()) / np.float16(7)))
    grid = O._torch_linspace_f32(np.float32(np.float16(np.float16(ms) / np.float16(32))), ms, 32)
    mses = [np.mean((e32[0] - np.clip(np.rint(e32[0] / g), -7, 7) * g) ** 2, dtype=np.float32) for g in grid]
    assert s[0] == np.float16(grid[int(np.argmin(mses))])
    # idempotent on an exactly representable residual
    s0 = np.float16(0.002); E2 = (rng.integers(-7, 8, (4, 64)) * np.float32(s0)).astype(np.float16)
    E2[:, 0] = np.float16(7 * np.float32(s0))
    q2, s2 = O.quantize_residual(E2)
    assert np.allclose(q2 * s2.astype(np.float32)[:, None], E2.astype(np.float32), atol=float(s0) * 0.51)


def test_reference_rounding_error_budget():
    """How far the reference's own fp16 arithmetic (dec.cu:248-275) sits from the exact value, under
    the metric the GPU tests use: this is what fixes the 10 % floor in tests/helpers.rel_err."""
    from tests.helpers import make_dec_layer, np_of, rel_err
    K, N, kc = 4096, 1024, 32
    L = make_dec_layer(K, N, seed=K + N + kc)
    rows, _, _ = O.select_channels(np_of(L["x"]), np_of(L["th"]), kc)
    want = O.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), rows)
    ref16 = O.dec_apply_reference_rounding(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), rows[:128], 16)
    strict = rel_err(ref16.astype(np.float64), want, floor=0.01)[0]
    used = rel_err(ref16.astype(np.float64), want)[0]
    assert used <= 1e-2 < strict * 2, (used, strict)       # passes with the 10 % floor, at or beyond 1e-2 with 1 %


# ---------------------------------------------------------------- any-precision bitplanes
@pytest.mark.parametrize("K", [1024, 2048 + 512, 1024 + 32])
@pytest.mark.parametrize("bits", [3, 4, 8])
def test_anyprec_two_readings_of_the_layout_agree(K, bits, c_oracle):
    rng = np.random.default_rng(K + bits)
    N = 12
    idx = rng.integers(0, 1 << bits, (N, K)).astype(np.uint8)
    q = O.anyprec_pack(idx, bits)
    assert np.array_equal(O.anyprec_unpack(q, bits), idx)
    lut = rng.standard_normal((N, 1 << bits)).astype(np.float16)
    x = O.make_activation(K, rng)
    via_store_addresses = O.anyprec_gemv(x, q, lut, bits)              # dequant_kbit_store's reading
    via_load_addresses = O.anyprec_gemv_kernel_order(x, q, lut, bits)   # matmul_kbit_32's reading
    assert np.allclose(via_store_addresses, via_load_addresses, rtol=1e-12, atol=1e-12)
    assert np.allclose(c_oracle.anyprec_gemv(x, q, lut, bits), via_store_addresses, rtol=1e-12, atol=1e-12)
    dense = np.take_along_axis(lut, idx.astype(np.int64), axis=1).astype(np.float64) @ x.astype(np.float64)
    assert np.allclose(dense, via_store_addresses, rtol=1e-12, atol=1e-12)


def test_anyprec_bit_position_spot_checks():
    """bit 31 of word t of chunk i is channel 1024 i + 8 t (j = e = 0); bit 0 is channel 1024 i + 768 + 8 t + 7;
    plane 0 is the MSB.  One weight set at a time."""
    K, N = 2048, 1
    for ch, (w, b) in {0: (0, 31), 7: (0, 24), 8: (1, 31), 256: (0, 23), 1023: (31, 0), 1024: (32, 31), 1024 + 768 + 15: (33, 0)}.items():
        idx = np.zeros((N, K), dtype=np.uint8); idx[0, ch] = 0b101
        q = O.anyprec_pack(idx, 3).view(np.uint32)
        assert q[0, 0, w] == (1 << b) and q[1, 0, w] == 0 and q[2, 0, w] == (1 << b), ch
        assert q.sum() == 2 * (1 << b)


# ---------------------------------------------------------------- LUT-GEMM BCQ
def test_bcq_reproduces_uniform_asymmetric_quantisation(c_oracle):
    rng = np.random.default_rng(17)
    N, K, bits, group = 16, 512, 3, 128
    W = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    q, s, z = O.awq_pseudo_quantize(W, bits, group)
    assert q.min() >= 0 and q.max() <= 7
    qw, alpha, q_bias = O.bcq_pack(q, s, z, bits)
    assert qw.shape == (K // 32, bits, N) and alpha.shape == (K // group, bits, N) and q_bias.shape == (K // group, N)
    Wd = O.lutgemm_dequant(qw, alpha, q_bias, group)
    want = ((q.reshape(N, K // group, group) - z[:, :, None]) * s[:, :, None]).reshape(N, K)   # scale * (q - zero)
    assert np.allclose(Wd, want, rtol=0, atol=1e-7)
    assert np.abs(Wd - W.astype(np.float64)).max() <= s.max() * 0.51                              # within half a step
    x = O.make_activation(K, rng)
    assert np.allclose(c_oracle.lutgemm_gemv(x, qw, alpha, q_bias, bits, group, "fp32"), want @ x.astype(np.float64), atol=1e-6)
    # LSB-first bit order inside a word: channel 32 t + j is bit j
    q1 = np.zeros((1, 64), dtype=np.int32); q1[0, 33] = 0b010
    qw1, _, _ = O.bcq_pack(q1, np.ones((1, 1), np.float32), np.zeros((1, 1), np.float32), 3)
    assert qw1.view(np.uint32)[1, 1, 0] == 2 and qw1.view(np.uint32).sum() == 2


# ---------------------------------------------------------------- SqueezeLLM
@pytest.mark.parametrize("bits", [3, 4])
def test_sqllm_pack_against_python_big_integers(bits, c_oracle):
    rng = np.random.default_rng(19 + bits)
    N, K = 6, 256
    idx = rng.integers(0, 1 << bits, (N, K)).astype(np.uint8)
    mat = O.sqllm_pack(idx, bits)
    assert mat.shape == (K * bits // 32, N)
    assert np.array_equal(O.sqllm_unpack(mat, bits), idx)
    u = mat.view(np.uint32)
    for n in range(N):
        per = 32 if bits == 3 else 8
        words = bits * per // 32
        for g in range(K // per):
            stream = sum(int(v) << (bits * j) for j, v in enumerate(idx[n, g * per:(g + 1) * per]))   # little-endian
            for w in range(words):
                assert int(u[g * words + w, n]) == (stream >> (32 * w)) & 0xFFFFFFFF
    lut = rng.standard_normal((N, 1 << bits)).astype(np.float16)
    x = O.make_activation(K, rng)
    dense = np.take_along_axis(lut, idx.astype(np.int64), axis=1).astype(np.float64) @ x.astype(np.float64)
    assert np.allclose(O.sqllm_gemv(x, mat, lut, bits), dense) and np.allclose(c_oracle.sqllm_gemv(x, mat, lut, bits), dense)
