"""GPU parity at the configuration shapes (Llama-3-8B, Phi-3-medium, Llama-3-70B linears) and at the operator
boundary: live launch geometry, the reference's custom-op wrapping, the dummy_* ops and side files.

Bar as in test_gpu_parity.py: selected channel indices bit-exact; outputs within 1e-2 of the float64 oracle
(relative, denominator floored at 10 % of max|y|).  Every output assertion reports the mean absolute error and
the same ratio with a 1 % floor.
"""
import numpy as np
import pytest
import torch

from decdec_amd import _lib, artifacts, ext, formats as F
from oracle import decdec_oracle as O
from tests.helpers import check_output, make_dec_layer, np_of

pytestmark = pytest.mark.gpu


def _ctx(n_tb, K, dtype=torch.float16):
    rows = torch.full((K,), -7, dtype=torch.int32, device="cuda")
    acts = torch.zeros(K, dtype=dtype, device="cuda")
    return ext.create_dec_context(n_tb, rows, acts), rows, acts


def _dec_only_layer(K, N, seed):
    """Activation, calibrated thresholds, random residual words and scales: what DEC alone needs (no base weight,
    so the 70B shapes stay cheap to build)."""
    g = torch.Generator().manual_seed(seed)
    cheat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=g, dtype=torch.int64).to(torch.int32)
    scales = (torch.rand(N, generator=g) * 1e-3 + 5e-4).half()
    x = F.make_activation(K, g)
    th = F.calibrate_thresholds(K, g, draws=16)
    return {"cheat": cheat.contiguous(), "scales": scales.contiguous(), "x": x, "th": th}


# --------------------------------------------------------------------------------------------------
# cheap ones first
# --------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 1024), (4096, 14336), (14336, 4096), (5120, 35840), (17920, 5120),
                                 (28672, 8192)])
def test_live_config_reports_the_reference_geometry(K, N):
    """read_dec_config of a live config (dec_config.cu:337-354): the nine keys equal the reference's launch
    geometry (dec_config.cu:34-115) at every n_tb, and follow an update_dec_config."""
    g = torch.Generator().manual_seed(K + N)
    cheat = torch.zeros(K, N // 8, dtype=torch.int32)
    scales = torch.rand(N, generator=g).half()
    th = F.calibrate_thresholds(K, g, draws=2)
    smem = getattr(torch.cuda.get_device_properties(0), "shared_memory_per_block", 65536)
    rows = torch.zeros(K, dtype=torch.int32, device="cuda"); acts = torch.zeros(K, dtype=torch.float16, device="cuda")
    cfg = None
    for n_tb in (8, 16, 32, 64):
        ctx = ext.create_dec_context(n_tb, rows, acts)
        if cfg is None:
            cfg = ext.create_dec_config(ctx, 32, cheat, scales, th)
        else:
            ext.update_dec_config(cfg, ctx, 32)
        got = ext.read_dec_config(cfg)
        want = O.dec_geometry(K, N, n_tb, 32, 2, smem)
        assert set(got) == set(_lib.REFERENCE_KEYS) and len(got) == 9
        assert got == {k: int(want[k]) for k in _lib.REFERENCE_KEYS}, (n_tb, got, want)
    ext.update_dec_config(cfg, ctx, 16)
    assert ext.read_dec_config(cfg) == {k: int(O.dec_geometry(K, N, 64, 16, 2, smem)[k]) for k in _lib.REFERENCE_KEYS}
    ext.destroy_dec_config(cfg)


def test_dummy_ops_run_each_base_gemv(c_oracle):
    """dummy_anyprec / dummy_lutgemm / dummy_sqllm (decdec.h:90-120): the base GEMV next to a spin kernel that
    holds `dummy_sm` compute units; the output is the GEMV's, with and without the spin kernel."""
    K, N = 4096, 1024
    L = make_dec_layer(K, N, seed=17)
    x = L["x"].cuda()
    xn = np_of(L["x"])
    q, s, z = F.awq_pseudo_quantize(L["W"], 3, 128)
    qw, alpha, q_bias = F.pack_bcq(q, s, z, 3)
    idx4, lut4 = F.quantize_uniform_rows(L["W"], 4)
    mat = F.pack_sqllm(idx4, 4)
    cases = {
        "anyprec": (lambda out, sm: ext.dummy_anyprec(x, out, L["qweight"].cuda(), L["lut"].cuda(), 3, sm, 2000),
                    c_oracle.anyprec_gemv(xn, L["qweight"].numpy(), np_of(L["lut"]), 3)),
        "lutgemm": (lambda out, sm: ext.dummy_lutgemm(x, out, qw.cuda(), alpha.cuda(), q_bias.cuda(), 3, 128, sm, 2000),
                    c_oracle.lutgemm_gemv(xn, qw.numpy(), np_of(alpha), np_of(q_bias), 3, 128)),
        "sqllm": (lambda out, sm: ext.dummy_sqllm(x, out, mat.cuda(), lut4.cuda(), 4, sm, 2000),
                  c_oracle.sqllm_gemv(xn, mat.numpy(), np_of(lut4), 4)),
    }
    for name, (run, want) in cases.items():
        for sm in (0, 8, 64):
            out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
            run(out, sm)
            torch.cuda.synchronize()
            check_output(np_of(out).reshape(-1), want, "fp16", (name, sm))


def test_ops_wrapped_as_custom_ops_trace_compile_and_capture(c_oracle):
    """The reference reaches the ops through torch.library.custom_op wrappers that mutate `output` and have an empty
    fake implementation (end-to-end/plugin.py:7-71), under torch.compile(fullgraph=True) and graph capture.  The
    same wrapping of this library's ops must trace with fake tensors, run compiled, and replay from a graph."""
    K, N, k_chunk = 4096, 1024, 16
    L = make_dec_layer(K, N, seed=41)
    ctx, rows, acts = _ctx(8, K)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])

    @torch.library.custom_op("decdec_test::dec_anyprec", mutates_args={"output"})
    def dec_anyprec_op(dec_config: int, x: torch.Tensor, output: torch.Tensor, q_weight: torch.Tensor,
                       lut: torch.Tensor, bitwidth: int) -> None:
        ext.dec_anyprec(dec_config, x, output, q_weight, lut, bitwidth)

    @dec_anyprec_op.register_fake
    def _(dec_config, x, output, q_weight, lut, bitwidth):
        return None

    @torch.library.custom_op("decdec_test::anyprec_gemv", mutates_args={"output"})
    def anyprec_gemv_op(x: torch.Tensor, output: torch.Tensor, q_weight: torch.Tensor, lut: torch.Tensor,
                        bitwidth: int) -> None:
        ext.anyprec_gemv(x, output, q_weight, lut, bitwidth)

    @anyprec_gemv_op.register_fake
    def _(x, output, q_weight, lut, bitwidth):
        return None

    qweight, lut = L["qweight"].cuda(), L["lut"].cuda()

    def layer(x):
        y = torch.zeros(1, 1, N, dtype=x.dtype, device=x.device)
        dec_anyprec_op(cfg, x, y, qweight, lut, 3)
        z = torch.zeros(1, 1, N, dtype=x.dtype, device=x.device)
        anyprec_gemv_op(x, z, qweight, lut, 3)
        return y, z

    xn = np_of(L["x"])
    want_rows, _, _ = O.select_channels(xn, np_of(L["th"]), k_chunk)
    base = c_oracle.anyprec_gemv(xn, L["qweight"].numpy(), np_of(L["lut"]), 3)
    want = base + c_oracle.dec_apply(xn, L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    x = L["x"].cuda()
    # fake-tensor tracing + functionalisation of the mutated argument, no code generation involved
    compiled = torch.compile(layer, backend="aot_eager", fullgraph=True, dynamic=False)
    for _ in range(2):
        y, z = compiled(x)
        torch.cuda.synchronize()
        check_output(np_of(y).reshape(-1), want, "fp16", "compiled dec_anyprec")
        check_output(np_of(z).reshape(-1), base, "fp16", "compiled anyprec_gemv")
    # graph capture of the wrapped ops, several replays with eager work between them
    static_x = x.clone()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        layer(static_x)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gy, gz = layer(static_x)
    for it in range(3):
        junk = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")
        graph.replay()
        torch.cuda.synchronize()
        check_output(np_of(gy).reshape(-1), want, "fp16", ("replay", it))
        check_output(np_of(gz).reshape(-1), base, "fp16", ("replay", it))
        del junk
    assert np.array_equal(rows.cpu().numpy()[:len(want_rows)], want_rows)
    ext.destroy_dec_config(cfg)


# --------------------------------------------------------------------------------------------------
# Llama-3-8B shapes at the benchmark's setting
# --------------------------------------------------------------------------------------------------
def test_anyprec_gemv_at_the_roofline_shape(c_oracle):
    """Any-precision 3-bit GEMV at 4096 -> 14336 (gate / up), the shape the roofline figure is quoted on."""
    K, N = 4096, 14336
    L = make_dec_layer(K, N, seed=K + N, random_residual=True)
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.anyprec_gemv(L["x"].cuda(), out, L["qweight"].cuda(), L["lut"].cuda(), 3)
    torch.cuda.synchronize()
    want = c_oracle.anyprec_gemv(np_of(L["x"]), L["qweight"].numpy(), np_of(L["lut"]), 3)
    check_output(np_of(out).reshape(-1), want, "fp16", (K, N))


@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096), (4096, 4096), (4096, 1024)])
def test_fused_dec_anyprec_at_the_benchmark_setting(K, N, c_oracle):
    """dec_anyprec at k_chunk 32, n_tb 32 on the Llama-3-8B linears: indices bit-exact, output against the oracle;
    and the compensated output is closer to the unquantised layer than the base GEMV alone."""
    k_chunk, n_tb = 32, 32
    L = make_dec_layer(K, N, seed=K + 3 * N)
    ctx, rows, acts = _ctx(n_tb, K)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dec_anyprec(cfg, L["x"].cuda(), out, L["qweight"].cuda(), L["lut"].cuda(), 3)
    torch.cuda.synchronize()
    xn = np_of(L["x"])
    want_rows, want_acts, _ = O.select_channels(xn, np_of(L["th"]), k_chunk)
    k = k_chunk * K // 1024
    assert np.array_equal(rows.cpu().numpy()[:k], want_rows[:k]), "selected channel indices differ from the oracle"
    assert np.array_equal(np_of(acts)[:k], want_acts[:k].astype(np.float16))
    base = c_oracle.anyprec_gemv(xn, L["qweight"].numpy(), np_of(L["lut"]), 3)
    want = base + c_oracle.dec_apply(xn, L["cheat"].numpy(), np_of(L["scales"]), want_rows)
    check_output(np_of(out).reshape(-1), want, "fp16", (K, N))
    exact = L["W"].double().numpy() @ xn.astype(np.float64).reshape(-1)
    assert np.abs(np_of(out).reshape(-1) - exact).mean() < np.abs(base - exact).mean()
    assert ext.read_dec_config(cfg, native=True)["hip_chunk_groups"] <= 4
    ext.destroy_dec_config(cfg)


@pytest.mark.parametrize("waves", [16, 8, 4])
@pytest.mark.parametrize("K,N,k_chunk", [(14336, 4096, 32), (14336, 4096, 20)])
def test_unfused_dec_with_magnitude_sorted_indices(K, N, k_chunk, waves, c_oracle):
    """Caller-supplied exact top-k indices in descending magnitude (evaluation/evaltools.py:327-343): the first
    chunk group then holds all the largest activations, the hardest case for the order of the output's atomic
    adds.  Every workgroup size."""
    L = make_dec_layer(K, N, seed=K + N + k_chunk, random_residual=True)
    _lib.set_option("dec_block_waves", waves)
    try:
        ctx, rows, acts = _ctx(24, K)
        cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
        assert ext.read_dec_config(cfg, native=True)["hip_chunk_groups"] <= 4
        k = k_chunk * K // 1024
        x = L["x"].cuda()
        topk = torch.topk(x[0, 0].abs().float(), k).indices.to(torch.int32)
        rows[:k] = topk
        out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
        ext.unfused_dec(cfg, x, out)
        torch.cuda.synchronize()
    finally:
        _lib.set_option("dec_block_waves", 16)
    want = c_oracle.dec_apply(np_of(L["x"]), L["cheat"].numpy(), np_of(L["scales"]), topk.cpu().numpy())
    check_output(np_of(out).reshape(-1), want, "fp16", (K, N, k_chunk, waves))
    ext.destroy_dec_config(cfg)


@pytest.mark.parametrize("dt,bits", [("fp16", 3), ("bf16", 3), ("fp16", 4), ("fp16", 5)])
def test_batched_layers_match_the_oracle_layer_by_layer(dt, bits, c_oracle):
    """dec_anyprec_batch: q | k | v of a Llama-3-8B layer (one input, three outputs) in one launch, every layer with
    its own config and context; then the same batch with DEC on the middle layer only, and without any config.
    Each output against the oracle, each context's selection bit-exact.  (5 bits: the per-layer fallback.)"""
    from tests.helpers import TORCH_DT
    dtype = TORCH_DT[dt]
    K, Ns, k_chunk = 4096, (4096, 1024, 1032), 32
    g = torch.Generator().manual_seed(7)
    x = F.make_activation(K, g, dtype=dtype)
    xn = np_of(x)
    layers = []
    for li, N in enumerate(Ns):
        W = (torch.randn(N, K, generator=g) * 0.02).half()
        idx, lut = F.quantize_uniform_rows(W, bits)
        cheat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=g, dtype=torch.int64).to(torch.int32)
        scales = (torch.rand(N, generator=g) * 1e-3 + 5e-4).to(dtype)
        th = F.calibrate_thresholds(K, g, draws=8, dtype=dtype)
        ctx, rows, acts = _ctx(16, K, dtype)
        cfg = ext.create_dec_config(ctx, k_chunk, cheat, scales, th)
        qweight = F.pack_anyprec(idx, bits)
        layers.append(dict(N=N, qweight=qweight, lut=lut.to(dtype), cheat=cheat, scales=scales, th=th, cfg=cfg, rows=rows, acts=acts,
                           base=c_oracle.anyprec_gemv(xn, qweight.numpy(), np_of(lut.to(dtype)), bits, dt)))
    qws = [l["qweight"].cuda() for l in layers]
    luts = [l["lut"].cuda() for l in layers]
    xc = x.cuda()
    for mode in ("all", "middle", "none"):
        outs = [torch.zeros(1, 1, l["N"], dtype=dtype, device="cuda") for l in layers]
        for l in layers:
            l["rows"].fill_(-7)
        cfgs = {"all": [l["cfg"] for l in layers], "middle": [0, layers[1]["cfg"], None], "none": None}[mode]
        ext.dec_anyprec_batch(cfgs, xc, outs, qws, luts, bits)
        torch.cuda.synchronize()
        for li, l in enumerate(layers):
            with_dec = cfgs is not None and bool(cfgs[li])
            want = l["base"]
            if with_dec:
                want_rows, _, _ = O.select_channels(xn, np_of(l["th"]), k_chunk, dt)
                k = k_chunk * K // 1024
                assert np.array_equal(l["rows"].cpu().numpy()[:k], want_rows[:k]), (mode, li)
                want = want + c_oracle.dec_apply(xn, l["cheat"].numpy(), np_of(l["scales"]), want_rows[:k], dt)
            else:
                assert (l["rows"].cpu().numpy() == -7).all(), (mode, li)
            check_output(np_of(outs[li]).reshape(-1), want, dt, (mode, li, bits))
    for l in layers:
        ext.destroy_dec_config(l["cfg"])


@pytest.mark.parametrize("kind,dt", [("lutgemm", "fp16"), ("lutgemm", "bf16"), ("lutgemm", "fp32"),
                                     ("sqllm", "fp16"), ("sqllm", "bf16"), ("sqllm", "fp32")])
def test_batched_lutgemm_and_sqllm_layers_match_the_oracle(kind, dt, c_oracle):
    """dec_lutgemm_batch / dec_sqllm_batch: three layers on one input in one launch (fp32: the per-layer path), DEC on
    all, on the middle one only, on none; every output against the oracle, every context's selection bit-exact."""
    from tests.helpers import TORCH_DT
    dtype = TORCH_DT[dt]
    K, Ns, k_chunk, group = 4096, (2048, 1024, 520), 32, 128
    bits = 3 if kind == "lutgemm" else 4
    g = torch.Generator().manual_seed(11)
    x = F.make_activation(K, g, dtype=dtype)
    xn = np_of(x)
    layers = []
    for N in Ns:
        W = (torch.randn(N, K, generator=g) * 0.02).half()
        cheat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=g, dtype=torch.int64).to(torch.int32)
        scales = (torch.rand(N, generator=g) * 1e-3 + 5e-4).to(dtype)
        th = F.calibrate_thresholds(K, g, draws=8, dtype=dtype)
        ctx, rows, acts = _ctx(16, K, dtype)
        cfg = ext.create_dec_config(ctx, k_chunk, cheat, scales, th)
        if kind == "lutgemm":
            q, s, z = F.awq_pseudo_quantize(W, bits, group)
            qw, alpha, q_bias = F.pack_bcq(q, s, z, bits, dtype=dtype)
            weights = (qw, alpha, q_bias)
            base = c_oracle.lutgemm_gemv(xn, qw.numpy(), np_of(alpha), np_of(q_bias), bits, group, dt)
        else:
            idx, lut = F.quantize_uniform_rows(W, bits)
            mat, lut = F.pack_sqllm(idx, bits), lut.to(dtype)
            weights = (mat, lut)
            base = c_oracle.sqllm_gemv(xn, mat.numpy(), np_of(lut), bits, dt)
        layers.append(dict(N=N, weights=[w.cuda() for w in weights], cheat=cheat, scales=scales, th=th, cfg=cfg, rows=rows,
                           acts=acts, base=base))
    xc = x.cuda()
    per_layer = list(zip(*[l["weights"] for l in layers]))             # one sequence per weight kind
    for mode in ("all", "middle", "none"):
        outs = [torch.zeros(1, 1, l["N"], dtype=dtype, device="cuda") for l in layers]
        for l in layers:
            l["rows"].fill_(-7)
        cfgs = {"all": [l["cfg"] for l in layers], "middle": [0, layers[1]["cfg"], None], "none": None}[mode]
        if kind == "lutgemm":
            ext.dec_lutgemm_batch(cfgs, xc, outs, *per_layer, bits, group)
        else:
            ext.dec_sqllm_batch(cfgs, xc, outs, *per_layer, bits)
        torch.cuda.synchronize()
        for li, l in enumerate(layers):
            with_dec = cfgs is not None and bool(cfgs[li])
            want = l["base"]
            if with_dec:
                want_rows, _, _ = O.select_channels(xn, np_of(l["th"]), k_chunk, dt)
                k = k_chunk * K // 1024
                assert np.array_equal(l["rows"].cpu().numpy()[:k], want_rows[:k]), (mode, li)
                want = want + c_oracle.dec_apply(xn, l["cheat"].numpy(), np_of(l["scales"]), want_rows[:k], dt)
            else:
                assert (l["rows"].cpu().numpy() == -7).all(), (mode, li)
            check_output(np_of(outs[li]).reshape(-1), want, dt, (kind, mode, li))
    for l in layers:
        ext.destroy_dec_config(l["cfg"])


def _random_anyprec3(K, N, g):
    """Random 3-bit planes and a sorted random LUT per row: everything the GEMV reads, without quantising a weight
    matrix (a 70B-size layer is built in a second)."""
    qweight = torch.randint(-2 ** 31, 2 ** 31 - 1, (3, N, K // 32), generator=g, dtype=torch.int64).to(torch.int32)
    lut = (torch.randn(N, 8, generator=g) * 0.02).sort(dim=1).values.half()
    return qweight.contiguous(), lut.contiguous()


@pytest.mark.parametrize("two_per_cu", [0, 1])
@pytest.mark.parametrize("Ns", [(14336, 14336), (4096, 1024, 1024)], ids=["gate_up", "q_k_v"])
def test_batched_launch_at_the_benchmark_shapes(Ns, two_per_cu, c_oracle):
    """dec_anyprec_batch as the benchmark launches it: gate | up = 2 x (4096 -> 14336) and q | k | v = 4096 -> (4096, 1024,
    1024) at k_chunk 32, n_tb 32, with the fused kernel instance chosen both ways.  Every layer's selection bit-exact,
    every output against the oracle; then the same batch with ONE context shared by all layers (the scratch read-back
    then belongs to whichever layer wrote last, the outputs must still be right)."""
    K, k_chunk, n_tb = 4096, 32, 32
    g = torch.Generator().manual_seed(sum(Ns) + two_per_cu)
    x = F.make_activation(K, g)
    xn = np_of(x)
    k = k_chunk * K // 1024
    layers = []
    for N in Ns:
        qweight, lut = _random_anyprec3(K, N, g)
        cheat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=g, dtype=torch.int64).to(torch.int32)
        scales = (torch.rand(N, generator=g) * 1e-3 + 5e-4).half()
        th = F.calibrate_thresholds(K, g, draws=8)
        want_rows, _, _ = O.select_channels(xn, np_of(th), k_chunk)
        want = c_oracle.anyprec_gemv(xn, qweight.numpy(), np_of(lut), 3) + \
            c_oracle.dec_apply(xn, cheat.numpy(), np_of(scales), want_rows[:k])
        layers.append(dict(N=N, qweight=qweight.cuda(), lut=lut.cuda(), cheat=cheat, scales=scales, th=th,
                           want_rows=want_rows, want=want))
    xc = x.cuda()
    _lib.set_option("fused_two_per_cu", two_per_cu)
    try:
        own = [_ctx(n_tb, K) for _ in layers]
        cfgs = [ext.create_dec_config(c[0], k_chunk, l["cheat"], l["scales"], l["th"]) for c, l in zip(own, layers)]
        outs = [torch.zeros(1, 1, l["N"], dtype=torch.float16, device="cuda") for l in layers]
        ext.dec_anyprec_batch(cfgs, xc, outs, [l["qweight"] for l in layers], [l["lut"] for l in layers], 3)
        torch.cuda.synchronize()
        for li, (l, c) in enumerate(zip(layers, own)):
            assert np.array_equal(c[1].cpu().numpy()[:k], l["want_rows"][:k]), ("selection", li)
            check_output(np_of(outs[li]).reshape(-1), l["want"], "fp16", ("own contexts", Ns, two_per_cu, li))
        for cfg in cfgs:
            ext.destroy_dec_config(cfg)
        shared = _ctx(n_tb, K)
        cfgs = [ext.create_dec_config(shared[0], k_chunk, l["cheat"], l["scales"], l["th"]) for l in layers]
        outs = [torch.zeros(1, 1, l["N"], dtype=torch.float16, device="cuda") for l in layers]
        ext.dec_anyprec_batch(cfgs, xc, outs, [l["qweight"] for l in layers], [l["lut"] for l in layers], 3)
        torch.cuda.synchronize()
        for li, l in enumerate(layers):
            check_output(np_of(outs[li]).reshape(-1), l["want"], "fp16", ("one shared context", Ns, two_per_cu, li))
        for cfg in cfgs:
            ext.destroy_dec_config(cfg)
    finally:
        _lib.set_option("fused_two_per_cu", -1)


@pytest.mark.parametrize("K,Ns,bits", [(4096, (14336, 14336), 3), (4096, (4096, 1024, 1024), 3), (4096, (14336, 40, 1000), 3),
                                       (2080, (3000, 17, 7000, 64), 3), (4096, (6000, 24, 1000), 4)],
                         ids=["gate_up", "q_k_v", "ragged", "ragged_k_tail", "ragged_4bit"])
def test_base_only_batch_planned_by_its_total_rows(K, Ns, bits, c_oracle):
    """A batch without DEC runs the layers' GEMVs in one launch of the standalone kernel's workgroups, every layer with
    the rows per wave that the rows of the whole launch call for: a 40-row layer beside a 14336-row one gets eight rows
    per wave and row tails in every workgroup.  Every output against the oracle."""
    g = torch.Generator().manual_seed(sum(Ns) + K + bits)
    x = F.make_activation(K, g)
    xn = np_of(x)
    qws, luts, wants = [], [], []
    for N in Ns:
        qweight = torch.randint(-2 ** 31, 2 ** 31 - 1, (bits, N, K // 32), generator=g, dtype=torch.int64).to(torch.int32).contiguous()
        lut = (torch.randn(N, 2 ** bits, generator=g) * 0.02).sort(dim=1).values.half().contiguous()
        wants.append(c_oracle.anyprec_gemv(xn, qweight.numpy(), np_of(lut), bits))
        qws.append(qweight.cuda()); luts.append(lut.cuda())
    outs = [torch.zeros(1, 1, N, dtype=torch.float16, device="cuda") for N in Ns]
    ext.dec_anyprec_batch(None, x.cuda(), outs, qws, luts, bits)
    torch.cuda.synchronize()
    for li, want in enumerate(wants):
        check_output(np_of(outs[li]).reshape(-1), want, "fp16", (K, Ns, bits, li))


@pytest.mark.parametrize("K,N", [(28672, 8192), (8192, 28672)])
def test_anyprec_at_llama3_70b_gate_and_down(K, N, c_oracle):
    """Any-precision 3-bit at the two large 70B linears (28672 -> 8192 is the 14-slice, 896-thread launch form):
    the GEMV alone, then dec_anyprec at k_chunk 16 and 32, against the oracle; indices bit-exact."""
    g = torch.Generator().manual_seed(K + N)
    qweight, lut = _random_anyprec3(K, N, g)
    L = _dec_only_layer(K, N, seed=K - N)
    xn = np_of(L["x"])
    xc, qc, lc = L["x"].cuda(), qweight.cuda(), lut.cuda()
    base = c_oracle.anyprec_gemv(xn, qweight.numpy(), np_of(lut), 3)
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.anyprec_gemv(xc, out, qc, lc, 3)
    torch.cuda.synchronize()
    check_output(np_of(out).reshape(-1), base, "fp16", ("anyprec_gemv", K, N))
    for k_chunk in (16, 32):
        ctx, rows, acts = _ctx(32, K)
        cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
        out.zero_()
        ext.dec_anyprec(cfg, xc, out, qc, lc, 3)
        torch.cuda.synchronize()
        k = k_chunk * K // 1024
        want_rows, _, _ = O.select_channels(xn, np_of(L["th"]), k_chunk)
        assert np.array_equal(rows.cpu().numpy()[:k], want_rows[:k]), (K, N, k_chunk)
        want = base + c_oracle.dec_apply(xn, L["cheat"].numpy(), np_of(L["scales"]), want_rows[:k])
        check_output(np_of(out).reshape(-1), want, "fp16", ("dec_anyprec", K, N, k_chunk))
        ext.destroy_dec_config(cfg)


# --------------------------------------------------------------------------------------------------
# Phi-3-medium: LUT-GEMM 3-bit, group 128, with DEC
# --------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("K,N", [(5120, 7680), (17920, 5120)])
def test_dec_lutgemm_at_phi3_shapes(K, N, c_oracle):
    """dec_lutgemm at k_chunk 32 on Phi-3-medium's fused qkv and down projections (17920 has a half-size last
    chunk: 16 picks written at offset 17 * 32)."""
    k_chunk, n_tb, bits, group = 32, 32, 3, 128
    L = make_dec_layer(K, N, seed=K + N)
    q, s, z = F.awq_pseudo_quantize(L["W"], bits, group)
    qw, alpha, q_bias = F.pack_bcq(q, s, z, bits)
    ctx, rows, acts = _ctx(n_tb, K)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dec_lutgemm(cfg, x, out, qw.cuda(), alpha.cuda(), q_bias.cuda(), bits, group)
    base_out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.lutgemm_gemv(x, base_out, qw.cuda(), alpha.cuda(), q_bias.cuda(), bits, group)
    torch.cuda.synchronize()
    xn = np_of(L["x"])
    want_rows, _, filled = O.select_channels(xn, np_of(L["th"]), k_chunk)
    k = k_chunk * K // 1024
    assert filled[:k].all() and np.array_equal(rows.cpu().numpy()[:k], want_rows[:k])
    base = c_oracle.lutgemm_gemv(xn, qw.numpy(), np_of(alpha), np_of(q_bias), bits, group)
    check_output(np_of(base_out).reshape(-1), base, "fp16", ("lutgemm_gemv", K, N))
    want = base + c_oracle.dec_apply(xn, L["cheat"].numpy(), np_of(L["scales"]), want_rows[:k])
    check_output(np_of(out).reshape(-1), want, "fp16", ("dec_lutgemm", K, N))
    ext.destroy_dec_config(cfg)


def test_dec_lutgemm_at_phi3_gate_up(c_oracle):
    """dec_lutgemm at Phi-3-medium's fused gate_up projection, 5120 -> 35840 (70 column segments of 512 outputs),
    k_chunk 32: indices bit-exact and the output against the oracle.  Random packed BCQ words, scales and offsets
    (what the kernel reads; no weight matrix is quantised), random residual words."""
    K, N, k_chunk, bits, group = 5120, 35840, 32, 3, 128
    g = torch.Generator().manual_seed(K + N)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, bits, N), generator=g, dtype=torch.int64).to(torch.int32)
    alpha = (torch.rand(K // group, bits, N, generator=g) * 4e-3 + 1e-3).half()
    q_bias = (torch.randn(K // group, N, generator=g) * 2e-3).half()
    L = _dec_only_layer(K, N, seed=N - K)
    ctx, rows, acts = _ctx(32, K)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dec_lutgemm(cfg, L["x"].cuda(), out, qw.cuda(), alpha.cuda(), q_bias.cuda(), bits, group)
    torch.cuda.synchronize()
    xn = np_of(L["x"])
    k = k_chunk * K // 1024
    want_rows, want_acts, _ = O.select_channels(xn, np_of(L["th"]), k_chunk)
    assert np.array_equal(rows.cpu().numpy()[:k], want_rows[:k])
    assert np.array_equal(np_of(acts)[:k], want_acts[:k].astype(np.float16))
    want = c_oracle.lutgemm_gemv(xn, qw.numpy(), np_of(alpha), np_of(q_bias), bits, group) + \
        c_oracle.dec_apply(xn, L["cheat"].numpy(), np_of(L["scales"]), want_rows[:k])
    check_output(np_of(out).reshape(-1), want, "fp16", ("dec_lutgemm", K, N))
    ext.destroy_dec_config(cfg)


# --------------------------------------------------------------------------------------------------
# Llama-3-70B shapes: DEC indices and output
# --------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("k_chunk", [16, 32])
@pytest.mark.parametrize("K,N", [(28672, 8192), (8192, 28672), (8192, 8192), (8192, 1024)])
def test_dec_at_llama3_70b_shapes(K, N, k_chunk, c_oracle):
    """dec at the 70B linears (28 chunks at the down projection; 3.5 MiB of residual rows per call at k_chunk 32):
    indices bit-exact, output against the oracle, and again from caller-supplied magnitude-sorted indices."""
    L = _dec_only_layer(K, N, seed=K + N + k_chunk)
    ctx, rows, acts = _ctx(32, K)
    cfg = ext.create_dec_config(ctx, k_chunk, L["cheat"], L["scales"], L["th"])
    assert ext.read_dec_config(cfg, native=True)["hip_chunk_groups"] <= 4
    x = L["x"].cuda()
    out = torch.zeros(1, 1, N, dtype=torch.float16, device="cuda")
    ext.dec(cfg, x, out)
    torch.cuda.synchronize()
    xn = np_of(L["x"])
    want_rows, want_acts, _ = O.select_channels(xn, np_of(L["th"]), k_chunk)
    k = k_chunk * K // 1024
    got_rows = rows.cpu().numpy()
    assert np.array_equal(got_rows[:k], want_rows[:k]), "selected channel indices differ from the oracle"
    assert np.array_equal(np_of(acts)[:k], want_acts[:k].astype(np.float16))
    assert (got_rows[k:] == -7).all(), "wrote past the k selected entries"
    want = c_oracle.dec_apply(xn, L["cheat"].numpy(), np_of(L["scales"]), want_rows[:k])
    check_output(np_of(out).reshape(-1), want, "fp16", ("dec", K, N, k_chunk))
    topk = torch.topk(x[0, 0].abs().float(), k).indices.to(torch.int32)
    rows[:k] = topk
    out.zero_()
    ext.unfused_dec(cfg, x, out)
    torch.cuda.synchronize()
    want = c_oracle.dec_apply(xn, L["cheat"].numpy(), np_of(L["scales"]), topk.cpu().numpy())
    check_output(np_of(out).reshape(-1), want, "fp16", ("unfused_dec", K, N, k_chunk))
    ext.destroy_dec_config(cfg)


# --------------------------------------------------------------------------------------------------
# side files -> model -> decode step
# --------------------------------------------------------------------------------------------------
def test_side_files_drive_a_decode_step(tmp_path, c_oracle):
    """cheatsheet.pt / thresholds.pt written per Hugging Face module (q, k, v, o, gate, up, down; the layout of
    decdec_setup/cheatsheet.py and thresholds.py), loaded and fused for the model (end-to-end/loader.py:114-193),
    then one decode step: every compensated linear against the oracle on the activations it saw, using the
    UNFUSED per-module residuals for the expected value."""
    from decdec_amd import generate as G
    from decdec_amd.model import DEC_MODULE_KEYS
    k_chunk = 8
    model = G.build_model("tiny-llama-test", "anyprec", 3, group_size=128, seed=9)
    model.setup_caches(1, 64)
    cfgm = model.config
    hd = cfgm.dim // cfgm.n_head
    dims = {"self_attn.q_proj": (cfgm.dim, cfgm.dim), "self_attn.k_proj": (cfgm.n_local_heads * hd, cfgm.dim),
            "self_attn.v_proj": (cfgm.n_local_heads * hd, cfgm.dim), "self_attn.o_proj": (cfgm.dim, cfgm.dim),
            "mlp.gate_proj": (cfgm.intermediate_size, cfgm.dim), "mlp.up_proj": (cfgm.intermediate_size, cfgm.dim),
            "mlp.down_proj": (cfgm.dim, cfgm.intermediate_size)}
    g = torch.Generator().manual_seed(4)
    layers, ths = [], []
    for _ in range(cfgm.n_layer):
        entry, th = {}, {}
        for name, (n, k) in dims.items():
            err = (torch.randn(n, k, generator=g) * 2e-3).half()
            entry[name] = artifacts.build_cheatsheet_entry(err, torch.zeros_like(err))
            th[name] = F.calibrate_thresholds(k, g, draws=4)
        layers.append(entry); ths.append(th)
    artifacts.save_cheatsheet(str(tmp_path), layers)
    artifacts.save_thresholds(str(tmp_path), ths)
    data = artifacts.load_dec_data(str(tmp_path))
    model.load_dec_data(data)
    model.create_dec_context(8, buffer_size=2048)
    model.set_dec_config([k_chunk] * 4)
    seen, hooks = {}, []
    for i, layer in enumerate(model.layers):
        for key, lin in zip(DEC_MODULE_KEYS, layer.dec_linears()):
            hooks.append(lin.register_forward_hook(
                lambda m, inp, out, name=(i, key): seen.__setitem__(name, (inp[0].detach().clone(), out.detach().clone()))))
    with torch.no_grad():
        model(torch.randint(0, cfgm.vocab_size, (1, 12), device="cuda"), torch.arange(12, device="cuda"))
        seen.clear()
        model(torch.tensor([[5]], device="cuda"), torch.tensor([12], device="cuda"))
        torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    parts = {"attention.wqkv": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"],
             "attention.wo": ["self_attn.o_proj"], "feed_forward.w1w3": ["mlp.gate_proj", "mlp.up_proj"],
             "feed_forward.w2": ["mlp.down_proj"]}
    assert len(seen) == 4 * cfgm.n_layer
    for i, layer in enumerate(model.layers):
        for key, lin in zip(DEC_MODULE_KEYS, layer.dec_linears()):
            x, y = seen[(i, key)]
            xn = np_of(x).reshape(-1)
            rows, _, _ = O.select_channels(xn, np_of(ths[i][parts[key][0]]), k_chunk)
            base = O.anyprec_dequant(lin.qweight.cpu().numpy(), np_of(lin.lut), 3).astype(np.float64) @ xn.astype(np.float64)
            dec = np.concatenate([c_oracle.dec_apply(xn, layers[i][m]["cheatsheet"].numpy(),
                                                     np_of(layers[i][m]["reordered_scales"]), rows) for m in parts[key]])
            check_output(np_of(y).reshape(-1), base + dec, "fp16", (i, key))
