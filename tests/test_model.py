"""Decode harness pieces that need no GPU: the decoder's cache / RoPE logic on dense fp32 linears, the model
table, and the DEC side-file formats."""
import math

import numpy as np
import pytest
import torch
import torch.nn as nn

from decdec_amd import artifacts, formats as F
from decdec_amd.model import ModelArgs, Transformer, apply_rope, rope_tables, RMSNorm
from oracle import decdec_oracle as O


def _dense_model(seed=0):
    torch.manual_seed(seed)
    cfg = ModelArgs.from_name("tiny-llama-test")
    m = Transformer(torch.float32, cfg, linear_class=nn.Linear,
                    linear_kwargs={"dtype": torch.float32, "device": "cpu"}, device="cpu")
    m.setup_caches(1, 64)
    return m, cfg


def test_model_table_matches_reference_shapes():
    # reference autotuner/README.md:56-60: fused qkv and gate_up widths of the three models
    for name, qkv, gu in (("Meta-Llama-3-8B-Instruct", 6144, 28672), ("Phi-3-medium-4k-instruct", 7680, 35840),
                          ("Meta-Llama-3-70B-Instruct", 10240, 57344)):
        c = ModelArgs.from_name(name)
        assert (c.n_head + 2 * c.n_local_heads) * c.head_dim == qkv
        assert 2 * c.intermediate_size == gu
    with pytest.raises(KeyError):
        ModelArgs.from_name("no-such-model")


def test_cached_decode_equals_full_causal_forward():
    m, cfg = _dense_model()
    tok = torch.randint(0, cfg.vocab_size, (1, 12))
    with torch.no_grad():
        full = m(tok, torch.arange(12))
        for b in m.layers:
            b.attention.kv_cache.k_cache.zero_(); b.attention.kv_cache.v_cache.zero_()
        outs = [m(tok[:, :8], torch.arange(8))[:, -1]]
        for t in range(8, 12):
            outs.append(m(tok[:, t:t + 1], torch.tensor([t]))[:, -1])
    assert torch.allclose(torch.stack(outs, 1), full[:, 7:], atol=1e-5)


def test_future_tokens_do_not_leak():
    m, cfg = _dense_model(1)
    a = torch.randint(0, cfg.vocab_size, (1, 10))
    b = a.clone(); b[0, 7:] = (b[0, 7:] + 1) % cfg.vocab_size
    with torch.no_grad():
        ya, yb = m(a, torch.arange(10)), m(b, torch.arange(10))
    assert torch.allclose(ya[:, :7], yb[:, :7], atol=1e-6) and not torch.allclose(ya[:, 7:], yb[:, 7:])


def test_rope_is_a_rotation_by_position_times_frequency():
    D, P, base = 16, 32, 10000.0
    cos, sin = rope_tables(D, P, base)
    x = torch.randn(1, 2, P, D)
    y = apply_rope(x, cos, sin)
    # closed form: complex multiplication of (x_i + i x_{i+D/2}) by exp(i pos base^(-2i/D))
    z = torch.complex(x[..., :D // 2], x[..., D // 2:])
    ang = torch.arange(P)[:, None] * (base ** (-torch.arange(0, D, 2) / D))[None, :]
    w = z * torch.polar(torch.ones_like(ang), ang)
    assert torch.allclose(y, torch.cat((w.real, w.imag), -1), atol=1e-5)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-5)
    # relative-position property: <rope(q, m), rope(k, n)> depends on m - n only
    q, k = torch.randn(D), torch.randn(D)
    rq = apply_rope(q.expand(1, 1, P, D), cos, sin)[0, 0]
    rk = apply_rope(k.expand(1, 1, P, D), cos, sin)[0, 0]
    assert math.isclose(float(rq[5] @ rk[2]), float(rq[20] @ rk[17]), rel_tol=1e-4, abs_tol=1e-4)


def test_rmsnorm():
    n = RMSNorm(8, eps=0.0)
    x = torch.randn(3, 8)
    assert torch.allclose(n(x).pow(2).mean(-1), torch.ones(3), atol=1e-5)


# ---- side files -------------------------------------------------------------------------------------
def _entry(N, K, seed):
    g = torch.Generator().manual_seed(seed)
    W = (torch.randn(N, K, generator=g) * 0.02).half()
    idx, lut = F.quantize_uniform_rows(W, 3)
    return W, F.dequant_lut(idx, lut), artifacts.build_cheatsheet_entry(W, F.dequant_lut(idx, lut))


def test_cheatsheet_entry_matches_oracle_quantiser_and_bounds_the_error():
    W, Wq, e = _entry(16, 64, 0)
    err = (W - Wq).half()
    q, s = O.quantize_residual(err.numpy())
    cheat, reordered = O.pack_residual(q, s)
    assert np.array_equal(e["cheatsheet"].numpy(), cheat) and np.array_equal(e["reordered_scales"].numpy(), reordered)
    dense = F.unpack_residual(e["cheatsheet"], e["reordered_scales"]).t()          # [N, K]
    sc = artifacts.natural_scales(e["reordered_scales"]).float()[:, None]
    inside = (err.float().abs() <= 7.5 * sc)                                        # not clamped
    assert torch.all(((dense - err.float()).abs() <= sc / 2 + 1e-6) | ~inside)


def test_fused_entry_is_the_residual_of_the_concatenated_module():
    parts = [_entry(n, 64, s)[2] for n, s in ((32, 1), (8, 2), (16, 3))]
    fused = artifacts.fuse_entries(parts)
    want = torch.cat([F.unpack_residual(p["cheatsheet"], p["reordered_scales"]) for p in parts], dim=1)
    got = F.unpack_residual(fused["cheatsheet"], fused["reordered_scales"])
    assert torch.equal(got, want)
    # joining the reordered vectors end to end is NOT the same thing
    naive = torch.cat([p["reordered_scales"] for p in parts])
    assert not torch.equal(naive, fused["reordered_scales"])
    assert torch.equal(artifacts.reorder_scales(artifacts.natural_scales(naive)), naive)


def test_side_files_round_trip(tmp_path):
    names = ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
             "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj"]
    dims = {"self_attn.q_proj": (32, 32), "self_attn.k_proj": (8, 32), "self_attn.v_proj": (8, 32),
            "self_attn.o_proj": (32, 32), "mlp.gate_proj": (64, 32), "mlp.up_proj": (64, 32), "mlp.down_proj": (32, 64)}
    layers = [{n: _entry(*dims[n], seed=10 * l + i)[2] for i, n in enumerate(names)} for l in range(2)]
    ths = [{n: torch.rand(dims[n][1]).sort(descending=True).values.half() for n in names} for _ in range(2)]
    artifacts.save_cheatsheet(str(tmp_path), layers)
    artifacts.save_thresholds(str(tmp_path), ths)
    d = artifacts.load_dec_data(str(tmp_path))
    assert len(d) == 2 * 4 * 3
    assert d["layers.1.attention.wqkv.q_residual"].shape == (32, 6) and d["layers.1.attention.wqkv.q_residual"].dtype == torch.int32
    assert d["layers.0.feed_forward.w1w3.scales"].shape == (128,)
    assert torch.equal(d["layers.1.feed_forward.w2.q_residual"], layers[1]["mlp.down_proj"]["cheatsheet"])
    assert torch.equal(d["layers.0.attention.wqkv.thresholds"], ths[0]["self_attn.q_proj"])
    assert torch.equal(d["layers.0.attention.wo.scales"], layers[0]["self_attn.o_proj"]["reordered_scales"])


def test_threshold_collector_is_the_running_max_of_sorted_magnitudes():
    lin = nn.Linear(16, 4)
    xs = [torch.randn(1, 5, 16), torch.randn(1, 3, 16)]
    th = artifacts.collect_thresholds([("m", lin)], lambda: [lin(x) for x in xs], dtype=torch.float32)["m"]
    allx = torch.cat([x.reshape(-1, 16) for x in xs]).abs()
    want = torch.stack([torch.sort(r, descending=True).values for r in allx]).amax(0)
    assert torch.equal(th, want)
    assert torch.all(th[:-1] >= th[1:])


def test_prefill_longer_than_the_cache_is_refused():
    """More prompt positions than cache rows must fail on the host, not index outside the mask on the device."""
    model, _ = _dense_model()                       # 64 cache rows
    with pytest.raises(AssertionError, match="do not fit a cache"):
        model(torch.zeros(1, 80, dtype=torch.int64), torch.arange(80))
