"""Decode-step helper kernels against plain fp32 torch references (these are floating-point kernels; the
tolerance is the rounding of their 16-bit outputs)."""
import math

import pytest
import torch

from decdec_amd import _lib, decode_ops as D, generate as G
from decdec_amd.model import apply_rope, rope_tables

pytestmark = pytest.mark.gpu


def _close(got, want, rtol):
    got, want = got.float(), want.float()
    return float((got - want).abs().max()) <= rtol * float(want.abs().max()) + 1e-6


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,Hkv,hd", [(8, 2, 64), (32, 8, 128), (4, 4, 128)])
def test_rope_cache_update(H, Hkv, hd, dt):
    S = 96
    g = torch.Generator(device="cuda").manual_seed(0)
    cos, sin = rope_tables(hd, S, 10000.0, "cuda")
    cos16, sin16 = cos.to(dt), sin.to(dt)
    kc = torch.randn(1, Hkv, S, hd, generator=g, device="cuda").to(dt)
    vc = torch.randn(1, Hkv, S, hd, generator=g, device="cuda").to(dt)
    for pos in (0, 5, S - 1):
        qkv = torch.randn((H + 2 * Hkv) * hd, generator=g, device="cuda").to(dt)
        k0, v0 = kc.clone(), vc.clone()
        q_out = torch.empty(H * hd, dtype=dt, device="cuda")
        p = torch.tensor([pos], device="cuda")
        D.rope_cache_update(qkv, cos16, sin16, p, q_out, kc, vc, H, Hkv)
        heads = qkv.float().view(H + 2 * Hkv, hd)
        want = apply_rope(heads[:H + Hkv].view(1, H + Hkv, 1, hd), cos16[pos:pos + 1].float(), sin16[pos:pos + 1].float())[0, :, 0]
        rt = 2e-2 if dt == torch.bfloat16 else 3e-3
        assert _close(q_out.view(H, hd), want[:H], rt)
        assert _close(kc[0, :, pos], want[H:], rt)
        assert torch.equal(vc[0, :, pos], heads[H + Hkv:].to(dt))
        keep = torch.ones(S, dtype=torch.bool, device="cuda"); keep[pos] = False
        assert torch.equal(kc[0][:, keep], k0[0][:, keep]) and torch.equal(vc[0][:, keep], v0[0][:, keep])
    k0, v0 = kc.clone(), vc.clone()
    for bad in (-1, S, S + 7):
        D.rope_cache_update(qkv, cos16, sin16, torch.tensor([bad], device="cuda"), q_out, kc, vc, H, Hkv)
    torch.cuda.synchronize()
    assert torch.equal(kc, k0) and torch.equal(vc, v0)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,Hkv,hd,S", [(8, 2, 64, 256), (32, 8, 128, 2048), (4, 4, 128, 80), (40, 10, 128, 520)])
def test_decode_attention(H, Hkv, hd, S, dt):
    g = torch.Generator(device="cuda").manual_seed(1)
    kc = torch.randn(1, Hkv, S, hd, generator=g, device="cuda").to(dt)
    vc = torch.randn(1, Hkv, S, hd, generator=g, device="cuda").to(dt)
    ws = D.attention_workspace(H, hd)
    for pos in sorted({0, 1, 15, 16, 63, 64, S // 2 + 3, S - 1}):
        q = (torch.randn(H * hd, generator=g, device="cuda") * 1.5).to(dt)
        out = torch.empty(H * hd, dtype=dt, device="cuda")
        D.decode_attention(q, kc, vc, torch.tensor([pos], device="cuda"), out, H, Hkv)
        # with a workspace: positions shared by up to 8 workgroups per head, short sequences (<= 512 positions by
        # default) scanned by the head's first workgroup alone; with the option at 0 every length is shared
        out_s, out_a = (torch.empty(H * hd, dtype=dt, device="cuda") for _ in range(2))
        D.decode_attention(q, kc, vc, torch.tensor([pos], device="cuda"), out_a, H, Hkv, ws)
        _lib.set_option("attention_single_below", 0)
        try:
            D.decode_attention(q, kc, vc, torch.tensor([pos], device="cuda"), out_s, H, Hkv, ws)
        finally:
            _lib.set_option("attention_single_below", 512)
        k = kc[0, :, :pos + 1].float().repeat_interleave(H // Hkv, dim=0)       # [H, L, hd]
        v = vc[0, :, :pos + 1].float().repeat_interleave(H // Hkv, dim=0)
        att = torch.softmax(torch.einsum("hd,hld->hl", q.float().view(H, hd), k) / math.sqrt(hd), dim=-1)
        want = torch.einsum("hl,hld->hd", att, v)
        assert _close(out.view(H, hd), want, 2e-2 if dt == torch.bfloat16 else 3e-3), (pos,)
        assert _close(out_s.view(H, hd), want, 2e-2 if dt == torch.bfloat16 else 3e-3), (pos, "split")
        assert _close(out_a.view(H, hd), want, 2e-2 if dt == torch.bfloat16 else 3e-3), (pos, "split or alone")
    # a position beyond the cache attends the whole cache and reads nothing outside it
    D.decode_attention(q, kc, vc, torch.tensor([S + 100], device="cuda"), out, H, Hkv)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,Hkv,hd,S", [(8, 2, 64, 256), (32, 8, 128, 2048), (4, 4, 128, 80), (40, 10, 128, 520)])
def test_rope_attention_equals_the_two_step_form(H, Hkv, hd, S, dt):
    """One launch for rotary embedding + cache append + attention against rope_cache_update followed by
    decode_attention (with and without the workspace) and against fp32 torch: same values row and same output to
    within rounding (a rotated value that sits within fp32 rounding error of a 16-bit tie may be rounded either
    way by either kernel), nothing but the new row touched."""
    g = torch.Generator(device="cuda").manual_seed(2)
    cos, sin = rope_tables(hd, S, 10000.0, "cuda")
    cos16, sin16 = cos.to(dt), sin.to(dt)
    kc = torch.randn(1, Hkv, S, hd, generator=g, device="cuda").to(dt)
    vc = torch.randn(1, Hkv, S, hd, generator=g, device="cuda").to(dt)
    ws = D.attention_workspace(H, hd)
    for pos in sorted({0, 1, 15, 16, 63, 64, S // 2 + 3, S - 1}):
        qkv = (torch.randn((H + 2 * Hkv) * hd, generator=g, device="cuda") * 1.5).to(dt)
        p = torch.tensor([pos], device="cuda")
        k2, v2 = kc.clone(), vc.clone()
        q_rot = torch.empty(H * hd, dtype=dt, device="cuda")
        want = torch.empty(H * hd, dtype=dt, device="cuda")
        D.rope_cache_update(qkv, cos16, sin16, p, q_rot, k2, v2, H, Hkv)
        D.decode_attention(q_rot, k2, v2, p, want, H, Hkv)
        for w in (None, ws):
            k1, v1 = kc.clone(), vc.clone()
            out = torch.empty(H * hd, dtype=dt, device="cuda")
            D.rope_attention(qkv, cos16, sin16, p, out, k1, v1, H, Hkv, w)
            torch.cuda.synchronize()
            assert torch.equal(v1, v2), (pos, w is not None)
            keep = torch.ones(S, dtype=torch.bool, device="cuda"); keep[pos] = False
            assert torch.equal(k1[0][:, keep], kc[0][:, keep]), pos
            ulp = 2.0 ** -7 if dt == torch.bfloat16 else 2.0 ** -10       # one unit in the last place, relative
            assert float(((k1 - k2).float().abs() / k2.float().abs().clamp_min(1e-3)).max()) <= ulp, pos
            assert int((k1 != k2).sum()) <= 4, pos
            assert _close(out, want, 2e-2 if dt == torch.bfloat16 else 3e-3), pos
        # fp32 torch on the rotated query and the updated cache
        k = k2[0, :, :pos + 1].float().repeat_interleave(H // Hkv, dim=0)
        v = v2[0, :, :pos + 1].float().repeat_interleave(H // Hkv, dim=0)
        att = torch.softmax(torch.einsum("hd,hld->hl", q_rot.float().view(H, hd), k) / math.sqrt(hd), dim=-1)
        ref = torch.einsum("hl,hld->hd", att, v)
        assert _close(out.view(H, hd), ref, 2e-2 if dt == torch.bfloat16 else 3e-3), pos
        kc, vc = k2, v2                                         # keep appending
    # a position outside the cache appends nothing and reads nothing outside it
    k0, v0 = kc.clone(), vc.clone()
    for bad in (-1, S, S + 100):
        D.rope_attention(qkv, cos16, sin16, torch.tensor([bad], device="cuda"), out, kc, vc, H, Hkv, ws)
    torch.cuda.synchronize()
    assert torch.equal(kc, k0) and torch.equal(vc, v0) and torch.isfinite(out.float()).all()


@pytest.mark.parametrize("H,Hkv,hd,S", [(32, 8, 128, 2048), (40, 10, 128, 1100)])
def test_attention_ranges_merged_in_kernel_over_many_calls(H, Hkv, hd, S):
    """The workgroup of a head that finishes last merges the head's ranges from results the others left in the
    workspace (no second kernel, no fence): several hundred calls in a row at random positions against the
    one-workgroup-per-head form, then the two-step form on the same workspace; the counters end at zero."""
    from decdec_amd import _lib
    g = torch.Generator(device="cuda").manual_seed(7)
    kc = torch.randn(1, Hkv, S, hd, generator=g, device="cuda").half()
    vc = torch.randn(1, Hkv, S, hd, generator=g, device="cuda").half()
    ws = D.attention_workspace(H, hd)
    one, many = (torch.empty(H * hd, dtype=torch.float16, device="cuda") for _ in range(2))
    positions = torch.randint(0, S, (400,), generator=g, device="cuda").tolist()
    try:
        for i, pos in enumerate(positions):
            if i == 100:
                _lib.set_option("attention_single_below", 0)      # from here on every length is shared
            if i == 300:
                _lib.set_option("attention_two_step", 1)
            q = (torch.randn(H * hd, generator=g, device="cuda") * 1.5).half()
            p = torch.tensor([pos], device="cuda")
            D.decode_attention(q, kc, vc, p, one, H, Hkv)
            D.decode_attention(q, kc, vc, p, many, H, Hkv, ws)
            assert _close(many, one, 3e-3), (i, pos)
    finally:
        _lib.set_option("attention_two_step", 0)
        _lib.set_option("attention_single_below", 512)
    assert int(ws.view(torch.int32)[:H].abs().sum()) == 0


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,K", [(640, 512), (1001, 4096), (32064, 5120), (7, 8), (130, 1032), (4099, 8192)])
def test_dense_gemv(N, K, dt):
    g = torch.Generator().manual_seed(N + K)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dt).cuda()
    x = torch.randn(K, generator=g).to(dt).cuda()
    out = torch.full((N,), 3.0, dtype=dt, device="cuda")
    D.dense_gemv(w, x, out)
    want = w.double() @ x.double()
    # one rounding of an fp32 sum: half a unit in the last place of the result plus the fp32 accumulation error
    ulp = 2.0 ** (-11 if dt == torch.float16 else -8)
    tol = ulp * want.abs() + 1e-5 * (w.double().abs() @ x.double().abs())
    assert bool(((out.double() - want).abs() <= 1.001 * tol).all()), float(((out.double() - want).abs() / tol).max())


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 12, 255, 1028, 14336, 17920])
def test_silu_mul(n, dt):
    gu = (torch.randn(2 * n, device="cuda") * 3).to(dt)
    out = torch.full((n,), 9.0, dtype=dt, device="cuda")
    D.silu_mul(gu, out)
    want = torch.nn.functional.silu(gu[:n].float()) * gu[n:].float()
    assert _close(out, want, 2e-3 if dt == torch.float16 else 1.6e-2)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,dim", [(1, 4096), (1, 512), (3, 5120), (2, 8192), (1, 68), (2, 14336)])
def test_add_rmsnorm(rows, dim, dt):
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn(rows, dim, generator=g, device="cuda").to(dt)
    y = (torch.randn(rows, dim, generator=g, device="cuda") * 0.5).to(dt)
    w = (1 + 0.1 * torch.randn(dim, generator=g, device="cuda")).to(dt)
    h, n = torch.empty_like(x), torch.empty_like(x)
    D.add_rmsnorm(x, y, w, h, n, 1e-5)
    want_h = (x.float() + y.float()).to(dt)
    assert torch.equal(h, want_h)
    hf = want_h.float()
    want_n = hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + 1e-5) * w.float()
    assert _close(n, want_n, 2e-2 if dt == torch.bfloat16 else 3e-3)
    n2 = torch.empty_like(x)
    D.add_rmsnorm(x, None, w, None, n2, 1e-5)
    xf = x.float()
    assert _close(n2, xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5) * w.float(), 2e-2 if dt == torch.bfloat16 else 3e-3)


def test_argument_checks():
    a = torch.zeros(8, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="twice as many"):
        D.silu_mul(a, a)
    with pytest.raises(RuntimeError, match="fp16 / bf16"):
        D.silu_mul(torch.zeros(16, device="cuda"), torch.zeros(8, device="cuda"))
    kc = torch.zeros(1, 2, 16, 32, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="head_dim must be 64 or 128"):
        D.decode_attention(torch.zeros(4 * 32, dtype=torch.float16, device="cuda"), kc, kc.clone(),
                           torch.tensor([0], device="cuda"), torch.zeros(4 * 32, dtype=torch.float16, device="cuda"), 4, 2)


def test_decode_step_on_helper_kernels_equals_the_torch_path():
    model = G.build_model("tiny-llama-test", "sqllm", 4, seed=9)
    model.setup_caches(1, 64)
    assert model.decode_kernels
    prompt = torch.randint(0, model.config.vocab_size, (1, 30), device="cuda")
    outs = {}
    for use in (True, False):
        model.decode_kernels = use
        for b in model.layers:
            b.attention.kv_cache.k_cache.zero_(); b.attention.kv_cache.v_cache.zero_()
        with torch.no_grad():
            model(prompt, torch.arange(30, device="cuda"))
            ys = [model(torch.tensor([[t]], device="cuda"), torch.tensor([30 + i], device="cuda")).float().clone()
                  for i, t in enumerate((3, 99, 250))]
        outs[use] = torch.stack(ys)
    assert _close(outs[True], outs[False], 1e-2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_greedy_pick_matches_argmax_and_keeps_the_books(dtype):
    ws = D.greedy_pick_workspace()
    g = torch.Generator().manual_seed(5)
    for n in (1, 7, 255, 4097, 32000, 128256):
        logits = torch.randn(n, generator=g).to(dtype).cuda()
        token = torch.full((1, 1), -1, dtype=torch.int64, device="cuda")
        seq = torch.full((4,), -1, dtype=torch.int64, device="cuda")
        count = torch.tensor([2], dtype=torch.int64, device="cuda")
        pos = torch.tensor([41], dtype=torch.int64, device="cuda")
        copy = torch.zeros(n, dtype=torch.float32, device="cuda")
        D.greedy_pick(logits, ws, token, seq, count, pos, copy)
        torch.cuda.synchronize()
        want = int(torch.argmax(logits.float()))
        assert float(logits[int(token)]) == float(logits[want])           # equal logits: any of them for torch
        assert int(token) == int((logits == logits[want]).nonzero()[0])   # the smallest index here
        assert seq.tolist() == [-1, -1, int(token), -1] and int(count) == 3 and int(pos) == 42
        assert torch.equal(copy, logits.float())
    # ties, a full sequence buffer, a NaN, optional arguments left out
    logits = torch.zeros(1000, dtype=dtype, device="cuda")
    logits[[17, 400, 999]] = 3.0
    token = torch.zeros(1, dtype=torch.int64, device="cuda")
    seq = torch.full((2,), -1, dtype=torch.int64, device="cuda")
    count = torch.tensor([2], dtype=torch.int64, device="cuda")
    D.greedy_pick(logits, ws, token, seq, count)
    torch.cuda.synchronize()
    assert int(token) == 17 and seq.tolist() == [-1, -1] and int(count) == 3
    logits[500] = float("nan")
    D.greedy_pick(logits, ws, token)
    torch.cuda.synchronize()
    assert int(token) == 500 == int(torch.argmax(logits))
    logits = -torch.rand(300, device="cuda").to(dtype) - 1.0          # all negative
    D.greedy_pick(logits, ws, token)
    torch.cuda.synchronize()
    assert int(token) == int((logits == logits.max()).nonzero()[0])
    with pytest.raises(RuntimeError):
        D.greedy_pick(logits, ws, token, seq)                        # seq without count
    with pytest.raises(RuntimeError):
        D.greedy_pick(logits, ws, token.int())
