"""Packers and quantisers for the data formats on either side of the DEC path (PyTorch, any device).

These produce the tensors the ops consume -- any-precision bitplanes, LUT-GEMM binary codes,
SqueezeLLM packed indices, and the 4-bit residual ("cheatsheet") with its reordered scales -- from
dense weights, and the calibration thresholds of the channel selector.  Layouts follow the
reference's kernels and offline tools (cited per function); the implementations are vectorised
torch code so that full-size layers can be built on the GPU in milliseconds.
"""
from __future__ import annotations

import torch

CHUNK_SIZE = 1024


def _to_int32(words: torch.Tensor) -> torch.Tensor:
    """Non-negative int64 values below 2^32 -> int32 with the same bit pattern."""
    return torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)


# ------------------------------------------------------------------------------------------------
# any-precision bitplanes (layout of reference decdec_extension/anyprec.cu:297-329, :411-475)
# ------------------------------------------------------------------------------------------------
def anyprec_channel_of(K: int, device=None) -> torch.Tensor:
    """chan[w, b] = input channel stored at bit b of word w of a row.
    Word w = 32 i + t of 1024-channel chunk i holds, at bit 31 - (8 j + e), channel
    1024 i + 8 eff j + 8 t + e with eff = 32 (full chunk) or (K % 1024) / 32 (tail chunk)."""
    assert K % 32 == 0
    W = K // 32
    w = torch.arange(W, device=device)
    i, t = w // 32, w % 32
    eff = torch.where(i == K // 1024, torch.full_like(i, (K % 1024) // 32), torch.full_like(i, 32))
    b = torch.arange(32, device=device)
    j, e = (31 - b) // 8, (31 - b) % 8
    return (1024 * i[:, None] + 8 * eff[:, None] * j[None, :] + 8 * t[:, None] + e[None, :]).long()


def pack_anyprec(idx: torch.Tensor, bits: int) -> torch.Tensor:
    """idx integer [N, K] in [0, 2^bits) -> qweight int32 [bits, N, K/32]; plane 0 = MSB."""
    N, K = idx.shape
    chan = anyprec_channel_of(K, idx.device)                      # [W, 32]
    gathered = idx.long()[:, chan.reshape(-1)].reshape(N, K // 32, 32)
    shifts = torch.arange(32, device=idx.device, dtype=torch.int64)
    planes = []
    for p in range(bits):
        bit = (gathered >> (bits - 1 - p)) & 1
        planes.append(_to_int32((bit << shifts).sum(dim=2)))
    return torch.stack(planes, dim=0).contiguous()


def unpack_anyprec(qweight: torch.Tensor, bits: int) -> torch.Tensor:
    """qweight int32 [>=bits, N, K/32] -> idx int64 [N, K]."""
    _, N, W = qweight.shape
    K = W * 32
    chan = anyprec_channel_of(K, qweight.device).reshape(-1)
    shifts = torch.arange(32, device=qweight.device, dtype=torch.int64)
    acc = torch.zeros((N, W, 32), dtype=torch.int64, device=qweight.device)
    for p in range(bits):
        plane = qweight[p].long() & 0xFFFFFFFF
        acc |= ((plane[:, :, None] >> shifts) & 1) << (bits - 1 - p)
    idx = torch.empty((N, K), dtype=torch.int64, device=qweight.device)
    idx[:, chan] = acc.reshape(N, K)
    return idx


def quantize_uniform_rows(W: torch.Tensor, bits: int):
    """Per-output-row uniform quantiser used to synthesise LUT layers: lut = linspace(min, max)
    in fp16, nearest level.  Returns (idx uint8 [N, K], lut [N, 2^bits] in W's dtype)."""
    W32 = W.float()
    lo = W32.amin(dim=1, keepdim=True)
    hi = W32.amax(dim=1, keepdim=True)
    L = 1 << bits
    steps = torch.arange(L, device=W.device, dtype=torch.float32) / (L - 1)
    lut = (lo + (hi - lo) * steps[None, :]).to(W.dtype)
    step = (hi - lo).clamp_min(1e-12) / (L - 1)
    idx = torch.clamp(torch.round((W32 - lo) / step), 0, L - 1).to(torch.uint8)
    return idx, lut


def dequant_lut(idx: torch.Tensor, lut: torch.Tensor) -> torch.Tensor:
    """W[n, c] = lut[n, idx[n, c]]."""
    return torch.gather(lut, 1, idx.long())


# ------------------------------------------------------------------------------------------------
# SqueezeLLM packed indices (reference decdec_extension/sqllm.cu:64-113, :152-166)
# ------------------------------------------------------------------------------------------------
def pack_sqllm(idx: torch.Tensor, bits: int) -> torch.Tensor:
    """idx integer [N, K] -> int32 [K*bits/32, N].  4-bit: word c/8, field 4 (c%8).
    3-bit: 32 channels = one 96-bit little-endian stream over 3 words, field at bit 3 (c%32)."""
    assert bits in (3, 4)
    N, K = idx.shape
    v = idx.long()
    if bits == 4:
        shifts = 4 * torch.arange(8, device=idx.device, dtype=torch.int64)
        words = (v.reshape(N, K // 8, 8) << shifts).sum(dim=2)
        return _to_int32(words).t().contiguous()
    g = v.reshape(N, K // 32, 32)
    out = torch.zeros((N, K // 32, 3), dtype=torch.int64, device=idx.device)
    for j in range(32):
        w, off = divmod(3 * j, 32)
        out[:, :, w] |= (g[:, :, j] << off) & 0xFFFFFFFF
        if off + 3 > 32:
            out[:, :, w + 1] |= g[:, :, j] >> (32 - off)
    return _to_int32(out.reshape(N, K // 32 * 3)).t().contiguous()


def unpack_sqllm(qweight: torch.Tensor, bits: int) -> torch.Tensor:
    """int32 [K*bits/32, N] -> idx int64 [N, K] (inverse of pack_sqllm)."""
    assert bits in (3, 4)
    w = qweight.long().t() & 0xFFFFFFFF                                       # [N, K*bits/32]
    N = w.shape[0]
    if bits == 4:
        shifts = 4 * torch.arange(8, device=w.device, dtype=torch.int64)
        return ((w[:, :, None] >> shifts) & 0xF).reshape(N, -1)
    g = w.reshape(N, -1, 3)
    out = torch.empty((N, g.shape[1], 32), dtype=torch.int64, device=w.device)
    for j in range(32):
        k, off = divmod(3 * j, 32)
        v = g[:, :, k] >> off
        if off + 3 > 32:
            v = v | (g[:, :, k + 1] << (32 - off))
        out[:, :, j] = v & 7
    return out.reshape(N, -1)


def dequant_sqllm(qweight: torch.Tensor, lut: torch.Tensor, bits: int) -> torch.Tensor:
    """Dense [N, K] weight of a SqueezeLLM layer, in the LUT's dtype (reference evaluation/evaltools.py:583-645)."""
    return dequant_lut(unpack_sqllm(qweight, bits), lut)


# ------------------------------------------------------------------------------------------------
# LUT-GEMM binary-coding format (reference decdec_setup/llm-awq/quantize/qmodule.py:61-92,
# quantizer.py:216-258)
# ------------------------------------------------------------------------------------------------
def awq_pseudo_quantize(W: torch.Tensor, bits: int, group_size: int):
    """Asymmetric uniform group quantisation: returns (q int64 [N, K], scales [N, G], zeros [N, G])."""
    N, K = W.shape
    G = K // group_size
    w = W.float().reshape(N * G, group_size)
    mx, mn = w.amax(dim=1, keepdim=True), w.amin(dim=1, keepdim=True)
    max_int = 2 ** bits - 1
    scales = (mx - mn).clamp(min=1e-5) / max_int
    zeros = (-torch.round(mn / scales)).clamp_(0, max_int)
    q = torch.clamp(torch.round(w / scales) + zeros, 0, max_int)
    return q.reshape(N, K).long(), scales.reshape(N, G), zeros.reshape(N, G)


def pack_bcq(q: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, bits: int, dtype=torch.float16):
    """(q, scales, zeros) -> (q_weight int32 [K/32, bits, N], alpha [G, bits, N], q_bias [G, N]).
    alpha[g, p, n] = scales/2 * 2^p (p = 0 is the LSB), q_bias = sum_p alpha - scales*zeros, and bit
    (c % 32) of q_weight[c/32, p, n] is bit p of q[n, c]; then w = sum_p alpha_p (2 bit_p - 1) + q_bias."""
    N, K = q.shape
    pw = 2.0 ** torch.arange(bits, device=q.device, dtype=torch.float32)
    alpha = (scales / 2.0)[:, :, None] * pw[None, None, :]                    # [N, G, B]
    q_bias = alpha.sum(-1) - scales * zeros                                   # [N, G]
    shifts = torch.arange(32, device=q.device, dtype=torch.int64)
    planes = []
    for p in range(bits):
        b = ((q >> p) & 1).reshape(N, K // 32, 32)
        planes.append(_to_int32((b << shifts).sum(dim=2)))                    # [N, K/32]
    q_weight = torch.stack(planes, dim=1).permute(2, 1, 0).contiguous()       # [K/32, B, N]
    return q_weight, alpha.permute(1, 2, 0).contiguous().to(dtype), q_bias.t().contiguous().to(dtype)


def dequant_bcq(q_weight: torch.Tensor, alpha: torch.Tensor, q_bias: torch.Tensor, group_size: int) -> torch.Tensor:
    """Dense [N, K] float32 weight of a BCQ layer (reference evaluation/evaltools.py:546-580)."""
    KT, B, N = q_weight.shape
    K = KT * 32
    shifts = torch.arange(32, device=q_weight.device, dtype=torch.int64)
    bits_ = ((q_weight.long()[:, :, :, None] & 0xFFFFFFFF) >> shifts) & 1    # [KT, B, N, 32]
    delta = bits_.permute(0, 3, 1, 2).reshape(K, B, N).float() * 2 - 1
    g = torch.arange(K, device=q_weight.device) // group_size
    w = (delta * alpha.float()[g]).sum(dim=1) + q_bias.float()[g]
    return w.t().contiguous()


# ------------------------------------------------------------------------------------------------
# 4-bit residual ("cheatsheet"), reference decdec_setup/cheatsheet.py:59-125
# ------------------------------------------------------------------------------------------------
def quantize_residual(E: torch.Tensor, grid_size: int = 32):
    """Per-output-row symmetric 4-bit quantisation of E [N, K]: 32 candidate scales up to
    max|e|/7, q = clamp(round(e/s), -7, 7), minimum float32 MSE.  Returns (q int8 [N, K],
    scales float16 [N])."""
    E16 = E.to(torch.float16)
    e32 = E16.float()
    max_scale = (E16.abs().amax(dim=1) / 7).float()                          # fp16 division, as the tool does
    start = (E16.abs().amax(dim=1) / 7 / grid_size).float()
    step = (max_scale - start) / (grid_size - 1)
    best_mse = torch.full((E.shape[0],), float("inf"), device=E.device)
    best_q = torch.zeros_like(e32)
    best_s = torch.zeros_like(max_scale)
    for i in range(grid_size):
        s = start + step * i if i < grid_size // 2 else max_scale - step * (grid_size - 1 - i)
        s_col = s[:, None]
        qc = torch.clamp(torch.round(e32 / s_col), -7, 7)
        mse = ((e32 - qc * s_col) ** 2).mean(dim=1)
        better = mse < best_mse
        best_mse = torch.where(better, mse, best_mse)
        best_s = torch.where(better, s, best_s)
        best_q = torch.where(better[:, None], qc, best_q)
    return torch.nan_to_num(best_q).to(torch.int8), best_s.to(torch.float16)


def pack_residual(q: torch.Tensor, scales: torch.Tensor):
    """q int [N, K] in [-7, 7], scales [N] -> (cheatsheet int32 [K, N/8], reordered_scales [N]).
    Nibble j of cheatsheet[c, m] is q[8m + j, c] + 8; reordered_scales[j N/8 + m] = scales[8m + j]."""
    N, K = q.shape
    assert N % 8 == 0
    nib = (q.long() + 8) & 0xF
    shifts = 4 * torch.arange(8, device=q.device, dtype=torch.int64)
    words = (nib.t().reshape(K, N // 8, 8) << shifts).sum(dim=2)
    reordered = scales.reshape(N // 8, 8).t().reshape(-1).contiguous()
    return _to_int32(words).contiguous(), reordered


def unpack_residual(cheatsheet: torch.Tensor, reordered_scales: torch.Tensor) -> torch.Tensor:
    """Dense dequantised residual [K, N] in float32."""
    K, M = cheatsheet.shape
    shifts = 4 * torch.arange(8, device=cheatsheet.device, dtype=torch.int64)
    nib = ((cheatsheet.long()[:, :, None] & 0xFFFFFFFF) >> shifts) & 0xF
    sc = reordered_scales.float().reshape(8, M).t()
    return ((nib - 8).float() * sc[None]).reshape(K, M * 8)


# ------------------------------------------------------------------------------------------------
# activations and selector thresholds
# ------------------------------------------------------------------------------------------------
def make_activation(K: int, generator: torch.Generator, dtype=torch.float16, device="cpu",
                    outlier_frac: float = 0.01, outlier_scale: float = 20.0) -> torch.Tensor:
    """x ~ N(0, 1) with a random 1 % of the channels scaled x20; shape [1, 1, K]."""
    x = torch.randn(K, generator=generator, dtype=torch.float32)
    n_out = max(1, int(round(K * outlier_frac)))
    pos = torch.randperm(K, generator=generator)[:n_out]
    x[pos] *= outlier_scale
    return x.to(dtype).reshape(1, 1, K).to(device)


def calibrate_thresholds(K: int, generator: torch.Generator, draws: int = 64, dtype=torch.float16) -> torch.Tensor:
    """thresholds[i] = max over calibration vectors of the i-th largest |x|
    (reference decdec_setup/thresholds.py:162-175).  CPU tensor [K]."""
    th = torch.zeros(K, dtype=torch.float32)
    for _ in range(draws):
        x = make_activation(K, generator, dtype=dtype).float().reshape(-1)
        th = torch.maximum(th, torch.sort(x.abs(), descending=True).values)
    return th.to(dtype)
