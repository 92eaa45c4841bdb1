"""Decode-step helpers of the library (rotary embedding + KV-cache append, one-token grouped-query
attention, gated activation) as functions on torch tensors.  They raise if the HIP library is missing;
there is no fallback."""
from __future__ import annotations

import torch

from . import _lib
from .ext import _check, _dt, _ptr, _stream


def _half_cuda(*ts):
    for t in ts:
        _check(t.is_cuda and t.is_contiguous(), "tensors must be contiguous CUDA tensors")
        _check(t.dtype == ts[0].dtype and t.dtype in (torch.float16, torch.bfloat16), "tensors must share an fp16 / bf16 dtype")


def rope_cache_update(qkv: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor, pos: torch.Tensor,
                      q_out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, n_head: int, n_kv_head: int) -> None:
    """qkv [(n_head + 2 n_kv_head) * D]; tables [max_seq, D]; pos int64 [1] on the device; caches [1, n_kv_head, max_seq, D]."""
    _half_cuda(qkv, cos_table, sin_table, q_out, k_cache, v_cache)
    _check(pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1, "pos must be one int64 on the device")
    D, max_seq = k_cache.shape[-1], k_cache.shape[-2]
    _check(qkv.numel() == (n_head + 2 * n_kv_head) * D and q_out.numel() == n_head * D, "qkv / q_out size mismatch")
    _check(k_cache.numel() == n_kv_head * max_seq * D and v_cache.shape == k_cache.shape, "cache shape mismatch")
    _check(tuple(cos_table.shape) == (max_seq, D) and tuple(sin_table.shape) == (max_seq, D), "rotary tables must be [max_seq, head_dim]")
    _lib.check(_lib.load().decdec_rope_cache_update(_ptr(qkv), _ptr(cos_table), _ptr(sin_table), _ptr(pos), _ptr(q_out),
                                                    _ptr(k_cache), _ptr(v_cache), _dt(qkv), n_head, n_kv_head, D, max_seq, _stream()))


def attention_workspace(n_head: int, head_dim: int, device="cuda") -> torch.Tensor:
    """Workspace that lets `decode_attention` / `rope_attention` share the positions of a head among up to 8
    workgroups.  It must be zero when first used (it starts with the heads' arrival counters, which every call leaves
    at zero)."""
    n = _lib.load().decdec_decode_attention_workspace_bytes(n_head, head_dim, 8)
    return torch.zeros(n // 4, dtype=torch.float32, device=device)


def decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, pos: torch.Tensor,
                     out: torch.Tensor, n_head: int, n_kv_head: int, workspace: torch.Tensor | None = None) -> None:
    _half_cuda(q, k_cache, v_cache, out)
    _check(pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1, "pos must be one int64 on the device")
    D, max_seq = k_cache.shape[-1], k_cache.shape[-2]
    _check(q.numel() == n_head * D and out.numel() == n_head * D, "q / out size mismatch")
    _check(k_cache.numel() == n_kv_head * max_seq * D and v_cache.shape == k_cache.shape, "cache shape mismatch")
    if workspace is not None:
        _check(workspace.is_cuda and workspace.is_contiguous() and workspace.dtype == torch.float32, "workspace must be a contiguous float32 CUDA tensor")
    _lib.check(_lib.load().decdec_decode_attention(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(pos), _ptr(out), _dt(q),
                                                   n_head, n_kv_head, D, max_seq,
                                                   _ptr(workspace) if workspace is not None else None,
                                                   workspace.numel() * 4 if workspace is not None else 0, _stream()))


def decode_attention_static(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, pos: torch.Tensor,
                            out: torch.Tensor, n_head: int, n_kv_head: int) -> None:
    """`decode_attention` with the library's own static workspace: nothing is allocated and no workspace is passed
    (at most 128 heads; calls on one GPU must not overlap in time)."""
    _half_cuda(q, k_cache, v_cache, out)
    _check(pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1, "pos must be one int64 on the device")
    D, max_seq = k_cache.shape[-1], k_cache.shape[-2]
    _check(q.numel() == n_head * D and out.numel() == n_head * D, "q / out size mismatch")
    _check(k_cache.numel() == n_kv_head * max_seq * D and v_cache.shape == k_cache.shape, "cache shape mismatch")
    _lib.check(_lib.load().decdec_decode_attention_static(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(pos), _ptr(out),
                                                          _dt(q), n_head, n_kv_head, D, max_seq, _stream()))


def rope_attention(qkv: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor, pos: torch.Tensor,
                   out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, n_head: int, n_kv_head: int,
                   workspace: torch.Tensor | None = None) -> None:
    """`rope_cache_update` + `decode_attention` in one launch: un-rotated qkv in, attention output out, the new key /
    value row appended to the caches."""
    _half_cuda(qkv, cos_table, sin_table, out, k_cache, v_cache)
    _check(pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1, "pos must be one int64 on the device")
    D, max_seq = k_cache.shape[-1], k_cache.shape[-2]
    _check(qkv.numel() == (n_head + 2 * n_kv_head) * D and out.numel() == n_head * D, "qkv / out size mismatch")
    _check(k_cache.numel() == n_kv_head * max_seq * D and v_cache.shape == k_cache.shape, "cache shape mismatch")
    _check(tuple(cos_table.shape) == (max_seq, D) and tuple(sin_table.shape) == (max_seq, D), "rotary tables must be [max_seq, head_dim]")
    if workspace is not None:
        _check(workspace.is_cuda and workspace.is_contiguous() and workspace.dtype == torch.float32, "workspace must be a contiguous float32 CUDA tensor")
    _lib.check(_lib.load().decdec_rope_attention(_ptr(qkv), _ptr(cos_table), _ptr(sin_table), _ptr(pos), _ptr(out),
                                                 _ptr(k_cache), _ptr(v_cache), _dt(qkv), n_head, n_kv_head, D, max_seq,
                                                 _ptr(workspace) if workspace is not None else None,
                                                 workspace.numel() * 4 if workspace is not None else 0, _stream()))


def dense_gemv(weight: torch.Tensor, x: torch.Tensor, out: torch.Tensor) -> None:
    """out[n] = sum_k weight[n, k] * x[k] for an unquantised fp16 / bf16 weight [N, K] (overwrites out)."""
    _half_cuda(weight, x, out)
    _check(weight.dim() == 2 and x.numel() == weight.shape[1] and out.numel() == weight.shape[0],
           "weight [N, K], x with K and out with N elements")
    _lib.check(_lib.load().decdec_dense_gemv(_ptr(weight), _ptr(x), _ptr(out), _dt(out), weight.shape[0],
                                             weight.shape[1], _stream()))


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _half_cuda(gate_up, out)
    _check(gate_up.numel() == 2 * out.numel(), "gate_up must hold twice as many elements as out")
    _lib.check(_lib.load().decdec_silu_mul(_ptr(gate_up), _ptr(out), _dt(out), out.numel(), _stream()))


def add_rmsnorm(x: torch.Tensor, y, weight: torch.Tensor, h_out, normed_out: torch.Tensor, eps: float) -> None:
    """Rows of x [..., dim]: h = x + y (written to h_out; y = h_out = None: h = x), normed_out = rmsnorm(h) * weight."""
    ts = [t for t in (x, y, weight, h_out, normed_out) if t is not None]
    _half_cuda(*ts)
    dim = x.shape[-1]
    _check(weight.numel() == dim and normed_out.shape == x.shape, "weight / normed_out shape mismatch")
    _check((y is None) == (h_out is None) and (y is None or (y.shape == x.shape and h_out.shape == x.shape)),
           "y and h_out go together and have the shape of x")
    _lib.check(_lib.load().decdec_add_rmsnorm(_ptr(x), _ptr(y) if y is not None else None, _ptr(weight),
                                              _ptr(h_out) if h_out is not None else None, _ptr(normed_out), _dt(x),
                                              x.numel() // dim, dim, float(eps), _stream()))



def greedy_pick_workspace(device="cuda") -> torch.Tensor:
    """Workspace of `greedy_pick` (contents irrelevant; one serves any number of calls that do not overlap)."""
    return torch.empty(int(_lib.load().decdec_greedy_pick_workspace_bytes()) // 8, dtype=torch.int64, device=device)


def greedy_pick(logits: torch.Tensor, workspace: torch.Tensor, token: torch.Tensor, seq=None, count=None, pos=None,
                logits_f32_out=None) -> None:
    """token[0] = argmax(logits) (smallest index among equal logits); seq[count[0]] = it and count[0] += 1 when seq and
    count are given; pos[0] += 1 when pos is given; logits_f32_out receives the logits as fp32 when given.  token, seq,
    count and pos are int64 tensors on the device."""
    _check(logits.is_cuda and logits.is_contiguous() and logits.dtype in (torch.float16, torch.bfloat16, torch.float32),
           "logits must be a contiguous fp16 / bf16 / fp32 CUDA tensor")
    for t in (token, seq, count, pos):
        _check(t is None or (t.is_cuda and t.is_contiguous() and t.dtype == torch.int64 and t.numel() >= 1),
               "token, seq, count and pos must be int64 CUDA tensors")
    _check((seq is None) == (count is None), "seq and count go together")
    _check(workspace.is_cuda and workspace.numel() * workspace.element_size() >= int(_lib.load().decdec_greedy_pick_workspace_bytes()),
           "workspace too small")
    _check(logits_f32_out is None or (logits_f32_out.is_cuda and logits_f32_out.is_contiguous() and
                                      logits_f32_out.dtype == torch.float32 and logits_f32_out.numel() >= logits.numel()),
           "logits_f32_out must be a contiguous fp32 CUDA tensor of at least as many elements")
    opt = lambda t: _ptr(t) if t is not None else None
    _lib.check(_lib.load().decdec_greedy_pick(_ptr(logits), logits.numel(), _dt(logits), _ptr(workspace), opt(logits_f32_out),
                                              _ptr(token), opt(seq), seq.numel() if seq is not None else 0, opt(count),
                                              opt(pos), _stream()))
