"""Decoder-only Transformer whose linear layers are the quantised DEC modules of ``decdec_amd.linear``.

Counterpart of the reference's end-to-end/model.py (a gpt-fast style Llama / Phi-3 decoder): same
``ModelArgs`` fields and model names, fused ``wqkv`` and ``w1w3`` projections, a static KV cache,
``load_dec_data`` / ``create_dec_context`` / ``set_dec_config`` / ``update_dec_config`` with the
reference's meaning (k_chunks = [qkv, o, gate_up, down]).  Everything that is not a linear layer is
plain torch: this file exists to drive the linear-layer hot path from a real decode step, not to be a
model zoo.  A decode step touches only static buffers, so it can be captured in a HIP graph; on the GPU
its residual adds + normalisations, rotary embedding, cache append, attention and gated activation run on the library's
helper kernels
(``decode_ops``), a prefill or CPU pass on torch ops.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F


def find_multiple(n: int, k: int) -> int:
    return n if n % k == 0 else n + k - n % k


@dataclass
class ModelArgs:
    block_size: int = 2048
    vocab_size: int = 32000
    n_layer: int = 32
    n_head: int = 32
    dim: int = 4096
    intermediate_size: Optional[int] = None
    n_local_heads: int = -1
    head_dim: int = 64
    rope_base: float = 10000
    norm_eps: float = 1e-5
    model_name: Optional[str] = None

    def __post_init__(self):
        if self.n_local_heads == -1:
            self.n_local_heads = self.n_head
        if self.intermediate_size is None:
            self.intermediate_size = find_multiple(int(2 * 4 * self.dim / 3), 256)
        self.head_dim = self.dim // self.n_head

    @classmethod
    def from_name(cls, name: str) -> "ModelArgs":
        if name not in transformer_configs:
            raise KeyError(f"Unknown model name: {name}, available: {sorted(transformer_configs)}")
        return cls(**transformer_configs[name])


# reference end-to-end/model.py:54-58, plus a small shape for tests
transformer_configs = {
    "Meta-Llama-3-8B-Instruct": dict(model_name="Meta-Llama-3-8B-Instruct", block_size=8192, n_layer=32, n_head=32,
                                     n_local_heads=8, dim=4096, intermediate_size=14336, vocab_size=128256,
                                     rope_base=500000),
    "Meta-Llama-3-70B-Instruct": dict(model_name="Meta-Llama-3-70B-Instruct", block_size=8192, n_layer=80, n_head=64,
                                      n_local_heads=8, dim=8192, intermediate_size=28672, vocab_size=128256,
                                      rope_base=500000),
    "Phi-3-medium-4k-instruct": dict(model_name="Phi-3-medium-4k-instruct", block_size=4096, n_layer=40, n_head=40,
                                     n_local_heads=10, dim=5120, intermediate_size=17920, vocab_size=32064,
                                     rope_base=10000),
    "tiny-llama-test": dict(model_name="tiny-llama-test", block_size=256, n_layer=2, n_head=8, n_local_heads=2,
                            dim=512, intermediate_size=1536, vocab_size=640, rope_base=10000),
}


class RMSNorm(nn.Module):
    """x / rms(x) * weight (one fused kernel; statistics in fp32)."""

    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.rms_norm(x, (x.shape[-1],), self.weight, self.eps)


def rope_tables(head_dim: int, max_pos: int, base: float, device=None):
    """cos / sin [max_pos, head_dim] in fp32 for the half-rotation form: pair (i, i + head_dim/2) is
    rotated by pos * base^(-2i/head_dim)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim))
    ang = torch.arange(max_pos, dtype=torch.float32, device=device)[:, None] * inv_freq[None, :]
    ang = torch.cat((ang, ang), dim=-1)
    return ang.cos(), ang.sin()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [..., S, D] with cos / sin [S, D] already gathered at the positions of the S tokens (same dtype)."""
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return x * cos + rot * sin


class KVCache(nn.Module):
    def __init__(self, max_batch_size: int, max_seq_length: int, n_heads: int, head_dim: int, dtype, device):
        super().__init__()
        shape = (max_batch_size, n_heads, max_seq_length, head_dim)
        self.register_buffer("k_cache", torch.zeros(shape, dtype=dtype, device=device), persistent=False)
        self.register_buffer("v_cache", torch.zeros(shape, dtype=dtype, device=device), persistent=False)

    def update(self, input_pos: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        self.k_cache.index_copy_(2, input_pos, k)
        self.v_cache.index_copy_(2, input_pos, v)
        return self.k_cache, self.v_cache


class Attention(nn.Module):
    def __init__(self, config: ModelArgs, linear_class, linear_kwargs):
        super().__init__()
        assert config.dim % config.n_head == 0 and config.n_head % config.n_local_heads == 0
        total = (config.n_head + 2 * config.n_local_heads) * config.head_dim
        self.wqkv = linear_class(config.dim, total, bias=False, **linear_kwargs)
        self.wo = linear_class(config.dim, config.dim, bias=False, **linear_kwargs)
        self.kv_cache: Optional[KVCache] = None
        self.n_head, self.n_local_heads, self.head_dim, self.dim = config.n_head, config.n_local_heads, config.head_dim, config.dim

    def forward(self, x: torch.Tensor, mask: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, input_pos: torch.Tensor,
                rope_tables_full=None):
        B, S, _ = x.shape
        kv = self.n_local_heads * self.head_dim
        qkv = self.wqkv(x)
        if rope_tables_full is not None:
            # one-token step on the library's helper kernel: rotate, append to the cache and attend in one launch
            from . import decode_ops
            y = torch.empty(1, 1, self.dim, dtype=x.dtype, device=x.device)
            decode_ops.rope_attention(qkv.view(-1), rope_tables_full[0], rope_tables_full[1], input_pos, y,
                                      self.kv_cache.k_cache, self.kv_cache.v_cache, self.n_head, self.n_local_heads,
                                      rope_tables_full[2])
            return self.wo(y)
        # RoPE on the query and key heads in one pass (they are neighbours in the fused projection)
        nqk = self.n_head + self.n_local_heads
        qk = apply_rope(qkv[..., :self.dim + kv].view(B, S, nqk, self.head_dim).transpose(1, 2), cos, sin)
        q, k = qk[:, :self.n_head], qk[:, self.n_head:]
        v = qkv[..., self.dim + kv:].view(B, S, self.n_local_heads, self.head_dim).transpose(1, 2)
        if self.kv_cache is not None:
            k, v = self.kv_cache.update(input_pos, k, v)
        # grouped-query attention over the whole (static) cache; rows of `mask` hide what is not yet written
        y = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, enable_gqa=self.n_head != self.n_local_heads)
        y = y.transpose(1, 2).reshape(B, S, self.dim)
        return self.wo(y)


class FeedForward(nn.Module):
    def __init__(self, config: ModelArgs, linear_class, linear_kwargs):
        super().__init__()
        self.inter = config.intermediate_size
        self.w1w3 = linear_class(config.dim, 2 * self.inter, bias=False, **linear_kwargs)
        self.w2 = linear_class(self.inter, config.dim, bias=False, **linear_kwargs)

    def forward(self, x: torch.Tensor, helper_kernels: bool = False) -> torch.Tensor:
        gu = self.w1w3(x)
        if helper_kernels:
            from . import decode_ops
            act = torch.empty(1, 1, self.inter, dtype=x.dtype, device=x.device)
            decode_ops.silu_mul(gu.view(-1), act.view(-1))
            return self.w2(act)
        a, b = gu.split([self.inter, self.inter], dim=-1)
        return self.w2(F.silu(a) * b)


class TransformerBlock(nn.Module):
    def __init__(self, config: ModelArgs, linear_class, linear_kwargs):
        super().__init__()
        self.attention = Attention(config, linear_class, linear_kwargs)
        self.feed_forward = FeedForward(config, linear_class, linear_kwargs)
        self.input_layernorm = RMSNorm(config.dim, config.norm_eps)
        self.post_attention_layernorm = RMSNorm(config.dim, config.norm_eps)

    def forward(self, x, mask, cos, sin, input_pos, rope_tables_full=None):
        h = x + self.attention(self.input_layernorm(x), mask, cos, sin, input_pos, rope_tables_full)
        return h + self.feed_forward(self.post_attention_layernorm(h), rope_tables_full is not None)

    def decode_step(self, h, branch, input_pos, rope_tables_full):
        """One token on the helper kernels.  `h` is the residual stream before this block, `branch` the output of
        the previous block's feed-forward that has not been added yet (None for the first block); returns the
        stream after this block's attention and this block's feed-forward output, again not yet added."""
        from . import decode_ops
        n1 = torch.empty_like(h)
        if branch is None:
            decode_ops.add_rmsnorm(h, None, self.input_layernorm.weight, None, n1, self.input_layernorm.eps)
            h0 = h
        else:
            h0 = torch.empty_like(h)
            decode_ops.add_rmsnorm(h, branch, self.input_layernorm.weight, h0, n1, self.input_layernorm.eps)
        a = self.attention(n1, None, None, None, input_pos, rope_tables_full)
        h1, n2 = torch.empty_like(h), torch.empty_like(h)
        decode_ops.add_rmsnorm(h0, a, self.post_attention_layernorm.weight, h1, n2, self.post_attention_layernorm.eps)
        return h1, self.feed_forward(n2, True)

    def dec_linears(self):
        """The four compensated linears in the order of the k_chunk lists: qkv, o, gate_up, down."""
        return [self.attention.wqkv, self.attention.wo, self.feed_forward.w1w3, self.feed_forward.w2]


DEC_MODULE_KEYS = ("attention.wqkv", "attention.wo", "feed_forward.w1w3", "feed_forward.w2")


class Transformer(nn.Module):
    def __init__(self, dtype, config: ModelArgs, linear_class=nn.Linear, linear_kwargs=None, device="cuda"):
        super().__init__()
        self.config, self.dtype = config, dtype
        linear_kwargs = dict(linear_kwargs or {})
        self.tok_embeddings = nn.Embedding(config.vocab_size, config.dim, dtype=dtype, device=device)
        self.layers = nn.ModuleList(TransformerBlock(config, linear_class, linear_kwargs) for _ in range(config.n_layer))
        self.norm = RMSNorm(config.dim, config.norm_eps)
        self.output = nn.Linear(config.dim, config.vocab_size, bias=False, dtype=dtype, device=device)
        self.max_batch_size = self.max_seq_length = -1
        self.dec_contexts = []
        # one-token steps use the library's rotary / attention / activation kernels instead of torch ops
        self.decode_kernels = (torch.device(device).type == "cuda" and dtype in (torch.float16, torch.bfloat16)
                               and config.head_dim in (64, 128))
        self.to(device)
        for m in self.modules():
            if isinstance(m, RMSNorm):
                m.weight.data = m.weight.data.to(dtype)

    @classmethod
    def from_name(cls, dtype, name: str, **kw) -> "Transformer":
        return cls(dtype, ModelArgs.from_name(name), **kw)

    def setup_caches(self, max_batch_size: int, max_seq_length: int):
        if self.max_seq_length >= max_seq_length and self.max_batch_size >= max_batch_size:
            return
        max_seq_length = find_multiple(max_seq_length, 8)
        self.max_seq_length, self.max_batch_size = max_seq_length, max_batch_size
        dev = self.tok_embeddings.weight.device
        for b in self.layers:
            b.attention.kv_cache = KVCache(max_batch_size, max_seq_length, self.config.n_local_heads,
                                           self.config.head_dim, self.dtype, dev)
        self.causal_mask = torch.tril(torch.ones(max_seq_length, max_seq_length, dtype=torch.bool, device=dev))
        cos, sin = rope_tables(self.config.head_dim, max_seq_length, self.config.rope_base, dev)
        self.rope_cos, self.rope_sin = cos.to(self.dtype), sin.to(self.dtype)
        self.attention_workspace = None
        # caches beyond 512 positions: with a workspace the kernel shares a head's positions among up to 8 workgroups
        # once the sequence is longer than that (8.9 against 17.0 us at position 2047; below, one workgroup per head
        # is faster: 5.9 against 8.0 us at 255)
        if self.decode_kernels and max_seq_length > 512:
            from . import decode_ops
            self.attention_workspace = decode_ops.attention_workspace(self.config.n_head, self.config.head_dim, dev)

    def share_output_arena(self):
        """Puts the persistent decode outputs of all quantised linears into one buffer that a decode step
        clears with a single fill, instead of one fill per linear."""
        lins = [l for layer in self.layers for l in layer.dec_linears() if hasattr(l, "external_zero")]
        if not lins:
            return
        total = sum(find_multiple(l.out_features, 64) for l in lins)
        self.output_arena = torch.zeros(total, dtype=self.dtype, device=self.tok_embeddings.weight.device)
        off = 0
        for l in lins:
            l.output = self.output_arena[off:off + l.out_features].view(1, 1, l.out_features)
            l.external_zero = True
            off += find_multiple(l.out_features, 64)

    def forward(self, idx: torch.Tensor, input_pos: torch.Tensor) -> torch.Tensor:
        """idx [B, S] token ids, input_pos [S] positions (int64); returns logits [B, S, vocab]."""
        assert self.max_seq_length > 0, "Caches must be initialized first"
        assert idx.shape[1] <= self.max_seq_length and input_pos.numel() == idx.shape[1], \
            f"{idx.shape[1]} positions do not fit a cache of {self.max_seq_length} (input_pos must hold one position per token)"
        if idx.shape[1] == 1 and getattr(self, "output_arena", None) is not None:
            self.output_arena.zero_()
        x = self.tok_embeddings(idx)
        if self.decode_kernels and idx.shape == (1, 1) and x.is_cuda:
            from . import decode_ops
            full = (self.rope_cos, self.rope_sin, self.attention_workspace)
            h, branch = x.contiguous(), None
            for layer in self.layers:
                h, branch = layer.decode_step(h, branch, input_pos, full)
            n = torch.empty_like(h)
            decode_ops.add_rmsnorm(h, branch, self.norm.weight, torch.empty_like(h), n, self.norm.eps)
            if self.output.bias is None and self.output.weight.dtype == n.dtype and self.config.dim % 8 == 0:
                # the unquantised head on the library's streaming GEMV (a gigabyte of weights per token at 8B)
                logits = torch.empty(1, 1, self.config.vocab_size, dtype=n.dtype, device=n.device)
                decode_ops.dense_gemv(self.output.weight, n.view(-1), logits.view(-1))
                return logits
            return self.output(n)
        mask = self.causal_mask.index_select(0, input_pos)                     # [S, max_seq]
        cos, sin = self.rope_cos.index_select(0, input_pos), self.rope_sin.index_select(0, input_pos)
        for layer in self.layers:
            x = layer(x, mask, cos, sin, input_pos)
        return self.output(self.norm(x))

    # ---- DEC plumbing (reference end-to-end/model.py:143-215) ----
    def load_dec_data(self, dec_data: dict):
        for i, layer in enumerate(self.layers):
            for key, lin in zip(DEC_MODULE_KEYS, layer.dec_linears()):
                p = f"layers.{i}.{key}."
                lin.load_dec_data(dec_data[p + "q_residual"], dec_data[p + "scales"], dec_data[p + "thresholds"])

    def create_dec_context(self, n_tbs, buffer_size: int = 1024):
        from . import ext
        n_tbs = [n_tbs] if isinstance(n_tbs, int) else list(n_tbs)
        dev = self.tok_embeddings.weight.device
        self.selected_rows_buffers = [torch.empty(buffer_size, dtype=torch.int32, device=dev) for _ in n_tbs]
        self.selected_activations_buffers = [torch.empty(buffer_size, dtype=self.dtype, device=dev) for _ in n_tbs]
        self.dec_contexts = [ext.create_dec_context(n, r, a) for n, r, a in
                             zip(n_tbs, self.selected_rows_buffers, self.selected_activations_buffers)]

    def update_dec_context(self, n_tbs):
        from . import ext
        n_tbs = [n_tbs] if isinstance(n_tbs, int) else list(n_tbs)
        assert len(n_tbs) == len(self.dec_contexts)
        old = self.dec_contexts
        self.dec_contexts = [ext.create_dec_context(n, r, a) for n, r, a in
                             zip(n_tbs, self.selected_rows_buffers, self.selected_activations_buffers)]
        self._stale_contexts = getattr(self, "_stale_contexts", []) + old      # configs may still point at them

    def _k_chunks(self, k_chunks):
        k_chunks = list(k_chunks)
        assert len(k_chunks) == 4, "k_chunks = [qkv, o, gate_up, down]"
        return k_chunks

    def set_dec_config(self, k_chunks):
        for layer in self.layers:
            for lin, k in zip(layer.dec_linears(), self._k_chunks(k_chunks)):
                lin.create_dec_config(self.dec_contexts[0], k)

    def update_dec_config(self, k_chunks):
        for layer in self.layers:
            for lin, k in zip(layer.dec_linears(), self._k_chunks(k_chunks)):
                lin.update_dec_config(self.dec_contexts[0], k)
