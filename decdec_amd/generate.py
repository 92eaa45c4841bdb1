"""Batch-1 greedy decode of a random-init decoder with DEC-compensated quantised linears: tokens/s with
and without DEC.

Counterpart of the reference's end-to-end/generate.py (prefill, then one token per step, the step captured
once in a graph and replayed).  Differences that matter on this machine: the whole step -- embedding,
32 layers, logits, argmax, feeding the token back and advancing the position -- lives in ONE HIP graph
that touches only static device buffers, so a run of tokens is a loop of graph replays without a host
round trip per token; weights are random (no checkpoint is read), the selector thresholds are calibrated
on the model's own activations.

    python -m decdec_amd.generate --model Meta-Llama-3-8B-Instruct --algo sqllm --bitwidth 4 \
        --k-chunk 8 --n-tb 16 --prompt-len 512 --max-new-tokens 256
"""
from __future__ import annotations

import argparse
import json
import sys
import time

import torch

from . import _lib, artifacts, decode_ops
from .linear import APLinear, LUTGEMMLinear, SQLLMLinear
from .model import DEC_MODULE_KEYS, Transformer

LINEAR_CLASSES = {"anyprec": APLinear, "lutgemm": LUTGEMMLinear, "sqllm": SQLLMLinear}


# ----------------------------------------------------------------------------------------------------
# random model
# ----------------------------------------------------------------------------------------------------
def _randint32(shape, gen, device):
    return torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int64, generator=gen, device=device).to(torch.int32)


def init_random_weights(model: Transformer, seed: int = 0, std: float = 0.02) -> None:
    """Random packed indices and LUTs / binary-coding scales with weight magnitudes around `std`."""
    dev = model.tok_embeddings.weight.device
    gen = torch.Generator(device=dev).manual_seed(seed)
    dt = model.dtype
    with torch.no_grad():
        model.tok_embeddings.weight.normal_(0, 1.0, generator=gen)
        model.output.weight.normal_(0, std, generator=gen)
        for layer in model.layers:
            for lin in layer.dec_linears():
                if isinstance(lin, torch.nn.Linear):
                    lin.weight.normal_(0, std, generator=gen)
                    continue
                lin.qweight.copy_(_randint32(tuple(lin.qweight.shape), gen, dev))
                if isinstance(lin, LUTGEMMLinear):
                    # uniform grid of 2^bits levels over about +-2.5 std: alpha_p = step 2^p / 2, centred
                    step = 5.0 * std / (2 ** lin.bitwidth - 1)
                    jitter = 0.75 + 0.5 * torch.rand(lin.alpha.shape[0], 1, lin.alpha.shape[2], generator=gen, device=dev)
                    pw = (2.0 ** torch.arange(lin.bitwidth, device=dev)).view(1, -1, 1)
                    lin.alpha.copy_((jitter * step / 2 * pw).to(dt))
                    lin.q_bias.copy_((torch.randn(lin.q_bias.shape, generator=gen, device=dev) * std * 0.05).to(dt))
                else:
                    lut = torch.randn(lin.lut.shape, generator=gen, device=dev).sort(dim=1).values * std
                    lin.lut.copy_(lut.to(dt))


def calibrate_thresholds(model: Transformer, seq_len: int = 256, passes: int = 2, seed: int = 1):
    """Thresholds of the four compensated linears of every layer from prefill passes over random tokens."""
    dev = model.tok_embeddings.weight.device
    seq_len = min(seq_len, model.max_seq_length)          # positions beyond the cache would index outside the mask
    gen = torch.Generator(device=dev).manual_seed(seed)
    named = [(f"layers.{i}.{key}", lin) for i, layer in enumerate(model.layers)
             for key, lin in zip(DEC_MODULE_KEYS, layer.dec_linears())]
    pos = torch.arange(seq_len, device=dev)

    def run():
        for _ in range(passes):
            tok = torch.randint(0, model.config.vocab_size, (1, seq_len), generator=gen, device=dev)
            model(tok, pos)
    return artifacts.collect_thresholds(named, run, dtype=model.dtype)


def random_dec_data(model: Transformer, thresholds: dict, seed: int = 2, residual_scale: float = 2e-4,
                    residual_device=None) -> dict:
    """Random 4-bit residual words and scales per module (one tensor per module shape, shared by the layers:
    every config pins its own copy) with the given thresholds.  With `residual_device` every layer gets a private
    copy of its residual on that device instead (the library then reads it in place: residuals resident in HBM)."""
    gen = torch.Generator().manual_seed(seed)
    per_shape = {}
    out = {}
    for i, layer in enumerate(model.layers):
        for key, lin in zip(DEC_MODULE_KEYS, layer.dec_linears()):
            K, N = lin.in_features, lin.out_features
            if (K, N) not in per_shape:
                q = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int64, generator=gen).to(torch.int32)
                s = (torch.rand(N, generator=gen) * residual_scale + residual_scale / 2).to(model.dtype)
                per_shape[(K, N)] = (q, s)
            q, s = per_shape[(K, N)]
            p = f"layers.{i}.{key}."
            if residual_device is not None:
                q = q.to(residual_device)                  # a new device tensor per layer
            out[p + "q_residual"], out[p + "scales"], out[p + "thresholds"] = q, s, thresholds[f"layers.{i}.{key}"]
    return out


# ----------------------------------------------------------------------------------------------------
# decode
# ----------------------------------------------------------------------------------------------------
class DecodeStep:
    """One greedy decode step on static buffers: logits of `token` at `pos`, argmax, the new token appended
    to `seq`, fed back into `token`, `pos` advanced.  `capture()` records it in a HIP graph."""

    def __init__(self, model: Transformer, max_tokens: int, keep_logits: bool = False):
        dev = model.tok_embeddings.weight.device
        self.model = model
        self.token = torch.zeros(1, 1, dtype=torch.int64, device=dev)
        self.pos = torch.zeros(1, dtype=torch.int64, device=dev)
        self.seq = torch.zeros(max_tokens, dtype=torch.int64, device=dev)
        self.count = torch.zeros(1, dtype=torch.int64, device=dev)
        self.logits = torch.zeros(1, model.config.vocab_size, dtype=torch.float32, device=dev) if keep_logits else None
        self.pick_workspace = decode_ops.greedy_pick_workspace(dev) if model.decode_kernels and dev.type == "cuda" else None
        self.graph = None

    def _step(self):
        logits = self.model(self.token, self.pos)[:, -1]
        if self.pick_workspace is not None and logits.dtype in (torch.float16, torch.bfloat16, torch.float32):
            # argmax and the bookkeeping below in two small launches
            decode_ops.greedy_pick(logits.contiguous(), self.pick_workspace, self.token, self.seq, self.count, self.pos,
                                   self.logits)
            return
        if self.logits is not None:
            self.logits.copy_(logits)
        nxt = torch.argmax(logits, dim=-1, keepdim=True)
        self.seq.index_copy_(0, self.count, nxt.view(1))
        self.token.copy_(nxt)
        self.pos.add_(1)
        self.count.add_(1)

    def start(self, token: int, pos: int):
        self.token.fill_(token)
        self.pos.fill_(pos)
        self.count.zero_()

    def capture(self):
        stream = torch.cuda.Stream()
        tok, pos, cnt = self.token.clone(), self.pos.clone(), self.count.clone()
        # everything queued so far (weights being initialised, the zero fill of the step's own buffers, a prefill)
        # must have run before the step does: an unordered step would read its token before it was written
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream), torch.no_grad():
            self._step()                      # warm-up: lazy initialisation must not happen under capture
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=stream), torch.no_grad():
            self._step()
        torch.cuda.current_stream().wait_stream(stream)
        self.token.copy_(tok); self.pos.copy_(pos); self.count.copy_(cnt)
        torch.cuda.synchronize()

    def run(self, n: int):
        with torch.no_grad():
            for _ in range(n):
                if self.graph is not None:
                    self.graph.replay()
                else:
                    self._step()


@torch.no_grad()
def generate(model: Transformer, prompt: torch.Tensor, max_new_tokens: int, use_graph: bool = True,
             max_seq_length: int | None = None):
    """Greedy decode; returns (tokens [T + max_new_tokens], seconds spent on the max_new_tokens - 1 decode steps)."""
    T = prompt.numel()
    total = T + max_new_tokens
    model.setup_caches(1, min(max_seq_length or total, model.config.block_size))
    assert total <= model.max_seq_length, "prompt + new tokens exceed the cache"
    dev = prompt.device
    logits = model(prompt.view(1, -1), torch.arange(T, device=dev))
    first = int(torch.argmax(logits[0, -1]))
    step = DecodeStep(model, max_new_tokens)
    step.start(first, T)
    if use_graph:
        step.capture()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    step.run(max_new_tokens - 1)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    seq = torch.cat((prompt.view(-1), torch.tensor([first], device=dev), step.seq[:max_new_tokens - 1]))
    return seq, dt


def build_model(name: str, algo: str, bitwidth: int, group_size: int = 128, dtype=torch.float16, seed: int = 0,
                n_layer: int | None = None) -> Transformer:
    from .model import ModelArgs
    cfg = ModelArgs.from_name(name)
    if n_layer is not None:
        cfg.n_layer = n_layer
    kw = {"bitwidth": bitwidth, "dtype": dtype}
    if algo == "lutgemm":
        kw["group_size"] = group_size
    model = Transformer(dtype, cfg, linear_class=LINEAR_CLASSES[algo], linear_kwargs=kw)
    init_random_weights(model, seed)
    model.share_output_arena()
    return model.eval()


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", default="Meta-Llama-3-8B-Instruct")
    ap.add_argument("--algo", choices=sorted(LINEAR_CLASSES), default="sqllm")
    ap.add_argument("--bitwidth", type=int, default=4)
    ap.add_argument("--group-size", type=int, default=128)
    ap.add_argument("--k-chunk", type=int, nargs="+", default=[8], help="one value, or groups of four (qkv o gate_up down); every group is one DEC run")
    ap.add_argument("--n-tb", type=int, default=16)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--max-new-tokens", type=int, default=256)
    ap.add_argument("--max-seq-length", type=int, default=2048)
    ap.add_argument("--n-layer", type=int, default=None, help="fewer layers than the named model (smoke runs)")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--residual-on-device", action="store_true",
                    help="keep every layer's residual in device memory instead of pinned host memory")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="library option (decdec_set_option), e.g. fusion=0; may be repeated")
    args = ap.parse_args(argv)
    for kv in args.option:
        name, _, value = kv.partition("=")
        _lib.set_option(name, int(value))
    if len(args.k_chunk) == 1:
        k_sets = [args.k_chunk * 4]
    else:
        assert len(args.k_chunk) % 4 == 0, "--k-chunk takes one value or groups of four (qkv o gate_up down)"
        k_sets = [args.k_chunk[i:i + 4] for i in range(0, len(args.k_chunk), 4)]
    log = lambda s: print(s, file=sys.stderr, flush=True)

    model = build_model(args.model, args.algo, args.bitwidth, args.group_size, n_layer=args.n_layer)
    gen = torch.Generator().manual_seed(3)
    prompt = torch.randint(0, model.config.vocab_size, (args.prompt_len,), generator=gen).cuda()
    log(f"model {args.model} ({model.config.n_layer} layers), {args.algo} {args.bitwidth}-bit; base-only run")
    seq0, t_base = generate(model, prompt, args.max_new_tokens, not args.no_graph, args.max_seq_length)
    n = args.max_new_tokens - 1
    log(f"base: {n / t_base:.1f} tokens/s; calibrating thresholds")
    th = calibrate_thresholds(model)
    model.load_dec_data(random_dec_data(model, th, residual_device="cuda" if args.residual_on_device else None))
    k_max = max(max(ks) for ks in k_sets)
    model.create_dec_context(args.n_tb, buffer_size=max(1024, k_max * (model.config.intermediate_size // 1024 + 1)))
    for i, ks in enumerate(k_sets):
        if i == 0:
            model.set_dec_config(ks)              # pins the residuals
        else:
            model.update_dec_config(ks)           # same pinned residuals, new k_chunk
        log(f"DEC run, k_chunk {ks}")
        seq1, t_dec = generate(model, prompt, args.max_new_tokens, not args.no_graph, args.max_seq_length)
        print(json.dumps({
            "metric": "tokens/s, batch-1 greedy decode", "model": args.model, "n_layer": model.config.n_layer,
            "algo": args.algo, "bitwidth": args.bitwidth, "k_chunk": ks, "n_tb": args.n_tb,
            "prompt_len": args.prompt_len, "new_tokens": args.max_new_tokens, "graph": not args.no_graph,
            "tokens_per_s_base": round(n / t_base, 2), "tokens_per_s_dec": round(n / t_dec, 2),
            "ms_per_token_base": round(t_base / n * 1e3, 4), "ms_per_token_dec": round(t_dec / n * 1e3, 4),
            "dec_slowdown_pct": round((t_dec / t_base - 1) * 100, 2), "data": "synthetic (random weights and prompt)",
            "residual": "device memory" if args.residual_on_device else "pinned host memory"}),
            flush=True)


if __name__ == "__main__":
    main()
