"""Choose n_tb and per-module k_chunk for a slowdown budget.

Counterpart of the reference's autotuner (autotuner/run_profile.py + tuner.py): it profiles a decode run
under Nsight Systems and parses the trace; here the library times its own layers (HIP-graph replay on
synthetic weights of the real shapes, nothing else is needed), and the same two-phase search then picks
the parameters:

  1. global search (tuner.py:150-262): for every n_tb cap, the largest k_chunk, equal for all modules,
     whose summed layer time stays within `baseline * (1 + budget)`; the cap that allows the largest
     k_chunk wins (ties: the faster one).  If not even k_chunk = 1 fits, the smallest module is taken out
     of compensation and the search repeats.
  2. fine-grained search (tuner.py:264-312): modules take further +1 steps of k_chunk, cheapest step
     first, while the layer stays within the budget.

`tune()` is pure Python on a timing table and runs anywhere; `measure()` (isolated launches) and
`measure_in_model()` (the modules inside the captured decode step, which is what a user will run) need the GPU.

    python -m decdec_amd.autotune --model llama3-8b --algo anyprec --bitwidth 3 --target-slowdown 2.5 [--in-model]
"""
from __future__ import annotations

import argparse
import time
import json
import sys

MODELS = {   # module -> (in_features, out_features); reference autotuner/README.md:56-60
    "llama3-8b": {"qkv": (4096, 6144), "o": (4096, 4096), "gu": (4096, 28672), "d": (14336, 4096)},
    "phi3-medium": {"qkv": (5120, 7680), "o": (5120, 5120), "gu": (5120, 35840), "d": (17920, 5120)},
    "llama3-70b": {"qkv": (8192, 10240), "o": (8192, 8192), "gu": (8192, 57344), "d": (28672, 8192)},
}
HBM_GBS, LINK_GBS = 8000.0, 64.0


def k_chunk_estimate(bitwidth: int, hbm_gbs: float = HBM_GBS, link_gbs: float = LINK_GBS) -> int:
    """Break-even k_chunk of the reference's rule (run_profile.py:26-30): the residual rows of a chunk cost
    as much link time as the chunk's base weights cost HBM time."""
    return int(bitwidth / (hbm_gbs / link_gbs) / 4 * 1024)


# ----------------------------------------------------------------------------------------------------
# search
# ----------------------------------------------------------------------------------------------------
def _time_at(table, n_tb_cap, k_chunk):
    """Time of a module at the largest measured n_tb not above the cap; None if not measured."""
    usable = [n for n in table if n <= n_tb_cap]
    if not usable:
        return None, None
    n = max(usable)
    return table[n].get(k_chunk), n


def tune(results: dict, target_slowdown: float, matrix_dims: dict) -> dict:
    """results[module] = (baseline_us, {n_tb: {k_chunk: us}}); target_slowdown is a factor (1.025 = +2.5 %).
    Returns best_max_n_tb, threadblocks_per_module, k_chunk_per_module, time_by_module, layer_time,
    layer_baseline -- the reference tuner's result dictionary."""
    modules = list(matrix_dims)
    baseline = {m: results[m][0] for m in modules}
    layer_baseline = sum(baseline.values())
    budget = layer_baseline * target_slowdown
    caps = sorted({n for m in modules for n in results[m][1]})
    k_values = sorted({k for m in modules for t in results[m][1].values() for k in t})
    by_size = sorted(modules, key=lambda m: matrix_dims[m][0] * matrix_dims[m][1])
    included = list(modules)

    best_cap, best_k, best_time = None, 0, layer_baseline
    while included:
        best_cap, best_k, best_time = None, 0, float("inf")
        for cap in caps:
            k_fit, t_fit = 0, layer_baseline
            for k in k_values:
                total = sum(baseline[m] for m in modules if m not in included)
                for m in included:
                    t, _ = _time_at(results[m][1], cap, k)
                    total += float("inf") if t is None else t
                if total > budget:
                    break
                k_fit, t_fit = k, total
            if k_fit > best_k or (k_fit == best_k and t_fit < best_time):
                best_cap, best_k, best_time = cap, k_fit, t_fit
        if best_k > 0:
            break
        included.remove(next(m for m in by_size if m in included))      # smallest module gives up compensation

    k_per, n_per, t_per = {}, {}, {}
    for m in modules:
        if m in included and best_k > 0:
            t, n = _time_at(results[m][1], best_cap, best_k)
            k_per[m], n_per[m], t_per[m] = best_k, n, t
        else:
            k_per[m], n_per[m], t_per[m] = 0, None, baseline[m]

    improved = best_k > 0
    while improved:                                  # fine-grained: cheapest +1 steps first
        improved = False
        steps = []
        for m in modules:
            if n_per[m] is None:
                continue
            nxt = [k for k in k_values if k > k_per[m]]
            if not nxt:
                continue
            t = results[m][1][n_per[m]].get(nxt[0])
            if t is not None:
                steps.append((t - t_per[m], m, nxt[0], t))
        for delta, m, k, t in sorted(steps):
            if sum(t_per.values()) + delta <= budget:
                k_per[m], t_per[m] = k, t
                improved = True
    return {"matrix_dims": matrix_dims, "best_max_n_tb": best_cap if best_k > 0 else None,
            "threadblocks_per_module": [n_per[m] for m in modules],
            "k_chunk_per_module": [k_per[m] for m in modules],
            "time_by_module": [t_per[m] for m in modules],
            "layer_time": sum(t_per.values()), "layer_baseline": layer_baseline}


# ----------------------------------------------------------------------------------------------------
# measurement (GPU)
# ----------------------------------------------------------------------------------------------------
def measure(matrix_dims: dict, algo: str, bitwidth: int, n_tb_values, k_chunk_values, group_size: int = 128,
            reps: int = 10, iters: int = 10, log=None, settle_ms: float = 20.0) -> dict:
    """Times base GEMV and fused DEC + GEMV of every module on synthetic data (fp16)."""
    import torch
    from . import ext, formats as F
    dev = "cuda"
    g = torch.Generator().manual_seed(0)

    def graph_time(fn):
        st = torch.cuda.Stream()
        st.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(st):
            for _ in range(2):
                fn()
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr, stream=st):
            for _ in range(reps):
                fn()
        # the shader clock takes some tens of milliseconds of load to settle after an idle period (the set-up between two
        # points is one): replay untimed first, or neighbouring points are timed at different clocks
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < settle_ms:
            gr.replay()
            torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(st):
            a.record(st)
            for _ in range(iters):
                gr.replay()
            b.record(st)
        torch.cuda.synchronize()
        return a.elapsed_time(b) / iters / reps * 1e3

    def randint(shape):
        return torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int32, device=dev)

    results = {}
    for name, (K, N) in matrix_dims.items():
        x = F.make_activation(K, g).to(dev)
        out = torch.zeros(1, 1, N, device=dev, dtype=torch.float16)
        nb = 6                                           # private weight copies: every launch reads HBM
        if algo == "anyprec":
            ws = [randint((bitwidth, N, K // 32)) for _ in range(nb)]
            lut = torch.randn(N, 1 << bitwidth, device=dev, dtype=torch.float16)
            base = lambda j: ext.anyprec_gemv(x, out, ws[j], lut, bitwidth)
            fused = lambda c, j: ext.dec_anyprec(c, x, out, ws[j], lut, bitwidth)
        elif algo == "lutgemm":
            ws = [randint((K // 32, bitwidth, N)) for _ in range(nb)]
            alpha = torch.rand(K // group_size, bitwidth, N, device=dev).half() * 0.01
            qb = torch.rand(K // group_size, N, device=dev).half() * 0.01
            base = lambda j: ext.lutgemm_gemv(x, out, ws[j], alpha, qb, bitwidth, group_size)
            fused = lambda c, j: ext.dec_lutgemm(c, x, out, ws[j], alpha, qb, bitwidth, group_size)
        elif algo == "sqllm":
            ws = [randint((K * bitwidth // 32, N)) for _ in range(nb)]
            lut = (torch.randn(N, 1 << bitwidth, device=dev) * 0.02).half()
            base = lambda j: ext.sqllm_gemv(x, out, ws[j], lut, bitwidth)
            fused = lambda c, j: ext.dec_sqllm(c, x, out, ws[j], lut, bitwidth)
        else:
            raise ValueError(f"unknown algo {algo}")
        i = [0]

        def run_base():
            i[0] += 1
            base(i[0] % nb)
        t_base = graph_time(run_base)
        if not n_tb_values:
            results[name] = (t_base, {})
            del ws
            continue
        rows = torch.zeros(K, dtype=torch.int32, device=dev)
        acts = torch.zeros(K, dtype=torch.float16, device=dev)
        th = F.calibrate_thresholds(K, g, draws=8)
        cheat = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), dtype=torch.int32)
        sc = torch.rand(N).half()
        table = {}
        cfg = None
        ctxs = []
        for n_tb in n_tb_values:
            ctx = ext.create_dec_context(n_tb, rows, acts)
            ctxs.append(ctx)
            table[n_tb] = {}
            for kc in k_chunk_values:
                if cfg is None:
                    cfg = ext.create_dec_config(ctx, kc, cheat, sc, th)     # the residual is pinned once
                else:
                    ext.update_dec_config(cfg, ctx, kc)

                def run_fused():
                    i[0] += 1
                    fused(cfg, i[0] % nb)
                table[n_tb][kc] = graph_time(run_fused)
            if log:
                log(f"{name} ({K} x {N}) base {t_base:.2f} us, n_tb {n_tb}: " +
                    " ".join(f"k{k}={t:.2f}" for k, t in table[n_tb].items()))
        ext.destroy_dec_config(cfg)
        for ctx in ctxs:
            ext.destroy_dec_context(ctx)
        results[name] = (t_base, table)
        del ws
    return results


FULL_NAMES = {"llama3-8b": "Meta-Llama-3-8B-Instruct", "phi3-medium": "Phi-3-medium-4k-instruct",
              "llama3-70b": "Meta-Llama-3-70B-Instruct"}


def measure_in_model(model: str, algo: str, bitwidth: int, n_tb_values, k_chunk_values, group_size: int = 128,
                     n_layer=None, prompt_len: int = 64, new_tokens: int = 49, log=None):
    """Times the modules where they run: inside the graph-captured decode step of the random-init model
    (the reference profiles its decode run, autotuner/run_profile.py:46-56).  For every n_tb and k_chunk, DEC is
    switched on for ONE module kind at a time; the change of the time per token, divided by the number of layers,
    is what that module's launch costs over its base GEMV in place.  Returns (results for `tune`, info) with
    info = {"token_us_base", "n_layer", "model", "evaluate": callable(k_chunks, n_tb) -> us per token}."""
    import torch
    from . import generate as G
    m = G.build_model(FULL_NAMES[model], algo, bitwidth, group_size, n_layer=n_layer)
    gen = torch.Generator().manual_seed(3)
    prompt = torch.randint(0, m.config.vocab_size, (prompt_len,), generator=gen).cuda()
    cache = max(256, prompt_len + new_tokens)

    def token_us():
        best = float("inf")
        for _ in range(2):
            _, dt = G.generate(m, prompt, new_tokens, True, cache)
            best = min(best, dt / (new_tokens - 1) * 1e6)
        return best

    t_base = token_us()
    m.load_dec_data(G.random_dec_data(m, G.calibrate_thresholds(m, seq_len=min(256, cache))))
    dims = MODELS[model]
    k_max = max(k_chunk_values)
    names = list(dims)
    base = measure(dims, algo, bitwidth, [], [], group_size)            # isolated base GEMV times
    tables = {name: {} for name in names}
    first = True
    for n_tb in n_tb_values:
        if first:
            m.create_dec_context(n_tb, buffer_size=max(1024, k_max * (m.config.intermediate_size // 1024 + 1)))
            m.set_dec_config([0, 0, 0, 0])                              # pins the residuals once
            first = False
        else:
            m.update_dec_context(n_tb)
        for i, name in enumerate(names):
            tables[name][n_tb] = {}
            for k in k_chunk_values:
                m.update_dec_config([k if j == i else 0 for j in range(4)])
                tables[name][n_tb][k] = base[name][0] + (token_us() - t_base) / m.config.n_layer
            if log:
                log(f"{name} base {base[name][0]:.2f} us, in-model, n_tb {n_tb}: " +
                    " ".join(f"k{k}={t:.2f}" for k, t in tables[name][n_tb].items()))

    def evaluate(k_chunks, n_tb):
        m.update_dec_context(n_tb)
        m.update_dec_config(list(k_chunks))
        return token_us()
    results = {name: (base[name][0], tables[name]) for name in names}
    return results, {"token_us_base": t_base, "n_layer": m.config.n_layer, "model": FULL_NAMES[model], "evaluate": evaluate}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", choices=sorted(MODELS), default="llama3-8b")
    ap.add_argument("--algo", choices=["anyprec", "lutgemm", "sqllm"], default="anyprec")
    ap.add_argument("--bitwidth", type=int, default=3)
    ap.add_argument("--target-slowdown", type=float, default=2.5, help="percent (reference default 2.5)")
    ap.add_argument("--min-n-tb", type=int, default=4)
    ap.add_argument("--max-n-tb", type=int, default=32)
    ap.add_argument("--n-tb-step", type=int, default=4)
    ap.add_argument("--max-k-chunk", type=int, default=0, help="0: twice the break-even estimate, at least 8")
    ap.add_argument("--in-model", action="store_true",
                    help="time the modules inside the graph-captured decode step of the random-init model")
    ap.add_argument("--n-layer", type=int, default=None, help="--in-model: build fewer layers than the model has")
    args = ap.parse_args(argv)
    dims = MODELS[args.model]
    k_max = args.max_k_chunk or max(8, 2 * k_chunk_estimate(args.bitwidth))
    n_tbs = list(range(args.min_n_tb, args.max_n_tb + 1, args.n_tb_step))
    ks = list(range(1, k_max + 1))
    print(f"break-even k_chunk estimate {k_chunk_estimate(args.bitwidth)}; sweeping k_chunk 1..{k_max}, n_tb {n_tbs}",
          file=sys.stderr)
    log = lambda s: print(s, file=sys.stderr, flush=True)
    if args.in_model:
        res, info = measure_in_model(args.model, args.algo, args.bitwidth, n_tbs, ks, n_layer=args.n_layer, log=log)
    else:
        res, info = measure(dims, args.algo, args.bitwidth, n_tbs, ks, log=log), None
    out = tune(res, 1 + args.target_slowdown / 100, dims)
    out["target_slowdown_pct"] = args.target_slowdown
    if info is not None:
        out["measured"] = "in the captured decode step"
        out["token_us_base"] = round(info["token_us_base"], 1)
        out["predicted_token_slowdown_pct"] = round(
            (out["layer_time"] - out["layer_baseline"]) * info["n_layer"] / info["token_us_base"] * 100, 2)
        if out["best_max_n_tb"] is not None:
            t = info["evaluate"](out["k_chunk_per_module"], out["best_max_n_tb"])
            out["measured_token_slowdown_pct"] = round((t / info["token_us_base"] - 1) * 100, 2)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
