"""Decode harness on the GPU: every compensated linear of a small decoder against the oracle on the very
activations it saw, and graph replays of the decode step against eager steps."""
import numpy as np
import pytest
import torch

from decdec_amd import generate as G
from decdec_amd.model import DEC_MODULE_KEYS
from oracle import decdec_oracle as O
from helpers import np_of, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _tiny(algo, bits, k_chunk=8, n_tb=8):
    model = G.build_model("tiny-llama-test", algo, bits, group_size=128, seed=5)
    model.setup_caches(1, 64)
    th = G.calibrate_thresholds(model, seq_len=48, passes=1)
    data = G.random_dec_data(model, th, residual_scale=2e-3)
    model.load_dec_data(data)
    model.create_dec_context(n_tb, buffer_size=1024)
    model.set_dec_config([k_chunk] * 4)
    return model, data


def _base_weight(lin, algo):
    if algo == "sqllm":
        return O.sqllm_dequant(lin.qweight.cpu().numpy(), np_of(lin.lut), lin.bitwidth)
    if algo == "anyprec":
        return O.anyprec_dequant(lin.qweight.cpu().numpy(), np_of(lin.lut), lin.bitwidth)
    return O.lutgemm_dequant(lin.qweight.cpu().numpy(), np_of(lin.alpha), np_of(lin.q_bias), lin.group_size)


@pytest.mark.parametrize("algo,bits", [("sqllm", 4), ("anyprec", 3), ("lutgemm", 3)])
def test_every_linear_of_a_decode_step_matches_the_oracle(algo, bits):
    k_chunk = 8
    model, data = _tiny(algo, bits, k_chunk)
    seen = {}
    hooks = []
    for i, layer in enumerate(model.layers):
        for key, lin in zip(DEC_MODULE_KEYS, layer.dec_linears()):
            name = f"layers.{i}.{key}"
            hooks.append(lin.register_forward_hook(
                lambda m, inp, out, name=name: seen.__setitem__(name, (inp[0].detach().clone(), out.detach().clone()))))
    with torch.no_grad():
        model(torch.randint(0, model.config.vocab_size, (1, 20), device="cuda"), torch.arange(20, device="cuda"))   # prefill
        seen.clear()
        model(torch.tensor([[7]], device="cuda"), torch.tensor([20], device="cuda"))
        torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    assert len(seen) == 4 * model.config.n_layer
    for i, layer in enumerate(model.layers):
        for key, lin in zip(DEC_MODULE_KEYS, layer.dec_linears()):
            name = f"layers.{i}.{key}"
            x, y = seen[name]
            assert x.shape == (1, 1, lin.in_features) and y.shape == (1, 1, lin.out_features)
            xn = np_of(x).reshape(-1)
            rows, _, _ = O.select_channels(xn, np_of(data[name + ".thresholds"]), k_chunk)
            want = _base_weight(lin, algo).astype(np.float64) @ xn.astype(np.float64)
            want = want + O.dec_apply(xn, data[name + ".q_residual"].numpy(), np_of(data[name + ".scales"]), rows)
            mre, mae = rel_err(np_of(y).reshape(-1), want)
            assert mre <= TOL, (name, mre, mae)


def test_graph_replays_equal_eager_steps():
    """A replay of the captured decode step against the same step run eagerly, first attempt, no retries.
    The step is made reproducible for this: every output of a linear layer receives exactly two atomic adds (one K
    range of the base GEMV, option sqllm_ktiles = 1, and one DEC chunk group, option dec_max_chunk_groups = 1), and a
    sum of two terms into a zeroed output does not depend on their order; the attention of this short sequence is
    scanned by one workgroup per head.  Run-to-run differences of a rounding step, which could move an activation
    across a bucket floor and make DEC pick another channel, therefore cannot arise, and a replay that reads stale
    memory or a stale pointer has nowhere to hide.  The thresholds are moved off the calibration values by 2^-6
    as well, so that no activation of the calibration pass sits exactly on a floor."""
    from decdec_amd import _lib
    model = G.build_model("tiny-llama-test", "sqllm", 4, group_size=128, seed=5)
    model.setup_caches(1, 64)
    th = G.calibrate_thresholds(model, seq_len=48, passes=1)
    th = {k: (v.float() * (1.0 + 2.0 ** -6)).to(v.dtype) for k, v in th.items()}
    _lib.set_option("sqllm_ktiles", 1)
    _lib.set_option("dec_max_chunk_groups", 1)
    try:
        model.load_dec_data(G.random_dec_data(model, th, residual_scale=2e-3))
        model.create_dec_context(8, buffer_size=1024)
        model.set_dec_config([8] * 4)
        with torch.no_grad():
            model(torch.randint(0, model.config.vocab_size, (1, 16), device="cuda"), torch.arange(16, device="cuda"))
        step = G.DecodeStep(model, max_tokens=16, keep_logits=True)
        step.start(3, 16)
        step.capture()
        exact = 0
        for it, (tok, pos) in enumerate([(3, 16), (11, 17), (5, 18), (3, 16)]):
            step.start(tok, pos)
            with torch.no_grad():
                step._step()
            torch.cuda.synchronize()
            eager = step.logits.clone()
            junk = torch.randn(512, 512, device="cuda") @ torch.randn(512, 512, device="cuda")  # unrelated work between
            step.start(tok, pos)
            step.graph.replay()
            torch.cuda.synchronize()
            assert int(step.pos) == pos + 1 and int(step.count) == 1
            assert int(step.seq[0]) == int(torch.argmax(step.logits))
            mre, _ = rel_err(step.logits.cpu().numpy().reshape(-1), eager.cpu().numpy().reshape(-1).astype(np.float64))
            exact += int(torch.equal(step.logits, eager))
            del junk
            assert mre <= TOL, (it, mre)
        print(f"replays bit-identical to the eager step: {exact} of 4")
    finally:
        _lib.set_option("sqllm_ktiles", 0)
        _lib.set_option("dec_max_chunk_groups", 0)


def test_generate_runs_prefill_and_graph_decode():
    model, _ = _tiny("sqllm", 4)
    prompt = torch.randint(0, model.config.vocab_size, (24,), device="cuda")
    seq, dt = G.generate(model, prompt, max_new_tokens=9, use_graph=True, max_seq_length=64)
    assert seq.shape == (33,) and torch.equal(seq[:24], prompt) and dt > 0
    assert int(seq.min()) >= 0 and int(seq.max()) < model.config.vocab_size
