"""DEC side files of a checkpoint directory: ``cheatsheet.pt`` and ``thresholds.pt``.

Formats (reference decdec_setup/cheatsheet.py:117-125, :176-190 and thresholds.py:148-200):

* ``cheatsheet.pt``  -- list over decoder layers of ``{module_name: {"cheatsheet": int32 [K, N/8],
  "reordered_scales": fp16 [N]}}``, module names as in the Hugging Face model
  (``self_attn.q_proj`` ... ``mlp.down_proj``, or the fused ``self_attn.qkv_proj`` / ``mlp.gate_up_proj``);
* ``thresholds.pt``  -- list over layers of ``{module_name: thresholds [K]}``, element i = the largest
  i-th largest |activation| seen at the module's input over the calibration tokens.

``build_cheatsheet_entry`` / ``collect_thresholds`` write these from weights and activations;
``load_dec_data`` reads them back into the flat dictionary ``Transformer.load_dec_data`` takes
(reference end-to-end/loader.py:114-193), fusing q|k|v and gate|up.  Files are read with
``torch.load(weights_only=True)``: they hold tensors in lists and dicts, nothing else.
"""
from __future__ import annotations

import os
from typing import Callable, Dict, Iterable, List

import torch

from . import formats

CHEATSHEET_FILE = "cheatsheet.pt"
THRESHOLDS_FILE = "thresholds.pt"


# ----------------------------------------------------------------------------------------------------
# builders
# ----------------------------------------------------------------------------------------------------
def build_cheatsheet_entry(weight: torch.Tensor, quantized_weight: torch.Tensor) -> Dict[str, torch.Tensor]:
    """4-bit residual of one module: weight, quantized_weight [N, K] (original and dequantised base).
    Per output row: 32 candidate scales up to max|e|/7, round and clamp to [-7, 7], least fp32 MSE;
    packed eight outputs per int32 with the nibble q + 8 (reference cheatsheet.py:59-125)."""
    assert weight.shape == quantized_weight.shape and weight.shape[0] % 8 == 0
    err = (weight.to(torch.float16) - quantized_weight.to(torch.float16))
    q, scales = formats.quantize_residual(err)
    cheat, reordered = formats.pack_residual(q, scales)
    return {"cheatsheet": cheat.cpu(), "reordered_scales": reordered.cpu()}


class ThresholdCollector:
    """Forward hooks on the given modules; after the calibration passes ``result()`` holds, per module,
    thresholds[i] = max over tokens of the i-th largest |x| at the module's input
    (reference thresholds.py:162-175).  Inputs are [1, S, K] or [S, K]."""

    def __init__(self, named_modules: Iterable):
        self._th: Dict[str, torch.Tensor] = {}
        self._hooks = []
        for name, module in named_modules:
            self._hooks.append(module.register_forward_hook(self._make(name)))

    def _make(self, name: str) -> Callable:
        def hook(module, inputs, output):
            x = inputs[0].detach()
            x = x.reshape(-1, x.shape[-1]).float().abs()
            ranked = torch.sort(x, dim=1, descending=True).values.amax(dim=0)
            prev = self._th.get(name)
            self._th[name] = ranked if prev is None else torch.maximum(prev, ranked)
        return hook

    def close(self):
        for h in self._hooks:
            h.remove()
        self._hooks = []

    def result(self, dtype=torch.float16) -> Dict[str, torch.Tensor]:
        return {k: v.to(dtype).cpu() for k, v in self._th.items()}


def collect_thresholds(named_modules: Iterable, run: Callable[[], None], dtype=torch.float16) -> Dict[str, torch.Tensor]:
    """Runs ``run()`` (the calibration forward passes) with the hooks in place."""
    c = ThresholdCollector(named_modules)
    try:
        with torch.no_grad():
            run()
    finally:
        c.close()
    return c.result(dtype)


# ----------------------------------------------------------------------------------------------------
# files
# ----------------------------------------------------------------------------------------------------
def save_cheatsheet(ckpt_dir: str, layers: List[Dict[str, Dict[str, torch.Tensor]]]) -> str:
    os.makedirs(ckpt_dir, exist_ok=True)
    path = os.path.join(ckpt_dir, CHEATSHEET_FILE)
    torch.save([{m: {k: t.cpu() for k, t in e.items()} for m, e in layer.items()} for layer in layers], path)
    return path


def save_thresholds(ckpt_dir: str, layers: List[Dict[str, torch.Tensor]]) -> str:
    os.makedirs(ckpt_dir, exist_ok=True)
    path = os.path.join(ckpt_dir, THRESHOLDS_FILE)
    torch.save([{m: t.cpu() for m, t in layer.items()} for layer in layers], path)
    return path


def load_cheatsheet(ckpt_dir: str):
    return torch.load(os.path.join(ckpt_dir, CHEATSHEET_FILE), map_location="cpu", weights_only=True)


def load_thresholds(ckpt_dir: str):
    return torch.load(os.path.join(ckpt_dir, THRESHOLDS_FILE), map_location="cpu", weights_only=True)


# ----------------------------------------------------------------------------------------------------
# fusing modules
# ----------------------------------------------------------------------------------------------------
def natural_scales(reordered: torch.Tensor) -> torch.Tensor:
    """reordered[j N/8 + m] -> scales[8 m + j]."""
    N = reordered.numel()
    return reordered.reshape(8, N // 8).t().reshape(-1).contiguous()


def reorder_scales(scales: torch.Tensor) -> torch.Tensor:
    N = scales.numel()
    return scales.reshape(N // 8, 8).t().reshape(-1).contiguous()


def fuse_entries(entries: List[Dict[str, torch.Tensor]]) -> Dict[str, torch.Tensor]:
    """Residual of the module whose outputs are those of `entries` one after the other.  The packed words
    concatenate along the output axis as they are; the scales are brought back to output order,
    concatenated and reordered for the fused width -- the DEC kernel reads the scale of output 8 m + j at
    j N/8 + m with the FUSED N, so joining the per-module reordered vectors end to end (as the reference
    loader does, loader.py:131-138) matches only for projections that were fused when the file was made."""
    cheat = torch.cat([e["cheatsheet"] for e in entries], dim=1).contiguous()
    scales = torch.cat([natural_scales(e["reordered_scales"]) for e in entries], dim=0)
    return {"cheatsheet": cheat, "reordered_scales": reorder_scales(scales)}


def load_dec_data(ckpt_dir: str, dtype=torch.float16) -> Dict[str, torch.Tensor]:
    """``{"layers.{i}.attention.wqkv.q_residual" | ".scales" | ".thresholds": tensor, ...}`` for wqkv, wo,
    w1w3 and w2 of every layer (CPU tensors; scales and thresholds cast to `dtype`)."""
    out: Dict[str, torch.Tensor] = {}
    for i, layer in enumerate(load_cheatsheet(ckpt_dir)):
        qkv = layer["self_attn.qkv_proj"] if "self_attn.qkv_proj" in layer else fuse_entries(
            [layer["self_attn.q_proj"], layer["self_attn.k_proj"], layer["self_attn.v_proj"]])
        gu = layer["mlp.gate_up_proj"] if "mlp.gate_up_proj" in layer else fuse_entries(
            [layer["mlp.gate_proj"], layer["mlp.up_proj"]])
        for key, e in (("attention.wqkv", qkv), ("attention.wo", layer["self_attn.o_proj"]),
                       ("feed_forward.w1w3", gu), ("feed_forward.w2", layer["mlp.down_proj"])):
            out[f"layers.{i}.{key}.q_residual"] = e["cheatsheet"].to(torch.int32).contiguous()
            out[f"layers.{i}.{key}.scales"] = e["reordered_scales"].to(dtype).contiguous()
    for i, layer in enumerate(load_thresholds(ckpt_dir)):
        # q, k, v (gate, up) see the same input: one module's thresholds serve the fused projection
        pick = lambda fused, first: layer[fused] if fused in layer else layer[first]
        out[f"layers.{i}.attention.wqkv.thresholds"] = pick("self_attn.qkv_proj", "self_attn.q_proj").to(dtype)
        out[f"layers.{i}.attention.wo.thresholds"] = layer["self_attn.o_proj"].to(dtype)
        out[f"layers.{i}.feed_forward.w1w3.thresholds"] = pick("mlp.gate_up_proj", "mlp.gate_proj").to(dtype)
        out[f"layers.{i}.feed_forward.w2.thresholds"] = layer["mlp.down_proj"].to(dtype)
    return out
