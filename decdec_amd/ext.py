"""The reference's ``decdec_ext`` op surface on top of libdecdec_hip.so.

Same function names, positional arguments and error behaviour (RuntimeError) as the reference's
pybind module (decdec_extension/bindings.cpp:19-40); the checks below follow the TORCH_CHECKs of
decdec_extension/decdec.cu, dec_config.cu and dec_context.cu in the same order.  PyTorch tensors
are only used for their device pointers, dtypes and shapes; all work happens in the HIP library.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib

_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_DT_NAME = {torch.float32: "FP32", torch.float16: "FP16", torch.bfloat16: "BF16"}

# config handle -> tensors whose storage the config borrows (thresholds) -- the reference leaves
# keeping them alive to the caller; holding a reference here costs nothing and removes a hazard
_KEEPALIVE: dict[int, tuple] = {}
# context handle -> the two scratch tensors the context borrows (same reasoning: a context whose buffers were
# garbage-collected would let DEC write its selection into whatever the allocator put there next)
_CONTEXT_KEEPALIVE: dict[int, tuple] = {}
_CONFIG_DTYPE: dict[int, torch.dtype] = {}
_CONFIG_SHAPE: dict[int, tuple[int, int]] = {}


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor) -> int:
    return t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    if t.dtype not in _DT:
        raise RuntimeError("Unsupported data type.")
    return _DT[t.dtype]


# ------------------------------------------------------------------------------------------------
# DECContext / DECConfig
# ------------------------------------------------------------------------------------------------
def create_dec_context(num_tb: int, selected_rows_buffer: torch.Tensor,
                       selected_activations_buffer: torch.Tensor) -> int:
    """dec_context.cu:62-103."""
    _check(selected_rows_buffer.is_cuda, "selected_rows_buffer must be on GPU.")
    _check(selected_activations_buffer.is_cuda, "selected_activations_buffer must be on GPU.")
    _check(selected_rows_buffer.numel() == selected_activations_buffer.numel(),
           "selected_rows_buffer and selected_activations_buffer must be of the same size.")
    _check(selected_rows_buffer.dtype == torch.int32, "selected_rows_buffer must be of type int.")
    _check(selected_rows_buffer.is_contiguous(), "selected_rows_buffer must be contiguous.")
    _check(selected_activations_buffer.is_contiguous(), "selected_activations_buffer must be contiguous.")
    dt = _dt(selected_activations_buffer)
    handle = ctypes.c_uint64(0)
    _lib.check(_lib.load().decdec_create_dec_context(
        int(num_tb), dt, selected_activations_buffer.numel(), _ptr(selected_rows_buffer),
        _ptr(selected_activations_buffer), ctypes.byref(handle)))
    _CONTEXT_KEEPALIVE[int(handle.value)] = (selected_rows_buffer, selected_activations_buffer)
    return int(handle.value)


def destroy_dec_context(dec_context: int) -> None:
    """Not in the reference (which leaks contexts); releases the sub-stream and event."""
    _lib.check(_lib.load().decdec_destroy_dec_context(int(dec_context)))
    _CONTEXT_KEEPALIVE.pop(int(dec_context), None)


def create_dec_config(dec_context: int, k_chunk: int, q_residual: torch.Tensor,
                      reordered_scales: torch.Tensor, thresholds: torch.Tensor) -> int:
    """dec_config.cu:247-292 (+ templated part :186-244)."""
    _check(thresholds.device.type == "cpu", "thresholds must be on CPU.")
    _check(reordered_scales.dtype == thresholds.dtype,
           "reordered_scales and thresholds must have the same data type.")
    _check(q_residual.dtype == torch.int32, "q_residual must be of type int.")
    _check(q_residual.is_contiguous(), "q_residual must be contiguous.")
    _check(reordered_scales.is_contiguous(), "reordered_scales must be contiguous.")
    _check(thresholds.is_contiguous(), "thresholds must be contiguous.")
    _check(reordered_scales.dtype in _DT, "Unsupported data type in create_dec_config.")
    _check(q_residual.dim() == 2 and reordered_scales.dim() == 1,
           "q_residual must be [in_features, out_features / 8] and reordered_scales [out_features].")
    num_rows = q_residual.size(0)
    num_cols = reordered_scales.size(0)
    _check(q_residual.size(1) == num_cols // 8 and num_cols % 8 == 0,
           "q_residual.size(1) must equal reordered_scales.size(0) / 8.")
    _check(thresholds.numel() >= num_rows, "thresholds must have in_features elements.")
    handle = ctypes.c_uint64(0)
    _lib.check(_lib.load().decdec_create_dec_config(
        int(dec_context), int(k_chunk), _DT[reordered_scales.dtype],
        _ptr(q_residual), int(q_residual.is_cuda),
        _ptr(reordered_scales), int(reordered_scales.is_cuda),
        _ptr(thresholds), num_rows, num_cols, ctypes.byref(handle)))
    h = int(handle.value)
    # a device-resident residual is used in place, so it must stay alive as well
    _KEEPALIVE[h] = (thresholds, q_residual if q_residual.is_cuda else None)
    _CONFIG_DTYPE[h] = reordered_scales.dtype
    _CONFIG_SHAPE[h] = (num_rows, num_cols)
    return h


def read_dec_config(dec_config: int, native: bool = False) -> dict:
    """dec_config.cu:337-354.  The nine reference keys; ``native=True`` adds the ``hip_*`` launch plan."""
    info = _lib.ConfigInfo()
    _lib.check(_lib.load().decdec_read_dec_config(int(dec_config), ctypes.byref(info)))
    out = {k: int(getattr(info, k)) for k in _lib.REFERENCE_KEYS}
    if native:
        out.update({name: int(getattr(info, name)) for name, _ in _lib.ConfigInfo._fields_
                    if name.startswith("hip_")})
    return out


def update_dec_config(dec_config: int, new_dec_context: int, k_chunk: int) -> None:
    """dec_config.cu:295-326."""
    _lib.check(_lib.load().decdec_update_dec_config(int(dec_config), int(new_dec_context), int(k_chunk)))


def destroy_dec_config(dec_config: int) -> None:
    """dec_config.cu:329-334."""
    _lib.check(_lib.load().decdec_destroy_dec_config(int(dec_config)))
    _KEEPALIVE.pop(int(dec_config), None)
    _CONFIG_DTYPE.pop(int(dec_config), None)
    _CONFIG_SHAPE.pop(int(dec_config), None)


# ------------------------------------------------------------------------------------------------
# shared checks
# ------------------------------------------------------------------------------------------------
def _check_dec_io(dec_config: int, input: torch.Tensor, output: torch.Tensor) -> None:
    """decdec.cu:99-126."""
    _check(input.dtype == output.dtype,
           f"Mismatched data types between input and output tensors. input type: {input.dtype}, "
           f"output type: {output.dtype}")
    _check(input.is_cuda and output.is_cuda, "input and output tensors must be on GPU.")
    cfg_dtype = _CONFIG_DTYPE.get(int(dec_config))
    _check(cfg_dtype is not None, "invalid DECConfig handle")
    _check(input.dtype in _DT, "Unsupported data type.")
    _check(input.dtype == cfg_dtype,
           "Mismatched data types between input tensor and DECConfig. input type: "
           f"{_DT_NAME[input.dtype]}, DECConfig type: {_DT_NAME[cfg_dtype]}")
    _check(input.dim() == 3, "input tensor must be of shape (batch_size, seq_len, hidden_size).")
    _check(output.dim() == 3, "output tensor must be of shape (batch_size, seq_len, hidden_size).")
    _check(input.size(0) == 1, "Batch size must be 1 for input tensor.")
    _check(output.size(0) == 1, "Batch size must be 1 for output tensor.")
    _check(input.size(1) == 1, "Sequence length must be 1 for input tensor.")
    _check(output.size(1) == 1, "Sequence length must be 1 for output tensor.")
    rows, cols = _CONFIG_SHAPE[int(dec_config)]
    _check(input.size(2) == rows,
           f"input tensor size does not match with DECConfig: input size: {input.size(2)}, DECConfig size: {rows}")
    _check(output.size(2) == cols,
           f"output tensor size does not match with DECConfig: output size: {output.size(2)}, DECConfig size: {cols}")
    _check(input.is_contiguous(), "input tensor must be contiguous.")
    _check(output.is_contiguous(), "output tensor must be contiguous.")


def _check_anyprec(input, output, qweight, lut, bitwidth) -> None:
    """decdec.cu:283-321."""
    _check(3 <= bitwidth <= 8, "Bitwidth must be between 3 and 8.")
    _check(input.dtype == lut.dtype and input.dtype == output.dtype,
           "Mismatched data types between input, lut, and output tensors.")
    _check(qweight.dtype == torch.int32, "qweight tensor must be of type int.")
    _check(input.dim() == 3, "input tensor must be of shape (batch_size, seq_len, hidden_size).")
    _check(output.dim() == 3, "output tensor must be of shape (batch_size, seq_len, hidden_size).")
    _check(lut.dim() == 2 and lut.size(1) == (1 << bitwidth) and lut.size(0) == output.size(2),
           f"lut tensor must be of shape (output_feat, 2 ** bitwidth). Expected ({output.size(2)}, "
           f"{1 << bitwidth}), got ({lut.size(0) if lut.dim() > 0 else '?'}, {lut.size(1) if lut.dim() > 1 else '?'}).")
    _check(qweight.dim() == 3 and qweight.size(0) >= bitwidth and qweight.size(2) == input.size(2) // 32
           and qweight.size(1) == output.size(2),
           "qweight tensor must be of shape (>=bitwidth, output_feat, input_feat / 32). Expected (>="
           f"{bitwidth}, {output.size(2)}, {input.size(2) // 32}), got {tuple(qweight.shape)}.")
    _check(input.size(1) == 1, "Only sequence length of 1 is supported.")
    _check(output.size(1) == 1, "Only sequence length of 1 is supported.")
    # the reference indexes rows of a batch (M <= 8) it never launches with; batch 1 is the op's contract
    _check(input.size(0) == 1 and output.size(0) == 1, "Batch size must be 1.")
    _check(input.is_cuda and output.is_cuda, "input and output tensors must be on GPU.")
    _check(qweight.is_cuda and lut.is_cuda, "qweight and lut tensors must be on GPU.")
    _check(input.is_contiguous(), "input tensor must be contiguous.")
    _check(output.is_contiguous(), "output tensor must be contiguous.")
    _check(qweight.is_contiguous(), "qweight tensor must be contiguous.")
    _check(lut.is_contiguous(), "lut tensor must be contiguous.")
    if input.dtype == torch.float32:
        raise RuntimeError("Any-Precision GEMV does not support float data type. Please use half or bfloat16.")
    _check(input.dtype in (torch.float16, torch.bfloat16), "Unsupported data type.")


def _check_lutgemm(input, output, q_weight, alpha, q_bias, bitwidth, group_size) -> None:
    """decdec.cu:440-482."""
    _check(1 <= bitwidth <= 8, "Bitwidth must be between 1 and 8.")
    _check(input.dtype == alpha.dtype and input.dtype == q_bias.dtype and input.dtype == output.dtype,
           "Mismatched data types between input, alpha, q_bias, and output tensors.")
    _check(input.dim() == 3, "input tensor must be of shape (batch_size, seq_len, input_feat).")
    _check(output.dim() == 3, "output tensor must be of shape (batch_size, seq_len, output_feat).")
    _check(input.size(0) == 1, "Batch size must be 1 for input tensor.")
    _check(input.size(1) == 1, "Sequence length must be 1 for input tensor.")
    _check(output.size(0) == 1, "Batch size must be 1 for output tensor.")
    _check(output.size(1) == 1, "Sequence length must be 1 for output tensor.")
    _check(input.is_cuda and output.is_cuda, "input and output tensors must be on GPU.")
    _check(q_weight.is_cuda and alpha.is_cuda and q_bias.is_cuda, "q_weight, alpha and q_bias tensors must be on GPU.")
    _check(input.is_contiguous(), "input tensor must be contiguous.")
    _check(output.is_contiguous(), "output tensor must be contiguous.")
    _check(q_weight.is_contiguous(), "q_weight tensor must be contiguous.")
    _check(alpha.is_contiguous(), "alpha tensor must be contiguous.")
    _check(q_bias.is_contiguous(), "q_bias tensor must be contiguous.")
    _check(q_weight.dtype == torch.int32, "q_weight tensor must be of type int.")
    _check(group_size > 0, "group_size must be positive.")
    k_size, m_size = input.size(2), output.size(2)
    num_groups = k_size // group_size
    _check(q_weight.dim() == 3 and q_weight.size(0) == k_size // 32 and q_weight.size(1) == bitwidth
           and q_weight.size(2) == m_size,
           "q_weight tensor must be of shape (input_feat / 32, bitwidth, output_feat). Expected ("
           f"{k_size // 32}, {bitwidth}, {m_size}), got {tuple(q_weight.shape)}.")
    _check(alpha.dim() == 3 and alpha.size(0) == num_groups and alpha.size(1) == bitwidth and alpha.size(2) == m_size,
           "alpha tensor must be of shape (num_groups, bitwidth, output_feat). Expected ("
           f"{num_groups}, {bitwidth}, {m_size}), got {tuple(alpha.shape)}.")
    _check(q_bias.dim() == 2 and q_bias.size(0) == num_groups and q_bias.size(1) == m_size,
           f"q_bias tensor must be of shape (num_groups, output_feat). Expected ({num_groups}, {m_size}), "
           f"got {tuple(q_bias.shape)}.")
    _check(input.dtype in _DT, "Unsupported data type.")


def _check_sqllm(input, output, qweight, lut, bitwidth) -> None:
    """decdec.cu:552-591."""
    _check(bitwidth in (3, 4), "Bitwidth must be 3 or 4.")
    _check(input.dtype == lut.dtype and input.dtype == output.dtype,
           "Mismatched data types between input, lut, and output tensors.")
    _check(qweight.dtype == torch.int32, "qweight tensor must be of type int.")
    _check(input.dim() == 3, "input tensor must be of shape (batch_size, seq_len, hidden_size).")
    _check(output.dim() == 3, "output tensor must be of shape (batch_size, seq_len, hidden_size).")
    _check(input.size(0) == 1, "Batch size must be 1 for input tensor.")
    _check(input.size(1) == 1, "Sequence length must be 1 for input tensor.")
    _check(output.size(0) == 1, "Batch size must be 1 for output tensor.")
    _check(output.size(1) == 1, "Sequence length must be 1 for output tensor.")
    _check(input.is_cuda and output.is_cuda, "input and output tensors must be on GPU.")
    _check(qweight.is_cuda and lut.is_cuda, "qweight and lut tensors must be on GPU.")
    _check(lut.dim() == 2 and lut.size(1) == (1 << bitwidth) and lut.size(0) == output.size(2),
           f"lut tensor must be of shape (output_feat, 2 ** bitwidth). Expected ({output.size(2)}, "
           f"{1 << bitwidth}), got {tuple(lut.shape)}.")
    _check(qweight.dim() == 2 and qweight.size(1) == lut.size(0)
           and qweight.size(0) == input.size(2) * bitwidth // 32,
           "qweight tensor must be of shape (input_feat * bitwidth / 32, output_feat). Expected ("
           f"{input.size(2) * bitwidth // 32}, {lut.size(0)}), got {tuple(qweight.shape)}.")
    _check(input.is_contiguous(), "input tensor must be contiguous.")
    _check(output.is_contiguous(), "output tensor must be contiguous.")
    _check(qweight.is_contiguous(), "qweight tensor must be contiguous.")
    _check(lut.is_contiguous(), "lut tensor must be contiguous.")
    _check(input.dtype in _DT, "Unsupported data type.")


# ------------------------------------------------------------------------------------------------
# ops
# ------------------------------------------------------------------------------------------------
def dec(dec_config: int, input: torch.Tensor, output: torch.Tensor) -> None:
    """decdec.cu:139-146."""
    _check_dec_io(dec_config, input, output)
    _lib.check(_lib.load().decdec_dec(int(dec_config), _ptr(input), _ptr(output), _dt(input),
                                      input.size(2), output.size(2), _stream()))


def unfused_dec(dec_config: int, input: torch.Tensor, output: torch.Tensor) -> None:
    """decdec.cu:238-245."""
    _check_dec_io(dec_config, input, output)
    _lib.check(_lib.load().decdec_unfused_dec(int(dec_config), _ptr(input), _ptr(output), _dt(input),
                                              input.size(2), output.size(2), _stream()))


def anyprec_gemv(input, output, qweight, lut, bitwidth: int) -> None:
    """decdec.cu:324-333."""
    _check_anyprec(input, output, qweight, lut, bitwidth)
    _lib.check(_lib.load().decdec_anyprec_gemv(_ptr(input), _ptr(output), _ptr(qweight), _ptr(lut), int(bitwidth),
                                               _dt(input), input.size(2), output.size(2), _stream()))


def anyprec_dequant(qweight: torch.Tensor, lut: torch.Tensor, bitwidth: int) -> torch.Tensor:
    """decdec.cu:386-393: returns the dense [out_features, in_features] weight."""
    _check(qweight.dim() == 3 and qweight.dtype == torch.int32, "qweight tensor must be a 3-D int tensor.")
    if lut.dtype == torch.float32:
        raise RuntimeError("Any-Precision Dequantization does not support float data type. "
                           "Please use half or bfloat16.")
    _check(lut.dtype in (torch.float16, torch.bfloat16), "Unsupported data type.")
    _check(qweight.is_cuda and lut.is_cuda and qweight.device == lut.device, "qweight and lut must be on the same GPU.")
    _check(3 <= bitwidth <= 8, "Bitwidth must be between 3 and 8.")
    _check(qweight.size(0) >= bitwidth, "qweight has fewer bit planes than bitwidth.")
    _check(lut.dim() == 2 and lut.size(0) == qweight.size(1) and lut.size(1) == (1 << bitwidth),
           "lut tensor must be of shape (output_feat, 2 ** bitwidth).")
    _check(qweight.is_contiguous() and lut.is_contiguous(), "qweight and lut must be contiguous.")
    n, k = qweight.size(1), qweight.size(2) * 32
    weight = torch.empty((n, k), dtype=lut.dtype, device=qweight.device)
    _lib.check(_lib.load().decdec_anyprec_dequant(_ptr(qweight), _ptr(lut), _ptr(weight), int(bitwidth),
                                                  _DT[lut.dtype], n, k, _stream()))
    return weight


def lutgemm_gemv(input, output, q_weight, alpha, q_bias, bitwidth: int, group_size: int) -> None:
    """decdec.cu:485-496."""
    _check_lutgemm(input, output, q_weight, alpha, q_bias, bitwidth, group_size)
    _lib.check(_lib.load().decdec_lutgemm_gemv(_ptr(input), _ptr(output), _ptr(q_weight), _ptr(alpha), _ptr(q_bias),
                                               int(bitwidth), int(group_size), _dt(input), input.size(2),
                                               output.size(2), _stream()))


def sqllm_gemv(input, output, qweight, lut, bitwidth: int) -> None:
    """decdec.cu:594-603."""
    _check_sqllm(input, output, qweight, lut, bitwidth)
    _lib.check(_lib.load().decdec_sqllm_gemv(_ptr(input), _ptr(output), _ptr(qweight), _ptr(lut), int(bitwidth),
                                             _dt(input), input.size(2), output.size(2), _stream()))


def dec_anyprec(dec_config: int, input, output, q_weight, lut, bitwidth: int) -> None:
    """decdec.cu:643-659."""
    _check(input.dtype in (torch.float16, torch.bfloat16), "Unsupported data type.")
    _check_dec_io(dec_config, input, output)
    _check_anyprec(input, output, q_weight, lut, bitwidth)
    _lib.check(_lib.load().decdec_dec_anyprec(int(dec_config), _ptr(input), _ptr(output), _ptr(q_weight), _ptr(lut),
                                              int(bitwidth), _dt(input), input.size(2), output.size(2), _stream()))


def dec_anyprec_batch(dec_configs, input, outputs, q_weights, luts, bitwidth: int) -> None:
    """Layers that read the same `input`, in one launch: layer i is dec_anyprec(dec_configs[i], input, outputs[i],
    q_weights[i], luts[i], bitwidth), or anyprec_gemv when dec_configs[i] is 0 / None (dec_configs may be None).
    Not in the reference (which concatenates such projections' weights instead)."""
    n = len(outputs)
    _check(1 <= n <= 4 and len(q_weights) == n and len(luts) == n, "a batch holds 1 to 4 layers")
    cfgs = [int(c) if c else 0 for c in (dec_configs if dec_configs is not None else [0] * n)]
    _check(len(cfgs) == n, "one config (or 0) per layer")
    _check(input.dtype in (torch.float16, torch.bfloat16), "Unsupported data type.")
    for c, out, qw, lut in zip(cfgs, outputs, q_weights, luts):
        if c:
            _check_dec_io(c, input, out)
        _check_anyprec(input, out, qw, lut, bitwidth)
    arr_c = (ctypes.c_uint64 * n)(*cfgs)
    arr_o = (ctypes.c_void_p * n)(*[_ptr(t) for t in outputs])
    arr_q = (ctypes.c_void_p * n)(*[_ptr(t) for t in q_weights])
    arr_l = (ctypes.c_void_p * n)(*[_ptr(t) for t in luts])
    arr_n = (ctypes.c_uint32 * n)(*[t.size(2) for t in outputs])
    _lib.check(_lib.load().decdec_dec_anyprec_batch(n, arr_c, _ptr(input), arr_o, arr_q, arr_l, int(bitwidth), _dt(input),
                                                    input.size(2), arr_n, _stream()))


def dec_lutgemm(dec_config: int, input, output, q_weight, alpha, q_bias, bitwidth: int, group_size: int) -> None:
    """decdec.cu:701-721."""
    _check(input.dtype in _DT, "Unsupported data type.")
    _check_dec_io(dec_config, input, output)
    _check_lutgemm(input, output, q_weight, alpha, q_bias, bitwidth, group_size)
    _lib.check(_lib.load().decdec_dec_lutgemm(int(dec_config), _ptr(input), _ptr(output), _ptr(q_weight), _ptr(alpha),
                                              _ptr(q_bias), int(bitwidth), int(group_size), _dt(input),
                                              input.size(2), output.size(2), _stream()))


def dec_sqllm(dec_config: int, input, output, q_weight, lut, bitwidth: int) -> None:
    """decdec.cu:761-779."""
    _check(input.dtype in _DT, "Unsupported data type.")
    _check_dec_io(dec_config, input, output)
    _check_sqllm(input, output, q_weight, lut, bitwidth)
    _lib.check(_lib.load().decdec_dec_sqllm(int(dec_config), _ptr(input), _ptr(output), _ptr(q_weight), _ptr(lut),
                                            int(bitwidth), _dt(input), input.size(2), output.size(2), _stream()))


def _batch_arrays(dec_configs, input, outputs, per_layer):
    n = len(outputs)
    _check(1 <= n <= 4 and all(len(seq) == n for seq in per_layer), "a batch holds 1 to 4 layers")
    cfgs = [int(c) if c else 0 for c in (dec_configs if dec_configs is not None else [0] * n)]
    _check(len(cfgs) == n, "one config (or 0) per layer")
    for c, out in zip(cfgs, outputs):
        if c:
            _check_dec_io(c, input, out)
    arr_c = (ctypes.c_uint64 * n)(*cfgs)
    arr_o = (ctypes.c_void_p * n)(*[_ptr(t) for t in outputs])
    arrs = [(ctypes.c_void_p * n)(*[_ptr(t) for t in seq]) for seq in per_layer]
    arr_n = (ctypes.c_uint32 * n)(*[t.size(2) for t in outputs])
    return n, arr_c, arr_o, arrs, arr_n


def dec_lutgemm_batch(dec_configs, input, outputs, q_weights, alphas, q_biases, bitwidth: int, group_size: int) -> None:
    """Layers that read the same `input`, in one launch: layer i is dec_lutgemm(dec_configs[i], input, outputs[i],
    q_weights[i], alphas[i], q_biases[i], bitwidth, group_size), or lutgemm_gemv when dec_configs[i] is 0 / None.
    Not in the reference."""
    _check(input.dtype in _DT, "Unsupported data type.")
    n, arr_c, arr_o, (arr_q, arr_a, arr_b), arr_n = _batch_arrays(dec_configs, input, outputs, (q_weights, alphas, q_biases))
    for out, qw, al, qb in zip(outputs, q_weights, alphas, q_biases):
        _check_lutgemm(input, out, qw, al, qb, bitwidth, group_size)
    _lib.check(_lib.load().decdec_dec_lutgemm_batch(n, arr_c, _ptr(input), arr_o, arr_q, arr_a, arr_b, int(bitwidth),
                                                    int(group_size), _dt(input), input.size(2), arr_n, _stream()))


def dec_sqllm_batch(dec_configs, input, outputs, q_weights, luts, bitwidth: int) -> None:
    """Layers that read the same `input`, in one launch: layer i is dec_sqllm(dec_configs[i], input, outputs[i],
    q_weights[i], luts[i], bitwidth), or sqllm_gemv when dec_configs[i] is 0 / None.  Not in the reference."""
    _check(input.dtype in _DT, "Unsupported data type.")
    n, arr_c, arr_o, (arr_q, arr_l), arr_n = _batch_arrays(dec_configs, input, outputs, (q_weights, luts))
    for out, qw, lut in zip(outputs, q_weights, luts):
        _check_sqllm(input, out, qw, lut, bitwidth)
    _lib.check(_lib.load().decdec_dec_sqllm_batch(n, arr_c, _ptr(input), arr_o, arr_q, arr_l, int(bitwidth), _dt(input),
                                                  input.size(2), arr_n, _stream()))


def dummy_anyprec(input, output, qweight, lut, bitwidth: int, dummy_sm: int, dummy_iters: int) -> None:
    """decdec.cu:874-893."""
    _check(input.dtype in (torch.float16, torch.bfloat16), "dummy_anyprec supports FP16/BF16 only.")
    _check_anyprec(input, output, qweight, lut, bitwidth)
    _lib.check(_lib.load().decdec_dummy_anyprec(_ptr(input), _ptr(output), _ptr(qweight), _ptr(lut), int(bitwidth),
                                                _dt(input), input.size(2), output.size(2), int(dummy_sm),
                                                int(dummy_iters), _stream()))


def dummy_lutgemm(input, output, qweight, alpha, qbias, bitwidth: int, group_size: int,
                  dummy_sm: int, dummy_iters: int) -> None:
    """decdec.cu:930-956."""
    _check(input.dtype in _DT, "Unsupported dtype for dummy_lutgemm")
    _check_lutgemm(input, output, qweight, alpha, qbias, bitwidth, group_size)
    _lib.check(_lib.load().decdec_dummy_lutgemm(_ptr(input), _ptr(output), _ptr(qweight), _ptr(alpha), _ptr(qbias),
                                                int(bitwidth), int(group_size), _dt(input), input.size(2),
                                                output.size(2), int(dummy_sm), int(dummy_iters), _stream()))


def dummy_sqllm(input, output, qweight, lut, bitwidth: int, dummy_sm: int, dummy_iters: int) -> None:
    """decdec.cu:990-1013."""
    _check(bitwidth in (3, 4), "SQLLM bitwidth must be 3 or 4.")
    _check(input.dtype in _DT, "Unsupported dtype for dummy_sqllm")
    _check_sqllm(input, output, qweight, lut, bitwidth)
    _lib.check(_lib.load().decdec_dummy_sqllm(_ptr(input), _ptr(output), _ptr(qweight), _ptr(lut), int(bitwidth),
                                              _dt(input), input.size(2), output.size(2), int(dummy_sm),
                                              int(dummy_iters), _stream()))


REFERENCE_API = (
    "create_dec_context", "create_dec_config", "read_dec_config", "update_dec_config", "destroy_dec_config",
    "dec", "unfused_dec", "anyprec_dequant", "anyprec_gemv", "lutgemm_gemv", "sqllm_gemv",
    "dec_anyprec", "dec_lutgemm", "dec_sqllm", "dummy_anyprec", "dummy_lutgemm", "dummy_sqllm",
)
__all__ = list(REFERENCE_API) + ["destroy_dec_context", "dec_anyprec_batch", "dec_lutgemm_batch", "dec_sqllm_batch"]
