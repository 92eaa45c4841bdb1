"""Argument checks of the decdec_ext op surface (no GPU): every violation raises RuntimeError before
anything is launched, with the reference's TORCH_CHECK wording (decdec.cu, dec_config.cu,
dec_context.cu)."""
import pytest
import torch

import decdec_ext
from decdec_amd import ext


def test_drop_in_module_exposes_the_reference_api():
    for name in ("create_dec_context", "create_dec_config", "read_dec_config", "update_dec_config",
                 "destroy_dec_config", "dec", "unfused_dec", "anyprec_dequant", "anyprec_gemv", "lutgemm_gemv",
                 "sqllm_gemv", "dec_anyprec", "dec_lutgemm", "dec_sqllm", "dummy_anyprec", "dummy_lutgemm",
                 "dummy_sqllm"):                               # bindings.cpp:19-40
        assert callable(getattr(decdec_ext, name)), name
    assert len(ext.REFERENCE_API) == 17


def test_create_dec_context_checks():
    rows = torch.zeros(16, dtype=torch.int32); acts = torch.zeros(16, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="selected_rows_buffer must be on GPU"):
        ext.create_dec_context(8, rows, acts)


def test_create_dec_config_checks():
    q = torch.zeros(64, 8, dtype=torch.int32); s = torch.zeros(64, dtype=torch.float16)
    th = torch.zeros(64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="same data type"):
        ext.create_dec_config(0, 8, q, s, th.float())
    with pytest.raises(RuntimeError, match="q_residual must be of type int"):
        ext.create_dec_config(0, 8, q.long(), s, th)
    with pytest.raises(RuntimeError, match="q_residual must be contiguous"):
        ext.create_dec_config(0, 8, torch.zeros(8, 64, dtype=torch.int32).t(), s, th)
    with pytest.raises(RuntimeError, match="Unsupported data type"):
        ext.create_dec_config(0, 8, q, s.double(), th.double())
    with pytest.raises(RuntimeError, match="invalid DECContext handle"):
        ext.create_dec_config(0, 8, q, s, th)


def _t(*shape, dtype=torch.float16):
    return torch.zeros(*shape, dtype=dtype)


def test_dec_checks_run_before_any_launch():
    with pytest.raises(RuntimeError, match="Mismatched data types between input and output"):
        ext.dec(0, _t(1, 1, 64), _t(1, 1, 64, dtype=torch.float32))
    with pytest.raises(RuntimeError, match="must be on GPU"):
        ext.dec(0, _t(1, 1, 64), _t(1, 1, 64))


def test_anyprec_checks():
    x, out = _t(1, 1, 1024), _t(1, 1, 8)
    qw, lut = torch.zeros(3, 8, 32, dtype=torch.int32), _t(8, 8)
    with pytest.raises(RuntimeError, match="Bitwidth must be between 3 and 8"):
        ext.anyprec_gemv(x, out, qw, lut, 2)
    with pytest.raises(RuntimeError, match="Mismatched data types"):
        ext.anyprec_gemv(x, out, qw, lut.float(), 3)
    with pytest.raises(RuntimeError, match="qweight tensor must be of type int"):
        ext.anyprec_gemv(x, out, qw.long(), lut, 3)
    with pytest.raises(RuntimeError, match="lut tensor must be of shape"):
        ext.anyprec_gemv(x, out, qw, _t(8, 16), 3)
    with pytest.raises(RuntimeError, match="qweight tensor must be of shape"):
        ext.anyprec_gemv(x, out, torch.zeros(3, 8, 16, dtype=torch.int32), lut, 3)
    with pytest.raises(RuntimeError, match="Only sequence length of 1"):
        ext.anyprec_gemv(_t(1, 2, 1024), out, qw, lut, 3)
    with pytest.raises(RuntimeError, match="must be on GPU"):
        ext.anyprec_gemv(x, out, qw, lut, 3)
    with pytest.raises(RuntimeError, match="does not support float"):
        ext.anyprec_dequant(qw, lut.float(), 3)


def test_lutgemm_and_sqllm_checks():
    x, out = _t(1, 1, 1024), _t(1, 1, 8)
    qw = torch.zeros(32, 3, 8, dtype=torch.int32); alpha = _t(8, 3, 8); qb = _t(8, 8)
    with pytest.raises(RuntimeError, match="Bitwidth must be between 1 and 8"):
        ext.lutgemm_gemv(x, out, qw, alpha, qb, 0, 128)
    with pytest.raises(RuntimeError, match="Batch size must be 1"):
        ext.lutgemm_gemv(_t(2, 1, 1024), out, qw, alpha, qb, 3, 128)
    with pytest.raises(RuntimeError, match="must be on GPU"):
        ext.lutgemm_gemv(x, out, qw, alpha, qb, 3, 128)
    with pytest.raises(RuntimeError, match="Bitwidth must be 3 or 4"):
        ext.sqllm_gemv(x, out, torch.zeros(96, 8, dtype=torch.int32), _t(8, 8), 5)
    with pytest.raises(RuntimeError, match="must be on GPU"):
        ext.sqllm_gemv(x, out, torch.zeros(96, 8, dtype=torch.int32), _t(8, 8), 3)
    # the reference's own tests/test_awq.py passes (x, qweight, alpha, q_bias, output, ...): with the binding's
    # real order (input, output, q_weight, alpha, q_bias) that call fails the dtype check, as it does upstream
    with pytest.raises(RuntimeError, match="Mismatched data types"):
        ext.lutgemm_gemv(x, qw, alpha, qb, out, 3, 128)
