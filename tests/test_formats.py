"""decdec_amd.formats (the product's torch packers) against the oracle's NumPy restatements."""
import numpy as np
import pytest
import torch

from decdec_amd import formats as F
from oracle import decdec_oracle as O


@pytest.mark.parametrize("K", [1024, 2048 + 512])
@pytest.mark.parametrize("bits", [3, 4, 8])
def test_anyprec_pack(K, bits):
    g = torch.Generator().manual_seed(K + bits)
    idx = torch.randint(0, 1 << bits, (24, K), generator=g, dtype=torch.int64)
    q = F.pack_anyprec(idx, bits)
    assert np.array_equal(q.numpy(), O.anyprec_pack(idx.numpy().astype(np.uint8), bits))
    assert torch.equal(F.unpack_anyprec(q, bits), idx)


@pytest.mark.parametrize("bits", [3, 4])
def test_sqllm_pack(bits):
    g = torch.Generator().manual_seed(bits)
    idx = torch.randint(0, 1 << bits, (10, 512), generator=g, dtype=torch.int64)
    assert np.array_equal(F.pack_sqllm(idx, bits).numpy(), O.sqllm_pack(idx.numpy().astype(np.uint8), bits))


def test_bcq_pack_and_dequant():
    g = torch.Generator().manual_seed(1)
    W = (torch.randn(16, 512, generator=g) * 0.02).half()
    q, s, z = F.awq_pseudo_quantize(W, 3, 128)
    qw, alpha, qb = F.pack_bcq(q, s, z, 3, torch.float32)
    q2, s2, z2 = O.awq_pseudo_quantize(W.numpy(), 3, 128)
    qw2, alpha2, qb2 = O.bcq_pack(q2, s2, z2, 3)
    assert np.array_equal(qw.numpy(), qw2) and np.array_equal(alpha.numpy(), alpha2) and np.array_equal(qb.numpy(), qb2)
    assert np.allclose(F.dequant_bcq(qw, alpha, qb, 128).numpy(), O.lutgemm_dequant(qw2, alpha2, qb2, 128), atol=1e-6)


def test_residual_quantise_and_pack():
    g = torch.Generator().manual_seed(2)
    E = (torch.randn(32, 384, generator=g) * 0.003).half()
    q, s = F.quantize_residual(E)
    q2, s2 = O.quantize_residual(E.numpy())
    assert np.array_equal(s.numpy(), s2) and np.array_equal(q.numpy(), q2)
    c, r = F.pack_residual(q, s)
    c2, r2 = O.pack_residual(q2, s2)
    assert np.array_equal(c.numpy(), c2) and np.array_equal(r.numpy(), r2)
    assert np.allclose(F.unpack_residual(c, r).numpy(), O.unpack_residual(c2, r2), atol=0)


def test_uniform_row_quantiser_and_thresholds():
    g = torch.Generator().manual_seed(3)
    W = (torch.randn(8, 256, generator=g) * 0.02).half()
    idx, lut = F.quantize_uniform_rows(W, 3)
    Wq = F.dequant_lut(idx, lut)
    step = (W.float().amax(1) - W.float().amin(1)) / 7
    assert ((W.float() - Wq.float()).abs().amax(1) <= step * 0.51 + 1e-3).all()
    th = F.calibrate_thresholds(1024, g, draws=4)
    assert th.dtype == torch.float16 and (th[:-1] >= th[1:]).all()        # sorted by construction
    x = F.make_activation(1024, g)
    assert x.shape == (1, 1, 1024) and (x.abs() > 10).sum() >= 1            # the x20 outliers
