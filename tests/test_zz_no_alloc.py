"""decdec_decode_attention_static (the entry point that allocates nothing: its workspace is a device array inside
the library image) against decdec_decode_attention with a caller-owned workspace, through the C ABI: two calls in
a row, the second on a smaller input, then a short sequence (one workgroup per head) and the size limit.

The two entry points run the same kernels; the partial results of a head are merged in a fixed order, so the outputs
are expected to be equal bit for bit, and they are checked to the floating-point bar of the other GPU tests: max
relative error 1e-2 (fp16) against the existing entry point's output."""
import ctypes

import numpy as np
import pytest
import torch

from decdec_amd import _lib, decode_ops as D
from tests.helpers import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _case(H, Hkv, hd, S, pos, seed, dtype=torch.float16):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = torch.randn(H * hd, device="cuda", generator=g).to(dtype)
    kc = torch.randn(1, Hkv, S, hd, device="cuda", generator=g).to(dtype)
    vc = torch.randn(1, Hkv, S, hd, device="cuda", generator=g).to(dtype)
    return q, kc, vc, torch.tensor([pos], device="cuda", dtype=torch.int64)


def _both(H, Hkv, hd, S, pos, seed):
    q, kc, vc, p = _case(H, Hkv, hd, S, pos, seed)
    ref = torch.zeros(H * hd, device="cuda", dtype=torch.float16)
    got = torch.full((H * hd,), 7.0, device="cuda", dtype=torch.float16)
    ws = D.attention_workspace(H, hd)
    D.decode_attention(q, kc, vc, p, ref, H, Hkv, ws)
    D.decode_attention_static(q, kc, vc, p, got, H, Hkv)
    torch.cuda.synchronize()
    # plain fp64 softmax attention as a sanity anchor for both
    G = H // Hkv
    K = kc[0].double()[:, :pos + 1]; V = vc[0].double()[:, :pos + 1]
    qh = q.double().view(H, hd)
    sc = torch.einsum("hd,hsd->hs", qh, K.repeat_interleave(G, 0)) / np.sqrt(hd)
    want = torch.einsum("hs,hsd->hd", torch.softmax(sc, -1), V.repeat_interleave(G, 0)).reshape(-1).cpu().numpy()
    return got.float().cpu().numpy(), ref.float().cpu().numpy(), want


def test_static_workspace_entry_point_matches_the_workspace_one():
    # first call: Llama-3-8B heads at a long sequence (positions of a head shared by 8 workgroups)
    got, ref, want = _both(32, 8, 128, 2048, 1500, seed=1)
    assert rel_err(got, ref.astype(np.float64))[0] <= TOL
    assert rel_err(ref, want)[0] <= TOL and rel_err(got, want)[0] <= TOL
    first_equal = np.array_equal(got, ref)
    # second call, smaller input: fewer and narrower heads, shorter cache
    got, ref, want = _both(8, 2, 64, 1024, 700, seed=2)
    assert rel_err(got, ref.astype(np.float64))[0] <= TOL
    assert rel_err(got, want)[0] <= TOL
    assert first_equal and np.array_equal(got, ref), "same kernels, fixed merge order: equal bit for bit"
    # a larger one again after the small one, and a short sequence (no sharing, no workspace traffic)
    got, ref, want = _both(40, 10, 128, 2048, 2047, seed=3)
    assert rel_err(got, ref.astype(np.float64))[0] <= TOL and rel_err(got, want)[0] <= TOL
    got, ref, want = _both(32, 8, 128, 2048, 100, seed=4)
    assert rel_err(got, ref.astype(np.float64))[0] <= TOL and rel_err(got, want)[0] <= TOL


def test_static_workspace_entry_point_refuses_sizes_beyond_its_array():
    q, kc, vc, p = _case(8, 8, 64, 512, 10, seed=5)
    out = torch.zeros(8 * 64, device="cuda", dtype=torch.float16)
    lib = _lib.load()
    rc = lib.decdec_decode_attention_static(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), p.data_ptr(), out.data_ptr(),
                                            1, 256, 8, 64, 512, None)
    assert rc != 0 and "exceeds the limit of 128 heads" in _lib.last_error()
