"""The model-side callers (sspmm_amd.layers) against dense torch arithmetic on the same weights."""
import numpy as np
import pytest
import torch

import sspmm_amd
from sspmm_amd import synth
from sspmm_amd.layers import SparseEncoderLayer, SparseLinear
from gpu_util import dev, max_rel_err

pytestmark = pytest.mark.gpu


def _vector_sparse_linear(out_f, in_f, V, sparsity, seed, **kw):
    vs = synth.vector_sparse(out_f, in_f, V, sparsity, seed=seed, std=0.05)
    return SparseLinear.from_cvse(in_f, V, dev(vs.row_offsets), dev(vs.col_idx), dev(vs.values), **kw)


@pytest.mark.parametrize("V", [8, 16])
def test_sparse_linear_from_cvse_matches_dense_matmul(built_library, V):
    lin = _vector_sparse_linear(256, 192, V, 0.8, seed=70, out_dtype=torch.float32)
    x = torch.randn(192, 136, device="cuda", generator=torch.Generator("cuda").manual_seed(1)).half()
    want = lin.dense_weight().float() @ x.float()
    got = lin(x)
    assert got.dtype == torch.float32 and got.shape == (256, 136)
    assert max_rel_err(got.cpu().numpy(), want.cpu().numpy()) <= 2e-5


def test_sparse_linear_from_unstructured_dense_weight(built_library):
    """A scalar-sparse weight goes through the SVC on the GPU; the layer still computes W @ x (+ bias)."""
    g = torch.Generator("cuda").manual_seed(2)
    W = torch.randn(128, 300, device="cuda", generator=g).half()
    W[torch.rand(128, 300, device="cuda", generator=g) < 0.9] = 0
    bias = torch.randn(128, device="cuda", generator=g).half()
    for order in ("sorted", "cpython"):
        lin = SparseLinear.from_dense(W, 8, bias=bias, order=order, out_dtype=torch.float32)
        assert torch.equal(lin.dense_weight(), W)
        x = torch.randn(300, 64, device="cuda", generator=g).half()
        want = W.float() @ x.float() + bias.float()[:, None]
        assert max_rel_err(lin(x).cpu().numpy(), want.cpu().numpy()) <= 2e-5
    with pytest.raises(ValueError):
        lin(torch.zeros(64, 300, device="cuda", dtype=torch.float16))


def test_encoder_layer_matches_the_same_layer_with_dense_products(built_library):
    hidden, heads, ffn, V, batch, seq = 256, 4, 1024, 16, 2, 64
    mk = lambda o, i, s: _vector_sparse_linear(o, i, V, 0.9, seed=s)
    layer = SparseEncoderLayer(hidden, heads, ffn, mk(hidden, hidden, 1), mk(hidden, hidden, 2), mk(hidden, hidden, 3),
                               mk(hidden, hidden, 4), mk(ffn, hidden, 5), mk(hidden, ffn, 6)).cuda().half()
    x = torch.randn(hidden, batch * seq, device="cuda", generator=torch.Generator("cuda").manual_seed(3)).half()
    dense = {n: getattr(layer, n).dense_weight() for n in ("q", "k", "v", "o", "ffn1", "ffn2")}
    with torch.no_grad():
        got = layer(x, batch, seq)
        want = layer(x, batch, seq, linear=lambda name, lin, t: (dense[name].float() @ t.float()).half())
    assert got.shape == (hidden, batch * seq)
    assert max_rel_err(got.float().cpu().numpy(), want.float().cpu().numpy()) <= 1e-2
