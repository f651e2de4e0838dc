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
    dense = {n: getattr(layer, n).dense_weight() for n in ("qkv", "o", "ffn1", "ffn2")}
    assert torch.equal(dense["qkv"], torch.cat([layer.q.dense_weight(), layer.k.dense_weight(), layer.v.dense_weight()]))
    with torch.no_grad():
        got = layer(x, batch, seq)
        gelu = torch.nn.functional.gelu
        want = layer(x, batch, seq, linear=lambda name, lin, t: (
            gelu(dense["ffn1"].float() @ t.float()) if name == "ffn1_gelu" else dense[name].float() @ t.float()).half())
    assert got.shape == (hidden, batch * seq)
    assert max_rel_err(got.float().cpu().numpy(), want.float().cpu().numpy()) <= 1e-2


@pytest.mark.parametrize("H,T", [(768, 4096), (256, 128), (100, 36), (1024, 68), (1, 4), (3072, 520), (4096, 16)])
@pytest.mark.parametrize("residual", [True, False])
def test_feature_major_add_layernorm_matches_torch(built_library, H, T, residual):
    """The fused kernel against torch's LayerNorm on the transposed sum: same fp16 sum, statistics in fp32."""
    from sspmm_amd.layers import add_layernorm
    g = torch.Generator("cuda").manual_seed(H + T)
    x = (torch.randn(H, T, device="cuda", generator=g) * 2 + 0.5).half()
    a = torch.randn(H, T, device="cuda", generator=g).half() if residual else None
    ln = torch.nn.LayerNorm(H).cuda().half()
    with torch.no_grad():
        ln.weight.copy_(torch.randn(H, device="cuda", generator=g))
        ln.bias.copy_(torch.randn(H, device="cuda", generator=g))
        got = add_layernorm(x, a, ln)
        s = x if a is None else x + a
        want = torch.nn.functional.layer_norm(s.t().float(), (H,), ln.weight.float(), ln.bias.float(), ln.eps).t()
    assert got.shape == (H, T) and got.dtype == torch.float16
    assert (got.float() - want).abs().max().item() <= 4e-3 * max(1.0, want.abs().max().item())
    # shapes outside the kernel's limits take torch and agree too
    if T % 4 == 0 and H > 1:
        odd = add_layernorm(x[:, :T - 1].contiguous(), None if a is None else a[:, :T - 1].contiguous(), ln)
        assert (odd.float() - want[:, :T - 1]).abs().max().item() <= 4e-3 * max(1.0, want.abs().max().item())


def _attention_reference(q, k, v, batch, heads, seq, scale):
    """fp32 attention of feature-major [heads * d, batch * seq] operands, written out with plain matmuls."""
    d = q.shape[0] // heads
    f = lambda t: t.float().view(heads, d, batch, seq).permute(2, 0, 3, 1)  # noqa: E731  [batch, heads, seq, d]
    p = torch.softmax(f(q) @ f(k).transpose(-1, -2) * scale, dim=-1)
    return (p @ f(v)).permute(1, 3, 0, 2).reshape(heads * d, batch * seq)


@pytest.mark.parametrize("batch,heads,seq", [(1, 1, 64), (2, 3, 128), (3, 2, 192), (8, 12, 512), (1, 2, 320), (1, 1, 1024)])
def test_feature_major_attention_matches_fp32_attention(built_library, batch, heads, seq):
    """sspmm_attention_fm_f16 through the C ABI, operands as three row ranges of one fused projection."""
    from sspmm_amd import _lib
    from sspmm_amd.layers import attention_fm
    hidden, T = heads * 64, batch * seq
    g = torch.Generator("cuda").manual_seed(seq + heads)
    qkv = torch.randn(3 * hidden, T, device="cuda", generator=g).half()
    qkv[:hidden] *= 2.0  # scores spread over several units, so the softmax is far from uniform
    scale = 0.125
    got = attention_fm(qkv, hidden, heads, batch, seq)
    assert got is not None and got.shape == (hidden, T) and got.dtype == torch.float16
    want = _attention_reference(qkv[:hidden], qkv[hidden:2 * hidden], qkv[2 * hidden:], batch, heads, seq, scale)
    assert (got.float() - want).abs().max().item() <= 2e-3 * max(1.0, want.abs().max().item())
    # separate operands with their own leading dimension, output into a wider array: the columns beyond stay untouched
    ld, ld_out = T + 24, T + 8
    q, k, v = (torch.randn(hidden, ld, device="cuda", generator=g).half() for _ in range(3))
    out = torch.full((hidden, ld_out), 7.0, dtype=torch.float16, device="cuda")
    rc = _lib.lib().sspmm_attention_fm_f16(batch, heads, seq, 64, q.data_ptr(), k.data_ptr(), v.data_ptr(), ld, out.data_ptr(),
                                           ld_out, scale, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    want = _attention_reference(q[:, :T], k[:, :T], v[:, :T], batch, heads, seq, scale)
    assert (out[:, :T].float() - want).abs().max().item() <= 2e-3 * max(1.0, want.abs().max().item())
    assert torch.all(out[:, T:] == 7.0)


def test_feature_major_attention_with_maxima_that_keep_growing(built_library):
    """Keys whose norm grows along the sequence: the running maximum of a query's scores rises by many units from one
    block of keys to the next, so the kernel moves the reference point of its exponentials again and again (it
    skips that step while the maximum grows by little)."""
    from sspmm_amd.layers import attention_fm
    batch, heads, seq = 2, 2, 512
    hidden, T = heads * 64, batch * seq
    g = torch.Generator("cuda").manual_seed(11)
    qkv = torch.randn(3 * hidden, T, device="cuda", generator=g)
    growth = 1.0 + 7.0 * (torch.arange(T, device="cuda") % seq).float() / seq
    qkv[hidden:2 * hidden] *= growth
    qkv[:hidden] = qkv[:hidden].abs() * 2.0   # same-sign queries and keys of growing size: scores rise with the position
    qkv[hidden:2 * hidden] = qkv[hidden:2 * hidden].abs()
    qkv = qkv.half()
    got = attention_fm(qkv, hidden, heads, batch, seq)
    want = _attention_reference(qkv[:hidden], qkv[hidden:2 * hidden], qkv[2 * hidden:], batch, heads, seq, 0.125)
    assert (got.float() - want).abs().max().item() <= 2e-3 * max(1.0, want.abs().max().item())


def test_feature_major_attention_rejects_what_it_does_not_cover(built_library):
    from sspmm_amd import _lib
    L = _lib.lib()
    t = torch.zeros(64, 1024, dtype=torch.float16, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    args = lambda **kw: [kw.get("batch", 1), kw.get("heads", 1), kw.get("seq", 64), kw.get("d", 64), t.data_ptr() + kw.get("off", 0),  # noqa: E731
                         t.data_ptr(), t.data_ptr(), kw.get("ld", 1024), t.data_ptr(), 1024, 0.125, s]
    assert L.sspmm_attention_fm_f16(*args()) == 0
    for bad in (dict(d=32), dict(seq=96), dict(seq=16448, ld=16448), dict(ld=1020), dict(off=2), dict(seq=512, batch=4, ld=1024), dict(batch=-1)):
        assert L.sspmm_attention_fm_f16(*args(**bad)) == 1, bad
    assert L.sspmm_attention_fm_f16(*args(batch=0)) == 0
    torch.cuda.synchronize()


def test_encoder_layer_at_the_benchmark_shape_takes_the_attention_kernel(built_library):
    """hidden 768, 12 heads, 8 x 512 tokens: the layer with the feature-major attention kernel against the same layer
    with torch's attention between relayout copies."""
    hidden, heads, ffn, V, batch, seq = 768, 12, 3072, 16, 8, 512
    mk = lambda o, i, s: _vector_sparse_linear(o, i, V, 0.9, seed=s)
    layer = SparseEncoderLayer(hidden, heads, ffn, mk(hidden, hidden, 1), mk(hidden, hidden, 2), mk(hidden, hidden, 3),
                               mk(hidden, hidden, 4), mk(ffn, hidden, 5), mk(hidden, ffn, 6)).cuda().half()
    x = torch.randn(hidden, batch * seq, device="cuda", generator=torch.Generator("cuda").manual_seed(5)).half()
    import sspmm_amd.layers as layers_mod
    with torch.no_grad():
        got = layer(x, batch, seq)
        kernel = layers_mod.attention_fm
        layers_mod.attention_fm = lambda *a, **kw: None
        try:
            want = layer(x, batch, seq)
        finally:
            layers_mod.attention_fm = kernel
    assert max_rel_err(got.float().cpu().numpy(), want.float().cpu().numpy()) <= 1e-2


def test_encoder_layer_at_the_benchmark_shape_matches_dense_products(built_library):
    """hidden 768, 12 heads, FFN 3072, 8 x 512 tokens, six weights V = 16 at 90 %: the layer against the same layer whose
    four products are dense fp32 matmuls on the densified weights (an independent check of the sparse products at the
    full shape: nothing of this library computes the comparison's products)."""
    hidden, heads, ffn, V, batch, seq = 768, 12, 3072, 16, 8, 512
    mk = lambda o, i, s: _vector_sparse_linear(o, i, V, 0.9, seed=s)
    layer = SparseEncoderLayer(hidden, heads, ffn, mk(hidden, hidden, 1), mk(hidden, hidden, 2), mk(hidden, hidden, 3),
                               mk(hidden, hidden, 4), mk(ffn, hidden, 5), mk(hidden, ffn, 6)).cuda().half()
    x = torch.randn(hidden, batch * seq, device="cuda", generator=torch.Generator("cuda").manual_seed(6)).half()
    dense = {n: getattr(layer, n).dense_weight().float() for n in ("qkv", "o", "ffn1", "ffn2")}
    assert torch.equal(dense["qkv"], torch.cat([layer.q.dense_weight(), layer.k.dense_weight(), layer.v.dense_weight()]).float())
    # the weights are held once: q, k and v are views of the fused layer's arrays, and state_dict names them once
    assert layer.q.values.data_ptr() == layer.qkv.values.data_ptr()
    assert not any(key.startswith(("q.", "k.", "v.", "ffn1_gelu.")) for key in layer.state_dict())
    gelu = torch.nn.functional.gelu
    with torch.no_grad():
        got = layer(x, batch, seq)
        want = layer(x, batch, seq, linear=lambda name, lin, t: (
            gelu(dense["ffn1"] @ t.float()) if name == "ffn1_gelu" else dense[name] @ t.float()).half())
    assert got.shape == (hidden, batch * seq)
    assert max_rel_err(got.float().cpu().numpy(), want.float().cpu().numpy()) <= 1e-2


def test_sparse_linear_drops_its_plan_when_the_buffers_move(built_library):
    lin = _vector_sparse_linear(256, 192, 16, 0.8, seed=72)
    lin.make_plan(64)
    assert lin.plan is not None
    lin = lin.half()   # any conversion or move goes through _apply
    assert lin.plan is None
    x = torch.randn(192, 64, device="cuda", generator=torch.Generator("cuda").manual_seed(7)).half()
    want = lin.dense_weight().float() @ x.float()
    assert max_rel_err(lin(x).float().cpu().numpy(), want.cpu().numpy()) <= 2e-3


@pytest.mark.parametrize("V,out_f,in_f,N", [(16, 3072, 768, 4096), (8, 64, 100, 72), (16, 128, 5000, 64), (8, 256, 96, 33)])
@pytest.mark.parametrize("activation", [None, "gelu"])
@pytest.mark.parametrize("with_bias", [False, True])
def test_linear_epilogue_matches_separate_bias_and_gelu(built_library, V, out_f, in_f, N, activation, with_bias):
    """sspmm_linear_f16 against the fp32 product with bias and erf-GELU applied in fp32: the gather kernel (wide N),
    the staged gather kernel (few waves, N <= 64, K above the split-row kernel's threshold) and the scalar kernel
    (N not a multiple of 8)."""
    from sspmm_amd.spmm import linear
    vs = synth.vector_sparse(out_f, in_f, V, 0.9, seed=out_f + N, std=0.05)
    g = torch.Generator("cuda").manual_seed(N)
    x = torch.randn(in_f, N, device="cuda", generator=g).half()
    bias = torch.randn(out_f, device="cuda", generator=g).half() if with_bias else None
    ro, ci, va = dev(vs.row_offsets), dev(vs.col_idx), dev(vs.values)
    got = linear(ro, ci, va, x, V, bias=bias, activation=activation)
    want = sspmm_amd.spmm(None, ro, ci, va, x, V, out_dtype=torch.float32)
    if bias is not None:
        want = want + bias.float()[:, None]
    if activation == "gelu":
        want = torch.nn.functional.gelu(want)
    assert got.dtype == torch.float16 and got.shape == (out_f, N)
    assert max_rel_err(got.float().cpu().numpy(), want.cpu().numpy()) <= 2e-3
    if bias is None and activation is None:
        assert torch.equal(got, sspmm_amd.spmm(None, ro, ci, va, x, V))


def test_sparse_linear_fuses_bias_and_activation(built_library):
    lin = _vector_sparse_linear(256, 192, 16, 0.8, seed=71, activation="gelu")
    lin.bias = torch.randn(256, device="cuda", generator=torch.Generator("cuda").manual_seed(4)).half()
    x = torch.randn(192, 200, device="cuda", generator=torch.Generator("cuda").manual_seed(5)).half()
    want = torch.nn.functional.gelu(lin.dense_weight().float() @ x.float() + lin.bias.float()[:, None])
    assert max_rel_err(lin(x).float().cpu().numpy(), want.cpu().numpy()) <= 2e-3
    from sspmm_amd import _lib
    L = _lib.lib()
    assert L.sspmm_linear_f16(1, 16, 8, 8, 0, 0, 0, 0, 0, 2, 0, 0) == 1  # unknown activation
