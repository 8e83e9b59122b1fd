"""Config 5: a decoder-only transformer forward pass built only from backend ops.
CPU part: the model under the oracle has the properties the construction implies (causality,
softmax rows summing to one). GPU part: logits under HIPBackend match the oracle's."""
import numpy as np
import pytest

from honeycrisp_amd.descriptors import DType
from honeycrisp_amd.nn import LayerNorm, Linear, Transformer
from honeycrisp_amd.tensor import Tensor
from backend_cases import assert_close_arrays


def logits(backend, dtype, ids, **cfg):
    with backend.use():
        model = Transformer(dtype=dtype, **cfg)
        return model(Tensor(data=ids)).numpy().astype(np.float32)


SMALL = dict(layers=2, d_model=64, heads=4, mlp=128, vocab=97, seq=16, seed=3)


def numpy_forward(model, ids):
    """The same decoder written directly in numpy float64 from the model's weights: no Tensor
    front-end, no backend calls, no descriptors. A lowering mistake in the front-end mirror (a
    wrong stride map, permutation or reduce axis) would hit both backends alike and cancel in a
    backend-against-backend comparison; it cannot cancel here."""
    f = lambda t: t.numpy().astype(np.float64)

    def layer_norm(x, ln):
        mean = x.mean(-1, keepdims=True)
        var = ((x - mean) ** 2).mean(-1, keepdims=True)
        return (x - mean) / np.sqrt(var + float(ln.eps)) * (f(ln.gain) + 1.0) + f(ln.bias)

    def linear(x, lin):
        return x @ f(lin.weight) + f(lin.bias)

    B, T = ids.shape
    x = f(model.table)[ids] + f(model.pos)[:T]
    mask = np.where(np.arange(T)[:, None] >= np.arange(T)[None, :], 0.0, -1e4)
    for blk in model.blocks:
        H = blk.heads
        hd = x.shape[-1] // H
        h = layer_norm(x, blk.ln1)
        q, k, v = (linear(h, w).reshape(B, T, H, hd).transpose(0, 2, 1, 3) for w in (blk.q, blk.k, blk.v))
        scores = q @ k.transpose(0, 1, 3, 2) / np.sqrt(hd) + mask
        scores = scores - scores.max(-1, keepdims=True)
        probs = np.exp(scores)
        probs /= probs.sum(-1, keepdims=True)
        ctx = (probs @ v).transpose(0, 2, 1, 3).reshape(B, T, H * hd)
        x = x + linear(ctx, blk.o)
        u = linear(layer_norm(x, blk.ln2), blk.fc1)
        u = 0.5 * u * (1.0 + np.tanh(0.797884561 * (u + 0.044715 * u ** 3)))      # GELU, tanh form (Elemwise.swift:109-111)
        x = x + linear(u, blk.fc2)
    return linear(layer_norm(x, model.ln_f), model.unembed)


def test_small_transformer_matches_an_independent_numpy_model(oracle_backend):
    ids = np.random.default_rng(0).integers(0, 97, size=(3, 16))
    with oracle_backend.use():
        model = Transformer(dtype=DType.float32, **SMALL)
        got = model(Tensor(data=ids)).numpy()
        want = numpy_forward(model, ids)
    assert_close_arrays(got, want, 1e-4, 1e-4)


def test_small_transformer_is_causal_under_the_oracle(oracle_backend):
    rng = np.random.default_rng(0)
    ids = rng.integers(0, 97, size=(3, 16))
    base = logits(oracle_backend, DType.float32, ids, **SMALL)
    assert base.shape == (3, 16, 97) and np.isfinite(base).all()
    changed = ids.copy()
    changed[:, 10:] = (changed[:, 10:] + 1) % 97
    other = logits(oracle_backend, DType.float32, changed, **SMALL)
    assert np.array_equal(base[:, :10], other[:, :10])      # the mask hides later tokens exactly
    assert not np.allclose(base[:, 10:], other[:, 10:])


def test_linear_and_layernorm_follow_their_definitions(oracle_backend):
    rng = np.random.default_rng(1)
    with oracle_backend.use():
        lin = Linear(24, 40, np.random.default_rng(5))
        x = rng.standard_normal((3, 7, 24)).astype(np.float32)
        w = lin.weight.numpy()
        assert np.abs(w).max() <= np.sqrt(3.0) / np.sqrt(24.0) + 1e-6     # uniform in +-sqrt(3/in)
        assert_close_arrays(lin(Tensor(data=x)).numpy(), x @ w, 1e-5, 1e-5)
        ln = LayerNorm([24], rng=np.random.default_rng(6))
        g, b = ln.gain.numpy(), ln.bias.numpy()
        mean = x.mean(-1, keepdims=True)
        var = ((x - mean) ** 2).mean(-1, keepdims=True)
        want = (x - mean) / np.sqrt(var + 1e-5) * (g + 1) + b
        assert_close_arrays(ln(Tensor(data=x)).numpy(), want, 1e-5, 1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(DType.float32, 1e-4), (DType.float16, 1e-2)], ids=["f32", "f16"])
def test_small_transformer_parity(hip_backend, oracle_backend, dtype, tol):
    ids = np.random.default_rng(0).integers(0, 97, size=(3, 16))
    got = logits(hip_backend, dtype, ids, **SMALL)
    want = logits(oracle_backend, dtype, ids, **SMALL)
    assert_close_arrays(got, want, tol, tol)


@pytest.mark.gpu
def test_config5_transformer_matches_an_independent_numpy_model(hip_backend):
    """Config 5 in fp32 on the device against the float64 numpy model (same weights): independent of
    the front-end mirror and of the oracle."""
    ids = np.random.default_rng(11).integers(0, 8192, size=(8, 256))
    with hip_backend.use():
        model = Transformer(dtype=DType.float32)
        got = model(Tensor(data=ids)).numpy()
        want = numpy_forward(model, ids)
    assert_close_arrays(got, want, 1e-4, 1e-4)
    assert float(np.max(np.abs(got - want))) / float(np.max(np.abs(want))) <= 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(DType.float32, 1e-4), (DType.float16, 1e-2)], ids=["f32", "f16"])
def test_config5_transformer_parity(hip_backend, oracle_backend, dtype, tol):
    """6 layers, d_model 512, 8 heads, MLP 2048, vocab 8192, batch 8 x seq 256, seeded weights."""
    ids = np.random.default_rng(11).integers(0, 8192, size=(8, 256))
    print("config 5", dtype.name, "gpu", flush=True)
    got = logits(hip_backend, dtype, ids)
    print("config 5", dtype.name, "oracle", flush=True)
    want = logits(oracle_backend, dtype, ids)
    assert got.shape == (8, 256, 8192)
    assert_close_arrays(got, want, tol, tol)
    scale = float(np.max(np.abs(want)))
    assert float(np.max(np.abs(got - want))) / scale <= tol
