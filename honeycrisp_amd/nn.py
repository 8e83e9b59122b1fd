"""`Linear`, `LayerNorm` and a decoder-only transformer built only from the Tensor ops of the
front-end mirror, i.e. from the backend calls a Honeycrisp model would emit.

`Linear` / `LayerNorm` restate Trainable.swift:508-547 and :787-829 (forward only). The
reference ships no transformer class; `Transformer` is the workload of the benchmark's
config 5 (6 layers, d_model 512, 8 heads, MLP 2048, vocab 8192, batch 8 x seq 256, causal
mask), written the way a Honeycrisp user would write it. Parameters are created on the host
from a numpy generator and uploaded, so that two backends can be given identical weights.
"""
import math
from typing import List, Optional

import numpy as np

from .descriptors import DType
from .tensor import NewAxis, Tensor


class Linear:
    """y = x @ W + b (Trainable.swift:508-547). Weight init (rand - 0.5) * (sqrt(3)/0.5/sqrt(in)),
    bias zeros in float32; `castParams` casts both at call time."""

    def __init__(self, inCount: int, outCount: int, rng: np.random.Generator, dtype=DType.float32,
                 castParams: Optional[DType] = None, bias: bool = True):
        self.castParams = castParams
        scale = np.float32(math.sqrt(3.0) / 0.5 / math.sqrt(float(inCount)))
        w = (rng.random((inCount, outCount), dtype=np.float32) - np.float32(0.5)) * scale
        self.weight = Tensor(data=w, dtype=dtype)
        self.bias = Tensor.zeros([outCount]) if bias else None

    def __call__(self, x: Tensor) -> Tensor:
        if len(x.shape) > 2:
            squashed = x.reshape([int(np.prod(x.shape[:-1])), x.shape[-1]])
            out = self(squashed)
            return out.reshape(x.shape[:-1] + [out.shape[-1]])
        h = Tensor.matmul(x, False, self.weight.cast(self.castParams or self.weight.dtype), False, False)
        if self.bias is not None:
            h = h + self.bias.cast(self.castParams or self.bias.dtype)
        return h


class LayerNorm:
    """Trainable.swift:787-829: cast -> normalize over the trailing axes -> (gain + 1) * x + bias
    -> cast back. gain and bias start at zero."""

    def __init__(self, shape: List[int], dtype=DType.float32, eps: float = 1e-5, affine: bool = True,
                 rng: Optional[np.random.Generator] = None):
        self.dtype, self.shape, self.eps = dtype, list(shape), np.float32(eps)
        if affine:
            # the reference initialises both to zero; a generator gives non-trivial values so
            # that parity tests exercise the affine part
            g = np.zeros(shape, np.float32) if rng is None else (rng.standard_normal(shape) * 0.1).astype(np.float32)
            b = np.zeros(shape, np.float32) if rng is None else (rng.standard_normal(shape) * 0.1).astype(np.float32)
            self.gain, self.bias = Tensor(data=g, dtype=dtype), Tensor(data=b, dtype=dtype)
        else:
            self.gain = self.bias = None

    def __call__(self, x: Tensor) -> Tensor:
        assert x.shape[len(x.shape) - len(self.shape):] == self.shape
        inType = x.dtype
        x = x.cast(self.dtype)
        batch = int(np.prod(x.shape[:len(x.shape) - len(self.shape)]))
        inner = int(np.prod(self.shape))
        normalized = x.reshape([batch, inner]).normalize(axis=1, eps=self.eps).reshape(x.shape)
        if self.gain is not None:
            return normalized.mul(self.gain + 1, thenAdd=self.bias).cast(inType)
        return normalized.cast(inType)


class Block:
    def __init__(self, d_model, heads, mlp, rng, dtype):
        cp = dtype if dtype != DType.float32 else None
        mk = lambda i, o: Linear(i, o, rng, dtype=dtype, castParams=cp)
        self.heads = heads
        self.ln1 = LayerNorm([d_model], rng=rng)
        self.q, self.k, self.v, self.o = mk(d_model, d_model), mk(d_model, d_model), mk(d_model, d_model), mk(d_model, d_model)
        self.ln2 = LayerNorm([d_model], rng=rng)
        self.fc1, self.fc2 = mk(d_model, mlp), mk(mlp, d_model)

    def __call__(self, x: Tensor, mask: Tensor) -> Tensor:
        B, T, D = x.shape
        H = self.heads
        hd = D // H
        h = self.ln1(x)
        # [B,T,D] -> [B,T,H,hd] -> swap -> [B,H,T,hd]: a gather of hd-element rows (Index.swift:365-376)
        q = self.q(h).reshape([B, T, H, hd]).swap(1, 2)
        k = self.k(h).reshape([B, T, H, hd]).swap(1, 2)
        v = self.v(h).reshape([B, T, H, hd]).swap(1, 2)
        scores = Tensor.batchedMatmul(q, False, k, True, False) * (1.0 / math.sqrt(hd))
        probs = (scores + mask).softmax()
        ctx = Tensor.batchedMatmul(probs, False, v, False, False).swap(1, 2).reshape([B, T, D])
        x = x + self.o(ctx)
        return x + self.fc2(self.fc1(self.ln2(x)).gelu())


class Transformer:
    def __init__(self, layers=6, d_model=512, heads=8, mlp=2048, vocab=8192, seq=256, seed=12,
                 dtype=DType.float32):
        rng = np.random.default_rng(seed)
        self.dtype, self.seq, self.d_model = dtype, seq, d_model
        self._masks = {}
        self.table = Tensor(data=(rng.standard_normal((vocab, d_model)) * 0.02).astype(np.float32), dtype=dtype)
        self.pos = Tensor(data=(rng.standard_normal((seq, d_model)) * 0.02).astype(np.float32), dtype=dtype)
        self.blocks = [Block(d_model, heads, mlp, rng, dtype) for _ in range(layers)]
        self.ln_f = LayerNorm([d_model], rng=rng)
        cp = dtype if dtype != DType.float32 else None
        self.unembed = Linear(d_model, vocab, rng, dtype=dtype, castParams=cp)

    def causal_mask(self, T: int) -> Tensor:
        # depends on T only: built once per length (also keeps host uploads out of the forward pass)
        if T not in self._masks:
            pos = Tensor(data=range(T))
            # finite in fp16; (pos[:, None] >= pos) is true on and below the diagonal
            self._masks[T] = (pos[..., NewAxis()] >= pos).when(0, -1e4, dtype=self.dtype)
        return self._masks[T]

    def __call__(self, ids: Tensor) -> Tensor:
        B, T = ids.shape
        x = self.table.gather(0, ids.reshape([B * T])).reshape([B, T, self.d_model])
        x = x + self.pos[0:T] if T != self.seq else x + self.pos
        mask = self.causal_mask(T)
        for block in self.blocks:
            x = block(x, mask)
        return self.unembed(self.ln_f(x))
