"""Random programs over the operations the rewrite of a recording knows (products, row and
matrix additions, GELU, LayerNorm, the scaled and masked softmax, row maxima), with random lifetimes of
the intermediates: results with several readers, results the program keeps, results released
at once. Whatever the rewrite merges or leaves alone, and wherever a batch happens to end, a
program's results must have the bits of the same calls issued one by one; here the same seeded
program runs call by call, under batching with random limits, and as a recording."""
import numpy as np
import pytest

from honeycrisp_amd.descriptors import DType
from honeycrisp_amd.nn import LayerNorm
from honeycrisp_amd.tensor import Tensor

pytestmark = pytest.mark.gpu


class Program:
    """`steps` operations on [m, d] tensors drawn from a seeded generator. A pool holds the tensors
    the program can still name; after every step a random part of it is dropped, which is what
    releases buffers (the front-end's tensors free their data when nobody holds them)."""

    def __init__(self, seed, dtype, m=192, d=128, steps=40):
        self.seed, self.dtype, self.m, self.d, self.steps = seed, dtype, m, d, steps
        rng = np.random.default_rng(seed)
        mk = lambda shape, scale=1.0: Tensor(data=(rng.standard_normal(shape) * scale).astype(np.float32), dtype=dtype)
        self.x0 = mk((m, d))
        self.weights = [mk((d, d), 1.0 / np.sqrt(d)) for _ in range(3)]
        self.rows = [mk((d,)) for _ in range(3)]
        self.norms = [LayerNorm([d], rng=rng) for _ in range(2)]
        mask = np.where(rng.random((m, d)) < 0.2, -1.0e4, 0.0).astype(np.float32)   # (finite: nothing here should make a NaN)
        self.mask = Tensor(data=mask, dtype=dtype)

    def run(self):
        rng = np.random.default_rng(self.seed + 1000)
        pool, kept = [self.x0], []
        for _ in range(self.steps):
            a = pool[rng.integers(len(pool))]
            op = rng.choice(["linear", "row", "matrix", "gelu", "norm", "softmax", "linear", "row", "center"])
            if op == "linear":
                t = Tensor.matmul(a, False, self.weights[rng.integers(3)], False, False)
            elif op == "row":
                t = a + self.rows[rng.integers(3)] if rng.random() < 0.5 else self.rows[rng.integers(3)] + a
            elif op == "matrix":
                t = a + pool[rng.integers(len(pool))]
            elif op == "gelu":
                t = a.gelu()
            elif op == "norm":
                t = self.norms[rng.integers(2)](a)
            elif op == "center":
                t = a - (a.max(axis=1, keepdims=True) if rng.random() < 0.5 else a.min(axis=1, keepdims=True))
            else:
                s = a * 0.125 if rng.random() < 0.7 else a
                if rng.random() < 0.5:
                    s = s + self.mask
                t = s.softmax()
            del a
            pool.append(t)
            if rng.random() < 0.15:
                kept.append(t)
            del t
            # drop a random part of the pool (never the newest, which the next step most likely reads)
            while len(pool) > 1 and rng.random() < 0.6:
                pool.pop(rng.integers(len(pool) - 1))
            if len(pool) > 4:
                pool.pop(0)
        return [pool[-1]] + kept


def same_bits(got, want, what):
    assert len(got) == len(want)
    for i, (g, w) in enumerate(zip(got, want)):
        assert np.array_equal(g.view(np.uint8), w.view(np.uint8)), "%s: result %d differs in %d of %d elements" % (
            what, i, int((g != w).sum()), w.size)


@pytest.mark.parametrize("dtype", [DType.float16, DType.float32], ids=["f16", "f32"])
@pytest.mark.parametrize("seed", range(12))
def test_random_program_batched_and_recorded(hip_backend, dtype, seed):
    with hip_backend.use():
        program = Program(seed, dtype)
        want = [t.numpy().copy() for t in program.run()]
        rng = np.random.default_rng(seed)
        listed, enqueued = hip_backend.batchingStats()
        for limit, idle_after in ((4096, 0), (int(rng.integers(2, 40)), 0), (int(rng.integers(8, 64)), int(rng.integers(1, 8)))):
            with hip_backend.batching(limit, idle_after):
                got = [t.numpy().copy() for t in program.run()]
            same_bits(got, want, "batching(%d, %d)" % (limit, idle_after))
        listed, enqueued = (b - a for a, b in zip((listed, enqueued), hip_backend.batchingStats()))
        with hip_backend.capture() as cap:
            outs = program.run()
        nodes = cap.graph.node_count()
        for replay in range(2):
            cap.graph.launch()
            same_bits([t.numpy() for t in outs], want, "replay %d" % replay)
        cap.graph.destroy()
        print("seed %d %s: %d launches listed over three batched runs, %d enqueued; recording: %d launches" % (
            seed, dtype.name, listed, enqueued, nodes), flush=True)
