"""Stream capture and graph replay (`HIPBackend.capture`): a replay must give exactly what the
same ops give when issued one by one, on every replay, with other work and synchronisations
in between, and with new contents in the input buffers. The allocator must keep a
recording's buffers away from everybody else while the graph exists."""
import numpy as np
import pytest

from honeycrisp_amd.descriptors import BackendError, DType
from honeycrisp_amd.nn import Transformer
from honeycrisp_amd.tensor import Tensor

pytestmark = pytest.mark.gpu


def chain(a, b, c):
    h = Tensor.matmul(a, False, b, False, False) + c
    return (h.gelu() * 0.5).sum(axis=1)


def test_replays_match_eager_with_new_inputs(hip_backend):
    rng = np.random.default_rng(0)
    with hip_backend.use():
        a = Tensor(data=rng.standard_normal((96, 64)).astype(np.float32))
        b = Tensor(data=rng.standard_normal((64, 128)).astype(np.float32))
        c = Tensor(data=rng.standard_normal((128,)).astype(np.float32))
        chain(a, b, c).wait()                       # warm the allocator and the kernel cache
        with hip_backend.capture() as cap:
            out = chain(a, b, c)
        for replay in range(4):
            fresh = rng.standard_normal((96, 64)).astype(np.float32)
            a.data.mutateOnCPU(lambda host: host.view(np.float32).__setitem__(slice(None), fresh.ravel()))
            cap.graph.launch()
            got = out.numpy().copy()
            # the program's own eager work between replays: same inputs, fresh buffers
            want = chain(a, b, c).numpy()
            assert np.array_equal(got, want), "replay %d differs from the eager result" % replay
            noise = [Tensor(data=rng.standard_normal((96, 128)).astype(np.float32)) for _ in range(3)]
            assert np.isfinite(sum(t.sum().numpy() for t in noise))
            hip_backend.sync()
        cap.graph.destroy()


def test_buffers_of_a_recording_are_not_handed_out(hip_backend):
    rng = np.random.default_rng(1)
    with hip_backend.use():
        a = Tensor(data=rng.standard_normal((64, 64)).astype(np.float32))
        with hip_backend.capture() as cap:
            out = ((a + 1.0) * 2.0) - 3.0           # two intermediates die inside the capture
        cap.graph.launch()
        want = out.numpy().copy()
        # same-size eager allocations must not land on the recording's intermediates
        held = [Tensor(data=np.full((64, 64), 7.0, np.float32)) for _ in range(8)]
        cap.graph.launch()
        assert np.array_equal(out.numpy(), want)
        assert all(np.all(t.numpy() == 7.0) for t in held)
        cap.graph.destroy()


def test_host_transfers_are_refused_while_capturing(hip_backend):
    with hip_backend.use():
        a = Tensor(data=np.ones((8, 8), np.float32))
        with pytest.raises(BackendError):
            with hip_backend.capture():
                Tensor(data=np.ones((8, 8), np.float32))    # an upload
        # the context is usable again and nothing was recorded
        assert np.all((a + 1.0).numpy() == 2.0)


@pytest.mark.parametrize("dtype", [DType.float32, DType.float16], ids=["f32", "f16"])
def test_transformer_forward_replay(hip_backend, dtype):
    cfg = dict(layers=2, d_model=64, heads=4, mlp=128, vocab=97, seq=16, seed=3)
    rng = np.random.default_rng(2)
    with hip_backend.use():
        model = Transformer(dtype=dtype, **cfg)
        ids = Tensor(data=rng.integers(0, 97, size=(3, 16)))
        model(ids).wait()
        with hip_backend.capture() as cap:
            logits = model(ids)
        for replay in range(3):
            fresh = rng.integers(0, 97, size=(3, 16)).astype(np.int64)
            ids.data.mutateOnCPU(lambda host: host.view(np.int64).__setitem__(slice(None), fresh.ravel()))
            cap.graph.launch()
            got = logits.numpy().copy()
            want = model(ids).numpy()
            assert np.array_equal(got, want), "replay %d" % replay
        cap.graph.destroy()


def test_a_graph_destroyed_during_another_recording(hip_backend):
    """hc_graph_destroy waits for the stream, which a capture in progress does not survive: a graph
    that its owner lets go of in the middle of a recording is destroyed when the recording ends."""
    rng = np.random.default_rng(21)
    with hip_backend.use():
        x = Tensor(data=rng.standard_normal((64, 64)).astype(np.float32))
        with hip_backend.capture() as first:
            y = x * 2.0
        first.graph.launch()
        assert np.array_equal(y.numpy(), x.numpy() * 2.0)
        with hip_backend.capture() as second:
            z = x + 1.0
            first.graph.destroy()          # in the middle of the second recording
            w = z * 3.0
        second.graph.launch()
        assert np.array_equal(w.numpy(), (x.numpy() + 1.0) * 3.0)
        second.graph.destroy()
