"""cg_argmax_into - the entry point that allocates nothing - against cg_argmax, through the C ABI.

Bit-exact (argmax is index work).  The cases are chosen so that the rows are split over workgroups
(few, long rows: the fixed scratch array is in use), two calls in a row, the second with a smaller
input, then shapes that take the unsplit kernels, and the errors.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(be, x_np):
    x = be.tensor(x_np)                               # uploaded: in memory
    want = be.to_vec(be.argmax(x))
    # a one-element upload is kept as a host-side constant until somebody needs memory for it
    out = be.realize(be.tensor(np.full(x_np.shape[:-1] + (1,), 0xFFFFFFFF, dtype=np.uint32)))
    before = be.stats()
    be.argmax_into(x, out)
    after = be.stats()
    got = be.to_vec(out)
    assert after["device_bytes"] == before["device_bytes"], "cg_argmax_into took device memory"
    assert after["pool_bytes"] == before["pool_bytes"], "cg_argmax_into took memory from the pool"
    assert after["launches"] > before["launches"]
    return want, got


@pytest.mark.parametrize("mode", ["f32", "bf16"])
def test_two_calls_in_a_row_second_smaller(hip, hip_bf16, oracle, mode):
    be = hip if mode == "f32" else hip_bf16
    rng = np.random.default_rng(5)
    first = rng.standard_normal((1, 1, 128256)).astype(np.float32)      # a vocabulary row: 62 chunks
    second = rng.standard_normal((1, 1, 40000)).astype(np.float32)      # fewer chunks, same scratch
    if mode == "bf16":  # values a bf16 store keeps exactly, so that the oracle sees the same numbers
        first = (first.view(np.uint32) & 0xFFFF0000).view(np.float32)
        second = (second.view(np.uint32) & 0xFFFF0000).view(np.float32)
    for x_np in (first, second):
        want, got = _both(be, x_np)
        assert np.array_equal(want, got)
        assert np.array_equal(got, oracle.to_vec(oracle.argmax(oracle.tensor(x_np))))


@pytest.mark.parametrize("shape", [(3, 65536), (2, 2, 20000), (7, 33), (1, 5), (300, 2048), (4, 1, 16385)])
def test_shapes_and_ties(hip, oracle, shape):
    rng = np.random.default_rng(shape[-1])
    x_np = rng.integers(-3, 4, size=shape).astype(np.float32)           # many ties: the last maximum wins
    want, got = _both(hip, x_np)
    assert np.array_equal(want, got)
    assert np.array_equal(got, oracle.to_vec(oracle.argmax(oracle.tensor(x_np))))


def test_u32_rows(hip, oracle):
    x_np = np.random.default_rng(2).integers(0, 1 << 32, size=(2, 50000), dtype=np.uint64).astype(np.uint32)
    want, got = _both(hip, x_np)
    assert np.array_equal(want, got)
    assert np.array_equal(got, oracle.to_vec(oracle.argmax(oracle.tensor(x_np))))


def test_rejects_what_it_cannot_do_without_allocating(hip, cg):
    x = hip.tensor(np.ones((2, 64), dtype=np.float32))
    out = hip.tensor(np.zeros((2, 1), dtype=np.uint32))
    with pytest.raises(cg.BackendPanic, match="deferred"):
        hip.argmax_into(hip.add(x, x), out)                             # not in memory yet
    with pytest.raises(cg.BackendPanic):
        hip.argmax_into(x, hip.tensor(np.zeros((2, 2), dtype=np.uint32)))   # wrong shape
    with pytest.raises(cg.BackendPanic):
        hip.argmax_into(x, hip.tensor(np.zeros((2, 1), dtype=np.float32)))  # wrong dtype
    with pytest.raises(cg.BackendPanic):
        hip.argmax_into(x, hip.zeros((2, 1), cg.U32))                   # a constant, not memory
    hip.argmax_into(hip.realize(hip.add(x, x)), out)                    # realised beforehand: fine
    assert list(hip.to_vec(out)) == [63, 63]


def test_two_backends_do_not_share_scratch(hip, hip_bf16, oracle):
    """Every backend owns a slice of the device's scratch array: split reductions of two backends (two
    streams), issued one behind the other without a wait in between, both give the right answer."""
    rng = np.random.default_rng(9)
    a_np = rng.standard_normal((1, 1, 128256)).astype(np.float32)
    b_np = (rng.standard_normal((1, 1, 128256)).astype(np.float32).view(np.uint32) & 0xFFFF0000).view(np.float32)
    a, b = hip.tensor(a_np), hip_bf16.tensor(b_np)
    oa = hip.realize(hip.tensor(np.full((1, 1, 1), 0xFFFFFFFF, dtype=np.uint32) + np.zeros((1, 1, 1), np.uint32)))
    ob = hip_bf16.realize(hip_bf16.tensor(np.full((1, 1, 1), 0xFFFFFFFF, dtype=np.uint32) + np.zeros((1, 1, 1), np.uint32)))
    for _ in range(8):
        hip.argmax_into(a, oa)
        hip_bf16.argmax_into(b, ob)
    assert hip.to_vec(oa)[0] == int(np.argmax(a_np)) and hip_bf16.to_vec(ob)[0] == int(np.argmax(b_np))
