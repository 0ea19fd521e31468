"""The reference's own test vectors and the stdlib definitions, on the HIP backend through the
C ABI and the native evaluator (deferred and eager)."""
import numpy as np
import pytest

import vectors

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["lazy", "eager", "nopat"])
def dev(request, hip, hip_eager, hip_nopat):
    return {"lazy": hip, "eager": hip_eager, "nopat": hip_nopat}[request.param]


def test_reference_backend_vectors(dev):
    vectors.check_backend_unit_vectors(dev)


def test_reference_interpreter_vectors(dev):
    vectors.check_interpreter_vectors(dev)


def test_reference_nn_vectors(dev):
    vectors.check_nn_vectors(dev)


def test_reference_legacy_shape_vectors(dev):
    vectors.check_legacy_shape_vectors(dev)


@pytest.mark.parametrize("name", ["sigmoid", "exp", "sqrt", "tanh", "gelu", "silu", "softmax"])
def test_stdlib_definitions_vs_oracle(oracle, dev, cg, name):
    mod = {m.name: m for m in vectors.nn.stdlib_definitions()}[name]
    g = np.random.default_rng(11)
    x = (g.standard_normal((2, 37, 64)) * 3).astype(np.float32)
    if name == "sqrt":
        x = np.abs(x)
    outs = []
    for be in (oracle, dev):
        it = cg.Interpreter(be, cg.stdlib())
        (y,) = it.run(mod.term(), [be.tensor(x)])
        outs.append(be.numpy(y))
    ref, got = outs
    assert np.allclose(got, ref, rtol=1e-4, atol=1e-6)


def test_softmax_masked_rows(oracle, dev):
    """scale + causal mask + softmax as llama emits it (models/llama.rs:97-107): masked entries
    are f32::MIN, never -inf; every row sums to one; masked probabilities are exactly 0."""
    g = np.random.default_rng(12)
    s = 19
    scores = (g.standard_normal((1, 3, s, s)) * 5).astype(np.float32)

    def f(b, a):
        lang = vectors.lang
        sh = lang.shape(b, a)
        _, _, n, _ = lang.unpack(b, 4, sh)
        a = a / lang.constant(b, 8.0, sh)
        mask = lang.broadcast(b, vectors.helpers.causal_mask(b, n), sh)
        return vectors.nn.softmax(b, a + mask)
    (ref,) = vectors.run(oracle, f, 1, scores)
    (got,) = vectors.run(dev, f, 1, scores)
    assert np.allclose(got, ref, rtol=1e-4, atol=1e-7)
    assert np.allclose(got.sum(-1), 1, atol=1e-5)
    assert np.all(got[0, 0][np.triu_indices(s, 1)] == 0)
