"""stdlib `nn`: activations, softmax and linear layers as op sequences.

Mirror of catgrad/src/stdlib/nn/mod.rs (same function names, argument order and emitted
operations).  The backend recognises these sequences and runs them as fused kernels; the
functions below must therefore keep emitting exactly what the reference emits.
"""
import math

import numpy as np

from .lang import (Module, TENSOR, broadcast, cast, constant, dtype, matmul, max, pack, param,
                   pow, reshape, shape, sum, to_nat, transpose, unpack)

E = float(np.float32(math.e))    # std::f32::consts::E
PI = float(np.float32(math.pi))  # std::f32::consts::PI


class _NNModule(Module):
    """trait NNModule (nn/mod.rs:12-34): one tensor in, one tensor out, path nn.<name>."""
    name = None
    fn = None

    def path(self):
        from .lang import path
        return path(["nn", self.name])

    def sort(self):
        return [TENSOR], [TENSOR]

    def def_(self, builder, args):
        (x,) = args
        return [type(self).fn(builder, x)]


# nn/mod.rs:117-121
def sqrt(builder, x):
    sh = shape(builder, x)
    e = constant(builder, 0.5, sh)
    return pow(builder, x, e)


# nn/mod.rs:123-128
def exp(builder, x):
    sh = shape(builder, x)
    e = constant(builder, E, sh)
    e = cast(builder, e, dtype(builder, x))
    return pow(builder, e, x)


# nn/mod.rs:130-136
def sigmoid(builder, x):
    sh = shape(builder, x)
    one = constant(builder, 1.0, sh)
    one = cast(builder, one, dtype(builder, x))
    return one / (one + exp(builder, -x))


# nn/mod.rs:138-144
def tanh(builder, x):
    sh = shape(builder, x)
    one = constant(builder, 1.0, sh)
    two = constant(builder, 2.0, sh)
    return two * sigmoid(builder, two * x) - one


# nn/mod.rs:146-148
def silu(builder, x):
    return x * sigmoid(builder, x)


# nn/mod.rs:150-160: tanh-approximated GELU
def gelu(builder, x):
    sh = shape(builder, x)
    c = constant(builder, float(np.sqrt(np.float32(2.0) / np.float32(PI))), sh)
    one = constant(builder, 1.0, sh)
    three = constant(builder, 3.0, sh)
    half = constant(builder, 0.5, sh)
    k = constant(builder, 0.044715, sh)
    return half * x * (one + tanh(builder, c * (x + k * pow(builder, x, three))))


# nn/mod.rs:162-171
def softmax(builder, x):
    x_shape = shape(builder, x)
    m = max(builder, x)
    bmax = broadcast(builder, m, x_shape)
    x = x - bmax
    ex = exp(builder, x)
    s = sum(builder, ex)
    bsum = broadcast(builder, s, x_shape)
    return ex / bsum


class Sigmoid(_NNModule):
    name, fn = "sigmoid", staticmethod(sigmoid)


class Exp(_NNModule):
    name, fn = "exp", staticmethod(exp)


class Sqrt(_NNModule):
    name, fn = "sqrt", staticmethod(sqrt)


class Gelu(_NNModule):
    name, fn = "gelu", staticmethod(gelu)


class Tanh(_NNModule):
    name, fn = "tanh", staticmethod(tanh)


class Silu(_NNModule):
    name, fn = "silu", staticmethod(silu)


class Softmax(_NNModule):
    name, fn = "softmax", staticmethod(softmax)


# nn/mod.rs:174-199
def linear_b_param(builder, in_dim, out_dim, weight, bias, x):
    w_t = transpose(builder, 0, 1, weight)
    sh = shape(builder, x)
    batch_size, _, _ = unpack(builder, 3, sh)
    in_dim = to_nat(builder, in_dim)
    out_dim = to_nat(builder, out_dim)
    sh = pack(builder, [batch_size, in_dim, out_dim])
    w_t = reshape(builder, sh, w_t)
    m = matmul(builder, x, w_t)
    if bias is not None:
        sh = shape(builder, m)
        bb = broadcast(builder, bias, sh)
        return m + bb
    return m


def linear_no_bias_param(builder, in_dim, out_dim, weight, x):
    return linear_b_param(builder, in_dim, out_dim, weight, None, x)


def linear_param(builder, in_dim, out_dim, weight, bias, x):
    return linear_b_param(builder, in_dim, out_dim, weight, bias, x)


# nn/mod.rs:222-238
def linear_b(builder, in_dim, out_dim, bias, p, x):
    weight = param(builder, p.extend(["weight"]))
    b = param(builder, p.extend(["bias"])) if bias else None
    return linear_b_param(builder, in_dim, out_dim, weight, b, x)


def linear_no_bias(builder, in_dim, out_dim, p, x):
    return linear_b(builder, in_dim, out_dim, False, p, x)


def linear(builder, in_dim, out_dim, p, x):
    return linear_b(builder, in_dim, out_dim, True, p, x)


def stdlib_definitions():
    """stdlib_definitions.rs:19-32: the definitions every Environment starts with."""
    return [Sigmoid(), Exp(), Sqrt(), Tanh(), Gelu(), Silu(), Softmax()]
