"""Inputs of the golden vectors for the elementwise / reduction / optimizer slots, regenerated
from the seeds tests/golden/make_golden.py used (the oracle's RNG restatement is pinned
against the reference's in test_oracle.py)."""
import numpy as np

BCAST = (((5, 7), (5, 7)), ((2, 3), (3,)), ((2, 1), (1, 3)), ((4, 1, 6), (3, 1)), ((2, 3, 4), (1,)),
         ((3, 8, 16), (8, 1)))
BINARY = ("add", "sub", "mul", "div", "equal", "greater")
UNARY = ("neg", "abs", "exp", "log", "sqrt", "square", "sigmoid", "tanh")
REDUCE_SHAPES = ((6, 10), (4, 5, 6), (3, 200))
SOFTMAX_SHAPES = ((5, 7), (3, 300), (2, 1000), (4, 64))
LAYERNORM_SHAPES = ((6, 16), (2, 5, 100), (3, 768))
OPTIMIZERS = {
    "opt_adam": ("adam", dict(lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)),
    "opt_adamw": ("adamw", dict(lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)),
    "opt_sgd_plain": ("sgd", dict(lr=5e-2, momentum=0.0, wd=0.0, nesterov=False)),
    "opt_sgd_momentum": ("sgd", dict(lr=5e-2, momentum=0.9, wd=0.01, nesterov=False)),
    "opt_sgd_nesterov": ("sgd", dict(lr=5e-2, momentum=0.9, wd=0.01, nesterov=True)),
}


def binary_inputs(oracle, case):
    sa, sb = BCAST[case]
    oracle.seed(7000 + case)
    a = np.round(oracle.uniform((int(np.prod(sa)),), -2.0, 2.0) * 4) / 4
    b = np.round(oracle.uniform((int(np.prod(sb)),), -2.0, 2.0) * 4) / 4
    return a.reshape(sa).astype(np.float32), b.reshape(sb).astype(np.float32)


def unary_input(oracle):
    oracle.seed(7100)
    return np.concatenate([oracle.uniform((200,), -4.0, 4.0),
                           np.array([0.0, -0.0, 1.0, -1.0, 30.0, -30.0, 1e-20], np.float32)])


def reduce_inputs(oracle):
    oracle.seed(7200)
    return [oracle.uniform(shp, -1.0, 1.0) for shp in REDUCE_SHAPES]


def softmax_inputs(oracle):
    oracle.seed(7300)
    return [oracle.uniform(shp, -6.0, 6.0) for shp in SOFTMAX_SHAPES]


def layernorm_inputs(oracle):
    oracle.seed(7400)
    return [(oracle.uniform(shp, -3.0, 5.0), oracle.uniform((shp[-1],), 0.5, 1.5), oracle.uniform((shp[-1],), -1.0, 1.0))
            for shp in LAYERNORM_SHAPES]


def optimizer_inputs(oracle):
    oracle.seed(7500)
    w0 = oracle.uniform((300,), -1.0, 1.0)
    return w0, [oracle.uniform((300,), -1.0, 1.0) for _ in range(3)]


def bias_corrections(beta1, beta2, step):
    """1 - beta^t in fp32, as adam_step computes them with powf (src/core/optim.c:270-271)."""
    b1, b2, t = np.float32(beta1), np.float32(beta2), np.float32(step)
    return float(np.float32(1) - np.power(b1, t, dtype=np.float32)), float(np.float32(1) - np.power(b2, t, dtype=np.float32))
