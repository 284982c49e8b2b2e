"""Seeded inputs of the five benchmark configurations (synthetic data of the stated shapes
and distributions), for benchmarks and examples that should not need the test oracle.

C1  y = tanh(a*x + b) * sigmoid(x), x fp32 [1024, 1024] ~ N(0, 1), a, b ~ U(-1, 1); seed 0
C2  batch-norm forward over x fp32 (C=256, H=56, W=56, N=64) ~ N(0.5, 2), gamma, beta ~
    U(0.5, 1.5); seed 1.  x is generated channel-major [C, H*W*N], the flattened view batch
    normalisation works on (ngraph/frontends/neon/layer.py:1242-1243)
C3  Adam over 25.6 M fp32 parameters: p ~ N(0, 0.02), grad ~ N(0, 1e-3), m = v = 0; seed 2
C4  LSTM cell: gates [4H, N] and c_prev [H, N] ~ N(0, 1), H = 1024, N = 64, both stored
    transposed ([N, 4H] and [N, H] in memory); seed 3
C5  flex16 relu(x*w + b) over 16 M elements: x ~ N(0, 1), w ~ N(0, 0.1), b ~ U(-0.1, 0.1); seed 4
"""
import numpy as np

f32 = np.float32


def c1_inputs(shape=(1024, 1024), seed=0):
    rs = np.random.RandomState(seed)
    x = rs.normal(0, 1, shape).astype(f32)
    a, b = rs.uniform(-1, 1, 2).astype(f32)
    return x, a, b


def c2_inputs(C=256, R=56 * 56 * 64, seed=1):
    rs = np.random.RandomState(seed)
    x = rs.normal(0.5, 2, (C, R)).astype(f32)
    gamma, beta = rs.uniform(0.5, 1.5, (2, C)).astype(f32)
    return x, gamma, beta


def c3_inputs(n=25600000, seed=2):
    rs = np.random.RandomState(seed)
    p = rs.normal(0, 0.02, n).astype(f32)
    g = rs.normal(0, 1e-3, n).astype(f32)
    return p, g, np.zeros(n, dtype=f32), np.zeros(n, dtype=f32)


def c4_inputs(H=1024, N=64, seed=3):
    rs = np.random.RandomState(seed)
    gates_store = rs.normal(0, 1, (N, 4 * H)).astype(f32)
    cprev_store = rs.normal(0, 1, (N, H)).astype(f32)
    return gates_store, cprev_store


def c5_inputs(n=16 * 1024 * 1024, seed=4):
    rs = np.random.RandomState(seed)
    x = rs.normal(0, 1, n).astype(f32)
    w = rs.normal(0, 0.1, n).astype(f32)
    b = rs.uniform(-0.1, 0.1, n).astype(f32)
    return x, w, b
