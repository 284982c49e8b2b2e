"""The five benchmark configurations as the reference CPU transformer runs them.

Oracle (test infrastructure).  Each `*_cpu` function issues, on float32
buffers with `out=`, the statement sequence that
ngraph/transformers/cputransform.py:512-761 generates for the graph the
reference front end builds:

  C1  tanh(a*x+b) * sigmoid(x)         sigmoid = reciprocal(exp(-x)+1), op_graph.py:4183-4197
  C2  BatchNorm forward (training)      frontends/neon/layer.py:1242-1257; mean = sum/size,
                                        variance two-pass, op_graph.py:4007-4009, 4252-4266
  C3  Adam update                       frontends/neon/optimizer.py:446-470
  C4  LSTM cell pointwise block         frontends/neon/layer.py:1630-1647 (gate order i,f,o,g :1615)
  C5  flex16 relu(x*w+b)                frontends/neon/activation.py:46; flex rules in flex_model.py

Inputs are seeded per configuration (seeds 0-4, NumPy RandomState).  Temporaries are preallocated
(the CPU transformer runs out of two preallocated float32 pools,
cputransform.py:998-1007), so timing one of these functions measures ufunc
work only.
"""
import numpy as np

f32 = np.float32


class Workspace(object):
    """Preallocated float32 temporaries, handed out by name."""

    def __init__(self):
        self._bufs = {}

    def get(self, name, shape):
        key = (name, tuple(shape))
        buf = self._bufs.get(key)
        if buf is None:
            buf = np.empty(shape, dtype=f32)
            self._bufs[key] = buf
        return buf


# --------------------------------------------------------------------------- C1
def c1_inputs(shape=(1024, 1024), seed=0):
    rs = np.random.RandomState(seed)
    x = rs.normal(0, 1, shape).astype(f32)
    a, b = rs.uniform(-1, 1, 2).astype(f32)
    return x, a, b


def c1_cpu(x, a, b, ws=None):
    ws = ws or Workspace()
    t = ws.get("t", x.shape)
    u = ws.get("u", x.shape)
    y = ws.get("y", x.shape)
    np.multiply(a, x, out=t)            # Multiply
    np.add(t, b, out=t)                 # Add
    np.tanh(t, out=t)                   # TanhOp
    np.negative(x, out=u)               # NegativeOp
    np.exp(u, out=u)                    # ExpOp
    np.add(u, f32(1), out=u)            # Add
    np.reciprocal(u, out=u)             # ReciprocalOp
    np.multiply(t, u, out=y)            # Multiply
    return y


# --------------------------------------------------------------------------- C2
def c2_inputs(C=256, R=56 * 56 * 64, seed=1):
    rs = np.random.RandomState(seed)
    # generated channel-major [C, H*W*N], the flattened view BatchNorm works on
    x = rs.normal(0.5, 2, (C, R)).astype(f32)
    gamma, beta = rs.uniform(0.5, 1.5, (2, C)).astype(f32)
    return x, gamma, beta


def c2_cpu(x, gamma, beta, eps=1e-5, ws=None):
    """Returns (y, mean, var); x is [C, R], reduced over axis 1."""
    ws = ws or Workspace()
    C, R = x.shape
    mean = ws.get("mean", (C,))
    var = ws.get("var", (C,))
    d = ws.get("d", x.shape)
    y = ws.get("y", x.shape)
    rstd = ws.get("rstd", (C,))
    np.sum(x, axis=1, out=mean)                       # Sum
    np.divide(mean, f32(R), out=mean)                 # Divide by TensorSizeOp
    np.subtract(x, mean[:, None], out=d)              # Subtract (broadcast view)
    np.square(d, out=y)                               # SquareOp
    np.sum(y, axis=1, out=var)                        # Sum
    np.divide(var, f32(R), out=var)                   # Divide
    np.add(var, f32(eps), out=rstd)                   # Add
    np.sqrt(rstd, out=rstd)                           # SqrtOp
    np.reciprocal(rstd, out=rstd)                     # ReciprocalOp
    np.multiply(d, rstd[:, None], out=y)              # Multiply
    np.multiply(gamma[:, None], y, out=y)             # Multiply
    np.add(y, beta[:, None], out=y)                   # Add
    return y, mean, var


# --------------------------------------------------------------------------- C3
def c3_inputs(n=25600000, seed=2):
    rs = np.random.RandomState(seed)
    p = rs.normal(0, 0.02, n).astype(f32)
    g = rs.normal(0, 1e-3, n).astype(f32)
    m = np.zeros(n, dtype=f32)
    v = np.zeros(n, dtype=f32)
    return p, g, m, v


def adam_ell(t, lr=1e-3, beta1=0.9, beta2=0.999):
    """ell = lr * sqrt(1 - beta2**t) / (1 - beta1**t) as float32 graph ops (optimizer.py:455)."""
    t = f32(t)
    b1, b2, one = f32(beta1), f32(beta2), f32(1)
    num = np.sqrt(np.subtract(one, np.power(b2, t, dtype=f32), dtype=f32), dtype=f32)
    den = np.subtract(one, np.power(b1, t, dtype=f32), dtype=f32)
    return np.divide(np.multiply(f32(lr), num, dtype=f32), den, dtype=f32)


def c3_cpu(p, g, m, v, t, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, ws=None):
    """One Adam step in place on p, m, v (optimizer.py:457-468, scale_factor = 1)."""
    ws = ws or Workspace()
    a = ws.get("a", p.shape)
    b = ws.get("b", p.shape)
    ell = adam_ell(t, lr, beta1, beta2)
    b1, b2 = f32(beta1), f32(beta2)
    omb1 = np.subtract(f32(1), b1, dtype=f32)         # (1 - beta_1) on float32 constants
    omb2 = np.subtract(f32(1), b2, dtype=f32)
    np.multiply(m, b1, out=a)                         # m * beta_1
    np.multiply(omb1, g, out=b)                       # (1 - beta_1) * grad
    np.add(a, b, out=m)                               # assign(m, ...)
    np.multiply(v, b2, out=a)                         # v * beta_2
    np.multiply(omb2, g, out=b)                       # (1 - beta_2) * grad
    np.multiply(b, g, out=b)                          # ... * grad
    np.add(a, b, out=v)                               # assign(v, ...)
    np.multiply(ell, m, out=a)                        # (scale_factor * ell) * m, x1 pruned
    np.sqrt(v, out=b)                                 # sqrt(v)
    np.add(b, f32(eps), out=b)                        # + epsilon
    np.divide(a, b, out=a)
    np.subtract(p, a, out=p)                          # assign(variable, ...)
    return p, m, v


# --------------------------------------------------------------------------- C4
def c4_inputs(H=1024, N=64, seed=3):
    """gates logical [4H, N] and c_prev logical [H, N], both stored transposed."""
    rs = np.random.RandomState(seed)
    gates_store = rs.normal(0, 1, (N, 4 * H)).astype(f32)     # memory layout [N, 4H]
    cprev_store = rs.normal(0, 1, (N, H)).astype(f32)
    return gates_store, cprev_store


def _sigmoid(x, out, tmp):
    np.negative(x, out=tmp)
    np.exp(tmp, out=tmp)
    np.add(tmp, f32(1), out=tmp)
    np.reciprocal(tmp, out=out)


def c4_cpu(gates_store, cprev_store, ws=None):
    """Returns (c, h, db) with c, h logical [H, N] (contiguous) and db [4H]."""
    ws = ws or Workspace()
    N, H4 = gates_store.shape
    H = H4 // 4
    gates = gates_store.T                 # logical [4H, N], strides (1, 4H) elements
    c_prev = cprev_store.T                # logical [H, N]
    gi, gf, go, gg = (gates[k * H:(k + 1) * H] for k in range(4))   # order i, f, o, g
    tmp = ws.get("tmp", (H, N))
    i = ws.get("i", (H, N))
    f = ws.get("f", (H, N))
    o = ws.get("o", (H, N))
    g = ws.get("g", (H, N))
    c = ws.get("c", (H, N))
    h = ws.get("h", (H, N))
    db = ws.get("db", (H4,))
    _sigmoid(gi, i, tmp)
    _sigmoid(gf, f, tmp)
    _sigmoid(go, o, tmp)
    np.tanh(gg, out=g)
    np.multiply(f, c_prev, out=c)
    np.multiply(i, g, out=tmp)
    np.add(c, tmp, out=c)
    np.tanh(c, out=tmp)
    np.multiply(o, tmp, out=h)
    np.sum(gates, axis=1, out=db)
    return c, h, db


# --------------------------------------------------------------------------- C5
def c5_inputs(n=16 * 1024 * 1024, seed=4):
    rs = np.random.RandomState(seed)
    x = rs.normal(0, 1, n).astype(f32)
    w = rs.normal(0, 0.1, n).astype(f32)
    b = rs.uniform(-0.1, 0.1, n).astype(f32)
    return x, w, b


def c5_cpu_float(xf, wf, bf, ws=None):
    """relu(x*w+b) on dequantised float32 operands, before output quantisation."""
    ws = ws or Workspace()
    t = ws.get("t", xf.shape)
    np.multiply(xf, wf, out=t)            # Multiply
    np.add(t, bf, out=t)                  # Add
    np.maximum(t, f32(0), out=t)          # Maximum(x, 0); slope*minimum(0, x) is pruned for slope 0
    return t
