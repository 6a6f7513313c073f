"""Plain, slow float64 statement of the Ditilix design, one function per mechanism, for the tests of the layer-stack model class.

It shares nothing with the product path: numpy only, whole sequences at once, no cache, no pages.  `forward` takes the config.json
dict of a model and its tensors (name -> float array) and returns the logits of every position of ONE sequence (and, on request, the
residual stream after every layer).

Notation: x residual stream [T, width]; h = norm(x); positions p = 0..T-1.
"""
import math

import numpy as np


def bf16_round(a):
    """nearest-even rounding of float32 values to bfloat16, returned as float32"""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32)


def position_vector(T, width, base=10000.0):
    """entry 2i: sin(p * base^(-2i/width)), entry 2i+1: cos of the same angle"""
    pe = np.zeros((T, width))
    p = np.arange(T, dtype=np.float64)[:, None]
    i = np.arange((width + 1) // 2, dtype=np.float64)[None]
    ang = p * base ** (-2.0 * i / width)
    pe[:, 0::2] = np.sin(ang)[:, : pe[:, 0::2].shape[1]]
    pe[:, 1::2] = np.cos(ang)[:, : pe[:, 1::2].shape[1]]
    return pe


def rms_div(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis"""
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)


def group_norm(x, w, groups, eps):
    T, width = x.shape
    parts = x.reshape(T, groups, width // groups)
    return rms_div(parts, eps).reshape(T, width) * w


def query_temperature(p, coef, every):
    return 1.0 + coef * np.log(np.floor((p + 1) / every) + 1.0)


def attention_core(q, k, v, mx, positions=None):
    """q [Tq, H, dim] at `positions` (default 0..Tq-1) over keys / values k [Tk, G, dim], v [Tk, G, vdim] at positions 0..Tk-1:
    temperature on q, scaled and soft-capped scores, key j visible to position p iff j <= p, ordinary softmax -> [Tq, H, vdim]"""
    Tq, H, _ = q.shape
    Tk, G, vdim = v.shape
    p = np.arange(Tq, dtype=np.float64) if positions is None else np.asarray(positions, np.float64)
    qt = mx.get("q_temp")
    if qt:
        q = q * query_temperature(p, qt["coef"], qt["every"])[:, None, None]
    out = np.zeros((Tq, H, vdim))
    j = np.arange(Tk, dtype=np.float64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * mx["scale"]
        cap = mx.get("softcap")
        if cap:
            s = cap * np.tanh(s / cap)
        s = np.where(j[None, :] <= p[:, None], s, -np.inf)
        s = s - s.max(-1, keepdims=True)
        e = np.exp(s)
        out[:, hd] = (e / e.sum(-1, keepdims=True)) @ v[:, g]
    return out


def attention(h, wq, wk, wv, wo, mx, kv=None):
    """causal softmax attention of one sequence; kv = (k, v) of another layer when this one has no projections of its own.
    Returns (output [T, width], (k, v))."""
    T = h.shape[0]
    H, G, dim, vdim = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
    q = (h @ wq.T).reshape(T, H, dim)
    if kv is None:
        kv = ((h @ wk.T).reshape(T, G, dim), (h @ wv.T).reshape(T, G, vdim))
    return attention_core(q, kv[0], kv[1], mx).reshape(T, H * vdim) @ wo.T, kv


def polynorm(z, coef, eps):
    a, b, c, e = [float(t) for t in coef]
    return a * rms_div(z, eps) + b * rms_div(z * z, eps) + c * rms_div(z * z * z, eps) + e


def dense_ff(h, w_up, w_down, coef, eps):
    return polynorm(h @ w_up.T, coef, eps) @ w_down.T


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def expert(hin, w_gate, w_up, w_down, limit):
    g = hin @ w_gate.T
    u = hin @ w_up.T
    if limit:
        g = np.minimum(g, limit)
        u = np.clip(u, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


def route(h, w_router, top):
    """-> (expert ids [T, top], weights [T, top]): the `top` largest sigmoid scores, not renormalised"""
    s = sigmoid(h @ w_router.T)
    idx = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    return idx, np.take_along_axis(s, idx, -1)


def moe_ff(h, tensors, prefix, ml):
    T, width = h.shape
    idx, wts = route(h, tensors[prefix + "router"], ml["router"].get("top", 1))
    out = np.zeros((T, width))
    lim = ml["expert"].get("limit")
    for t in range(T):
        for e, w in zip(idx[t], wts[t]):
            pe = "%se%d." % (prefix, e)
            out[t] += expert(w * h[t:t + 1], tensors[pe + "gate"], tensors[pe + "up"], tensors[pe + "down"], lim)[0]
    sh = ml.get("shared")
    if sh:
        ps = prefix + "shared."
        gate = sigmoid(h @ tensors[ps + "sg"].reshape(1, -1).T)
        out = out + gate * expert(h, tensors[ps + "gate"], tensors[ps + "up"], tensors[ps + "down"], sh.get("limit"))
    return out


def forward(cfg, tensors, tokens, layers_out=None):
    """logits [T, vocab] (float64) of one whole sequence"""
    tw = {k: np.asarray(v, np.float64) for k, v in tensors.items()}
    norm = cfg.get("norm") or {}
    eps, groups = norm.get("eps", 1e-6), norm.get("groups", 1)
    width = cfg["width"]
    T = len(tokens)
    x = tw["embed"][np.asarray(tokens)] + position_vector(T, width)
    kv = {}
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        h = group_norm(x, tw[p + "norm1"], groups, eps)
        mx = layer["mixer"]
        src = mx.get("kv_from")
        o, kv_i = attention(h, tw[p + "mix.q"], tw.get(p + "mix.k"), tw.get(p + "mix.v"), tw[p + "mix.o"], mx, kv[src] if src is not None else None)
        if src is None:
            kv[i] = kv_i
        ml = layer.get("mlp")
        if not ml:
            ff = 0.0
        elif ml["kind"] == "dense":
            ff = dense_ff(h, tw[p + "mlp.up"], tw[p + "mlp.down"], tw[p + "mlp.act"], eps)
        else:
            ff = moe_ff(h, tw, p + "mlp.", ml)
        x = x + cfg.get("residual_mult", 1.0) * (o + ff)
        if layers_out is not None:
            layers_out.append(x.copy())
    h = group_norm(x, tw["final.norm"], groups, eps)
    return (h @ tw["head"].T) * cfg.get("logit_scale", 1.0)


# ------------------------------------------------------------------------------------------------ small random models
def tensor_shapes(cfg):
    """name -> shape of every tensor a model of this config has"""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        mx = layer["mixer"]
        H, G, dim, vdim = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
        out[p + "norm1"] = (W,)
        out[p + "mix.q"] = (H * dim, W)
        if mx.get("kv_from") is None:
            out[p + "mix.k"], out[p + "mix.v"] = (G * dim, W), (G * vdim, W)
        out[p + "mix.o"] = (W, H * vdim)
        ml = layer.get("mlp")
        if ml and ml["kind"] == "dense":
            out[p + "mlp.up"], out[p + "mlp.down"], out[p + "mlp.act"] = (ml["ff"], W), (W, ml["ff"]), (4,)
        elif ml:
            out[p + "mlp.router"] = (ml["router"]["experts"], W)
            for e in range(ml["router"]["experts"]):
                f = ml["expert"]["ff"]
                out["%smlp.e%d.gate" % (p, e)], out["%smlp.e%d.up" % (p, e)], out["%smlp.e%d.down" % (p, e)] = (f, W), (f, W), (W, f)
            if ml.get("shared"):
                f = ml["shared"]["ff"]
                out[p + "mlp.shared.gate"], out[p + "mlp.shared.up"], out[p + "mlp.shared.down"], out[p + "mlp.shared.sg"] = (f, W), (f, W), (W, f), (1, W)
    return out


def random_tensors(cfg, seed):
    """bfloat16-representable float32 tensors: projections ~ N(0, 1.5 / sqrt(fan in)) so that attention is peaked and routers decide"""
    r = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith("norm1") or name == "final.norm":
            a = 1.0 + 0.2 * r.standard_normal(shape)
        elif name.endswith("mlp.act"):
            a = np.array([0.7, 0.4, 0.2, 0.05]) + 0.05 * r.standard_normal(4)
        elif name == "embed":
            a = r.standard_normal(shape)
        elif name.endswith("router") or name.endswith(".sg"):
            a = 3.0 * r.standard_normal(shape) / math.sqrt(shape[-1])
        else:
            a = 1.5 * r.standard_normal(shape) / math.sqrt(shape[-1])
        out[name] = bf16_round(a.astype(np.float32))
    return out
