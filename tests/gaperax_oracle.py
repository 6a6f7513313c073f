"""Plain, slow float64 statement of the Gaperax design, one function per mechanism, for the tests of the layer-stack model class.

It shares nothing with the product path: numpy only, whole sequences at once, no cache, no pages, no absorbed projections.
`forward` takes the config.json dict of a model and its tensors (name -> float array) and returns the logits of every position of ONE
sequence (and, on request, the residual stream after every layer).

Notation: x residual stream [T, width]; positions p = 0..T-1; a layer is  x <- x + mixer(N1(x)),  x <- x + ff(N2(x)).
"""
import math

import numpy as np

from tests.stack_oracle import bf16_round  # noqa: F401  (re-exported: the tests round their random tensors with it)


def sigmoid(z):
    return 0.5 * (1.0 + np.tanh(0.5 * np.asarray(z, np.float64)))  # (= 1 / (1 + e^-z), without the overflow of e^-z far below 0)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_norm(v, w, eps):
    """v / sqrt(mean(v^2) + eps) * w over the last axis"""
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps) * w


def dyt(x, w, b, alpha):
    """Dynamic Tanh: no statistics of x, an element-wise squash with a learned slope"""
    return np.tanh(float(np.asarray(alpha).reshape(-1)[0]) * x) * w + b


def rotary_table(rot, positions):
    """-> (cos, sin) [T, dims / 2] of the angles p * f_i with the frequencies of `rot` (base, dims, optional YaRN scaling)"""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def turn_dim(t):  # the (fractional) pair index whose wavelength makes t turns over the original length
            return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))
        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = np.asarray(positions, np.float64)[:, None] * f[None]
    return np.cos(ang) * mag, np.sin(ang) * mag


def rotate_pairs(v, cos, sin):
    """v [T, ..., n] with n >= 2 * cos.shape[1]: dimensions (2i, 2i+1) of the first 2 * pairs are turned by the angle of pair i, the
    rest pass.  cos / sin [T, pairs]."""
    out = np.array(v, np.float64)
    n = 2 * cos.shape[1]
    shape = (v.shape[0],) + (1,) * (v.ndim - 2) + (cos.shape[1],)
    c, s = cos.reshape(shape), sin.reshape(shape)
    a, b = v[..., 0:n:2], v[..., 1:n:2]
    out[..., 0:n:2] = a * c - b * s
    out[..., 1:n:2] = b * c + a * s
    return out


def latent_attention(h, tw, p, mx, eps):
    """queries and keys / values through low-rank latents; a rotated key part shared by all heads; causal softmax whose denominator
    also holds exp(sink_h)"""
    T = h.shape[0]
    H, dim, rd, vdim, kr = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    cq = rms_norm(h @ tw[p + "dq"].T, tw[p + "dq.norm"], eps)
    q = (cq @ tw[p + "uq"].T).reshape(T, H, dim + rd)
    ckv = h @ tw[p + "dkv"].T
    c = rms_norm(ckv[:, :kr], tw[p + "dkv.norm"], eps)
    k_rot = ckv[:, kr:]
    k_un = (c @ tw[p + "uk"].T).reshape(T, H, dim)
    v = (c @ tw[p + "uv"].T).reshape(T, H, vdim)
    cos, sin = rotary_table(mx["rot"], np.arange(T))
    q_rot = rotate_pairs(q[:, :, dim:], cos, sin)
    k_rot = rotate_pairs(k_rot, cos, sin)
    scores = [(q[:, hd, :dim] @ k_un[:, hd].T + q_rot[:, hd] @ k_rot.T) * mx["scale"] for hd in range(H)]
    return softmax_with_sink(np.stack(scores), v, tw[p + "sink"]).reshape(T, H * vdim) @ tw[p + "o"].T


def softmax_with_sink(scores, v, sink, positions=None):
    """scores [H, Tq, Tk] (already scaled), v [Tk, H, vdim], queries at `positions` (default 0..Tq-1): causal softmax whose denominator
    also holds exp(sink_h) — a term without key or value -> [Tq, H, vdim]"""
    H, Tq, Tk = scores.shape
    p = np.arange(Tq) if positions is None else np.asarray(positions)
    seen = np.arange(Tk)[None, :] <= p[:, None]
    out = np.zeros((Tq, H, v.shape[2]))
    for hd in range(H):
        s = np.where(seen, scores[hd], -np.inf)
        m = np.maximum(s.max(-1, keepdims=True), sink[hd])
        e = np.exp(s - m)
        out[:, hd] = (e / (e.sum(-1, keepdims=True) + np.exp(sink[hd] - m))) @ v[:, hd]
    return out


def visible(T, mask, positions=None):
    """[Tq, T] bool: key j is seen from position i (queries at `positions`, default 0..T-1)"""
    i = (np.arange(T) if positions is None else np.asarray(positions))[:, None]
    j = np.arange(T)[None, :]
    vis = j <= i
    if mask:
        vis = vis & ((i - j < int(mask["size"])) | (j < int(mask.get("keep_first", 0))))
    return vis


def sigmoid_weighted_values(q, k, v, scale, mask, head_bias, talk, positions=None):
    """q [Tq, H, dim] at `positions` over k [Tk, G, dim], v [Tk, G, vdim] at 0..Tk-1: every visible key weighs
    sigmoid(q . k * scale - slope_h * distance + head_bias_h) (no normalisation over keys), slope_h = 2^(-8 (h + 1) / H); the heads'
    weights are mixed by `talk`; head h sums the values of its own key/value head -> [Tq, H, vdim]"""
    Tq, H, _ = q.shape
    Tk, G, _ = k.shape
    p = np.arange(Tq) if positions is None else np.asarray(positions)
    vis = visible(Tk, mask, p)
    dist = (p[:, None] - np.arange(Tk)[None, :]).astype(np.float64)
    w = np.zeros((H, Tq, Tk))
    for hd in range(H):
        slope = 2.0 ** (-8.0 * (hd + 1) / H)
        s = (q[:, hd] @ k[:, hd // (H // G)].T) * scale - slope * dist
        w[hd] = np.where(vis, sigmoid(s + head_bias[hd]), 0.0)
    w = np.einsum("hg,gij->hij", talk, w)
    return np.stack([w[hd] @ v[:, hd // (H // G)] for hd in range(H)], 1)


def gated_sigmoid_attention(h, tw, p, mx, eps):
    """biased projections, one RMS norm over all of q and one over all of k, no rotation; sigmoid weights in a window that also keeps the
    first tokens; a sigmoid gate on the concatenated heads"""
    T = h.shape[0]
    H, G, dim, vdim = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    q = rms_norm(h @ tw[p + "q"].T + tw[p + "q.b"], tw[p + "q.norm"], eps).reshape(T, H, dim)
    k = rms_norm(h @ tw[p + "k"].T + tw[p + "k.b"], tw[p + "k.norm"], eps).reshape(T, G, dim)
    v = (h @ tw[p + "v"].T + tw[p + "v.b"]).reshape(T, G, vdim)
    out = sigmoid_weighted_values(q, k, v, mx["scale"], mx.get("mask"), tw[p + "pb"], tw[p + "talk"]).reshape(T, H * vdim)
    return (out * sigmoid(h @ tw[p + "g"].T)) @ tw[p + "o"].T


def gated_ff(h, tw, p):
    return (gelu_tanh(h @ tw[p + "gate"].T) * (h @ tw[p + "up"].T)) @ tw[p + "down"].T


def forward(cfg, tensors, tokens, layers_out=None):
    """logits [T, vocab] (float64) of one whole sequence"""
    tw = {k: np.asarray(v, np.float64) for k, v in tensors.items()}
    eps = (cfg.get("norm") or {}).get("eps", 1e-6)
    x = tw["embed"][np.asarray(tokens)]

    def norm(name, v):
        return dyt(v, tw[name], tw[name + ".b"], tw[name + ".alpha"])
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % (layer["weights_of"] if layer.get("weights_of") is not None else i)
        h = norm(p + "norm1", x)
        if layer["type"] == "latent_attention":
            x = x + latent_attention(h, tw, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "attention":
            x = x + gated_sigmoid_attention(h, tw, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp"):
            x = x + gated_ff(norm(p + "norm2", x), tw, p + "mlp.")
        if layers_out is not None:
            layers_out.append(x.copy())
    return norm("final.norm", x) @ tw["head"].T


# ------------------------------------------------------------------------------------------------ small random models
def tensor_shapes(cfg):
    """name -> shape of every tensor a model of this config has"""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,), "final.norm.b": (W,), "final.norm.alpha": ()}
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p = "l%d." % i
        mx = layer["mixer"]
        for n in ("norm1", "norm2") if layer.get("mlp") else ("norm1",):
            out[p + n], out[p + n + ".b"], out[p + n + ".alpha"] = (W,), (W,), ()
        H, dim, vdim = mx["heads"], mx["dim"], mx["vdim"]
        if layer["type"] == "latent_attention":
            rd, kr, qr = mx["rot_dim"], mx["kv_rank"], mx["q_rank"]
            out.update({p + "mix.dq": (qr, W), p + "mix.dq.norm": (qr,), p + "mix.uq": (H * (dim + rd), qr), p + "mix.dkv": (kr + rd, W),
                        p + "mix.dkv.norm": (kr,), p + "mix.uk": (H * dim, kr), p + "mix.uv": (H * vdim, kr), p + "mix.sink": (H,),
                        p + "mix.o": (W, H * vdim)})
        else:
            G = mx.get("kv_heads", H)
            out.update({p + "mix.q": (H * dim, W), p + "mix.q.b": (H * dim,), p + "mix.k": (G * dim, W), p + "mix.k.b": (G * dim,),
                        p + "mix.v": (G * vdim, W), p + "mix.v.b": (G * vdim,), p + "mix.q.norm": (H * dim,), p + "mix.k.norm": (G * dim,),
                        p + "mix.talk": (H, H), p + "mix.pb": (H,), p + "mix.g": (H * vdim, W), p + "mix.o": (W, H * vdim)})
        if layer.get("mlp"):
            f = layer["mlp"]["ff"]
            out.update({p + "mlp.gate": (f, W), p + "mlp.up": (f, W), p + "mlp.down": (W, f)})
    return out


def random_tensors(cfg, seed):
    """bfloat16-representable float32 tensors; projections ~ N(0, 1.5 / sqrt(fan in)) so that scores spread and gates decide"""
    r = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(".alpha"):
            a = np.array(0.6 + 0.3 * r.random())
        elif name.endswith(".norm") or name.endswith("norm1") or name.endswith("norm2"):
            a = 1.0 + 0.2 * r.standard_normal(shape)
        elif name.endswith(".b"):
            a = 0.1 * r.standard_normal(shape)
        elif name.endswith(".sink") or name.endswith(".pb"):
            a = r.standard_normal(shape)
        elif name.endswith(".talk"):
            a = np.eye(shape[0]) + 0.3 * r.standard_normal(shape)
        elif name == "embed":
            a = r.standard_normal(shape)
        else:
            a = 1.5 * r.standard_normal(shape) / math.sqrt(shape[-1])
        out[name] = bf16_round(np.asarray(a, np.float32))
    return out
