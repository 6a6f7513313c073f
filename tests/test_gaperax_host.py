"""CPU tests of the Gaperax design in the layer-stack model class: the reader of its config.json (every size and constant, optional
mechanisms), the native parser of the layer list it writes (host-only engine: no GPU touched), and the float64 oracle's mechanisms
checked by hand (tests/gaperax_oracle.py)."""
import ctypes as C
import math

import numpy as np
import pytest

from tests import gaperax_oracle as go
from vllm_rs_amd import _lib, checkpoint
from vllm_rs_amd.engine import model_config


def latent(heads=3, dim=8, rot_dim=4, vdim=6, kv_rank=10, q_rank=12, scale=0.3, scaling=True, base=5000.0):
    rot = dict(base=base, dims=rot_dim)
    if scaling:
        rot["scaling"] = dict(factor=3.0, original=64, fast=16.0, slow=2.0)
    return dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale, rot=rot)


def windowed(heads=4, kv_heads=2, dim=6, vdim=5, scale=0.4, size=7, keep_first=2):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if size:
        m["mask"] = dict(size=size, keep_first=keep_first)
    return m


def small_config():
    return dict(architecture="Gaperax", width=24, vocab=50, norm=dict(eps=1e-5), layers=[
        dict(type="attention", mixer=windowed(), mlp=dict(kind="dense", ff=20)),
        dict(type="latent_attention", mixer=latent(), mlp=dict(kind="dense", ff=12)),
        dict(type="attention", mixer=windowed(), mlp=dict(kind="dense", ff=20), weights_of=0),
        dict(type="latent_attention", mixer=latent(scaling=False), mlp=None),
        dict(type="attention", mixer=windowed(heads=2, kv_heads=2, size=0), mlp=None),
    ])


def fields(line):
    return dict(kv.split("=") for kv in line.split()[1:])


def test_config_reader_takes_every_size_and_constant_from_the_config():
    cfg = checkpoint.parse_config(small_config())
    assert cfg["arch"] == "stack" and cfg["design"] == "Gaperax" and cfg["hidden_size"] == 24 and cfg["vocab_size"] == 50 and cfg["num_layers"] == 5
    lines = cfg["spec"].strip().split("\n")
    top = fields(lines[0])
    assert (top["block"], top["norm"], top["pos"], float(top["eps"])) == ("sequential", "dyt", "none", 1e-5)
    l0, l1, l2, l3, l4 = (fields(x) for x in lines[1:])
    assert (l0["mixer"], int(l0["heads"]), int(l0["kv_heads"]), int(l0["dim"]), int(l0["vdim"]), float(l0["scale"])) == ("sigmoid", 4, 2, 6, 5, 0.4)
    assert (int(l0["window"]), int(l0["keep_first"]), float(l0["slope_exp"]), l0["mlp"], int(l0["ff"])) == (7, 2, 8.0, "gated", 20)
    assert (l1["mixer"], int(l1["rot_dim"]), int(l1["kv_rank"]), int(l1["q_rank"]), int(l1["rot_dims"]), float(l1["rot_base"])) == ("latent", 4, 10, 12, 4, 5000.0)
    assert (float(l1["yarn_factor"]), float(l1["yarn_original"]), float(l1["yarn_fast"]), float(l1["yarn_slow"]), int(l1["sink"])) == (3.0, 64.0, 16.0, 2.0, 1)
    assert int(l2["weights_of"]) == 0 and "weights_of" not in l0
    # mechanisms the config leaves out are off: no frequency scaling, no window, no feed-forward
    assert "yarn_factor" not in l3 and l3["mlp"] == "none"
    assert int(l4["window"]) == 0 and int(l4["keep_first"]) == 0
    assert checkpoint.parse_config(small_config(), "float32")["dtype"] == checkpoint.F32


def test_config_reader_rejects_what_the_design_does_not_have():
    bad = small_config()
    bad["layers"][0]["type"] = "recurrent"
    with pytest.raises(ValueError):
        checkpoint.parse_config(bad)
    bad = small_config()
    bad["layers"][1]["mlp"]["kind"] = "moe"
    with pytest.raises(ValueError):
        checkpoint.parse_config(bad)
    with pytest.raises(ValueError):
        checkpoint.parse_config(small_config(), "float16")


def create(spec, cfg):
    L = _lib.load()
    mc = model_config(cfg)
    ec = _lib.EngineConfig(block_size=64, max_num_seqs=4, max_model_len=256, num_gpu_blocks=8, prefill_chunk=8192, device=-1)
    h = L.vra_engine_create_spec(C.byref(mc), C.byref(ec), spec.encode())
    assert h
    return L, h


def test_native_parser_accepts_the_layer_list():
    cfg = checkpoint.parse_config(small_config())
    L, h = create(cfg["spec"], cfg)
    assert L.vra_engine_finalize_weights(h) == 0, L.vra_engine_last_error(h).decode()
    L.vra_engine_destroy(h)


@pytest.mark.parametrize("edit,why", [
    (lambda s: s.replace("weights_of=0", "weights_of=1"), "shapes of the layer it names"),
    (lambda s: s.replace("weights_of=0", "weights_of=2"), "another layer with tensors of its own"),
    (lambda s: s.replace("heads=4 ", "heads=3 ", 1), "multiple of kv_heads"),
    (lambda s: s.replace("rot_dims=4", "rot_dims=6", 1), "rot_dims"),
    (lambda s: s.replace("block=sequential", "block=parallel"), "sequential blocks"),
    (lambda s: s.replace("norm=dyt", "norm=layer"), "norm must be"),
    (lambda s: s.replace("mixer=latent", "mixer=conv", 1), "unknown mixer"),
])
def test_native_parser_refuses_inconsistent_lists(edit, why):
    """the refusal surfaces at the first call that needs the model (loading a tensor), with the reason"""
    cfg = checkpoint.parse_config(small_config())
    L, h = create(edit(cfg["spec"]), cfg)
    a = np.zeros((50, 24), np.uint16)
    shape = (C.c_int64 * 2)(50, 24)
    assert L.vra_engine_load_tensor(h, b"embed", a.ctypes.data_as(C.c_void_p), shape, 2, 2) != 0
    assert why in L.vra_engine_last_error(h).decode()
    L.vra_engine_destroy(h)


# ------------------------------------------------------------------------------------------------ the oracle's mechanisms by hand
def test_dynamic_tanh_and_gated_feed_forward():
    x = np.array([[0.0, 1.0, -2.0]])
    assert np.allclose(go.dyt(x, np.array([2.0, 2.0, 2.0]), np.array([0.5, 0.0, 0.0]), 0.5), [[0.5, 2 * math.tanh(0.5), 2 * math.tanh(-1.0)]])
    assert abs(go.gelu_tanh(np.array([1.0]))[0] - 0.841192) < 1e-6 and go.gelu_tanh(np.array([0.0]))[0] == 0.0
    tw = {"gate": np.eye(2), "up": np.array([[2.0, 0.0], [0.0, 3.0]]), "down": np.array([[1.0, 1.0]])}
    h = np.array([[1.0, -1.0]])
    assert np.allclose(go.gated_ff(h, tw, ""), go.gelu_tanh(np.array([1.0]))[0] * 2.0 + go.gelu_tanh(np.array([-1.0]))[0] * -3.0)


def test_rotary_table_plain_and_scaled():
    rot = dict(base=100.0, dims=4)
    cos, sin = go.rotary_table(rot, [0, 3])
    assert np.allclose(cos[0], 1) and np.allclose(sin[0], 0)
    assert np.allclose(cos[1], [math.cos(3.0), math.cos(0.3)]) and np.allclose(sin[1], [math.sin(3.0), math.sin(0.3)])
    # pairs are neighbours (2i, 2i + 1); what lies behind the rotated dimensions passes
    v = np.array([[1.0, 0.0, 0.0, 2.0, 7.0]])
    out = go.rotate_pairs(v, *go.rotary_table(rot, [3]))
    assert np.allclose(out[0], [math.cos(3.0), math.sin(3.0), -2 * math.sin(0.3), 2 * math.cos(0.3), 7.0])
    # scaling: fast pairs keep their frequency, slow pairs are divided by the factor, both parts grow by 0.1 ln(factor) + 1
    rot = dict(base=10000.0, dims=16, scaling=dict(factor=8.0, original=256, fast=32.0, slow=1.0))
    cos, sin = go.rotary_table(rot, [1])
    mag = 0.1 * math.log(8.0) + 1.0
    f = 10000.0 ** (-2.0 * np.arange(8) / 16)
    ang = np.arctan2(sin[0], cos[0])
    assert np.allclose(np.hypot(cos[0], sin[0]), mag)
    assert np.isclose(ang[0], f[0]) and np.isclose(ang[7], f[7] / 8.0)
    assert np.all(ang <= f + 1e-12) and np.all(ang >= f / 8.0 - 1e-12)


def test_window_keeps_the_first_tokens():
    vis = go.visible(12, dict(size=3, keep_first=2))
    assert vis[10].nonzero()[0].tolist() == [0, 1, 8, 9, 10]
    assert vis[2].nonzero()[0].tolist() == [0, 1, 2] and vis[4].nonzero()[0].tolist() == [0, 1, 2, 3, 4]
    assert vis[5].nonzero()[0].tolist() == [0, 1, 3, 4, 5]
    assert go.visible(5, None)[4].all() and not go.visible(5, None)[2, 3]


def test_sink_counts_once_and_has_no_value():
    """one head, one key: the weight of the key is e^s / (e^s + e^sink)"""
    cfg = dict(heads=1, dim=2, rot_dim=0, vdim=1, kv_rank=2, q_rank=2, scale=1.0, rot=dict(base=10.0, dims=0))
    eye = np.eye(2)
    tw = {"dq": eye, "dq.norm": np.ones(2), "uq": eye, "dkv": eye, "dkv.norm": np.ones(2), "uk": eye, "uv": np.array([[1.0, 0.0]]),
          "sink": np.array([0.7]), "o": np.array([[1.0]])}
    h = np.array([[3.0, 4.0]])
    c = h / np.sqrt((h * h).mean())
    s = float((c * c).sum())
    out = go.latent_attention(h, tw, "", cfg, 0.0)
    assert np.allclose(out, math.exp(s) / (math.exp(s) + math.exp(0.7)) * c[0, 0])


def test_sigmoid_attention_by_hand():
    """two tokens, two heads on one key/value head: weights are plain sigmoids with the distance penalty, mixed by the matrix, gated"""
    mx = dict(heads=2, kv_heads=1, dim=1, vdim=1, scale=2.0)
    one = np.ones((1, 1))
    tw = {"q": np.ones((2, 1)), "q.b": np.zeros(2), "k": one, "k.b": np.zeros(1), "v": one, "v.b": np.array([0.5]), "q.norm": np.ones(2), "k.norm": np.ones(1),
          "pb": np.array([0.1, -0.2]), "talk": np.array([[1.0, 0.5], [0.0, 2.0]]), "g": np.zeros((2, 1)), "o": np.eye(2)}
    h = np.array([[1.0], [-2.0]])
    out = go.gated_sigmoid_attention(h, tw, "", mx, 0.0)
    # q rows are [1, 1] and [-2, -2] before the norm, +-1 after it; k = sign(h); v = h + 0.5
    sl = [2.0 ** -4, 2.0 ** -8]
    w = np.zeros((2, 2, 2))
    for hd in range(2):
        w[hd, 0, 0] = go.sigmoid(2.0 + tw["pb"][hd])
        w[hd, 1, 0] = go.sigmoid(-2.0 - sl[hd] + tw["pb"][hd])
        w[hd, 1, 1] = go.sigmoid(2.0 + tw["pb"][hd])
    mixed = np.einsum("hg,gij->hij", tw["talk"], w)
    v = np.array([1.5, -1.5])
    assert np.allclose(out, 0.5 * np.stack([mixed[0] @ v, mixed[1] @ v], 1))


def test_latent_scores_equal_their_absorbed_form():
    """q_h . (W_uk_h c) = (W_uk_h^T q_h) . c, and the values may be projected after the weighted sum: the cache needs the latent alone"""
    r = np.random.default_rng(0)
    H, dim, kr, vdim, T = 2, 3, 4, 5, 6
    q, c = r.standard_normal((T, H, dim)), r.standard_normal((T, kr))
    uk, uv = r.standard_normal((H * dim, kr)), r.standard_normal((H * vdim, kr))
    for hd in range(H):
        ukh, uvh = uk[hd * dim:(hd + 1) * dim], uv[hd * vdim:(hd + 1) * vdim]
        s1 = q[:, hd] @ (c @ ukh.T).T
        s2 = (q[:, hd] @ ukh) @ c.T
        assert np.allclose(s1, s2)
        w = r.random((T, T))
        assert np.allclose(w @ (c @ uvh.T), (w @ c) @ uvh.T)


def test_oracle_is_causal_and_shares_weights_not_caches():
    cfg = small_config()
    tensors = go.random_tensors(cfg, 3)
    assert not any(n.startswith("l2.") for n in tensors)
    toks = np.random.default_rng(0).integers(0, 50, 30).tolist()
    whole = go.forward(cfg, tensors, toks)
    for n in (1, 2, 9, 17):
        assert np.abs(go.forward(cfg, tensors, toks[:n]) - whole[:n]).max() < 1e-9
    # layer 2 runs with layer 0's tensors on its own input: changing them changes both layers' work
    t2 = dict(tensors)
    t2["l0.mix.talk"] = tensors["l0.mix.talk"].T.copy()
    a, b = [], []
    go.forward(cfg, tensors, toks, a), go.forward(cfg, t2, toks, b)
    assert np.abs(a[0] - b[0]).max() > 1e-4
    # a token outside every window and behind the kept ones does not reach position 20 through layer 0 alone
    cfg1 = dict(cfg, layers=cfg["layers"][:1])
    t_a, t_b = list(toks), list(toks)
    t_b[5] = (toks[5] + 1) % 50
    la, lb = go.forward(cfg1, tensors, t_a), go.forward(cfg1, tensors, t_b)
    assert np.abs(la[11] - lb[11]).max() > 1e-9 and np.abs(la[12:] - lb[12:]).max() == 0.0
    t_b = list(toks)
    t_b[1] = (toks[1] + 1) % 50  # a kept token is seen from everywhere
    assert np.abs(go.forward(cfg1, tensors, t_b)[29] - la[29]).max() > 1e-9
