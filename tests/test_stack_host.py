"""CPU tests of the layer-stack model class: the reader of a Ditilix config.json (every key, optional mechanisms switched off when
absent), the native parser of the layer list it writes (host-only engine: no GPU touched), and the float64 oracle's own consistency
(a prompt's prefix gives the same logits as the whole prompt: causality of every mechanism)."""
import ctypes as C

import numpy as np
import pytest

from tests import stack_oracle as so
from vllm_rs_amd import _lib, checkpoint
from vllm_rs_amd.engine import model_config


def small_config():
    return dict(architecture="Ditilix", width=48, vocab=60, residual_mult=0.5, logit_scale=0.25, norm=dict(eps=1e-5, groups=4), layers=[
        dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.35, softcap=5.0, q_temp=dict(coef=0.2, every=4)),
             mlp=dict(kind="moe", expert=dict(ff=20, limit=1.0), router=dict(experts=4, top=2), shared=dict(ff=8, limit=0.5))),
        dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.35, kv_from=0), mlp=dict(kind="dense", ff=30)),
        dict(type="attention", mixer=dict(heads=2, kv_heads=2, dim=6, scale=0.4), mlp=None),
    ])


def fields(line):
    return dict(kv.split("=") for kv in line.split()[1:])


def test_config_reader_takes_every_size_and_constant_from_the_config():
    cfg = checkpoint.parse_config(small_config())
    assert cfg["arch"] == "stack" and cfg["hidden_size"] == 48 and cfg["vocab_size"] == 60 and cfg["num_layers"] == 3
    lines = cfg["spec"].strip().split("\n")
    assert lines[0].split()[0] == "stack" and len(lines) == 4
    top = fields(lines[0])
    assert (int(top["width"]), int(top["vocab"]), int(top["groups"])) == (48, 60, 4)
    assert (float(top["eps"]), float(top["residual_mult"]), float(top["logit_scale"])) == (1e-5, 0.5, 0.25)
    l0, l1, l2 = (fields(x) for x in lines[1:])
    assert (int(l0["heads"]), int(l0["kv_heads"]), int(l0["dim"]), int(l0["vdim"])) == (4, 2, 8, 12)
    assert (float(l0["scale"]), float(l0["softcap"]), float(l0["temp_coef"]), int(l0["temp_every"]), int(l0["kv_from"])) == (0.35, 5.0, 0.2, 4, -1)
    assert (l0["mlp"], int(l0["experts"]), int(l0["top"]), int(l0["ff"]), float(l0["limit"]), int(l0["shared_ff"]), float(l0["shared_limit"])) == \
        ("moe", 4, 2, 20, 1.0, 8, 0.5)
    # mechanisms the config leaves out are off: no soft cap, no temperature; the value size defaults to the key size
    assert float(l1["softcap"]) == 0.0 and "temp_coef" not in l1 and int(l1["kv_from"]) == 0 and l1["mlp"] == "dense" and int(l1["ff"]) == 30
    assert l2["mlp"] == "none" and int(l2["vdim"]) == 6 and int(l2["kv_heads"]) == 2
    assert checkpoint.parse_config(small_config(), "float32")["dtype"] == checkpoint.F32


def test_config_reader_rejects_what_the_design_does_not_have():
    bad = small_config()
    bad["layers"][0]["type"] = "recurrent"
    with pytest.raises(ValueError):
        checkpoint.parse_config(bad)
    bad = small_config()
    bad["layers"][1]["mlp"]["kind"] = "glu"
    with pytest.raises(ValueError):
        checkpoint.parse_config(bad)
    with pytest.raises(ValueError):
        checkpoint.parse_config(small_config(), "float16")


def host_engine(cfg, spec=None):
    L = _lib.load()
    mc = model_config(cfg)
    ec = _lib.EngineConfig(block_size=64, max_num_seqs=4, max_model_len=256, num_gpu_blocks=8, prefill_chunk=8192, device=-1)
    h = L.vra_engine_create_spec(C.byref(mc), C.byref(ec), (cfg["spec"] if spec is None else spec).encode())
    assert h
    rc = L.vra_engine_finalize_weights(h)  # a host-only engine: scheduler and block manager, no model memory
    return L, h, rc


def test_native_parser_accepts_the_layer_list():
    cfg = checkpoint.parse_config(small_config())
    L, h, rc = host_engine(cfg)
    assert rc == 0, L.vra_engine_last_error(h).decode()
    L.vra_engine_destroy(h)


@pytest.mark.parametrize("edit,why", [
    (lambda s: s.replace("kv_from=0", "kv_from=2"), "earlier layer"),
    (lambda s: s.replace("heads=4 kv_heads=2", "heads=3 kv_heads=2", 1), "multiple of kv_heads"),
    (lambda s: s.replace("groups=4", "groups=5"), "norm groups"),
    (lambda s: s.replace("top=2", "top=9"), "top"),
    (lambda s: s.replace("mlp=dense", "mlp=conv"), "feed-forward kind"),
])
def test_native_parser_refuses_inconsistent_lists(edit, why):
    """the refusal surfaces at the first call that needs the model (loading a tensor), with the reason"""
    cfg = checkpoint.parse_config(small_config())
    L = _lib.load()
    mc = model_config(cfg)
    ec = _lib.EngineConfig(block_size=64, max_num_seqs=4, max_model_len=256, num_gpu_blocks=8, prefill_chunk=8192, device=-1)
    h = L.vra_engine_create_spec(C.byref(mc), C.byref(ec), edit(cfg["spec"]).encode())
    assert h
    a = np.zeros((60, 48), np.uint16)
    shape = (C.c_int64 * 2)(60, 48)
    assert L.vra_engine_load_tensor(h, b"embed", a.ctypes.data_as(C.c_void_p), shape, 2, 2) != 0
    assert why in L.vra_engine_last_error(h).decode()
    L.vra_engine_destroy(h)


def test_oracle_is_causal_and_reads_borrowed_keys():
    cfg = small_config()
    tensors = so.random_tensors(cfg, 3)
    toks = np.random.default_rng(0).integers(0, 60, 40).tolist()
    whole = so.forward(cfg, tensors, toks)
    for n in (1, 4, 5, 17):
        assert np.abs(so.forward(cfg, tensors, toks[:n]) - whole[:n]).max() < 1e-9
    # layer 1 borrows layer 0's keys and values: changing layer 0's key projection changes what layer 1 sees
    t2 = dict(tensors)
    t2["l0.mix.k"] = tensors["l0.mix.k"][::-1].copy()
    layers_a, layers_b = [], []
    so.forward(cfg, tensors, toks, layers_a), so.forward(cfg, t2, toks, layers_b)
    h_same = np.abs(layers_a[0] - layers_b[0]).max()
    assert h_same > 1e-3 and np.abs(layers_a[1] - layers_b[1]).max() > 1e-3


def test_oracle_mechanisms_by_hand():
    # grouped norm: every part ends with unit mean square
    x = np.arange(1, 13, dtype=np.float64).reshape(1, 12)
    h = so.group_norm(x, np.ones(12), 3, 0.0)
    assert np.allclose((h.reshape(3, 4) ** 2).mean(-1), 1.0)
    # query temperature steps at multiples of `every` (p + 1 counts tokens)
    t = so.query_temperature(np.array([0, 2, 3, 6, 7]), 0.5, 4)
    assert np.allclose(t, [1, 1, 1 + 0.5 * np.log(2), 1 + 0.5 * np.log(2), 1 + 0.5 * np.log(3)])
    # PolyNorm of a constant vector: every normalised power is 1
    assert np.allclose(so.polynorm(np.full((1, 8), 2.0), [0.5, 0.25, 0.125, 0.1], 0.0), 0.975)
    # expert: gate clamped from above only, up on both sides
    w1 = np.eye(2)
    y = so.expert(np.array([[5.0, -5.0]]), w1, w1, w1, 2.0)
    g = np.array([2.0, -5.0])
    assert np.allclose(y, g * so.sigmoid(1.702 * g) * (np.array([2.0, -2.0]) + 1))
    # router: top scores, weights are the sigmoids themselves
    idx, w = so.route(np.array([[1.0, 0.0]]), np.array([[0.5, 0], [2.0, 0], [-1.0, 0]]), 2)
    assert idx.tolist() == [[1, 0]] and np.allclose(w, so.sigmoid(np.array([[2.0, 0.5]])))
