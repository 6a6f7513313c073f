"""GPU tests of the layer-stack model class (Ditilix design): every operator of vllm_rs_amd/csrc/stack_ops.hip alone, then whole
models of small random configurations through the engine — against tests/stack_oracle.py (float64, no cache, no pages).

f32 models must agree with the oracle to f32 rounding; bf16 models to bf16 rounding; and whatever the element type, the logits of a
position must not depend on how its prompt was cut, on the rest of the batch or on the pages it got: f32 steps of the prefill form are
compared EXACTLY; decode steps (another reduction order in the attention) and bf16 steps (the row count of a step picks the matrix
kernel) to rounding.
"""
import ctypes as C
import math

import numpy as np
import pytest

from tests import stack_oracle as so
from vllm_rs_amd import _lib, checkpoint

pytestmark = pytest.mark.gpu
BF16, F32 = 0, 2


# ------------------------------------------------------------------------------------------------ helpers
_KEEP = []  # device buffers of the running test: an argument like `raw(x).ptr` must outlive the launch that reads it


@pytest.fixture(autouse=True)
def _buffers_live_until_the_test_ends():
    yield
    _lib.load().vra_device_sync()
    _KEEP.clear()


def keep(buf):
    _KEEP.append(buf)
    return buf


def to_dev(a, dt):
    """float array -> device buffer in the element type dt"""
    from vllm_rs_amd.ops import DevBuf
    a = np.ascontiguousarray(a, np.float32)
    return keep(DevBuf(array=checkpoint.f32_to_bf16_bits(a) if dt == BF16 else a))


def from_dev(buf, shape, dt):
    if dt == BF16:
        return (buf.numpy(np.uint16, shape).astype(np.uint32) << 16).view(np.float32)
    return buf.numpy(np.float32, shape)


def raw(a, dtype):
    from vllm_rs_amd.ops import DevBuf
    return keep(DevBuf(array=np.ascontiguousarray(a, dtype)))


def empty(nbytes):
    from vllm_rs_amd.ops import DevBuf
    return keep(DevBuf(nbytes=nbytes).fill_bytes(0xFF))


def check():
    from vllm_rs_amd.ops import check_error
    check_error()


def rel(got, ref):
    """rms of the difference over the rms of the reference"""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return float(np.sqrt(((got - ref) ** 2).mean()) / max(np.sqrt((ref ** 2).mean()), 1e-30))


TOL = {F32: 3e-5, BF16: 2.5e-2}


def agree(got, ref, dt, what=""):
    """a model's rows against the oracle's.  f32: every row to f32 rounding.  bf16: rounding may turn a close call of a router (a discrete
    choice, which then changes that token a lot and, through its keys and values, the tokens behind it a little), so the rows are judged
    one by one: the typical row to bf16 rounding, three in four within a few times that (the f32 runs of the same tests are the sharp ones)"""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    got, ref = got.reshape(-1, got.shape[-1]), ref.reshape(-1, ref.shape[-1])
    rows = np.sqrt(((got - ref) ** 2).mean(-1)) / np.maximum(np.sqrt((ref ** 2).mean(-1)), 1e-30)
    if dt == F32:
        assert rows.max() < 1e-4 and rel(got, ref) < TOL[F32], (what, rows.max())
    else:
        assert np.median(rows) < 1.5e-2 and np.quantile(rows, 0.75) < 5e-2, (what, float(np.median(rows)), float(np.quantile(rows, 0.75)))


def mixer(heads=6, kv_heads=3, dim=16, vdim=24, scale=0.3, softcap=8.0, q_temp=(0.25, 5), kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if softcap:
        m["softcap"] = softcap
    if q_temp:
        m["q_temp"] = dict(coef=q_temp[0], every=q_temp[1])
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(experts=5, top=2, ff=40, limit=1.5, shared=(24, 1.0)):
    m = dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, top=top))
    if shared:
        m["shared"] = dict(ff=shared[0], limit=shared[1])
    return m


def config_a():
    """other sizes than any shipped model: 3 norm groups, 2 query heads per kv head, key size != value size, top-2 routing, an expert width
    that is no multiple of 16, layers that borrow keys / values, a layer without feed-forward, a layer with as many kv heads as heads"""
    return dict(architecture="Ditilix", width=96, vocab=160, residual_mult=0.4, logit_scale=0.7, norm=dict(eps=1e-5, groups=3), layers=[
        dict(type="attention", mixer=mixer(), mlp=dict(kind="dense", ff=72)),
        dict(type="attention", mixer=mixer(), mlp=moe()),
        dict(type="attention", mixer=mixer(kv_from=1), mlp=moe(shared=None)),
        dict(type="attention", mixer=mixer(kv_from=1, softcap=0, q_temp=None), mlp=None),
        # (key size a multiple of 8, value size a multiple of 16: the bf16 model runs this layer's prompt portions on the matrix-core kernel)
        dict(type="attention", mixer=mixer(heads=4, kv_heads=4, dim=24, vdim=16, scale=0.5, softcap=4.0, q_temp=(0.5, 64)), mlp=dict(kind="dense", ff=16)),
    ])


def config_b():
    """sizes that leave the 16-byte fast paths: width 50, key size 5, value size 7, one norm group, one kv head, top-1 of 3 experts"""
    return dict(architecture="Ditilix", width=50, vocab=70, residual_mult=1.0, logit_scale=1.0, norm=dict(eps=1e-6, groups=1), layers=[
        dict(type="attention", mixer=mixer(heads=2, kv_heads=1, dim=5, vdim=7, scale=0.6, softcap=3.0, q_temp=(0.3, 3)), mlp=moe(experts=3, top=1, ff=9, limit=0.8, shared=(5, 0.5))),
        dict(type="attention", mixer=mixer(heads=2, kv_heads=1, dim=5, vdim=7, scale=0.6, softcap=0, q_temp=None, kv_from=0), mlp=dict(kind="dense", ff=11)),
    ])


def build(cfg_json, tensors, dt, blocks=24, max_model_len=1024, **kw):
    from vllm_rs_amd.engine import Engine
    cfg = checkpoint.parse_config(cfg_json, "float32" if dt == F32 else None)
    eng = Engine(cfg, num_gpu_blocks=blocks, max_num_seqs=4, max_model_len=max_model_len, **dict(dict(use_graph=False), **kw))
    bits = {n: checkpoint.to_engine_tensor(n, checkpoint.f32_to_bf16_bits(a), "bf16", cfg["dtype"]) for n, a in tensors.items()}
    return eng.load_weights(bits)


def tokens_of(cfg_json, n, seed):
    return np.random.default_rng(seed).integers(0, cfg_json["vocab"], n).tolist()


# ------------------------------------------------------------------------------------------------ operators alone
@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("W", [96, 51])
def test_embed_sinusoidal_positions(dt, W):
    L = _lib.load()
    r = np.random.default_rng(1)
    V, T = 40, 9
    emb = so.bf16_round(r.standard_normal((V, W)).astype(np.float32))
    ids = r.integers(0, V, T).astype(np.uint32)
    pos = np.array([0, 1, 2, 63, 64, 65, 700, 4095, 3], np.int64)
    inv = (10000.0 ** (-2.0 * np.arange((W + 1) // 2) / W)).astype(np.float32)
    x = empty(T * W * 4)
    L.vra_stack_op_embed_sinpos(raw(ids, np.uint32).ptr, raw(pos, np.int64).ptr, to_dev(emb, dt).ptr, raw(inv, np.float32).ptr, x.ptr, T, W, V, dt, 0)
    check()
    ref = emb[ids] + np.stack([so.position_vector(int(p) + 1, W)[int(p)] for p in pos])
    assert np.abs(x.numpy(np.float32, (T, W)) - ref).max() < 2e-4  # (f32 angle p * f at p = 4095: half an ulp of 4095 in the sine)


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("W,groups", [(96, 3), (96, 1), (50, 5), (1024, 2)])
def test_group_norm(dt, W, groups):
    L = _lib.load()
    r = np.random.default_rng(2)
    T = 7
    x = (r.standard_normal((T, W)) * np.linspace(0.1, 30, W)).astype(np.float32)  # parts of very different size: a norm over the wrong part shows
    w = (1 + 0.3 * r.standard_normal(W)).astype(np.float32)
    h = empty(T * W * 4)
    L.vra_stack_op_group_norm(raw(x, np.float32).ptr, raw(w, np.float32).ptr, h.ptr, T, W, groups, 1e-5, None, 0, 0, 0, None, None, None, dt, 0)
    check()
    assert rel(from_dev(h, (T, W), dt), so.group_norm(x.astype(np.float64), w, groups, 1e-5)) < (1e-6 if dt == F32 else 4e-3)


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("top,gate_row", [(1, 1), (2, 0), (3, 1)])
def test_router_in_the_norm_launch(dt, top, gate_row):
    L = _lib.load()
    r = np.random.default_rng(3)
    T, W, E = 33, 64, 7
    x = r.standard_normal((T, W)).astype(np.float32)
    w = np.ones(W, np.float32)
    rw = so.bf16_round((3 * r.standard_normal((E + gate_row, W)) / 8).astype(np.float32))
    h, pe, pw, gt = empty(T * W * 4), empty(T * top * 4), empty(T * top * 4), empty(T * 4)
    L.vra_stack_op_group_norm(raw(x, np.float32).ptr, raw(w, np.float32).ptr, h.ptr, T, W, 2, 1e-6, to_dev(rw, dt).ptr, E, top, gate_row, pe.ptr, pw.ptr,
                              gt.ptr, dt, 0)
    check()
    hn = so.group_norm(x.astype(np.float64), w, 2, 1e-6)
    idx, wts = so.route(hn, rw[:E].astype(np.float64), top)
    got_e, got_w = pe.numpy(np.int32, (T, top)), pw.numpy(np.float32, (T, top))
    assert (got_e == idx).all()  # (weights are random: no near ties)
    assert np.abs(got_w - wts).max() < 1e-5
    if gate_row:
        assert np.abs(gt.numpy(np.float32, (T,)) - so.sigmoid(hn @ rw[E].astype(np.float64))).max() < 1e-5


GEMM_SHAPES = [(1, 64, 96), (5, 200, 96), (16, 48, 144), (33, 130, 96), (100, 72, 256), (300, 160, 96), (7, 33, 50), (70, 19, 27)]


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_plain(dt, M, N, K):
    L = _lib.load()
    r = np.random.default_rng(M * 7 + N)
    a = so.bf16_round(r.standard_normal((M, K)).astype(np.float32))
    w = so.bf16_round(r.standard_normal((N, K)).astype(np.float32))
    out = empty(M * N * 4)
    L.vra_stack_op_gemm(to_dev(a, dt).ptr, K, to_dev(w, dt).ptr, 0, out.ptr, N, 1, M, N, K, 0.5, None, 0, None, None, None, 0, 0.0, dt, 0)
    check()
    assert rel(out.numpy(np.float32, (M, N)), 0.5 * (a.astype(np.float64) @ w.astype(np.float64).T)) < 2e-6
    # a row's result does not depend on the number of rows around it (the kernels pick tiles by M)
    if M > 33:
        out2 = empty(3 * N * 4)
        L.vra_stack_op_gemm(to_dev(a[:3], dt).ptr, K, to_dev(w, dt).ptr, 0, out2.ptr, N, 1, 3, N, K, 0.5, None, 0, None, None, None, 0, 0.0, dt, 0)
        check()
        if dt == F32:
            assert (out2.numpy(np.float32, (3, N)) == out.numpy(np.float32, (M, N))[:3]).all()
        else:  # (bf16: few rows split K over the waves of a workgroup, many rows run one chain: the same sum in another order)
            assert rel(out2.numpy(np.float32, (3, N)), out.numpy(np.float32, (M, N))[:3]) < 2e-6


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("granule,P,E,top", [(16, 37, 5, 2), (64, 900, 3, 1), (16, 4, 6, 1)])
def test_moe_sort_and_grouped_gemm(dt, granule, P, E, top):
    """pairs sorted by expert into padded granules; gather + weight on the way in, scatter on the way out; gated pair both fused and apart"""
    L = _lib.load()
    r = np.random.default_rng(P)
    W, F = 96, 40
    Fp = (F + 15) // 16 * 16
    T = P // top
    P = T * top
    pe = r.integers(0, E, P).astype(np.int32)
    pw = r.uniform(0.2, 1.0, P).astype(np.float32)
    rows = (P + E * (granule - 1) + granule - 1) // granule * granule
    rt, rs, rp, tg = empty(rows * 4), empty(rows * 4), empty(rows * 4), empty(rows // granule * 4)
    L.vra_stack_op_moe_sort(raw(pe, np.int32).ptr, raw(pw, np.float32).ptr, P, top, E, granule, rows, rt.ptr, rs.ptr, rp.ptr, tg.ptr, 0)
    check()
    row_pair, row_token, tile = rp.numpy(np.int32, (rows,)), rt.numpy(np.int32, (rows,)), tg.numpy(np.int32, (rows // granule,))
    assert sorted(row_pair[row_pair >= 0].tolist()) == list(range(P))
    for i, p in enumerate(row_pair):
        if p >= 0:
            assert tile[i // granule] == pe[p] and row_token[i] == p // top
    h = so.bf16_round(r.standard_normal((T, W)).astype(np.float32))
    gate = so.bf16_round((r.standard_normal((E, F, W)) / 5).astype(np.float32))
    up = so.bf16_round((r.standard_normal((E, F, W)) / 5).astype(np.float32))
    gu = np.zeros((E, 2 * Fp, W), np.float32)
    for f in range(F):
        gu[:, (2 * (f // 16)) * 16 + f % 16], gu[:, (2 * (f // 16) + 1) * 16 + f % 16] = gate[:, f], up[:, f]
    hd, gud = to_dev(h, dt), to_dev(gu, dt)
    ref = np.zeros((P, F))
    for p in range(P):
        hin = pw[p].astype(np.float64) * h[p // top].astype(np.float64)
        hin = so.bf16_round(hin.astype(np.float32)).astype(np.float64) if dt == BF16 else hin
        g, u = np.minimum(gate[pe[p]] @ hin, 1.5), np.clip(up[pe[p]] @ hin, -1.5, 1.5)
        ref[p] = g * so.sigmoid(1.702 * g) * (u + 1)
    # apart: product into f32, then the activation
    z, y = empty(rows * 2 * Fp * 4), empty(rows * Fp * 4)
    L.vra_stack_op_gemm(hd.ptr, W, gud.ptr, 2 * Fp * W, z.ptr, 2 * Fp, 1, rows, 2 * Fp, W, 1.0, tg.ptr, granule, rt.ptr, rs.ptr, None, 0, 0.0, dt, 0)
    L.vra_stack_op_gated_act(z.ptr, y.ptr, rows, F, 1.5, 1.702, dt, 0)
    check()
    got = from_dev(y, (rows, Fp), dt)
    sel = row_pair >= 0
    assert rel(got[sel][:, :F], ref[row_pair[sel]]) < (1e-5 if dt == F32 else 6e-3)
    assert (got[sel][:, F:] == 0).all()
    if dt == BF16:  # fused: the activation as the product's epilogue gives the same numbers
        y2 = empty(rows * Fp * 2)
        L.vra_stack_op_gemm(hd.ptr, W, gud.ptr, 2 * Fp * W, y2.ptr, Fp, 0, rows, 2 * Fp, W, 1.0, tg.ptr, granule, rt.ptr, rs.ptr, None, 1, 1.5, dt, 0)
        check()
        assert (from_dev(y2, (rows, Fp), dt)[sel] == got[sel]).all()
    # the way out: rows of the padded space land on their pair's row
    down = so.bf16_round((r.standard_normal((E, W, Fp)) / 6).astype(np.float32))
    o = empty(P * W * 4)
    L.vra_stack_op_gemm(y.ptr, Fp, to_dev(down, dt).ptr, W * Fp, o.ptr, W, 1, rows, W, Fp, 1.0, tg.ptr, granule, None, None, rp.ptr, 0, 0.0, dt, 0)
    check()
    want = np.stack([down[pe[p]].astype(np.float64) @ got[np.nonzero(row_pair == p)[0][0]].astype(np.float64) for p in range(P)])
    assert rel(o.numpy(np.float32, (P, W)), want) < 1e-5


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("F", [72, 11, 1000])
def test_polynorm(dt, F):
    L = _lib.load()
    r = np.random.default_rng(F)
    M = 5
    z = (2 * r.standard_normal((M, F))).astype(np.float32)
    coef = np.array([0.7, -0.4, 0.2, 0.05], np.float32)
    out = empty(M * F * 4)
    L.vra_stack_op_polynorm(raw(z, np.float32).ptr, out.ptr, raw(coef, np.float32).ptr, M, F, 1e-5, dt, 0)
    check()
    assert rel(from_dev(out, (M, F), dt), so.polynorm(z.astype(np.float64), coef, 1e-5)) < (2e-6 if dt == F32 else 4e-3)


def test_residual_combine():
    L = _lib.load()
    r = np.random.default_rng(5)
    T, W, n1 = 9, 50, 3
    x, o, p1, p2, g = [r.standard_normal(s).astype(np.float32) for s in ((T, W), (T, W), (T * n1, W), (T, W), (T,))]
    xd = raw(x, np.float32)
    L.vra_stack_op_residual_combine(xd.ptr, raw(o, np.float32).ptr, raw(p1, np.float32).ptr, n1, raw(p2, np.float32).ptr, raw(g, np.float32).ptr, 0.3, T, W, 0)
    check()
    ref = x + 0.3 * (o + p1.reshape(T, n1, W).sum(1) + g[:, None] * p2)
    assert np.abs(xd.numpy(np.float32, (T, W)) - ref).max() < 1e-5


def paged(k, v, BS, r, dt, extra_blocks=3):
    """k / v of ONE sequence [Tk, G, *] -> caches over shuffled pages (+ block table), unused slots poisoned"""
    Tk, G, dim = k.shape
    vdim = v.shape[2]
    nb = (Tk + BS - 1) // BS
    total = nb + extra_blocks
    table = r.permutation(total)[:nb].astype(np.uint32)
    kc = np.full((total * BS, G * dim), 1e4, np.float32)
    vc = np.full((total * BS, G * vdim), -1e4, np.float32)
    for j in range(Tk):
        s = int(table[j // BS]) * BS + j % BS
        kc[s], vc[s] = k[j].reshape(-1), v[j].reshape(-1)
    return to_dev(kc, dt), to_dev(vc, dt), table


def run_attention(L, q, positions, k, v, mx, dt, decode, r, BS=64):
    """one sequence: queries q [Tq, H, dim] at `positions`, all keys / values of positions 0..Tk-1 in the cache"""
    Tq, H, dim = q.shape
    G, vdim = v.shape[1], v.shape[2]
    kc, vc, table = paged(k, v, BS, r, dt)
    out = empty(Tq * H * vdim * 4)
    qt = mx.get("q_temp") or {}
    qd = to_dev(q.reshape(Tq, H * dim), dt)
    if decode:
        res = []
        for i in range(Tq):  # one launch per token: the decode form takes one token per sequence
            o1 = empty(H * vdim * 4)
            qi = to_dev(q[i].reshape(1, H * dim), dt)
            L.vra_stack_op_attention(qi.ptr, H * dim, o1.ptr, kc.ptr, vc.ptr, raw([positions[i]], np.int64).ptr, raw(table, np.uint32).ptr,
                                     raw([positions[i] + 1], np.uint32).ptr, None, 1, 1, 1, H, G, dim, vdim, BS, len(table), mx["scale"],
                                     mx.get("softcap", 0.0), qt.get("coef", 0.0), qt.get("every", 0), dt, 0)
            check()
            res.append(from_dev(o1, (H, vdim), dt))
        return np.stack(res)
    L.vra_stack_op_attention(qd.ptr, H * dim, out.ptr, kc.ptr, vc.ptr, raw(positions, np.int64).ptr, raw(table, np.uint32).ptr,
                             raw([k.shape[0]], np.uint32).ptr, raw([0, Tq], np.uint32).ptr, 1, Tq, Tq, H, G, dim, vdim, BS, len(table), mx["scale"],
                             mx.get("softcap", 0.0), qt.get("coef", 0.0), qt.get("every", 0), dt, 0)
    check()
    return from_dev(out, (Tq, H, vdim), dt)


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("H,G,dim,vdim", [(6, 3, 16, 24), (4, 4, 8, 8), (2, 1, 5, 7), (8, 2, 128, 128), (3, 1, 40, 200), (6, 2, 32, 48), (4, 2, 64, 16),
                                          (2, 1, 160, 144), (5, 5, 72, 80)])
def test_attention_random(dt, decode, H, G, dim, vdim):
    L = _lib.load()
    r = np.random.default_rng(H * 100 + dim)
    Tk = 150
    mx = dict(scale=1.3 / math.sqrt(dim), softcap=6.0, q_temp=dict(coef=0.4, every=7))
    k = so.bf16_round(r.standard_normal((Tk, G, dim)).astype(np.float32))
    v = so.bf16_round(r.standard_normal((Tk, G, vdim)).astype(np.float32))
    positions = np.array([0, 1, 5, 6, 7, 62, 63, 64, 65, 127, 128, 149] if decode else list(range(110, 150)), np.int64)
    q = so.bf16_round(r.standard_normal((len(positions), H, dim)).astype(np.float32))
    got = run_attention(L, q, positions, k, v, mx, dt, decode, r)
    ref = so.attention_core(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), mx, positions)
    assert rel(got, ref) < (2e-6 if dt == F32 else 4e-3)


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("softcap,temp", [(0.0, None), (20.0, dict(coef=0.3, every=64))])
def test_attention_planted_key(dt, decode, softcap, temp):
    """One key is made to stand out among 900 (its value is a marker): wherever it lies — first token, around page borders, far back, the
    query's own position — a query that may see it returns the marker; one position before it, the query must not feel it at all (the
    key is already in the cache, as in a prompt's portion)."""
    L = _lib.load()
    r = np.random.default_rng(11)
    Tk, H, G = 900, 4, 2
    dim, vdim = (32, 16) if temp else (16, 8)  # (the first pair runs the bf16 prompt form on the matrix-core kernel, the second on FMA)
    mx = dict(scale=0.25, softcap=softcap)
    if temp:
        mx["q_temp"] = temp
    base_k = so.bf16_round((0.1 * r.standard_normal((Tk, G, dim))).astype(np.float32))
    base_v = so.bf16_round((0.1 * r.standard_normal((Tk, G, vdim))).astype(np.float32))
    u = np.zeros(dim, np.float32)
    u[3] = 1.0
    for j in (0, 1, 63, 64, 65, 127, 128, 300, 766, 898):
        k, v = base_k.copy(), base_v.copy()
        k[j, :, :] = 16.0 * u  # score = 8 * 16 * 0.25 = 32 against |scores| < 1 elsewhere: weight 1 - 900 e^-31 (or, soft-capped at 20, 1 - 900 e^-17)
        v[j, :, :] = 5.0
        positions = np.array(sorted({max(j - 1, 0), j, j + 1, 899}), np.int64)
        q = np.tile(8.0 * u, (len(positions), H, 1)).astype(np.float32)
        got = run_attention(L, q, positions, k, v, mx, dt, decode, r)
        ref = so.attention_core(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), mx, positions)
        assert np.abs(got - ref).max() < (1e-4 if dt == F32 else 3e-2), (j, np.abs(got - ref).max())
        for i, p in enumerate(positions):
            if p >= j:
                assert np.abs(got[i] - 5.0).max() < 0.05, (j, p)
            else:
                assert np.abs(got[i]).max() < 0.6, (j, p)  # (the other values are 0.1 N(0, 1); the marker is 5)


# ------------------------------------------------------------------------------------------------ whole models through the engine
@pytest.fixture(scope="module", params=[("a", F32), ("a", BF16), ("b", F32), ("b", BF16)], ids=["a-f32", "a-bf16", "b-f32", "b-bf16"])
def model(request):
    name, dt = request.param
    cfg = config_a() if name == "a" else config_b()
    tensors = so.random_tensors(cfg, 7 if name == "a" else 8)
    eng = build(cfg, tensors, dt, blocks=12, max_model_len=512)
    yield cfg, tensors, dt, eng
    eng.close()


def test_layers_one_by_one(model):
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 23, 1)
    eng.layer_trace(True)
    got = eng.replay_step([(1, toks, list(range(len(toks))))], [1])
    trace = eng.read_layer_trace(len(toks))
    eng.layer_trace(False)
    layers = []
    ref = so.forward(cfg, tensors, toks, layers)
    for i, x in enumerate(layers):
        agree(trace[i], x, dt, f"layer {i}")
    agree(got, ref, dt)


def test_prefill_against_token_by_token_decoding(model):
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 150, 2)  # crosses two page borders and many temperature steps
    ref = so.forward(cfg, tensors, toks)
    whole = eng.replay_step([(1, toks, list(range(len(toks))))], [1])
    agree(whole, ref, dt, "whole")
    rows = [eng.replay_step([(2, toks[:1], [0])], [])[0]]
    for p in range(1, len(toks)):
        rows.append(eng.replay_step([(2, toks[p:p + 1], [0])], [2] if p == len(toks) - 1 else [])[0])
    one = np.stack(rows)
    agree(one, ref, dt, "token by token")
    if dt == F32:
        assert rel(one, whole) < 1e-5
    else:
        agree(one, whole, dt, "token by token against whole")


@pytest.mark.parametrize("sizes", [[2] * 30, [37, 3, 37, 2, 5], [64, 64, 2], [63, 2, 63, 2], [1, 5, 1, 1, 70, 1]])
def test_portions(model, sizes):
    """a prompt cut anywhere (down to two tokens, at and across page borders) gives the logits of the whole prompt — exactly, where the
    portions run in the prefill form"""
    cfg, tensors, dt, eng = model
    n = sum(sizes)
    toks = tokens_of(cfg, n, 3)
    whole = eng.replay_step([(1, toks, list(range(n)))], [1])
    got, at = [], 0
    for i, c in enumerate(sizes):
        got.append(eng.replay_step([(2, toks[at:at + c], list(range(c)))], [2] if i == len(sizes) - 1 else []))
        at += c
    got = np.concatenate(got)
    at, exact = 0, True
    for c in sizes:
        # a single token behind a cached context runs the decode kernels: another order of the same sums, for that token and (through
        # the keys and values it leaves in the deeper layers' caches) for the tokens behind it
        exact = exact and (c > 1 or at == 0) and dt == F32  # (bf16: steps of up to 32 rows sum their matrix products in another order)
        if exact:
            assert (got[at:at + c] == whole[at:at + c]).all(), f"portion at {at} of {c} tokens differs from the whole prompt"
        else:
            assert rel(got[at:at + c], whole[at:at + c]) < (1e-5 if dt == F32 else 1.5e-2)
        at += c


def test_unequal_batch_against_each_alone(model):
    cfg, tensors, dt, eng = model
    lens = [70, 3, 129, 1]
    prompts = [tokens_of(cfg, n, 10 + i) for i, n in enumerate(lens)]
    alone = [eng.replay_step([(1, p, list(range(len(p))))], [1]) for p in prompts]
    # all four in one batch; then the same with every prompt cut in two and the second parts beside each other
    batch = eng.replay_step([(10 + i, p, list(range(len(p)))) for i, p in enumerate(prompts)], [10, 11, 12, 13])
    same = (lambda x, y: (x == y).all()) if dt == F32 else (lambda x, y: rel(x, y) < 1.5e-2)  # (bf16: the row count of a step picks the kernel)
    at = 0
    for i, p in enumerate(prompts):
        assert same(batch[at:at + len(p)], alone[i]), f"request {i} depends on its batch"
        at += len(p)
    cut = [n // 2 for n in lens]
    first = eng.replay_step([(20 + i, p[:c], list(range(c))) for i, (p, c) in enumerate(zip(prompts, cut)) if c], [])
    second = eng.replay_step([(20 + i, p[c:], list(range(len(p) - c))) for i, (p, c) in enumerate(zip(prompts, cut))], [20, 21, 22, 23])
    a1 = a2 = 0
    for i, (p, c) in enumerate(zip(prompts, cut)):
        got = np.concatenate([first[a1:a1 + c], second[a2:a2 + len(p) - c]])
        a1, a2 = a1 + c, a2 + len(p) - c
        if len(p) - c > 1 or c == 0:
            assert same(got, alone[i]), f"request {i} depends on its cut or its batch"
        else:
            assert rel(got, alone[i]) < (1e-5 if dt == F32 else 1.5e-2)


def test_mixed_steps_and_reused_pages(model):
    """12 pages for requests that come and go: decoded tokens beside portions of prompts, pages handed back and taken again in another
    order; every logit row equals the request's own run"""
    cfg, tensors, dt, eng = model
    r = np.random.default_rng(4)
    lens = [130, 60, 200, 90, 33, 150, 64, 128]
    prompts = [tokens_of(cfg, n, 40 + i) for i, n in enumerate(lens)]
    ref = [so.forward(cfg, tensors, p) for p in prompts]
    waiting, live, nxt = list(range(len(prompts))), {}, 100
    got_rows, ref_rows = [], []
    while waiting or live:
        while waiting and len(live) < 4 and sum((lens[i] + 63) // 64 for i in list(live) + [waiting[0]]) <= 12:
            live[waiting.pop(0)] = 0
        entries, ends, spans = [], [], []
        for i, at in live.items():
            left = lens[i] - at
            c = 1 if (at > 0 and r.random() < 0.5) else int(min(left, r.choice([2, 3, 17, 64, 100])))
            entries.append((1000 + i, prompts[i][at:at + c], list(range(c))))
            spans.append((i, at, c))
            if at + c == lens[i]:
                ends.append(1000 + i)
        out = eng.replay_step(entries, ends)
        o = 0
        for i, at, c in spans:
            got_rows.append(out[o:o + c]), ref_rows.append(ref[i][at:at + c])
            o += c
            live[i] = at + c
            if live[i] == lens[i]:
                del live[i]
    agree(np.concatenate(got_rows), np.concatenate(ref_rows), dt)


def test_long_decoding(model):
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 330, 5)
    ref = so.forward(cfg, tensors, toks)
    eng.replay_step([(1, toks[:20], [])], [])
    rows = [eng.replay_step([(1, toks[p:p + 1], [0])], [1] if p == len(toks) - 1 else [])[0] for p in range(20, len(toks))]
    agree(np.stack(rows), ref[20:], dt)


@pytest.mark.parametrize("use_graph", [False, True])
def test_greedy_generation_through_the_scheduler(use_graph):
    """Engine.generate: the engine's own scheduler, block manager, prefill and decode steps (captured decode graphs when asked) and its
    argmax — against the oracle's greedy continuation, f32 so that near ties do not decide"""
    cfg = config_a()
    tensors = so.random_tensors(cfg, 9)
    eng = build(cfg, tensors, F32, blocks=16, max_model_len=256, use_graph=use_graph)
    prompts = [tokens_of(cfg, n, 60 + n) for n in (5, 70, 31)]
    outs = eng.generate(prompts, max_tokens=12, ignore_eos=True)
    eng.close()
    for p, out in zip(prompts, outs):
        seq = list(p)
        for t in out:
            lg = so.forward(cfg, tensors, seq)[-1]
            top2 = np.sort(lg)[-2:]
            assert int(t) == int(lg.argmax()) or top2[1] - top2[0] < 1e-3, (len(p), len(seq))
            seq.append(int(t))
        assert len(out) == 12


def test_synthetic_weights_and_cache_plan():
    """random weights of a configured shape load, the cache plan follows the layers that own a cache, a generation runs"""
    from vllm_rs_amd.engine import Engine
    cfg = checkpoint.parse_config(config_a())
    eng = Engine(cfg, max_num_seqs=4, max_model_len=256, kv_fraction=0.01, use_graph=False).init_synthetic()
    assert eng.num_gpu_blocks > 16
    out = eng.generate([list(range(1, 40))], max_tokens=5, ignore_eos=True)[0]
    assert len(out) == 5
    eng.close()
