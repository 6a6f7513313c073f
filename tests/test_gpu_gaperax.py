"""GPU tests of the Gaperax design in the layer-stack model class: the operators it adds (vllm_rs_amd/csrc/stack_mixers.hip and the new
options of stack_ops.hip) one by one, then whole models of small random configurations through the engine — against
tests/gaperax_oracle.py (float64, no cache, no pages, no absorbed projections).

f32 models must agree with the oracle to f32 rounding; bf16 models to bf16 rounding; and the logits of a position must not depend on how
its prompt was cut, on the rest of the batch or on the pages it got: f32 steps of the prefill form are compared EXACTLY; decode steps
(another kernel form) and bf16 steps (the row count of a step picks the matrix kernel) to rounding.
"""
import math

import numpy as np
import pytest

from tests import gaperax_oracle as go
from tests.test_gpu_stack import _KEEP, BF16, F32, TOL, build, check, empty, from_dev, paged, raw, rel, to_dev, tokens_of
from vllm_rs_amd import _lib, checkpoint

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _buffers_live_until_the_test_ends():
    yield
    _lib.load().vra_device_sync()
    _KEEP.clear()


def f32(a):
    return raw(a, np.float32)


def agree(got, ref, dt, what=""):
    """a model's rows against the oracle's.  f32: every row to f32 rounding.  bf16: to what the rounding of the activations causes in
    these random models — rounding them to bfloat16 inside the float64 oracle itself (norm outputs, values, mixer and feed-forward
    activations) moves the typical logit row by 3.4 % and three rows in four by less than 4.5 %; the f32 runs of the same tests are the
    sharp ones."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    got, ref = got.reshape(-1, got.shape[-1]), ref.reshape(-1, ref.shape[-1])
    rows = np.sqrt(((got - ref) ** 2).mean(-1)) / np.maximum(np.sqrt((ref ** 2).mean(-1)), 1e-30)
    if dt == F32:
        assert rows.max() < 1e-4 and rel(got, ref) < TOL[F32], (what, rows.max())
    else:
        assert np.median(rows) < 5e-2 and np.quantile(rows, 0.75) < 8e-2, (what, float(np.median(rows)), float(np.quantile(rows, 0.75)))


def rnd(r, shape, sd=1.0):
    return go.bf16_round((sd * r.standard_normal(shape)).astype(np.float32))


def freq_pair(rot):
    """the rotary frequencies of `rot` as f32 hi + lo pairs and the factor on cos / sin, as the operators take them; formed here from the
    definition and checked against the oracle's table at position 1"""
    dims, base = rot["dims"], rot["base"]
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        def td(t):
            return dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))
        lo, hi = max(math.floor(td(sc["fast"])), 0), min(math.ceil(td(sc["slow"])), dims - 1)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0, 1)
        f = f / sc["factor"] * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(sc["factor"]) + 1.0
    cos, sin = go.rotary_table(rot, [1])
    assert np.allclose(np.cos(f) * mag, cos[0]) and np.allclose(np.sin(f) * mag, sin[0])
    fh = f.astype(np.float32)
    return fh, (f - fh.astype(np.float64)).astype(np.float32), mag


# ------------------------------------------------------------------------------------------------ operators alone
@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("W,with_add", [(96, True), (51, False)])
def test_dynamic_tanh_with_residual_sum(dt, W, with_add):
    L = _lib.load()
    r = np.random.default_rng(1)
    T = 9
    x, add = (3 * r.standard_normal((T, W))).astype(np.float32), r.standard_normal((T, W)).astype(np.float32)
    w, b = (1 + 0.3 * r.standard_normal(W)).astype(np.float32), (0.2 * r.standard_normal(W)).astype(np.float32)
    xd, h = f32(x), empty(T * W * 4)
    L.vra_stack_op_dyt(xd.ptr, f32(add).ptr if with_add else None, f32(w).ptr, f32(b).ptr, 0.37, h.ptr, T, W, dt, 0)
    check()
    xs = x + add if with_add else x
    assert (xd.numpy(np.float32, (T, W)) == xs).all()
    assert rel(from_dev(h, (T, W), dt), go.dyt(xs.astype(np.float64), w, b, np.float32(0.37))) < (1e-6 if dt == F32 else 4e-3)


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("M", [3, 70, 300])
def test_gemm_bias_and_heads_as_a_batch(dt, M):
    L = _lib.load()
    r = np.random.default_rng(M)
    # bias in the epilogue
    K, N = 96, 72
    a, w, bias = rnd(r, (M, K)), rnd(r, (N, K)), r.standard_normal(N).astype(np.float32)
    out = empty(M * N * 4)
    L.vra_stack_op_gemm_ex(to_dev(a, dt).ptr, K, to_dev(w, dt).ptr, out.ptr, N, 1, M, N, K, 1.0, f32(bias).ptr, 0, 0, 1, 0, 0, 0, dt, 0)
    check()
    assert rel(out.numpy(np.float32, (M, N)), a.astype(np.float64) @ w.astype(np.float64).T + bias) < 2e-6
    # one product per head in one launch: head z reads columns z * hs .. of the rows, its own weights, and writes its own columns
    for H, hs, kd, n, os_ in [(3, 24, 16, 40, 48), (5, 7, 5, 9, 11)]:  # (the second: nothing a multiple of 8)
        a, w = rnd(r, (M, H * hs)), rnd(r, (H, n, kd))
        out = empty(M * H * os_ * 4).fill_bytes(0)
        L.vra_stack_op_gemm_ex(to_dev(a, dt).ptr, H * hs, to_dev(w, dt).ptr, out.ptr, H * os_, 1, M, n, kd, 1.0, None, 0, 0, H, hs, n * kd, os_, dt, 0)
        check()
        got = out.numpy(np.float32, (M, H, os_))
        for z in range(H):
            assert rel(got[:, z, :n], a.reshape(M, H, hs)[:, z, :kd].astype(np.float64) @ w[z].astype(np.float64).T) < 2e-6
            assert (got[:, z, n:] == 0).all()


@pytest.mark.parametrize("dt", [F32, BF16])
def test_gated_gelu_feed_forward_pair(dt):
    """gate / up rows interleaved in blocks of 16: gelu_tanh(gate) * up, as the product's epilogue (bf16) and as a launch of its own"""
    L = _lib.load()
    r = np.random.default_rng(7)
    M, W, F = 37, 96, 40
    Fp = 48
    h, gate, up = rnd(r, (M, W)), rnd(r, (F, W), 0.2), rnd(r, (F, W), 0.2)
    gu = np.zeros((2 * Fp, W), np.float32)
    for f in range(F):
        gu[(2 * (f // 16)) * 16 + f % 16], gu[(2 * (f // 16) + 1) * 16 + f % 16] = gate[f], up[f]
    ref = go.gelu_tanh(h.astype(np.float64) @ gate.T.astype(np.float64)) * (h.astype(np.float64) @ up.T.astype(np.float64))
    z, y = empty(M * 2 * Fp * 4), empty(M * Fp * 4)
    L.vra_stack_op_gemm_ex(to_dev(h, dt).ptr, W, to_dev(gu, dt).ptr, z.ptr, 2 * Fp, 1, M, 2 * Fp, W, 1.0, None, 0, 0, 1, 0, 0, 0, dt, 0)
    check()
    zz = z.numpy(np.float32, (M, 2 * Fp)).reshape(M, Fp // 16, 2, 16)
    got = go.gelu_tanh(zz[:, :, 0].astype(np.float64)) * zz[:, :, 1]
    assert rel(got.reshape(M, Fp)[:, :F], ref) < 1e-5
    if dt == BF16:
        L.vra_stack_op_gemm_ex(to_dev(h, dt).ptr, W, to_dev(gu, dt).ptr, y.ptr, Fp, 0, M, 2 * Fp, W, 1.0, None, 1, 1, 1, 0, 0, 0, dt, 0)
        check()
        assert rel(from_dev(y, (M, Fp), dt)[:, :F], ref) < 6e-3


ROTS = [dict(base=1e4, dims=8), dict(base=5e5, dims=12, scaling=dict(factor=6.0, original=128, fast=24.0, slow=1.5)), dict(base=10.0, dims=2)]


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("rot", ROTS, ids=["plain", "scaled", "one-pair"])
def test_latent_rows_norms_rotary_cache(dt, rot):
    """the two latent norms, the rotated key part at the token's position (far positions included: the angle must not lose the
    frequency's low bits), the cache row [latent | rotated part] at the token's slot; a slot < 0 writes nothing"""
    L = _lib.load()
    r = np.random.default_rng(3)
    qr, kr, rd = 20, 13, rot["dims"] + 2  # (two dimensions behind the rotated ones pass unchanged)
    pos = np.array([0, 1, 63, 64, 700, 4095, 100000, 5], np.int64)
    T = len(pos)
    slots = np.array([5, 0, 17, 3, 9, 11, 2, -1], np.int64)
    raw_rows = r.standard_normal((T, qr + kr + rd)).astype(np.float32) * 3
    qn, kn = (1 + 0.2 * r.standard_normal(qr)).astype(np.float32), (1 + 0.2 * r.standard_normal(kr)).astype(np.float32)
    fh, fl, mag = freq_pair(rot)
    cq, cache = empty(T * qr * 4), empty(20 * (kr + rd) * 4)
    L.vra_stack_op_latent_prep(f32(raw_rows).ptr, qr + kr + rd, qr, kr, rd, f32(qn).ptr, f32(kn).ptr, 1e-5, cq.ptr, cache.ptr, kr + rd, raw(slots, np.int64).ptr,
                               raw(pos, np.int64).ptr, f32(fh).ptr, f32(fl).ptr, rot["dims"] // 2, mag, T, dt, 0)
    check()
    x = raw_rows.astype(np.float64)
    tol = 2e-6 if dt == F32 else 4e-3
    assert rel(from_dev(cq, (T, qr), dt), go.rms_norm(x[:, :qr], qn, 1e-5)) < tol
    rows = from_dev(cache, (20, kr + rd), dt)
    cos, sin = go.rotary_table(rot, pos)
    want = np.concatenate([go.rms_norm(x[:, qr:qr + kr], kn, 1e-5), go.rotate_pairs(x[:, qr + kr:], cos, sin)], 1)
    for t in range(T):
        if slots[t] >= 0:
            assert np.abs(rows[slots[t]] - want[t]).max() < (3e-5 if dt == F32 else 6e-2), (t, np.abs(rows[slots[t]] - want[t]).max())
    untouched = [s for s in range(20) if s not in slots.tolist()]
    assert np.isnan(rows[untouched]).all() or (np.abs(rows[untouched]) > 1e30).all()  # (the buffer was filled with 0xFF bytes)


@pytest.mark.parametrize("dt", [F32, BF16])
def test_rotary_on_head_rows(dt):
    L = _lib.load()
    r = np.random.default_rng(4)
    rot = ROTS[1]
    H, hs_in, off_in, hs_out, off_out, n = 3, 20, 6, 30, 16, 14
    pos = np.array([0, 3, 64, 999, 70000], np.int64)
    T = len(pos)
    x = rnd(r, (T, H, hs_in))
    out = empty(T * H * hs_out * 4).fill_bytes(0)
    fh, fl, mag = freq_pair(rot)
    L.vra_stack_op_rope_heads(to_dev(x.reshape(T, -1), dt).ptr, H * hs_in, hs_in, off_in, out.ptr, H * hs_out, hs_out, off_out, n, H, raw(pos, np.int64).ptr,
                              f32(fh).ptr, f32(fl).ptr, rot["dims"] // 2, mag, T, dt, 0)
    check()
    got = from_dev(out, (T, H, hs_out), dt)
    want = go.rotate_pairs(x[:, :, off_in:off_in + n].astype(np.float64), *go.rotary_table(rot, pos))
    assert np.abs(got[:, :, off_out:off_out + n] - want).max() < (2e-5 if dt == F32 else 4e-2)
    assert (got[:, :, :off_out] == 0).all()


@pytest.mark.parametrize("dt", [F32, BF16])
def test_whole_projection_norms_and_cache_rows(dt):
    L = _lib.load()
    r = np.random.default_rng(5)
    nq, nk, nv, ng, T = 36, 18, 21, 10, 6
    x = (r.standard_normal((T, nq + nk + nv + ng)) * np.concatenate([np.full(nq, 5.0), np.full(nk, 0.2), np.ones(nv + ng)])).astype(np.float32)
    qw, kw = (1 + 0.2 * r.standard_normal(nq)).astype(np.float32), (1 + 0.2 * r.standard_normal(nk)).astype(np.float32)
    slots = np.array([4, 1, -1, 0, 7, 2], np.int64)
    q, kc, vc = empty(T * nq * 4), empty(8 * nk * 4), empty(8 * nv * 4)
    L.vra_stack_op_qk_norm_store(f32(x).ptr, nq + nk + nv + ng, nq, nk, nv, f32(qw).ptr, f32(kw).ptr, 1e-6, q.ptr, kc.ptr, vc.ptr, raw(slots, np.int64).ptr, T, dt, 0)
    check()
    xx = x.astype(np.float64)
    tol = 2e-6 if dt == F32 else 4e-3
    assert rel(from_dev(q, (T, nq), dt), go.rms_norm(xx[:, :nq], qw, 1e-6)) < tol
    ks, vs = from_dev(kc, (8, nk), dt), from_dev(vc, (8, nv), dt)
    keep = slots >= 0
    assert rel(ks[slots[keep]], go.rms_norm(xx[keep, nq:nq + nk], kw, 1e-6)) < tol and rel(vs[slots[keep]], xx[keep, nq + nk:nq + nk + nv]) < tol


def latent_rows(c, k_rot, BS, r, dt, extra=3):
    """cache rows [c | k_rot] of ONE sequence over shuffled pages"""
    Tk = c.shape[0]
    nb = (Tk + BS - 1) // BS
    table = r.permutation(nb + extra)[:nb].astype(np.uint32)
    rows = np.full(((nb + extra) * BS, c.shape[1] + k_rot.shape[1]), 1e4, np.float32)
    for j in range(Tk):
        rows[int(table[j // BS]) * BS + j % BS] = np.concatenate([c[j], k_rot[j]])
    return to_dev(rows, dt), table


def run_sink_attention(L, q, positions, c, k_rot, scale, sink, dt, decode, r, BS=64):
    """absorbed latent attention of one sequence: q [Tq, H, kr + rd] over cache rows [c | k_rot]; values = the first kr columns"""
    Tq, H, kd = q.shape
    kr = c.shape[1]
    cache, table = latent_rows(c, k_rot, BS, r, dt)
    sk = f32(sink)
    if decode:
        res = []
        for i in range(Tq):
            o1 = empty(H * kr * 4)
            L.vra_stack_op_attention_ex(to_dev(q[i].reshape(1, -1), dt).ptr, H * kd, o1.ptr, cache.ptr, cache.ptr, raw([positions[i]], np.int64).ptr,
                                        raw(table, np.uint32).ptr, raw([positions[i] + 1], np.uint32).ptr, None, 1, 1, 1, H, 1, kd, kr, BS, len(table), scale,
                                        sk.ptr, kd, kd, dt, 0)
            check()
            res.append(from_dev(o1, (H, kr), dt))
        return np.stack(res)
    out = empty(Tq * H * kr * 4)
    L.vra_stack_op_attention_ex(to_dev(q.reshape(Tq, -1), dt).ptr, H * kd, out.ptr, cache.ptr, cache.ptr, raw(positions, np.int64).ptr, raw(table, np.uint32).ptr,
                                raw([c.shape[0]], np.uint32).ptr, raw([0, Tq], np.uint32).ptr, 1, Tq, Tq, H, 1, kd, kr, BS, len(table), scale, sk.ptr, kd, kd, dt, 0)
    check()
    return from_dev(out, (Tq, H, kr), dt)


def sink_reference(q, positions, c, k_rot, scale, sink):
    rows = np.concatenate([c, k_rot], 1).astype(np.float64)
    scores = np.stack([(q[:, hd].astype(np.float64) @ rows.T) * scale for hd in range(q.shape[1])])
    v = np.repeat(c.astype(np.float64)[:, None, :], q.shape[1], 1)
    return go.softmax_with_sink(scores, v, sink, positions)


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("H,kr,rd", [(3, 32, 8), (2, 13, 6), (4, 80, 48), (1, 160, 16)])
def test_softmax_sink_over_latent_rows(dt, decode, H, kr, rd):
    L = _lib.load()
    r = np.random.default_rng(H * 10 + kr)
    Tk = 150
    c, k_rot = rnd(r, (Tk, kr)), rnd(r, (Tk, rd))
    positions = np.array([0, 1, 5, 63, 64, 65, 127, 128, 149] if decode else list(range(100, 150)), np.int64)
    q = rnd(r, (len(positions), H, kr + rd))
    sink = np.linspace(-1.0, 3.0, H).astype(np.float32)
    scale = 1.3 / math.sqrt(kr + rd)
    got = run_sink_attention(L, q, positions, c, k_rot, scale, sink, dt, decode, r)
    assert rel(got, sink_reference(q, positions, c, k_rot, scale, sink)) < (2e-6 if dt == F32 else 4e-3)


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("decode", [False, True])
def test_sink_and_planted_latent_key(dt, decode):
    """a key made to stand out among 900 returns its latent wherever it lies (first token, page borders, far back, the query's own
    position) and is not felt one position earlier; a sink that dominates every score empties the output; a sink far below leaves the
    plain softmax"""
    L = _lib.load()
    r = np.random.default_rng(12)
    Tk, H, kr, rd = 900, 2, 16, 8
    base_c, base_rot = rnd(r, (Tk, kr), 0.1), rnd(r, (Tk, rd), 0.1)
    u = np.zeros(kr + rd, np.float32)
    u[kr + 3] = 1.0  # (the stand-out score lives in the rotated part: the marker in the latent stays a plain value)
    for j in (0, 1, 63, 64, 128, 300, 898):
        c, k_rot = base_c.copy(), base_rot.copy()
        k_rot[j] = 16.0 * u[kr:]
        c[j] = 5.0
        positions = np.array(sorted({max(j - 1, 0), j, j + 1, 899}), np.int64)
        q = np.tile(8.0 * u, (len(positions), H, 1)).astype(np.float32)
        for sink, kind in ((np.full(H, -30.0, np.float32), "plain"), (np.full(H, 3.0, np.float32), "mild"), (np.full(H, 60.0, np.float32), "dominant")):
            got = run_sink_attention(L, q, positions, c, k_rot, 0.25, sink, dt, decode, r)
            ref = sink_reference(q, positions, c, k_rot, 0.25, sink)
            assert np.abs(got - ref).max() < (1e-4 if dt == F32 else 3e-2), (j, kind)
            for i, p in enumerate(positions):
                if kind == "dominant":
                    assert np.abs(got[i]).max() < 1e-3, (j, p)
                elif p >= j:
                    assert np.abs(got[i] - 5.0).max() < 0.05, (j, p, kind)
                else:
                    assert np.abs(got[i]).max() < 0.6, (j, p, kind)


def run_sigmoid_attention(L, q, positions, k, v, scale, mask, pb, talk, gate, dt, decode, r, BS=64, scratch=True):
    Tq, H, dim = q.shape
    G, vdim = v.shape[1], v.shape[2]
    kc, vc, table = paged(k, v, BS, r, dt)
    slopes = np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], np.float32)
    win, keep_first = (int(mask["size"]), int(mask.get("keep_first", 0))) if mask else (0, 0)
    args = (H, G, dim, vdim, BS, len(table), scale, win, keep_first, f32(slopes).ptr, f32(pb).ptr, f32(talk).ptr)
    # scratch for the two-launch forms (the kernels' own one-launch form runs without: scratch=False)
    nbytes = max(Tq * H * G * vdim, 64 * H * vdim) * 4
    sc = (empty(nbytes).ptr, nbytes, k.shape[0]) if scratch else (None, 0, 0)
    if decode:
        res = []
        for i in range(Tq):
            o1 = empty(H * vdim * 4)
            L.vra_stack_op_sigmoid_attention(to_dev(q[i].reshape(1, -1), dt).ptr, H * dim, o1.ptr, kc.ptr, vc.ptr, raw([positions[i]], np.int64).ptr,
                                             raw(table, np.uint32).ptr, raw([positions[i] + 1], np.uint32).ptr, None, 1, 1, 1, *args,
                                             f32(gate[i]).ptr if gate is not None else None, H * vdim, *sc, dt, 0)
            check()
            res.append(from_dev(o1, (H, vdim), dt))
        return np.stack(res)
    out = empty(Tq * H * vdim * 4)
    L.vra_stack_op_sigmoid_attention(to_dev(q.reshape(Tq, -1), dt).ptr, H * dim, out.ptr, kc.ptr, vc.ptr, raw(positions, np.int64).ptr, raw(table, np.uint32).ptr,
                                     raw([k.shape[0]], np.uint32).ptr, raw([0, Tq], np.uint32).ptr, 1, Tq, Tq, *args,
                                     f32(gate).ptr if gate is not None else None, H * vdim, *sc, dt, 0)
    check()
    return from_dev(out, (Tq, H, vdim), dt)


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("H,G,dim,vdim,mask", [(6, 3, 16, 24, dict(size=40, keep_first=5)), (4, 4, 8, 8, dict(size=70, keep_first=0)), (2, 1, 5, 7, dict(size=3, keep_first=2)),
                                               (8, 2, 64, 64, None), (3, 3, 40, 100, dict(size=64, keep_first=64)), (16, 4, 32, 96, dict(size=1, keep_first=1)),
                                               (4, 1, 128, 128, dict(size=33, keep_first=40)), (4, 4, 72, 80, dict(size=100, keep_first=3)),
                                               (8, 8, 32, 32, dict(size=50, keep_first=2)), (6, 3, 32, 32, dict(size=90, keep_first=0)), (12, 3, 64, 32, None)])
def test_sigmoid_attention_random(dt, decode, H, G, dim, vdim, mask):
    L = _lib.load()
    r = np.random.default_rng(H * 100 + dim)
    Tk = 200
    k, v = rnd(r, (Tk, G, dim)), rnd(r, (Tk, G, vdim))
    positions = np.array([0, 1, 2, 5, 63, 64, 65, 127, 128, 199] if decode else list(range(150, 200)), np.int64)
    Tq = len(positions)
    q = rnd(r, (Tq, H, dim))
    pb = (-2.0 + r.standard_normal(H)).astype(np.float32)
    talk = (np.eye(H) + 0.3 * r.standard_normal((H, H))).astype(np.float32)
    gate = r.standard_normal((Tq, H * vdim)).astype(np.float32)
    scale = 1.5 / math.sqrt(dim)
    ref = go.sigmoid_weighted_values(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), scale, mask, pb, talk, positions)
    ref = ref * go.sigmoid(gate.astype(np.float64)).reshape(Tq, H, vdim)
    for scratch in (True, False):  # the two-launch forms (matrix cores for bf16 prompts, key tiles over workgroups for single tokens) and the plain one
        got = run_sigmoid_attention(L, q, positions, k, v, scale, mask, pb, talk, gate, dt, decode, r, scratch=scratch)
        assert rel(got, ref) < (3e-6 if dt == F32 else 5e-3), scratch


@pytest.mark.parametrize("dt", [F32, BF16])
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("H,G,dim,vdim", [(2, 1, 8, 4), (4, 2, 16, 16), (2, 2, 16, 16)])  # (bf16 prompts: FMA kernel, all-heads and per-head matrix-core kernels)
def test_sigmoid_attention_window_edges_and_kept_tokens(dt, decode, H, G, dim, vdim):
    """Every key weighs about e^-12 except ONE, whose score is made large: the output is its value (a marker) exactly when the design
    lets the query see it — the last key inside the window and the first one outside, the last kept first token and the one after it, at
    page borders, far back, the query's own position and the position before the key arrives."""
    L = _lib.load()
    r = np.random.default_rng(13)
    Tk = 700
    size, keep_first = 150, 12
    mask = dict(size=size, keep_first=keep_first)
    pb, talk = np.full(H, -12.0, np.float32), np.eye(H, dtype=np.float32)
    u = np.zeros(dim, np.float32)
    u[2] = 1.0
    base_k, base_v = rnd(r, (Tk, G, dim), 0.05), rnd(r, (Tk, G, vdim), 0.1)
    cases = []  # (key, query position, seen)
    for p in (699, 300, 200, 191):
        cases += [(p - size + 1, p, True), (p - size, p, False), (p, p, True), (keep_first - 1, p, True), (keep_first, p, False), (0, p, True)]
    cases += [(64, 63, False), (64, 64, True), (63, 64, True), (128, 277, True), (127, 277, False), (5, 5, True), (19, 19, True), (25, 100, True), (25, 175, False)]
    for j, p, seen in cases:
        k, v = base_k.copy(), base_v.copy()
        k[j, :] = 16.0 * u
        v[j, :] = 5.0
        q = np.tile(8.0 * u, (1, H, 1)).astype(np.float32)  # score 8 * 16 * 0.25 = 32, minus the distance penalty (at most 700 / 16), plus -12
        positions = np.array([p], np.int64)
        # (bf16 prompts: with scratch short steps take the per-head matrix-core kernel, without it the all-heads one where the shape allows)
        got = run_sigmoid_attention(L, q, positions, k, v, 0.25, mask, pb, talk, None, dt, decode, r, scratch=(j + p) % 2 == 0)
        ref = go.sigmoid_weighted_values(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), 0.25, mask, pb, talk, positions)
        assert np.abs(got - ref).max() < (1e-4 if dt == F32 else 3e-2), (j, p)
        # the last head (slope 2^-8) always keeps the planted weight near 1 when the key is seen
        assert (np.abs(got[0, H - 1] - 5.0).max() < 0.1) == seen, (j, p, seen, got[0, H - 1])
        if not seen:
            assert np.abs(got).max() < 0.05, (j, p)


def test_mixed_heads_use_their_own_values():
    """the mixing matrix moves weights between heads, never values: with talk = a permutation, head h weighs with head perm(h)'s scores
    and still sums the values of its OWN key/value head"""
    L = _lib.load()
    r = np.random.default_rng(14)
    Tk, H, G, dim, vdim = 40, 4, 2, 8, 4
    k, v, q = rnd(r, (Tk, G, dim)), rnd(r, (Tk, G, vdim)), rnd(r, (Tk, H, dim))
    pb = r.standard_normal(H).astype(np.float32)
    talk = np.eye(H, dtype=np.float32)[[2, 3, 0, 1]]
    pos = np.arange(Tk, dtype=np.int64)
    got = run_sigmoid_attention(L, q, pos, k, v, 0.4, None, pb, talk, None, F32, False, r)
    plain = go.sigmoid_weighted_values(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), 0.4, None, pb, np.eye(H), pos)
    ref = go.sigmoid_weighted_values(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), 0.4, None, pb, talk, pos)
    assert rel(got, ref) < 3e-6 and rel(got, plain) > 0.1


# ------------------------------------------------------------------------------------------------ whole models through the engine
def latent(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=24, scale=0.2, scaling=True, base=5e4):
    rot = dict(base=base, dims=rot_dim)
    if scaling:
        rot["scaling"] = dict(factor=5.0, original=96, fast=20.0, slow=1.5)
    return dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale, rot=rot)


def windowed(heads=6, kv_heads=3, dim=16, vdim=24, scale=0.3, size=70, keep_first=5):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if size:
        m["mask"] = dict(size=size, keep_first=keep_first)
    return m


def config_a():
    """other sizes than any shipped model: two query heads per key/value head, a window longer than a page, a layer that runs with another
    layer's tensors, a latent layer without frequency scaling and without feed-forward, a windowless layer with as many kv heads as heads"""
    return dict(architecture="Gaperax", width=96, vocab=160, norm=dict(eps=1e-5), layers=[
        dict(type="attention", mixer=windowed(), mlp=dict(kind="dense", ff=72)),
        dict(type="latent_attention", mixer=latent(), mlp=dict(kind="dense", ff=40)),
        dict(type="attention", mixer=windowed(), mlp=dict(kind="dense", ff=72), weights_of=0),
        dict(type="latent_attention", mixer=latent(heads=2, dim=8, rot_dim=16, vdim=16, kv_rank=48, q_rank=32, scaling=False), mlp=None),
        dict(type="latent_attention", mixer=latent(), mlp=dict(kind="dense", ff=40), weights_of=1),
        dict(type="attention", mixer=windowed(heads=4, kv_heads=4, dim=24, vdim=16, size=0), mlp=dict(kind="dense", ff=16)),
    ])


def config_b():
    """sizes that leave every 16-byte path: width 50, key size 5, value size 7, latent ranks 9 and 7, a window of 9 tokens that keeps 3"""
    return dict(architecture="Gaperax", width=50, vocab=70, norm=dict(eps=1e-6), layers=[
        dict(type="latent_attention", mixer=latent(heads=2, dim=6, rot_dim=2, vdim=5, kv_rank=9, q_rank=7, scale=0.4, base=100.0), mlp=dict(kind="dense", ff=11)),
        dict(type="attention", mixer=windowed(heads=2, kv_heads=1, dim=5, vdim=7, scale=0.6, size=9, keep_first=3), mlp=dict(kind="dense", ff=9)),
        dict(type="attention", mixer=windowed(heads=2, kv_heads=1, dim=5, vdim=7, scale=0.6, size=9, keep_first=3), mlp=dict(kind="dense", ff=9), weights_of=1),
    ])


@pytest.fixture(scope="module", params=[("a", F32), ("a", BF16), ("b", F32), ("b", BF16)], ids=["a-f32", "a-bf16", "b-f32", "b-bf16"])
def model(request):
    name, dt = request.param
    cfg = config_a() if name == "a" else config_b()
    tensors = go.random_tensors(cfg, 17 if name == "a" else 18)
    eng = build(cfg, tensors, dt, blocks=12, max_model_len=512)
    yield cfg, tensors, dt, eng
    eng.close()


def test_layers_one_by_one(model):
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 90, 1)  # (longer than every window but the unwindowed layer's)
    eng.layer_trace(True)
    got = eng.replay_step([(1, toks, list(range(len(toks))))], [1])
    trace = eng.read_layer_trace(len(toks))
    eng.layer_trace(False)
    layers = []
    ref = go.forward(cfg, tensors, toks, layers)
    for i, x in enumerate(layers):
        agree(trace[i], x, dt, f"layer {i}")
    agree(got, ref, dt)


def test_prefill_against_token_by_token_decoding(model):
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 150, 2)  # crosses two page borders and every window
    ref = go.forward(cfg, tensors, toks)
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


@pytest.mark.parametrize("sizes", [[2] * 30, [37, 3, 37, 2, 5], [64, 64, 2], [63, 2, 63, 2], [1, 5, 1, 1, 70, 1], [71, 9, 2, 70]])
def test_portions(model, sizes):
    """a prompt cut anywhere (down to two tokens, at and across page borders and window edges) gives the logits of the whole prompt —
    exactly, where the portions run in the prefill form"""
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
        # a single token behind a cached context runs the decode form: another order of the same sums, for that token and (through the
        # cache rows it leaves in the deeper layers) for the tokens behind it
        exact = exact and (c > 1 or at == 0) and dt == F32  # (bf16: steps of up to 32 rows sum their matrix products in another order)
        if exact:
            assert (got[at:at + c] == whole[at:at + c]).all(), f"portion at {at} of {c} tokens differs from the whole prompt"
        else:
            assert rel(got[at:at + c], whole[at:at + c]) < (1e-5 if dt == F32 else 3e-2)
        at += c


def test_unequal_batch_against_each_alone(model):
    cfg, tensors, dt, eng = model
    lens = [70, 3, 129, 1]
    prompts = [tokens_of(cfg, n, 10 + i) for i, n in enumerate(lens)]
    alone = [eng.replay_step([(1, p, list(range(len(p))))], [1]) for p in prompts]
    batch = eng.replay_step([(10 + i, p, list(range(len(p)))) for i, p in enumerate(prompts)], [10, 11, 12, 13])
    same = (lambda x, y: (x == y).all()) if dt == F32 else (lambda x, y: rel(x, y) < 3e-2)  # (bf16: the row count of a step picks the kernel)
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
            assert rel(got, alone[i]) < (1e-5 if dt == F32 else 3e-2)


def test_mixed_steps_and_reused_pages(model):
    """12 pages for requests that come and go: decoded tokens beside portions of prompts, pages handed back and taken again in another
    order; every logit row equals the request's own run"""
    cfg, tensors, dt, eng = model
    r = np.random.default_rng(4)
    lens = [130, 60, 200, 90, 33, 150, 64, 128]
    prompts = [tokens_of(cfg, n, 40 + i) for i, n in enumerate(lens)]
    ref = [go.forward(cfg, tensors, p) for p in prompts]
    waiting, live = list(range(len(prompts))), {}
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


def test_long_prompt_in_one_step_and_in_portions():
    """a 1700-token prompt: bf16 steps of this size run the sigmoid attention's all-heads kernel, shorter portions the per-head one; both agree
    with the oracle, and the long step with its portions"""
    cfg = dict(config_a(), layers=[dict(type="attention", mixer=windowed(heads=8, kv_heads=2, dim=32, vdim=32, size=300, keep_first=7), mlp=dict(kind="dense", ff=64)),
                                   dict(type="latent_attention", mixer=latent(), mlp=None)])
    tensors = go.random_tensors(cfg, 23)
    toks = tokens_of(cfg, 1700, 8)
    want = list(range(0, 1700, 53)) + [1699]
    ref = go.forward(cfg, tensors, toks)[want]
    for dt in (F32, BF16):
        eng = build(cfg, tensors, dt, blocks=56, max_model_len=1792)
        whole = eng.replay_step([(1, toks, want)], [1])
        agree(whole, ref, dt, "whole")
        parts, at = [], 0
        for c in (700, 40, 960):
            parts.append(eng.replay_step([(2, toks[at:at + c], [w - at for w in want if at <= w < at + c])], [2] if at + c == 1700 else []))
            at += c
        eng.close()
        parts = np.concatenate(parts)
        agree(parts, ref, dt, "portions")
        assert rel(parts, whole) < (1e-5 if dt == F32 else 3e-2)


def test_long_decoding(model):
    """310 decoded tokens: every window passes over decoded tokens, the kept first tokens stay"""
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 330, 5)
    ref = go.forward(cfg, tensors, toks)
    eng.replay_step([(1, toks[:20], [])], [])
    rows = [eng.replay_step([(1, toks[p:p + 1], [0])], [1] if p == len(toks) - 1 else [])[0] for p in range(20, len(toks))]
    agree(np.stack(rows), ref[20:], dt)


def test_a_far_token_reaches_the_end_through_the_latent_layers_only():
    """changing token 30 of a 400-token prompt: the windowed layers alone (window 70, 5 kept tokens) do not carry it to the last position,
    a latent layer does — in one whole prompt and in token-by-token decoding"""
    cfg = config_a()
    tensors = go.random_tensors(cfg, 21)
    sig_only = dict(cfg, layers=[cfg["layers"][0]])
    with_latent = dict(cfg, layers=cfg["layers"][:2])
    toks = tokens_of(cfg, 400, 6)
    other = list(toks)
    other[30] = (toks[30] + 7) % cfg["vocab"]
    for sub, reaches in ((sig_only, False), (with_latent, True)):
        names = go.tensor_shapes(sub)
        eng = build(sub, {n: tensors[n] for n in names}, F32, blocks=16, max_model_len=512)
        a = eng.replay_step([(1, toks, [399])], [1])
        b = eng.replay_step([(2, other, [399])], [2])
        eng.replay_step([(3, other[:380], [])], [])
        d = np.stack([eng.replay_step([(3, other[p:p + 1], [0])], [3] if p == 399 else [])[0] for p in range(380, 400)])[-1:]
        eng.close()
        ref_a, ref_b = go.forward(sub, tensors, toks)[399:], go.forward(sub, tensors, other)[399:]
        assert rel(a, ref_a) < 3e-5 and rel(b, ref_b) < 3e-5 and rel(d, ref_b) < 3e-5
        assert (np.abs(a - b).max() > 1e-4) == reaches and (np.abs(ref_a - ref_b).max() > 1e-9) == reaches


@pytest.mark.parametrize("use_graph", [False, True])
def test_greedy_generation_through_the_scheduler(use_graph):
    """Engine.generate: the engine's own scheduler, block manager, prefill and decode steps (captured decode graphs when asked) and its
    argmax — against the oracle's greedy continuation, f32 so that near ties do not decide"""
    cfg = config_a()
    tensors = go.random_tensors(cfg, 19)
    eng = build(cfg, tensors, F32, blocks=16, max_model_len=256, use_graph=use_graph)
    prompts = [tokens_of(cfg, n, 60 + n) for n in (5, 70, 31)]
    outs = eng.generate(prompts, max_tokens=12, ignore_eos=True)
    eng.close()
    for p, out in zip(prompts, outs):
        seq = list(p)
        for t in out:
            lg = go.forward(cfg, tensors, seq)[-1]
            top2 = np.sort(lg)[-2:]
            assert int(t) == int(lg.argmax()) or top2[1] - top2[0] < 1e-3, (len(p), len(seq))
            seq.append(int(t))
        assert len(out) == 12


def test_synthetic_weights_and_cache_plan():
    """random weights of a configured shape load, the cache plan follows the layers' rows (a latent layer keeps one row per token and no
    value blocks), a generation runs"""
    from vllm_rs_amd.engine import Engine
    cfg = checkpoint.parse_config(config_a())
    eng = Engine(cfg, max_num_seqs=4, max_model_len=256, kv_fraction=0.01, use_graph=False).init_synthetic()
    assert eng.num_gpu_blocks > 16
    out = eng.generate([list(range(1, 40))], max_tokens=5, ignore_eos=True)[0]
    assert len(out) == 5
    eng.close()


def test_trace_runner_on_a_model_folder(tmp_path):
    """bin/trace_run as a user starts it: config.json + model.safetensors (bfloat16 tensors, scalar slopes of the norms as 0-d tensors) in a
    folder, steps on standard input (a prompt in portions beside another request's single tokens, pages given back and taken again in a
    pool of three), logits files out — against the oracle, in both dtypes"""
    import json
    import os
    import struct
    import subprocess
    import sys
    cfg = config_a()
    tensors = go.random_tensors(cfg, 31)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfg))
    header, blobs, off = {}, [], 0
    for name, a in tensors.items():
        b = checkpoint.f32_to_bf16_bits(np.asarray(a, np.float32)).tobytes()
        header[name] = dict(dtype="BF16", shape=list(np.shape(a)), data_offsets=[off, off + len(b)])
        off += len(b)
        blobs.append(b)
    h = json.dumps(header).encode()
    (model_dir / "model.safetensors").write_bytes(struct.pack("<Q", len(h)) + h + b"".join(blobs))
    p1, p2, p3 = tokens_of(cfg, 100, 1), tokens_of(cfg, 40, 2), tokens_of(cfg, 64, 3)
    every = lambda n: list(range(n))
    steps = [dict(entries=[dict(id="x", tokens=p1[:37], want=every(37)), dict(id="y", tokens=p2[:39], want=[])], end=[]),
             dict(entries=[dict(id="x", tokens=p1[37:99], want=every(62)), dict(id="y", tokens=p2[39:], want=[0])], end=["y"]),
             dict(entries=[dict(id="x", tokens=p1[99:], want=[0])], end=["x"]),
             dict(entries=[dict(id="z", tokens=p3, want=every(64))], end=["z"])]
    for i, s in enumerate(steps):
        s["step"] = i
    r1, r2, r3 = (go.forward(cfg, tensors, p) for p in (p1, p2, p3))
    want = [r1[:37], np.concatenate([r1[37:99], r2[39:]]), r1[99:], r3]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype, dt in (("float32", F32), ("bfloat16", BF16)):
        out = tmp_path / ("out_" + dtype)
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype, "--out", str(out),
                            "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps).encode() + b"\n", capture_output=True, timeout=110)
        assert r.returncode == 0, r.stderr.decode()[-1500:]
        assert [ln for ln in r.stdout.decode().split("\n") if ln.startswith("done")] == ["done %d" % i for i in range(4)]
        got = [np.fromfile(out / ("%d.f32" % i), "<f4").reshape(-1, cfg["vocab"]) for i in range(4)]
        assert [g.shape[0] for g in got] == [w.shape[0] for w in want]
        agree(np.concatenate(got), np.concatenate(want), dt, dtype)
