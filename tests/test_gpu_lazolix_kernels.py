"""Each mechanism of the Lazolix design alone: the HIP kernel behind its one-sequence C entry (csrc/capi_stream32.hip) against the float64 oracle.
Where random inputs would hide a fault -- a far key among hundreds, a window's edge, a sink -- one query / key pair is scaled so that one score stands out."""
import ctypes as C

import numpy as np
import pytest

import lazolix_oracle as O
from uzu_amd import _ffi

pytestmark = pytest.mark.gpu


def ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def linear(ctx, x, w, bias=None, residual=None, batch=1, act=0, bf16=0, form=0):
    rows = x.shape[0]
    n, k = w.shape[-2], w.shape[-1]
    y = np.empty((rows, n * batch), dtype=np.float32)
    wb, bb = O.bf16_bits(w), None if bias is None else O.bf16_bits(bias)
    _ffi.call("uzu_hip_s32_linear", ctx._h, ptr(f32(x)), ptr(wb), ptr(bb), ptr(None if residual is None else f32(residual)), ptr(y), C.c_uint32(rows), C.c_uint32(n), C.c_uint32(k),
              C.c_uint32(batch), C.c_uint32(act), C.c_uint32(bf16), C.c_uint32(form))
    return y


@pytest.mark.parametrize("rows,n,k", [(1, 7, 24), (3, 33, 40), (16, 64, 72), (17, 5, 9), (70, 130, 100), (129, 64, 64), (300, 96, 136)])
def test_linear_true_f32_every_row_count(hip_ctx, rows, n, k):
    rng = np.random.default_rng(rows)
    x, w, b, res = rng.standard_normal((rows, k)), O.to_bf16(rng.standard_normal((n, k))), O.to_bf16(rng.standard_normal(n)), rng.standard_normal((rows, n))
    want = np.maximum(f32(x).astype(np.float64) @ w.T.astype(np.float64) + b, 0) ** 2 + f32(res)
    got = linear(hip_ctx, x, w, b, res, act=1)
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("rows,n,k,batch", [(32, 64, 64, 1), (200, 200, 72, 1), (130, 48, 24, 3), (257, 128, 320, 1), (64, 320, 128, 2), (1000, 130, 136, 1)])
def test_linear_matrix_core_form_equals_the_plain_form(hip_ctx, rows, n, k, batch):
    """bf16 products: the matrix-core tiles against the same products without the matrix cores, every tile shape, ragged edges, the batched per-head form"""
    rng = np.random.default_rng(n)
    x = rng.standard_normal((rows, k * batch))
    w = O.to_bf16(rng.standard_normal((batch, n, k)))
    b = O.to_bf16(rng.standard_normal(n)) if batch == 1 else None
    res = rng.standard_normal((rows, n)) if batch == 1 else None
    a = linear(hip_ctx, x, w, b, res, batch=batch, act=0, bf16=1, form=1)
    c = linear(hip_ctx, x, w, b, res, batch=batch, act=0, bf16=1, form=2)
    xb = O.to_bf16(x).astype(np.float64)
    want = np.concatenate([xb[:, z * k:(z + 1) * k] @ w[z].T.astype(np.float64) for z in range(batch)], axis=1)
    if batch == 1:
        want = want + b + f32(res)
    assert np.isfinite(a).all()
    assert np.abs(a - want).max() <= 3e-5 * max(1.0, np.abs(want).max()) and np.abs(c - want).max() <= 3e-5 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("rows,start", [(1, 0), (1, 5), (6, 0), (9, 3)])
def test_dyn_tanh_and_token_shift_with_state(hip_ctx, rows, start):
    rng = np.random.default_rng(rows + start)
    d = 70
    x, w, b, mu, prev = rng.standard_normal((rows, d)) * 2, 1 + 0.2 * rng.standard_normal(d), 0.1 * rng.standard_normal(d), rng.random(d), rng.standard_normal(d)
    alpha = 0.7
    h = O.dyn_tanh(f32(x), f32(w), f32(b), np.float32(alpha))
    want, last = O.token_shift(h, f32(mu), prev=f32(prev) if start else None)
    out, state = np.empty((rows, d), dtype=np.float32), f32(prev).copy()
    _ffi.call("uzu_hip_s32_dyn_tanh", hip_ctx._h, ptr(f32(x)), ptr(f32(w)), ptr(f32(b)), C.c_float(alpha), ptr(f32(mu)), ptr(state), C.c_uint32(start), ptr(out), C.c_uint32(rows),
              C.c_uint32(d))
    assert np.abs(out - want).max() < 5e-6 and np.abs(state - last).max() < 5e-6   # position 0 ignores what the state row held
    plain = np.empty((rows, d), dtype=np.float32)
    _ffi.call("uzu_hip_s32_dyn_tanh", hip_ctx._h, ptr(f32(x)), ptr(f32(w)), None, C.c_float(alpha), None, None, C.c_uint32(0), ptr(plain), C.c_uint32(rows), C.c_uint32(d))
    assert np.abs(plain - O.dyn_tanh(f32(x), f32(w), None, np.float32(alpha))).max() < 5e-6


def test_depth_mix(hip_ctx):
    rng = np.random.default_rng(5)
    slots, w = f32(rng.standard_normal((4, 7, 33))), f32(rng.standard_normal(4))
    out = np.empty((7, 33), dtype=np.float32)
    _ffi.call("uzu_hip_s32_depth_mix", hip_ctx._h, ptr(slots), ptr(w), C.c_uint32(4), ptr(out), C.c_uint32(7), C.c_uint32(33))
    assert np.abs(out - O.depth_mix(list(slots.astype(np.float64)), w)).max() < 1e-5


@pytest.mark.parametrize("bf16", [0, 1])
def test_latent_norm_append_keeps_earlier_rows(hip_ctx, bf16):
    rng = np.random.default_rng(6)
    start, rows, rank = 5, 4, 40
    cache = f32(O.to_bf16(rng.standard_normal((start + rows, rank))))
    before = cache.copy()
    u, g = f32(rng.standard_normal((rows, rank)) * 3), f32(1 + 0.2 * rng.standard_normal(rank))
    _ffi.call("uzu_hip_s32_latent_norm_append", hip_ctx._h, ptr(u), ptr(g), C.c_float(1e-3), ptr(cache), C.c_uint32(bf16), C.c_uint32(start), C.c_uint32(rows), C.c_uint32(rank))
    want = O.rms_latent(u.astype(np.float64), g, 1e-3)
    assert np.array_equal(cache[:start], before[:start])
    assert np.abs(cache[start:] - want).max() <= (2e-2 if bf16 else 5e-6)


def core(ctx, qlat, cache, sinks, rows, start, heads, rank, window, scale, bf16, form):
    out = np.empty((rows, heads * rank), dtype=np.float32)
    _ffi.call("uzu_hip_s32_latent_attention", ctx._h, ptr(f32(qlat)), ptr(f32(cache)), ptr(None if sinks is None else f32(sinks)), ptr(out), C.c_uint32(rows), C.c_uint32(start),
              C.c_uint32(heads), C.c_uint32(rank), C.c_uint32(window), C.c_float(scale), C.c_uint32(bf16), C.c_uint32(form))
    return out


FORMS = [(0, 1), (1, 1), (1, 2), (1, 3)]  # (bf16 cache, form): f32 simple, bf16 simple, bf16 tiled, bf16 tiled with the keys split over workgroups


@pytest.mark.parametrize("bf16,form", FORMS)
@pytest.mark.parametrize("rows,start,heads,rank,window", [(1, 0, 3, 40, 0), (7, 0, 3, 40, 4), (1, 9, 5, 24, 4), (40, 3, 3, 72, 9), (5, 130, 2, 128, 0), (150, 0, 8, 128, 33), (33, 64, 16, 256, 32), (3, 2, 2, 1100, 0), (2, 6, 3, 320, 5)])
def test_latent_core_against_the_oracle(hip_ctx, bf16, form, rows, start, heads, rank, window):
    rng = np.random.default_rng(rows * 7 + start)
    if form >= 2 and (rank > 256 or rank % 8):  # the matrix-core form refuses what it does not cover (the dispatcher then takes the simple form)
        with pytest.raises(_ffi.UzuHipError):
            core(hip_ctx, np.zeros((rows, heads * rank)), np.zeros((start + rows, rank)), None, rows, start, heads, rank, window, 1.0, bf16, form)
        return
    cache = O.to_bf16(rng.standard_normal((start + rows, rank)))
    qlat = O.to_bf16(rng.standard_normal((rows, heads * rank)) * 1.5)   # bf16-representable queries: the tiled form's rounding of them is then exact
    sinks = rng.standard_normal(heads) if rows % 2 else None
    got = core(hip_ctx, qlat, cache, sinks, rows, start, heads, rank, window, rank ** -0.5, bf16, form)
    want = O.latent_core(qlat, cache, heads, rank ** -0.5, window, sinks, start)
    assert np.isfinite(got).all() and np.abs(got - want).max() < (2e-4 if form >= 2 else 2e-5)


@pytest.mark.parametrize("bf16,form", FORMS)
@pytest.mark.parametrize("rows,start", [(1, 299), (300, 0), (45, 255)])   # decoding alone, a whole prompt, a portion behind a prefix
def test_latent_core_one_key_stands_out_at_every_edge(hip_ctx, bf16, form, rows, start):
    """The last row's query is aligned with ONE key.  Just inside the window (and at a block border, and far back without a window) the output must be that key's
    latent; just outside, the key must leave no trace."""
    rng = np.random.default_rng(9)
    heads, rank, T = 2, 64, start + rows
    t = T - 1
    for window, j, inside in [(40, t - 39, True), (40, t - 40, False), (0, 3, True), (200, t - 199, True), (200, t - 200, False), (33, t - 32, True), (1, t, True), (1, t - 1, False),
                              (64, t - 63, True), (65, t - 64, True), (64, t - 64, False)]:
        cache = O.to_bf16(rng.standard_normal((T, rank)))
        qlat = O.to_bf16(rng.standard_normal((rows, heads * rank)) * 0.3)
        qlat[-1, :rank] = O.to_bf16(cache[j] * 4.0)                       # head 0 of the last row: score ~ 4 * 64 * scale above everything else
        got = core(hip_ctx, qlat, cache, np.zeros(heads), rows, start, heads, rank, window, 0.5, bf16, form)
        want = O.latent_core(qlat, cache, heads, 0.5, window, np.zeros(heads), start)
        assert np.abs(got - want).max() < 3e-4, (window, j)
        hit = np.abs(got[-1, :rank] - cache[j]).max() < 1e-2
        assert hit == inside, (window, j, inside)


@pytest.mark.parametrize("bf16,form", FORMS)
def test_latent_core_sink_takes_weight_and_first_tokens(hip_ctx, bf16, form):
    rng = np.random.default_rng(10)
    heads, rank = 4, 32
    cache, qlat = O.to_bf16(rng.standard_normal((6, rank))), O.to_bf16(rng.standard_normal((6, heads * rank)))
    sinks = np.array([-30.0, 0.0, 5.0, 30.0])
    got = core(hip_ctx, qlat, cache, sinks, 6, 0, heads, rank, 3, 0.2, bf16, form)
    assert np.abs(got - O.latent_core(qlat, cache, heads, 0.2, 3, sinks)).max() < 2e-4
    assert np.abs(got[0, :rank] - cache[0]).max() < 1e-3        # position 0, a negligible sink: the only key gets all the weight
    assert np.abs(got[:, 3 * rank:]).max() < 1e-6               # a dominant sink: (almost) nothing is left for the keys
    no_sink = core(hip_ctx, qlat, cache, None, 6, 0, heads, rank, 3, 0.2, bf16, form)
    assert np.abs(no_sink[0].reshape(heads, rank) - cache[0]).max() < 1e-3


@pytest.mark.parametrize("routed,identity,top,ff", [(4, 0, 1, 16), (3, 2, 2, 24), (1, 1, 2, 8), (0, 3, 2, 0), (9, 1, 4, 40), (5, 1, 4, 3200)])
def test_score_routed_experts(hip_ctx, routed, identity, top, ff):
    rng = np.random.default_rng(routed * 10 + top)
    rows, d = 13, 48
    x = f32(rng.standard_normal((rows, d)))
    wr = O.to_bf16(rng.standard_normal((routed + identity, d)) * 0.5)
    corr = f32(0.3 * rng.standard_normal(routed + identity))
    experts = [tuple(O.to_bf16(rng.standard_normal(s) / np.sqrt(s[1])) for s in ((ff, d), (ff, d), (d, ff))) for _ in range(routed)]
    w13 = np.stack([np.concatenate([O.bf16_bits(u), O.bf16_bits(g)]) for g, u, _ in experts]) if routed else None
    w2 = np.stack([O.bf16_bits(dn) for _, _, dn in experts]) if routed else None
    res = f32(rng.standard_normal((rows, d)))
    y, ids, wts = np.empty((rows, d), dtype=np.float32), np.empty((rows, top), dtype=np.int32), np.empty((rows, top), dtype=np.float32)
    _ffi.call("uzu_hip_s32_moe", hip_ctx._h, ptr(x), ptr(O.bf16_bits(wr)), ptr(corr), ptr(w13), ptr(w2), ptr(res), ptr(y), ptr(ids), ptr(wts), C.c_uint32(rows), C.c_uint32(d),
              C.c_uint32(ff), C.c_uint32(routed), C.c_uint32(identity), C.c_uint32(top), C.c_uint32(0))
    want_ids, want_w = O.route(x.astype(np.float64), wr, corr, top)
    assert np.array_equal(ids, want_ids) and np.abs(wts - want_w).max() < 1e-5
    want = res + O.moe_mlp(x.astype(np.float64), wr, corr, experts, top)
    assert np.abs(y - want).max() < 3e-5 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("rows,routed,identity,top,ff,d", [(64, 4, 1, 2, 32, 64), (300, 3, 0, 1, 40, 72), (257, 8, 2, 3, 64, 128), (100, 5, 1, 2, 24, 48)])
def test_grouped_expert_form_equals_the_per_row_form(hip_ctx, rows, routed, identity, top, ff, d):
    """prefill-sized row counts, bf16 products: buckets per expert through the matrix-core linear against the per-row kernels and the oracle on rounded operands"""
    rng = np.random.default_rng(rows)
    x = f32(rng.standard_normal((rows, d)))
    wr = O.to_bf16(rng.standard_normal((routed + identity, d)) * 0.5)
    corr = f32(0.1 * rng.standard_normal(routed + identity))
    experts = [tuple(O.to_bf16(rng.standard_normal(s) / np.sqrt(s[1])) for s in ((ff, d), (ff, d), (d, ff))) for _ in range(routed)]
    w13 = np.stack([np.concatenate([O.bf16_bits(u), O.bf16_bits(g)]) for g, u, _ in experts])
    w2 = np.stack([O.bf16_bits(dn) for _, _, dn in experts])
    res = f32(rng.standard_normal((rows, d)))
    outs = []
    for mode in (1, 2):
        y, ids, wts = np.empty((rows, d), dtype=np.float32), np.empty((rows, top), dtype=np.int32), np.empty((rows, top), dtype=np.float32)
        _ffi.call("uzu_hip_s32_moe", hip_ctx._h, ptr(x), ptr(O.bf16_bits(wr)), ptr(corr), ptr(w13), ptr(w2), ptr(res), ptr(y), ptr(ids), ptr(wts), C.c_uint32(rows), C.c_uint32(d),
                  C.c_uint32(ff), C.c_uint32(routed), C.c_uint32(identity), C.c_uint32(top), C.c_uint32(mode))
        outs.append(y)
    assert np.isfinite(outs[1]).all() and np.abs(outs[0] - outs[1]).max() < 2e-4 * max(1.0, np.abs(outs[0]).max())
