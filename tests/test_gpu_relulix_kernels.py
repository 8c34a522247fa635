"""Each new mechanism of the Relulix design alone: the HIP kernel behind its one-sequence C entry (csrc/capi_stream32.hip) against the float64 oracle, and
the forms of one kernel against each other.  Where random inputs would hide a fault -- a far key among hundreds, a window's edge, the sink, a far token in a
slowly decaying state -- one query / key pair is scaled so that one term stands out."""
import ctypes as C

import numpy as np
import pytest

import relulix_oracle as O
from uzu_amd import _ffi

pytestmark = pytest.mark.gpu
u32, f32c = C.c_uint32, C.c_float


def ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def tables(rot, positions):
    """cos / sin tables [positions][dims] with both halves filled, from the oracle's frequencies (float64, then rounded)"""
    f, m = O.frequencies(rot)
    ang = np.arange(positions, dtype=np.float64)[:, None] * f[None, :]
    c, s = np.cos(ang) * m, np.sin(ang) * m
    return f32(np.concatenate([c, c], axis=1)), f32(np.concatenate([s, s], axis=1))


def rotate(ctx, q, k, rot, start, key_scale):
    rows, H, dim = q.shape
    G = k.shape[1]
    packed = f32(np.concatenate([q.reshape(rows, -1), k.reshape(rows, -1)], axis=1))
    cs, sn = tables(rot, start + rows)
    _ffi.call("uzu_hip_s32_rotate", ctx._h, ptr(packed), ptr(cs), ptr(sn), u32(rows), u32(start), u32(H), u32(G), u32(dim), u32(rot["dims"]), f32c(key_scale))
    return packed[:, :H * dim].reshape(rows, H, dim), packed[:, H * dim:].reshape(rows, G, dim)


def attention(ctx, q, K, V, mx, start, sinks="unit", bf16=0, form=0):
    rows, H, dim = q.shape
    G, vd = K.shape[1], V.shape[2]
    out = np.empty((rows, H * vd), dtype=np.float32)
    sk = f32(np.zeros(H)) if isinstance(sinks, str) else (None if sinks is None else f32(sinks))
    _ffi.call("uzu_hip_s32_window_attention", ctx._h, ptr(f32(q)), ptr(f32(K)), ptr(f32(V)), ptr(sk), ptr(out), u32(rows), u32(start), u32(H), u32(G), u32(dim), u32(vd),
              u32(int((mx.get("mask") or {}).get("size") or 0)), f32c(mx["scale"]), f32c(mx.get("softcap") or 0.0), u32(bf16), u32(form))
    return out.reshape(rows, H, vd)


def retention(ctx, q, k, v, decay, state, start, form):
    rows, H, dim = q.shape
    vd = v.shape[2]
    out = np.empty((rows, H * vd), dtype=np.float32)
    st = f32(state).copy()
    _ffi.call("uzu_hip_s32_retention", ctx._h, ptr(f32(q)), ptr(f32(k)), ptr(f32(v)), ptr(f32(decay)), ptr(st), ptr(out), u32(rows), u32(start), u32(H), u32(dim), u32(vd), u32(form))
    return out.reshape(rows, H, vd), st.reshape(H, dim, vd)


YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}


@pytest.mark.parametrize("dims,dim,scaling,start", [(8, 8, None, 0), (4, 12, None, 7), (16, 24, YARN, 300), (2, 8, YARN, 1), (32, 32, {"factor": 3.0, "original": 256, "fast": 24.0, "slow": 2.0}, 1000)])
def test_rotation_partial_and_scaled(hip_ctx, dims, dim, scaling, start):
    rng = np.random.default_rng(dims + start)
    rot = O.rot(dims, 10000.0 if dims != 4 else 500.0, scaling)
    q, k = rng.standard_normal((5, 3, dim)), rng.standard_normal((5, 2, dim))
    pos = np.arange(start, start + 5)
    gq, gk = rotate(hip_ctx, q, k, rot, start, 0.25)
    wq, wk = O.rotate(f32(q), pos, rot), O.rotate(f32(k), pos, rot) * 0.25
    tol = 3e-6
    assert np.abs(gq - wq).max() < tol * np.abs(wq).max() and np.abs(gk - wk).max() < tol * np.abs(wk).max()
    assert np.array_equal(gq[..., dims:], f32(q)[..., dims:])  # what does not turn passes unchanged


def qkv(rng, T, H, G, dim, vd):
    return rng.standard_normal((T, H, dim)), rng.standard_normal((T, G, dim)), rng.standard_normal((T, G, vd))


CASES = [  # heads, kv heads, dim, vdim, window, cap, positions, start
    (4, 4, 8, 8, 5, 0.0, 40, 0), (6, 2, 16, 8, 0, 3.0, 150, 0), (3, 1, 24, 40, 33, 0.0, 100, 0), (2, 2, 64, 64, 70, 5.0, 200, 0),
    (8, 2, 32, 16, 64, 0.0, 130, 100), (4, 4, 8, 16, 1, 2.0, 20, 0), (4, 1, 16, 16, 129, 0.0, 300, 290), (2, 1, 128, 128, 200, 30.0, 260, 0),
]


@pytest.mark.parametrize("H,G,dim,vd,window,cap,T,start", CASES)
def test_attention_simple_form_true_f32(hip_ctx, H, G, dim, vd, window, cap, T, start):
    rng = np.random.default_rng(H * 100 + T)
    q, K, V = qkv(rng, T, H, G, dim, vd)
    mx = {"heads": H, "kv_heads": G, "scale": 1.7 / np.sqrt(dim), "mask": {"size": window}, "softcap": cap}
    want = O.attention_core(f32(q)[start:], f32(K), f32(V), mx, start)
    got = attention(hip_ctx, q[start:], K, V, mx, start, form=1)
    assert np.abs(got - want).max() < 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("H,G,dim,vd,window,cap,T,start", [c for c in CASES if c[2] % 8 == 0 and c[3] % 8 == 0])
def test_attention_matrix_core_form_equals_the_simple_form(hip_ctx, H, G, dim, vd, window, cap, T, start):
    rng = np.random.default_rng(H * 100 + T + 1)
    q, K, V = qkv(rng, T, H, G, dim, vd)
    mx = {"heads": H, "kv_heads": G, "scale": 1.7 / np.sqrt(dim), "mask": {"size": window}, "softcap": cap}
    Kb, Vb = O.to_bf16(K), O.to_bf16(V)
    want = O.attention_core(f32(q)[start:], Kb, Vb, mx, start)
    if T - start < 16:
        pytest.skip("decode-sized passes take the simple form")
    a = attention(hip_ctx, q[start:], K, V, mx, start, bf16=1, form=2)
    b = attention(hip_ctx, q[start:], K, V, mx, start, bf16=1, form=1)
    assert np.isfinite(a).all()
    assert np.abs(b - want).max() < 2e-5 * np.abs(want).max()
    assert np.abs(a - want).max() < 6e-5 * np.abs(want).max()  # the query as hi + lo bf16: 16 significant bits


@pytest.mark.parametrize("H,G,dim,vd,window,cap,T,start", [c for c in CASES if c[2] % 8 == 0 and c[3] % 8 == 0])
def test_attention_split_keys_form_on_few_rows(hip_ctx, H, G, dim, vd, window, cap, T, start):
    """a decode-sized pass: the last one to three rows of the sequence, their key blocks spread over five workgroups and merged"""
    rng = np.random.default_rng(H * 100 + T + 2)
    q, K, V = qkv(rng, T, H, G, dim, vd)
    mx = {"heads": H, "kv_heads": G, "scale": 1.7 / np.sqrt(dim), "mask": {"size": window}, "softcap": cap}
    for rows in (1, 3):
        want = O.attention_core(f32(q)[T - rows:], O.to_bf16(K), O.to_bf16(V), mx, T - rows)
        got = attention(hip_ctx, q[T - rows:], K, V, mx, T - rows, bf16=1, form=3)
        assert np.isfinite(got).all() and np.abs(got - want).max() < 6e-5 * np.abs(want).max()


@pytest.mark.parametrize("bf16,form", [(0, 1), (1, 1), (1, 2)])
@pytest.mark.parametrize("window", [1, 2, 31, 32, 33, 64, 65, 130])
def test_one_key_stands_out_just_inside_and_just_outside_the_window(hip_ctx, bf16, form, window):
    """Position t sees t - window + 1 .. t.  A key with a huge score is planted one step inside the edge and one step outside: inside it owns the output,
    outside the output must not know it -- for rows in a prompt and for one decoded row, with the edge at and around key-block borders."""
    H, G, dim, vd, T = 2, 1, 16, 16, 330
    rng = np.random.default_rng(window)
    q, K, V = qkv(rng, T, H, G, dim, vd)
    q, K = q * 0.1, K * 0.1
    mx = {"heads": H, "kv_heads": G, "scale": 1.0, "mask": {"size": window}}
    for t in (window + 3, 200, T - 1):
        for inside in (True, False):
            j = t - window + 1 if inside else t - window
            if j < 0:
                continue
            K2, V2, q2 = K.copy(), V.copy(), q.copy()
            K2[j, 0] = 0.0
            K2[j, 0, 3] = 8.0
            q2[t, :, 3] = 8.0       # score 64 against O(1) elsewhere
            V2[j, 0] = 100.0 + np.arange(vd)
            for start in (0, t):    # the row inside a prompt from position 0, and decoded alone
                got = attention(hip_ctx, q2[start:t + 1], K2[:t + 1], V2[:t + 1], mx, start, bf16=bf16, form=form if (start == 0 and t + 1 >= 16) else (3 if form == 2 else 1))[-1]
                if inside:
                    assert np.abs(got - V2[j, 0]).max() < 1e-2, (t, start)
                else:
                    assert np.abs(got).max() < 20.0, (t, start)
                    want = O.attention_core(f32(q2[t:t + 1]), O.to_bf16(K2[:t + 1]) if bf16 else f32(K2[:t + 1]), O.to_bf16(V2[:t + 1]) if bf16 else f32(V2[:t + 1]), mx, t)[0]
                    assert np.abs(got - want).max() < 1e-4 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("bf16,form", [(0, 1), (1, 2)])
def test_far_key_among_hundreds_without_a_window_and_the_first_tokens(hip_ctx, bf16, form):
    H, G, dim, vd, T = 4, 2, 32, 24 if form == 1 else 32, 700
    rng = np.random.default_rng(5)
    q, K, V = qkv(rng, T, H, G, dim, vd)
    q, K = q * 0.05, K * 0.05
    mx = {"heads": H, "kv_heads": G, "scale": 1.0}
    for j in (0, 1, 31, 32, 63, 64, 377):
        K2, V2, q2 = K.copy(), V.copy(), q.copy()
        K2[j, 1] = 0.0
        K2[j, 1, 0] = 9.0
        q2[T - 1, 2:, 0] = 9.0      # heads 2 and 3 read key / value head 1
        V2[j, 1] = -50.0
        got = attention(hip_ctx, q2, K2, V2, mx, 0, bf16=bf16, form=form)[-1]
        assert np.abs(got[2:] + 50.0).max() < 1e-2 and np.abs(got[:2]).max() < 5.0, j
    # position 0 sees itself and the sink only: softmax weight e^s / (1 + e^s)
    got = attention(hip_ctx, q[:20], K[:20], V[:20], mx, 0, bf16=bf16, form=form)[0]
    Kr, Vr = (O.to_bf16(K), O.to_bf16(V)) if bf16 else (f32(K), f32(V))
    for a in range(H):
        s = float(f32(q)[0, a].astype(np.float64) @ Kr[0, a // 2].astype(np.float64))
        assert np.abs(got[a] - np.exp(s) / (1 + np.exp(s)) * Vr[0, a // 2]).max() < 1e-4


@pytest.mark.parametrize("bf16,form", [(0, 1), (1, 2)])
def test_the_sink_takes_weight_and_has_no_value(hip_ctx, bf16, form):
    """All scores far below zero: the unit sink owns the denominator and the output shrinks to nothing; without a sink the same rows are plain softmax averages;
    a per-head sink logit shifts the balance."""
    H, G, dim, vd, T = 2, 2, 16, 16, 48
    rng = np.random.default_rng(9)
    q, K, V = qkv(rng, T, H, G, dim, vd)
    K[:] = 0.0
    K[..., 0] = -1.0
    q[:] = 0.0
    q[..., 0] = 12.0                 # every score is -12
    V = np.abs(V) + 1.0
    mx = {"heads": H, "kv_heads": G, "scale": 1.0}
    unit = attention(hip_ctx, q, K, V, mx, 0, sinks="unit", bf16=bf16, form=form)
    none = attention(hip_ctx, q, K, V, mx, 0, sinks=None, bf16=bf16, form=form)
    big = attention(hip_ctx, q, K, V, mx, 0, sinks=np.array([-12.0, -30.0]), bf16=bf16, form=form)
    Vr = O.to_bf16(V) if bf16 else f32(V)
    assert np.abs(unit).max() < 48 * np.exp(-12.0) * Vr.max() * 1.01
    for t in (0, 7, 47):
        mean = Vr[:t + 1].mean(0)
        assert np.abs(none[t] - mean).max() < 1e-4 * mean.max()
        assert np.abs(big[t, 0] - mean[0] * (t + 1) / (t + 2)).max() < 1e-4 * mean.max()   # a sink as heavy as one key
        assert np.abs(big[t, 1] - mean[1]).max() < 1e-4 * mean.max()                        # a sink too light to matter


def test_score_cap_bounds_a_huge_score(hip_ctx):
    """cap * tanh(s / cap): two keys with scores 400 and 40 end at cap and cap * tanh(40 / cap) -- near a tie under a small cap -- where plain softmax would give
    the first everything"""
    H, G, dim, vd, T = 1, 1, 8, 8, 3
    K, V, q = np.zeros((T, 1, dim)), np.zeros((T, 1, vd)), np.zeros((T, 1, dim))
    K[0, 0, 0], K[1, 0, 0], q[2, 0, 0] = 20.0, 2.0, 20.0
    V[0], V[1] = 1.0, -1.0
    for bf16, form in ((0, 1), (1, 1)):
        for cap in (5.0, 50.0):
            mx = {"heads": 1, "kv_heads": 1, "scale": 1.0, "softcap": cap}
            got = attention(hip_ctx, q, K, V, mx, 0, bf16=bf16, form=form)[2, 0, 0]
            s = cap * np.tanh(np.array([400.0, 40.0, 0.0]) / cap)
            e = np.exp(s - s.max())
            want = (e[0] - e[1]) / (e.sum() + np.exp(-s.max()))
            assert abs(got - want) < 1e-5, (cap, got, want)


RET = [(2, 8, 8, 5, 0), (3, 16, 24, 70, 0), (1, 64, 64, 200, 0), (4, 24, 8, 129, 0), (2, 128, 128, 64, 0), (2, 8, 40, 33, 50), (5, 12, 20, 1, 9), (2, 96, 72, 150, 30),
       (1, 136, 16, 70, 0), (1, 100, 128, 65, 3)]


@pytest.mark.parametrize("H,dim,vd,T,start", RET)
@pytest.mark.parametrize("form", [1, 2, 3])
def test_retention_both_forms_against_the_recurrence(hip_ctx, H, dim, vd, T, start, form):
    rng = np.random.default_rng(H + T)
    q, k, v = rng.standard_normal((T, H, dim)), rng.standard_normal((T, H, dim)) / np.sqrt(dim), rng.standard_normal((T, H, vd))
    decay = np.array([0.9, 0.999, 0.5, 0.9375, 1.0][:H])
    state = rng.standard_normal((H, dim, vd)) if start else np.full((H, dim, vd), np.nan)   # at position 0 whatever the state holds is ignored
    want, S = O.retention_core(f32(q), f32(k), f32(v), decay, f32(state) if start else None)
    got, gs = retention(hip_ctx, q, k, v, decay, state, start, form)
    assert np.isfinite(got).all() and np.isfinite(gs).all()
    assert np.abs(got - want).max() < 3e-5 * np.abs(want).max() and np.abs(gs - S).max() < 3e-5 * np.abs(S).max()


@pytest.mark.parametrize("form", [1, 2, 3])
def test_retention_state_carries_a_far_token_through_portions(hip_ctx, form):
    """One early token writes a large outer product into a slowly decaying head; 500 positions later a query along its key reads its value back, scaled by
    decay^distance -- across portions of 64, 1, 2, 200, ... rows that hand the state on.  The fast head has forgotten it."""
    H, dim, vd, T = 2, 16, 16, 520
    rng = np.random.default_rng(2)
    q, k, v = rng.standard_normal((T, H, dim)) * 0.01, rng.standard_normal((T, H, dim)) * 0.01, rng.standard_normal((T, H, vd)) * 0.01
    decay = np.array([0.999, 0.9])
    k[5, :, :] = 0.0
    k[5, :, 2] = 10.0
    v[5] = 7.0 + np.arange(vd)
    q[505, :, :] = 0.0
    q[505, :, 2] = 10.0
    want, _ = O.retention_core(f32(q), f32(k), f32(v), decay)
    assert np.abs(want[505, 0] - 100.0 * 0.999 ** 500 * v[5, 0]).max() < 0.05 and np.abs(want[505, 1]).max() < 2e-2
    state, at, rows = np.zeros((H, dim, vd)), 0, []
    for n in (64, 1, 2, 200, 63, 65, 1, 1, 123):
        o, state = retention(hip_ctx, q[at:at + n], k[at:at + n], v[at:at + n], decay, state, at, form)
        rows.append(o)
        at += n
    got = np.concatenate(rows)
    assert at == T and np.abs(got - want).max() < 3e-5 * np.abs(want).max()
