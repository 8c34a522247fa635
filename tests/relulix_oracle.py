"""A plain, slow statement of the Relulix design in float64 NumPy: one function per mechanism, whole sequences at a time, no cache, no batching.

It shares no code with the engine or with uzu_amd.relulix (which only reads and writes files): configurations and weights for the tests are made here.
Equations, for a sequence of T positions (position 0 first), width d; `rms(u) = u / sqrt(mean(u^2) + eps)`:

  embedding          x_t = E[token_t] * s_in
  norm               n(x) = g * rms(x)                      one gain g for all coordinates
  rotation           on the first R coordinates of a head: (a_i, a_(i+R/2)) <- (a_i c - a_(i+R/2) s, a_(i+R/2) c + a_i s),  angle = t * f_i, f_i = base^(-2i/R);
                     scaled frequencies (factor F, original length L, fast b_f, slow b_s): D(b) = R ln(L / (2 pi b)) / (2 ln base),
                     lo = max(floor D(b_f), 0), hi = min(ceil D(b_s), R - 1), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
                     f_i <- f_i / F * r_i + f_i (1 - r_i), and c, s are multiplied by 0.1 ln F + 1
  retention, head a  S_t = lambda_a S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t,  k scaled by dim^(-1/2) behind its rotation,  S_(-1) = 0;
                     out = W_o (concat_a rms(o_t[a]) * silu(W_g h_t))
  attention, head a  key / value head floor(a / (H / G)); s_tj = cap * tanh(scale <q_t, k_j> / cap) for 0 <= t - j < window;
                     p_tj = exp(s_tj) / (1 + sum_j' exp(s_tj'));  out = W_o concat_a sum_j p_tj v_j;  a sharing layer reads another layer's k_j, v_j
  experts            z = W_r h + b_r; the `top` largest z win, weights = softmax over the winners' z;
                     expert e: g = min(W_gate h, lim), u = clamp(W_up h, -lim, lim), W_down (g * sigmoid(1.702 g) * (u + 1))
  layer              h = n(x);  x <- x + (mixer(h) + experts(h))
  logits             = W_head n_final(x)
"""
import json
import os

import numpy as np

F = np.float64


def to_bf16(a):
    """values of `a` rounded to bf16 (round to nearest even), as float32"""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32) << 16
    return r.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def bf16_bits(a):
    return (to_bf16(a).view(np.uint32) >> 16).astype(np.uint16)


# ------------------------------------------------------------------------------------------------ mechanisms
def unit_rms(u, eps):
    return u / np.sqrt((u * u).mean(-1, keepdims=True) + eps)


def scalar_norm(x, g, eps):
    return unit_rms(x.astype(F), eps) * F(g)


def frequencies(rot):
    """the R / 2 angular frequencies of a rotation and the factor on cos / sin"""
    R, base = int(rot["dims"]), F(rot["base"])
    i = np.arange(R // 2, dtype=F)
    f = base ** (-2.0 * i / R)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, L = F(sc["factor"]), F(sc["original"])
    D = lambda b: R * np.log(L / (2.0 * np.pi * F(b))) / (2.0 * np.log(base))
    lo = max(np.floor(D(sc["fast"])), 0.0)
    hi = min(np.ceil(D(sc["slow"])), R - 1.0)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * np.log(factor) + 1.0


def rotate(a, positions, rot):
    """a [T, heads, dim]: the first R coordinates of every head turn by the angle of the row's position"""
    R = int(rot["dims"])
    f, m = frequencies(rot)
    ang = np.asarray(positions, dtype=F)[:, None] * f[None, :]
    c, s = (np.cos(ang) * m)[:, None, :], (np.sin(ang) * m)[:, None, :]
    out = a.astype(F).copy()
    u, v = a[..., :R // 2].astype(F), a[..., R // 2:R].astype(F)
    out[..., :R // 2] = u * c - v * s
    out[..., R // 2:R] = v * c + u * s
    return out


def silu(z):
    return z / (1.0 + np.exp(-z))


def retention_core(q, k, v, decay, state=None):
    """q, k [T, heads, dim], v [T, heads, vdim] (k already scaled); returns (o [T, heads, vdim], the state behind the last position [heads, dim, vdim])"""
    T, H, dim = q.shape
    S = np.zeros((H, dim, v.shape[2]), dtype=F) if state is None else state.astype(F).copy()
    o = np.zeros((T, H, v.shape[2]), dtype=F)
    for t in range(T):
        for a in range(H):
            S[a] = F(decay[a]) * S[a] + np.outer(k[t, a], v[t, a])
            o[t, a] = S[a].T @ q[t, a]
    return o, S


def retention(h, W, mx, eps, start=0, state=None):
    """h [T, d] at positions start ..; W: q, k, v, g, o matrices; returns (out [T, d], state)"""
    H, dim, vd = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    T = h.shape[0]
    pos = np.arange(start, start + T)
    q = rotate((h @ W["q"].astype(F).T).reshape(T, H, dim), pos, mx["rot"])
    k = rotate((h @ W["k"].astype(F).T).reshape(T, H, dim), pos, mx["rot"]) * F(dim) ** -0.5
    v = (h @ W["v"].astype(F).T).reshape(T, H, vd)
    o, S = retention_core(q, k, v, mx["decay"], state)
    o = unit_rms(o, eps).reshape(T, H * vd) * silu(h @ W["g"].astype(F).T)
    return o @ W["o"].astype(F).T, S


def attention_keys_values(h, W, mx, start=0):
    """keys (rotated) [T, G, dim] and values [T, G, vdim] of rows at positions start .."""
    G, dim, vd = int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    T = h.shape[0]
    k = (h @ W["k"].astype(F).T + W["k.b"].astype(F)).reshape(T, G, dim)
    v = (h @ W["v"].astype(F).T + W["v.b"].astype(F)).reshape(T, G, vd)
    return rotate(k, np.arange(start, start + T), mx["rot"]), v


def attention_core(q, K, V, mx, start=0):
    """q [T, H, dim] (rotated) at positions start ..; K [start + T, G, dim], V [start + T, G, vdim]: capped scores, window, one in the denominator"""
    H, G = int(mx["heads"]), int(mx["kv_heads"])
    window = int((mx.get("mask") or {}).get("size") or 0)
    cap = F(mx.get("softcap") or 0.0)
    scale = F(mx["scale"])
    T = q.shape[0]
    out = np.zeros((T, H, V.shape[2]), dtype=F)
    for i in range(T):
        t = start + i
        lo = max(0, t - window + 1) if window else 0
        for a in range(H):
            g = a // (H // G)
            s = (K[lo:t + 1, g] @ q[i, a]) * scale
            if cap:
                s = cap * np.tanh(s / cap)
            m = max(s.max(), 0.0)
            e = np.exp(s - m)
            out[i, a] = (e / (np.exp(-m) + e.sum())) @ V[lo:t + 1, g]
    return out


def attention(h, W, mx, K, V, start=0):
    """h [T, d]; K, V hold positions 0 .. start + T - 1 (the layer's own or another layer's)"""
    H, dim = int(mx["heads"]), int(mx["dim"])
    T = h.shape[0]
    q = rotate((h @ W["q"].astype(F).T + W["q.b"].astype(F)).reshape(T, H, dim), np.arange(start, start + T), mx["rot"])
    o = attention_core(q, K, V, mx, start)
    return o.reshape(T, -1) @ W["o"].astype(F).T


def route(h, w_router, b_router, top):
    """ids [T, top] by falling logit (ties: the lower index), weights = softmax over the winners' logits"""
    z = h @ w_router.astype(F).T + b_router.astype(F)
    ids = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zw = np.take_along_axis(z, ids, -1)
    e = np.exp(zw - zw.max(-1, keepdims=True))
    return ids, e / e.sum(-1, keepdims=True)


def expert(h, gate, up, down, limit):
    g = np.minimum(h @ gate.astype(F).T, limit)
    u = np.clip(h @ up.astype(F).T, -limit, limit)
    return (g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)) @ down.astype(F).T


def experts_mlp(h, W, ml):
    top, limit = int(ml["router"]["top"]), F(ml["expert"]["limit"])
    ids, wts = route(h, W["router"], W["router.b"], top)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            out[t] += wts[t, j] * expert(h[t:t + 1], W[f"e{e}.gate"], W[f"e{e}.up"], W[f"e{e}.down"], limit)[0]
    return out


# ------------------------------------------------------------------------------------------------ the whole model
def sub(W, prefix):
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def forward(cfg, W, tokens, layers_out=None):
    """logits [T, vocab] of a whole sequence from position 0; layers_out (a list) receives the residual rows behind every layer"""
    eps = F(cfg["norm"]["eps"])
    x = W["embed"].astype(F)[np.asarray(tokens)] * F(cfg["embedding"]["scale"])
    kv = {}
    for i, lc in enumerate(cfg["layers"]):
        mx = lc["mixer"]
        h = scalar_norm(x, W[f"l{i}.norm1"], eps)
        Wm = sub(W, f"l{i}.mix.")
        if lc["type"] == "retention":
            y, _ = retention(h, Wm, mx, eps)
        else:
            if mx.get("kv_from") is None:
                kv[i] = attention_keys_values(h, Wm, mx)
            K, V = kv[i if mx.get("kv_from") is None else int(mx["kv_from"])]
            y = attention(h, Wm, mx, K, V)
        if lc.get("mlp") is not None:
            y = y + experts_mlp(h, sub(W, f"l{i}.mlp."), lc["mlp"])
        x = x + y
        if layers_out is not None:
            layers_out.append(x.copy())
    return scalar_norm(x, W["final.norm"], eps) @ W["head"].astype(F).T


def greedy(cfg, W, prompt, steps):
    toks = list(prompt)
    for _ in range(steps):
        toks.append(int(np.argmax(forward(cfg, W, toks)[-1])))
    return toks[len(prompt):]


# ------------------------------------------------------------------------------------------------ configurations and weights for tests
def rot(dims, base=10000.0, scaling=None):
    r = {"dims": int(dims), "base": float(base)}
    if scaling:
        r["scaling"] = dict(scaling)
    return r


def attention_layer(heads, kv_heads, dim, vdim, rotation, window=None, scale=None, softcap=None, kv_from=None, mlp=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rotation, "scale": float(scale if scale is not None else dim ** -0.5)}
    if window:
        mx["mask"] = {"size": int(window)}
    if softcap:
        mx["softcap"] = float(softcap)
    if kv_from is not None:
        mx["kv_from"] = int(kv_from)
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def retention_layer(heads, dim, vdim, rotation, decay, mlp=None):
    assert len(decay) == heads
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "rot": rotation, "decay": [float(x) for x in decay]}, "mlp": mlp}


def moe(experts, top, ff, limit=7.0):
    return {"kind": "moe", "expert": {"ff": int(ff), "limit": float(limit)}, "router": {"experts": int(experts), "top": int(top)}}


def config(vocab, width, layers, eps=1e-6, embed_scale=None):
    return {"architecture": "Relulix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": float(embed_scale if embed_scale is not None else width ** 0.5)},
            "layers": layers}


def weights(cfg, seed, logit_gain=1.0):
    """bf16-representable float32 tensors of every name the configuration implies"""
    rng = np.random.default_rng(seed)
    d, V = cfg["width"], cfg["vocab"]
    W = {}

    def lin(name, n, k, gain=1.0, bias=False):
        W[name] = to_bf16(rng.standard_normal((n, k)) * gain / np.sqrt(k))
        if bias:
            W[name + ".b"] = to_bf16(rng.standard_normal(n) * 0.2)

    W["embed"] = to_bf16(rng.standard_normal((V, d)) / cfg["embedding"]["scale"])
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        W[p + "norm1"] = to_bf16(np.float32(0.8 + 0.4 * rng.random())).reshape(())
        H, dim, vd = mx["heads"], mx["dim"], mx["vdim"]
        if lc["type"] == "retention":
            lin(p + "mix.q", H * dim, d, 1.5)
            lin(p + "mix.k", H * dim, d, 1.5)
            lin(p + "mix.v", H * vd, d)
            lin(p + "mix.g", H * vd, d, 2.0)
            lin(p + "mix.o", d, H * vd)
        else:
            G = mx["kv_heads"]
            lin(p + "mix.q", H * dim, d, 2.0, bias=True)
            if mx.get("kv_from") is None:
                lin(p + "mix.k", G * dim, d, 2.0, bias=True)
                lin(p + "mix.v", G * vd, d, bias=True)
            lin(p + "mix.o", d, H * vd)
        ml = lc.get("mlp")
        if ml is not None:
            ff = ml["expert"]["ff"]
            for e in range(ml["router"]["experts"]):
                lin(f"{p}mlp.e{e}.gate", ff, d, 1.5)
                lin(f"{p}mlp.e{e}.up", ff, d, 1.5)
                lin(f"{p}mlp.e{e}.down", d, ff)
            lin(p + "mlp.router", ml["router"]["experts"], d, 2.0, bias=True)
    W["final.norm"] = to_bf16(np.float32(0.8 + 0.4 * rng.random())).reshape(())
    lin("head", V, d, logit_gain)
    return W


def write_model_dir(path, cfg, W):
    """config.json + model.safetensors (bf16) in the design's layout, written with nothing but the file format"""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name in sorted(W):
        b = bf16_bits(W[name]).tobytes()
        header[name] = {"dtype": "BF16", "shape": list(np.shape(W[name])), "data_offsets": [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(len(hj).to_bytes(8, "little") + hj + b"".join(blobs))


def logit_error(got, want):
    """per row: RMS over the vocabulary of the difference with its mean taken off, relative to the RMS of the centred expected row"""
    d = np.asarray(got, dtype=F) - np.asarray(want, dtype=F)
    d = d - d.mean(-1, keepdims=True)
    w = np.asarray(want, dtype=F)
    w = w - w.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / np.sqrt((w * w).mean(-1) + 1e-30)
