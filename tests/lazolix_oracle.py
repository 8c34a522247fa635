"""A plain, slow statement of the Lazolix design in float64 NumPy: one function per mechanism, whole sequences at a time, no cache, no batching.

It shares no code with the engine or with uzu_amd.lazolix (which only reads and writes files): configurations and weights for the tests are made here.
Equations, for a sequence of T positions (position 0 first), width d:

  dyn_tanh(x)        = tanh(alpha x) * w + b
  shift(h)_t         = h_t + (h_(t-1) - h_t) * mu,   h_(-1) = 0
  latent c_t         = g * u_t / sqrt(mean(u_t^2) + eps),   u_t = W_dkv h_t
  head a: k_j = W_uk[a] c_j, v_j = W_uv[a] c_j, s_tj = scale <q_t[a], k_j> for t - window < j <= t (no window: 0 <= j <= t)
          p_tj = exp(s_tj) / (sum_j' exp(s_tj') + exp(sink_a)),   out_t[a] = sum_j p_tj v_j
  dense  = W_down relu(W_up h + b_up)^2 + b_down
  moe    : z = W_r h, s = softmax(z) over experts + identity; the `top` largest s + correction win; weight = s / (sum of the winners' s + 1e-20);
           expert e: W_down[e] (silu(W_gate[e] h) * (W_up[e] h)); an identity expert returns h
  layer i: y = x + W_o attention(shift(dyn_tanh_1(x)));  X_(i+1) = y + mlp(dyn_tanh_2(y)) (or y);  x <- sum_(j <= i+1) dwa[j] X_j
  logits = embed dyn_tanh_final(x)
"""
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
def dyn_tanh(x, w, b, alpha):
    return np.tanh(F(alpha) * x.astype(F)) * w.astype(F) + (0.0 if b is None else b.astype(F))


def token_shift(h, mu, prev=None):
    """h [T, d]; prev = the normalised row of the position before h[0] (None: position 0).  Returns (shifted rows, the last unshifted row)."""
    before = np.concatenate([np.zeros_like(h[:1]) if prev is None else prev[None].astype(F), h[:-1]])
    return h + (before - h) * mu.astype(F), h[-1].copy()


def rms_latent(u, g, eps):
    return u / np.sqrt((u * u).mean(-1, keepdims=True) + eps) * g.astype(F)


def visible(t, j, window):
    return (j <= t) and (window == 0 or t - j < window)


def latent_attention(q, c, w_uk, w_uv, heads, scale, window, sinks, start=0):
    """q [T, heads * dim] for positions start .. start + T - 1, c [start + T, rank]; keys and values are expanded per head (the direct form)."""
    T = q.shape[0]
    dim = w_uk.shape[0] // heads
    vd = w_uv.shape[0] // heads
    k = (c @ w_uk.astype(F).T).reshape(-1, heads, dim)
    v = (c @ w_uv.astype(F).T).reshape(-1, heads, vd)
    out = np.zeros((T, heads, vd), dtype=F)
    for i in range(T):
        t = start + i
        js = [j for j in range(t + 1) if visible(t, j, window)]
        for a in range(heads):
            s = np.array([scale * (q[i, a * dim:(a + 1) * dim] @ k[j, a]) for j in js])
            m = max(s.max(), sinks[a]) if sinks is not None else s.max()
            e = np.exp(s - m)
            den = e.sum() + (np.exp(F(sinks[a]) - m) if sinks is not None else 0.0)
            out[i, a] = (e / den) @ v[js, a]
    return out.reshape(T, heads * vd)


def latent_core(qlat, c, heads, scale, window, sinks, start=0):
    """The same attention with keys = values = the latents themselves: qlat [T, heads * rank] -> [T, heads * rank]."""
    T, rank = qlat.shape[0], c.shape[1]
    out = np.zeros((T, heads, rank), dtype=F)
    for i in range(T):
        t = start + i
        js = [j for j in range(t + 1) if visible(t, j, window)]
        for a in range(heads):
            s = scale * (c[js].astype(F) @ qlat[i, a * rank:(a + 1) * rank].astype(F))
            m = max(s.max(), sinks[a]) if sinks is not None else s.max()
            e = np.exp(s - m)
            den = e.sum() + (np.exp(F(sinks[a]) - m) if sinks is not None else 0.0)
            out[i, a] = (e / den) @ c[js].astype(F)
    return out.reshape(T, heads * rank)


def dense_mlp(h, w_up, b_up, w_down, b_down):
    u = h @ w_up.astype(F).T + (0.0 if b_up is None else b_up.astype(F))
    return (np.maximum(u, 0.0) ** 2) @ w_down.astype(F).T + (0.0 if b_down is None else b_down.astype(F))


def route(h, w_router, correction, top):
    """-> ids [T, top] (descending choice score), weights [T, top]"""
    z = h @ w_router.astype(F).T
    s = np.exp(z - z.max(-1, keepdims=True))
    s /= s.sum(-1, keepdims=True)
    choice = s + (0.0 if correction is None else correction.astype(F))
    ids = np.argsort(-choice, axis=-1, kind="stable")[:, :top]
    w = np.take_along_axis(s, ids, -1)
    return ids, w / (w.sum(-1, keepdims=True) + 1e-20)


def moe_mlp(h, w_router, correction, experts, top):
    """experts: list of (gate, up, down) for the experts that have tensors; router rows beyond them are identity experts."""
    ids, w = route(h, w_router, correction, top)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(ids[t], w[t]):
            if e >= len(experts):
                out[t] += we * h[t]
            else:
                g, u, dn = (m.astype(F) for m in experts[e])
                a = g @ h[t]
                out[t] += we * (dn @ (a / (1.0 + np.exp(-a)) * (u @ h[t])))
    return out


def depth_mix(xs, w):
    return sum(F(w[j]) * xs[j] for j in range(len(xs)))


# ------------------------------------------------------------------------------------------------ the model
def forward(cfg, W, tokens, layers_out=None):
    """logits [T, vocab] of a whole sequence; layers_out (a list) receives what every layer hands on."""
    x = W["embed"][np.asarray(tokens)].astype(F)
    eps = cfg["norm"]["eps"]
    xs, latents = [x], {}
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        h = dyn_tanh(x, W[p + "norm1"], W.get(p + "norm1.b"), W[p + "norm1.alpha"])
        h, _ = token_shift(h, W[p + "shift"])
        q = h @ W[p + "mix.q"].astype(F).T
        if mx.get("kv_from") is None:
            latents[i] = rms_latent(h @ W[p + "mix.dkv"].astype(F).T, W[p + "mix.dkv.norm"], eps)
            c = latents[i]
        else:
            c = latents[mx["kv_from"]]
        window = (mx.get("mask") or {}).get("size") or 0
        a = latent_attention(q, c, W[p + "mix.uk"], W[p + "mix.uv"], mx["heads"], mx["scale"], window, W.get(p + "mix.sink"))
        y = x + a @ W[p + "mix.o"].astype(F).T
        ml = lc.get("mlp")
        if ml is not None:
            h2 = dyn_tanh(y, W[p + "norm2"], W.get(p + "norm2.b"), W[p + "norm2.alpha"])
            if ml["kind"] == "dense":
                y = y + dense_mlp(h2, W[p + "mlp.up"], W.get(p + "mlp.up.b"), W[p + "mlp.down"], W.get(p + "mlp.down.b"))
            else:
                r = ml["router"]
                experts = [(W[f"{p}mlp.e{e}.gate"], W[f"{p}mlp.e{e}.up"], W[f"{p}mlp.e{e}.down"]) for e in range(r["experts"])]
                y = y + moe_mlp(h2, W[p + "mlp.router"], W.get(p + "mlp.correction"), experts, r["top"])
        xs.append(y)
        x = depth_mix(xs, W[p + "dwa"])
        if layers_out is not None:
            layers_out.append(x.copy())
    hf = dyn_tanh(x, W["final.norm"], W.get("final.norm.b"), W["final.norm.alpha"])
    return hf @ W["embed"].astype(F).T


def greedy(cfg, W, prompt, steps):
    toks = list(prompt)
    out = []
    for _ in range(steps):
        t = int(np.argmax(forward(cfg, W, toks)[-1]))
        out.append(t)
        toks.append(t)
    return out


# ------------------------------------------------------------------------------------------------ configurations and weights of the tests
def layer(heads, dim, vdim, rank, window=None, scale=None, kv_from=None, mlp=None):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": float(dim ** -0.5 if scale is None else scale)}
    if window:
        mixer["mask"] = {"size": window}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=0):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}


def config(vocab, width, layers, eps=1e-6):
    return {"architecture": "Lazolix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def weights(cfg, seed, logit_gain=1.0):
    """bf16-representable float32 tensors by name.  Queries and key projections get a gain so that attention is not uniform (a wrong key or a window that is one
    off moves the logits), routers a gain so that choices have margins."""
    rng = np.random.default_rng(seed)
    V, d = cfg["vocab"], cfg["width"]
    W = {}

    def lin(name, n, k, gain=1.0, bias=False):
        W[name] = to_bf16(rng.standard_normal((n, k)) * gain / np.sqrt(k))
        if bias:
            W[name + ".b"] = to_bf16(rng.standard_normal(n) * 0.2)

    def norm(name):
        W[name] = to_bf16(1.0 + 0.2 * rng.standard_normal(d))
        W[name + ".b"] = to_bf16(0.1 * rng.standard_normal(d))
        W[name + ".alpha"] = to_bf16(np.float32(0.4 + 0.6 * rng.random())).reshape(())

    W["embed"] = to_bf16(rng.standard_normal((V, d)) * logit_gain)
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        H, dim, vd, r = mx["heads"], mx["dim"], mx["vdim"], mx["kv_rank"]
        norm(p + "norm1")
        lin(p + "mix.q", H * dim, d, gain=3.0)
        if mx.get("kv_from") is None:
            lin(p + "mix.dkv", r, d)
            W[p + "mix.dkv.norm"] = to_bf16(1.0 + 0.2 * rng.standard_normal(r))
        lin(p + "mix.uk", H * dim, r, gain=3.0)
        lin(p + "mix.uv", H * vd, r)
        W[p + "mix.sink"] = to_bf16(rng.standard_normal(H))
        lin(p + "mix.o", d, H * vd)
        W[p + "shift"] = to_bf16(rng.random(d))
        W[p + "dwa"] = to_bf16(1.0 / (i + 2) + 0.3 * rng.standard_normal(i + 2))
        ml = lc.get("mlp")
        if ml is None:
            continue
        norm(p + "norm2")
        if ml["kind"] == "dense":
            lin(p + "mlp.up", ml["ff"], d, bias=True)
            lin(p + "mlp.down", d, ml["ff"], bias=True)
        else:
            r_ = ml["router"]
            for e in range(r_["experts"]):
                lin(f"{p}mlp.e{e}.gate", ml["expert"]["ff"], d)
                lin(f"{p}mlp.e{e}.up", ml["expert"]["ff"], d)
                lin(f"{p}mlp.e{e}.down", d, ml["expert"]["ff"])
            lin(p + "mlp.router", r_["experts"] + r_.get("identity", 0), d, gain=4.0)
            W[p + "mlp.correction"] = to_bf16(0.05 * rng.standard_normal(r_["experts"] + r_.get("identity", 0)))
    norm("final.norm")
    return W


def write_model_dir(path, cfg, W):
    """config.json + model.safetensors (bf16) through the package's file writer (file format only, no arithmetic)."""
    import json
    import os
    from uzu_amd.loader import write_safetensors
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(path, "model.safetensors"), {k: ("BF16", bf16_bits(v).reshape(np.shape(v))) for k, v in W.items()}, {})


def logit_error(got, want):
    """rms over the vocabulary of the difference (means removed), relative to the rms of the expected logits: per row"""
    d = np.asarray(got, dtype=F) - np.asarray(want, dtype=F)
    d = d - d.mean(-1, keepdims=True)
    w = np.asarray(want, dtype=F)
    w = w - w.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / np.sqrt((w * w).mean())
