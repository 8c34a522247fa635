"""Lazolix: a decoder-only design with an f32 residual stream (include/uzu_model_desc.h: ``f32_stream``), read from its own ``config.json`` schema.

A model directory holds ``config.json`` (``"architecture": "Lazolix"``) and ``model.safetensors`` (bf16 tensors, linear weights ``[out, in]``).  This module
turns it into the engine's :class:`uzu_amd.desc.ModelBundle` -- the same object every other model becomes, so `HipModel`, states, batched steps, sampling and
the generate loop are the engine's own -- and writes such a directory from a configuration and random weights (tests, benchmarks).

The design, in this package's terms (all sizes and constants come from ``config.json`` or from tensor shapes, nothing is assumed):

* ``embed [vocab, width]`` is the input table and, behind ``final.norm``, the read-out.
* ``layers[i]``: ``x <- x + mixer(shift(norm1(x)))``, then (unless ``mlp`` is null) ``x <- x + mlp(norm2(x))``, then the depth mix
  ``x <- sum_j dwa[j] * X_j`` over the embedding rows X_0 and every layer's own result X_1 .. X_(i+1).
* norms are dynamic-tanh norms: ``tanh(alpha * x) * w + b`` (tensors ``<name>``, ``<name>.alpha``, ``<name>.b``).
* token shift (``l<i>.shift``): the mixer reads ``h + (h_prev - h) * shift`` with ``h_prev`` the previous position's normalised row (zeros at position 0).
* mixer ``latent_attention``: queries ``mix.q``, a cached latent ``c = RMSNorm(mix.dkv h) * mix.dkv.norm`` of ``kv_rank`` numbers per token, per-head keys
  ``mix.uk c`` and values ``mix.uv c``, scores ``q.k * scale`` over a causal sliding window of ``mask.size`` positions (none: all earlier positions), a
  per-head sink logit ``mix.sink`` in the softmax denominator, output ``mix.o``.  ``kv_from: j`` = no ``mix.dkv`` of its own: layer j's cached latents.
* ``mlp.kind = dense``: ``down(relu(up h + b)^2) + b``;  ``moe``: router scores = softmax over ``experts + identity`` outputs, the ``top`` largest
  ``score + correction`` win, weights = winners' scores / their sum; experts ``down(silu(gate h) * up h)`` without biases; identity experts return ``h``.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import desc as D
from .design_tensors import Tensors as _Tensors, bits_to_f32 as _bits_to_f32, f32_to_bf16_bits as _f32_to_bf16_bits, full_linear as _full

ARCHITECTURE = "Lazolix"


def _dyn_tanh(t: _Tensors, name: str, width: int, eps: float) -> D.NormWeights:
    alpha = float(t.f32(name + ".alpha").reshape(-1)[0])
    return D.NormWeights(present=True, epsilon=eps, scales=t.f32(name, (width,)), biases=t.f32(name + ".b", (width,)) if t.has(name + ".b") else None,
                         kind=D.NORM_DYNAMIC_TANH, alpha=alpha)


def load(path: str, cfg: dict, st, max_context_length: Optional[int], name: Optional[str], errors) -> D.ModelBundle:
    """config.json (already parsed) + model.safetensors (uzu_amd.loader.SafeTensors) -> ModelBundle.  `errors` = (ModelFormatError, UnsupportedModelError)."""
    bad, unsupported = errors
    t = _Tensors(st, bad)
    vocab, width = t.shape("embed")
    for key, have in (("vocab", vocab), ("width", width)):
        if cfg.get(key) is not None and int(cfg[key]) != have:
            raise bad(f"config.json: {key} = {cfg[key]} but 'embed' is {[vocab, width]}")
    eps = float((cfg.get("norm") or {}).get("eps", 1e-6))
    layer_cfgs = cfg.get("layers")
    if not isinstance(layer_cfgs, list) or not layer_cfgs:
        raise bad("config.json: 'layers' must be a non-empty array")
    layers: List[D.LayerWeights] = []
    for i, lc in enumerate(layer_cfgs):
        p = f"l{i}."
        if lc.get("type") != "latent_attention":
            raise unsupported(f"config.json: layers[{i}].type = {lc.get('type')!r}: this design's mixer here is 'latent_attention'")
        mx = lc.get("mixer") or {}
        q_rows = t.shape(p + "mix.q")[0]
        heads = int(mx["heads"]) if mx.get("heads") is not None else int(t.shape(p + "mix.sink")[0])
        dim = int(mx["dim"]) if mx.get("dim") is not None else q_rows // heads
        uv_rows, rank_t = t.shape(p + "mix.uv")
        rank = int(mx["kv_rank"]) if mx.get("kv_rank") is not None else int(rank_t)
        vdim = int(mx["vdim"]) if mx.get("vdim") is not None else uv_rows // heads
        kv_from = mx.get("kv_from")
        mask = mx.get("mask") or {}
        window = int(mask.get("size") or 0)
        scale = float(mx["scale"]) if mx.get("scale") is not None else float(dim) ** -0.5
        if kv_from is not None and not (0 <= int(kv_from) < i):
            raise bad(f"config.json: layers[{i}].mixer.kv_from = {kv_from} must name an earlier layer")
        lw = D.LayerWeights(
            mixer_kind=D.MIXER_LATENT_ATTENTION, hidden_dim=0, activation=D.ACT_RELU_SQUARED,
            pre_mixer_norm=_dyn_tanh(t, p + "norm1", width, eps), pre_mlp_norm=D.ABSENT_NORM, up_projection=None, down_projection=None,
            num_heads=heads, num_groups=1, head_dim=dim, attention_scale=scale,
            qkv_projection=_full(t.bits(p + "mix.q", (heads * dim, width))), out_projection=_full(t.bits(p + "mix.o", (width, heads * vdim))),
            sliding_window_size=window, sinks=t.bits(p + "mix.sink", (heads,)) if t.has(p + "mix.sink") else None,
            kv_source_layer_index=None if kv_from is None else int(kv_from),
            latent_rank=rank, value_head_dim=vdim,
            latent_up_keys=_full(t.bits(p + "mix.uk", (heads * dim, rank))), latent_up_values=_full(t.bits(p + "mix.uv", (heads * vdim, rank))),
            token_shift=t.f32(p + "shift", (width,)) if t.has(p + "shift") else None,
            depth_weights=t.f32(p + "dwa", (i + 2,)) if t.has(p + "dwa") else None)
        if kv_from is None:
            lw.latent_down = _full(t.bits(p + "mix.dkv", (rank, width)))
            lw.latent_norm = D.NormWeights(present=True, epsilon=eps, scales=t.f32(p + "mix.dkv.norm", (rank,)))
        ml = lc.get("mlp")
        if ml is None:
            lw.no_mlp = True
        else:
            lw.pre_mlp_norm = _dyn_tanh(t, p + "norm2", width, eps)
            kind = ml.get("kind")
            if kind == "dense":
                ff = int(ml["ff"]) if ml.get("ff") is not None else int(t.shape(p + "mlp.up")[0])
                lw.hidden_dim, lw.mlp_plain = ff, True
                lw.up_projection = _full(t.bits(p + "mlp.up", (ff, width)), t.bits(p + "mlp.up.b", (ff,)) if t.has(p + "mlp.up.b") else None)
                lw.down_projection = _full(t.bits(p + "mlp.down", (width, ff)), t.bits(p + "mlp.down.b", (width,)) if t.has(p + "mlp.down.b") else None)
            elif kind == "moe":
                r = ml.get("router") or {}
                experts, identity, top = int(r["experts"]), int(r.get("identity") or 0), int(r["top"])
                routed = experts  # `experts` counts the experts that have tensors; the router has experts + identity outputs
                ff = int((ml.get("expert") or {}).get("ff") or (t.shape(p + "mlp.e0.gate")[0] if routed else 0))
                outputs = t.shape(p + "mlp.router")[0]
                if outputs != routed + identity:
                    raise bad(f"config.json: layers[{i}].mlp.router: {routed} experts + {identity} identity experts, but '{p}mlp.router' has {outputs} rows")
                if not 0 < top <= outputs:
                    raise bad(f"config.json: layers[{i}].mlp.router.top = {top} of {outputs} router outputs")
                w13 = np.empty((routed, 2 * ff, width), dtype=np.uint16) if routed else None
                w2 = np.empty((routed, width, ff), dtype=np.uint16) if routed else None
                for e in range(routed):  # the engine's expert layout: per expert [up rows ; gate rows] and the down matrix
                    w13[e, :ff] = t.bits(f"{p}mlp.e{e}.up", (ff, width))
                    w13[e, ff:] = t.bits(f"{p}mlp.e{e}.gate", (ff, width))
                    w2[e] = t.bits(f"{p}mlp.e{e}.down", (width, ff))
                lw.moe = D.MoeWeights(num_routed_experts=routed, num_active_experts=top, expert_hidden_dim=ff, router_weights=t.bits(p + "mlp.router", (outputs, width)),
                                      router_biases=None, w13=w13, w2=w2, up_biases=None, down_biases=None, router_renorm=False, gating_sel=2,
                                      routing=D.MOE_ROUTE_SCORES, num_identity_experts=identity,
                                      selection_bias=t.f32(p + "mlp.correction", (outputs,)) if t.has(p + "mlp.correction") else None)
            else:
                raise unsupported(f"config.json: layers[{i}].mlp.kind = {kind!r} (dense | moe)")
        layers.append(lw)
    for i, lw in enumerate(layers):
        j = lw.kv_source_layer_index
        if j is not None and (layers[j].kv_source_layer_index is not None or layers[j].latent_rank != lw.latent_rank):
            raise bad(f"config.json: layers[{i}].mixer.kv_from = {j}: that layer must own latents of the same kv_rank")
    bundle = D.ModelBundle(name=name or os.path.basename(os.path.normpath(path)), vocab_size=int(vocab), model_dim=int(width),
                           max_context_length=int(max_context_length or cfg.get("max_context_length") or 4096), rope=D.RopeConfig(),
                           embedding=_full(t.bits("embed", (vocab, width))), output_norm=_dyn_tanh(t, "final.norm", width, eps), layers=layers, tied_embeddings=True,
                           f32_stream=True, architecture=ARCHITECTURE)
    st.assert_all_consumed()
    return bundle


# ------------------------------------------------------------------------------------------------ writer: a configuration + random weights -> a model directory
def random_tensors(cfg: dict, seed: int = 0) -> Dict[str, np.ndarray]:
    """f32 values (already bf16-representable) of every tensor a configuration names, from a seeded generator: linear weights ~ N(0, 1/in), norm weights near 1,
    shifts in (0, 1), depth weights near an average, sinks / corrections small."""
    rng = np.random.default_rng(seed)
    rb = lambda a: _bits_to_f32(_f32_to_bf16_bits(np.asarray(a, dtype=np.float32)))
    vocab, width = int(cfg["vocab"]), int(cfg["width"])
    out: Dict[str, np.ndarray] = {}

    def lin(name, n, k, bias=False, gain=1.0):
        out[name] = rb(rng.standard_normal((n, k)) * gain / np.sqrt(k))
        if bias:
            out[name + ".b"] = rb(rng.standard_normal(n) * 0.1)

    def norm(name):
        out[name] = rb(1.0 + 0.1 * rng.standard_normal(width))
        out[name + ".b"] = rb(0.05 * rng.standard_normal(width))
        out[name + ".alpha"] = rb(np.float32(0.5 + 0.5 * rng.random())).reshape(())

    out["embed"] = rb(rng.standard_normal((vocab, width)))
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        H, dim, vd, rank = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"]), int(mx["kv_rank"])
        norm(p + "norm1")
        lin(p + "mix.q", H * dim, width, gain=2.0)
        if mx.get("kv_from") is None:
            lin(p + "mix.dkv", rank, width)
            out[p + "mix.dkv.norm"] = rb(1.0 + 0.1 * rng.standard_normal(rank))
        lin(p + "mix.uk", H * dim, rank, gain=2.0)
        lin(p + "mix.uv", H * vd, rank)
        out[p + "mix.sink"] = rb(rng.standard_normal(H))
        lin(p + "mix.o", width, H * vd)
        out[p + "shift"] = rb(rng.random(width))
        out[p + "dwa"] = rb(1.0 / (i + 2) + 0.2 * rng.standard_normal(i + 2))
        ml = lc.get("mlp")
        if ml is None:
            continue
        norm(p + "norm2")
        if ml["kind"] == "dense":
            lin(p + "mlp.up", int(ml["ff"]), width, bias=True)
            lin(p + "mlp.down", width, int(ml["ff"]), bias=True)
        else:
            r = ml["router"]
            E, I, ff = int(r["experts"]), int(r.get("identity") or 0), int(ml["expert"]["ff"])
            for e in range(E):
                lin(f"{p}mlp.e{e}.gate", ff, width)
                lin(f"{p}mlp.e{e}.up", ff, width)
                lin(f"{p}mlp.e{e}.down", width, ff)
            lin(p + "mlp.router", E + I, width, gain=2.0)
            out[p + "mlp.correction"] = rb(0.05 * rng.standard_normal(E + I))
    norm("final.norm")
    return out


def save(path: str, cfg: dict, tensors: Dict[str, np.ndarray]):
    """Write config.json + model.safetensors (every tensor as bf16) in this design's layout."""
    from .loader import write_safetensors
    os.makedirs(path, exist_ok=True)
    full = dict(cfg)
    full["architecture"] = ARCHITECTURE
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(full, f, indent=1, sort_keys=True)
    write_safetensors(os.path.join(path, "model.safetensors"), {k: ("BF16", _f32_to_bf16_bits(v).reshape(np.shape(v))) for k, v in tensors.items()}, {})


def layer_config(heads: int, dim: int, vdim: int, kv_rank: int, window: Optional[int], scale: Optional[float] = None, kv_from: Optional[int] = None,
                 mlp: Optional[dict] = None) -> dict:
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": float(scale if scale is not None else dim ** -0.5)}
    if window:
        mixer["mask"] = {"size": int(window)}
    if kv_from is not None:
        mixer["kv_from"] = int(kv_from)
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def dense_mlp(ff: int) -> dict:
    return {"kind": "dense", "ff": int(ff)}


def moe_mlp(experts: int, top: int, ff: int, identity: int = 0) -> dict:
    return {"kind": "moe", "expert": {"ff": int(ff)}, "router": {"experts": int(experts), "identity": int(identity), "top": int(top)}}
