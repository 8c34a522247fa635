"""Relulix: a decoder-only design of parallel blocks over an f32 residual stream (include/uzu_model_desc.h: ``f32_stream``), read from its own ``config.json`` schema.

A model directory holds ``config.json`` (``"architecture": "Relulix"``) and ``model.safetensors`` (bf16 tensors, linear weights ``[out, in]``).  This module turns
it into the engine's :class:`uzu_amd.desc.ModelBundle` -- the object every other model becomes, so `HipModel`, states, batched steps, sampling and the generate loop
are the engine's own -- and writes such a directory from a configuration and random weights (tests, benchmarks).

The design, in this package's terms (every size comes from ``config.json`` or a tensor's shape, every constant that can differ between models from ``config.json``):

* ``x = embed[token] * embedding.scale``; the read-out is ``head`` behind ``final.norm``.
* norms (``l<i>.norm1``, ``final.norm``) are RMS norms with ONE gain: ``g * x / sqrt(mean(x^2) + norm.eps)`` (desc.NORM_RMS_SCALAR).
* ``layers[i]`` is a parallel block: ``h = norm1(x)``, ``x <- x + (mixer(h) + mlp(h))`` (``mlp`` null: the mixer alone).
* ``type: attention`` (desc.MIXER_ATTENTION): ``mix.q / k / v`` with biases ``.b`` (packed into one projection: queries | keys | values), ``heads`` query heads on
  ``kv_heads`` key / value heads of widths ``dim`` / ``vdim``, rotation of the first ``rot.dims`` coordinates of queries and keys (``rot.base``; ``rot.scaling``
  = YaRN frequencies), scores ``scale * q.k`` capped by ``softcap * tanh(s / softcap)``, a causal window of ``mask.size`` positions, one more ``exp(0)`` in the
  softmax denominator, ``mix.o``.  ``kv_from: j`` = no key / value projections: layer j's cached (rotated) keys and values.
* ``type: retention`` (desc.MIXER_RETENTION): ``mix.q / k / v / g`` without biases (packed: queries | keys | values | gate), rotation as above (no scaling), keys
  times ``dim^(-1/2)``, per head ``S <- decay S + k v^T``, ``o = S^T q``, ``o / rms(o) * silu(g h)``, ``mix.o``.
* ``mlp.kind = moe``: logits ``router h + router.b``, the ``top`` largest win with the softmax over the winners as weights; expert
  ``down(g * sigmoid(1.702 g) * (u + 1))`` with ``g = min(gate h, limit)``, ``u = clamp(up h, -limit, limit)``, no biases.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import numpy as np

from . import desc as D
from .design_tensors import Tensors as _Tensors, bits_to_f32 as _bits_to_f32, f32_to_bf16_bits as _f32_to_bf16_bits, full_linear as _full

ARCHITECTURE = "Relulix"
GATE_ALPHA = 1.702  # the sigmoid's slope in an expert's gate
UP_OFFSET = 1.0     # an expert's up branch enters the product as (u + 1)


def _rope(rot: dict, max_positions: int) -> D.RopeConfig:
    sc = rot.get("scaling")
    if not sc:
        return D.RopeConfig(kind=D.ROPE_UNSCALED, head_dim=int(rot["dims"]), max_sequence_length=max_positions, base=float(rot["base"]))
    return D.RopeConfig(kind=D.ROPE_YARN, head_dim=int(rot["dims"]), max_sequence_length=max_positions, base=float(rot["base"]), scaling_factor=float(sc["factor"]),
                        original_context_length=int(sc["original"]), beta_fast=float(sc["fast"]), beta_slow=float(sc["slow"]), truncate=True)


def _gain(t: _Tensors, name: str, eps: float) -> D.NormWeights:
    return D.NormWeights(present=True, epsilon=eps, kind=D.NORM_RMS_SCALAR, alpha=float(t.f32(name).reshape(-1)[0]))


def _packed(t: _Tensors, names: List[str], rows: List[int], width: int, biases: bool) -> D.LinearWeights:
    """several [out_i, width] matrices stacked into one projection (and their biases into one vector)"""
    w = np.concatenate([t.bits(n, (r, width)) for n, r in zip(names, rows)], axis=0)
    b = np.concatenate([t.bits(n + ".b", (r,)) for n, r in zip(names, rows)]) if biases else None
    return _full(np.ascontiguousarray(w), None if b is None else np.ascontiguousarray(b))


def load(path: str, cfg: dict, st, max_context_length: Optional[int], name: Optional[str], errors) -> D.ModelBundle:
    """config.json (already parsed) + model.safetensors (uzu_amd.loader.SafeTensors) -> ModelBundle.  `errors` = (ModelFormatError, UnsupportedModelError)."""
    bad, unsupported = errors
    t = _Tensors(st, bad)
    vocab, width = t.shape("embed")
    for key, have in (("vocab", vocab), ("width", width)):
        if cfg.get(key) is not None and int(cfg[key]) != have:
            raise bad(f"config.json: {key} = {cfg[key]} but 'embed' is {[vocab, width]}")
    eps = float((cfg.get("norm") or {}).get("eps", 1e-6))
    max_ctx = int(max_context_length or cfg.get("max_context_length") or 4096)
    layer_cfgs = cfg.get("layers")
    if not isinstance(layer_cfgs, list) or not layer_cfgs:
        raise bad("config.json: 'layers' must be a non-empty array")
    ropes: List[D.RopeConfig] = []

    def rope_index(rot: Optional[dict], dim: int, where: str) -> Optional[int]:
        if not rot or not int(rot.get("dims") or 0):
            return None
        dims = int(rot["dims"])
        if dims % 2 or dims > dim:
            raise bad(f"config.json: {where}.rot.dims = {dims}: an even number of at most dim = {dim} coordinates turns")
        r = _rope(rot, max_ctx)
        for i, have in enumerate(ropes):
            if have == r:
                return i
        ropes.append(r)
        return len(ropes) - 1

    layers: List[D.LayerWeights] = []
    for i, lc in enumerate(layer_cfgs):
        p, kind, mx = f"l{i}.", lc.get("type"), lc.get("mixer") or {}
        where = f"layers[{i}].mixer"
        if kind not in ("attention", "retention"):
            raise unsupported(f"config.json: layers[{i}].type = {kind!r} (attention | retention)")
        heads, dim, vdim = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
        ri = rope_index(mx.get("rot"), dim, where)
        lw = D.LayerWeights(
            mixer_kind=D.MIXER_ATTENTION if kind == "attention" else D.MIXER_RETENTION, hidden_dim=0, activation=D.ACT_SILU,
            pre_mixer_norm=_gain(t, p + "norm1", eps), pre_mlp_norm=D.ABSENT_NORM, up_projection=None, down_projection=None,
            num_heads=heads, head_dim=dim, value_head_dim=vdim, use_rope=ri is not None, rope_index=ri or 0, parallel_block=True,
            out_projection=_full(t.bits(p + "mix.o", (width, heads * vdim))))
        if kind == "attention":
            groups = int(mx.get("kv_heads") or heads)
            if heads % groups:
                raise bad(f"config.json: {where}: {heads} heads on {groups} kv_heads")
            kv_from = mx.get("kv_from")
            lw.num_groups = groups
            lw.attention_scale = float(mx["scale"]) if mx.get("scale") is not None else float(dim) ** -0.5
            lw.score_soft_cap = float(mx.get("softcap") or 0.0)
            lw.sliding_window_size = int((mx.get("mask") or {}).get("size") or 0)
            lw.unit_sink = True
            if kv_from is None:
                lw.qkv_projection = _packed(t, [p + "mix.q", p + "mix.k", p + "mix.v"], [heads * dim, groups * dim, groups * vdim], width, biases=True)
            else:
                if not 0 <= int(kv_from) < i:
                    raise bad(f"config.json: {where}.kv_from = {kv_from} must name an earlier layer")
                lw.kv_source_layer_index = int(kv_from)
                lw.qkv_projection = _packed(t, [p + "mix.q"], [heads * dim], width, biases=True)
        else:
            decay = np.asarray(mx.get("decay") or [], dtype=np.float32)
            if decay.shape != (heads,):
                raise bad(f"config.json: {where}.decay must list one decay per head ({heads})")
            lw.num_groups = heads
            lw.retention_decay = np.ascontiguousarray(decay)
            lw.key_scale = float(dim) ** -0.5
            lw.head_norm_epsilon = eps
            lw.qkv_projection = _packed(t, [p + "mix.q", p + "mix.k", p + "mix.v", p + "mix.g"], [heads * dim, heads * dim, heads * vdim, heads * vdim], width, biases=False)
        ml = lc.get("mlp")
        if ml is None:
            lw.no_mlp = True
        elif ml.get("kind") == "moe":
            r = ml.get("router") or {}
            experts, top = int(r["experts"]), int(r["top"])
            ex = ml.get("expert") or {}
            ff = int(ex.get("ff") or t.shape(p + "mlp.e0.gate")[0])
            limit = float(ex["limit"]) if ex.get("limit") is not None else float("inf")
            if not 0 < top <= experts:
                raise bad(f"config.json: layers[{i}].mlp.router.top = {top} of {experts} experts")
            w13 = np.empty((experts, 2 * ff, width), dtype=np.uint16)
            w2 = np.empty((experts, width, ff), dtype=np.uint16)
            for e in range(experts):  # the engine's expert layout: per expert [up rows ; gate rows] and the down matrix
                w13[e, :ff] = t.bits(f"{p}mlp.e{e}.up", (ff, width))
                w13[e, ff:] = t.bits(f"{p}mlp.e{e}.gate", (ff, width))
                w2[e] = t.bits(f"{p}mlp.e{e}.down", (width, ff))
            lw.moe = D.MoeWeights(num_routed_experts=experts, num_active_experts=top, expert_hidden_dim=ff, router_weights=t.bits(p + "mlp.router", (experts, width)),
                                  router_biases=t.bits(p + "mlp.router.b", (experts,)), w13=w13, w2=w2, up_biases=None, down_biases=None, router_renorm=True, gating_sel=2,
                                  silu_alpha=GATE_ALPHA, gate_clip=(float("-inf"), limit), up_clip=(-limit, limit), routing=D.MOE_ROUTE_TOPK_LOGITS, up_offset=UP_OFFSET)
        else:
            raise unsupported(f"config.json: layers[{i}].mlp.kind = {ml.get('kind')!r} (moe, or mlp: null)")
        layers.append(lw)
    for i, lw in enumerate(layers):
        j = lw.kv_source_layer_index
        if j is None:
            continue
        src = layers[j]
        if src.mixer_kind != D.MIXER_ATTENTION or src.kv_source_layer_index is not None or (src.num_groups, src.head_dim, src.value_head_dim) != (lw.num_groups, lw.head_dim, lw.value_head_dim):
            raise bad(f"config.json: layers[{i}].mixer.kv_from = {j}: that layer must be an attention layer with keys and values of its own and the same kv_heads / dim / vdim")
    bundle = D.ModelBundle(name=name or os.path.basename(os.path.normpath(path)), vocab_size=int(vocab), model_dim=int(width), max_context_length=max_ctx,
                           rope=D.RopeConfig(), embedding=_full(t.bits("embed", (vocab, width))), output_norm=_gain(t, "final.norm", eps), layers=layers,
                           tied_embeddings=False, output_embedding=_full(t.bits("head", (vocab, width))), input_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                           ropes=ropes or None, f32_stream=True, architecture=ARCHITECTURE)
    st.assert_all_consumed()
    return bundle


# ------------------------------------------------------------------------------------------------ writer: a configuration + random weights -> a model directory
def random_tensors(cfg: dict, seed: int = 0) -> Dict[str, np.ndarray]:
    """f32 values (already bf16-representable) of every tensor a configuration names, from a seeded generator: linear weights ~ N(0, gain^2 / in), gains near 1"""
    rng = np.random.default_rng(seed)
    rb = lambda a: _bits_to_f32(_f32_to_bf16_bits(np.asarray(a, dtype=np.float32)))
    vocab, width = int(cfg["vocab"]), int(cfg["width"])
    out: Dict[str, np.ndarray] = {}

    def lin(name, n, k, bias=False, gain=1.0):
        out[name] = rb(rng.standard_normal((n, k)) * gain / np.sqrt(k))
        if bias:
            out[name + ".b"] = rb(rng.standard_normal(n) * 0.1)

    out["embed"] = rb(rng.standard_normal((vocab, width)) / float(cfg["embedding"]["scale"]))
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        H, dim, vd = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
        out[p + "norm1"] = rb(np.float32(0.9 + 0.2 * rng.random())).reshape(())
        if lc["type"] == "retention":
            lin(p + "mix.q", H * dim, width, gain=1.5)
            lin(p + "mix.k", H * dim, width, gain=1.5)
            lin(p + "mix.v", H * vd, width)
            lin(p + "mix.g", H * vd, width, gain=2.0)
        else:
            G = int(mx["kv_heads"])
            lin(p + "mix.q", H * dim, width, bias=True, gain=2.0)
            if mx.get("kv_from") is None:
                lin(p + "mix.k", G * dim, width, bias=True, gain=2.0)
                lin(p + "mix.v", G * vd, width, bias=True)
        lin(p + "mix.o", width, H * vd)
        ml = lc.get("mlp")
        if ml is None:
            continue
        E, ff = int(ml["router"]["experts"]), int(ml["expert"]["ff"])
        for e in range(E):
            lin(f"{p}mlp.e{e}.gate", ff, width, gain=1.5)
            lin(f"{p}mlp.e{e}.up", ff, width, gain=1.5)
            lin(f"{p}mlp.e{e}.down", width, ff)
        lin(p + "mlp.router", E, width, bias=True, gain=2.0)
    out["final.norm"] = rb(np.float32(0.9 + 0.2 * rng.random())).reshape(())
    lin("head", vocab, width)
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


def rotation(dims: int, base: float = 10000.0, scaling: Optional[dict] = None) -> dict:
    r = {"dims": int(dims), "base": float(base)}
    if scaling:
        r["scaling"] = {k: scaling[k] for k in ("factor", "original", "fast", "slow")}
    return r


def attention_layer(heads: int, kv_heads: int, dim: int, vdim: int, rot: dict, window: Optional[int] = None, scale: Optional[float] = None, softcap: Optional[float] = None,
                    kv_from: Optional[int] = None, mlp: Optional[dict] = None) -> dict:
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": float(scale if scale is not None else dim ** -0.5)}
    if window:
        mixer["mask"] = {"size": int(window)}
    if softcap:
        mixer["softcap"] = float(softcap)
    if kv_from is not None:
        mixer["kv_from"] = int(kv_from)
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def retention_layer(heads: int, dim: int, vdim: int, rot: dict, decay, mlp: Optional[dict] = None) -> dict:
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "rot": rot, "decay": [float(x) for x in decay]}, "mlp": mlp}


def moe_mlp(experts: int, top: int, ff: int, limit: float = 7.0) -> dict:
    return {"kind": "moe", "expert": {"ff": int(ff), "limit": float(limit)}, "router": {"experts": int(experts), "top": int(top)}}


def config(vocab: int, width: int, layers: List[dict], eps: float = 1e-6, embed_scale: Optional[float] = None) -> dict:
    return {"vocab": int(vocab), "width": int(width), "norm": {"eps": float(eps)}, "embedding": {"scale": float(embed_scale if embed_scale is not None else width ** 0.5)},
            "layers": layers}
