"""Relulix on the host: identities of the float64 oracle (what the GPU tests lean on), and the config.json reader -- every branch of the schema, the engine
description it produces, its refusals, and the writer's round trip.  No GPU."""
import json
import os

import numpy as np
import pytest

import relulix_oracle as O
from uzu_amd import desc as D, loader, relulix

YARN = {"factor": 6.0, "original": 48, "fast": 12.0, "slow": 1.5}


def test_oracle_retention_portions_hand_the_state_on():
    rng = np.random.default_rng(0)
    q, k, v = rng.standard_normal((50, 2, 6)), rng.standard_normal((50, 2, 6)), rng.standard_normal((50, 2, 4))
    whole, S = O.retention_core(q, k, v, [0.9, 0.99])
    a, Sa = O.retention_core(q[:17], k[:17], v[:17], [0.9, 0.99])
    b, Sb = O.retention_core(q[17:], k[17:], v[17:], [0.9, 0.99], Sa)
    assert np.allclose(np.concatenate([a, b]), whole, atol=1e-12) and np.allclose(Sb, S, atol=1e-12)
    # the closed form of one output: sum_j decay^(t - j) <q_t, k_j> v_j
    t = 30
    direct = sum(0.9 ** (t - j) * (q[t, 0] @ k[j, 0]) * v[j, 0] for j in range(t + 1))
    assert np.allclose(whole[t, 0], direct, atol=1e-10)


def test_oracle_attention_rows_do_not_depend_on_where_the_call_starts():
    rng = np.random.default_rng(1)
    q, K, V = rng.standard_normal((40, 4, 8)), rng.standard_normal((40, 2, 8)), rng.standard_normal((40, 2, 6))
    mx = {"heads": 4, "kv_heads": 2, "scale": 0.3, "mask": {"size": 7}, "softcap": 2.0}
    whole = O.attention_core(q, K, V, mx)
    assert np.allclose(O.attention_core(q[25:], K, V, mx, start=25), whole[25:], atol=1e-12)
    # one more term in the denominator: the weights of a row sum to less than one
    mx1 = {"heads": 1, "kv_heads": 1, "scale": 1.0}
    out = O.attention_core(np.zeros((3, 1, 4)), np.zeros((3, 1, 4)), np.ones((3, 1, 2)), mx1)
    assert np.allclose(out[:, 0, 0], [1 / 2, 2 / 3, 3 / 4])


def test_oracle_rotation_and_scaled_frequencies():
    rot = O.rot(8, 10000.0)
    a = np.random.default_rng(2).standard_normal((5, 2, 12))
    r = O.rotate(a, [0, 1, 7, 100, 1000], rot)
    assert np.allclose(r[0], a[0]) and np.allclose(r[..., 8:], a[..., 8:])
    assert np.allclose((r[..., :8] ** 2).sum(-1), (a[..., :8] ** 2).sum(-1))
    # the scalar product of a rotated query and key depends on the distance only
    q, k = a[:1], a[1:2]
    d1 = (O.rotate(q, [13], rot) * O.rotate(k, [10], rot)).sum()
    d2 = (O.rotate(q, [503], rot) * O.rotate(k, [500], rot)).sum()
    assert np.isclose(d1, d2)
    f, m = O.frequencies(O.rot(16, 10000.0, YARN))
    f0, _ = O.frequencies(O.rot(16, 10000.0))
    assert np.isclose(m, 0.1 * np.log(6.0) + 1.0)
    assert np.isclose(f[0], f0[0]) and np.isclose(f[-1], f0[-1] / 6.0) and np.all(f <= f0 + 1e-15) and np.all(f >= f0 / 6.0 - 1e-15)


def test_oracle_routing_and_expert():
    h = np.array([[1.0, 0.0], [0.0, 1.0]])
    w = np.array([[1.0, 0.0], [1.0, 0.0], [0.0, 2.0]])
    ids, wt = O.route(h, w, np.array([0.0, 0.0, 0.5]), 2)
    assert ids.tolist() == [[0, 1], [2, 0]]                      # a tie goes to the lower index
    assert np.allclose(wt[0], [0.5, 0.5]) and np.isclose(wt[1].sum(), 1.0) and np.isclose(wt[1, 0] / wt[1, 1], np.exp(2.5))
    g = O.expert(np.array([[10.0]]), np.array([[1.0]]), np.array([[-1.0]]), np.array([[1.0]]), 2.0)   # gate 10 -> 2, up -10 -> -2
    assert np.isclose(g[0, 0], 2.0 / (1 + np.exp(-1.702 * 2.0)) * (-2.0 + 1.0))


def cfg_full():
    return O.config(vocab=29, width=24, eps=2e-6, embed_scale=1.25, layers=[
        O.retention_layer(3, 4, 6, O.rot(4, 777.0), [0.5, 0.75, 0.875], mlp=O.moe(3, 2, 8, limit=1.25)),
        O.attention_layer(4, 2, 6, 10, O.rot(2, 10000.0, YARN), window=9, softcap=3.0, scale=0.37, mlp=None),
        O.attention_layer(4, 2, 6, 10, O.rot(2, 10000.0, YARN), kv_from=1, mlp=O.moe(2, 1, 4)),
        O.attention_layer(1, 1, 8, 8, O.rot(8, 10000.0), mlp=None),
    ])


def write(tmp_path, cfg, W=None, name="m"):
    path = str(tmp_path / name)
    O.write_model_dir(path, cfg, W if W is not None else O.weights(cfg, 3))
    return path


def test_reader_maps_every_branch_of_the_schema(tmp_path):
    cfg = cfg_full()
    W = O.weights(cfg, 3)
    b = loader.load_model_dir(write(tmp_path, cfg, W), max_context_length=100)
    assert b.architecture == "Relulix" and b.f32_stream and not b.tied_embeddings and b.vocab_size == 29 and b.model_dim == 24 and b.input_scale == 1.25
    assert b.output_norm.kind == D.NORM_RMS_SCALAR and np.isclose(b.output_norm.alpha, W["final.norm"]) and np.isclose(b.output_norm.epsilon, 2e-6)
    assert b.output_embedding.n == 29 and b.output_embedding.k == 24
    assert len(b.ropes) == 3 and [r.kind for r in b.ropes] == [D.ROPE_UNSCALED, D.ROPE_YARN, D.ROPE_UNSCALED] and [l.rope_index for l in b.layers] == [0, 1, 1, 2]
    y = b.ropes[1]
    assert (y.head_dim, y.scaling_factor, y.original_context_length, y.beta_fast, y.beta_slow) == (2, 6.0, 48, 12.0, 1.5)
    r, a, s, last = b.layers
    assert all(l.parallel_block and l.pre_mixer_norm.kind == D.NORM_RMS_SCALAR and not l.pre_mlp_norm.present for l in b.layers)
    assert r.mixer_kind == D.MIXER_RETENTION and r.qkv_projection.n == 3 * (4 + 4 + 6 + 6) and r.qkv_projection.out_biases is None
    assert np.allclose(r.retention_decay, [0.5, 0.75, 0.875]) and np.isclose(r.key_scale, 0.5) and np.isclose(r.head_norm_epsilon, 2e-6)
    assert a.mixer_kind == D.MIXER_ATTENTION and (a.num_heads, a.num_groups, a.head_dim, a.value_head_dim) == (4, 2, 6, 10)
    assert a.qkv_projection.n == 4 * 6 + 2 * 6 + 2 * 10 and a.qkv_projection.out_biases.shape == (56,) and a.no_mlp
    assert (a.sliding_window_size, a.unit_sink, a.kv_source_layer_index) == (9, True, None) and np.isclose(a.score_soft_cap, 3.0) and np.isclose(a.attention_scale, 0.37)
    # the packed projection is queries | keys | values, row for row
    assert np.array_equal(a.qkv_projection.weights[24:36], O.bf16_bits(W["l1.mix.k"])) and np.array_equal(a.qkv_projection.out_biases[36:], O.bf16_bits(W["l1.mix.v.b"]))
    assert s.kv_source_layer_index == 1 and s.qkv_projection.n == 24 and s.sliding_window_size == 0 and s.score_soft_cap == 0.0
    mo = r.moe
    assert (mo.num_routed_experts, mo.num_active_experts, mo.expert_hidden_dim, mo.routing, mo.router_renorm) == (3, 2, 8, D.MOE_ROUTE_TOPK_LOGITS, True)
    assert np.isclose(mo.silu_alpha, 1.702) and mo.up_offset == 1.0 and mo.gate_clip == (float("-inf"), 1.25) and mo.up_clip == (-1.25, 1.25)
    assert np.array_equal(mo.w13[1, :8], O.bf16_bits(W["l0.mlp.e1.up"])) and np.array_equal(mo.w13[1, 8:], O.bf16_bits(W["l0.mlp.e1.gate"]))
    assert last.sliding_window_size == 0 and last.num_groups == 1
    d = b.desc()  # the C description builds
    assert d.num_layers == 4 and d.layers[0].mixer_kind == D.MIXER_RETENTION and d.layers[2].is_kv_sharing == 1 and d.num_ropes == 3


def test_reader_refusals(tmp_path):
    def broken(change, name):
        cfg = cfg_full()
        W = O.weights(cfg, 3)
        change(cfg, W)
        return write(tmp_path, cfg, W, name)

    def decay(c, W): c["layers"][0]["mixer"]["decay"] = [0.5, 0.5]
    def later(c, W): c["layers"][2]["mixer"]["kv_from"] = 3
    def from_retention(c, W): c["layers"][2]["mixer"]["kv_from"] = 0
    def kind(c, W): c["layers"][3]["type"] = "convolution"
    def dense(c, W): c["layers"][0]["mlp"]["kind"] = "dense"
    def shape(c, W): W["l1.mix.k"] = W["l1.mix.k"][:-1]
    def extra(c, W): W["l3.mix.extra"] = W["l3.mix.q"]
    def odd(c, W): c["layers"][3]["mixer"]["rot"]["dims"] = 3
    def groups(c, W): c["layers"][2]["mixer"]["kv_heads"] = 4; W["unused"] = W["final.norm"]
    for i, (change, err) in enumerate([(decay, loader.ModelFormatError), (later, loader.ModelFormatError), (from_retention, loader.ModelFormatError), (kind, loader.UnsupportedModelError),
                                       (dense, loader.UnsupportedModelError), (shape, loader.ModelFormatError), (extra, loader.ModelFormatError), (odd, loader.ModelFormatError),
                                       (groups, loader.ModelFormatError)]):
        with pytest.raises(err):
            loader.load_model_dir(broken(change, f"bad{i}"), max_context_length=64)


def test_writer_round_trip(tmp_path):
    cfg = relulix.config(37, 16, [
        relulix.retention_layer(2, 4, 4, relulix.rotation(4, 1e4), [0.9, 0.99], mlp=relulix.moe_mlp(2, 1, 8, limit=2.0)),
        relulix.attention_layer(2, 1, 8, 4, relulix.rotation(4, 1e4, YARN), window=3, softcap=9.0, mlp=None)])
    T = relulix.random_tensors(cfg, seed=4)
    relulix.save(str(tmp_path / "w"), cfg, T)
    assert json.load(open(os.path.join(str(tmp_path / "w"), "config.json")))["architecture"] == "Relulix"
    b = loader.load_model_dir(str(tmp_path / "w"), max_context_length=32)
    assert b.layers[0].mixer_kind == D.MIXER_RETENTION and b.layers[1].sliding_window_size == 3 and b.layers[0].moe.gate_clip[1] == 2.0
    assert np.array_equal(b.embedding.weights, O.bf16_bits(T["embed"]))
    # the oracle reads what the writer wrote: both sides agree on names and shapes
    full = dict(cfg, architecture="Relulix")
    assert O.forward(full, {k: v.astype(np.float64) for k, v in T.items()}, [1, 2, 3]).shape == (3, 37)
