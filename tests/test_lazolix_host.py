"""Lazolix on the host: the plain oracle against algebraic identities of the design, and the model-directory reader on every branch of the configuration."""
import json
import os

import numpy as np
import pytest

import lazolix_oracle as O
from uzu_amd import desc as D
from uzu_amd import lazolix, loader


def small_cfg():
    return O.config(vocab=50, width=24, layers=[
        O.layer(3, 8, 6, 16, window=4, mlp=O.dense(40)),
        O.layer(2, 4, 10, 16, window=None, kv_from=0, scale=0.3, mlp=O.moe(3, 2, 12, identity=1)),
        O.layer(1, 8, 8, 8, window=1, mlp=None),
        O.layer(3, 8, 6, 16, window=7, kv_from=0, mlp=O.moe(2, 1, 8, identity=0)),
    ])


def test_oracle_latent_space_form_equals_expanded_keys_and_values():
    rng = np.random.default_rng(0)
    T, H, dim, vd, r = 9, 3, 4, 5, 6
    q, c = rng.standard_normal((T, H * dim)), rng.standard_normal((T + 2, r))
    uk, uv, sinks = rng.standard_normal((H * dim, r)), rng.standard_normal((H * vd, r)), rng.standard_normal(H)
    for window in (0, 1, 3):
        direct = O.latent_attention(q, c, uk, uv, H, 0.4, window, sinks, start=2)
        qlat = np.concatenate([q[:, a * dim:(a + 1) * dim] @ uk[a * dim:(a + 1) * dim] for a in range(H)], axis=1)
        ctx = O.latent_core(qlat, c, H, 0.4, window, sinks, start=2)
        folded = np.concatenate([ctx[:, a * r:(a + 1) * r] @ uv[a * vd:(a + 1) * vd].T for a in range(H)], axis=1)
        assert np.allclose(direct, folded, atol=1e-12)


def test_oracle_window_sink_and_shift_edges():
    assert O.visible(5, 5, 1) and not O.visible(5, 4, 1) and O.visible(5, 3, 3) and not O.visible(5, 2, 3) and O.visible(5, 0, 0) and not O.visible(5, 6, 0)
    # a sink far above every score takes all the weight and has no value: the output vanishes
    rng = np.random.default_rng(1)
    out = O.latent_core(rng.standard_normal((2, 4)), rng.standard_normal((2, 4)), 1, 1.0, 0, np.array([60.0]))
    assert np.abs(out).max() < 1e-20
    h = rng.standard_normal((3, 5))
    mu = rng.random(5)
    s, last = O.token_shift(h, mu)
    assert np.allclose(s[0], h[0] * (1 - mu)) and np.allclose(s[2], h[2] + (h[1] - h[2]) * mu) and np.allclose(last, h[2])
    s2, _ = O.token_shift(h[1:], mu, prev=h[0])
    assert np.allclose(s2, s[1:])


def test_oracle_routing_identity_experts_and_weights():
    rng = np.random.default_rng(2)
    h = rng.standard_normal((6, 8))
    wr = rng.standard_normal((5, 8))
    ids, w = O.route(h, wr, np.array([0, 0, 0, 0, 10.0]), 2)
    assert (ids[:, 0] == 4).all() and np.allclose(w.sum(-1), 1.0)  # the correction decides the choice ...
    ids0, w0 = O.route(h, wr, None, 5)
    z = h @ wr.T
    s = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    assert np.allclose(np.take_along_axis(s, ids0, -1), w0)        # ... and never the weights
    only_identity = O.moe_mlp(h, wr[:1], None, [], 1)
    assert np.allclose(only_identity, h)


def test_model_dir_round_trip_every_branch(tmp_path):
    cfg = small_cfg()
    W = O.weights(cfg, 3)
    O.write_model_dir(str(tmp_path / "m"), cfg, W)
    b = loader.load_model_dir(str(tmp_path / "m"), max_context_length=64)
    assert b.f32_stream and b.architecture == "Lazolix" and b.vocab_size == 50 and b.model_dim == 24 and b.max_context_length == 64
    l0, l1, l2, l3 = b.layers
    assert all(l.mixer_kind == D.MIXER_LATENT_ATTENTION for l in b.layers)
    assert (l0.num_heads, l0.head_dim, l0.value_head_dim, l0.latent_rank, l0.sliding_window_size) == (3, 8, 6, 16, 4)
    assert l0.mlp_plain and l0.hidden_dim == 40 and l0.up_projection.out_biases is not None and l0.latent_down is not None
    assert l1.kv_source_layer_index == 0 and l1.latent_down is None and l1.sliding_window_size == 0 and abs(l1.attention_scale - 0.3) < 1e-7
    assert l1.moe.routing == D.MOE_ROUTE_SCORES and l1.moe.num_routed_experts == 3 and l1.moe.num_identity_experts == 1 and l1.moe.num_active_experts == 2
    assert l1.moe.router_weights.shape == (4, 24) and l1.moe.w13.shape == (3, 24, 24) and l1.moe.w2.shape == (3, 24, 12)
    assert np.array_equal(l1.moe.w13[2, :12], O.bf16_bits(W["l1.mlp.e2.up"])) and np.array_equal(l1.moe.w13[2, 12:], O.bf16_bits(W["l1.mlp.e2.gate"]))
    assert l2.no_mlp and l2.sliding_window_size == 1 and l3.moe.num_identity_experts == 0
    assert l0.pre_mixer_norm.kind == D.NORM_DYNAMIC_TANH and abs(l0.pre_mixer_norm.alpha - float(W["l0.norm1.alpha"])) < 1e-7
    assert l3.depth_weights.shape == (5,) and l2.token_shift.shape == (24,)
    d = b.desc()
    assert d.f32_stream == 1 and d.layers[1].is_kv_sharing == 1 and d.layers[2].no_mlp == 1 and d.layers[1].moe.num_identity_experts == 1


def test_model_dir_errors(tmp_path):
    cfg = small_cfg()
    W = O.weights(cfg, 4)
    bad = dict(W)
    del bad["l0.mix.dkv"]
    O.write_model_dir(str(tmp_path / "a"), cfg, bad)
    with pytest.raises(loader.ModelFormatError):
        loader.load_model_dir(str(tmp_path / "a"))
    extra = dict(W)
    extra["l1.mix.dkv"] = W["l0.mix.dkv"]  # a sharing layer has no down projection: an unread tensor is an error
    O.write_model_dir(str(tmp_path / "b"), cfg, extra)
    with pytest.raises(loader.ModelFormatError):
        loader.load_model_dir(str(tmp_path / "b"))
    other = dict(cfg)
    other["architecture"] = "Nonesuch"
    O.write_model_dir(str(tmp_path / "c"), other, W)
    with pytest.raises(loader.UnsupportedModelError):
        loader.load_model_dir(str(tmp_path / "c"))
    fwd = json.loads(json.dumps(cfg))
    fwd["layers"][1]["mixer"]["kv_from"] = 2
    O.write_model_dir(str(tmp_path / "d"), fwd, W)
    with pytest.raises(loader.ModelFormatError):
        loader.load_model_dir(str(tmp_path / "d"))


def test_package_writer_makes_loadable_models(tmp_path):
    cfg = {"vocab": 40, "width": 16, "norm": {"eps": 1e-5},
           "layers": [lazolix.layer_config(2, 8, 4, 8, window=3, mlp=lazolix.dense_mlp(24)), lazolix.layer_config(2, 8, 4, 8, None, kv_from=0, mlp=lazolix.moe_mlp(2, 1, 8, 1))]}
    lazolix.save(str(tmp_path / "w"), cfg, lazolix.random_tensors(cfg, seed=1))
    b = loader.load_model_dir(str(tmp_path / "w"))
    assert len(b.layers) == 2 and b.layers[1].kv_source_layer_index == 0 and abs(b.output_norm.epsilon - 1e-5) < 1e-12
    W = {k: v.astype(np.float64) for k, v in lazolix.random_tensors(cfg, seed=1).items()}
    full = dict(cfg, architecture="Lazolix")
    assert np.isfinite(O.forward(full, W, [1, 2, 3, 4, 5])).all()


def test_trace_runner_is_an_executable_script():
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    assert os.access(path, os.X_OK)
