"""Relulix through the engine (HipModel: states, batched steps, prefill / decode, sampling, the generate loops) against the float64 oracle on small models of
the tests' own making: odd sizes, head widths that differ between keys and values, grouped and single key / value heads, layers with and without window /
cap / scaling / experts / shared caches, retention layers in front, between and behind attention layers, one and several winners."""

import numpy as np
import pytest

import relulix_oracle as O
from uzu_amd import loader
from uzu_amd.engine import MODEL_BATCH, MODEL_DEBUG_TAPS, MODEL_FULL_F32, HipModel

pytestmark = pytest.mark.gpu

TOL = {True: 4e-5, False: 6e-2}  # full f32 / bf16 products: rms logit error relative to the rms of the logits
YARN = {"factor": 6.0, "original": 48, "fast": 12.0, "slow": 1.5}


def rows_ok(err, full, tol=None):
    """True f32: every row inside the tolerance.  bf16 products: a router's choice between two experts of nearly equal logit may fall the other way for a token
    (a discontinuity of the design, not an error of the arithmetic), so nine rows in ten must be inside and the median well inside."""
    err, tol = np.asarray(err), TOL[full] if tol is None else tol
    return bool(err.max() < tol) if full else bool(np.median(err) < tol / 2 and np.mean(err < tol) >= 0.9)


def cfg_a():  # odd sizes: nothing is a multiple of 8, so every kernel runs its general form
    return O.config(vocab=61, width=36, eps=1e-5, embed_scale=3.5, layers=[
        O.retention_layer(3, 6, 10, O.rot(6, 5000.0), [0.9, 0.99, 0.75], mlp=O.moe(3, 2, 12, limit=1.0)),
        O.attention_layer(6, 2, 10, 6, O.rot(4, 10000.0, YARN), window=5, softcap=4.0, scale=0.4, mlp=O.moe(5, 1, 20, limit=0.7)),
        O.attention_layer(6, 2, 10, 6, O.rot(4, 10000.0, YARN), window=None, softcap=None, kv_from=1, mlp=None),
        O.attention_layer(2, 2, 12, 12, O.rot(12, 100.0), window=1, mlp=O.moe(2, 2, 8, limit=50.0)),
        O.retention_layer(1, 12, 6, O.rot(2, 10000.0), [0.999], mlp=None),
    ])


def cfg_b():  # matrix-core friendly sizes, windows that span several key blocks, a cache shared across a retention layer
    return O.config(vocab=97, width=64, layers=[
        O.attention_layer(4, 2, 16, 16, O.rot(8, 10000.0, {"factor": 3.0, "original": 64, "fast": 24.0, "slow": 2.0}), window=40, softcap=15.0, mlp=O.moe(4, 2, 32, limit=1.75)),
        O.retention_layer(2, 32, 32, O.rot(32, 1e6), [0.9375, 0.998046875], mlp=O.moe(6, 3, 16, limit=2.0)),
        O.attention_layer(4, 2, 16, 16, O.rot(8, 10000.0, {"factor": 3.0, "original": 64, "fast": 24.0, "slow": 2.0}), window=70, softcap=15.0, kv_from=0, mlp=O.moe(1, 1, 16)),
        O.attention_layer(8, 8, 8, 16, O.rot(8, 10000.0), window=None, mlp=None),
    ])


@pytest.fixture(scope="module")
def models(hip_ctx, tmp_path_factory):
    out = {}
    for name, cfg, seed in (("a", cfg_a(), 11), ("b", cfg_b(), 12)):
        W = O.weights(cfg, seed)
        path = str(tmp_path_factory.mktemp("relulix") / name)
        O.write_model_dir(path, cfg, W)
        bundle = loader.load_model_dir(path, max_context_length=512)
        W64 = {k: v.astype(np.float64) for k, v in W.items()}
        out[name] = (cfg, W64, {full: HipModel(hip_ctx, bundle, MODEL_BATCH(6) | MODEL_DEBUG_TAPS | (MODEL_FULL_F32 if full else 0)) for full in (True, False)})
    yield out
    for _, _, ms in out.values():
        for m in ms.values():
            m.close()


def prompt(cfg, n, seed):
    return list(np.random.default_rng(seed).integers(0, cfg["vocab"], size=n))


@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("full", [True, False])
def test_whole_prompt_every_position_and_every_layer(models, name, full):
    cfg, W, ms = models[name]
    m = ms[full]
    toks = prompt(cfg, 150, 1)
    layers = []
    want = O.forward(cfg, W, toks, layers)
    st = m.new_state()
    got, _ = m.step_batch([st], [toks], [list(range(len(toks)))])
    for l, ref in enumerate(layers):  # the residual stream behind every layer: names the first layer that differs
        err = np.abs(m.read_layer_output_f32(l) - ref).max(-1) / np.abs(ref).max()
        assert rows_ok(err, full, 2e-5 if full else 5e-2), (l, err.max(), np.median(err))
    assert rows_ok(O.logit_error(got, want), full)
    st.close()


def one_layer(layer, vocab=53, width=40):
    return O.config(vocab=vocab, width=width, layers=[layer])


MECHANISMS = {
    "retention": O.retention_layer(2, 8, 12, O.rot(8, 1e4), [0.95, 0.999]),
    "retention_partial_rotation": O.retention_layer(3, 12, 4, O.rot(6, 1e3), [0.5, 1.0, 0.9]),
    "attention_plain": O.attention_layer(2, 2, 8, 8, O.rot(8, 1e4)),
    "attention_grouped_window_cap": O.attention_layer(4, 2, 12, 20, O.rot(6, 1e4), window=7, softcap=1.5, scale=0.9),
    "attention_scaled_rotation": O.attention_layer(2, 1, 16, 8, O.rot(16, 1e4, YARN), window=50),
    "experts_alone_top1": O.attention_layer(1, 1, 8, 8, O.rot(2, 1e4), window=1, mlp=O.moe(7, 1, 12, limit=0.5)),
    "experts_all_chosen": O.attention_layer(1, 1, 8, 8, O.rot(2, 1e4), window=1, mlp=O.moe(3, 3, 20, limit=3.0)),
}


@pytest.mark.parametrize("which", sorted(MECHANISMS))
def test_each_mechanism_alone_in_a_one_layer_model(hip_ctx, tmp_path, which):
    cfg = one_layer(MECHANISMS[which])
    W = O.weights(cfg, 5)
    O.write_model_dir(str(tmp_path / "m"), cfg, W)
    W64 = {k: v.astype(np.float64) for k, v in W.items()}
    m = HipModel(hip_ctx, loader.load_model_dir(str(tmp_path / "m"), max_context_length=256), MODEL_BATCH(2) | MODEL_DEBUG_TAPS | MODEL_FULL_F32)
    toks = prompt(cfg, 90, 3)
    layers = []
    want = O.forward(cfg, W64, toks, layers)
    st = m.new_state()
    got, _ = m.step_batch([st], [toks], [list(range(len(toks)))])
    assert np.abs(m.read_layer_output_f32(0) - layers[0]).max() < 2e-5 * np.abs(layers[0]).max()
    assert O.logit_error(got, want).max() < TOL[True]
    st.close()
    m.close()


@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("full", [True, False])
def test_prefill_then_token_by_token_and_portions_down_to_two_tokens(models, name, full):
    cfg, W, ms = models[name]
    m = ms[full]
    toks = prompt(cfg, 120, 2)
    want = O.forward(cfg, W, toks)
    for cuts in ([100] + [1] * 20, [1] * 30 + [90], [2, 3, 2, 50, 7, 2, 54], [33, 31, 17, 39], [64, 1, 55]):
        assert sum(cuts) == len(toks)
        st, rows, at = m.new_state(), [], 0
        for n in cuts:
            lg, _ = m.step_batch([st], [toks[at:at + n]], [list(range(n))])
            rows.append(lg)
            at += n
        assert st.context_length == len(toks)
        assert rows_ok(O.logit_error(np.concatenate(rows), want), full), cuts
        st.close()


@pytest.mark.parametrize("name", ["a", "b"])
def test_unequal_batch_equals_each_request_alone_and_reused_states(models, name):
    cfg, W, ms = models[name]
    m = ms[True]
    reqs = [prompt(cfg, n, 10 + n) for n in (1, 37, 90, 5, 64)]
    alone = []
    for r in reqs:
        st = m.new_state()
        first, _ = m.step_batch([st], [r[:-3]] if len(r) > 3 else [r], [[len(r) - 4] if len(r) > 3 else [0]])
        tail = [m.step_batch([st], [[t]], [[0]])[0] for t in (r[-3:] if len(r) > 3 else [])]
        alone.append(np.concatenate([first] + tail))
        st.close()
    pool = [m.new_state() for _ in reqs]
    for round_ in range(2):  # the second round reuses the states the first one gave back (reset), in another order: caches and retention states of other requests
        states = pool if round_ == 0 else pool[::-1]
        heads = [r[:-3] if len(r) > 3 else r for r in reqs]
        lg, _ = m.step_batch(states, heads, [[len(h) - 1] for h in heads])
        got = [[lg[i]] for i in range(len(reqs))]
        for step in range(3):  # decoded together; the one-token request has left the batch
            live = [i for i, r in enumerate(reqs) if len(r) > 3]
            lg, _ = m.step_batch([states[i] for i in live], [[reqs[i][len(reqs[i]) - 3 + step]] for i in live], [[0]] * len(live))
            for row, i in zip(lg, live):
                got[i].append(row)
        for i in range(len(reqs)):
            assert np.abs(np.stack(got[i]) - alone[i]).max() < 2e-4 * np.abs(alone[i]).max(), (round_, i)
            assert O.logit_error(np.stack(got[i])[-1:], O.forward(cfg, W, reqs[i])[-1:]).max() < TOL[True]
        for st in states:
            st.reset()
    for st in pool:
        st.close()


def test_more_requests_than_a_pass_carries_and_prompts_longer_than_a_pass(hip_ctx, tmp_path):
    cfg = O.config(vocab=31, width=16, layers=[
        O.attention_layer(2, 1, 8, 8, O.rot(4, 1e4), window=6, mlp=O.moe(2, 1, 8)),
        O.retention_layer(2, 8, 8, O.rot(8, 1e4), [0.9, 0.998], mlp=None),
        O.attention_layer(2, 1, 8, 8, O.rot(4, 1e4), window=None, kv_from=0, mlp=None)])
    W = O.weights(cfg, 21)
    O.write_model_dir(str(tmp_path / "m"), cfg, W)
    W64 = {k: v.astype(np.float64) for k, v in W.items()}
    m = HipModel(hip_ctx, loader.load_model_dir(str(tmp_path / "m"), max_context_length=3000), MODEL_BATCH(2) | MODEL_FULL_F32)
    reqs = [prompt(cfg, n, n) for n in (9, 2100, 4, 30, 2)]  # 2100 > one pass of 2048 rows; five requests > two per pass
    states = [m.new_state() for _ in reqs]
    lg, sampled = m.step_batch(states, reqs, [[len(r) - 1] for r in reqs], sample=True)
    for i, r in enumerate(reqs):
        want = O.forward(cfg, W64, r)[-1:] if len(r) < 200 else None
        if want is not None:
            assert O.logit_error(lg[i:i + 1], want).max() < TOL[True] and int(sampled[i]) == int(np.argmax(want))
        assert states[i].context_length == len(r)
    # the long prompt: against the same prompt through two explicit portions
    st = m.new_state()
    m.step_batch([st], [reqs[1][:1500]], [[]])
    two, _ = m.step_batch([st], [reqs[1][1500:]], [[599]])
    assert np.abs(two[0] - lg[1]).max() < 2e-4 * np.abs(two).max()
    m.close()


@pytest.mark.parametrize("full", [True, False])
def test_long_decoding_across_windows(models, full):
    cfg, W, ms = models["b"]
    m = ms[full]
    toks = prompt(cfg, 230, 5)
    want = O.forward(cfg, W, toks)
    st = m.new_state()
    m.step_batch([st], [toks[:10]], [[]])
    rows = [m.step_batch([st], [[t]], [[0]])[0][0] for t in toks[10:]]  # 220 decoded tokens: every window (40, 70) slides over decoded tokens only
    assert rows_ok(O.logit_error(np.stack(rows), want[10:]), full)
    st.close()


def test_a_far_token_reaches_the_logits_only_through_the_retention_state(hip_ctx, tmp_path):
    """Windows of 4: the attention layers cannot see position 3 from position 400; the slow retention head can.  Changing that one token must change the last
    logits, by prompt and by decoding alike, exactly as the oracle says."""
    cfg = O.config(vocab=41, width=32, layers=[
        O.attention_layer(2, 2, 8, 8, O.rot(8, 1e4), window=4, mlp=None),
        O.retention_layer(2, 16, 16, O.rot(16, 1e6), [0.5, 0.9995], mlp=None),
        O.attention_layer(2, 2, 8, 8, O.rot(8, 1e4), window=4, mlp=None)])
    W = O.weights(cfg, 8)
    O.write_model_dir(str(tmp_path / "m"), cfg, W)
    W64 = {k: v.astype(np.float64) for k, v in W.items()}
    m = HipModel(hip_ctx, loader.load_model_dir(str(tmp_path / "m"), max_context_length=512), MODEL_BATCH(2) | MODEL_FULL_F32)
    base = prompt(cfg, 401, 4)
    other = list(base)
    other[3] = (base[3] + 7) % cfg["vocab"]
    want = [O.forward(cfg, W64, t)[-1] for t in (base, other)]
    assert O.logit_error(want[0][None], want[1][None]).max() > 1e-3, "the oracle itself does not carry the token: strengthen the weights"
    for toks, ref in zip((base, other), want):
        st = m.new_state()
        whole, _ = m.step_batch([st], [toks], [[400]])
        st.reset()
        m.step_batch([st], [toks[:100]], [[]])
        for t in toks[100:-1]:
            m.step_batch([st], [[t]], [[]])
        dec, _ = m.step_batch([st], [[toks[-1]]], [[0]])
        assert O.logit_error(whole, ref[None]).max() < TOL[True] and O.logit_error(dec, ref[None]).max() < TOL[True]
        st.close()
    m.close()


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation_through_prefill_and_decode(models, name):
    """The engine's own entry points: HipModel.prefill + chained decode (the sampled token is fed back on the device), then the stochastic sampler's plumbing."""
    cfg, W, ms = models[name]
    m = ms[True]
    p = prompt(cfg, 25, 7)
    m.reset()
    m.set_sampling(None)
    first = m.prefill(np.asarray(p, dtype=np.uint32))
    rest, _ = m.decode(9)
    got = [int(first)] + [int(t) for t in rest]
    want, margin_ok = [], True
    toks = list(p)
    for _ in range(10):
        row = O.forward(cfg, W, toks)[-1]
        top2 = np.sort(row)[-2:]
        margin_ok = margin_ok and (top2[1] - top2[0]) > 1e-3 * np.abs(row).max()
        want.append(int(np.argmax(row)))
        toks.append(want[-1])
    assert margin_ok, "the oracle's own greedy stream has a near tie: pick another seed"
    assert got == want and m.context_length == len(p) + 9
    assert np.argmax(m.read_logits_f32()) == want[-1]
    m.reset()
    m.set_sampling(seed=3, temperature=1e-4)  # temperature -> 0 of the stochastic sampler is greedy
    s1 = [int(m.prefill(np.asarray(p, dtype=np.uint32)))] + [int(t) for t in m.decode(4)[0]]
    assert s1 == want[:5]
    m.set_sampling(None)
    m.reset()


def test_generate_loop_of_the_text_front_end_and_the_pool(hip_ctx, tmp_path):
    """LanguageModel.generate on a directory without tokenizer.json, and SequencePool.generate: prompts of unequal length prefilled in one batch and decoded
    together, requests leaving as they finish (one by a stop token), their states reused by a second round -- against each prompt generated alone by the oracle"""
    from uzu_amd.language_model import LanguageModel
    from uzu_amd.serving import SequencePool
    cfg = cfg_a()
    W = O.weights(cfg, 31, logit_gain=3.0)
    O.write_model_dir(str(tmp_path / "g"), cfg, W)
    W64 = {k: v.astype(np.float64) for k, v in W.items()}
    lm = LanguageModel(hip_ctx, str(tmp_path / "g"), max_context_length=128, flags=MODEL_FULL_F32, tokenizer_required=False)
    p = prompt(cfg, 12, 3)
    res = lm.generate(p, max_tokens=11, chunk=4)
    assert res.token_ids == O.greedy(cfg, W64, p, 11) and res.prompt_tokens == 12
    lm.close()
    m = HipModel(hip_ctx, loader.load_model_dir(str(tmp_path / "g"), max_context_length=128), MODEL_BATCH(4) | MODEL_FULL_F32)
    prompts = {"x": prompt(cfg, 3, 41), "y": prompt(cfg, 40, 42), "z": prompt(cfg, 17, 43)}
    want = {k: O.greedy(cfg, W64, q, 8) for k, q in prompts.items()}
    stop = want["y"][4]
    cut = lambda seq: seq[:seq.index(stop)] if stop in seq else seq
    pool = SequencePool(m)
    for _ in range(2):
        got = pool.generate(prompts, max_tokens=8, stop_token_ids=[stop])
        assert got == {k: cut(v) for k, v in want.items()}
        assert not pool.live and len(pool.free) == 3
    pool.close()
    m.close()


@pytest.mark.parametrize("full", [True, False])
def test_decode_graph_replays_equal_plain_launches(hip_ctx, tmp_path, full):
    """The chained decode step is ONE captured hipGraph per state that reads its position from device memory.  Replayed in several calls, with eager batched
    steps of OTHER states (which overwrite the model's pass tables) and synchronisations between them, every token and the logits after every call must equal
    those of a model that decodes with plain launches."""
    from uzu_amd.engine import MODEL_NO_GRAPH
    cfg = cfg_b()
    W = O.weights(cfg, 77)
    O.write_model_dir(str(tmp_path / "m"), cfg, W)
    bundle = loader.load_model_dir(str(tmp_path / "m"), max_context_length=256)
    base = MODEL_BATCH(4) | (MODEL_FULL_F32 if full else 0)
    graph, plain = HipModel(hip_ctx, bundle, base), HipModel(hip_ctx, bundle, base | MODEL_NO_GRAPH)
    p, other = prompt(cfg, 70, 8), prompt(cfg, 33, 9)
    firsts = [m.prefill(np.asarray(p, dtype=np.uint32)) for m in (graph, plain)]
    assert firsts[0] == firsts[1]
    side = [m.new_state() for m in (graph, plain)]
    for call in range(4):
        toks = [m.decode(5)[0] for m in (graph, plain)]
        assert list(toks[0]) == list(toks[1]), call
        assert np.array_equal(graph.read_logits_f32(), plain.read_logits_f32()), call
        for m, st in zip((graph, plain), side):  # eager work on another state between the replays
            m.step_batch([st], [other[call * 8:(call + 1) * 8]], [[7]])
    assert graph.context_length == 70 + 20
    for m in (graph, plain):
        m.close()
