"""Pins of the plain Budorax implementation (tests/plain/budorax_plain.py) that need no GPU: special cases against
library routines, and properties chosen so that a plausible misreading of a mechanism fails them; then the
configuration class (keys, checks, tensor names, the order of the runs and their caches)."""
import numpy as np
import pytest
import torch

from plain import budorax_plain as P

RNG = np.random.default_rng(31)


def test_the_norm_takes_every_element_on_its_own():
    x = RNG.normal(size=(3, 8)) * 3
    w, b = RNG.normal(size=8), RNG.normal(size=8)
    y = P.tanh_norm(x, w, b, 0.7)
    np.testing.assert_allclose(y, torch.tanh(torch.from_numpy(0.7 * x)).numpy() * w + b, rtol=1e-12)
    moved = x.copy()
    moved[0, 0] += 100.0                                   # no mean, no variance: the other elements do not notice
    assert np.array_equal(P.tanh_norm(moved, w, b, 0.7)[:, 1:], y[:, 1:])
    np.testing.assert_allclose(P.tanh_norm(np.zeros(4), np.ones(4), np.full(4, 0.25), 9.0), 0.25)
    assert np.all(np.abs(P.tanh_norm(x * 1e6, np.ones(8), np.zeros(8), 1.0)) <= 1.0)       # saturates, never explodes


def test_root_mean_square_has_eps_inside_the_root():
    x = RNG.normal(size=(2, 6))
    want = torch.nn.functional.rms_norm(torch.from_numpy(x), (6,), eps=1e-3).numpy()
    np.testing.assert_allclose(P.over_rms(x, 1e-3), want, rtol=1e-12)
    np.testing.assert_allclose(P.over_rms(np.zeros((1, 4)), 1e-4), 0.0)


def test_rotation_pairs_neighbours_and_leaves_the_rest():
    x = np.zeros((1, 1, 10))
    x[0, 0, 2] = 1.0                                        # pairs (0,1) (2,3) (4,5): channel 2 is the first of pair 1
    x[0, 0, 7] = 5.0
    angle = 3 * 100.0 ** (-2 / 6)
    y = P.turn_pairs(x, [3], 6, 100.0)
    assert y[0, 0, 2] == pytest.approx(np.cos(angle)) and y[0, 0, 3] == pytest.approx(np.sin(angle))
    assert y[0, 0, 7] == 5.0 and np.count_nonzero(y) == 3
    assert np.array_equal(P.turn_pairs(x, [0], 6, 100.0), x)                     # position 0: nothing turns
    q, k = RNG.normal(size=(1, 2, 8)), RNG.normal(size=(1, 2, 8))
    a = np.sum(P.turn_pairs(q, [9], 8, 50.0) * P.turn_pairs(k, [4], 8, 50.0))
    b = np.sum(P.turn_pairs(q, [25], 8, 50.0) * P.turn_pairs(k, [20], 8, 50.0))
    assert a == pytest.approx(b)                                                  # scores depend on distances only
    c = np.sum(P.turn_pairs(q, [4], 8, 50.0) * P.turn_pairs(k, [9], 8, 50.0))
    assert a != pytest.approx(c)                                                  # and on their sign


def test_blocks_are_counted_from_position_zero():
    seen = P.seen_in_block(7, 3)
    assert seen[2].tolist() == [True, True, True, False, False, False, False]
    assert seen[3].tolist() == [False, False, False, True, False, False, False]     # a block's first position sees itself alone
    assert seen[5].tolist() == [False, False, False, True, True, True, False]
    assert np.array_equal(P.seen_in_block(5, 100), P.seen_causal(5))
    assert np.array_equal(P.seen_in_block(4, 1), np.eye(4, dtype=bool))
    p = P.masked_softmax(np.zeros((7, 7)), seen)
    np.testing.assert_allclose(p[4], [0, 0, 0, 0.5, 0.5, 0, 0])


def attention_weights(cfg, width):
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    w = dict(q=RNG.normal(size=(H * 2 * D, width)), k=RNG.normal(size=(G * 2 * D, width)), v=RNG.normal(size=(G * V, width)),
             o=RNG.normal(size=(width, H * V)))
    for n in ("lq1", "lk1", "lq2", "lk2"):
        w[n] = RNG.normal(size=D) * 0.3
    return w


def test_differential_attention_against_the_library_one_map_at_a_time():
    cfg = dict(heads=2, kv_heads=1, dim=4, vdim=6, diff=0.3, scale=0.5, rot=dict(dims=4, base=100.0), mask=dict(size=100))
    width, T = 5, 9
    x = RNG.normal(size=(T, width))
    w = attention_weights(cfg, width)
    got = P.block_differential_attention(x, w, cfg, 1e-5)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    pos = np.arange(T)
    q = P.turn_pairs((x @ w["q"].T).reshape(T, 2, 2, 4), pos, 4, 100.0)
    k = P.turn_pairs((x @ w["k"].T).reshape(T, 1, 2, 4), pos, 4, 100.0)
    v = (x @ w["v"].T).reshape(T, 1, 6)
    lam = np.exp(w["lq1"] @ w["lk1"]) - np.exp(w["lq2"] @ w["lk2"]) + 0.3
    assert P.differential_factor(w, 0.3) == pytest.approx(lam)
    heads = []
    for h in range(2):
        maps = [torch.nn.functional.scaled_dot_product_attention(t(q[:, h, m])[None], t(k[:, 0, m])[None], t(v[:, 0])[None],
                                                                 is_causal=True, scale=0.5)[0].numpy() for m in (0, 1)]
        o = maps[0] - lam * maps[1]
        heads.append(o / np.sqrt((o * o).mean(axis=1, keepdims=True) + 1e-5) * 0.7)
    np.testing.assert_allclose(got, np.concatenate(heads, axis=1) @ w["o"].T, rtol=1e-9, atol=1e-9)
    # a block of three positions: the fourth token sees itself alone, so both maps give its own value
    small = dict(cfg, mask=dict(size=3))
    out = P.block_differential_attention(x, w, small, 1e-5)
    own = v[3, 0] * (1.0 - lam)
    np.testing.assert_allclose(out[3], np.concatenate([own / np.sqrt((own * own).mean() + 1e-5) * 0.7] * 2) @ w["o"].T, rtol=1e-9)
    assert not np.allclose(out[4], got[4])


def test_latent_attention_by_hand_for_one_head():
    cfg = dict(heads=1, dim=3, rot_dim=2, vdim=4, kv_rank=5, q_rank=4, scale=0.4, rot=dict(dims=2, base=10.0))
    width, T = 6, 5
    x = RNG.normal(size=(T, width))
    w = {"dq": RNG.normal(size=(4, width)), "dq.norm": RNG.normal(size=4), "uq": RNG.normal(size=(5, 4)),
         "dkv": RNG.normal(size=(7, width)), "dkv.norm": RNG.normal(size=5), "uk": RNG.normal(size=(3, 5)),
         "uv": RNG.normal(size=(4, 5)), "g": RNG.normal(size=(1, width)), "o": RNG.normal(size=(width, 4))}
    got = P.latent_attention(x, w, cfg, 1e-5)
    rms = lambda a: a / np.sqrt((a * a).mean(axis=-1, keepdims=True) + 1e-5)
    q = (rms(x @ w["dq"].T) * w["dq.norm"]) @ w["uq"].T
    down = x @ w["dkv"].T
    c = rms(down[:, :5]) * w["dkv.norm"]                       # the rotated key part is not normed
    t = 4
    scores = []
    for j in range(t + 1):
        turned_q = P.turn_pairs(q[t:t + 1, 3:], [t], 2, 10.0)[0]
        turned_k = P.turn_pairs(down[j:j + 1, 5:], [j], 2, 10.0)[0]
        scores.append((q[t, :3] @ (w["uk"] @ c[j]) + turned_q @ turned_k) * 0.4)
    p = np.exp(scores - np.max(scores))
    p /= p.sum()
    o = sum(p[j] * (w["uv"] @ c[j]) for j in range(t + 1)) * P.sigmoid(x[t] @ w["g"][0])
    np.testing.assert_allclose(got[t], w["o"] @ o, rtol=1e-9)


def test_short_convolution_matches_the_library():
    x, taps = RNG.normal(size=(9, 5)), RNG.normal(size=(5, 3))
    want = torch.nn.functional.conv1d(torch.from_numpy(x.T)[None], torch.from_numpy(taps)[:, None, :], padding=2, groups=5)[0, :, :9].numpy().T
    np.testing.assert_allclose(P.short_convolution(x, taps), want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(P.short_convolution(x[:2], RNG.normal(size=(5, 8)) * 0 + 1.0)[1], x[0] + x[1])     # more taps than tokens
    np.testing.assert_allclose(P.short_convolution(x, taps[:, -1:]), x * taps[:, -1])


def test_delta_rule_overwrites_what_a_key_held_and_reads_after_it_wrote():
    k = np.array([[1.0, 0.0], [1.0, 0.0], [0.0, 1.0]])
    v = np.array([[1.0, 2.0, 3.0], [10.0, 20.0, 30.0], [7.0, 7.0, 7.0]])
    out = P.delta_walk(k, k, v, np.ones(3), np.ones(3))
    np.testing.assert_allclose(out[0], v[0])                   # the read-out sees the token's own write
    np.testing.assert_allclose(out[1], v[1])                   # full strength: the key's old value is gone
    np.testing.assert_allclose(out[2], v[2])
    half = P.delta_walk(k, k, v, np.full(3, 0.5), np.ones(3))
    np.testing.assert_allclose(half[1], 0.5 * v[0] + 0.5 * (v[1] - 0.5 * v[0]))
    faded = P.delta_walk(k, k, v, np.ones(3), np.array([1.0, 0.25, 1.0]))        # the decay comes before the write
    np.testing.assert_allclose(faded[1], v[1])
    q = np.array([[0.0, 1.0], [1.0, 0.0], [1.0, 0.0]])
    read = P.delta_walk(q, k, v, np.ones(3), np.array([1.0, 1.0, 0.5]))
    np.testing.assert_allclose(read[2], 0.5 * v[1])


def test_gated_delta_shares_keys_between_heads_and_norms_each_head():
    cfg = dict(heads=4, kv_heads=2, dim=3, vdim=5, conv=2)
    width, T = 6, 7
    x = RNG.normal(size=(T, width))
    w = {"q": RNG.normal(size=(6, width)), "k": RNG.normal(size=(6, width)), "v": RNG.normal(size=(20, width)),
         "q.conv": RNG.normal(size=(6, 2)), "k.conv": RNG.normal(size=(6, 2)), "v.conv": RNG.normal(size=(20, 2)),
         "b": RNG.normal(size=(4, width)), "a": RNG.normal(size=(4, width)), "A_log": RNG.normal(size=4),
         "dt_bias": RNG.normal(size=4), "norm": RNG.normal(size=5), "g": RNG.normal(size=(20, width)), "o": np.eye(20)}
    got = P.gated_delta(x, w, cfg, 1e-5).reshape(T, 4, 5)
    conv = lambda name: P.silu(P.short_convolution(x @ w[name].T, w[name + ".conv"]))
    unit = lambda a: a / np.sqrt((a * a).sum(axis=-1, keepdims=True) + 1e-6)
    h = 3                                                       # uses q/k head 1
    q, k = unit(conv("q")[:, 3:6]) * 3 ** -0.5, unit(conv("k")[:, 3:6])
    g = np.exp(-np.exp(w["A_log"][h]) * np.log1p(np.exp(x @ w["a"][h] + w["dt_bias"][h])))
    o = P.delta_walk(q, k, conv("v")[:, 15:20], P.sigmoid(x @ w["b"][h]), g)
    gate = (x @ w["g"].T)[:, 15:20]
    want = o / np.sqrt((o * o).mean(axis=1, keepdims=True) + 1e-5) * w["norm"] * gate * P.sigmoid(gate)
    np.testing.assert_allclose(got[:, h], want, rtol=1e-9, atol=1e-12)
    assert np.all((g > 0) & (g < 1))


def test_experts_are_chosen_by_corrected_scores_and_weighted_by_plain_ones():
    x = np.eye(4)
    router = np.array([[2.0, 0, 0, 0], [1.0, 0, 0, 0], [0.0, 0, 0, 0], [-1.0, 0, 0, 0]])      # token 0 scores the experts 2, 1, 0, -1
    w = dict(router=router, correction=np.array([0.0, 0.0, 0.0, 10.0]))
    ids, weights = P.choose_experts(x[:1], w, dict(top=2, scale=3.0))
    assert ids[0].tolist() == [3, 0]                           # the correction lifts expert 3 into the choice ...
    s = P.sigmoid(np.array([-1.0, 2.0]))
    np.testing.assert_allclose(weights[0], s / s.sum() * 3.0)   # ... and stays out of its weight
    ids, weights = P.choose_experts(x[1:2], w, dict(top=4, scale=1.0))               # equal scores: the lowest numbers first
    assert ids[0].tolist() == [3, 0, 1, 2] and weights[0].sum() == pytest.approx(1.0)
    width, ff = 4, 3
    for e in range(4):
        w.update({f"e{e}.gate": RNG.normal(size=(ff, width)), f"e{e}.up": RNG.normal(size=(ff, width)), f"e{e}.down": RNG.normal(size=(width, ff))})
    tokens = RNG.normal(size=(5, width))
    got = P.expert_mixture(tokens, w, dict(router=dict(experts=4, top=2, scale=1.5)))
    ids, weights = P.choose_experts(tokens, w, dict(top=2, scale=1.5))
    for t in range(5):
        want = sum(a * (torch.nn.functional.silu(torch.from_numpy(w[f"e{e}.gate"] @ tokens[t])).numpy() * (w[f"e{e}.up"] @ tokens[t]))
                   @ w[f"e{e}.down"].T for e, a in zip(ids[t], weights[t]))
        np.testing.assert_allclose(got[t], want, rtol=1e-9)
    margins = P.choice_margin(tokens, w, dict(top=2))
    assert margins.shape == (5,) and np.all(margins > 0) and np.all(np.isinf(P.choice_margin(tokens, w, dict(top=4))))


def small_config():
    attention = dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=8, vdim=6, diff=0.25, scale=0.3, rot=dict(dims=4, base=100.0),
                                                  mask=dict(size=5)), mlp=dict(kind="moe", expert=dict(ff=10), router=dict(experts=3, top=2, scale=1.5)))
    latent = dict(type="latent_attention", mixer=dict(heads=2, dim=6, rot_dim=4, vdim=5, kv_rank=7, q_rank=3, scale=0.2,
                                                      rot=dict(dims=4, base=50.0)), mlp=None)
    delta = dict(type="delta", mixer=dict(heads=2, kv_heads=1, dim=4, vdim=6, conv=3), mlp=dict(kind="moe", expert=dict(ff=4),
                                                                                                 router=dict(experts=2, top=1, scale=1.0)))
    return dict(architecture="Budorax", vocab=19, width=12, norm=dict(eps=1e-5), logit_softcap=7.0, loop=dict(start=1, stop=3, times=3),
                layers=[attention, latent, delta, attention])


def test_the_runs_follow_the_loop_and_the_stream_takes_the_embedding_again():
    cfg = small_config()
    assert P.run_order(cfg) == [(0, 0, False), (1, 0, True), (2, 0, False), (1, 1, True), (2, 1, False), (1, 2, True), (2, 2, False),
                                (3, 0, False)]
    assert [r[0] for r in P.run_order(dict(cfg, loop=dict(start=0, stop=4, times=2)))] == [0, 1, 2, 3, 0, 1, 2, 3]
    assert [r[0] for r in P.run_order({k: v for k, v in cfg.items() if k != "loop"})] == [0, 1, 2, 3]
    assert [r[0] for r in P.run_order(dict(cfg, loop=dict(start=2, stop=2, times=5)))] == [0, 1, 2, 3]
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.weights import random_tensors
    from mini_llm_runtime_amd.parts import expected_tensors
    tensors = {n: t.double().numpy() for n, t in random_tensors(expected_tensors(config_from_dict(cfg)), 5, matrix_std=0.3).items()}
    tokens = [3, 1, 4, 1, 5, 9, 2, 6]
    streams = []
    logits = P.forward(cfg, tensors, tokens, streams=streams)
    assert len(streams) == 8 and logits.shape == (8, 19) and np.all(np.abs(logits) < 7.0)          # the cap bounds every logit
    once = dict(cfg, loop=dict(start=1, stop=3, times=1))
    first = []
    P.forward(once, tensors, tokens, streams=first)
    np.testing.assert_allclose(first[2], streams[2])            # the first pass knows nothing of the others
    # the second pass starts from the first pass's stream plus the embedding's output: feed that by hand
    x0 = tensors["embed"][np.asarray(tokens)]
    by_hand = streams[2] + x0
    normed = P.named_norm(tensors, "l1.norm1", by_hand)
    mixed = P.latent_attention(normed, P.part_weights(tensors, "l1.mix."), cfg["layers"][1]["mixer"], 1e-5)
    np.testing.assert_allclose(streams[3], by_hand + P.named_norm(tensors, "l1.norm1b", mixed), rtol=1e-9)
    # the prefix property: a token's logits do not depend on what follows
    np.testing.assert_allclose(P.forward(cfg, tensors, tokens[:5])[4], logits[4], rtol=1e-9, atol=1e-12)


def test_configuration_names_every_tensor_and_gives_every_run_a_cache_of_its_own():
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.parts import expected_tensors
    cfg = config_from_dict(small_config())
    assert cfg.to_dict() == small_config() and config_from_dict(cfg.to_dict()) == cfg
    spec = cfg.model_spec()
    assert [(r.layer, r.cache, r.add_embedding) for r in spec.schedule] == \
        [(0, 0, False), (1, 1, False), (2, 2, False), (1, 3, True), (2, 4, False), (1, 5, True), (2, 6, False), (3, 7, False)]
    names = expected_tensors(cfg)
    for name, shape in {"embed": (19, 12), "final.norm": (12,), "final.norm.b": (12,), "final.norm.alpha": (),
                        "l0.norm1": (12,), "l0.norm1b.b": (12,), "l0.norm2.alpha": (), "l0.norm2b": (12,),
                        "l0.mix.q": (64, 12), "l0.mix.k": (32, 12), "l0.mix.v": (12, 12), "l0.mix.lq1": (8,), "l0.mix.o": (12, 24),
                        "l0.mlp.router": (3, 12), "l0.mlp.correction": (3,), "l0.mlp.e2.gate": (10, 12), "l0.mlp.e2.up": (10, 12),
                        "l0.mlp.e2.down": (12, 10),
                        "l1.mix.dq": (3, 12), "l1.mix.dq.norm": (3,), "l1.mix.uq": (20, 3), "l1.mix.dkv": (11, 12), "l1.mix.dkv.norm": (7,),
                        "l1.mix.uk": (12, 7), "l1.mix.uv": (10, 7), "l1.mix.g": (2, 12), "l1.mix.o": (12, 10),
                        "l2.mix.q": (4, 12), "l2.mix.q.conv": (4, 3), "l2.mix.v": (12, 12), "l2.mix.v.conv": (12, 3), "l2.mix.b": (2, 12),
                        "l2.mix.a": (2, 12), "l2.mix.A_log": (2,), "l2.mix.dt_bias": (2,), "l2.mix.norm": (6,), "l2.mix.g": (12, 12),
                        "l2.mix.o": (12, 12)}.items():
        assert tuple(names[name].shape) == shape, name
    assert "l1.norm2" not in names and "l1.mlp.router" not in names and "l0.mix.g" not in names      # no feed-forward, no gate
    assert names["head"].optional and not any(n.startswith("l4.") for n in names)
    plain = config_from_dict({k: v for k, v in small_config().items() if k not in ("loop", "logit_softcap")})
    assert [(r.layer, r.cache, r.add_embedding) for r in plain.model_spec().schedule] == [(i, i, False) for i in range(4)]
    assert plain.model_spec().head.softcap is None and "loop" not in plain.to_dict()


def test_configuration_refuses_what_it_cannot_mean():
    from mini_llm_runtime_amd.config import ConfigError, config_from_dict
    import copy

    def broken(change):
        cfg = copy.deepcopy(small_config())
        change(cfg)
        with pytest.raises(ConfigError):
            config_from_dict(cfg)
    broken(lambda c: c["layers"][0]["mixer"].update(heads=3))                    # no multiple of kv_heads
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=3))              # odd
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10))             # more than a map has
    broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=2))              # latent attention turns its whole rotated part
    broken(lambda c: c["layers"][0]["mixer"].pop("mask"))
    broken(lambda c: c["layers"][0]["mixer"].pop("diff"))
    broken(lambda c: c["layers"][2]["mixer"].update(kv_heads=3))
    broken(lambda c: c["layers"][2].update(type="channel_delta"))
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=4))              # more choices than experts
    broken(lambda c: c["layers"][0]["mlp"].update(kind="dense"))
    broken(lambda c: c["loop"].update(stop=5))
    broken(lambda c: c["loop"].update(start=3, stop=2))
    broken(lambda c: c["loop"].update(times=0))
    broken(lambda c: c.update(logit_softcap=0.0))
    broken(lambda c: c.pop("norm"))
    cfg = small_config()
    cfg["layers"][1]["mixer"]["rot"].pop("dims")                                 # (it is rot_dim)
    assert config_from_dict(cfg).model_spec().layers[1].mixer.position.dim == 4
