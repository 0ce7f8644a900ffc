"""Pins of the plain Tigelorn implementation (tests/plain/tigelorn_plain.py) that need no GPU: special cases against
library routines, and properties chosen so that a plausible misreading of a mechanism fails them; then the
configuration class (keys, checks, tensor names, layers that share tensors) and the position part's frequencies."""
import numpy as np
import pytest
import torch

from plain import tigelorn_plain as P

RNG = np.random.default_rng(23)


def test_norms_have_eps_inside_the_root_and_differ_in_what_the_weight_means():
    x = RNG.normal(size=(3, 8))
    want = torch.nn.functional.rms_norm(torch.from_numpy(x), (8,), torch.full((8,), 2.0, dtype=torch.float64), eps=1e-5).numpy()
    np.testing.assert_allclose(P.norm_plain(x, np.full(8, 2.0), 1e-5), want, rtol=1e-12)
    np.testing.assert_allclose(P.norm_around_zero(x, np.full(8, 1.0), 1e-5), want, rtol=1e-12)
    assert np.allclose(P.norm_plain(x, np.zeros(8), 1e-5), 0.0)
    np.testing.assert_allclose(P.norm_around_zero(x, np.zeros(8), 1e-5), x / P.rms(x, 1e-5))      # zero weight: factor one
    assert np.allclose(P.norm_plain(np.zeros((1, 4)), np.ones(4), 1e-4), 0.0)


def test_activations_match_the_library():
    z = torch.from_numpy(RNG.normal(size=50) * 4)
    np.testing.assert_allclose(P.gelu_tanh(z.numpy()), torch.nn.functional.gelu(z, approximate="tanh").numpy(), rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(P.silu(z.numpy()), torch.nn.functional.silu(z).numpy(), rtol=1e-12)
    np.testing.assert_allclose(P.softplus(z.numpy()), torch.nn.functional.softplus(z).numpy(), rtol=1e-12)
    assert P.softplus(np.array([800.0]))[0] == 800.0 and P.softplus(np.array([-800.0]))[0] == 0.0
    assert abs(P.gelu_tanh(np.array([1.0]))[0] - 0.8411919906) < 1e-9            # not the erf form (0.8413447)


def test_pair_rows_hash_the_token_before_and_the_token():
    rows = P.bigram_rows([5, 9, 9, 0], buckets=11, mul_prev=7, mul_cur=3)
    assert rows.tolist() == [11, (5 * 7 + 9 * 3) % 11, (9 * 7 + 9 * 3) % 11, (9 * 7) % 11]
    table, pairs = RNG.normal(size=(12, 4)), RNG.normal(size=(12, 4))
    x = P.embed([5, 9], table, pairs, dict(bigram=dict(buckets=11, mul_prev=7, mul_cur=3)))
    np.testing.assert_allclose(x[0], table[5] + pairs[11])                        # a sequence's first token: the last row
    np.testing.assert_allclose(x[1], table[9] + pairs[(35 + 27) % 11])
    assert P.bigram_rows([3], 1, 5, 5).tolist() == [1] and P.bigram_rows([3, 4], 1, 5, 5).tolist() == [1, 0]


def test_rotation_pairs_halves_or_neighbours_and_leaves_the_rest():
    x = np.zeros((1, 1, 10))
    x[0, 0, 1] = 1.0
    x[0, 0, 7] = 5.0
    angle = 3 * 100.0 ** (-2 / 6)
    y = P.rotate(x, [3], 6, 100.0, interleaved=False)                            # pairs (0,3) (1,4) (2,5); 6.. pass
    assert y[0, 0, 1] == pytest.approx(np.cos(angle)) and y[0, 0, 4] == pytest.approx(np.sin(angle))
    assert y[0, 0, 7] == 5.0 and np.count_nonzero(y) == 3
    x2 = np.zeros((1, 1, 10))
    x2[0, 0, 2] = 1.0                                                             # pairs (0,1) (2,3) (4,5): channel 2 is u of pair 1
    y2 = P.rotate(x2, [3], 6, 100.0, interleaved=True)
    assert y2[0, 0, 2] == pytest.approx(np.cos(angle)) and y2[0, 0, 3] == pytest.approx(np.sin(angle))
    assert np.count_nonzero(y2) == 2
    assert np.array_equal(P.rotate(x, [0], 6, 100.0, True), x)                  # position 0: nothing turns
    q, k = RNG.normal(size=(1, 1, 8)), RNG.normal(size=(1, 1, 8))
    for inter in (False, True):
        a = np.sum(P.rotate(q, [9], 8, 50.0, inter) * P.rotate(k, [4], 8, 50.0, inter))
        b = np.sum(P.rotate(q, [25], 8, 50.0, inter) * P.rotate(k, [20], 8, 50.0, inter))
        assert a == pytest.approx(b)                                             # scores depend on distances only
        assert np.sum(P.rotate(q, [9], 8, 50.0, inter) ** 2) == pytest.approx(np.sum(q ** 2))


def test_stretched_frequencies_keep_the_fast_pairs_and_slow_the_others():
    scaling = dict(factor=4.0, original=64, fast=8.0, slow=1.0)
    f, amp = P.yarn_frequencies(16, 100.0, scaling)
    plain, one = P.yarn_frequencies(16, 100.0, None)
    assert one == 1.0 and amp == pytest.approx(0.1 * np.log(4.0) + 1.0)
    np.testing.assert_allclose(plain, 100.0 ** (-np.arange(8) / 8.0))
    place = lambda t: 16 * np.log(64 / (2 * np.pi * t)) / (2 * np.log(100.0))
    lo, hi = max(np.floor(place(8.0)), 0), min(np.ceil(place(1.0)), 15)
    assert lo < hi
    for i in range(8):
        ramp = min(max((i - lo) / (hi - lo), 0.0), 1.0)
        assert f[i] == pytest.approx(plain[i] * (1 - ramp) + plain[i] / 4.0 * ramp)
    assert f[0] == plain[0] and f[7] == pytest.approx(plain[7] / 4.0)            # the two ends of the ramp
    same, amp1 = P.yarn_frequencies(16, 100.0, dict(factor=1.0, original=64, fast=8.0, slow=1.0))
    np.testing.assert_allclose(same, plain)
    assert amp1 == 1.0
    # cosines and sines carry the factor: a turned vector grows by it
    x = RNG.normal(size=(1, 1, 16))
    assert np.sum(P.rotate(x, [5], 16, 100.0, True, scaling) ** 2) == pytest.approx(amp ** 2 * np.sum(x ** 2))
    # lo == hi: the ramp's width falls back to 0.001, a step
    step, _ = P.yarn_frequencies(8, 10.0, dict(factor=2.0, original=2 * np.pi * 10.0, fast=1.0, slow=1.0))
    base = 10.0 ** (-np.arange(4) / 4.0)
    np.testing.assert_allclose(step, base, rtol=1e-9)                            # lo = hi = 4: every pair lies below the step


def test_masks_and_softmax():
    w = P.seen_in_window(10, 4)
    assert w[3, 0] and not w[4, 0] and w[4, 1] and w[9, 6] and not w[9, 5] and not w[2, 3] and w[0, 0]
    assert np.array_equal(P.seen_in_window(5, 1), np.eye(5, dtype=bool))
    assert np.array_equal(P.seen_causal(4), np.tril(np.ones((4, 4), dtype=bool)))
    s = RNG.normal(size=(4, 4))
    p = P.masked_softmax(s, P.seen_causal(4))
    want = torch.softmax(torch.from_numpy(np.where(P.seen_causal(4), s, -np.inf)), dim=1).numpy()
    np.testing.assert_allclose(p, want, rtol=1e-12)


def test_window_attention_against_the_library_and_its_order_of_rotation_and_norm():
    T, E = 9, 12
    cfg = dict(heads=4, kv_heads=2, dim=6, vdim=5, scale=0.7, rot=dict(dims=4, base=50.0), mask=dict(size=3))
    w = {n: RNG.normal(size=s) * 0.5 for n, s in dict(q=(24, E), k=(12, E), v=(10, E), g=(20, E), o=(E, 20)).items()}
    w.update({"q.b": RNG.normal(size=24), "k.b": RNG.normal(size=12), "v.b": RNG.normal(size=10)})
    x = RNG.normal(size=(T, E))
    got = P.window_attention(x, w, cfg, 1e-5)
    q = (x @ w["q"].T + w["q.b"]).reshape(T, 4, 6)
    k = (x @ w["k"].T + w["k.b"]).reshape(T, 2, 6)
    v = (x @ w["v"].T + w["v.b"]).reshape(T, 2, 5)
    q, k = P.rotate(q, np.arange(T), 4, 50.0, False), P.rotate(k, np.arange(T), 4, 50.0, False)
    q, k = q / P.rms(q, 1e-5), k / P.rms(k, 1e-5)
    tq, tk, tv = (torch.from_numpy(a.transpose(1, 0, 2)) for a in (q, np.repeat(k, 2, axis=1), np.repeat(v, 2, axis=1)))
    mask = torch.from_numpy(P.seen_in_window(T, 3))
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask, scale=0.7).numpy().transpose(1, 0, 2)
    want = (ref.reshape(T, 20) * P.sigmoid(x @ w["g"].T)) @ w["o"].T
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)
    # a query's own length does not matter (it is normed), the values' does
    w2 = dict(w, q=w["q"] * 3.0)
    w2["q.b"] = w["q.b"] * 3.0
    np.testing.assert_allclose(P.window_attention(x, w2, cfg, 1e-12), P.window_attention(x, w, cfg, 1e-12), rtol=1e-6)


def test_latent_attention_by_hand_for_one_head_and_in_the_form_that_reads_only_the_cache_row():
    T, E = 7, 10
    cfg = dict(heads=2, dim=4, rot_dim=4, vdim=3, kv_rank=5, q_rank=6, scale=0.4,
               rot=dict(dims=4, base=30.0, scaling=dict(factor=2.0, original=8, fast=4.0, slow=1.0)))
    w = {n: RNG.normal(size=s) * 0.6 for n, s in dict(dq=(6, E), uq=(16, 6), dkv=(9, E), uk=(8, 5), uv=(6, 5), o=(E, 6)).items()}
    w["dq.norm"], w["dkv.norm"] = RNG.normal(size=6) + 1, RNG.normal(size=5) + 1
    x = RNG.normal(size=(T, E))
    got = P.latent_attention(x, w, cfg, 1e-5)
    # the other form: the key up-projection moved to the query, attention over [latent | rotated part] rows
    q = (P.norm_plain(x @ w["dq"].T, w["dq.norm"], 1e-5) @ w["uq"].T).reshape(T, 2, 8)
    down = x @ w["dkv"].T
    lat = P.norm_plain(down[:, :5], w["dkv.norm"], 1e-5)
    sc = cfg["rot"]["scaling"]
    kr = P.rotate(down[:, None, 5:], np.arange(T), 4, 30.0, True, sc)[:, 0]
    qr = P.rotate(q[..., 4:], np.arange(T), 4, 30.0, True, sc)
    heads = []
    for h in range(2):
        q_lat = q[:, h, :4] @ w["uk"].reshape(2, 4, 5)[h]                        # [T, rank]
        s = (q_lat @ lat.T + qr[:, h] @ kr.T) * 0.4
        heads.append((P.masked_softmax(s, P.seen_causal(T)) @ lat) @ w["uv"].reshape(2, 3, 5)[h].T)
    np.testing.assert_allclose(got, np.concatenate(heads, axis=1) @ w["o"].T, rtol=1e-9, atol=1e-12)
    # the first token attends to itself alone: its heads are its own values
    v0 = (lat[:1] @ w["uv"].T)
    np.testing.assert_allclose(got[0], (v0 @ w["o"].T)[0], rtol=1e-9)


def test_short_convolution_matches_the_library():
    x, taps = RNG.normal(size=(11, 3)), RNG.normal(size=(3, 4))
    want = torch.nn.functional.conv1d(torch.from_numpy(x.T)[None], torch.from_numpy(taps)[:, None, :], padding=3, groups=3)[0, :, :11].numpy().T
    np.testing.assert_allclose(P.short_convolution(x, taps), want, rtol=1e-12, atol=1e-14)
    assert np.allclose(P.short_convolution(x, taps)[0], x[0] * taps[:, -1])       # the last column is the current token's
    np.testing.assert_allclose(P.short_convolution(x, taps[:, -1:]), x * taps[:, -1])


def test_decayed_sum_attention_is_its_unrolled_sum():
    T, E = 8, 6
    cfg = dict(heads=2, dim=3, vdim=4, decay=[0.5, 1.0])
    w = {n: RNG.normal(size=s) for n, s in dict(q=(6, E), k=(6, E), v=(8, E), g=(8, E), o=(E, 8)).items()}
    w["norm"] = RNG.normal(size=8) + 1
    x = RNG.normal(size=(T, E))
    q, k, v = (P.silu(x @ w[n].T).reshape(T, 2, -1) for n in "qkv")
    out = np.zeros((T, 2, 4))
    for h in range(2):
        for t in range(T):
            for s in range(t + 1):
                out[t, h] += cfg["decay"][h] ** (t - s) * (q[t, h] @ k[s, h]) * v[s, h]
    want = (P.norm_plain(out.reshape(T, 8), w["norm"], 1e-5) * P.sigmoid(x @ w["g"].T)) @ w["o"].T
    np.testing.assert_allclose(P.decayed_sum_attention(x, w, cfg, 1e-5), want, rtol=1e-10)


def test_delta_rule_overwrites_what_a_key_held_and_reads_after_it_wrote():
    D, V = 4, 3
    keys = np.eye(D)
    ones, no_decay = np.ones(5), np.ones((5, D))
    k = np.stack([keys[0], keys[1], keys[0], keys[2], keys[0]])
    v = RNG.normal(size=(5, V))
    out = P.delta_rule(k, k, v, ones, no_decay)                                  # beta 1, unit keys: a key holds its last value
    np.testing.assert_allclose(out, v, atol=1e-12)                              # the read-out sees the token's own write
    q = np.stack([keys[0]] * 5)
    got = P.delta_rule(q, k, v, ones, no_decay)
    np.testing.assert_allclose(got, [v[0], v[0], v[2], v[2], v[4]], atol=1e-12)   # overwritten, not added up
    half = P.delta_rule(q, k, v, np.full(5, 0.5), no_decay)
    np.testing.assert_allclose(half[2], 0.5 * v[2] + 0.25 * v[0], atol=1e-12)     # beta: how much of the difference is written
    g = np.ones((5, D))
    g[1:, 0] = 0.5                                                               # channel 0 decays, the others do not
    decayed = P.delta_rule(q, k, v, ones, g)
    np.testing.assert_allclose(decayed[1], 0.5 * v[0], atol=1e-12)              # decay comes before the token's write and read
    np.testing.assert_allclose(decayed[2], v[2], atol=1e-12)
    # two tokens in closed form with general vectors
    q2, k2, v2, b2, g2 = RNG.normal(size=(2, D)), RNG.normal(size=(2, D)), RNG.normal(size=(2, V)), RNG.random(2), RNG.random((2, D))
    S1 = np.outer(k2[0], b2[0] * v2[0])
    S1d = g2[1][:, None] * S1
    S2 = S1d + np.outer(k2[1], b2[1] * (v2[1] - S1d.T @ k2[1]))
    np.testing.assert_allclose(P.delta_rule(q2, k2, v2, b2, g2), [S1.T @ q2[0], S2.T @ q2[1]], rtol=1e-12)


def test_channel_delta_shares_keys_between_heads_and_norms_each_head():
    T, E = 6, 8
    cfg = dict(heads=4, kv_heads=2, dim=3, vdim=2, conv=3)
    shapes = dict(q=(6, E), k=(6, E), v=(8, E), b=(4, E), a1=(2, E), a2=(12, 2), g1=(2, E), g2=(8, 2), o=(E, 8))
    w = {n: RNG.normal(size=s) * 0.7 for n, s in shapes.items()}
    w.update({"q.conv": RNG.normal(size=(6, 3)), "k.conv": RNG.normal(size=(6, 3)), "v.conv": RNG.normal(size=(8, 3)),
              "dt_bias": RNG.normal(size=12), "A_log": RNG.normal(size=4), "norm": RNG.normal(size=2) + 1})
    x = RNG.normal(size=(T, E))
    got = P.channel_delta(x, w, cfg, 1e-5)
    q = P.silu(P.short_convolution(x @ w["q"].T, w["q.conv"])).reshape(T, 2, 3)
    k = P.silu(P.short_convolution(x @ w["k"].T, w["k.conv"])).reshape(T, 2, 3)
    v = P.silu(P.short_convolution(x @ w["v"].T, w["v.conv"])).reshape(T, 4, 2)
    q = q / np.sqrt((q ** 2).sum(-1, keepdims=True) + 1e-6) / np.sqrt(3.0)
    k = k / np.sqrt((k ** 2).sum(-1, keepdims=True) + 1e-6)
    beta = P.sigmoid(x @ w["b"].T)
    g = np.exp(-np.exp(w["A_log"])[None, :, None] * P.softplus((x @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).reshape(T, 4, 3))
    assert (g > 0).all() and (g < 1).all()
    heads = []
    for h in range(4):
        o = P.delta_rule(q[:, h // 2], k[:, h // 2], v[:, h], beta[:, h], g[:, h])
        heads.append(o / np.sqrt((o ** 2).mean(-1, keepdims=True) + 1e-5) * w["norm"])
    want = (np.concatenate(heads, axis=1) * P.sigmoid((x @ w["g1"].T) @ w["g2"].T)) @ w["o"].T
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)
    # causal: a later token changes nothing before it
    x2 = x.copy()
    x2[4] += 1.0
    np.testing.assert_allclose(P.channel_delta(x2, w, cfg, 1e-5)[:4], got[:4], rtol=1e-12)


# ---- the configuration --------------------------------------------------------------------------------------
def tiny_config():
    left = dict(heads=4, kv_heads=2, dim=8, vdim=4, scale=0.3, rot=dict(dims=4, base=100.0), mask=dict(size=5))
    right = dict(heads=2, dim=4, vdim=6, decay=[0.9, 1.0])
    par = dict(type="parallel", mixer=dict(left=left, right=right, left_scale=0.5, right_scale=2.0), mlp=dict(kind="dense", ff=24))
    delta = dict(type="channel_delta", mixer=dict(heads=2, kv_heads=1, dim=4, vdim=6, conv=3, decay_rank=3, gate_rank=2), mlp=None)
    lat = dict(type="latent_attention", mlp=dict(kind="dense", ff=20),
               mixer=dict(heads=2, dim=4, rot_dim=2, vdim=6, kv_rank=5, q_rank=7, scale=0.4,
                          rot=dict(dims=2, base=10.0, scaling=dict(factor=2.0, original=16, fast=4.0, slow=1.0))))
    return dict(architecture="Tigelorn", vocab=50, width=16, norm=dict(eps=1e-5),
                embedding=dict(bigram=dict(buckets=13, mul_prev=3, mul_cur=5)),
                layers=[par, delta, lat, dict(delta, weights_of=1), dict(par, weights_of=0)])


def test_configuration_names_every_tensor_and_runs_shared_layers_against_caches_of_their_own():
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.parts import expected_tensors
    cfg = config_from_dict(tiny_config())
    assert config_from_dict(cfg.to_dict()) == cfg
    spec = cfg.model_spec()
    assert [(r.layer, r.cache) for r in spec.schedule] == [(0, 0), (1, 1), (2, 2), (1, 3), (0, 4)]
    assert len(spec.layers) == 3 and spec.layers[1].ffn is None and spec.layers[1].norm2 is None
    names = expected_tensors(cfg)
    assert names["bigram"].shape == (14, 16) and names["embed"].shape == (50, 16) and names["final.norm"].shape == (16,)
    assert names["l0.mix.left.q"].shape == (32, 16) and names["l0.mix.left.q.b"].shape == (32,)
    assert names["l0.mix.left.g"].shape == (16, 16) and names["l0.mix.left.o"].shape == (16, 16)
    assert names["l0.mix.right.norm"].shape == (12,) and names["l0.mix.right.o"].shape == (16, 12)
    assert names["l0.mlp.gate"].shape == (24, 16) and names["l0.mlp.down"].shape == (16, 24)
    assert names["l1.mix.q.conv"].shape == (4, 3) and names["l1.mix.v.conv"].shape == (12, 3)
    assert names["l1.mix.a2"].shape == (8, 3) and names["l1.mix.dt_bias"].shape == (8,) and names["l1.mix.A_log"].shape == (2,)
    assert names["l1.mix.g2"].shape == (12, 2) and names["l1.mix.b"].shape == (2, 16) and names["l1.mix.norm"].shape == (6,)
    assert "l1.norm2" not in names and "l1.mlp.gate" not in names
    assert names["l2.mix.dq"].shape == (7, 16) and names["l2.mix.uq"].shape == (12, 7) and names["l2.mix.dkv"].shape == (7, 16)
    assert names["l2.mix.dkv.norm"].shape == (5,) and names["l2.mix.uk"].shape == (8, 5) and names["l2.mix.uv"].shape == (12, 5)
    assert not any(n.startswith(("l3.", "l4.")) for n in names)                  # they use other layers' tensors
    assert "l0.mix.left.sink" not in names and "l0.mix.left.q.norm" not in names
    # without the ranks the tensors say them
    plain = tiny_config()
    for key in ("decay_rank", "gate_rank"):
        plain["layers"][1]["mixer"].pop(key)                                     # (layer 3's entry is the same object)
        assert key not in plain["layers"][3]["mixer"]
    open_names = expected_tensors(config_from_dict(plain))
    assert open_names["l1.mix.a1"].shape == (None, 16) and open_names["l1.mix.a2"].shape == (8, None)


def test_configuration_refuses_what_it_cannot_mean():
    from mini_llm_runtime_amd.config import ConfigError, config_from_dict

    def broken(change):
        cfg = tiny_config()
        change(cfg)
        with pytest.raises(ConfigError):
            config_from_dict(cfg)
    broken(lambda c: c.pop("embedding"))
    broken(lambda c: c["layers"][0].update(type="attention"))
    broken(lambda c: c["layers"][0]["mixer"]["left"].update(heads=3))
    broken(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=10))
    broken(lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5]))
    broken(lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5, 1.5]))
    broken(lambda c: c["layers"][0]["mixer"].pop("left_scale"))
    broken(lambda c: c["layers"][2]["mixer"]["rot"].update(dims=4))
    broken(lambda c: c["layers"][2]["mixer"].pop("q_rank"))
    broken(lambda c: c["layers"][3].update(weights_of=3))
    broken(lambda c: c["layers"][3].update(weights_of=9))
    broken(lambda c: c["layers"][3].update(weights_of=0))
    broken(lambda c: c["layers"][0].update(mlp=dict(kind="moe", ff=8)))


def test_position_part_computes_the_plain_frequencies_in_32_bit():
    from mini_llm_runtime_amd.config.specs import FrequencyStretch, PositionSpec
    from mini_llm_runtime_amd.parts.rope import Rope
    for dims, base, scaling in ((24, 5000.0, dict(factor=3.0, original=1024, fast=16.0, slow=1.0)), (6, 50.0, None),
                                (16, 100.0, dict(factor=1.5, original=64, fast=8.0, slow=2.0))):
        stretch = FrequencyStretch(**scaling) if scaling else None
        freq, amp = Rope(PositionSpec("rope", dims, base, interleaved=True, stretch=stretch)).frequencies()
        want, want_amp = P.yarn_frequencies(dims, base, scaling)
        assert freq.dtype == np.float32
        np.testing.assert_allclose(freq, want, rtol=1e-7)
        assert amp == pytest.approx(want_amp)
