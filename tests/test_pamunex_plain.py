"""Pins of the plain Pamunex implementation (tests/plain/pamunex_plain.py) that need no GPU: special cases against
library routines, and properties chosen so that a plausible misreading of a mechanism fails them; then the
configuration class: keys, checks and tensor names."""
import numpy as np
import pytest
import torch

from plain import pamunex_plain as P

RNG = np.random.default_rng(11)


def test_layer_norm_matches_the_library_and_norms_what_it_is_given():
    x = RNG.normal(size=(5, 12)) * 3 + 1
    w, b = RNG.normal(size=12), RNG.normal(size=12)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x), (12,), torch.from_numpy(w), torch.from_numpy(b), 1e-5).numpy()
    np.testing.assert_allclose(P.layer_norm(x, w, b, 1e-5), want, rtol=1e-12)
    assert np.allclose(P.layer_norm(np.full((1, 4), 7.0), np.ones(4), np.full(4, 0.5), 1e-5), 0.5)   # a constant row: the bias


def test_rms_norm_has_eps_inside_the_root_and_a_plain_weight():
    x = RNG.normal(size=(3, 8))
    want = torch.nn.functional.rms_norm(torch.from_numpy(x), (8,), torch.full((8,), 2.0, dtype=torch.float64), eps=1e-5).numpy()
    np.testing.assert_allclose(P.rms_norm(x, np.full(8, 2.0), 1e-5), want, rtol=1e-12)
    assert np.allclose(P.rms_norm(np.zeros((1, 4)), np.ones(4), 1e-4), 0.0)
    assert np.allclose(P.rms_norm(x, np.zeros(8), 1e-5), 0.0)                  # the weight itself, not one plus it


def test_rotation_turns_the_first_channels_in_halves_and_leaves_the_rest():
    x = np.zeros((1, 1, 10))
    x[0, 0, 1] = 1.0
    x[0, 0, 7] = 5.0
    y = P.rotate_half_prefix(x, [3], 6, 100.0)                                  # pairs (0,3) (1,4) (2,5); 6.. pass
    angle = 3 * 100.0 ** (-2 / 6)
    assert y[0, 0, 1] == pytest.approx(np.cos(angle)) and y[0, 0, 4] == pytest.approx(np.sin(angle))
    assert y[0, 0, 7] == 5.0 and np.count_nonzero(y) == 3
    assert np.array_equal(P.rotate_half_prefix(x, [0], 6, 100.0), x)            # position 0: nothing turns
    q, k = RNG.normal(size=(2, 1, 8)), RNG.normal(size=(2, 1, 8))
    a = np.sum(P.rotate_half_prefix(q[:1], [9], 8, 50.0) * P.rotate_half_prefix(k[:1], [4], 8, 50.0))
    b = np.sum(P.rotate_half_prefix(q[:1], [25], 8, 50.0) * P.rotate_half_prefix(k[:1], [20], 8, 50.0))
    assert a == pytest.approx(b)                                                # scores depend on distances only


def test_masks_at_their_edges():
    c = P.seen_in_chunk(np.arange(10), 4)
    assert c[3, 0] and c[3, 3] and not c[4, 3] and c[4, 4] and c[7, 4] and not c[8, 7] and not c[2, 3]
    w = P.seen_in_window(np.arange(10), 4)
    assert w[3, 0] and not w[4, 0] and w[4, 1] and w[9, 6] and not w[9, 5] and not w[2, 3] and w[0, 0]
    assert np.array_equal(P.seen_in_window(np.arange(5), 1), np.eye(5, dtype=bool))
    assert np.array_equal(P.seen_in_chunk(np.arange(5), 1), np.eye(5, dtype=bool))
    cut = P.seen_in_chunk(np.arange(6, 10), 4)                                  # positions count from the sequence's start
    assert not cut[2, 1] and cut[2, 2] and cut[1, 0]


def test_sink_softmax_is_a_softmax_with_one_more_summand():
    s = RNG.normal(size=(4, 6))
    seen = np.tril(np.ones((4, 6), dtype=bool), 2)
    p = P.sink_softmax(s, seen, 0.3)
    wide = np.where(seen, s, -np.inf)
    full = torch.softmax(torch.from_numpy(np.concatenate([wide, np.full((4, 1), 0.3)], axis=1)), dim=1).numpy()
    np.testing.assert_allclose(p, full[:, :6], rtol=1e-12)
    assert np.all(p.sum(1) < 1.0)
    np.testing.assert_allclose(P.sink_softmax(s, seen, -1e9).sum(1), 1.0)       # a sink far below: the usual softmax
    assert np.all(P.sink_softmax(s, seen, 50.0).sum(1) < 1e-15 * np.exp(50) )   # a large sink takes nearly everything
    assert P.sink_softmax(s * 0 + 1000.0, seen, 0.0).sum(1).max() <= 1.0        # no overflow


def _attention_weights(H, G, D, V, E, bias=True):
    w = {"q": RNG.normal(size=(H * D, E)), "k": RNG.normal(size=(G * D, E)), "v": RNG.normal(size=(G * V, E)),
         "o": RNG.normal(size=(E, H * V)), "q.norm": RNG.normal(size=D) + 1, "k.norm": RNG.normal(size=D) + 1,
         "sink": RNG.normal(size=H)}
    for n, width in (("q.b", H * D), ("k.b", G * D), ("v.b", G * V)):
        w[n] = RNG.normal(size=width) if bias else np.zeros(width)
    return w


def test_chunked_attention_sees_its_own_chunk_only_and_shares_kv_heads_in_blocks():
    H, G, D, V, E, T = 4, 2, 6, 5, 16, 11
    cfg = dict(heads=H, kv_heads=G, dim=D, vdim=V, scale=0.4, rot=dict(dims=4, base=100.0), mask=dict(size=4))
    w = _attention_weights(H, G, D, V, E)
    x = RNG.normal(size=(T, E))
    out = P.chunked_attention(x, w, cfg, 1e-5)
    again = P.chunked_attention(x[4:8], w, cfg, 1e-5, positions=np.arange(4, 8))
    np.testing.assert_allclose(out[4:8], again, rtol=1e-9)                      # a chunk does not look back
    moved = x.copy()
    moved[3] += 1.0
    assert np.allclose(P.chunked_attention(moved, w, cfg, 1e-5)[4:], out[4:])
    # query heads 0, 1 read kv head 0; heads 2, 3 kv head 1: changing v of kv head 1 leaves the first heads' part of o's input
    w2 = dict(w, o=np.concatenate([w["o"][:, :2 * V], np.zeros((E, 2 * V))], axis=1))
    w3 = dict(w2, v=np.concatenate([w["v"][:V], w["v"][V:] * 2], axis=0))
    np.testing.assert_allclose(P.chunked_attention(x, w2, cfg, 1e-5), P.chunked_attention(x, w3, cfg, 1e-5))


def test_latent_attention_is_attention_with_made_up_keys_and_values():
    H, D, R, V, C, E, T = 3, 4, 6, 5, 7, 12, 9
    cfg = dict(heads=H, dim=D, rot_dim=R, vdim=V, kv_rank=C, scale=0.3, rot=dict(dims=R, base=1000.0), mask=dict(size=3))
    w = {"q": RNG.normal(size=(H * (D + R), E)), "dkv": RNG.normal(size=(C + R, E)), "dkv.norm": RNG.normal(size=C) + 1,
         "uk": RNG.normal(size=(H * D, C)), "uv": RNG.normal(size=(H * V, C)), "sink": RNG.normal(size=H),
         "o": RNG.normal(size=(E, H * V))}
    x = RNG.normal(size=(T, E))
    out = P.latent_attention(x, w, cfg, 1e-5)
    # by hand for the last token and head 1: keys 6, 7, 8
    down = x @ w["dkv"].T
    lat = P.rms_norm(down[:, :C], w["dkv.norm"], 1e-5)
    q = (x[8] @ w["q"].T).reshape(H, D + R)[1]
    q_rot = P.rotate_half_prefix(q[None, None, D:], [8], R, 1000.0)[0, 0]
    scores = []
    for j in (6, 7, 8):
        k_rot = P.rotate_half_prefix(down[j][None, None, C:], [j], R, 1000.0)[0, 0]
        scores.append((q[:D] @ (w["uk"][D:2 * D] @ lat[j]) + q_rot @ k_rot) * 0.3)
    e = np.exp(scores)
    p = e / (e.sum() + np.exp(w["sink"][1]))
    head = sum(pj * (w["uv"][V:2 * V] @ lat[j]) for pj, j in zip(p, (6, 7, 8)))
    rest = dict(w, o=np.concatenate([np.zeros((E, V)), w["o"][:, V:2 * V], np.zeros((E, V))], axis=1))
    np.testing.assert_allclose(P.latent_attention(x, rest, cfg, 1e-5)[8], w["o"][:, V:2 * V] @ head, rtol=1e-9)
    far = x.copy()
    far[5] += 1.0                                                               # outside the last token's window of 3
    np.testing.assert_allclose(P.latent_attention(far, w, cfg, 1e-5)[8], out[8], rtol=1e-9)


def test_routing_keeps_the_best_groups_and_uses_scores_as_weights():
    E = 6
    router = dict(experts=8, top=3, groups=dict(count=4, keep=2))
    w = {"router": np.eye(8, E + 2)[:, :E] * 0}
    z = np.array([[3.0, -1.0, 2.5, 2.4, 0.1, 0.2, 2.9, -3.0]])                  # groups (0,1) (2,3) (4,5) (6,7)
    w = {"router": z.T @ np.ones((1, E)) / E}
    chosen, weights = P.route(np.ones((1, E)), w, router)
    s = 1 / (1 + np.exp(-z[0]))
    # group sums of their two largest: 0: s0+s1, 1: s2+s3 (largest), 3: s6+s7; the best two groups are 1 and 0
    assert sorted(chosen[0].tolist()) == [0, 2, 3] and chosen[0, 0] == 0        # expert 6 scores high but its group is out
    np.testing.assert_allclose(weights[0], s[chosen[0]])
    assert weights.sum() > 1.0                                                  # not renormalized
    one = dict(experts=8, top=2, groups=dict(count=8, keep=3))                  # groups of one expert: its own score
    chosen, _ = P.route(np.ones((1, E)), w, one)
    assert chosen[0].tolist() == [0, 6]
    x = RNG.normal(size=(5, E))
    we = {"router": RNG.normal(size=(8, E))}
    for e in range(8):
        we[f"e{e}.up"], we[f"e{e}.down"] = RNG.normal(size=(7, E)), RNG.normal(size=(E, 7))
    everything = dict(experts=8, top=8, groups=dict(count=1, keep=1))
    s = 1 / (1 + np.exp(-(x @ we["router"].T)))
    want = sum(s[:, e:e + 1] * (np.maximum(x @ we[f"e{e}.up"].T, 0) ** 2 @ we[f"e{e}.down"].T) for e in range(8))
    np.testing.assert_allclose(P.moe_ffn(x, we, dict(kind="moe", router=everything)), want, rtol=1e-9)


# ---- the configuration class ---------------------------------------------------------------------------------
def tiny_config():
    return dict(architecture="Pamunex", vocab=50, width=24, norm=dict(eps=1e-5), logit_scale=0.5, layers=[
        dict(type="latent_attention", mixer=dict(heads=2, dim=4, rot_dim=6, vdim=5, kv_rank=9, scale=0.3, rot=dict(dims=6, base=100.0),
                                                 mask=dict(size=7)), mlp=dict(kind="dense", ff=20)),
        dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=6, vdim=3, scale=0.4, rot=dict(dims=4, base=1000.0), mask=dict(size=5)),
             mlp=dict(kind="moe", expert=dict(ff=10), router=dict(experts=6, top=2, groups=dict(count=3, keep=2)))),
        dict(type="attention", mixer=dict(heads=1, kv_heads=1, dim=8, vdim=8, scale=0.35, rot=dict(dims=8, base=10.0), mask=dict(size=1)),
             mlp=None)])


def test_configuration_reads_every_size_and_names_every_tensor():
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.parts import expected_tensors
    config = config_from_dict(tiny_config())
    assert config.to_dict() == tiny_config()
    spec = config.model_spec()
    assert spec.layers[0].mixer.rank == 9 and spec.layers[0].mixer.mask.kind == "window" and spec.layers[0].mixer.mask.size == 7
    assert spec.layers[1].mixer.mask.kind == "chunk" and spec.layers[1].mixer.position.dim == 4
    assert spec.layers[1].ffn.group_count == 3 and spec.layers[1].ffn.group_keep == 2 and spec.layers[2].ffn is None
    assert spec.head.scale == 0.5 and spec.head.tied
    names = {n: tuple(ws.shape) for n, ws in expected_tensors(config).items() if not ws.optional}
    assert names["l0.mix.q"] == (20, 24) and names["l0.mix.dkv"] == (15, 24) and names["l0.mix.dkv.norm"] == (9,)
    assert names["l0.mix.uk"] == (8, 9) and names["l0.mix.uv"] == (10, 9) and names["l0.mix.sink"] == (2,)
    assert names["l1.mix.q.b"] == (24,) and names["l1.mix.v"] == (6, 24) and names["l1.mix.k.norm"] == (6,)
    assert names["l1.mlp.e5.down"] == (24, 10) and names["l1.mlp.router"] == (6, 24) and names["l0.mlp.up"] == (20, 24)
    assert names["l2.norm1.b"] == (24,) and "l2.norm2" not in names and names["final.norm.b"] == (24,) and names["embed"] == (50, 24)


@pytest.mark.parametrize("change,text", [
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=4), "rot_dim"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=8), "exceeds"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "choices"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "choices"),
    (lambda c: c["layers"][2].update(type="conv"), "none of"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "mask"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_configuration_refuses_what_does_not_fit(change, text):
    from mini_llm_runtime_amd.config import ConfigError, config_from_dict
    cfg = tiny_config()
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(cfg)
