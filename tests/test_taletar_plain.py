"""Pins of the plain Taletar implementation (tests/plain/taletar_plain.py) that need no GPU: special cases
against library routines, and properties chosen so that a plausible misreading of a mechanism fails them."""
import numpy as np
import pytest
import torch

from plain import taletar_plain as P

RNG = np.random.default_rng(3)


def test_rms_unit_has_eps_inside_the_root_and_matches_the_library():
    x = RNG.normal(size=(5, 12))
    got = P.rms_norm(x, np.ones(12), 1e-5)
    want = torch.nn.functional.rms_norm(torch.from_numpy(x), (12,), eps=1e-5).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-12)
    assert np.allclose(P.rms_unit(np.zeros((1, 4)), 1e-4), 0.0)         # a zero row stays zero: eps is under the root
    tiny = np.full((1, 4), 1e-3)
    assert np.allclose(P.rms_unit(tiny, 1e-2), 1e-3 / np.sqrt(1e-6 + 1e-2))


def test_query_temperature_steps_with_the_position():
    t = P.query_temperature(np.arange(40), 0.5, 8)
    assert np.all(t[:7] == 1.0) and t[7] == pytest.approx(1 + 0.5 * np.log(2))      # position 7: (7 + 1) / 8 = 1
    assert t[14] == t[7] and t[15] == pytest.approx(1 + 0.5 * np.log(3))


def test_capped_scores_stay_below_the_cap_and_are_linear_near_zero():
    q, k = RNG.normal(size=(3, 8)) * 30, RNG.normal(size=(6, 8)) * 30
    s = P.capped_scores(q, k, 0.5, 7.0)
    assert np.abs(s).max() <= 7.0 and np.abs(P.capped_scores(q / 30, k / 30, 0.5, 7.0)).max() < 7.0
    small = P.capped_scores(q * 1e-4, k * 1e-4, 0.5, 7.0)
    np.testing.assert_allclose(small, (q @ k.T) * 0.5e-8, rtol=1e-6)


def test_causal_softmax_matches_the_library_and_sees_its_own_position():
    s = RNG.normal(size=(6, 6))
    p = P.causal_softmax(s)
    assert np.allclose(np.triu(p, 1), 0.0) and np.allclose(p.sum(1), 1.0) and p[0, 0] == 1.0
    q, k, v = (torch.from_numpy(RNG.normal(size=(1, 6, 4))) for _ in range(3))
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.3)[0].numpy()
    got = P.causal_softmax((q[0].numpy() @ k[0].numpy().T) * 0.3) @ v[0].numpy()
    np.testing.assert_allclose(got, want, rtol=1e-10)
    # a portion that starts at position 2 sees keys 0..2 in its first row
    assert np.count_nonzero(P.causal_softmax(RNG.normal(size=(2, 6)), first_position=2)[0]) == 3


def _attention_weights(H, G, D, V, E):
    w = {"q": RNG.normal(size=(H * 2 * D, E)), "k": RNG.normal(size=(G * 2 * D, E)), "v": RNG.normal(size=(G * V, E)),
         "g": RNG.normal(size=(H * V, E)), "o": RNG.normal(size=(E, H * V))}
    for n in ("lq1", "lk1", "lq2", "lk2"):
        w[n] = RNG.normal(size=D) * 0.2
    return w


def test_differential_attention_cancels_when_both_maps_are_equal_and_lambda_is_one():
    H, G, D, V, E = 2, 1, 4, 6, 10
    w = _attention_weights(H, G, D, V, E)
    q = w["q"].reshape(H, 2, D, E)
    q[:, 1] = q[:, 0]
    k = w["k"].reshape(G, 2, D, E)
    k[:, 1] = k[:, 0]
    for n in ("lq1", "lk1", "lq2", "lk2"):
        w[n] = np.zeros(D)                       # lam = 1 - 1 + diff
    cfg = dict(heads=H, kv_heads=G, dim=D, vdim=V, scale=0.5, softcap=20.0, diff=1.0, q_temp=dict(coef=0.3, every=4))
    out = P.differential_attention(RNG.normal(size=(7, E)), w, cfg, 1e-5)
    assert np.abs(out).max() < 1e-9              # o = a - 1 * a = 0; and the factor 1 - diff is 0 too
    cfg["diff"] = 0.25                           # lam = 0.25: o = 0.75 a, normed to unit rms, times 0.75
    h = RNG.normal(size=(7, E))
    one_map = dict(cfg, diff=0.0)                # lam = 0: the first map alone, normed, times 1
    w_o = w["o"]
    a = P.differential_attention(h, w, one_map, 0.0) @ np.linalg.pinv(w_o).T
    b = P.differential_attention(h, w, cfg, 0.0) @ np.linalg.pinv(w_o).T
    np.testing.assert_allclose(b, 0.75 * a, rtol=1e-6, atol=1e-9)


def test_differential_lambda():
    w = dict(lq1=np.array([1.0, 2.0]), lk1=np.array([0.5, 0.25]), lq2=np.array([0.0, 1.0]), lk2=np.array([3.0, -1.0]))
    assert P.differential_lambda(w, 0.6) == pytest.approx(np.exp(1.0) - np.exp(-1.0) + 0.6)


def test_the_recurrence_equals_its_unrolled_sum_and_carries_its_state():
    T, N, V = 9, 3, 4
    q, k, a = RNG.normal(size=(T, N)), RNG.normal(size=(T, N)), RNG.uniform(0.5, 1.0, size=(T, N))
    v = RNG.normal(size=(T, V))
    out, last = P.linear_recurrence(q, k, v, a)
    for t in range(T):
        want = np.zeros(V)
        for s in range(t + 1):
            decay = np.prod(a[s + 1:t + 1], axis=0)          # the decay acts on the key channels, from s + 1 on
            want += (q[t] * decay * k[s]).sum() * v[s]
        np.testing.assert_allclose(out[t], want, rtol=1e-10)
    first, state = P.linear_recurrence(q[:4], k[:4], v[:4], a[:4])
    second, state = P.linear_recurrence(q[4:], k[4:], v[4:], a[4:], state)
    np.testing.assert_allclose(np.concatenate([first, second]), out, rtol=1e-12)
    np.testing.assert_allclose(state, last, rtol=1e-12)


def test_gla_decay_is_a_root_of_the_sigmoid():
    h = RNG.normal(size=(3, 5))
    w = {"a1": RNG.normal(size=(2, 5)), "a2": RNG.normal(size=(6, 2)), "a2.b": RNG.normal(size=6)}
    alpha = P.gla_decay(h, w, dict(heads=2, dim=3, tau=4.0))
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    np.testing.assert_allclose(alpha.reshape(3, 6) ** 4.0, 1 / (1 + np.exp(-z)), rtol=1e-10)
    assert alpha.min() > 0 and alpha.max() < 1


def test_causal_conv_matches_the_library_and_puts_the_last_tap_on_the_current_token():
    T, C, taps = 11, 5, 4
    x, w, b = RNG.normal(size=(T, C)), RNG.normal(size=(C, taps)), RNG.normal(size=C)
    want = torch.nn.functional.conv1d(torch.from_numpy(x.T)[None], torch.from_numpy(w)[:, None, :], torch.from_numpy(b),
                                      padding=taps - 1, groups=C)[0, :, :T].T.numpy()
    np.testing.assert_allclose(P.causal_conv(x, w, b), want, rtol=1e-10)
    only_last = np.zeros((C, taps))
    only_last[:, -1] = 1.0
    np.testing.assert_allclose(P.causal_conv(x, only_last, np.zeros(C)), x)


def test_mamba2_with_one_token_is_its_closed_form():
    H, V, N, G, E = 2, 3, 4, 1, 6
    inner = H * V
    w = {"in": RNG.normal(size=(2 * inner + 2 * G * N + H, E)), "conv": RNG.normal(size=(inner + 2 * G * N, 3)),
         "conv.b": RNG.normal(size=inner + 2 * G * N), "dt_bias": RNG.normal(size=H), "A_log": RNG.normal(size=H),
         "D": RNG.normal(size=H), "norm": RNG.normal(size=inner), "o": np.eye(inner)}
    cfg = dict(heads=H, vdim=V, state=N, groups=G, conv=3, norm_groups=2)
    h = RNG.normal(size=(1, E))
    p = (h @ w["in"].T)[0]
    z, xbc, dt = p[:inner], p[inner:inner + inner + 2 * N], p[-H:]
    xbc = P.silu(xbc * w["conv"][:, -1] + w["conv.b"])            # one token: only the last tap meets an input
    x, B, C = xbc[:inner].reshape(H, V), xbc[inner:inner + N], xbc[inner + N:]
    dt = np.log1p(np.exp(dt + w["dt_bias"]))
    y = (dt[:, None] * x) * (B @ C) + w["D"][:, None] * x          # S_1 = dt B x^T, whatever the decay
    y = (y.reshape(-1) * P.silu(z)).reshape(2, -1)                 # the gate comes before the norm
    y = (y / np.sqrt((y * y).mean(axis=1, keepdims=True) + 1e-5)).reshape(-1) * w["norm"]
    np.testing.assert_allclose(P.mamba2(h, w, cfg, 1e-5)[0], y, rtol=1e-9)


def test_clamped_glu_clamps_one_side_of_the_gate_and_both_of_up():
    w = {"gate": np.eye(2), "up": np.eye(2), "down": np.eye(2)}
    h = np.array([[-5.0, 5.0], [0.5, -0.5]])
    got = P.clamped_glu(h, w, dict(limit=1.0))
    g = np.array([[-5.0, 1.0], [0.5, -0.5]])          # the gate is only clamped from above
    u = np.array([[-1.0, 1.0], [0.5, -0.5]])
    np.testing.assert_allclose(got, g / (1 + np.exp(-1.702 * g)) * (u + 1))
