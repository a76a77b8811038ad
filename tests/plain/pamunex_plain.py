"""A plain, slow implementation of the Pamunex decoder in float64 numpy: whole sequences, no cache, no
batching, one function per mechanism.  It shares no code with the engine; the engine's tests compare
against it.

Notation: x [T, E] is the residual stream of one sequence, positions count from 0, linear weights are
[out, in] and applied as x @ W.T.  `cfg` is a mixer's (or feed-forward's) entry of config.json, `w` maps
the last part of a tensor's name ("q", "q.b", "dkv.norm", "e3.up", ...) to an array.
"""
from __future__ import annotations

import numpy as np


def rms_norm(x, weight, eps):
    """x over its root mean square along the last axis (eps inside the root), times the weight itself."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * weight


def layer_norm(x, weight, bias, eps):
    """Mean taken off, divided by the root of the mean squared deviation plus eps; weight and bias."""
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * weight + bias


def rotate_half_prefix(x, positions, dims, base):
    """x [T, heads, D]: the first `dims` channels of every head turned by the token's position, channel i
    paired with channel i + dims/2, angle position * base^(-2 i / dims); the other channels pass."""
    half = dims // 2
    freq = base ** (-2.0 * np.arange(half) / dims)
    angle = np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :]
    c, s = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    out = np.array(x, dtype=np.float64, copy=True)
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def seen_in_chunk(positions, size):
    """[T, T] mask: query i sees key j when j <= i and both lie in the same block of `size` positions."""
    p = np.asarray(positions)
    return (p[None, :] <= p[:, None]) & ((p[None, :] // size) == (p[:, None] // size))


def seen_in_window(positions, size):
    """[T, T] mask: query i sees key j when 0 <= i - j < size."""
    p = np.asarray(positions)
    d = p[:, None] - p[None, :]
    return (d >= 0) & (d < size)


def sink_softmax(scores, seen, sink):
    """Softmax over the seen keys of each row with one more summand exp(sink) in the denominator, which
    stands for no key and brings no value."""
    s = np.where(seen, scores, -np.inf)
    top = np.maximum(s.max(axis=1, keepdims=True), sink)
    p = np.exp(s - top)
    return p / (p.sum(axis=1, keepdims=True) + np.exp(sink - top))


def chunked_attention(x, w, cfg, eps, positions=None):
    """The mixer `attention`: biased q/k/v, a norm per head of q and k, a rotation of a head's first channels,
    keys of the query's own block of positions, a sink in the softmax."""
    T = x.shape[0]
    positions = np.arange(T) if positions is None else positions
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = (x @ w["q"].T + w["q.b"]).reshape(T, H, D)
    k = (x @ w["k"].T + w["k.b"]).reshape(T, G, D)
    v = (x @ w["v"].T + w["v.b"]).reshape(T, G, V)
    q = rms_norm(q, w["q.norm"], eps)
    k = rms_norm(k, w["k.norm"], eps)
    q = rotate_half_prefix(q, positions, cfg["rot"]["dims"], cfg["rot"]["base"])
    k = rotate_half_prefix(k, positions, cfg["rot"]["dims"], cfg["rot"]["base"])
    seen = seen_in_chunk(positions, cfg["mask"]["size"])
    heads = []
    for head in range(H):
        g = head // (H // G)
        p = sink_softmax((q[:, head] @ k[:, g].T) * cfg["scale"], seen, w["sink"][head])
        heads.append(p @ v[:, g])
    return np.concatenate(heads, axis=1) @ w["o"].T


def latent_attention(x, w, cfg, eps, positions=None):
    """The mixer `latent_attention`: keys and values of all heads made from one normed latent vector a token,
    plus one rotated key part that all heads share; a sliding window; a sink in the softmax."""
    T = x.shape[0]
    positions = np.arange(T) if positions is None else positions
    H, D, R, V, C = cfg["heads"], cfg["dim"], cfg["rot_dim"], cfg["vdim"], cfg["kv_rank"]
    q = (x @ w["q"].T).reshape(T, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    down = x @ w["dkv"].T
    latent = rms_norm(down[:, :C], w["dkv.norm"], eps)
    k_rot = down[:, None, C:]                                        # [T, 1, R]
    q_rot = rotate_half_prefix(q_rot, positions, R, cfg["rot"]["base"])
    k_rot = rotate_half_prefix(k_rot, positions, R, cfg["rot"]["base"])[:, 0]
    k_plain = (latent @ w["uk"].T).reshape(T, H, D)
    v = (latent @ w["uv"].T).reshape(T, H, V)
    seen = seen_in_window(positions, cfg["mask"]["size"])
    heads = []
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * cfg["scale"]
        heads.append(sink_softmax(s, seen, w["sink"][head]) @ v[:, head])
    return np.concatenate(heads, axis=1) @ w["o"].T


def relu_squared(z):
    return np.maximum(z, 0.0) ** 2


def dense_ffn(x, w):
    return relu_squared(x @ w["up"].T) @ w["down"].T


def route(x, w, router):
    """(chosen experts [T, top], their weights [T, top]): sigmoid scores; experts in `groups.count` blocks of
    neighbours, a block's score the sum of its two largest scores, only the best `groups.keep` blocks stay;
    of the experts that stay the `top` largest scores, used as weights as they are."""
    n, top = router["experts"], router["top"]
    count, keep = router["groups"]["count"], router["groups"]["keep"]
    s = 1.0 / (1.0 + np.exp(-(x @ w["router"].T)))                   # [T, n]
    per = n // count
    blocks = s.reshape(-1, count, per)
    best_two = np.sort(blocks, axis=2)[:, :, -2:].sum(axis=2) if per >= 2 else blocks.sum(axis=2)
    order = np.argsort(-best_two, axis=1, kind="stable")[:, :keep]
    allowed = np.zeros((s.shape[0], count), dtype=bool)
    np.put_along_axis(allowed, order, True, axis=1)
    masked = np.where(np.repeat(allowed, per, axis=1), s, -np.inf)
    chosen = np.argsort(-masked, axis=1, kind="stable")[:, :top]
    return chosen, np.take_along_axis(s, chosen, axis=1)


def route_margin(x, w, router, rounding=2.0 ** -8):
    """[T]: how far each token's choice is from another one, in units of what rounding x to `rounding` (relative,
    per element) may move a score: the smaller of the gap between the last group kept and the first one dropped and
    the gap between the last expert chosen and the best one left (infinite where nothing is left out), over the
    largest such move among the token's scores.  A test that compares a rounded engine with this file may not rest
    on tokens whose margin is a small number."""
    n, top = router["experts"], router["top"]
    count, keep = router["groups"]["count"], router["groups"]["keep"]
    s = 1.0 / (1.0 + np.exp(-(x @ w["router"].T)))
    moved = (s * (1.0 - s) * rounding * np.sqrt((x * x) @ (w["router"] ** 2).T)).max(axis=1) + 1e-300
    per = n // count
    blocks = s.reshape(-1, count, per)
    best_two = np.sort(blocks, axis=2)[:, :, -2:].sum(axis=2) if per >= 2 else blocks.sum(axis=2)
    ranked = -np.sort(-best_two, axis=1)
    group_gap = ranked[:, keep - 1] - ranked[:, keep] if keep < count else np.full(s.shape[0], np.inf)
    order = np.argsort(-best_two, axis=1, kind="stable")[:, :keep]
    allowed = np.zeros((s.shape[0], count), dtype=bool)
    np.put_along_axis(allowed, order, True, axis=1)
    masked = -np.sort(-np.where(np.repeat(allowed, per, axis=1), s, -np.inf), axis=1)
    expert_gap = masked[:, top - 1] - masked[:, top] if top < keep * per else np.full(s.shape[0], np.inf)
    return np.minimum(group_gap, expert_gap) / moved


def moe_ffn(x, w, cfg):
    chosen, weights = route(x, w, cfg["router"])
    out = np.zeros_like(x)
    for t in range(x.shape[0]):
        for e, a in zip(chosen[t], weights[t]):
            out[t] += a * (relu_squared(x[t] @ w[f"e{e}.up"].T) @ w[f"e{e}.down"].T)
    return out


def feed_forward(x, w, cfg):
    return dense_ffn(x, w) if cfg["kind"] == "dense" else moe_ffn(x, w, cfg)


MIXERS = {"attention": chunked_attention, "latent_attention": latent_attention}


def layer_weights(weights, layer, part):
    prefix = f"l{layer}.{part}."
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


def forward(config, weights, tokens, streams=None, margins=None):
    """Logits [T, vocab] of one sequence from position 0.  `weights`: {tensor name: float64 array}.
    `streams`, a list, receives the residual stream after every layer; `margins`, a list, the routing margin
    [T] of every layer that routes."""
    eps = config["norm"]["eps"]
    x = weights["embed"][np.asarray(tokens)]
    for i, layer in enumerate(config["layers"]):
        mixed = MIXERS[layer["type"]](x, layer_weights(weights, i, "mix"), layer["mixer"], eps)
        x = x + layer_norm(mixed, weights[f"l{i}.norm1"], weights[f"l{i}.norm1.b"], eps)
        if layer.get("mlp") is not None:
            fed = feed_forward(x, layer_weights(weights, i, "mlp"), layer["mlp"])
            if margins is not None and layer["mlp"]["kind"] == "moe":
                margins.append(route_margin(x, layer_weights(weights, i, "mlp"), layer["mlp"]["router"]))
            x = x + layer_norm(fed, weights[f"l{i}.norm2"], weights[f"l{i}.norm2.b"], eps)
        if streams is not None:
            streams.append(x.copy())
    x = layer_norm(x, weights["final.norm"], weights["final.norm.b"], eps)
    return (x @ weights["embed"].T) * config["logit_scale"]


class PlainPamunex:
    """A model folder (config.json, model.safetensors) run by the functions above."""

    def __init__(self, folder):
        import json
        import os

        import torch
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            self.cfg = json.load(f)
        self.tensors = {n: (t.to(torch.float64) if t.dtype.is_floating_point else t).numpy()
                        for n, t in load_file(os.path.join(folder, "model.safetensors")).items()}

    def logits(self, tokens, want=None):
        rows = forward(self.cfg, self.tensors, tokens)
        return rows if want is None else rows[np.asarray(want, dtype=np.int64)]

    def routing_margins(self, tokens):
        """[T]: the smallest routing margin of every position over the layers that route (see `route_margin`);
        None for a model that routes nowhere."""
        margins = []
        forward(self.cfg, self.tensors, tokens, margins=margins)
        return np.min(margins, axis=0) if margins else None

    def decisive(self, tokens, rng, least=40.0, tries=2000):
        """`tokens` with the token at every position whose routing is a close call (a margin below `least`) drawn
        again, from left to right (a position's margins depend on the tokens up to it only), so that an engine that
        rounds chooses the experts this file chooses: no comparison then rests on a close call."""
        tokens = list(tokens)
        vocab = self.tensors["embed"].shape[0]
        for _ in range(tries):
            margins = self.routing_margins(tokens)
            near = [] if margins is None else np.nonzero(margins < least)[0]
            if len(near) == 0:
                return tokens
            tokens[int(near[0])] = int(rng.integers(0, vocab))
        raise ValueError("no decisive sequence found")

    def greedy(self, prompt, n):
        tokens, out = list(prompt), []
        for _ in range(n):
            t = int(np.argmax(self.logits(tokens, [len(tokens) - 1])[0]))
            out.append(t)
            tokens.append(t)
        return out
