"""A plain, slow implementation of the Taletar decoder in float64 numpy: whole sequences, no cache, no
batching, one function per mechanism.  It shares no code with the engine; the engine's tests compare
against it.

Notation: h [T, E] is a sequence's input of a mixer, positions count from 0, linear weights are [out, in]
and applied as x @ W.T.  `cfg` is the mixer's (or feed-forward's) entry of config.json, `w` maps the
tensor's last name part ("q", "conv.b", ...) to an array.
"""
from __future__ import annotations

import numpy as np


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return np.logaddexp(0.0, x)


def rms_unit(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x, weight, eps):
    return rms_unit(x, eps) * weight


# ---- differential attention ----------------------------------------------------------------------
def query_temperature(positions, coef, every):
    """Factor on the query at each position: 1 + coef * ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * np.log(np.floor((positions + 1) / every) + 1.0)


def capped_scores(q, k, scale, softcap):
    """[Tq, Tk] scores of one map of one head: scaled, then squashed into (-softcap, softcap) (None: no cap)."""
    s = (q @ k.T) * scale
    return s if softcap is None else softcap * np.tanh(s / softcap)


def causal_softmax(s, first_position=0):
    """Row i (position first_position + i) sees the keys 0 .. first_position + i."""
    tq, tk = s.shape
    seen = np.arange(tk)[None, :] <= (first_position + np.arange(tq))[:, None]
    s = np.where(seen, s, -np.inf)
    s = s - s.max(axis=1, keepdims=True)
    p = np.exp(s)
    return p / p.sum(axis=1, keepdims=True)


def differential_lambda(w, diff):
    return np.exp(np.sum(w["lq1"] * w["lk1"])) - np.exp(np.sum(w["lq2"] * w["lk2"])) + diff


def differential_attention(h, w, cfg, eps):
    T = h.shape[0]
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = (h @ w["q"].T).reshape(T, H, 2, D)
    k = (h @ w["k"].T).reshape(T, G, 2, D)
    v = (h @ w["v"].T).reshape(T, G, V)
    temp = cfg.get("q_temp")
    if temp:
        q = q * query_temperature(np.arange(T), temp["coef"], temp["every"])[:, None, None, None]
    lam = differential_lambda(w, cfg["diff"])
    heads = []
    for head in range(H):
        g = head // (H // G)
        maps = [causal_softmax(capped_scores(q[:, head, m], k[:, g, m], cfg["scale"], cfg.get("softcap"))) @ v[:, g]
                for m in range(2)]
        o = maps[0] - lam * maps[1]
        heads.append(rms_unit(o, eps) * (1.0 - cfg["diff"]))
    o = np.concatenate(heads, axis=1)
    o = o * sigmoid(h @ w["g"].T)
    return o @ w["o"].T


# ---- gated linear attention ------------------------------------------------------------------------
def gla_decay(h, w, cfg):
    """[T, heads, dim] decays in (0, 1): sigmoid(z)^(1/tau), z from the low-rank pair a1, a2 with a bias."""
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    return (sigmoid(z) ** (1.0 / cfg["tau"])).reshape(h.shape[0], cfg["heads"], cfg["dim"])


def linear_recurrence(q, k, v, decay, state=None):
    """One head.  S_t = decay_t[:, None] * S_(t-1) + outer(k_t, v_t); o_t = S_t^T q_t.  q, k, decay [T, N],
    v [T, V].  Returns (o [T, V], the last S)."""
    T, N = k.shape
    S = np.zeros((N, v.shape[1])) if state is None else state.copy()
    out = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = decay[t][:, None] * S + np.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out, S


def gated_linear_attention(h, w, cfg, eps):
    T = h.shape[0]
    H, D, V = cfg["heads"], cfg["dim"], cfg["vdim"]
    q = (h @ w["q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).reshape(T, H, D)
    v = (h @ w["v"].T).reshape(T, H, V)
    alpha = gla_decay(h, w, cfg)
    heads = [rms_norm(linear_recurrence(q[:, i], k[:, i], v[:, i], alpha[:, i])[0], w["norm"], eps) for i in range(H)]
    o = np.concatenate(heads, axis=1) * silu(h @ w["g"].T)
    return o @ w["o"].T


# ---- Mamba-2 ---------------------------------------------------------------------------------------
def causal_conv(x, weight, bias):
    """Per channel: y_t = bias + sum_j weight[:, j] * x_(t - (taps - 1) + j), zeros before the start."""
    T, C = x.shape
    taps = weight.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), x], axis=0)
    y = np.tile(bias, (T, 1)).astype(np.float64)
    for j in range(taps):
        y += padded[j:j + T] * weight[:, j]
    return y


def grouped_rms_norm(x, weight, parts, eps):
    T, W = x.shape
    return (rms_unit(x.reshape(T, parts, W // parts), eps).reshape(T, W)) * weight


def mamba2(h, w, cfg, eps):
    T = h.shape[0]
    H, V, N, G = cfg["heads"], cfg["vdim"], cfg["state"], cfg["groups"]
    inner = H * V
    p = h @ w["in"].T
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w["conv"], w["conv.b"]))
    x = xbc[:, :inner].reshape(T, H, V)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w["dt_bias"])                                   # [T, H]
    decay = np.exp(-np.exp(w["A_log"]) * dt)                          # [T, H]
    heads = []
    for i in range(H):
        g = i // (H // G)
        y, _ = linear_recurrence(C[:, g], B[:, g], dt[:, i, None] * x[:, i], np.repeat(decay[:, i, None], N, axis=1))
        heads.append(y + w["D"][i] * x[:, i])
    y = np.concatenate(heads, axis=1) * silu(z)
    y = grouped_rms_norm(y, w["norm"], cfg["norm_groups"], eps)
    return y @ w["o"].T


# ---- feed-forward ----------------------------------------------------------------------------------
def clamped_glu(h, w, cfg):
    g = np.minimum(h @ w["gate"].T, cfg["limit"])
    u = np.clip(h @ w["up"].T, -cfg["limit"], cfg["limit"])
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


# ---- the model --------------------------------------------------------------------------------------
MIXERS = {"attention": differential_attention, "gla": gated_linear_attention, "mamba2": mamba2}


def part_weights(tensors, prefix):
    """{name below `prefix`: float64 array} of the tensors whose names start with `prefix`."""
    return {name[len(prefix):]: np.asarray(t, dtype=np.float64) for name, t in tensors.items() if name.startswith(prefix)}


def forward(config, tensors, tokens, residuals=None):
    """Logits [T, vocab] of a whole sequence; `residuals`, a list, receives the stream after every layer."""
    eps = config["norm"]["eps"]
    x = np.asarray(tensors["embed"], dtype=np.float64)[np.asarray(tokens)]
    for i, layer in enumerate(config["layers"]):
        name = f"l{i}."
        mixed = MIXERS[layer["type"]](rms_norm(x, np.asarray(tensors[name + "norm1"], np.float64), eps),
                                      part_weights(tensors, name + "mix."), layer["mixer"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"feed-forward kind {layer['mlp']['kind']!r}")
            mixed = mixed + clamped_glu(rms_norm(x, np.asarray(tensors[name + "norm2"], np.float64), eps),
                                        part_weights(tensors, name + "mlp."), layer["mlp"])
        x = x + mixed
        if residuals is not None:
            residuals.append(x.copy())
    x = rms_norm(x, np.asarray(tensors["final.norm"], np.float64), eps)
    return x @ np.asarray(tensors["head"], dtype=np.float64).T


class PlainTaletar:
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

    def greedy(self, prompt, n):
        tokens, out = list(prompt), []
        for _ in range(n):
            t = int(np.argmax(self.logits(tokens, [len(tokens) - 1])[0]))
            out.append(t)
            tokens.append(t)
        return out
