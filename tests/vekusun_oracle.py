"""Plain whole-sequence implementation of the Vekusun decoder, one function
per mechanism, float64 numpy throughout, no cache, no state slots and no
batching. It exists to be compared with the engine and shares no code with it.

A model is (cfg, W): cfg the parsed config.json, W {tensor name: float64
array}. Every function takes whole-sequence arrays [n, ...].
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(x, w, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return np.logaddexp(0.0, x)


def gelu_exact(x):
    erf = np.vectorize(math.erf)
    return 0.5 * x * (1.0 + erf(x / math.sqrt(2.0)))


# ---------------------------------------------------------------------------
# rotation
# ---------------------------------------------------------------------------
def ramped_frequencies(rot):
    """(frequencies per pair, multiplier of cos and sin) of a rotation spec
    {base, dims, scaling: {factor, original, fast, slow} | absent}."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = sc["factor"], sc["original"]

    def pair_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(sc["fast"])), 0)
    hi = min(math.ceil(pair_of(sc["slow"])), dims - 1)
    i = np.arange(dims // 2)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, pos, freqs, mult):
    """x [n, ..., 2 * len(freqs)]: dimension 2i is paired with 2i + 1."""
    a = pos.astype(np.float64).reshape((-1,) + (1,) * (x.ndim - 1)) * freqs
    c, s = np.cos(a) * mult, np.sin(a) * mult
    u, v = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = u * c - v * s
    out[..., 1::2] = v * c + u * s
    return out


# ---------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------
def causal_softmax(scores, sink=None):
    """scores [n, n] of one head; row i sees columns j <= i. sink: a score
    that joins the denominator only."""
    n = scores.shape[0]
    out = np.zeros_like(scores)
    for i in range(n):
        row = scores[i, : i + 1]
        m = row.max() if sink is None else max(row.max(), sink)
        e = np.exp(row - m)
        den = e.sum() + (0.0 if sink is None else math.exp(sink - m))
        out[i, : i + 1] = e / den
    return out


def query_latent_attention(h, W, p, mx, eps):
    """Latent attention without positions: queries through a normed latent,
    keys and values up-projected from a normed latent, a sink per head."""
    n = h.shape[0]
    H, D, Dv = mx["heads"], mx["dim"], mx["vdim"]
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).reshape(n, H, D)
    c = rms_norm(h @ W[p + "dkv"].T, W[p + "dkv.norm"], eps)
    k = (c @ W[p + "uk"].T).reshape(n, H, D)
    v = (c @ W[p + "uv"].T).reshape(n, H, Dv)
    out = np.zeros((n, H, Dv))
    for hd in range(H):
        s = q[:, hd] @ k[:, hd].T * mx["scale"]
        out[:, hd] = causal_softmax(s, sink=float(W[p + "sink"][hd])) @ v[:, hd]
    return out.reshape(n, H * Dv) @ W[p + "o"].T


def rotated_latent_attention(h, W, p, mx, eps):
    """Latent attention with rot_dim rotated query dims per head against one
    rotated key part shared by the heads, and a sigmoid gate per head."""
    n = h.shape[0]
    H, D, Dr, Dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    pos = np.arange(n)
    q = (h @ W[p + "q"].T).reshape(n, H, D + Dr)
    down = h @ W[p + "dkv"].T
    c = rms_norm(down[:, :R], W[p + "dkv.norm"], eps)
    k = (c @ W[p + "uk"].T).reshape(n, H, D)
    v = (c @ W[p + "uv"].T).reshape(n, H, Dv)
    if Dr:
        f, mult = ramped_frequencies(mx["rot"])
        q_rot = rotate_pairs(q[..., D:], pos, f, mult)
        k_rot = rotate_pairs(down[:, R:], pos, f, mult)
    gate = sigmoid(h @ W[p + "g"].T)  # [n, H]
    out = np.zeros((n, H, Dv))
    for hd in range(H):
        s = q[:, hd, :D] @ k[:, hd].T
        if Dr:
            s = s + q_rot[:, hd] @ k_rot.T
        out[:, hd] = (causal_softmax(s * mx["scale"]) @ v[:, hd]) * gate[:, hd : hd + 1]
    return out.reshape(n, H * Dv) @ W[p + "o"].T


# ---------------------------------------------------------------------------
# gated delta rule
# ---------------------------------------------------------------------------
def short_conv_silu(x, w):
    """x [n, C], w [C, taps]: the last column weighs the current token."""
    n, taps = x.shape[0], w.shape[1]
    y = np.zeros_like(x)
    for t in range(n):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                y[t] += w[:, j] * x[src]
    return silu(y)


def delta_recurrence(q, k, v, beta, g):
    """One head: q, k [n, D], v [n, Dv], beta, g [n]. Returns o [n, Dv]."""
    S = np.zeros((q.shape[1], v.shape[1]))
    o = np.zeros_like(v)
    for t in range(q.shape[0]):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o


def delta_mixer(h, W, p, mx, eps):
    n = h.shape[0]
    H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = short_conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).reshape(n, G, D)
    k = short_conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).reshape(n, G, D)
    v = short_conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).reshape(n, H, Dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ W[p + "b"].T)
    g = np.exp(-np.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    out = np.zeros((n, H, Dv))
    for hd in range(H):
        kv = hd // (H // G)
        out[:, hd] = delta_recurrence(q[:, kv], k[:, kv], v[:, hd], beta[:, hd], g[:, hd])
    out = out / np.sqrt((out * out).mean(-1, keepdims=True) + eps) * W[p + "norm"]
    return (out.reshape(n, H * Dv) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


# ---------------------------------------------------------------------------
# feed-forward
# ---------------------------------------------------------------------------
def dense_feed_forward(h, W, p):
    return gelu_exact(h @ W[p + "up"].T) @ W[p + "down"].T


def route(h, W, p, mlp):
    """(chosen experts [n, top], their weights [n, top])."""
    z = h @ W[p + "router"].T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    choice = s + W[p + "correction"]
    top = mlp["router"]["top"]
    idx = np.argsort(-choice, axis=-1, kind="stable")[:, :top]
    return idx, np.take_along_axis(s, idx, axis=-1)


def routed_feed_forward(h, W, p, mlp):
    idx, w = route(h, W, p, mlp)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(idx[t], w[t]):
            a = silu(W[f"{p}e{e}.gate"] @ h[t]) * (W[f"{p}e{e}.up"] @ h[t])
            out[t] += we * (W[f"{p}e{e}.down"] @ a)
    return out


# ---------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------
def layer(cfg, W, i, x):
    L, p, eps = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"]
    h = rms_norm(x, W[p + "norm1"], eps)
    mixer = {"latent_attention": query_latent_attention,
             "latent_attention_2": rotated_latent_attention,
             "delta": delta_mixer}[L["type"]]
    y = mixer(h, W, p + "mix.", L["mixer"], eps) * W[p + "ls1"]
    mlp = L.get("mlp")
    if mlp is not None:
        f = (dense_feed_forward(h, W, p + "mlp.") if mlp["kind"] == "dense"
             else routed_feed_forward(h, W, p + "mlp.", mlp))
        y = y + f * W[p + "ls2"]
    return x + cfg.get("residual_mult", 1.0) * y


def forward(cfg, W, tokens, capture=None):
    """Logits [n, vocab]; capture (a list) receives the residual stream
    after every layer run."""
    x = W["embed"][np.asarray(tokens)]
    first = x.copy()
    n_layers = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}

    def run(i, x):
        x = layer(cfg, W, i, x)
        if capture is not None:
            capture.append(x.copy())
        return x

    for i in range(loop["start"]):
        x = run(i, x)
    if loop["stop"] > loop["start"]:
        for t in range(loop["times"]):
            if t > 0:
                x = x + first
            x = x + W["loop.step"][t]
            for i in range(loop["start"], loop["stop"]):
                x = run(i, x)
    for i in range(loop["stop"], n_layers):
        x = run(i, x)
    z = rms_norm(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(z / cap) if cap else z


def random_weights(cfg, seed):
    """{name: bfloat16 torch tensor} for a config."""
    import torch

    g = torch.Generator().manual_seed(seed)
    W = {}

    def mat(name, n_out, n_in, gain=1.0):
        W[name] = (torch.randn(n_out, n_in, generator=g) * gain * n_in ** -0.5).bfloat16()

    def vec(name, n, center, spread=0.2):
        W[name] = (center + spread * torch.randn(n, generator=g)).bfloat16()

    width, vocab = cfg["width"], cfg["vocab"]
    W["embed"] = torch.randn(vocab, width, generator=g).bfloat16()
    mat("head", vocab, width, 2.0)
    vec("final.norm", width, 1.0)
    loop = cfg.get("loop")
    if loop:
        W["loop.step"] = (0.5 * torch.randn(loop["times"], width, generator=g)).bfloat16()
    for i, L in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", L["mixer"]
        vec(p + "norm1", width, 1.0)
        vec(p + "ls1", width, 1.0, 0.3)
        q = p + "mix."
        if L["type"] == "latent_attention":
            H, D, Dv, R, Q = mx["heads"], mx["dim"], mx["vdim"], mx["kv_rank"], mx["q_rank"]
            mat(q + "dq", Q, width)
            vec(q + "dq.norm", Q, 1.0)
            mat(q + "uq", H * D, Q, 2.0)
            mat(q + "dkv", R, width)
            vec(q + "dkv.norm", R, 1.0)
            mat(q + "uk", H * D, R, 2.0)
            mat(q + "uv", H * Dv, R)
            vec(q + "sink", H, 0.5, 1.0)
            mat(q + "o", width, H * Dv)
        elif L["type"] == "latent_attention_2":
            H, D, Dr, Dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
            mat(q + "q", H * (D + Dr), width, 2.0)
            mat(q + "dkv", R + Dr, width, 2.0)
            vec(q + "dkv.norm", R, 1.0)
            mat(q + "uk", H * D, R, 2.0)
            mat(q + "uv", H * Dv, R)
            mat(q + "g", H, width, 2.0)
            mat(q + "o", width, H * Dv)
        else:
            H, G, D, Dv, taps = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"], mx["conv"]
            for name, n_out in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                mat(q + name, n_out, width, 2.0)
                W[q + name + ".conv"] = (0.6 * torch.randn(n_out, taps, generator=g)).bfloat16()
            mat(q + "b", H, width, 2.0)
            mat(q + "a", H, width, 2.0)
            vec(q + "A_log", H, -0.5, 1.0)
            vec(q + "dt_bias", H, 0.0, 1.0)
            vec(q + "norm", Dv, 1.0)
            mat(q + "g", H * Dv, width, 2.0)
            mat(q + "o", width, H * Dv)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        vec(p + "ls2", width, 1.0, 0.3)
        q = p + "mlp."
        if mlp["kind"] == "dense":
            mat(q + "up", mlp["ff"], width, 2.0)
            mat(q + "down", width, mlp["ff"])
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            for e in range(E):
                mat(f"{q}e{e}.gate", ff, width, 2.0)
                mat(f"{q}e{e}.up", ff, width, 2.0)
                mat(f"{q}e{e}.down", width, ff)
            mat(q + "router", E, width, 3.0)
            vec(q + "correction", E, 0.0, 0.1)
    return W


def as_float64(W):
    return {k: v.double().numpy() for k, v in W.items()}
