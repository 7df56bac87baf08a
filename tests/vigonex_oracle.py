"""Plain float64 implementation of the Vigonex decoder, whole sequences only:
one function per mechanism, numpy, no code shared with the engine. Weights
are a dict of checkpoint names -> arrays, sizes and constants the config dict.

Notation: T tokens, C model width, H query heads, G key/value heads, D key
size, Dv value size, S residual streams, E experts.
"""
from __future__ import annotations

import math

import numpy as np


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def unit_rms(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def position_vectors(n, width):
    """Row p, column c: sin (c even) or cos (c odd) of p * 10000^(-2 (c // 2) / width)."""
    p = np.arange(n, dtype=np.float64)[:, None]
    c = np.arange(width)
    ang = p * 10000.0 ** (-2.0 * (c // 2) / width)
    return np.where(c % 2 == 0, np.sin(ang), np.cos(ang))


def embed(cfg, W, tokens):
    x = W["embed"][np.asarray(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    return x + position_vectors(len(tokens), x.shape[1])


def token_shift(h, mu):
    """Every token moves towards its predecessor (zeros before the first) by
    the per-channel fraction mu."""
    prev = np.concatenate([np.zeros_like(h[:1]), h[:-1]])
    return h + (prev - h) * mu


def query_temperature(n, qt):
    if not qt:
        return np.ones(n)
    p = np.arange(n)
    return 1.0 + float(qt["coef"]) * np.log(np.floor((p + 1) / int(qt["every"])) + 1.0)


def causal_softmax_attention(q, k, v, scale, softcap):
    """q [T, D], k [T, D], v [T, Dv] of one head -> [T, Dv]."""
    s = (q @ k.T) * scale
    if softcap:
        s = softcap * np.tanh(s / softcap)
    T = q.shape[0]
    s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(-1, keepdims=True)
    return p @ v


def differential_attention(h, W, pre, m, eps):
    """Two softmax maps per head over shared values, subtracted."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ W[pre + "q"].T + W[pre + "q.b"]).reshape(T, H, 2, D)
    k = (h @ W[pre + "k"].T + W[pre + "k.b"]).reshape(T, G, 2, D)
    v = (h @ W[pre + "v"].T + W[pre + "v.b"]).reshape(T, G, Dv)
    q = q * query_temperature(T, m.get("q_temp"))[:, None, None, None]
    diff = float(m["diff"])
    lam = (math.exp(float((W[pre + "lq1"] * W[pre + "lk1"]).sum()))
           - math.exp(float((W[pre + "lq2"] * W[pre + "lk2"]).sum())) + diff)
    out = np.zeros((T, H, Dv))
    for hd in range(H):
        g = hd // (H // G)
        a = [causal_softmax_attention(q[:, hd, i], k[:, g, i], v[:, g], float(m["scale"]),
                                      float(m.get("softcap") or 0.0)) for i in range(2)]
        out[:, hd] = unit_rms(a[0] - lam * a[1], eps) * (1.0 - diff)
    return out.reshape(T, H * Dv) @ W[pre + "o"].T + W[pre + "o.b"]


def general_delta_recurrence(r, k, v, w, a, key_eps=1e-6):
    """One head. r, k, w, a [T, D]; v [T, Dv]. The state S [D, Dv] starts at
    zero; per token, with n the key scaled to unit length,
    S <- diag(w) S - (a * n) (n^T S) + k v^T (both first terms read the old
    S) and the read-out is S^T r."""
    T, D = k.shape
    S = np.zeros((D, v.shape[1]))
    out = np.zeros((T, v.shape[1]))
    for t in range(T):
        n = k[t] / math.sqrt(float((k[t] * k[t]).sum()) + key_eps)
        S = w[t][:, None] * S - np.outer(a[t] * n, n @ S) + np.outer(k[t], v[t])
        out[t] = r[t] @ S
    return out


def general_delta(h, W, pre, m, eps):
    T = h.shape[0]
    H, D = int(m["heads"]), int(m["dim"])
    r, k, v, g = (h @ W[pre + n].T for n in "rkvg")
    w = np.exp(-math.exp(-0.5) * sigmoid(np.tanh(h @ W[pre + "w1"].T) @ W[pre + "w2"].T
                                         + W[pre + "w0"]))
    a = sigmoid(h @ W[pre + "a"].T + W[pre + "a.b"])
    o = np.zeros((T, H, D))
    for hd in range(H):
        sl = slice(hd * D, (hd + 1) * D)
        o[:, hd] = unit_rms(general_delta_recurrence(r[:, sl], k[:, sl], v[:, sl],
                                                     w[:, sl], a[:, sl]), eps)
    y = o.reshape(T, H * D) * W[pre + "norm"] * sigmoid(g)
    return y @ W[pre + "o"].T


def dense_ff(h, W, pre):
    z = h @ W[pre + "gate"].T
    return (z * sigmoid(z) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def clamped_expert(h, W, pre, limit):
    g = np.minimum(h @ W[pre + "gate"].T, limit)
    u = np.clip(h @ W[pre + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[pre + "down"].T


def routed_ff(h, W, pre, mlp):
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ W[pre + "router"].T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s /= s.sum(-1, keepdims=True)
    out = np.zeros((h.shape[0], W[pre + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        chosen = np.argsort(-s[t], kind="stable")[:top]
        for e in chosen:
            out[t] += s[t, e] * float(mlp["router"].get("scale", 1.0)) * clamped_expert(
                h[t : t + 1], W, f"{pre}e{e}.", float(mlp["expert"]["limit"]))[0]
    if mlp.get("shared"):
        sh = clamped_expert(h, W, pre + "shared.", float(mlp["shared"]["limit"]))
        out += sh * sigmoid(h @ W[pre + "shared.sg"].T)
    return out


def feed_forward(h, W, pre, mlp):
    if mlp["kind"] == "dense":
        return dense_ff(h, W, pre)
    if mlp["kind"] == "moe":
        return routed_ff(h, W, pre, mlp)
    raise ValueError(mlp["kind"])


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence. layers_out (a list) receives
    the sum of the streams after every layer."""
    eps = float(cfg["norm"]["eps"])
    S = int(cfg.get("streams", 1))
    x0 = embed(cfg, W, tokens)
    X = np.stack([x0] * S)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        for q, sub in ((1, "mixer"), (2, "mlp")):
            if sub == "mlp" and L.get("mlp") is None:
                continue
            u = np.tensordot(W[f"{p}hc{q}.in"], X, axes=1)
            h = unit_rms(u, eps) * W[f"{p}norm{q}"]
            if sub == "mixer":
                hin = token_shift(h, W[p + "shift"])
                if L["type"] == "attention":
                    y = differential_attention(hin, W, p + "mix.", L["mixer"], eps)
                elif L["type"] == "general_delta":
                    y = general_delta(hin, W, p + "mix.", L["mixer"], eps)
                else:
                    raise ValueError(L["type"])
            else:
                y = feed_forward(h, W, p + "mlp.", L["mlp"])
            y = y * sigmoid(h @ W[f"{p}rg{q}"].T + W[f"{p}rg{q}.b"])
            X = (np.einsum("st,snc->tnc", W[f"{p}hc{q}.mix"], X)
                 + W[f"{p}hc{q}.out"][:, None, None] * y[None])
        if layers_out is not None:
            layers_out.append(X.sum(0))
    h = unit_rms(X.sum(0), eps) * W["final.norm"]
    return (h @ W["head"].T) * float(cfg.get("logit_scale", 1.0))


def random_weights(cfg, seed):
    """{name: bfloat16 torch tensor} for a config; the decay bottleneck of a
    delta layer has mixer["lowrank"] rows (default 5)."""
    import torch

    g = torch.Generator().manual_seed(seed)
    W = {}

    def mat(name, n_out, n_in, gain=1.0):
        W[name] = (torch.randn(n_out, n_in, generator=g) * gain * n_in ** -0.5).bfloat16()

    def vec(name, n, center, spread=0.2):
        W[name] = (center + spread * torch.randn(n, generator=g)).bfloat16()

    width, vocab, S = cfg["width"], cfg["vocab"], int(cfg.get("streams", 1))
    W["embed"] = torch.randn(vocab, width, generator=g).bfloat16()
    mat("head", vocab, width, 2.0)
    vec("final.norm", width, 1.0)
    for i, L in enumerate(cfg["layers"]):
        p, mx, q = f"l{i}.", L["mixer"], f"l{i}.mix."
        W[p + "shift"] = torch.rand(width, generator=g).bfloat16()
        for n in (1, 2):
            if n == 2 and L.get("mlp") is None:
                continue
            vec(f"{p}norm{n}", width, 1.0)
            vec(f"{p}hc{n}.in", S, 1.0 / S, 0.3)
            vec(f"{p}hc{n}.out", S, 1.0, 0.4)
            W[f"{p}hc{n}.mix"] = (torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)).bfloat16()
            mat(f"{p}rg{n}", width, width, 2.0)
            vec(f"{p}rg{n}.b", width, 0.5, 1.0)
        if L["type"] == "attention":
            H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            for name, n_out in (("q", 2 * H * D), ("k", 2 * G * D), ("v", G * Dv)):
                mat(q + name, n_out, width, 2.0)
                vec(q + name + ".b", n_out, 0.0, 0.3)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                vec(q + name, D, 0.0, 0.5 * D ** -0.5)
            mat(q + "o", width, H * Dv)
            vec(q + "o.b", width, 0.0, 0.3)
        else:
            H, D = mx["heads"], mx["dim"]
            R = int(mx.get("lowrank", 5))
            for name in "rkvga":
                mat(q + name, H * D, width, 2.0)
            vec(q + "a.b", H * D, 0.0, 1.0)
            mat(q + "w1", R, width, 2.0)
            mat(q + "w2", H * D, R, 2.0)
            vec(q + "w0", H * D, -0.5, 1.5)
            vec(q + "norm", H * D, 1.0)
            mat(q + "o", width, H * D)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        q = p + "mlp."
        if mlp["kind"] == "dense":
            mat(q + "gate", mlp["ff"], width, 2.0)
            mat(q + "up", mlp["ff"], width, 2.0)
            mat(q + "down", width, mlp["ff"])
        else:
            names = [f"{q}e{e}." for e in range(mlp["router"]["experts"])]
            sizes = [mlp["expert"]["ff"]] * len(names)
            if mlp.get("shared"):
                names.append(q + "shared.")
                sizes.append(mlp["shared"]["ff"])
                mat(q + "shared.sg", 1, width, 3.0)
            for n, ff in zip(names, sizes):
                mat(n + "gate", ff, width, 3.0)
                mat(n + "up", ff, width, 3.0)
                mat(n + "down", width, ff)
            mat(q + "router", mlp["router"]["experts"], width, 4.0)
    return W


def as_float64(W):
    return {k: v.double().numpy() for k, v in W.items()}
