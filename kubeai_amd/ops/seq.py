"""Sequence-state ops: recurrences, short convolutions and chunk-masked
attention over the token-packed batch.

A packed step holds several *runs*: the tokens one sequence contributes
this step (one token for a decoding sequence, a prompt portion for a
prefilling one). Everything that carries per-sequence state across steps
takes a ``SeqMeta`` describing the runs and a state tensor indexed by the
sequence's *state slot* (engine/statecache.py). Conventions:

  - state tensors are fp32, ``[num_slots, ...]``; a run with slot -1 (bucket
    padding) reads zeros and writes nothing;
  - a run whose first token sits at position 0 starts from zero state
    whatever the slot holds, so a slot can be handed to a new sequence
    without clearing it;
  - activations are bf16 or fp32 (the serving dtype); recurrences, decays,
    gates of a recurrence, norms and attention scores are fp32 inside.

Dispatch follows kubeai_amd.ops: CPU tensors run the torch references below
(also the numerics reference of the kernels); GPU tensors require the
``kubeai_amd._C_seq`` HIP extension and fail loudly without it.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Optional

import torch

_C = None
_C_IMPORT_ERROR: Exception | None = None
try:
    from kubeai_amd import _C_seq as _C  # type: ignore[attr-defined,no-redef]
except Exception as e:  # pragma: no cover
    _C_IMPORT_ERROR = e


def have_seq_ext() -> bool:
    return _C is not None


def _require_ext() -> None:
    if _C is None:
        raise RuntimeError(
            "kubeai_amd._C_seq (sequence-state HIP kernels) is not built but a "
            "GPU tensor reached the ops layer. Build it with "
            "`KUBEAI_BUILD_ONLY=_C_seq python setup.py build_ext --inplace`. "
            f"Original import error: {_C_IMPORT_ERROR!r}"
        )


@dataclasses.dataclass
class SeqMeta:
    """Runs of the packed token stream, in packing order."""

    start_loc: torch.Tensor   # int32 [n_seq + 1] offsets into the stream
    slots: torch.Tensor       # int32 [n_seq] state slot, -1 = none
    token_seq: torch.Tensor   # int32 [T] run index of every token
    positions: torch.Tensor   # int32 [T] position of every token in its sequence
    block_tables: Optional[torch.Tensor]  # int32 [n_seq, max_blocks]
    n_seq: int
    max_len: int              # longest run (host value, sizes grids)

    def runs(self):
        """(start, length, slot, first position) per run — host values, for
        the CPU references only."""
        sl = self.start_loc.tolist()
        slots = self.slots.tolist()
        pos = self.positions
        for i in range(self.n_seq):
            s0, n = sl[i], sl[i + 1] - sl[i]
            if n > 0:
                yield s0, n, slots[i], int(pos[s0])

    @staticmethod
    def build(runs, positions, device, block_tables=None) -> "SeqMeta":
        """runs: list of (length, slot). positions: int32 tensor [T]."""
        import numpy as np

        lens = np.asarray([r[0] for r in runs], dtype=np.int64)
        start = np.zeros(len(runs) + 1, dtype=np.int32)
        np.cumsum(lens, out=start[1:])
        tok = np.repeat(np.arange(len(runs), dtype=np.int32), lens)
        return SeqMeta(
            start_loc=torch.from_numpy(start).to(device),
            slots=torch.tensor([r[1] for r in runs], dtype=torch.int32, device=device),
            token_seq=torch.from_numpy(tok).to(device),
            positions=positions,
            block_tables=block_tables,
            n_seq=len(runs),
            max_len=int(lens.max()) if len(runs) else 0,
        )


# ---------------------------------------------------------------------------
# norms
# ---------------------------------------------------------------------------

def add_layernorm(branch, residual, weight, bias, eps: float, out_dtype):
    """residual (fp32, in place) += branch; returns LayerNorm(residual) * w + b
    in ``out_dtype``. The variance is the mean squared deviation. branch may
    be None (first norm of the model)."""
    if residual.is_cuda:
        _require_ext()
        out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
        _C.add_layernorm(out, branch, residual, weight, bias, eps)
        return out
    if branch is not None:
        residual.add_(branch.float())
    mu = residual.mean(-1, keepdim=True)
    d = residual - mu
    var = (d * d).mean(-1, keepdim=True)
    return (d * torch.rsqrt(var + eps) * weight + bias).to(out_dtype)


def gated_rmsnorm(o, weight, gate, groups: int, gate_act: str, eps: float,
                  out, out_scale: float = 1.0):
    """out = o / rms(o over each of `groups` equal slices) * weight
    * act(gate) * out_scale. o is fp32 [T, C]; gate [T, C] may be a strided
    column view; out [T, C] may be a strided column view of a wider buffer.
    gate_act: "none" (gate already activated), "sigmoid" or "silu"."""
    if o.is_cuda:
        _require_ext()
        _C.gated_rmsnorm(out, o, weight, gate, groups,
                         {"none": 0, "sigmoid": 1, "silu": 2}[gate_act], eps,
                         out_scale)
        return out
    T, C = o.shape
    og = o.view(T, groups, C // groups)
    n = og * torch.rsqrt((og * og).mean(-1, keepdim=True) + eps)
    g = gate.float()
    if gate_act == "sigmoid":
        g = torch.sigmoid(g)
    elif gate_act == "silu":
        g = g * torch.sigmoid(g)
    out.copy_((n.reshape(T, C) * weight * g * out_scale).to(out.dtype))
    return out


def relu_squared(x):
    """relu(x)^2, elementwise (fp32 inside)."""
    if x.is_cuda:
        _require_ext()
        out = torch.empty_like(x)
        _C.relu_squared(out, x)
        return out
    r = torch.relu(x.float())
    return (r * r).to(x.dtype)


def gelu(x):
    """Exact GELU, x * Phi(x) = x/2 (1 + erf(x / sqrt 2)), elementwise (fp32
    inside)."""
    if x.is_cuda:
        _require_ext()
        out = torch.empty_like(x)
        _C.gelu(out, x)
        return out
    xf = x.float()
    return (0.5 * xf * (1.0 + torch.erf(xf * 0.7071067811865476))).to(x.dtype)


def rmsnorm_rows(x, weight, eps: float):
    """x / sqrt(mean(x^2) + eps) * weight per row, fp32 inside. x [T, C] may
    be a strided column view; returns a dense [T, C] of x's dtype."""
    if x.is_cuda:
        _require_ext()
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _C.rmsnorm_rows(out, x, weight, eps)
        return out
    xf = x.float()
    return (xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps) * weight).to(x.dtype)


def scaled_add_rmsnorm(residual, a, a_scale, b, b_scale, mult: float, extra,
                       extra_row, weight, eps: float, out_dtype):
    """Residual update of a layer whose sublayers read one norm and are
    summed, fused with the next norm:

        residual (fp32, in place) += mult * (a * a_scale + b * b_scale)
        residual += extra + extra_row
        returns residual / sqrt(mean(residual^2) + eps) * weight  (out_dtype)

    a, b: branch outputs [T, C] (serving dtype or fp32), either may be None;
    a_scale, b_scale: fp32 [C] per-channel scales (None = 1); extra: fp32
    [T, C] or None; extra_row: fp32 [C] or None."""
    if residual.is_cuda:
        _require_ext()
        out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
        _C.scaled_add_rmsnorm(out, residual, a, a_scale, b, b_scale, mult, extra,
                              extra_row, weight, eps)
        return out
    br = None
    for t, sc in ((a, a_scale), (b, b_scale)):
        if t is None:
            continue
        t = t.float() if sc is None else t.float() * sc
        br = t if br is None else br + t
    if br is not None:
        residual.add_(br * mult)
    if extra is not None:
        residual.add_(extra)
    if extra_row is not None:
        residual.add_(extra_row)
    r = torch.rsqrt((residual * residual).mean(-1, keepdim=True) + eps)
    return (residual * r * weight).to(out_dtype)


def tanh_cap(x, cap: float):
    """cap * tanh(x / cap) on an fp32 tensor, in place."""
    if x.is_cuda:
        _require_ext()
        _C.tanh_cap(x, cap)
        return x
    return x.copy_(cap * torch.tanh(x / cap))


# ---------------------------------------------------------------------------
# short causal convolutions with carried tails
# ---------------------------------------------------------------------------

def causal_conv(x, w, tails, meta: SeqMeta, residual: bool, act: str = "none"):
    """Depthwise causal convolution over time inside every run, followed by
    an optional activation (act: "none" or "silu", applied to the sum).

    x [T, C] (row-strided view allowed); w fp32 [C, taps]:
    y_t = sum_j w[:, j] * x_(t - taps + 1 + j)  (+ x_t if residual).
    tails fp32 [slots, taps-1, C] holds each sequence's last taps-1 inputs
    (row i = input at position P - (taps-1) + i, P = the next position) and
    is advanced past this step's tokens. Inputs before position 0 are zero.
    """
    taps = w.shape[1]
    if x.is_cuda:
        _require_ext()
        y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _C.causal_conv(y, x, w, tails, meta.start_loc, meta.slots,
                       meta.token_seq, meta.positions, residual,
                       {"none": 0, "silu": 1}[act])
        return y
    y = torch.empty(x.shape, dtype=x.dtype)
    C = x.shape[1]
    for s0, n, slot, p0 in meta.runs():
        xs = x[s0 : s0 + n].float()
        hist = torch.zeros(taps - 1, C)
        if slot >= 0:
            hist = tails[slot].clone()
            for i in range(taps - 1):
                if p0 - (taps - 1) + i < 0:
                    hist[i] = 0
        full = torch.cat([hist, xs])
        acc = xs.clone() if residual else torch.zeros_like(xs)
        for j in range(taps):
            acc += w[:, j] * full[j : j + n]
        if act == "silu":
            acc = acc * torch.sigmoid(acc)
        elif act != "none":
            raise ValueError(f"unknown activation {act!r}")
        y[s0 : s0 + n] = acc.to(x.dtype)
        if slot >= 0:
            tails[slot] = full[n : n + taps - 1]
    return y


def token_shift_mix(h, mu, prev, meta: SeqMeta):
    """mixes[s] = h + (h' - h) * mu[s], h' the previous token's h (zeros at
    position 0; across steps it comes from prev fp32 [slots, 1, C], which is
    advanced). h [T, C], mu fp32 [S, C] -> [S, T, C]."""
    if h.is_cuda:
        _require_ext()
        out = torch.empty((mu.shape[0],) + tuple(h.shape), dtype=h.dtype,
                          device=h.device)
        _C.token_shift_mix(out, h, mu, prev, meta.start_loc, meta.slots,
                           meta.token_seq, meta.positions)
        return out
    out = torch.empty((mu.shape[0],) + tuple(h.shape), dtype=h.dtype)
    for s0, n, slot, p0 in meta.runs():
        hs = h[s0 : s0 + n].float()
        first = torch.zeros(1, h.shape[1])
        if slot >= 0 and p0 > 0:
            first = prev[slot].clone()
        hp = torch.cat([first, hs[:-1]])
        out[:, s0 : s0 + n] = (hs + (hp - hs) * mu.unsqueeze(1)).to(h.dtype)
        if slot >= 0:
            prev[slot] = hs[-1:]
    return out


# ---------------------------------------------------------------------------
# recurrences
# ---------------------------------------------------------------------------

def mingru_scan(zxg, bz, bx, state, meta: SeqMeta):
    """Elementwise gated recurrence over packed projections zxg [T, 3n]
    (z | x | g): z = sigmoid(z + bz), u = x + bx,
    c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0),
    S_t = (1 - z) S_(t-1) + z c, y_t = S_t * silu(g). state fp32 [slots, n]."""
    n = bz.numel()
    if zxg.is_cuda:
        _require_ext()
        y = torch.empty((zxg.shape[0], n), dtype=zxg.dtype, device=zxg.device)
        _C.mingru_scan(y, zxg, bz, bx, state, meta.start_loc, meta.slots,
                       meta.positions, meta.max_len)
        return y
    y = torch.empty((zxg.shape[0], n), dtype=zxg.dtype)
    for s0, ln, slot, p0 in meta.runs():
        blk = zxg[s0 : s0 + ln].float()
        z = torch.sigmoid(blk[:, :n] + bz)
        u = blk[:, n : 2 * n] + bx
        g = blk[:, 2 * n :]
        c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        S = state[slot].clone() if (slot >= 0 and p0 > 0) else torch.zeros(n)
        for t in range(ln):
            S = (1 - z[t]) * S + z[t] * c[t]
            y[s0 + t] = (S * (g[t] * torch.sigmoid(g[t]))).to(zxg.dtype)
        if slot >= 0:
            state[slot] = S
    return y


def linear_attn_scan(q, k, v, decay, bonus, state, meta: SeqMeta, *,
                     w_bias=None, silu_inputs: bool = False):
    """Matrix-state linear attention, per head S [D, Dv] (fp32).

    Two forms share the kernel:
      * per-token channel decay (decay [T, H, D] holds pre-activations,
        w = exp(-exp(decay + w_bias))) with a bonus u [H, D] for the current
        token: o_t = (S + diag(u) k v^T)^T q, then S <- diag(w) S + k v^T;
      * constant per-head decay (decay fp32 [H], bonus None):
        S <- decay S + k v^T, then o_t = S^T q.
    silu_inputs applies silu to q, k, v first. q, k [T, H, D], v [T, H, Dv]
    (strided views allowed); returns o fp32 [T, H, Dv].
    """
    T, H, D = q.shape
    Dv = v.shape[2]
    per_token = decay.dim() == 3
    if q.is_cuda:
        _require_ext()
        o = torch.empty((T, H, Dv), dtype=torch.float32, device=q.device)
        _C.linear_attn_scan(o, q, k, v, decay, bonus, w_bias, state,
                            meta.start_loc, meta.slots, meta.positions,
                            silu_inputs, meta.max_len)
        return o
    o = torch.empty((T, H, Dv), dtype=torch.float32)
    act = (lambda a: a * torch.sigmoid(a)) if silu_inputs else (lambda a: a)
    for s0, n, slot, p0 in meta.runs():
        qs, ks, vs = (act(a[s0 : s0 + n].float()) for a in (q, k, v))
        if per_token:
            w = torch.exp(-torch.exp(decay[s0 : s0 + n].float() + w_bias.view(H, D)))
        S = (state[slot].clone() if (slot >= 0 and p0 > 0)
             else torch.zeros(H, D, Dv))
        for t in range(n):
            kv = ks[t].unsqueeze(-1) * vs[t].unsqueeze(-2)
            if per_token:
                o[s0 + t] = torch.einsum(
                    "hkv,hk->hv", S + bonus.unsqueeze(-1) * kv, qs[t])
                S = w[t].unsqueeze(-1) * S + kv
            else:
                S = decay.view(H, 1, 1) * S + kv
                o[s0 + t] = torch.einsum("hkv,hk->hv", S, qs[t])
        if slot >= 0:
            state[slot] = S
    return o


def gated_delta_scan(q, k, v, beta_pre, decay_pre, a_log, dt_bias, state,
                     meta: SeqMeta, norm_eps: float = 1e-6):
    """Gated delta rule, per head a matrix state S [D, Dv] (fp32):

        q <- q / sqrt(|q|^2 + norm_eps) * D^(-1/2),  k <- k / sqrt(|k|^2 + norm_eps)
        beta = sigmoid(beta_pre),  g = exp(-exp(a_log_h) softplus(decay_pre + dt_bias_h))
        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q

    so a token's read-out sees its own write. q, k [T, G, D] with H a
    multiple of G (head h uses q/k head h // (H/G)), v [T, H, Dv], beta_pre
    and decay_pre [T, H] (strided column views allowed), a_log and dt_bias
    fp32 [H], state fp32 [slots, H, D, Dv]. Everything but the loads is fp32.
    Returns o fp32 [T, H, Dv]."""
    T, G, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    if q.is_cuda:
        _require_ext()
        o = torch.empty((T, H, Dv), dtype=torch.float32, device=q.device)
        _C.gated_delta_scan(o, q, k, v, beta_pre, decay_pre, a_log, dt_bias,
                            state, meta.start_loc, meta.slots, meta.positions,
                            norm_eps, meta.max_len)
        return o
    o = torch.empty((T, H, Dv), dtype=torch.float32)
    rep = H // G
    for s0, n, slot, p0 in meta.runs():
        qs, ks, vs = (a[s0 : s0 + n].float() for a in (q, k, v))
        qs = qs * torch.rsqrt((qs * qs).sum(-1, keepdim=True) + norm_eps) * D ** -0.5
        ks = ks * torch.rsqrt((ks * ks).sum(-1, keepdim=True) + norm_eps)
        qs = qs.repeat_interleave(rep, dim=1)
        ks = ks.repeat_interleave(rep, dim=1)
        beta = torch.sigmoid(beta_pre[s0 : s0 + n].float())
        g = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(
            decay_pre[s0 : s0 + n].float() + dt_bias))
        S = (state[slot].clone() if (slot >= 0 and p0 > 0)
             else torch.zeros(H, D, Dv))
        for t in range(n):
            S = S * g[t].view(H, 1, 1)
            u = beta[t].view(H, 1) * (vs[t] - torch.einsum("hkv,hk->hv", S, ks[t]))
            S = S + ks[t].unsqueeze(-1) * u.unsqueeze(-2)
            o[s0 + t] = torch.einsum("hkv,hk->hv", S, qs[t])
        if slot >= 0:
            state[slot] = S
    return o


# ---------------------------------------------------------------------------
# rotary (interleaved pairs, leading dims) + paged cache write
# ---------------------------------------------------------------------------

def rope_pairs_and_cache(q, k, v, positions, inv_freq, k_cache, v_cache,
                         slot_mapping):
    """Rotate adjacent pairs (2i, 2i+1) of the first 2*len(inv_freq) dims of
    every q and k head by angle position * inv_freq[i] (fp32 angles); q is
    rotated in place, rotated k and v go to the paged caches
    (k_cache [blocks, G, block, D], v_cache [blocks, G, block, Dv]) at
    slot_mapping (slot < 0: no write). q [T, H, D], k [T, G, D],
    v [T, G, Dv] may be strided views."""
    if q.is_cuda:
        _require_ext()
        _C.rope_pairs_and_cache(q, k, v, positions, inv_freq, k_cache, v_cache,
                                slot_mapping)
        return q
    half = inv_freq.numel()
    a = positions.float().unsqueeze(-1) * inv_freq  # [T, half]
    c, s = torch.cos(a).unsqueeze(1), torch.sin(a).unsqueeze(1)

    def rot(x):
        xf = x.float()
        u = xf[..., 0 : 2 * half : 2]
        w = xf[..., 1 : 2 * half : 2]
        out = xf.clone()
        out[..., 0 : 2 * half : 2] = u * c - w * s
        out[..., 1 : 2 * half : 2] = w * c + u * s
        return out.to(x.dtype)

    q.copy_(rot(q))
    kr = rot(k)
    bs = k_cache.shape[2]
    ok = slot_mapping >= 0
    blk = (slot_mapping[ok] // bs).long()
    off = (slot_mapping[ok] % bs).long()
    k_cache[blk, :, off] = kr[ok].to(k_cache.dtype)
    v_cache[blk, :, off] = v[ok].to(v_cache.dtype)
    return q


def qknorm_rope_half_and_cache(q, k, v, q_weight, k_weight, eps: float, positions,
                               inv_freq, k_cache, v_cache, slot_mapping):
    """Whole-row RMS norm of q and of k (over all heads at once, plain fp32
    weights of the row's size; None skips the norm), then rotary on the
    first 2*len(inv_freq) dims of every head with dimension i paired with
    i + len(inv_freq): (u, w) -> (u cos a - w sin a, w cos a + u sin a),
    a = position * inv_freq[i] in fp32. q is rewritten in place; k and v go
    to the paged caches at slot_mapping (slot < 0: no write)."""
    if q.is_cuda:
        _require_ext()
        _C.qknorm_rope_half_and_cache(q, k, v, q_weight, k_weight, eps, positions,
                                      inv_freq, k_cache, v_cache, slot_mapping)
        return q
    T, H, D = q.shape
    G = k.shape[1]
    half = inv_freq.numel()
    a = positions.float().unsqueeze(-1) * inv_freq
    c, s = torch.cos(a).unsqueeze(1), torch.sin(a).unsqueeze(1)

    def prep(x, w, n):
        xf = x.float().reshape(T, -1)
        if w is not None:
            xf = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps) * w
        xf = xf.view(T, n, D)
        out = xf.clone()
        u, ww = xf[..., :half], xf[..., half : 2 * half]
        out[..., :half] = u * c - ww * s
        out[..., half : 2 * half] = ww * c + u * s
        return out.to(x.dtype)

    q.copy_(prep(q, q_weight, H))
    kr = prep(k, k_weight, G)
    bs = k_cache.shape[2]
    ok = slot_mapping >= 0
    blk = (slot_mapping[ok] // bs).long()
    off = (slot_mapping[ok] % bs).long()
    k_cache[blk, :, off] = kr[ok].to(k_cache.dtype)
    v_cache[blk, :, off] = v[ok].to(v_cache.dtype)
    return q


# ---------------------------------------------------------------------------
# norms around both sides of a sublayer, cached latents, gates
# ---------------------------------------------------------------------------

def sandwich_rmsnorm(branch, post_weight, residual, pre_weight, eps: float,
                     out_dtype):
    """residual (fp32, in place) += branch / rms(branch) * post_weight, then
    returns residual / rms(residual) * pre_weight in ``out_dtype``. rms(x) =
    sqrt(mean(x^2) + eps). Weights are fp32 multipliers (a checkpoint that
    stores them around zero adds the one when it is loaded). branch (serving
    dtype or fp32) may be None: only the second norm runs."""
    if residual.is_cuda:
        _require_ext()
        out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
        _C.sandwich_rmsnorm(out, branch, post_weight if branch is not None else None,
                            residual, pre_weight, eps)
        return out
    if branch is not None:
        b = branch.float()
        residual.add_(b * torch.rsqrt((b * b).mean(-1, keepdim=True) + eps)
                      * post_weight)
    r = torch.rsqrt((residual * residual).mean(-1, keepdim=True) + eps)
    return (residual * r * pre_weight).to(out_dtype)


def rmsnorm_to_cache(x, weight, eps: float, cache, slot_mapping):
    """cache row at slot_mapping[t] = x[t] / rms(x[t]) * weight (fp32 inside).
    x [T, C] may be a strided column view; cache [blocks, 1, block, C]."""
    if x.is_cuda:
        _require_ext()
        _C.rmsnorm_to_cache(cache, x, weight, slot_mapping, eps)
        return
    xf = x.float()
    y = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps) * weight
    ok = slot_mapping >= 0
    flat = cache.view(-1, cache.shape[-1])
    flat[slot_mapping[ok].long()] = y[ok].to(cache.dtype)


def latent_rope_to_cache(x, weight, eps: float, q_rot, q_out, positions,
                         inv_freq, rot_mult: float, cache, slot_mapping):
    """Cache row of a latent-attention layer with a shared rotated key part.

    x [T, R + r] (strided rows fine): the first R = len(weight) columns are
    RMS-normed (times weight) into the cache row's first R columns; the last
    r = 2 len(inv_freq) columns are rotated and written behind them. The
    rotation pairs dimension 2i with 2i+1: (u, w) -> (u cos a - w sin a,
    w cos a + u sin a) * rot_mult, a = position * inv_freq[i], fp32. The same
    rotation is applied to q_rot [T, H, r] (a strided slice of the query
    heads), written to q_out [T, H, r] (a strided slice of the folded query).
    r may be 0 (q_rot/q_out None): only the norm runs. cache
    [blocks, 1, block, R + r]; rows with slot < 0 are not written."""
    R = weight.numel()
    half = inv_freq.numel()
    if x.is_cuda:
        _require_ext()
        _C.latent_rope_to_cache(cache, x, weight, eps, q_rot, q_out, positions,
                                inv_freq, rot_mult, slot_mapping)
        return
    xf = x.float()
    c = xf[:, :R]
    row = [c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * weight]
    if half:
        a = positions.float().unsqueeze(-1) * inv_freq
        cs, sn = torch.cos(a) * rot_mult, torch.sin(a) * rot_mult

        def rot(t, cs, sn):
            u, w = t[..., 0::2], t[..., 1::2]
            o = torch.empty_like(t)
            o[..., 0::2] = u * cs - w * sn
            o[..., 1::2] = w * cs + u * sn
            return o

        row.append(rot(xf[:, R:], cs, sn))
        q_out.copy_(rot(q_rot.float(), cs.unsqueeze(1), sn.unsqueeze(1)).to(q_out.dtype))
    y = torch.cat(row, dim=-1)
    ok = slot_mapping >= 0
    flat = cache.view(-1, cache.shape[-1])
    flat[slot_mapping[ok].long()] = y[ok].to(cache.dtype)


def sigmoid_gate(x, gate, out=None):
    """x * sigmoid(gate), elementwise; gate may be a strided column view."""
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    if x.is_cuda:
        _require_ext()
        _C.sigmoid_gate(out, x, gate)
        return out
    out.copy_((x.float() * torch.sigmoid(gate.float())).to(x.dtype))
    return out


def head_linear(x, w, gate=None, out=None):
    """y[t, h, :] = w[h] @ x[t, h, :], times sigmoid of a gate if one is
    given: gate [T, H*B] gates every output channel, gate [T, H] a whole
    head. x [T, H, A] and out [T, H, B] may be views whose token and head
    strides are larger than their sizes (a slice of every head of a wider
    buffer); w [H, B, A]; gate rows may be strided. fp32 accumulation."""
    T, H, _ = x.shape
    B = w.shape[1]
    if out is None:
        out = torch.empty((T, H, B), dtype=x.dtype, device=x.device)
    if x.is_cuda:
        _require_ext()
        _C.head_linear(out, x, w, gate)
        return out
    y = torch.einsum("tha,hba->thb", x.float(), w.float())
    if gate is not None:
        g = torch.sigmoid(gate.float())
        y = y * (g.reshape(T, H, 1) if gate.shape[1] == H and B != 1 else g.reshape(T, H, B))
    out.copy_(y.to(x.dtype))
    return out


# ---------------------------------------------------------------------------
# mixture-of-experts routing
# ---------------------------------------------------------------------------

def router_topk(logits, top: int):
    """fp32 router logits [T, E] -> (dense [T, E], weights [T, top],
    index int32 [T, top]): the `top` largest logits of every row (equal
    logits: lower index first), weights = softmax over the chosen logits
    only, dense = the same weights scattered to the experts' columns."""
    T, E = logits.shape
    if logits.is_cuda:
        _require_ext()
        dense = torch.empty((T, E), dtype=torch.float32, device=logits.device)
        w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
        idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
        _C.router_topk(logits.contiguous(), dense, w, idx)
        return dense, w, idx
    order = torch.sort(logits, dim=-1, descending=True, stable=True)
    idx = order.indices[:, :top]
    w = torch.softmax(order.values[:, :top], dim=-1)
    dense = torch.zeros((T, E), dtype=torch.float32)
    dense.scatter_(1, idx, w)
    return dense, w, idx.to(torch.int32)


def relu_squared_weighted(u, w, group: int):
    """out[t, c] = relu(u[t, c])^2 * w[t, c // group]; columns past
    w.shape[1] * group get weight 1. u [T, C]; w fp32 [T, groups]."""
    if u.is_cuda:
        _require_ext()
        out = torch.empty_like(u)
        _C.relu_squared_weighted(out, u, w, group)
        return out
    r = torch.relu(u.float())
    r = r * r
    n = w.shape[1] * group
    r[:, :n] = (r[:, :n].view(u.shape[0], w.shape[1], group) * w.unsqueeze(-1)).view(
        u.shape[0], n)
    return r.to(u.dtype)


def router_scores_topk(logits, top: int, bias=None, scale: float = 1.0):
    """Routing by scores: s = softmax(logits) over all experts (fp32); the
    `top` experts with the largest s + bias are chosen (equal values: lower
    index first; bias fp32 [E] or None), and their weights are their scores
    s themselves times `scale`, not renormalised. Returns (dense [T, E] with the weights at
    the chosen experts' columns, weights [T, top], index int32 [T, top])."""
    T, E = logits.shape
    if logits.is_cuda:
        _require_ext()
        dense = torch.empty((T, E), dtype=torch.float32, device=logits.device)
        w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
        idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
        _C.router_scores_topk(logits.contiguous(), bias, dense, w, idx, scale)
        return dense, w, idx
    s = torch.softmax(logits.float(), dim=-1)
    choice = s if bias is None else s + bias
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    w = torch.gather(s, 1, idx) * scale
    dense = torch.zeros((T, E), dtype=torch.float32)
    dense.scatter_(1, idx, w)
    return dense, w, idx.to(torch.int32)


def silu_mul_weighted(gu, w, group: int):
    """Gated expert activation with the routing weight folded in. gu
    [T, n * 2 * group] holds, per expert e, `group` gate columns followed by
    `group` up columns; out[t, e * group + c] = silu(gate) * up * w[t, e].
    w fp32 [T, n] (a strided column view is fine)."""
    return glu_weighted(gu, w, group)


def glu_weighted(gu, w, group: int, *, alpha: float = 1.0, limit: float = 0.0,
                 up_shift: float = 0.0, w_sigmoid: bool = False, out=None):
    """Gated activation over blocks of `group` gate columns followed by
    `group` up columns (gu [T, n * 2 * group], rows may be strided):

        g = gate, u = up;  with limit > 0: g = min(g, limit), u = clamp(u, -limit, limit)
        out[t, e * group + c] = g * sigmoid(alpha * g) * (u + up_shift) * w[t, e]

    alpha = 1 is silu. w fp32 [T, n] (strided columns view fine) or None (no
    weight); with w_sigmoid the weight is sigmoid(w). out [T, n * group] may
    be a strided column view of a wider buffer. fp32 inside."""
    T, C2 = gu.shape
    n = C2 // (2 * group)
    if out is None:
        out = torch.empty((T, n * group), dtype=gu.dtype, device=gu.device)
    if gu.is_cuda:
        _require_ext()
        _C.glu_weighted(out, gu, w, group, alpha, limit, up_shift, w_sigmoid)
        return out
    g = gu.float().reshape(T, n, 2, group)
    gate, up = g[:, :, 0], g[:, :, 1]
    if limit > 0:
        gate = gate.clamp(max=limit)
        up = up.clamp(-limit, limit)
    a = gate * torch.sigmoid(alpha * gate) * (up + up_shift)
    if w is not None:
        wf = torch.sigmoid(w.float()) if w_sigmoid else w.float()
        a = a * wf.unsqueeze(-1)
    out.copy_(a.reshape(T, n * group).to(out.dtype))
    return out


# ---------------------------------------------------------------------------
# masked paged attention (decode tokens and prompt portions alike)
# ---------------------------------------------------------------------------

def masked_paged_attention(q, k_cache, v_cache, meta: SeqMeta, scale: float,
                           out, *, softcap: float = 0.0, chunk: int = 0,
                           window: int = 0, out_scale: float = 1.0,
                           sink: Optional[torch.Tensor] = None):
    """Softmax attention of every packed token over its own sequence's cached
    keys. The token at position i sees j <= i with, when chunk > 0,
    floor(j / chunk) == floor(i / chunk) (position-aligned chunks) and, when
    window > 0, j > i - window. Scores are (q . k) * scale, then
    softcap * tanh(score / softcap) if softcap > 0; all in fp32. With sink
    (fp32 [H]), the softmax of head h has one more key whose score is
    sink[h] as it stands (not scaled, not capped) and that carries no value:
    the denominator grows by exp(sink[h]).
    q [T, H, D] (strided ok), caches [blocks, G, block, D | Dv]; v_cache may
    be the leading Dv columns of the key rows (a view of k_cache), or have
    fewer heads than k_cache (Gv dividing G: query head h reads key head
    h // (H / G) and value head h // (H / Gv), so several score maps share
    one value head);
    out [T, H, Dv] may be a strided view; out = attention * out_scale.
    sink=True stands for a score of 0 on every head."""
    if sink is True:
        sink = torch.zeros(q.shape[1], dtype=torch.float32, device=q.device)
    elif sink is False:
        sink = None
    if q.is_cuda:
        _require_ext()
        _C.masked_paged_attention(out, q, k_cache, v_cache, meta.block_tables,
                                  meta.start_loc, meta.token_seq, meta.positions,
                                  meta.max_len, scale, softcap, chunk, window,
                                  out_scale, sink)
        return out
    T, H, D = q.shape
    G, bs = k_cache.shape[1], k_cache.shape[2]
    rep, rep_v = H // G, H // v_cache.shape[1]
    bt = meta.block_tables
    sl = meta.start_loc.tolist()
    for si in range(meta.n_seq):
        s0, n = sl[si], sl[si + 1] - sl[si]
        if n == 0:
            continue
        pos = meta.positions[s0 : s0 + n].long()
        L = int(pos.max()) + 1
        lo = 0
        if chunk > 0:
            lo = (int(pos.min()) // chunk) * chunk
        if window > 0:
            lo = max(lo, int(pos.min()) - window + 1)
        j = torch.arange(lo, L)
        blk = bt[si][(j // bs)].long()
        ks = k_cache[blk, :, j % bs].float()  # [L', G, D]
        vs = v_cache[blk, :, j % bs].float()
        ks = ks.repeat_interleave(rep, dim=1)
        vs = vs.repeat_interleave(rep_v, dim=1)
        s = torch.einsum("thd,lhd->htl", q[s0 : s0 + n].float(), ks) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        vis = j.view(1, -1) <= pos.view(-1, 1)
        if chunk > 0:
            vis &= (j.view(1, -1) // chunk) == (pos.view(-1, 1) // chunk)
        if window > 0:
            vis &= j.view(1, -1) > pos.view(-1, 1) - window
        s = s.masked_fill(~vis.unsqueeze(0), float("-inf"))
        if sink is not None:
            s = torch.cat(
                [s, sink.float().view(H, 1, 1).expand(H, s.shape[1], 1)], dim=-1)
        p = torch.softmax(s, dim=-1)
        if sink is not None:
            p = p[..., :-1]
        o = torch.einsum("htl,lhd->thd", p, vs) * out_scale
        out[s0 : s0 + n] = o.to(out.dtype)
    return out


# ---------------------------------------------------------------------------
# sinusoidal positions, residual streams, differential attention, the
# generalized delta rule
# ---------------------------------------------------------------------------

def embed_sinusoid(ids, table, scale: float, positions, freqs, copies: int = 1):
    """fp32 [T, copies, C], every copy table[ids] * scale plus a position
    vector whose column c is sin (c even) or cos (c odd) of
    position * freqs[c // 2]. table [V, C] in the serving dtype, freqs
    float64 [ceil(C / 2)]: the angle is formed in double and reduced to one
    turn before the fp32 sine and cosine."""
    T, C = ids.shape[0], table.shape[1]
    if table.is_cuda:
        _require_ext()
        out = torch.empty((T, copies, C), dtype=torch.float32, device=table.device)
        _C.embed_sinusoid(out, ids, table, scale, positions, freqs)
        return out
    ang = torch.remainder(positions.double().unsqueeze(-1) * freqs, 2.0 * math.pi).float()
    pe = torch.stack([torch.sin(ang), torch.cos(ang)], dim=-1).reshape(T, -1)[:, :C]
    x = table[ids.long()].float() * scale + pe
    return x.unsqueeze(1).repeat(1, copies, 1)


def hyper_mix_rmsnorm(streams, y, gate, mix, out_w, in_w, weight, eps: float,
                      out_dtype):
    """Residual streams (hyper-connections) around a sublayer, fused with the
    next sublayer's input norm. streams fp32 [T, S, C], updated in place:

        z = y * sigmoid(gate)                  (gate None: z = y)
        streams[:, t] <- sum_s mix[s, t] streams[:, s] + out_w[t] * z
        u = sum_s in_w[s] streams[:, s]
        returns u / sqrt(mean(u^2) + eps) * weight      (out_dtype)

    y [T, C] is the previous sublayer's output (serving dtype or fp32; None:
    the streams stay as they are), gate [T, C] its gate's pre-activation (rows
    may be strided), mix fp32 [S, S] indexed [from, to], out_w and in_w fp32
    [S], weight fp32 [C]. All sums are fp32."""
    if streams.is_cuda:
        _require_ext()
        out = torch.empty((streams.shape[0], streams.shape[2]), dtype=out_dtype,
                          device=streams.device)
        _C.hyper_mix_rmsnorm(out, streams, y, gate, mix, out_w, in_w, weight, eps)
        return out
    if y is not None:
        z = y.float()
        if gate is not None:
            z = z * torch.sigmoid(gate.float())
        new = torch.einsum("st,nsc->ntc", mix, streams) + out_w.view(1, -1, 1) * z.unsqueeze(1)
        streams.copy_(new)
    u = torch.einsum("s,nsc->nc", in_w, streams)
    return (u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps) * weight).to(out_dtype)


def scale_q_and_cache(q, k, v, positions, coef: float, every: int, k_cache,
                      v_cache, slot_mapping):
    """Position-dependent query temperature fused with the paged cache write:
    q[t] *= 1 + coef * ln(floor((p + 1) / every) + 1) at position p (fp32; in
    place; coef 0 leaves q alone); k and v rows go to their caches at
    slot_mapping (slot < 0: no write). q [T, H, D], k [T, G, D], v [T, Gv, Dv]
    may be strided views; the caches are [blocks, G | Gv, block, D | Dv]."""
    if q.is_cuda:
        _require_ext()
        _C.scale_q_and_cache(q, k, v, positions, coef, every, k_cache, v_cache,
                             slot_mapping)
        return q
    if coef != 0.0:
        p = positions.long()
        temp = 1.0 + coef * torch.log(
            torch.div(p + 1, int(every), rounding_mode="floor").float() + 1.0)
        q.copy_((q.float() * temp.view(-1, 1, 1)).to(q.dtype))
    bs = k_cache.shape[2]
    ok = slot_mapping >= 0
    blk = (slot_mapping[ok] // bs).long()
    off = (slot_mapping[ok] % bs).long()
    k_cache[blk, :, off] = k[ok].to(k_cache.dtype)
    v_cache[blk, :, off] = v[ok].to(v_cache.dtype)
    return q


def diff_combine(att, lam: float, gain: float, eps: float, out):
    """Differential attention's join: att [T, G, 2, R, Dv] holds, per group
    of R query heads, the outputs of the two softmax maps; for head (g, r)

        o = att[:, g, 0, r] - lam * att[:, g, 1, r]
        out[:, g * R + r] = o / sqrt(mean(o^2) + eps) * gain

    in fp32. out [T, G * R, Dv] may be a strided view."""
    T, G, _, R, Dv = att.shape
    if att.is_cuda:
        _require_ext()
        _C.diff_combine(out, att, lam, gain, eps)
        return out
    a = att.float()
    o = a[:, :, 0] - lam * a[:, :, 1]
    o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps) * gain
    out.copy_(o.reshape(T, G * R, Dv).to(out.dtype))
    return out


def diag_rank1_scan(r, k, v, w_pre, a_pre, w_bias, a_bias, state, meta: SeqMeta,
                    decay_scale: float, key_eps: float = 1e-6):
    """Generalized delta rule: per head a matrix state S [D, Dv] (fp32) whose
    transition is a diagonal decay plus a rank-one removal along the unit key,
    both applied to the old state, followed by the write:

        w = exp(-decay_scale * sigmoid(w_pre + w_bias)),  a = sigmoid(a_pre + a_bias)
        n = k / sqrt(|k|^2 + key_eps)
        S <- diag(w) S - (a * n) (n^T S) + k v^T;   o = S^T r

    r, k, w_pre, a_pre [T, H, D], v [T, H, Dv] (strided column views of one
    projection are fine), w_bias, a_bias fp32 [H * D], state fp32
    [slots, H, D, Dv]. Everything but the loads is fp32. Returns o fp32
    [T, H, Dv]."""
    T, H, D = k.shape
    Dv = v.shape[2]
    if k.is_cuda:
        _require_ext()
        o = torch.empty((T, H, Dv), dtype=torch.float32, device=k.device)
        _C.diag_rank1_scan(o, r, k, v, w_pre, a_pre, w_bias, a_bias, state,
                           meta.start_loc, meta.slots, meta.positions, decay_scale,
                           key_eps, meta.max_len)
        return o
    o = torch.empty((T, H, Dv), dtype=torch.float32)
    for s0, n, slot, p0 in meta.runs():
        rs, ks, vs = (x[s0 : s0 + n].float() for x in (r, k, v))
        w = torch.exp(-decay_scale * torch.sigmoid(
            w_pre[s0 : s0 + n].float() + w_bias.view(H, D)))
        a = torch.sigmoid(a_pre[s0 : s0 + n].float() + a_bias.view(H, D))
        un = ks * torch.rsqrt((ks * ks).sum(-1, keepdim=True) + key_eps)
        S = (state[slot].clone() if (slot >= 0 and p0 > 0)
             else torch.zeros(H, D, Dv))
        for t in range(n):
            proj = torch.einsum("hk,hkv->hv", un[t], S)
            S = (w[t].unsqueeze(-1) * S
                 - (a[t] * un[t]).unsqueeze(-1) * proj.unsqueeze(-2)
                 + ks[t].unsqueeze(-1) * vs[t].unsqueeze(-2))
            o[s0 + t] = torch.einsum("hkv,hk->hv", S, rs[t])
        if slot >= 0:
            state[slot] = S
    return o
