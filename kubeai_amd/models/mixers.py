"""Token mixers beyond plain causal attention, for hybrid layer stacks.

Each mixer is parameterised by its own sizes and constants (never by a
particular checkpoint) and declares what it carries between steps:

  state_spec()  -> {name: per-slot shape}  fp32 tensors [slots, *shape]
  kv_spec()     -> None | (kv_heads, key_dim, value_dim) for a paged cache

forward() gets the activations h [T, C] of the packed step, the ForwardBatch
(whose .seq describes the runs and their state slots), this layer's state
tensors and paged cache. Projections are library GEMMs in the serving dtype;
everything inside a recurrence, every norm and every attention score is fp32
in the kernels (kubeai_amd.ops.seq).
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from kubeai_amd.ops import seq as sops


def _f32(*shape):
    return nn.Parameter(torch.zeros(*shape, dtype=torch.float32), requires_grad=False)


class Proj(nn.Module):
    """Bias-free linear layer [out, in] in the serving dtype."""

    def __init__(self, n_in: int, n_out: int):
        super().__init__()
        self.weight = nn.Parameter(torch.empty(n_out, n_in), requires_grad=False)
        nn.init.normal_(self.weight, std=n_in ** -0.5)

    def forward(self, x):
        return F.linear(x, self.weight)


class CausalConvTails(nn.Module):
    """Depthwise causal convolution over time whose last taps-1 inputs are
    sequence state (the layer-input convolution and the q/k/v convolutions)."""

    def __init__(self, channels: int, taps: int, residual: bool, act: str = "none"):
        super().__init__()
        self.taps = taps
        self.residual = residual
        self.act = act
        self.weight = _f32(channels, taps)
        nn.init.normal_(self.weight, std=0.3)
        self.channels = channels

    def state_shape(self):
        return (self.taps - 1, self.channels)

    def forward(self, x, fb, tails):
        return sops.causal_conv(x, self.weight, tails, fb.seq, self.residual, self.act)


class MinGRUMixer(nn.Module):
    """minGRU: elementwise recurrent state whose gate and candidate are
    functions of the input at t alone, which is what lets a run be scanned
    segment-parallel."""

    def __init__(self, width: int, n: int):
        super().__init__()
        self.n = n
        self.in_proj = Proj(width, 3 * n)  # z | x | g
        self.bias_z = _f32(n)
        self.bias_x = _f32(n)
        self.o_proj = Proj(n, width)

    def state_spec(self):
        return {"s": (self.n,)}

    def kv_spec(self):
        return None

    def forward(self, h, fb, state, kv_cache):
        zxg = self.in_proj(h)
        y = sops.mingru_scan(zxg, self.bias_z, self.bias_x, state["s"], fb.seq)
        return self.o_proj(y)


class WKVMixer(nn.Module):
    """Matrix-state time mixing with token shift and data-dependent
    per-channel decay; the current token gets a bonus instead of the state."""

    STREAMS = "rkvgw"

    def __init__(self, width: int, heads: int, dim: int, lowrank: int, eps: float):
        super().__init__()
        self.width, self.heads, self.dim, self.eps = width, heads, dim, eps
        n = heads * dim
        self.mu = _f32(5, width)
        # r, k, v, g share the output size: stacked [4, n, width]
        self.rkvg = nn.Parameter(torch.empty(4, n, width), requires_grad=False)
        nn.init.normal_(self.rkvg, std=width ** -0.5)
        self.w1 = Proj(width, lowrank)
        self.w2 = Proj(lowrank, n)
        self.w0 = _f32(n)
        self.u = _f32(heads, dim)
        self.norm = _f32(n)
        self.o_proj = Proj(n, width)

    def state_spec(self):
        return {"prev": (1, self.width), "s": (self.heads, self.dim, self.dim)}

    def kv_spec(self):
        return None

    def forward(self, h, fb, state, kv_cache):
        T = h.shape[0]
        H, D = self.heads, self.dim
        mixes = sops.token_shift_mix(h, self.mu, state["prev"], fb.seq)
        # four plain GEMMs (the library path every other family uses; the
        # strided-batched path is not exercised under the tuned-GEMM table)
        rkvg = [F.linear(mixes[i], self.rkvg[i]) for i in range(4)]
        lr = torch.tanh(self.w1(mixes[4]).float()).to(h.dtype)
        wpre = self.w2(lr)
        o = sops.linear_attn_scan(
            rkvg[0].view(T, H, D), rkvg[1].view(T, H, D), rkvg[2].view(T, H, D),
            wpre.view(T, H, D), self.u, state["s"], fb.seq, w_bias=self.w0,
        )
        y = torch.empty((T, H * D), dtype=h.dtype, device=h.device)
        sops.gated_rmsnorm(o.view(T, H * D), self.norm, rkvg[3], H, "silu",
                           self.eps, y)
        return self.o_proj(y)


class ChunkedAttention(nn.Module):
    """Softmax attention restricted to position-aligned chunks, with grouped
    key/value heads, separate key and value sizes, short convolutions on the
    projected q/k/v, rotary on leading interleaved pairs and a tanh cap.
    Projections are owned by the caller (so they can be fused with a
    sibling's); this module takes the projected [T, q|k|v] block."""

    def __init__(self, heads, kv_heads, dim, vdim, conv_taps, rot_dims, rot_base,
                 scale, softcap, chunk, window=0):
        super().__init__()
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.softcap = float(scale), float(softcap or 0.0)
        self.chunk, self.window = int(chunk or 0), int(window or 0)
        self.sizes = (heads * dim, kv_heads * dim, kv_heads * vdim)
        self.n_in = sum(self.sizes)
        self.n_out = heads * vdim
        self.conv = (
            CausalConvTails(self.n_in, conv_taps, residual=False)
            if conv_taps and conv_taps > 0 else None
        )
        half = int(rot_dims) // 2
        i = torch.arange(half, dtype=torch.float64)
        inv = float(rot_base) ** (-2.0 * i / max(int(rot_dims), 1))
        self.register_buffer("inv_freq", inv.to(torch.float32), persistent=False)

    def state_spec(self):
        return {"conv": self.conv.state_shape()} if self.conv is not None else {}

    def kv_spec(self):
        return (self.kv_heads, self.dim, self.vdim)

    def forward(self, qkv, fb, state, kv_cache, out, out_scale=1.0):
        T = qkv.shape[0]
        if self.conv is not None:
            qkv = self.conv(qkv, fb, state["conv"])
        nq, nk, nv = self.sizes
        q = qkv[:, :nq].unflatten(-1, (self.heads, self.dim))
        k = qkv[:, nq : nq + nk].unflatten(-1, (self.kv_heads, self.dim))
        v = qkv[:, nq + nk :].unflatten(-1, (self.kv_heads, self.vdim))
        k_cache, v_cache = kv_cache
        sops.rope_pairs_and_cache(q, k, v, fb.positions, self.inv_freq, k_cache,
                                  v_cache, fb.slot_mapping)
        sops.masked_paged_attention(
            q, k_cache, v_cache, fb.seq, self.scale,
            out.unflatten(-1, (self.heads, self.vdim)),
            softcap=self.softcap, chunk=self.chunk, window=self.window,
            out_scale=out_scale,
        )
        return out


class LightningAttention(nn.Module):
    """Linear attention with a constant per-head state decay, silu on q/k/v,
    an RMS norm over the concatenated heads and a sigmoid output gate.
    Takes the projected [T, q|k|v|g] block."""

    def __init__(self, heads, dim, vdim, decay, eps):
        super().__init__()
        self.heads, self.dim, self.vdim, self.eps = heads, dim, vdim, eps
        self.sizes = (heads * dim, heads * dim, heads * vdim, heads * vdim)
        self.n_in = sum(self.sizes)
        self.n_out = heads * vdim
        self.register_buffer(
            "decay", torch.tensor(list(decay), dtype=torch.float32), persistent=False
        )
        self.norm = _f32(self.n_out)

    def state_spec(self):
        return {"s": (self.heads, self.dim, self.vdim)}

    def kv_spec(self):
        return None

    def forward(self, qkvg, fb, state, out, out_scale=1.0):
        T = qkvg.shape[0]
        H, D, Dv = self.heads, self.dim, self.vdim
        a, b, c, _ = self.sizes
        q = qkvg[:, :a].unflatten(-1, (H, D))
        k = qkvg[:, a : a + b].unflatten(-1, (H, D))
        v = qkvg[:, a + b : a + b + c].unflatten(-1, (H, Dv))
        g = qkvg[:, a + b + c :]
        o = sops.linear_attn_scan(q, k, v, self.decay, None, state["s"], fb.seq,
                                  silu_inputs=True)
        sops.gated_rmsnorm(o.view(T, H * Dv), self.norm, g, 1, "sigmoid",
                           self.eps, out, out_scale)
        return out


class ParallelMixer(nn.Module):
    """Chunked softmax attention and lightning attention fed by one input
    and summed with fixed scales. Both input projections are one
    GEMM; both output projections are one GEMM over the concatenated
    (pre-scaled) branch outputs."""

    def __init__(self, width, left: ChunkedAttention, right: LightningAttention,
                 left_scale: float, right_scale: float):
        super().__init__()
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.in_proj = Proj(width, left.n_in + right.n_in)
        self.o_proj = Proj(left.n_out + right.n_out, width)

    def state_spec(self):
        spec = {"left." + k: v for k, v in self.left.state_spec().items()}
        spec.update({"right." + k: v for k, v in self.right.state_spec().items()})
        return spec

    def kv_spec(self):
        return self.left.kv_spec()

    def forward(self, h, fb, state, kv_cache):
        T = h.shape[0]
        proj = self.in_proj(h)
        nl = self.left.n_in
        cat = torch.empty((T, self.left.n_out + self.right.n_out), dtype=h.dtype,
                          device=h.device)
        ls = {k[5:]: v for k, v in state.items() if k.startswith("left.")}
        rs = {k[6:]: v for k, v in state.items() if k.startswith("right.")}
        self.left(proj[:, :nl], fb, ls, kv_cache, cat[:, : self.left.n_out],
                  self.left_scale)
        self.right(proj[:, nl:], fb, rs, cat[:, self.left.n_out :],
                   self.right_scale)
        return self.o_proj(cat)


class SquaredReluMLP(nn.Module):
    """Dense feed-forward: down(relu(up(h))^2)."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.up = Proj(width, ff)
        self.down = Proj(ff, width)

    def forward(self, h):
        return self.down(sops.relu_squared(self.up(h)))


def scaled_rotary_frequencies(dims: int, base: float, scaling: dict | None):
    """fp32 [dims/2] rotary frequencies base^(-2i/dims), optionally rescaled
    by wavelength (scaling = {factor, low, high, original}): wavelengths
    below original/high keep their frequency, those above original/low are
    divided by factor, and the band between is interpolated linearly in
    original/wavelength."""
    import math

    out = []
    for i in range(int(dims) // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high = (float(scaling[k]) for k in ("factor", "low", "high"))
            orig = float(scaling["original"])
            lam = 2.0 * math.pi / f
            if lam > orig / low:
                f = f / factor
            elif lam >= orig / high:
                s = (orig / lam - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float32)


class SinkWindowAttention(nn.Module):
    """Softmax attention over a sliding window of cached keys with grouped
    key/value heads and separate key and value sizes. Options, each a
    constructor argument: an RMS norm over the whole q and the whole k
    projection (all heads at once) before rotation, rotary on the leading
    dims of every head in the split-half pairing with wavelength-dependent
    frequency scaling, and a sink (a value-less key of score 0)."""

    def __init__(self, width, heads, kv_heads, dim, vdim, scale, window=0,
                 sink=False, qk_norm=False, rot_dims=0, rot_base=10000.0,
                 rot_scaling=None, eps=1e-5):
        super().__init__()
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.window, self.sink, self.eps = float(scale), int(window or 0), bool(sink), eps
        self.sizes = (heads * dim, kv_heads * dim, kv_heads * vdim)
        self.in_proj = Proj(width, sum(self.sizes))  # q | k | v
        self.o_proj = Proj(heads * vdim, width)
        self.q_norm = self.k_norm = None
        if qk_norm:
            self.q_norm, self.k_norm = _f32(heads * dim), _f32(kv_heads * dim)
            nn.init.ones_(self.q_norm)
            nn.init.ones_(self.k_norm)
        self.register_buffer(
            "inv_freq", scaled_rotary_frequencies(rot_dims, rot_base, rot_scaling),
            persistent=False)
        # the sink of this mixer is a key of score 0 for every head
        self.sink_scores = _f32(heads) if self.sink else None

    def state_spec(self):
        return {}

    def kv_spec(self):
        return (self.kv_heads, self.dim, self.vdim)

    def forward(self, h, fb, state, kv_cache):
        T = h.shape[0]
        nq, nk, nv = self.sizes
        qkv = self.in_proj(h)
        q = qkv[:, :nq].unflatten(-1, (self.heads, self.dim))
        k = qkv[:, nq : nq + nk].unflatten(-1, (self.kv_heads, self.dim))
        v = qkv[:, nq + nk :].unflatten(-1, (self.kv_heads, self.vdim))
        k_cache, v_cache = kv_cache
        sops.qknorm_rope_half_and_cache(q, k, v, self.q_norm, self.k_norm, self.eps,
                                        fb.positions, self.inv_freq, k_cache, v_cache,
                                        fb.slot_mapping)
        out = torch.empty((T, self.heads, self.vdim), dtype=h.dtype, device=h.device)
        sops.masked_paged_attention(q, k_cache, v_cache, fb.seq, self.scale, out,
                                    window=self.window, sink=self.sink_scores)
        return self.o_proj(out.view(T, self.heads * self.vdim))


def ramped_rotary_frequencies(dims: int, base: float, scaling: dict | None):
    """fp32 [dims/2] rotary frequencies f_i = base^(-2i/dims) and the factor
    that multiplies cos and sin. With scaling = {factor, original, fast,
    slow}, pair i is interpolated between its own frequency and f_i / factor
    by a ramp over the pair index: the ramp runs from the pair that turns
    `fast` times within `original` positions to the one that turns `slow`
    times, d(t) = dims ln(original / (2 pi t)) / (2 ln base),
    lo = max(floor d(fast), 0), hi = min(ceil d(slow), dims - 1),
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i); the multiplier is
    0.1 ln(factor) + 1 (1 without scaling)."""
    import math

    f = [float(base) ** (-2.0 * i / dims) for i in range(int(dims) // 2)]
    mult = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def d(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(d(float(scaling["fast"]))), 0)
        hi = min(math.ceil(d(float(scaling["slow"]))), dims - 1)
        for i, fi in enumerate(f):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = fi / factor * ramp + fi * (1.0 - ramp)
        mult = 0.1 * math.log(factor) + 1.0
    return torch.tensor(f, dtype=torch.float32), mult


class LatentAttention(nn.Module):
    """Causal attention whose keys and values are per-head up-projections of
    one low-rank latent per token; only the (RMS-normed) latent is cached,
    as a one-head paged cache. Options, each a constructor argument:

      q_rank    queries go through a latent of their own: an RMS-normed
                down-projection followed by an up-projection (0 = one matrix)
      rot_dim   every query head has rot_dim more dimensions that are rotated
                by position, against one rotated key part shared by all heads
                and cached behind the latent (0 = no positions enter)
      sink      a learned score per head that joins the softmax denominator
                without a value
      gate      "channel": every output channel times sigmoid of a projection
                of the input; "head": one such gate per head; None

    The kernel attends in latent space: the key up-projection is folded into
    the query (q_h W_uk_h, one product per head), scores and the weighted sum
    run against the cached rows (the rotated parts just extend the dot
    product), and the value up-projection is applied to the attended latent.
    With own_latent=False the layer has no down-projection and reads the
    cache of another layer (bound by the model)."""

    def __init__(self, width, heads, dim, vdim, kv_rank, scale, own_latent=True,
                 eps=1e-5, q_rank=0, rot_dim=0, rot_base=10000.0, rot_scaling=None,
                 sink=False, gate="channel"):
        super().__init__()
        self.heads, self.dim, self.vdim, self.rank = heads, dim, vdim, kv_rank
        self.scale, self.own_latent, self.eps = float(scale), bool(own_latent), eps
        self.q_rank, self.rot_dim, self.gate = int(q_rank or 0), int(rot_dim or 0), gate
        if gate not in ("channel", "head", None):
            raise ValueError(f"unknown gate {gate!r}")
        if self.rot_dim % 2:
            raise ValueError("rot_dim must be even")
        if self.rot_dim and not own_latent:
            raise ValueError("a borrowed latent carries no rotated key part")
        qd = dim + self.rot_dim
        n_q = self.q_rank if self.q_rank else heads * qd
        n_g = {"channel": heads * vdim, "head": heads, None: 0}[gate]
        self.sizes = (n_q, n_g, kv_rank + self.rot_dim if own_latent else 0)
        self.in_proj = Proj(width, sum(self.sizes))  # q (or its latent) | gate | latent
        self.q_norm = self.q_up = None
        if self.q_rank:
            self.q_norm = _f32(self.q_rank)
            nn.init.ones_(self.q_norm)
            self.q_up = Proj(self.q_rank, heads * qd)
        self.latent_norm = None
        if own_latent:
            self.latent_norm = _f32(kv_rank)
            nn.init.ones_(self.latent_norm)
        # per-head up-projections as Linear-style weights of the folded maps:
        # uk_r [H, rank, dim] takes q_h into latent space (the transposed key
        # up-projection), uv [H, vdim, rank] takes the attended latent out
        self.uk_r = nn.Parameter(torch.empty(heads, kv_rank, dim), requires_grad=False)
        self.uv = nn.Parameter(torch.empty(heads, vdim, kv_rank), requires_grad=False)
        nn.init.normal_(self.uk_r, std=kv_rank ** -0.5)
        nn.init.normal_(self.uv, std=kv_rank ** -0.5)
        self.sink_scores = _f32(heads) if sink else None
        freqs, self.rot_mult = ramped_rotary_frequencies(
            max(self.rot_dim, 1), rot_base, rot_scaling)
        self.register_buffer("inv_freq", freqs[: self.rot_dim // 2], persistent=False)
        self.o_proj = Proj(heads * vdim, width)

    def state_spec(self):
        return {}

    def kv_spec(self):
        # one "head" of kv_rank (+ rot_dim) dims; keys and values are the same
        # rows, the values their first kv_rank columns
        return (1, self.rank + self.rot_dim, 0) if self.own_latent else None

    def forward(self, h, fb, state, kv_cache):
        T = h.shape[0]
        H, D, Dv, R, r = self.heads, self.dim, self.vdim, self.rank, self.rot_dim
        nq, ng, _ = self.sizes
        proj = self.in_proj(h)
        c_cache = kv_cache[0]
        if self.q_rank:
            q = self.q_up(sops.rmsnorm_rows(proj[:, :nq], self.q_norm, self.eps))
        else:
            q = proj[:, :nq]
        q = q.unflatten(-1, (H, D + r))
        ql = torch.empty((T, H, R + r), dtype=h.dtype, device=h.device)
        if self.own_latent and r:
            sops.latent_rope_to_cache(proj[:, nq + ng :], self.latent_norm, self.eps,
                                      q[..., D:], ql[..., R:], fb.positions,
                                      self.inv_freq, self.rot_mult, c_cache,
                                      fb.slot_mapping)
        elif self.own_latent:
            sops.rmsnorm_to_cache(proj[:, nq + ng :], self.latent_norm, self.eps,
                                  c_cache, fb.slot_mapping)
        sops.head_linear(q[..., :D], self.uk_r, out=ql[..., :R])  # [T, H, R]
        lat = torch.empty((T, H, R), dtype=h.dtype, device=h.device)
        sops.masked_paged_attention(ql, c_cache, c_cache[..., :R] if r else c_cache,
                                    fb.seq, self.scale, lat, sink=self.sink_scores)
        o = sops.head_linear(lat, self.uv,
                             gate=proj[:, nq : nq + ng] if ng else None)  # [T, H, Dv]
        return self.o_proj(o.view(T, H * Dv))


class GatedDeltaMixer(nn.Module):
    """Gated delta rule: a matrix state per head that decays by a
    data-dependent factor and is corrected towards the current value along
    the current key (S <- g S; S += k (beta (v - S^T k))^T; o = S^T q).
    q and k have kv_heads heads shared by groups of value heads; q, k and v
    pass a short causal convolution with silu; q and k are unit vectors per
    head (q times dim^-1/2). The read-out is RMS-normed per head (one weight
    vector shared by the heads) and gated by silu of a projection."""

    def __init__(self, width, heads, kv_heads, dim, vdim, conv_taps, eps):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kv_heads, self.dim, self.vdim, self.eps = heads, kv_heads, dim, vdim, eps
        nqk, nv = kv_heads * dim, heads * vdim
        self.sizes = (nqk, nqk, nv, nv, heads, heads)  # q | k | v | gate | beta | decay
        self.in_proj = Proj(width, sum(self.sizes))
        self.conv = CausalConvTails(2 * nqk + nv, conv_taps, residual=False, act="silu")
        self.a_log = _f32(heads)
        self.dt_bias = _f32(heads)
        self.norm = _f32(nv)  # the per-head weight, repeated for every head
        nn.init.ones_(self.norm)
        self.o_proj = Proj(nv, width)

    def state_spec(self):
        return {"conv": self.conv.state_shape(),
                "s": (self.heads, self.dim, self.vdim)}

    def kv_spec(self):
        return None

    def forward(self, h, fb, state, kv_cache):
        T = h.shape[0]
        H, G, D, Dv = self.heads, self.kv_heads, self.dim, self.vdim
        nqk, nv = G * D, H * Dv
        proj = self.in_proj(h)
        qkv = self.conv(proj[:, : 2 * nqk + nv], fb, state["conv"])
        at = 2 * nqk + 2 * nv
        o = sops.gated_delta_scan(
            qkv[:, :nqk].unflatten(-1, (G, D)), qkv[:, nqk : 2 * nqk].unflatten(-1, (G, D)),
            qkv[:, 2 * nqk :].unflatten(-1, (H, Dv)), proj[:, at : at + H],
            proj[:, at + H : at + 2 * H], self.a_log, self.dt_bias,
            state["s"], fb.seq)
        y = torch.empty((T, nv), dtype=h.dtype, device=h.device)
        sops.gated_rmsnorm(o.view(T, nv), self.norm, proj[:, 2 * nqk + nv : at], H,
                           "silu", self.eps, y)
        return self.o_proj(y)


class GeluMLP(nn.Module):
    """Dense feed-forward: down(gelu(up(h))), the exact (erf) GELU."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.up = Proj(width, ff)
        self.down = Proj(ff, width)

    def forward(self, h):
        return self.down(sops.gelu(self.up(h)))


class RoutedSquaredReluMoE(nn.Module):
    """Mixture of squared-ReLU experts (down(relu(up h)^2), no biases) with
    fp32 top-k routing, weights = softmax over the chosen logits, plus an
    optional shared expert that every token uses.

    All up-projections are one stacked matrix [E*ff + shared_ff, width] and
    all down-projections one [width, E*ff + shared_ff]. Small steps (decode)
    run them as two GEMMs over every expert with the routing weight (0 for
    experts a token did not choose) folded into the activation, so the sum
    over experts happens inside the second GEMM's fp32 accumulation and the
    step has no data-dependent shapes. Large steps gather each expert's
    tokens and run its slice of the stacked matrices."""

    DENSE_MAX_TOKENS = 256

    def __init__(self, width, experts, top, ff, shared_ff=0):
        super().__init__()
        self.experts, self.top, self.ff, self.shared_ff = experts, top, ff, int(shared_ff or 0)
        n = experts * ff + self.shared_ff
        self.router = nn.Parameter(torch.empty(experts, width, dtype=torch.float32),
                                   requires_grad=False)
        nn.init.normal_(self.router, std=width ** -0.5)
        self.up = Proj(width, n)
        self.down = Proj(n, width)

    def forward(self, h):
        T = h.shape[0]
        E, ff = self.experts, self.ff
        logits = F.linear(h.float(), self.router)
        dense, w, idx = sops.router_topk(logits, self.top)
        if T <= self.DENSE_MAX_TOKENS:
            a = sops.relu_squared_weighted(self.up(h), dense, ff)
            return self.down(a)
        out = torch.zeros((T, h.shape[1]), dtype=torch.float32, device=h.device)
        flat = idx.flatten().long()
        order = torch.argsort(flat, stable=True)
        counts = torch.bincount(flat, minlength=E).tolist()
        tok = order // self.top
        wrow = w.flatten()[order].unsqueeze(1)
        s = 0
        for e in range(E):
            n = counts[e]
            if n == 0:
                continue
            rows = tok[s : s + n]
            u = F.linear(h.index_select(0, rows), self.up.weight[e * ff : (e + 1) * ff])
            a = sops.relu_squared_weighted(u, wrow[s : s + n], ff)
            y = F.linear(a, self.down.weight[:, e * ff : (e + 1) * ff])
            out.index_add_(0, rows, y.float())
            s += n
        if self.shared_ff:
            u = F.linear(h, self.up.weight[E * ff :])
            y = F.linear(sops.relu_squared(u), self.down.weight[:, E * ff :])
            out.add_(y)
        return out


class RoutedGatedMoE(nn.Module):
    """Mixture of gated experts (down(act(gate h) * (up h)), no biases).
    Routing: fp32 logits, scores = softmax over all experts; the `top`
    experts with the largest score + correction (a per-expert bias that only
    steers the choice) are used, weighted by their scores as they are (times
    weight_scale).

    The activation is g * sigmoid(act_alpha * g) * (u + up_shift), with
    g = min(gate, act_limit) and u = clamp(up, +-act_limit) when act_limit > 0
    (defaults: silu(gate) * up). shared_ff > 0 adds one expert of that size
    that every token uses (its own clamp shared_limit), weighted by the
    sigmoid of one more router row when shared_gate is set.

    Expert e's gate and up matrices are rows [e*2ff, e*2ff + ff) and
    [e*2ff + ff, (e+1)*2ff) of one stacked matrix (the shared expert's follow
    them), all down-projections one [width, E*ff + shared_ff]. Small steps
    (decode) run two GEMMs over every expert with the routing weight (0 for
    experts a token did not choose) folded into the activation, so the
    weighted sum happens inside the second GEMM's fp32 accumulation and the
    step has no data-dependent shapes. Large steps gather each expert's
    tokens and run its slice.

    extra_out > 0 appends that many rows (with a bias) to the stacked input
    matrix for a projection of the same input that the caller owns (a
    residual gate); forward then returns (output, that projection)."""

    DENSE_MAX_TOKENS = 256

    def __init__(self, width, experts, top, ff, correction=True, act_alpha=1.0,
                 act_limit=0.0, up_shift=0.0, weight_scale=1.0, shared_ff=0,
                 shared_limit=0.0, shared_gate=False, extra_out=0):
        super().__init__()
        self.experts, self.top, self.ff = experts, top, ff
        self.act = dict(alpha=float(act_alpha), limit=float(act_limit or 0.0),
                        up_shift=float(up_shift))
        self.weight_scale = float(weight_scale)
        self.shared_ff = int(shared_ff or 0)
        self.shared_act = dict(self.act, limit=float(shared_limit or 0.0))
        self.shared_gate = bool(shared_gate) and self.shared_ff > 0
        # the shared expert's gate is one more row behind the experts'
        self.router = nn.Parameter(
            torch.empty(experts + int(self.shared_gate), width, dtype=torch.float32),
            requires_grad=False)
        nn.init.normal_(self.router, std=width ** -0.5)
        self.correction = _f32(experts) if correction else None
        self.extra_out = int(extra_out or 0)
        n_in = experts * 2 * ff + 2 * self.shared_ff + self.extra_out
        self.gate_up = BiasProj(width, n_in) if self.extra_out else Proj(width, n_in)
        self.down = Proj(experts * ff + self.shared_ff, width)

    def forward(self, h):
        T = h.shape[0]
        E, ff, sff = self.experts, self.ff, self.shared_ff
        logits = F.linear(h.float(), self.router)
        sg = logits[:, E:] if self.shared_gate else None
        dense, w, idx = sops.router_scores_topk(
            logits[:, :E] if self.shared_gate else logits, self.top, self.correction,
            self.weight_scale)
        at = E * 2 * ff + 2 * sff  # where the caller's extra projection starts
        if T <= self.DENSE_MAX_TOKENS:
            gu = self.gate_up(h)
            a = torch.empty((T, E * ff + sff), dtype=h.dtype, device=h.device)
            sops.glu_weighted(gu[:, : E * 2 * ff], dense, ff, out=a[:, : E * ff],
                              **self.act)
            if sff:
                sops.glu_weighted(gu[:, E * 2 * ff : at], sg, sff, w_sigmoid=True,
                                  out=a[:, E * ff :], **self.shared_act)
            y = self.down(a)
            return (y, gu[:, at:]) if self.extra_out else y
        out = torch.zeros((T, h.shape[1]), dtype=torch.float32, device=h.device)
        flat = idx.flatten().long()
        order = torch.argsort(flat, stable=True)
        counts = torch.bincount(flat, minlength=E).tolist()
        tok = order // self.top
        wrow = w.flatten()[order].unsqueeze(1)
        s = 0
        for e in range(E):
            n = counts[e]
            if n == 0:
                continue
            rows = tok[s : s + n]
            gu = F.linear(h.index_select(0, rows),
                          self.gate_up.weight[e * 2 * ff : (e + 1) * 2 * ff])
            a = sops.glu_weighted(gu, wrow[s : s + n], ff, **self.act)
            y = F.linear(a, self.down.weight[:, e * ff : (e + 1) * ff])
            out.index_add_(0, rows, y.float())
            s += n
        extra = None
        if sff or self.extra_out:
            # the shared expert's rows and the caller's are one product
            bias = self.gate_up.bias[E * 2 * ff :] if self.extra_out else None
            gu = F.linear(h, self.gate_up.weight[E * 2 * ff :], bias)
            if sff:
                a = sops.glu_weighted(gu[:, : 2 * sff], sg, sff, w_sigmoid=True,
                                      **self.shared_act)
                out.add_(F.linear(a, self.down.weight[:, E * ff :]))
            extra = gu[:, 2 * sff :]
        return (out, extra) if self.extra_out else out


class SiluGatedMLP(nn.Module):
    """Dense gated feed-forward: down(silu(gate h) * (up h)); the gate and up
    matrices are one stacked [2 ff, width] product. extra_out > 0 appends
    that many rows (with a bias) for a projection of the same input that the
    caller owns; forward then returns (output, that projection)."""

    def __init__(self, width: int, ff: int, extra_out: int = 0):
        super().__init__()
        self.ff, self.extra_out = ff, int(extra_out or 0)
        n_in = 2 * ff + self.extra_out
        self.gate_up = BiasProj(width, n_in) if self.extra_out else Proj(width, n_in)
        self.down = Proj(ff, width)

    def forward(self, h):
        gu = self.gate_up(h)
        y = self.down(sops.glu_weighted(gu[:, : 2 * self.ff], None, self.ff))
        return (y, gu[:, 2 * self.ff :]) if self.extra_out else y


class BiasProj(nn.Module):
    """Linear layer [out, in] with a bias, both in the serving dtype (the
    bias is added in the product's epilogue)."""

    def __init__(self, n_in: int, n_out: int):
        super().__init__()
        self.weight = nn.Parameter(torch.empty(n_out, n_in), requires_grad=False)
        nn.init.normal_(self.weight, std=n_in ** -0.5)
        self.bias = nn.Parameter(torch.zeros(n_out), requires_grad=False)

    def forward(self, x):
        return F.linear(x, self.weight, self.bias)


class DifferentialAttention(nn.Module):
    """Causal softmax attention in which every query head computes two score
    maps (two query and two key vectors per head) over the same values and
    outputs their difference, map 1 - lam * map 2, RMS-normed per head
    (no weight) and scaled by `gain`. Grouped key/value heads, separate key
    and value sizes, a tanh cap on the scores, biases on every projection.
    Positions enter only through a query temperature
    1 + coef * ln(floor((p + 1) / every) + 1) (coef 0: none).

    lam is one number for the layer: exp(lq1 . lk1) - exp(lq2 . lk2) + lam0.

    The two maps are ordinary attention heads to the kernels: the cache keeps
    2 G key heads (head 2 g + m is map m of group g) and G value heads; the
    query rows are ordered (group, map, head in group), so that query head j
    reads key head j // R and value head j // 2R (R = heads per group)."""

    def __init__(self, width, heads, kv_heads, dim, vdim, scale, softcap=0.0,
                 lam0=0.0, gain=1.0, temp_coef=0.0, temp_every=1, eps=1e-6):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.softcap = float(scale), float(softcap or 0.0)
        self.lam0, self.gain, self.eps = float(lam0), float(gain), eps
        self.temp_coef, self.temp_every = float(temp_coef or 0.0), max(1, int(temp_every))
        self.sizes = (2 * heads * dim, 2 * kv_heads * dim, kv_heads * vdim)
        self.in_proj = BiasProj(width, sum(self.sizes))  # q | k | v
        self.o_proj = BiasProj(heads * vdim, width)
        self.lam_q = _f32(2, dim)
        self.lam_k = _f32(2, dim)
        self._lam = None

    def state_spec(self):
        return {}

    def kv_spec(self):
        # (key heads, key size, value size, value heads)
        return (2 * self.kv_heads, self.dim, self.vdim, self.kv_heads)

    def query_row_order(self):
        """Index of the checkpoint's query rows (head, map, dim) in the
        engine's order (group, map, head in group, dim)."""
        H, G, D = self.heads, self.kv_heads, self.dim
        idx = torch.arange(2 * H * D).view(G, H // G, 2, D)
        return idx.permute(0, 2, 1, 3).reshape(-1)

    @property
    def lam(self) -> float:
        if self._lam is None:
            dots = (self.lam_q.double() * self.lam_k.double()).sum(-1).float()
            e = torch.exp(dots)
            self._lam = float(e[0] - e[1]) + self.lam0
        return self._lam

    def forward(self, h, fb, state, kv_cache):
        T = h.shape[0]
        H, G, D, Dv = self.heads, self.kv_heads, self.dim, self.vdim
        nq, nk, _ = self.sizes
        qkv = self.in_proj(h)
        q = qkv[:, :nq].unflatten(-1, (2 * H, D))
        k = qkv[:, nq : nq + nk].unflatten(-1, (2 * G, D))
        v = qkv[:, nq + nk :].unflatten(-1, (G, Dv))
        k_cache, v_cache = kv_cache
        sops.scale_q_and_cache(q, k, v, fb.positions, self.temp_coef, self.temp_every,
                               k_cache, v_cache, fb.slot_mapping)
        att = torch.empty((T, 2 * H, Dv), dtype=h.dtype, device=h.device)
        sops.masked_paged_attention(q, k_cache, v_cache, fb.seq, self.scale, att,
                                    softcap=self.softcap)
        out = torch.empty((T, H, Dv), dtype=h.dtype, device=h.device)
        sops.diff_combine(att.view(T, G, 2, H // G, Dv), self.lam, self.gain, self.eps,
                          out)
        return self.o_proj(out.view(T, H * Dv))


class GeneralDeltaMixer(nn.Module):
    """Generalized delta rule: a matrix state per head with a per-channel,
    data-dependent decay (through a low-rank tanh bottleneck) and a
    per-channel removal rate along the unit key:
    S <- diag(w) S - (a * n)(n^T S) + k v^T, o = S^T r (ops.seq.diag_rank1_scan).
    r, k, v have heads x dim channels; the read-out is RMS-normed per head,
    times a weight over all heads, times sigmoid of a gate projection."""

    def __init__(self, width, heads, dim, lowrank, eps, decay_scale=0.6065306597126334,
                 key_eps=1e-6):
        super().__init__()
        self.heads, self.dim, self.lowrank, self.eps = heads, dim, int(lowrank), eps
        self.decay_scale, self.key_eps = float(decay_scale), float(key_eps)
        n = heads * dim
        self.in_proj = Proj(width, 5 * n + self.lowrank)  # r | k | v | g | a | w1
        self.w2 = Proj(self.lowrank, n)
        self.w0 = _f32(n)
        self.a_bias = _f32(n)
        self.norm = _f32(n)
        nn.init.ones_(self.norm)
        self.o_proj = Proj(n, width)

    def set_lowrank(self, lowrank: int):
        """Resize the decay bottleneck (a checkpoint gives its size by the
        shape of its tensors)."""
        if int(lowrank) == self.lowrank:
            return
        n, w = self.heads * self.dim, self.in_proj.weight
        self.lowrank = int(lowrank)
        self.in_proj.weight = nn.Parameter(
            torch.zeros((5 * n + self.lowrank, w.shape[1]), dtype=w.dtype, device=w.device),
            requires_grad=False)
        self.w2.weight = nn.Parameter(
            torch.zeros((n, self.lowrank), dtype=w.dtype, device=w.device),
            requires_grad=False)

    def state_spec(self):
        return {"s": (self.heads, self.dim, self.dim)}

    def kv_spec(self):
        return None

    def forward(self, h, fb, state, kv_cache):
        T = h.shape[0]
        H, D = self.heads, self.dim
        n = H * D
        proj = self.in_proj(h)
        w_pre = self.w2(torch.tanh(proj[:, 5 * n :]))
        part = lambda i: proj[:, i * n : (i + 1) * n].unflatten(-1, (H, D))
        o = sops.diag_rank1_scan(part(0), part(1), part(2), w_pre.view(T, H, D), part(4),
                                 self.w0, self.a_bias, state["s"], fb.seq,
                                 self.decay_scale, self.key_eps)
        y = torch.empty((T, n), dtype=h.dtype, device=h.device)
        sops.gated_rmsnorm(o.view(T, n), self.norm, proj[:, 3 * n : 4 * n], H, "sigmoid",
                           self.eps, y)
        return self.o_proj(y)
