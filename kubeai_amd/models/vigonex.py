"""Vigonex: a decoder whose config lists its layers, built around several
residual streams (hyper-connections). Every sublayer q of a layer reads a
learned combination of the streams and writes back into all of them:

    u = sum_s in_q[s] x_s;  h = rmsnorm(u) * w_q
    y = sublayer(h) * sigmoid(R_q h + b_q)                 (gated residual)
    x_t <- sum_s mix_q[s, t] x_s + out_q[t] * y            (all t at once)

The mixer reads h after a token shift (h + (h_prev - h) * mu, the previous
token's h being sequence state); the gate reads h as it is. Mixers:
differential attention (two softmax maps per head over shared values, query
temperature by position, tanh-capped scores) and the generalized delta rule
(matrix state with per-channel decay and removal along the unit key);
feed-forwards: a dense silu-gated layer or a mixture of clamped gated
experts with a sigmoid-gated shared expert (kubeai_amd.models.mixers). The
embedding is scaled and gets a sinusoidal position vector; the logits are
scaled.

Same execution model as the other layer-list decoders: one token-packed
forward per engine step, GEMMs through the BLAS library in the serving dtype,
everything else in the gfx950 kernels of kubeai_amd.ops.seq. The streams are
fp32; a sublayer's write into the streams, the read for the next sublayer
and its norm are one kernel.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from kubeai_amd.engine.batch import ForwardBatch
from kubeai_amd.ops import seq as sops
from .config import HybridLayerSpec, ModelArchConfig
from .mixers import (
    BiasProj,
    DifferentialAttention,
    GeneralDeltaMixer,
    RoutedGatedMoE,
    SiluGatedMLP,
    _f32,
)


def build_mixer(spec: HybridLayerSpec, width: int, eps: float) -> nn.Module:
    m = spec.mixer
    if spec.type == "attention":
        qt = m.get("q_temp") or {}
        diff = float(m.get("diff", 0.0))
        return DifferentialAttention(
            width, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
            dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=m["scale"],
            softcap=m.get("softcap") or 0.0, lam0=diff, gain=1.0 - diff,
            temp_coef=float(qt.get("coef", 0.0)), temp_every=int(qt.get("every", 1)),
            eps=eps,
        )
    if spec.type == "general_delta":
        return GeneralDeltaMixer(width, heads=int(m["heads"]), dim=int(m["dim"]),
                                 lowrank=int(m.get("lowrank") or max(8, width // 16)),
                                 eps=eps)
    raise ValueError(f"unknown mixer type {spec.type!r}")


def build_mlp(mlp: dict | None, width: int):
    if mlp is None:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        return SiluGatedMLP(width, int(mlp["ff"]), extra_out=width)
    if kind == "moe":
        shared = mlp.get("shared") or {}
        return RoutedGatedMoE(
            width, experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
            ff=int(mlp["expert"]["ff"]), correction=False, act_alpha=1.702,
            act_limit=float(mlp["expert"].get("limit") or 0.0), up_shift=1.0,
            weight_scale=float(mlp["router"].get("scale", 1.0)),
            shared_ff=int(shared.get("ff", 0)),
            shared_limit=float(shared.get("limit") or 0.0), shared_gate=True,
            extra_out=width,
        )
    raise ValueError(f"unknown feed-forward kind {kind!r}")


class HyperConnection(nn.Module):
    """Read weights, write weights and the stream-to-stream matrix of one
    sublayer, with its input norm and residual gate (own_gate=False: the
    sublayer computes the gate's projection inside its own input product)."""

    def __init__(self, width: int, streams: int, own_gate: bool = True):
        super().__init__()
        self.norm = _f32(width)
        nn.init.ones_(self.norm)
        self.read = _f32(streams)
        self.write = _f32(streams)
        self.mix = _f32(streams, streams)
        nn.init.constant_(self.read, 1.0 / streams)
        nn.init.ones_(self.write)
        self.mix.data.copy_(torch.eye(streams))
        self.gate = BiasProj(width, width) if own_gate else None


class VigonexLayer(nn.Module):
    def __init__(self, spec: HybridLayerSpec, width: int, eps: float, streams: int):
        super().__init__()
        self.mixer = build_mixer(spec, width, eps)
        self.mlp = build_mlp(spec.mlp, width)
        self.hc1 = HyperConnection(width, streams)
        # the feed-forward's gate reads the feed-forward's input: one product
        self.hc2 = (HyperConnection(width, streams, own_gate=False)
                    if self.mlp is not None else None)
        self.shift = _f32(1, width)

    def state_spec(self):
        spec = dict(self.mixer.state_spec())
        spec["prev"] = (1, self.shift.shape[1])
        return spec


def sinusoid_frequencies(width: int, base: float = 10000.0) -> torch.Tensor:
    """float64 [ceil(width / 2)]: base^(-2 i / width)."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    return float(base) ** (-2.0 * i / width)


class VigonexForCausalLM(nn.Module):
    #: token shifts and delta-rule layers carry state: the engine gives every
    #: live sequence a state slot and builds fb.seq
    has_seq_state = True

    def __init__(self, cfg: ModelArchConfig, device=None, dtype=torch.bfloat16):
        super().__init__()
        assert cfg.hybrid is not None
        self.cfg = cfg
        self.dtype = dtype
        hs = cfg.hybrid
        W = cfg.hidden_size
        self.eps = hs.norm_eps
        self.streams = int(hs.streams)
        self.logit_scale = float(hs.logit_scale)
        prev_dtype = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            with torch.device(device if device is not None else "cpu"):
                self.embed_tokens = nn.Embedding(cfg.vocab_size, W)
                self.layers = nn.ModuleList(
                    [VigonexLayer(spec, W, hs.norm_eps, self.streams) for spec in hs.layers]
                )
                self.final_norm = _f32(W)
                nn.init.ones_(self.final_norm)
                self.final_read = _f32(self.streams)
                nn.init.ones_(self.final_read)  # the streams are summed at the end
                self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W),
                                            requires_grad=False)
                nn.init.normal_(self.lm_head, std=W ** -0.5)
                self.register_buffer("pos_freqs", sinusoid_frequencies(W),
                                     persistent=False)
        finally:
            torch.set_default_dtype(prev_dtype)
        self.capture_layers = None  # set to a list to record per-layer residuals

    # -- what the runner allocates per layer -----------------------------
    def kv_cache_specs(self):
        return [layer.mixer.kv_spec() for layer in self.layers]

    def state_specs(self):
        return [layer.state_spec() for layer in self.layers]

    def bind_kv_caches(self, kv_caches):
        self.kv_caches = kv_caches

    def bind_states(self, states):
        self.states = states

    # --------------------------------------------------------------------
    def _streams_after(self, X, y, gate, hc):
        z = y.float() * torch.sigmoid(gate.float())
        return (torch.einsum("st,nsc->ntc", hc.mix, X)
                + hc.write.view(1, -1, 1) * z.unsqueeze(1)).sum(1)

    @torch.inference_mode()
    def forward(self, fb: ForwardBatch) -> torch.Tensor:
        hs = self.cfg.hybrid
        X = sops.embed_sinusoid(fb.input_ids, self.embed_tokens.weight,
                                hs.embedding_scale, fb.positions, self.pos_freqs,
                                self.streams)  # [T, S, C] fp32
        y = gate = hc = None  # the sublayer output not yet written to the streams

        def read(nxt):
            return sops.hyper_mix_rmsnorm(
                X, y, gate, hc.mix if hc is not None else None,
                hc.write if hc is not None else None, nxt.read, nxt.norm, self.eps,
                self.dtype)

        for i, layer in enumerate(self.layers):
            state = self.states[i]
            h = read(layer.hc1)
            hc, gate = layer.hc1, layer.hc1.gate(h)
            hin = sops.token_shift_mix(h, layer.shift, state["prev"], fb.seq)[0]
            y = layer.mixer(hin, fb, state, self.kv_caches[i])
            if layer.mlp is not None:
                h = read(layer.hc2)
                hc = layer.hc2
                y, gate = layer.mlp(h)
            if self.capture_layers is not None:
                self.capture_layers.append(self._streams_after(X, y, gate, hc))
        return sops.hyper_mix_rmsnorm(
            X, y, gate, hc.mix if hc is not None else None,
            hc.write if hc is not None else None, self.final_read, self.final_norm,
            self.eps, self.dtype)

    @torch.inference_mode()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = F.linear(hidden, self.lm_head).float()
        if self.logit_scale != 1.0:
            logits.mul_(self.logit_scale)
        return logits

    # -- checkpoint names -> fused engine layout -----------------------------
    def load_named_tensors(self, tensors) -> int:
        """tensors: iterable of (name, tensor) with the design's names
        ('embed', 'l<i>.norm1', 'l<i>.hc1.in', 'l<i>.rg1', 'l<i>.shift',
        'l<i>.mix.q', 'l<i>.mlp.e<k>.gate', 'final.norm', 'head', ...)."""
        W = {k: v for k, v in tensors}
        used = set()

        def get(name):
            used.add(name)
            try:
                return W[name]
            except KeyError:
                raise ValueError(f"checkpoint lacks tensor {name!r}") from None

        def put(param, value):
            value = value.to(device=param.device, dtype=param.dtype)
            if param.shape != value.shape:
                raise ValueError(
                    f"checkpoint tensor of shape {tuple(value.shape)} does not fit "
                    f"{tuple(param.shape)}")
            param.data.copy_(value)

        put(self.embed_tokens.weight, get("embed"))
        put(self.lm_head, get("head"))
        put(self.final_norm, get("final.norm"))
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            put(layer.shift, get(p + "shift").reshape(1, -1))
            for q, hc in ((1, layer.hc1), (2, layer.hc2)):
                if hc is None:
                    continue
                put(hc.norm, get(f"{p}norm{q}"))
                if f"{p}hc{q}.in" in W or self.streams != 1:
                    put(hc.read, get(f"{p}hc{q}.in"))
                    put(hc.write, get(f"{p}hc{q}.out"))
                    put(hc.mix, get(f"{p}hc{q}.mix"))
                else:  # one stream without learned connections: a plain residual sum
                    hc.read.data.fill_(1.0)
                    hc.write.data.fill_(1.0)
                    hc.mix.data.fill_(1.0)
                if hc.gate is not None:
                    put(hc.gate.weight, get(f"{p}rg{q}"))
                    put(hc.gate.bias, get(f"{p}rg{q}.b"))
            m, q = layer.mixer, p + "mix."
            if isinstance(m, DifferentialAttention):
                order = m.query_row_order()
                put(m.in_proj.weight, torch.cat(
                    [get(q + "q")[order], get(q + "k"), get(q + "v")]))
                put(m.in_proj.bias, torch.cat(
                    [get(q + "q.b")[order], get(q + "k.b"), get(q + "v.b")]))
                put(m.lam_q, torch.stack([get(q + "lq1"), get(q + "lq2")]))
                put(m.lam_k, torch.stack([get(q + "lk1"), get(q + "lk2")]))
                m._lam = None
                put(m.o_proj.weight, get(q + "o"))
                put(m.o_proj.bias, get(q + "o.b"))
            else:
                m.set_lowrank(get(q + "w1").shape[0])
                put(m.in_proj.weight,
                    torch.cat([get(q + n) for n in ("r", "k", "v", "g", "a", "w1")]))
                put(m.w2.weight, get(q + "w2"))
                put(m.w0, get(q + "w0"))
                put(m.a_bias, get(q + "a.b"))
                put(m.norm, get(q + "norm"))
                put(m.o_proj.weight, get(q + "o"))
            f, q = layer.mlp, p + "mlp."
            if f is None:
                continue
            rg, rg_b = get(p + "rg2"), get(p + "rg2.b")

            def with_gate_bias(n_rows):
                return torch.cat([torch.zeros(n_rows, dtype=rg_b.dtype), rg_b])

            if isinstance(f, SiluGatedMLP):
                put(f.gate_up.weight, torch.cat([get(q + "gate"), get(q + "up"), rg]))
                put(f.gate_up.bias, with_gate_bias(2 * f.ff))
                put(f.down.weight, get(q + "down"))
            else:
                names = [f"{q}e{e}." for e in range(f.experts)]
                router = [get(q + "router")]
                if f.shared_ff:
                    names.append(q + "shared.")
                    router.append(get(q + "shared.sg").reshape(1, -1))
                put(f.gate_up.weight, torch.cat(
                    [get(n + part) for n in names for part in ("gate", "up")] + [rg]))
                put(f.gate_up.bias, with_gate_bias(f.experts * 2 * f.ff + 2 * f.shared_ff))
                put(f.down.weight, torch.cat([get(n + "down") for n in names], dim=1))
                put(f.router, torch.cat(router))
        missing = set(W) - used
        if missing:
            raise ValueError(f"checkpoint tensors not consumed: {sorted(missing)[:8]}")
        return len(used)
