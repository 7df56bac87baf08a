"""Vekusun: a decoder whose config lists its layers. A layer has ONE RMS
norm whose output feeds both of its sublayers, and adds their sum:

    h = norm(x);  x <- x + m * (ls1 * mixer(h) + ls2 * ff(h))

with per-channel layer scales ls1, ls2 and one residual multiplier m for the
whole model. The mixer is latent attention with a query latent and a learned
sink per head, latent attention with a rotated key part shared by the heads
and a sigmoid gate per head, or the gated delta rule (kubeai_amd.models.mixers);
the feed-forward is a dense GELU layer or a mixture of gated experts routed
by biased softmax scores. A span of layers may run several times in a row
with the same weights: every pass has caches and state of its own, gets a
learned vector added to the stream before its first layer, and every pass
after the first gets the embedding output added as well. The logits pass a
tanh cap.

Same execution model as the other layer-list decoders: one token-packed
forward per engine step, GEMMs through the BLAS library in the serving dtype,
everything else in the gfx950 kernels of kubeai_amd.ops.seq. The residual
stream is fp32; a layer's residual update, the additions before a pass and
the next layer's norm are one kernel.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from kubeai_amd.engine.batch import ForwardBatch
from kubeai_amd.ops import seq as sops
from .config import HybridLayerSpec, ModelArchConfig
from .mixers import GatedDeltaMixer, GeluMLP, LatentAttention, RoutedGatedMoE, _f32


def build_mixer(spec: HybridLayerSpec, width: int, eps: float) -> nn.Module:
    m = spec.mixer
    if spec.type == "latent_attention":
        return LatentAttention(
            width, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
            kv_rank=int(m["kv_rank"]), scale=m["scale"], eps=eps,
            q_rank=int(m["q_rank"]), sink=True, gate=None,
        )
    if spec.type == "latent_attention_2":
        rot = m.get("rot") or {}
        rot_dim = int(m.get("rot_dim", 0))
        if rot_dim and int(rot.get("dims", rot_dim)) != rot_dim:
            raise ValueError("the rotated key part is rotated as a whole")
        return LatentAttention(
            width, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
            kv_rank=int(m["kv_rank"]), scale=m["scale"], eps=eps,
            rot_dim=rot_dim, rot_base=float(rot.get("base", 10000.0)),
            rot_scaling=rot.get("scaling"), gate="head",
        )
    if spec.type == "delta":
        return GatedDeltaMixer(
            width, heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
            dim=int(m["dim"]), vdim=int(m["vdim"]), conv_taps=int(m["conv"]), eps=eps,
        )
    raise ValueError(f"unknown mixer type {spec.type!r}")


def build_mlp(mlp: dict | None, width: int):
    if mlp is None:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        return GeluMLP(width, int(mlp["ff"]))
    if kind == "moe":
        return RoutedGatedMoE(
            width, experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
            ff=int(mlp["expert"]["ff"]), correction=True,
        )
    raise ValueError(f"unknown feed-forward kind {kind!r}")


class VekusunLayer(nn.Module):
    def __init__(self, spec: HybridLayerSpec, width: int, eps: float):
        super().__init__()
        self.mixer = build_mixer(spec, width, eps)
        self.mlp = build_mlp(spec.mlp, width)
        self.norm1 = _f32(width)
        nn.init.ones_(self.norm1)
        self.ls1 = _f32(width)
        nn.init.ones_(self.ls1)
        self.ls2 = None
        if self.mlp is not None:
            self.ls2 = _f32(width)
            nn.init.ones_(self.ls2)


class VekusunForCausalLM(nn.Module):
    #: the delta-rule layers carry state: the engine gives every live
    #: sequence a state slot and builds fb.seq
    has_seq_state = True

    def __init__(self, cfg: ModelArchConfig, device=None, dtype=torch.bfloat16):
        super().__init__()
        assert cfg.hybrid is not None
        self.cfg = cfg
        self.dtype = dtype
        hs = cfg.hybrid
        W = cfg.hidden_size
        self.eps = hs.norm_eps
        self.mult = float(hs.residual_mult)
        self.cap = float(hs.logit_softcap or 0.0)
        start, stop, times = hs.loop
        prev_dtype = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            with torch.device(device if device is not None else "cpu"):
                self.embed_tokens = nn.Embedding(cfg.vocab_size, W)
                self.layers = nn.ModuleList(
                    [VekusunLayer(spec, W, hs.norm_eps) for spec in hs.layers]
                )
                self.loop_step = _f32(times, W) if stop > start else None
                self.final_norm = _f32(W)
                nn.init.ones_(self.final_norm)
                self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W),
                                            requires_grad=False)
                nn.init.normal_(self.lm_head, std=W ** -0.5)
        finally:
            torch.set_default_dtype(prev_dtype)
        # layer runs in execution order: (layer index, pass number or None);
        # the pass number is set on the first layer of every pass
        self.schedule = [(i, None) for i in range(start)]
        for t in range(times if stop > start else 0):
            self.schedule += [(i, t if i == start else None) for i in range(start, stop)]
        self.schedule += [(i, None) for i in range(stop, len(hs.layers))]
        self.capture_layers = None  # set to a list to record per-run residuals

    # -- what the runner allocates per layer run -------------------------
    def kv_cache_specs(self):
        return [self.layers[i].mixer.kv_spec() for i, _ in self.schedule]

    def state_specs(self):
        return [self.layers[i].mixer.state_spec() for i, _ in self.schedule]

    def bind_kv_caches(self, kv_caches):
        self.kv_caches = kv_caches

    def bind_states(self, states):
        self.states = states

    # --------------------------------------------------------------------
    @torch.inference_mode()
    def forward(self, fb: ForwardBatch) -> torch.Tensor:
        residual = self.embed_tokens(fb.input_ids.long()).float()
        # later passes add the embedding output again
        emb = residual.clone() if any(t for _, t in self.schedule) else None
        a = b = ls1 = ls2 = None
        for r, (i, t) in enumerate(self.schedule):
            layer = self.layers[i]
            h = sops.scaled_add_rmsnorm(
                residual, a, ls1, b, ls2, self.mult,
                emb if t else None, self.loop_step[t] if t is not None else None,
                layer.norm1, self.eps, self.dtype)
            a = layer.mixer(h, fb, self.states[r], self.kv_caches[r])
            b = layer.mlp(h) if layer.mlp is not None else None
            ls1, ls2 = layer.ls1, layer.ls2
            if self.capture_layers is not None:
                x = a.float() * ls1
                if b is not None:
                    x = x + b.float() * ls2
                self.capture_layers.append(residual + self.mult * x)
        return sops.scaled_add_rmsnorm(residual, a, ls1, b, ls2, self.mult, None, None,
                                       self.final_norm, self.eps, self.dtype)

    @torch.inference_mode()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = F.linear(hidden, self.lm_head).float()
        if self.cap > 0:
            sops.tanh_cap(logits, self.cap)
        return logits

    # -- checkpoint names -> fused engine layout -----------------------------
    def load_named_tensors(self, tensors) -> int:
        """tensors: iterable of (name, tensor) with the design's names
        ('embed', 'loop.step', 'l<i>.norm1', 'l<i>.ls1', 'l<i>.mix.dkv',
        'l<i>.mlp.e<k>.gate', 'final.norm', 'head', ...)."""
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
        if self.loop_step is not None:
            put(self.loop_step, get("loop.step"))
        else:
            used.add("loop.step")  # no layer is looped: the vector is never added
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            put(layer.norm1, get(p + "norm1"))
            put(layer.ls1, get(p + "ls1"))
            m, q = layer.mixer, p + "mix."
            if isinstance(m, LatentAttention):
                H, D, Dv, R = m.heads, m.dim, m.vdim, m.rank
                if m.q_rank:
                    parts = [get(q + "dq")]
                    put(m.q_norm, get(q + "dq.norm"))
                    put(m.q_up.weight, get(q + "uq"))
                else:
                    parts = [get(q + "q")]
                if m.gate is not None:
                    parts.append(get(q + "g"))
                parts.append(get(q + "dkv"))
                put(m.in_proj.weight, torch.cat(parts))
                put(m.latent_norm, get(q + "dkv.norm"))
                put(m.uk_r, get(q + "uk").reshape(H, D, R).transpose(1, 2))
                put(m.uv, get(q + "uv").reshape(H, Dv, R))
                if m.sink_scores is not None:
                    put(m.sink_scores, get(q + "sink"))
                put(m.o_proj.weight, get(q + "o"))
            else:
                put(m.in_proj.weight,
                    torch.cat([get(q + n) for n in ("q", "k", "v", "g", "b", "a")]))
                put(m.conv.weight,
                    torch.cat([get(q + n + ".conv") for n in ("q", "k", "v")]))
                put(m.a_log, get(q + "A_log"))
                put(m.dt_bias, get(q + "dt_bias"))
                put(m.norm, get(q + "norm").repeat(m.heads))
                put(m.o_proj.weight, get(q + "o"))
            f, q = layer.mlp, p + "mlp."
            if f is None:
                used.add(p + "ls2")  # nothing to scale
                continue
            put(layer.ls2, get(p + "ls2"))
            if isinstance(f, GeluMLP):
                put(f.up.weight, get(q + "up"))
                put(f.down.weight, get(q + "down"))
            else:
                put(f.gate_up.weight, torch.cat(
                    [get(f"{q}e{e}.{n}") for e in range(f.experts) for n in ("gate", "up")]))
                put(f.down.weight,
                    torch.cat([get(f"{q}e{e}.down") for e in range(f.experts)], dim=1))
                put(f.router, get(q + "router"))
                put(f.correction, get(q + "correction"))
        missing = set(W) - used
        if missing:
            raise ValueError(f"checkpoint tensors not consumed: {sorted(missing)[:8]}")
        return len(used)
