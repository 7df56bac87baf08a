"""Prefill and decode throughput of a layer-list design (Dulotar, Nugopel,
Vekusun, Vigonex) beside the closest existing stack of equal width, depth and
(about) parameter count, random weights, one GPU: a dense Llama for Dulotar,
a Mixtral-style routed Llama (same number of experts and choices) for
Nugopel, Nugopel itself (latent attention, routed experts) for Vekusun, and
Vekusun (full causal attention, a delta rule, dense and routed gated
feed-forwards, sequence state) for Vigonex; the feed-forward sizes of the
last two are scaled so that the parameter counts agree.

    python bench.py --compare-hybrid [--compare-design dulotar|nugopel|vekusun|vigonex]
                    [--compare-sizes 1k,2k,4k]

Prefill: one sequence's whole prompt as a single fixed step (both families
go through LLMEngine.step_fixed, i.e. the packed forward without sampling).
Decode: B sequences admitted through the scheduler, then timed pure-decode
engine steps (captured graphs, greedy sampling). One JSON line per
measurement on stdout.
"""
from __future__ import annotations

import json
import sys
import time

import torch

from kubeai_amd.models.config import PRESETS, ModelArchConfig

SIZES = {"1k": (1024, 12), "2k": (2048, 12), "4k": (4096, 6)}


def _log(msg: str) -> None:
    print(f"[compare t={time.monotonic():.1f}] {msg}", file=sys.stderr, flush=True)


def _params(model) -> int:
    seen, n = set(), 0
    for p in model.parameters():
        if id(p) not in seen:
            seen.add(id(p))
            n += p.numel()
    return n


def _llama_like(width: int, layers: int, vocab: int, target_params: int,
                experts: int = 0, top: int = 2) -> ModelArchConfig:
    """experts > 0: every feed-forward is a routed mixture of that many gated
    experts (the Mixtral layout), sized to the same parameter count."""
    heads = width // 128
    kv = max(1, heads // 4)
    attn = width * (heads + 2 * kv) * 128 + heads * 128 * width
    fixed = 2 * vocab * width + layers * attn
    per_inter = 3 * width * layers * max(1, experts)
    inter = max(256, int((target_params - fixed) / per_inter) // 256 * 256)
    return ModelArchConfig(
        architecture="mixtral" if experts else "llama", vocab_size=vocab,
        hidden_size=width, intermediate_size=inter, num_hidden_layers=layers,
        num_attention_heads=heads, num_key_value_heads=kv, head_dim=128,
        max_position_embeddings=16384, rope_theta=10000.0, eos_token_id=2,
        bos_token_id=1, num_local_experts=experts, num_experts_per_tok=top,
    )


def _meta_params(arch: ModelArchConfig) -> int:
    """Parameter count of an architecture without allocating it."""
    from kubeai_amd.models.registry import model_class

    return _params(model_class(arch.architecture)(arch, device="meta"))


def _sized_like(preset, width: int, layers: int, target_params: int) -> ModelArchConfig:
    """preset(width, layers, ff_scale=...) with its feed-forward sizes scaled
    to the target parameter count (the count is linear in the scale)."""
    p1 = _meta_params(preset(width, layers, ff_scale=1.0))
    p2 = _meta_params(preset(width, layers, ff_scale=2.0))
    scale = 1.0 + (target_params - p1) / max(p2 - p1, 1)
    return preset(width, layers, ff_scale=max(scale, 0.1))


def _vekusun_sized_like(width: int, layers: int, target_params: int) -> ModelArchConfig:
    from kubeai_amd.models.config import vekusun_preset

    return _sized_like(vekusun_preset, width, layers, target_params)


def _engine(name: str, device: str, blocks: int, seqs: int, max_len: int):
    from kubeai_amd.engine import EngineConfig, LLMEngine

    return LLMEngine(EngineConfig(
        model=name, device=device, dtype="bfloat16", num_gpu_blocks=blocks,
        max_num_seqs=seqs, max_model_len=max_len, max_num_batched_tokens=max_len,
        enable_prefix_caching=False, enable_graphs=True))


def _sync(device):
    if device.startswith("cuda"):
        torch.cuda.synchronize()


def _prefill(eng, device, vocab, n_tokens, reps=4):
    g = torch.Generator().manual_seed(n_tokens)
    best = None
    for r in range(reps + 1):
        toks = torch.randint(10, vocab - 10, (n_tokens,), generator=g).tolist()
        _sync(device)
        t0 = time.perf_counter()
        eng.step_fixed([("p%d" % r, toks, [n_tokens - 1])], ["p%d" % r])
        _sync(device)
        dt = time.perf_counter() - t0
        if r > 0:  # the first run warms allocator and GEMM algorithm selection
            best = dt if best is None else min(best, dt)
    return n_tokens / best


def _decode(eng, device, vocab, batch, context, steps=48):
    from kubeai_amd.engine import SamplingParams

    g = torch.Generator().manual_seed(batch)
    for i in range(batch):
        toks = torch.randint(10, vocab - 10, (context,), generator=g).tolist()
        eng.add_request(toks, SamplingParams(max_tokens=steps + 24, ignore_eos=True),
                        request_id="d%d" % i)
    guard = 0
    while (eng.scheduler.num_waiting or any(r.in_prefill for r in eng.scheduler.running)):
        eng.step()
        guard += 1
        assert guard < 10000
    for _ in range(8):
        eng.step()  # graph capture + warm replays
    _sync(device)
    t0 = time.perf_counter()
    n = 0
    for _ in range(steps):
        n += len(eng.step())
    _sync(device)
    dt = time.perf_counter() - t0
    for i in range(batch):
        eng.abort_request("d%d" % i)
    eng.step()
    return n / dt, dt / steps * 1e3


def main(args) -> None:
    device = "cuda" if torch.cuda.is_available() else "cpu"
    sizes = [s for s in (args.compare_sizes or "1k,2k,4k").split(",") if s]
    prefill_lens = [2048, 8192] if device == "cuda" else [64]
    batches = [(64, 1536), (8, 3584)] if device == "cuda" else [(2, 32)]
    design = getattr(args, "compare_design", None) or "dulotar"
    if design not in ("dulotar", "nugopel", "vekusun", "vigonex"):
        raise SystemExit(f"unknown design {design!r}")
    for key in sizes:
        width, layers = SIZES[key]
        name = f"{design}-{key}" if device == "cuda" else f"{design}-tiny"
        if design == "vekusun" and device == "cuda":
            name = f"vekusun-like-nugopel-{key}"
            PRESETS[name] = _vekusun_sized_like(
                width, layers, _meta_params(PRESETS[f"nugopel-{key}"]))
        if design == "vigonex" and device == "cuda":
            from kubeai_amd.models.config import vigonex_preset

            name = f"vigonex-like-vekusun-{key}"
            PRESETS[name] = _sized_like(vigonex_preset, width, layers,
                                        _meta_params(PRESETS[f"vekusun-{key}"]))
        arch = PRESETS[name]
        max_len = 8192 + 256
        blocks = (max(b * (c + 128) for b, c in batches) + max_len) // 16 + 64
        _log(f"{design} {key}: building engine ({name})")
        eng = _engine(name, device, blocks, 64, max_len)
        n_params = _params(eng.runner.model)
        ref_name = f"llama-like-{key}"
        ref_fam = "llama"
        moe = arch.hybrid.layers[0].mlp if design == "nugopel" else None
        if design == "vekusun":
            ref_fam = "nugopel"
            ref_name = f"nugopel-{key}" if device == "cuda" else "nugopel-tiny"
        elif design == "vigonex":
            ref_fam = "vekusun"
            ref_name = f"vekusun-{key}" if device == "cuda" else "vekusun-tiny"
        elif moe:
            ref_fam = "mixtral"
            PRESETS[ref_name] = _llama_like(
                arch.hidden_size, arch.num_hidden_layers, arch.vocab_size, n_params,
                experts=int(moe["router"]["experts"]), top=int(moe["router"]["top"]))
        else:
            PRESETS[ref_name] = _llama_like(
                arch.hidden_size, arch.num_hidden_layers, arch.vocab_size, n_params)
        for fam, model_name in ((design, name), (ref_fam, ref_name)):
            if fam == ref_fam:
                del eng
                if device == "cuda":
                    torch.cuda.empty_cache()
                eng = _engine(model_name, device, blocks, 64, max_len)
            params = _params(eng.runner.model)
            for n in prefill_lens:
                _log(f"{fam} {key}: prefill {n}")
                tps = _prefill(eng, device, arch.vocab_size, n)
                print(json.dumps({"bench": "prefill", "family": fam, "size": key,
                                  "params_m": round(params / 1e6, 1), "tokens": n,
                                  "tokens_per_s": round(tps, 1)}), flush=True)
            for b, c in batches:
                _log(f"{fam} {key}: decode batch {b} context {c}")
                tps, ms = _decode(eng, device, arch.vocab_size, b, c)
                print(json.dumps({"bench": "decode", "family": fam, "size": key,
                                  "params_m": round(params / 1e6, 1), "batch": b,
                                  "context": c, "tokens_per_s": round(tps, 1),
                                  "ms_per_step": round(ms, 3)}), flush=True)
        del eng
        if device == "cuda":
            torch.cuda.empty_cache()
