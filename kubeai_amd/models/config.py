"""Model architecture configs.

Mirrors the fields of HF `config.json` that the engine needs; presets cover
the BASELINE.json configs (Llama-3 8B / 70B, plus tiny variants for tests).
"""
from __future__ import annotations

import dataclasses
import json
import os


@dataclasses.dataclass
class ModelArchConfig:
    architecture: str = "llama"
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    max_position_embeddings: int = 8192
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    tie_word_embeddings: bool = False
    bos_token_id: int = 128000
    eos_token_id: int = 128001
    # MoE (Mixtral-style); n_experts == 0 means dense MLP
    num_local_experts: int = 0
    num_experts_per_tok: int = 2
    # Qwen2-style: q/k/v projections carry a bias
    attention_bias: bool = False
    # HF rope_scaling dict (llama3 / linear), None = unscaled
    rope_scaling: dict | None = None
    # sliding-window attention (Mistral family; Gemma2 uses it on
    # alternate layers): 0 = full causal
    sliding_window: int = 0
    # "all": every layer windowed (Mistral); "even": layers 0,2,4,..
    # windowed (Gemma2 layer_types pattern)
    sliding_window_pattern: str = "all"
    # gemma3: every Nth layer is GLOBAL attention (no window, global
    # rope base); the rest are windowed with rope_local_base_freq.
    # 0 disables the pattern.
    global_layer_interval: int = 0
    rope_local_base_freq: float = 0.0
    # gemma3: per-head RMSNorm on q and k before rope
    qk_norm: bool = False
    # granite-3 scalar multipliers (0 = disabled/default)
    embedding_multiplier: float = 0.0
    residual_multiplier: float = 0.0
    logits_scaling: float = 0.0
    attention_multiplier: float = 0.0
    # gemma2 family knobs
    hidden_act: str = "silu"  # or "gelu_pytorch_tanh" (GeGLU)
    norm_plus_one: bool = False  # RMSNorm multiplies by (1 + w)
    scale_embeddings: bool = False  # x *= sqrt(hidden) after embedding
    post_norms: bool = False  # extra post-attn/pre+post-FFN norms
    attn_logit_softcap: float = 0.0  # s = c*tanh(s/c) on attention logits
    final_logit_softcap: float = 0.0  # same cap on lm_head logits
    query_pre_attn_scalar: float = 0.0  # 0 -> head_dim (scale = x^-0.5)
    # multimodal (LLaVA-style): vision-tower config dict + the token id
    # that marks an image slot in the prompt (expanded to n_patches
    # placeholder positions at admission; models/vision.py)
    vision: dict | None = None
    image_token_id: int = -1
    # hybrid designs (per-layer mixers: recurrences, chunked attention, ...):
    # the list of HybridLayerSpec plus the design's scalar constants.
    # None for the homogeneous attention families above.
    hybrid: "HybridSpec | None" = None

    @property
    def n_kv_heads(self) -> int:
        return self.num_key_value_heads

    @staticmethod
    def from_hf_config(path: str) -> "ModelArchConfig":
        with open(os.path.join(path, "config.json")) as f:
            cfg = json.load(f)
        if cfg.get("architecture") == "Dulotar":
            return dulotar_arch_config(cfg)
        if cfg.get("architecture") == "Nugopel":
            return nugopel_arch_config(cfg)
        if cfg.get("architecture") == "Vekusun":
            return vekusun_arch_config(cfg)
        if cfg.get("architecture") == "Vigonex":
            return vigonex_arch_config(cfg)
        hidden = cfg["hidden_size"]
        n_heads = cfg["num_attention_heads"]
        arch = (cfg.get("architectures") or ["LlamaForCausalLM"])[0]
        gemma2 = arch == "Gemma2ForCausalLM"
        gemma1 = arch == "GemmaForCausalLM"
        gemma3 = arch in ("Gemma3ForCausalLM", "Gemma3ForConditionalGeneration")
        granite = arch == "GraniteForCausalLM"
        vision = None
        image_token_id = -1
        if arch == "Gemma3ForConditionalGeneration":
            # text-only serving of the text tower (the gemma3 SigLIP
            # vision tower is not implemented; LLaVA covers multimodal)
            cfg = {**cfg, **(cfg.get("text_config") or {})}
            hidden = cfg["hidden_size"]
            n_heads = cfg["num_attention_heads"]
        if arch == "LlavaForConditionalGeneration":
            # llava config nests text_config + vision_config
            vision = dict(cfg.get("vision_config") or {})
            vision.setdefault(
                "vision_feature_layer", cfg.get("vision_feature_layer", -2)
            )
            image_token_id = cfg.get("image_token_index", 32000)
            cfg = {**cfg, **(cfg.get("text_config") or {})}
            hidden = cfg["hidden_size"]
            n_heads = cfg["num_attention_heads"]
        eos = cfg.get("eos_token_id", 2)
        if isinstance(eos, list):
            eos = eos[0]
        return ModelArchConfig(
            architecture="mixtral" if "Mixtral" in arch else "llama",
            # Qwen2 always uses qkv bias; Llama-family configs may say so
            attention_bias=bool(
                cfg.get("attention_bias", arch.startswith("Qwen2"))
            ),
            vocab_size=cfg["vocab_size"],
            hidden_size=hidden,
            intermediate_size=cfg["intermediate_size"],
            num_hidden_layers=cfg["num_hidden_layers"],
            num_attention_heads=n_heads,
            num_key_value_heads=cfg.get("num_key_value_heads", n_heads),
            head_dim=cfg.get("head_dim", hidden // n_heads),
            max_position_embeddings=cfg.get("max_position_embeddings", 8192),
            rms_norm_eps=cfg.get("rms_norm_eps", 1e-5),
            rope_theta=cfg.get("rope_theta", 10000.0),
            tie_word_embeddings=cfg.get(
                "tie_word_embeddings", gemma2 or gemma1 or gemma3
            ),
            bos_token_id=cfg.get("bos_token_id", 1),
            eos_token_id=eos,
            num_local_experts=cfg.get("num_local_experts", 0),
            num_experts_per_tok=cfg.get("num_experts_per_tok", 2),
            rope_scaling=cfg.get("rope_scaling"),
            sliding_window=int(cfg.get("sliding_window") or 0),
            sliding_window_pattern="even" if gemma2 else "all",
            hidden_act=(
                "gelu_pytorch_tanh"
                if gemma2 or gemma1 or gemma3
                or "gelu" in str(cfg.get("hidden_act") or "")
                else "silu"
            ),
            norm_plus_one=gemma2 or gemma1 or gemma3,
            scale_embeddings=gemma2 or gemma1 or gemma3,
            post_norms=gemma2 or gemma3,
            global_layer_interval=(
                int(cfg.get("sliding_window_pattern") or 6) if gemma3 else 0
            ),
            rope_local_base_freq=(
                float(cfg.get("rope_local_base_freq") or 10000.0)
                if gemma3 else 0.0
            ),
            qk_norm=gemma3,
            embedding_multiplier=float(
                cfg.get("embedding_multiplier") or 0.0
            ) if granite else 0.0,
            residual_multiplier=float(
                cfg.get("residual_multiplier") or 0.0
            ) if granite else 0.0,
            logits_scaling=float(
                cfg.get("logits_scaling") or 0.0
            ) if granite else 0.0,
            attention_multiplier=float(
                cfg.get("attention_multiplier") or 0.0
            ) if granite else 0.0,
            attn_logit_softcap=float(
                cfg.get("attn_logit_softcapping") or 0.0
            ) if gemma2 else 0.0,
            final_logit_softcap=float(
                cfg.get("final_logit_softcapping") or 0.0
            ) if gemma2 else 0.0,
            query_pre_attn_scalar=float(
                cfg.get("query_pre_attn_scalar") or 0.0
            ) if (gemma2 or gemma3) else 0.0,
            vision=vision,
            image_token_id=image_token_id,
        )


@dataclasses.dataclass
class HybridLayerSpec:
    """One layer of a hybrid design: which mixer, its sizes/constants as the
    checkpoint's config gives them, its feed-forward (None = the layer has
    only the mixer sublayer), and the layer whose tensors it uses."""

    type: str
    mixer: dict
    mlp: dict | None
    weights_of: int  # own index unless the layer shares another's tensors


@dataclasses.dataclass
class HybridSpec:
    layers: list
    norm_eps: float
    embedding_scale: float
    canon_taps: int  # taps of the per-layer input convolution (0 = none)
    # multiplier on every layer's summed sublayer outputs
    residual_mult: float = 1.0
    # logits <- cap * tanh(logits / cap); 0 = none
    logit_softcap: float = 0.0
    # (start, stop, times): layers start..stop-1 run `times` times in a row
    # with the same weights, every pass with cache and state of its own
    loop: tuple = (0, 0, 1)
    # residual streams (hyper-connections); 1 = one stream
    streams: int = 1
    # multiplier on the logits
    logit_scale: float = 1.0


def dulotar_arch_config(cfg: dict) -> ModelArchConfig:
    """Dulotar config.json -> arch config. Every size and constant comes
    from the file; nothing is defaulted to a particular checkpoint."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        layers.append(
            HybridLayerSpec(
                type=L["type"],
                mixer=L["mixer"],
                mlp=L.get("mlp"),
                weights_of=int(L.get("weights_of", i)),
            )
        )
    return ModelArchConfig(
        architecture="dulotar",
        vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]),
        num_hidden_layers=len(layers),
        intermediate_size=0,
        num_attention_heads=0,
        num_key_value_heads=0,
        head_dim=0,
        max_position_embeddings=1 << 30,  # no learned/cached position table
        bos_token_id=-1,
        eos_token_id=-1,  # the design defines no end token
        hybrid=HybridSpec(
            layers=layers,
            norm_eps=float(cfg["norm"]["eps"]),
            embedding_scale=float(cfg["embedding"]["scale"]),
            canon_taps=int((cfg.get("canon") or {}).get("taps", 0)),
        ),
    )


def nugopel_arch_config(cfg: dict) -> ModelArchConfig:
    """Nugopel config.json -> arch config: the list of layers (mixer type,
    the mixer's sizes and constants, the feed-forward) and the norm epsilon,
    all as the file gives them."""
    layers = [
        HybridLayerSpec(type=L["type"], mixer=L["mixer"], mlp=L.get("mlp"), weights_of=i)
        for i, L in enumerate(cfg["layers"])
    ]
    return ModelArchConfig(
        architecture="nugopel",
        vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]),
        num_hidden_layers=len(layers),
        intermediate_size=0,
        num_attention_heads=0,
        num_key_value_heads=0,
        head_dim=0,
        max_position_embeddings=1 << 30,  # positions are computed, not tabulated
        bos_token_id=-1,
        eos_token_id=-1,  # the design defines no end token
        hybrid=HybridSpec(
            layers=layers,
            norm_eps=float(cfg["norm"]["eps"]),
            embedding_scale=1.0,
            canon_taps=0,
        ),
    )


def vekusun_arch_config(cfg: dict) -> ModelArchConfig:
    """Vekusun config.json -> arch config: the list of layers (mixer type, the
    mixer's sizes and constants, the feed-forward), the looped span, the
    residual multiplier, the logit cap and the norm epsilon, all as the file
    gives them."""
    layers = [
        HybridLayerSpec(type=L["type"], mixer=L["mixer"], mlp=L.get("mlp"), weights_of=i)
        for i, L in enumerate(cfg["layers"])
    ]
    loop = cfg.get("loop") or {}
    start, stop = int(loop.get("start", 0)), int(loop.get("stop", 0))
    times = int(loop.get("times", 1))
    if not (0 <= start <= stop <= len(layers)) or times < 1:
        raise ValueError(f"loop {loop!r} does not fit {len(layers)} layers")
    if start == stop:
        start, stop, times = 0, 0, 1
    return ModelArchConfig(
        architecture="vekusun",
        vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]),
        num_hidden_layers=len(layers),
        intermediate_size=0,
        num_attention_heads=0,
        num_key_value_heads=0,
        head_dim=0,
        max_position_embeddings=1 << 30,  # positions are computed, not tabulated
        bos_token_id=-1,
        eos_token_id=-1,  # the design defines no end token
        hybrid=HybridSpec(
            layers=layers,
            norm_eps=float(cfg["norm"]["eps"]),
            embedding_scale=1.0,
            canon_taps=0,
            residual_mult=float(cfg.get("residual_mult", 1.0)),
            logit_softcap=float(cfg.get("logit_softcap") or 0.0),
            loop=(start, stop, times),
        ),
    )


def vigonex_arch_config(cfg: dict) -> ModelArchConfig:
    """Vigonex config.json -> arch config: the list of layers (mixer type, the
    mixer's sizes and constants, the feed-forward), the number of residual
    streams, the embedding and logit scales and the norm epsilon, all as the
    file gives them."""
    layers = [
        HybridLayerSpec(type=L["type"], mixer=L["mixer"], mlp=L.get("mlp"), weights_of=i)
        for i, L in enumerate(cfg["layers"])
    ]
    streams = int(cfg.get("streams", 1))
    if streams < 1:
        raise ValueError("streams must be at least 1")
    return ModelArchConfig(
        architecture="vigonex",
        vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]),
        num_hidden_layers=len(layers),
        intermediate_size=0,
        num_attention_heads=0,
        num_key_value_heads=0,
        head_dim=0,
        max_position_embeddings=1 << 30,  # positions are computed, not tabulated
        bos_token_id=-1,
        eos_token_id=-1,  # the design defines no end token
        hybrid=HybridSpec(
            layers=layers,
            norm_eps=float(cfg["norm"]["eps"]),
            embedding_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
            canon_taps=0,
            streams=streams,
            logit_scale=float(cfg.get("logit_scale", 1.0)),
        ),
    )


# Presets (BASELINE.json configs + test-size models)
PRESETS: dict[str, ModelArchConfig] = {
    "llama-3-8b": ModelArchConfig(
        # Llama-3.1-8B-Instruct shape (the BASELINE model): 128k context
        # via llama3 rope scaling
        max_position_embeddings=131072,
        rope_scaling={"rope_type": "llama3", "factor": 8.0,
                      "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                      "original_max_position_embeddings": 8192},
    ),
    "llama-3-70b": ModelArchConfig(
        hidden_size=8192,
        intermediate_size=28672,
        num_hidden_layers=80,
        num_attention_heads=64,
        num_key_value_heads=8,
        max_position_embeddings=131072,
        rope_scaling={"rope_type": "llama3", "factor": 8.0,
                      "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                      "original_max_position_embeddings": 8192},
    ),
    # tiny: CPU tests / smoke; same head_dim=128 so HIP kernel paths match
    # Qwen2 family (also the DeepSeek-R1-Distill-Qwen arch): qkv bias,
    # tied embeddings on the small models
    "qwen2-tiny": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=128,
        max_position_embeddings=2048,
        bos_token_id=1,
        eos_token_id=2,
        attention_bias=True,
        tie_word_embeddings=True,
        rope_theta=1000000.0,
    ),
    "qwen2-7b": ModelArchConfig(
        vocab_size=152064,
        hidden_size=3584,
        intermediate_size=18944,
        num_hidden_layers=28,
        num_attention_heads=28,
        num_key_value_heads=4,
        head_dim=128,
        max_position_embeddings=32768,
        rms_norm_eps=1e-6,
        rope_theta=1000000.0,
        bos_token_id=151643,
        eos_token_id=151645,
        attention_bias=True,
    ),
    "llama-tiny": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=128,
        max_position_embeddings=2048,
        bos_token_id=1,
        eos_token_id=2,
    ),
    # Gemma-2b (v1) shape: MQA (1 kv head, G=8), GeGLU, (1+w) norms,
    # scaled embeddings, head_dim 256 — no post-norms/softcaps/window
    "gemma-2b": ModelArchConfig(
        vocab_size=256000,
        hidden_size=2048,
        intermediate_size=16384,
        num_hidden_layers=18,
        num_attention_heads=8,
        num_key_value_heads=1,
        head_dim=256,
        max_position_embeddings=8192,
        rope_theta=10000.0,
        rms_norm_eps=1e-6,
        tie_word_embeddings=True,
        bos_token_id=2,
        eos_token_id=1,
        hidden_act="gelu_pytorch_tanh",
        norm_plus_one=True,
        scale_embeddings=True,
    ),
    "gemma-tiny": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=256,
        max_position_embeddings=2048,
        rope_theta=10000.0,
        rms_norm_eps=1e-6,
        tie_word_embeddings=True,
        bos_token_id=2,
        eos_token_id=1,
        hidden_act="gelu_pytorch_tanh",
        norm_plus_one=True,
        scale_embeddings=True,
    ),
    # Phi-4 shape (Phi3ForCausalLM): llama structure with fused
    # qkv_proj / gate_up_proj checkpoint tensors, untied head
    "phi-4": ModelArchConfig(
        vocab_size=100352,
        hidden_size=5120,
        intermediate_size=17920,
        num_hidden_layers=40,
        num_attention_heads=40,
        num_key_value_heads=10,
        head_dim=128,
        max_position_embeddings=16384,
        rope_theta=250000.0,
        rms_norm_eps=1e-5,
        bos_token_id=100257,
        eos_token_id=100257,
    ),
    # Gemma2-2b shape: GeGLU, (1+w) norms, post-norms, logit softcaps,
    # head_dim 256, alternate-layer sliding window
    "gemma2-2b": ModelArchConfig(
        vocab_size=256000,
        hidden_size=2304,
        intermediate_size=9216,
        num_hidden_layers=26,
        num_attention_heads=8,
        num_key_value_heads=4,
        head_dim=256,
        max_position_embeddings=8192,
        rope_theta=10000.0,
        rms_norm_eps=1e-6,
        tie_word_embeddings=True,
        bos_token_id=2,
        eos_token_id=1,
        sliding_window=4096,
        sliding_window_pattern="even",
        hidden_act="gelu_pytorch_tanh",
        norm_plus_one=True,
        scale_embeddings=True,
        post_norms=True,
        attn_logit_softcap=50.0,
        final_logit_softcap=30.0,
        query_pre_attn_scalar=256.0,
    ),
    # tiny gemma2 for CPU tests: every architectural wrinkle, small dims
    "gemma2-tiny": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=256,
        max_position_embeddings=2048,
        rope_theta=10000.0,
        rms_norm_eps=1e-6,
        tie_word_embeddings=True,
        bos_token_id=2,
        eos_token_id=1,
        sliding_window=64,
        sliding_window_pattern="even",
        hidden_act="gelu_pytorch_tanh",
        norm_plus_one=True,
        scale_embeddings=True,
        post_norms=True,
        attn_logit_softcap=50.0,
        final_logit_softcap=30.0,
        query_pre_attn_scalar=256.0,
    ),
    # Granite-3.1-8b dense shape: llama structure + scalar multipliers
    "granite-3-8b": ModelArchConfig(
        vocab_size=49155,
        hidden_size=4096,
        intermediate_size=12800,
        num_hidden_layers=40,
        num_attention_heads=32,
        num_key_value_heads=8,
        head_dim=128,
        max_position_embeddings=131072,
        rope_theta=10000000.0,
        tie_word_embeddings=True,
        bos_token_id=0,
        eos_token_id=0,
        embedding_multiplier=12.0,
        residual_multiplier=0.22,
        logits_scaling=16.0,
        attention_multiplier=0.0078125,
    ),
    "granite-tiny": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=128,
        max_position_embeddings=2048,
        tie_word_embeddings=True,
        bos_token_id=1,
        eos_token_id=2,
        embedding_multiplier=12.0,
        residual_multiplier=0.22,
        logits_scaling=16.0,
        attention_multiplier=0.0078125,
    ),
    # Gemma3-4b text shape: qk-norm, 5 local(1024-window, theta 10k) :
    # 1 global(theta 1M, linear x8) layer pattern, post-norms, GeGLU
    "gemma3-4b": ModelArchConfig(
        vocab_size=262208,
        hidden_size=2560,
        intermediate_size=10240,
        num_hidden_layers=34,
        num_attention_heads=8,
        num_key_value_heads=4,
        head_dim=256,
        max_position_embeddings=131072,
        rope_theta=1000000.0,
        rope_scaling={"rope_type": "linear", "factor": 8.0},
        rope_local_base_freq=10000.0,
        rms_norm_eps=1e-6,
        tie_word_embeddings=True,
        bos_token_id=2,
        eos_token_id=1,
        sliding_window=1024,
        global_layer_interval=6,
        hidden_act="gelu_pytorch_tanh",
        norm_plus_one=True,
        scale_embeddings=True,
        post_norms=True,
        qk_norm=True,
        query_pre_attn_scalar=256.0,
    ),
    "gemma3-tiny": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=3,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=256,
        max_position_embeddings=2048,
        rope_theta=1000000.0,
        rope_local_base_freq=10000.0,
        rms_norm_eps=1e-6,
        tie_word_embeddings=True,
        bos_token_id=2,
        eos_token_id=1,
        sliding_window=32,
        global_layer_interval=3,
        hidden_act="gelu_pytorch_tanh",
        norm_plus_one=True,
        scale_embeddings=True,
        post_norms=True,
        qk_norm=True,
        query_pre_attn_scalar=256.0,
    ),
    # Mistral-7B v0.1/v0.2 shape: llama arch + 4096-token sliding window
    "mistral-7b": ModelArchConfig(
        vocab_size=32000,
        hidden_size=4096,
        intermediate_size=14336,
        num_hidden_layers=32,
        num_attention_heads=32,
        num_key_value_heads=8,
        head_dim=128,
        max_position_embeddings=32768,
        rope_theta=10000.0,
        sliding_window=4096,
        bos_token_id=1,
        eos_token_id=2,
    ),
    # tiny windowed model for CPU tests (window smaller than the
    # prompts the tests use, so masking actually bites)
    "mistral-tiny": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=128,
        max_position_embeddings=2048,
        rope_theta=10000.0,
        sliding_window=64,
        bos_token_id=1,
        eos_token_id=2,
    ),
    # multimodal tiny: llama-tiny text + 2-layer CLIP tower; 16 patches
    # per image (64px / 16px patches). Image slot token = 99 (synthetic
    # tokenizer's char region stops at 97).
    "llava-tiny": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=128,
        max_position_embeddings=2048,
        bos_token_id=1,
        eos_token_id=2,
        image_token_id=99,
        vision={
            "image_size": 64,
            "patch_size": 16,
            "hidden_size": 128,
            "num_hidden_layers": 2,
            "num_attention_heads": 2,
            "intermediate_size": 256,
        },
    ),
    # LLaVA-1.5-7B shape: Vicuna-7B text + CLIP ViT-L/14-336 (576
    # patches/image, features from the penultimate layer)
    "llava-1.5-7b": ModelArchConfig(
        vocab_size=32064,
        hidden_size=4096,
        intermediate_size=11008,
        num_hidden_layers=32,
        num_attention_heads=32,
        num_key_value_heads=32,
        head_dim=128,
        max_position_embeddings=4096,
        rope_theta=10000.0,
        bos_token_id=1,
        eos_token_id=2,
        image_token_id=32000,
        vision={
            "image_size": 336,
            "patch_size": 14,
            "hidden_size": 1024,
            "num_hidden_layers": 24,
            "num_attention_heads": 16,
            "intermediate_size": 4096,
        },
    ),
    # long-context tiny model: exercises chunked prefill + paged decode
    # at tens of thousands of tokens without big weights (the engine
    # sizes KV from free HBM; presets elsewhere are 8k-faithful)
    "llama-tiny-32k": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=128,
        max_position_embeddings=32768,
        bos_token_id=1,
        eos_token_id=2,
    ),
    # small: 1-GPU quick bench model (head_dim=128 to stay on the HIP path)
    "llama-1b": ModelArchConfig(
        vocab_size=128256,
        hidden_size=2048,
        intermediate_size=8192,
        num_hidden_layers=16,
        num_attention_heads=16,
        num_key_value_heads=4,
        head_dim=128,
    ),
    # tiny with 2 KV heads so TP=2 shards cleanly (tests/test_tp.py)
    "llama-tiny-tp": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=4,
        num_key_value_heads=2,
        head_dim=128,
        max_position_embeddings=2048,
        bos_token_id=1,
        eos_token_id=2,
    ),
    # TP-shardable multimodal tiny (2 kv heads so TP=2 splits evenly)
    "llava-tiny-tp": ModelArchConfig(
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=4,
        num_key_value_heads=2,
        head_dim=128,
        max_position_embeddings=2048,
        bos_token_id=1,
        eos_token_id=2,
        image_token_id=99,
        vision={
            "image_size": 64,
            "patch_size": 16,
            "hidden_size": 128,
            "num_hidden_layers": 2,
            "num_attention_heads": 2,
            "intermediate_size": 256,
        },
    ),
    "mixtral-tiny": ModelArchConfig(
        architecture="mixtral",
        vocab_size=2048,
        hidden_size=256,
        intermediate_size=512,
        num_hidden_layers=2,
        num_attention_heads=2,
        num_key_value_heads=1,
        head_dim=128,
        max_position_embeddings=2048,
        bos_token_id=1,
        eos_token_id=2,
        num_local_experts=4,
        num_experts_per_tok=2,
    ),
    "mixtral-8x7b": ModelArchConfig(
        architecture="mixtral",
        vocab_size=32000,
        hidden_size=4096,
        intermediate_size=14336,
        num_hidden_layers=32,
        num_attention_heads=32,
        num_key_value_heads=8,
        head_dim=128,
        rope_theta=1000000.0,
        bos_token_id=1,
        eos_token_id=2,
        num_local_experts=8,
        num_experts_per_tok=2,
    ),
}


def nugopel_preset(width: int, layers: int, vocab: int = 32000, head_dim: int = 128,
                   window: int = 1024, kv_rank: int = 128, experts: int = 8,
                   top: int = 2) -> ModelArchConfig:
    """A Nugopel stack of the given size with random-init weights: the layer
    pattern (window attention, latent attention with its own latent, window
    attention, latent attention reading the earlier latent) repeats to the
    requested depth; every layer has a routed feed-forward. Attention has
    width/head_dim query heads over a quarter as many key/value heads. The
    experts are sized so that the feed-forward work per token (chosen
    experts + shared) is that of a dense 3.5 x width gated feed-forward."""
    heads = max(1, width // head_dim)
    # a gated dense layer moves 3 * width * 3.5 width weights per token; the
    # squared-ReLU experts have two matrices: (top + 1) * ff * 2 = 10.5 width
    ff = max(16, int(10.5 * width / (2 * (top + 1))) // 16 * 16)
    mlp = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "top": top}, "shared": {"ff": ff}}
    attn = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": head_dim,
            "vdim": head_dim, "scale": head_dim ** -0.5, "mask": {"size": window},
            "rot": {"base": 500000.0, "dims": head_dim // 2,
                    "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0,
                                "original": 8192}}}
    lat = {"heads": heads, "dim": head_dim, "vdim": head_dim, "kv_rank": kv_rank,
           "scale": head_dim ** -0.5}
    out = []
    for i in range(layers):
        if i % 2 == 0:
            out.append({"type": "attention", "mixer": attn, "mlp": mlp})
        elif i % 4 == 1:
            out.append({"type": "latent_attention", "mixer": dict(lat), "mlp": mlp})
        else:
            out.append({"type": "latent_attention",
                        "mixer": dict(lat, kv_from=i - 2), "mlp": mlp})
    return nugopel_arch_config({
        "architecture": "Nugopel", "vocab": vocab, "width": width,
        "norm": {"eps": 1e-5}, "layers": out,
    })


def vekusun_preset(width: int, layers: int, vocab: int = 32000, head_dim: int = 128,
                   kv_rank: int = 128, rot_dim: int = 64, experts: int = 8,
                   top: int = 2, loop_times: int = 1,
                   ff_scale: float = 1.0) -> ModelArchConfig:
    """A Vekusun stack of the given size with random-init weights: the layer
    pattern (latent attention with a query latent and sinks + dense
    feed-forward, latent attention with a rotated key part and head gates +
    routed experts, gated delta rule + dense feed-forward, latent attention +
    routed experts) repeats to the requested depth. The feed-forward work per
    token is that of a dense 3.5 x width gated layer in either kind (times
    ff_scale, for matching another model's size); with loop_times > 1 the
    first two layers run that many times."""
    heads = max(1, width // head_dim)
    ff_dense = max(16, int(5.25 * ff_scale * width) // 16 * 16)     # two matrices
    ff_exp = max(16, int(3.5 * ff_scale * width / top) // 16 * 16)  # three, top experts
    dense = {"kind": "dense", "ff": ff_dense}
    moe = {"kind": "moe", "expert": {"ff": ff_exp},
           "router": {"experts": experts, "top": top}}
    lat1 = {"heads": heads, "dim": head_dim, "vdim": head_dim, "kv_rank": kv_rank,
            "q_rank": max(64, width // 2), "scale": head_dim ** -0.5}
    lat2 = {"heads": heads, "dim": head_dim, "rot_dim": rot_dim, "vdim": head_dim,
            "kv_rank": kv_rank, "scale": (head_dim + rot_dim) ** -0.5,
            "rot": {"base": 10000.0, "dims": rot_dim,
                    "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0,
                                "slow": 1.0}}}
    delta = {"heads": heads, "kv_heads": max(1, heads // 2), "dim": head_dim,
             "vdim": head_dim, "conv": 4}
    pattern = [
        {"type": "latent_attention", "mixer": lat1, "mlp": dense},
        {"type": "latent_attention_2", "mixer": lat2, "mlp": moe},
        {"type": "delta", "mixer": delta, "mlp": dense},
        {"type": "latent_attention", "mixer": lat1, "mlp": moe},
    ]
    cfg = {
        "architecture": "Vekusun", "vocab": vocab, "width": width,
        "norm": {"eps": 1e-5}, "residual_mult": 1.0, "logit_softcap": 30.0,
        "layers": [dict(pattern[i % 4]) for i in range(layers)],
    }
    if loop_times > 1:
        cfg["loop"] = {"start": 0, "stop": min(2, layers), "times": loop_times}
    return vekusun_arch_config(cfg)


def vigonex_preset(width: int, layers: int, vocab: int = 32000, head_dim: int = 128,
                   experts: int = 8, top: int = 2, streams: int = 2,
                   ff_scale: float = 1.0) -> ModelArchConfig:
    """A Vigonex stack of the given size with random-init weights: the layer
    pattern (differential attention + dense feed-forward, differential
    attention + routed experts with a shared one, generalized delta rule +
    routed experts, differential attention + routed experts) repeats to the
    requested depth. Differential heads have head_dim / 2 key dims per map
    and head_dim value dims, 4:1 grouped keys; delta heads are 64 wide. The
    feed-forward work per token is that of a dense 3.5 x width gated layer
    in either kind (times ff_scale, for matching another model's size)."""
    heads = max(1, width // head_dim)
    kv = max(1, heads // 4)
    dim = max(8, head_dim // 2)
    ff_dense = max(16, int(3.5 * ff_scale * width) // 16 * 16)
    ff_exp = max(16, int(3.5 * ff_scale * width / (top + 1)) // 16 * 16)
    dense = {"kind": "dense", "ff": ff_dense}
    moe = {"kind": "moe", "expert": {"ff": ff_exp, "limit": 7.0},
           "router": {"experts": experts, "top": top, "scale": 1.0},
           "shared": {"ff": ff_exp, "limit": 7.0}}
    att = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": head_dim, "diff": 0.2,
           "scale": dim ** -0.5, "softcap": 30.0, "q_temp": {"coef": 0.1, "every": 1024}}
    ddim = min(64, head_dim)
    delta = {"heads": max(1, width // ddim), "dim": ddim, "lowrank": max(16, width // 32)}
    pattern = [
        {"type": "attention", "mixer": att, "mlp": dense},
        {"type": "attention", "mixer": att, "mlp": moe},
        {"type": "general_delta", "mixer": delta, "mlp": moe},
        {"type": "attention", "mixer": att, "mlp": moe},
    ]
    return vigonex_arch_config({
        "architecture": "Vigonex", "vocab": vocab, "width": width,
        "norm": {"eps": 1e-6}, "streams": streams, "embedding": {"scale": 1.0},
        "logit_scale": 1.0, "layers": [dict(pattern[i % 4]) for i in range(layers)],
    })


def dulotar_preset(width: int, layers: int, vocab: int = 32000, head_dim: int = 128,
                   chunk: int = 1024, ff_mult: int = 4) -> ModelArchConfig:
    """A Dulotar stack of the given size with random-init weights: the
    pattern (wkv, mingru, parallel + feed-forward) repeated; sizes follow
    common practice (head_dim-wide heads, 4:1 grouped keys, ff = 4 x width)."""
    heads = max(1, width // head_dim)
    kv = max(1, heads // 4)
    lin_dim = min(head_dim, 128)
    pattern = [
        {"type": "wkv", "mlp": None,
         "mixer": {"heads": max(1, width // 64), "dim": 64, "lowrank": max(16, width // 32)}},
        {"type": "mingru", "mlp": None, "mixer": {"width": width}},
        {"type": "parallel", "mlp": {"kind": "dense", "ff": ff_mult * width},
         "mixer": {
             "left": {"heads": heads, "kv_heads": kv, "dim": head_dim, "vdim": head_dim,
                      "conv": 4, "mask": {"size": chunk},
                      "rot": {"base": 10000.0, "dims": head_dim // 2},
                      "scale": head_dim ** -0.5, "softcap": 50.0},
             "left_scale": 1.0,
             "right": {"heads": heads, "dim": lin_dim, "vdim": head_dim,
                       "decay": [1.0 - 2.0 ** (-5 - 3 * i / max(1, heads - 1))
                                 for i in range(heads)]},
             "right_scale": 1.0}},
    ]
    return dulotar_arch_config({
        "architecture": "Dulotar", "vocab": vocab, "width": width,
        "canon": {"taps": 4}, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
        "layers": [dict(pattern[i % 3]) for i in range(layers)],
    })


PRESETS.update({
    "nugopel-tiny": nugopel_preset(128, 4, vocab=512, head_dim=32, window=48,
                                   kv_rank=64, experts=4, top=2),
    "nugopel-1k": nugopel_preset(1024, 12),
    "nugopel-2k": nugopel_preset(2048, 12),
    "nugopel-4k": nugopel_preset(4096, 6),
    "vekusun-tiny": vekusun_preset(128, 4, vocab=512, head_dim=32, kv_rank=48,
                                   rot_dim=16, experts=4, top=2, loop_times=2),
    "vekusun-1k": vekusun_preset(1024, 12),
    "vekusun-2k": vekusun_preset(2048, 12),
    "vekusun-4k": vekusun_preset(4096, 6),
    "vigonex-tiny": vigonex_preset(128, 4, vocab=512, head_dim=32, experts=4, top=2),
    "vigonex-1k": vigonex_preset(1024, 12),
    "vigonex-2k": vigonex_preset(2048, 12),
    "vigonex-4k": vigonex_preset(4096, 6),
    "dulotar-tiny": dulotar_preset(128, 3, vocab=512, head_dim=32, chunk=64),
    "dulotar-1k": dulotar_preset(1024, 12),
    "dulotar-2k": dulotar_preset(2048, 12),
    "dulotar-4k": dulotar_preset(4096, 6),
})

