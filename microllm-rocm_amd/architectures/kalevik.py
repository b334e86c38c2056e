"""The Kalevik decoder as a ``ModelSpec``.

Token embedding times a factor; layers with an RMS norm before and after each sublayer (the ``sandwich_norm``
arrangement with a factor of one); per layer one of two mixers: a causal attention through cached latents (queries
straight from the input, a rotated key part shared by all heads, neighbouring channels turned together, no gate), or a
parallel mixer of a softmax attention inside chunks of positions (grouped key/value heads, a norm of queries and keys,
a partial split-half rotation with stretched positions, one added to the softmax's denominator, a gate a head) beside a
retention (linear attention with one fixed decay a head, its result of unit root mean square a head, a SiLU gate); a
dense gated feed-forward, a mixture of experts (softmax scores, groups of experts of which only the best can be chosen,
experts of one inner weight with the exact gelu, a gated shared expert) or none; a range of layers that may run several
times in a row, the embedding's output joining the stream again before every pass but the first; a final norm and an
untied head.

Tensor names: ``embed``, ``head``, ``final.norm``; per layer ``l<i>.norm1``, ``l<i>.norm1b`` (after the mixer),
``l<i>.norm2``, ``l<i>.norm2b`` (after the feed-forward), ``l<i>.mix.*`` (the parallel mixer's members under ``.left``
and ``.right``), ``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.{router,e<n>.up,e<n>.down,shared.up,shared.down,shared.sg}``.
"""
from __future__ import annotations

from ..config.kalevik import (ChunkAttentionConfig, DenseMlpConfig, KalevikConfig, LatentAttentionConfig, MoeMlpConfig, ParallelConfig,
                              RetentionConfig)
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..weights.random_init import InitRule

MAX_POSITIONS = 1 << 20     # no part has a longest position; block tables and requests need a bound
SINK_SCORE = 0.0            # the score of the softmax's further term without key or value: exp(0) = 1 in the denominator


def _latent_spec(width: int, prefix: str, mixer: LatentAttentionConfig, eps: float) -> PartSpec:
    names = {role: f"{prefix}.{role}" for role in ("q", "dkv", "uk", "uv", "o")}
    names["dkv_norm"] = f"{prefix}.dkv.norm"
    return PartSpec("latent_attention", {
        "hidden_size": width, "heads": mixer.heads, "dim": mixer.dim, "rot_dim": mixer.rot_dim, "vdim": mixer.vdim,
        "q_rank": None, "kv_rank": mixer.kv_rank, "scale": mixer.scale, "window": None, "eps": eps,
        "owns_kv": True, "output_gate": False,
        "position": PartSpec("rope_neighbours", {"theta": mixer.rot_base, "head_dim": mixer.rot_dim, "rotary_dim": mixer.rot_dims})}, names)


def _chunk_attention_spec(width: int, prefix: str, mixer: ChunkAttentionConfig, eps: float) -> PartSpec:
    names = {role: f"{prefix}.{role}" for role in ("q", "k", "v", "g", "o")}
    names.update({"q_norm": f"{prefix}.q.norm", "k_norm": f"{prefix}.k.norm"})
    return PartSpec("bucket_bias_attention", {
        "hidden_size": width, "heads": mixer.heads, "kv_heads": mixer.kv_heads, "key_dim": mixer.dim, "value_dim": mixer.vdim,
        "scale": mixer.scale, "qk_norm": True, "qk_norm_weight": True, "eps": eps, "sink": False, "sink_value": SINK_SCORE,
        "chunk": mixer.chunk, "head_gate": True,
        "position": PartSpec("rope_split_half", {"theta": mixer.rot_base, "head_dim": mixer.dim, "rotary_dim": mixer.rot_dims,
                                                 "scaling_factor": mixer.rot_factor})}, names)


def _retention_spec(width: int, prefix: str, mixer: RetentionConfig, eps: float) -> PartSpec:
    names = {role: f"{prefix}.{role}" for role in ("q", "k", "v", "g", "o")}
    # the keys' factor dim^(-1/2) is applied to the read-out, which is linear in the keys
    return PartSpec("gated_linear_attention", {
        "hidden_size": width, "heads": mixer.heads, "key_dim": mixer.dim, "value_dim": mixer.vdim, "fixed_decay": list(mixer.decay),
        "norm_weight": False, "eps": eps, "query_scale": mixer.dim ** -0.5}, names)


def _mlp_spec(width: int, prefix: str, mlp) -> PartSpec:
    if isinstance(mlp, DenseMlpConfig):
        return PartSpec("swiglu", {"hidden_size": width, "intermediate_size": mlp.ff},
                        {"gate_proj.weight": f"{prefix}.gate", "up_proj.weight": f"{prefix}.up", "down_proj.weight": f"{prefix}.down"})
    assert isinstance(mlp, MoeMlpConfig)
    names = {"router": f"{prefix}.router"}
    for expert in range(mlp.experts):
        for role in ("up", "down"):
            names[f"expert{expert}.{role}"] = f"{prefix}.e{expert}.{role}"
    if mlp.shared_ff is not None:
        names.update({"shared.up": f"{prefix}.shared.up", "shared.down": f"{prefix}.shared.down", "shared.scale": f"{prefix}.shared.sg"})
    return PartSpec("routed_experts", {
        "hidden_size": width, "experts": mlp.experts, "top": mlp.top, "expert_size": mlp.expert_ff, "shared_size": mlp.shared_ff,
        "score": "softmax", "renormalize": False, "weight_on": "output", "expert_form": "plain", "activation": "gelu_erf",
        "groups": mlp.groups if mlp.groups > 1 else 0, "keep_groups": mlp.keep_groups if mlp.groups > 1 else 0,
        "shared_scale": "sigmoid" if mlp.shared_ff is not None else None}, names)


def build_spec(config: KalevikConfig) -> ModelSpec:
    width, eps = config.width, config.norm_eps
    norm = {"size": width, "eps": eps}
    layers = []
    for index, layer in enumerate(config.layers):
        prefix = f"l{index}"
        mixer = layer.mixer
        if isinstance(mixer, LatentAttentionConfig):
            mixer_spec = _latent_spec(width, f"{prefix}.mix", mixer, eps)
        else:
            assert isinstance(mixer, ParallelConfig)
            mixer_spec = PartSpec("parallel", {"members": (
                (_chunk_attention_spec(width, f"{prefix}.mix.left", mixer.left, eps), mixer.left_scale),
                (_retention_spec(width, f"{prefix}.mix.right", mixer.right, eps), mixer.right_scale))})
        extra = {"mixer_after": ("norm", PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm1b"}))}
        ffn = ffn_norm = None
        if layer.mlp is not None:
            ffn = _mlp_spec(width, f"{prefix}.mlp", layer.mlp)
            ffn_norm = PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm2"})
            extra["ffn_after"] = ("norm", PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm2b"}))
        layers.append(LayerSpec(arrangement="sandwich_norm", mixer_norm=PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm1"}),
                                mixer=mixer_spec, ffn_norm=ffn_norm, ffn=ffn, extra=extra, params={"residual_mult": 1.0}))
    order = tuple(RunEntry(layer=index, adds_embedding=again) for index, again in config.run_order())
    sizes = {"vocab_size": config.vocab, "hidden_size": width}
    return ModelSpec(
        architecture=config.architecture, vocab_size=config.vocab, hidden_size=width, max_positions=MAX_POSITIONS,
        embedding=PartSpec("token_embedding", {**sizes, "scale": config.embedding_scale}, {"weight": "embed"}),
        layers=tuple(layers), order=order,
        final_norm=PartSpec("rms_norm", norm, {"weight": "final.norm"}),
        head=PartSpec("lm_head", sizes, {"weight": "head"}))


def init_rules(config: KalevikConfig):
    """Random weights: norm weights around one; every matrix ~ N(0, std)."""
    return [
        InitRule(suffix="norm", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm1", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm2", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm1b", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm2b", mean=1.0, std_key="norm_std"),
        InitRule(suffix="", mean=0.0, std_key="std"),
    ]


register_architecture(Architecture(
    name="Kalevik",
    config_from_dict=KalevikConfig.from_dict,
    build_spec=build_spec,
    init_rules=init_rules,
))
