"""The Zabozen decoder as a ``ModelSpec``.

Token embedding; layers with an RMS norm before and after each sublayer and a factor on what joins the residual stream
(the ``sandwich_norm`` arrangement); per layer one of three mixers: a causal attention through cached latents (queries
straight from the input, a rotated key part shared by all heads, a gate of one number a head), a softmax attention over
a sliding window (grouped key/value heads, projection biases, queries and keys of unit root mean square, a slope a
head times the distance taken off the scores; a layer may read the keys and values another layer cached), or the gated
delta rule behind short convolutions; a dense gated feed-forward or none; a final norm, an untied head and a soft cap
``c * tanh(logits / c)`` on the logits.

Tensor names: ``embed``, ``head``, ``final.norm``; per layer ``l<i>.norm1``, ``l<i>.norm1b`` (after the mixer),
``l<i>.norm2``, ``l<i>.norm2b`` (after the feed-forward), ``l<i>.mix.*`` and ``l<i>.mlp.{gate,up,down}``; a projection's
bias is its weight's name with ``.b``, a convolution's taps its projection's name with ``.conv``.
"""
from __future__ import annotations

from ..config.registry import Architecture, register_architecture
from ..config.zabozen import DeltaConfig, LatentAttentionConfig, WindowAttentionConfig, ZabozenConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..weights.random_init import InitRule

MAX_POSITIONS = 1 << 20     # no part has a longest position; block tables and requests need a bound
SLOPE_EXPONENT = 8.0        # head h of H takes slope 2^(-SLOPE_EXPONENT (h + 1) / H) off the score per token of distance
UNIT_EPS = 1e-6             # inside the root that makes the delta rule's queries and keys unit vectors


def distance_slopes(heads: int):
    return [2.0 ** (-SLOPE_EXPONENT * (head + 1) / heads) for head in range(heads)]


def build_spec(config: ZabozenConfig) -> ModelSpec:
    width = config.width
    norm = {"size": width, "eps": config.norm_eps}
    # A layer that lends its keys and values keeps them as long as the widest window among itself and its borrowers.
    kept_window = {}
    for index, layer in enumerate(config.layers):
        if isinstance(layer.mixer, WindowAttentionConfig):
            owner = layer.mixer.kv_from if layer.mixer.kv_from is not None else index
            kept_window[owner] = max(kept_window.get(owner, 0), layer.mixer.window)
    layers, order = [], []
    for index, layer in enumerate(config.layers):
        prefix = f"l{index}"
        mixer = layer.mixer
        reads = None
        if isinstance(mixer, LatentAttentionConfig):
            names = {role: f"{prefix}.mix.{role}" for role in ("q", "dkv", "uk", "uv", "g", "o")}
            names["dkv_norm"] = f"{prefix}.mix.dkv.norm"
            mixer_spec = PartSpec("latent_attention", {
                "hidden_size": width, "heads": mixer.heads, "dim": mixer.dim, "rot_dim": mixer.rot_dim, "vdim": mixer.vdim,
                "q_rank": None, "kv_rank": mixer.kv_rank, "scale": mixer.scale, "window": None, "eps": config.norm_eps,
                "owns_kv": True, "output_gate": True, "gate_a_head": True,
                "position": PartSpec("rope_split_half", {"theta": mixer.rot_base, "head_dim": mixer.rot_dim,
                                                         "rotary_dim": mixer.rot_dims})}, names)
        elif isinstance(mixer, WindowAttentionConfig):
            owns = mixer.kv_from is None
            reads = mixer.kv_from
            names = {}
            for role in ("q", "o") + (("k", "v") if owns else ()):
                names[role] = f"{prefix}.mix.{role}"
                names[f"{role}_bias"] = f"{prefix}.mix.{role}.b"
            mixer_spec = PartSpec("bucket_bias_attention", {
                "hidden_size": width, "heads": mixer.heads, "kv_heads": mixer.kv_heads, "key_dim": mixer.dim, "value_dim": mixer.vdim,
                "scale": mixer.scale, "qk_norm": True, "qk_norm_weight": False, "eps": config.norm_eps, "projection_bias": True,
                "slopes": distance_slopes(mixer.heads), "window": mixer.window,
                "kept_window": kept_window[index if owns else mixer.kv_from], "owns_kv": owns, "sink": False}, names)
        else:
            assert isinstance(mixer, DeltaConfig)
            names = {role: f"{prefix}.mix.{role}" for role in ("q", "k", "v", "g", "o", "norm", "A_log", "dt_bias")}
            names.update({"beta": f"{prefix}.mix.b", "step": f"{prefix}.mix.a"})
            names.update({f"{role}_conv": f"{prefix}.mix.{role}.conv" for role in ("q", "k", "v")})
            mixer_spec = PartSpec("gated_delta_rule", {
                "hidden_size": width, "heads": mixer.heads, "key_heads": mixer.kv_heads, "key_dim": mixer.dim, "value_dim": mixer.vdim,
                "taps": mixer.conv, "eps": config.norm_eps, "unit_eps": UNIT_EPS, "query_scale": mixer.dim ** -0.5}, names)
        extra = {"mixer_after": ("norm", PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm1b"}))}
        ffn = ffn_norm = None
        if layer.mlp is not None:
            ffn = PartSpec("swiglu", {"hidden_size": width, "intermediate_size": layer.mlp.ff},
                           {"gate_proj.weight": f"{prefix}.mlp.gate", "up_proj.weight": f"{prefix}.mlp.up",
                            "down_proj.weight": f"{prefix}.mlp.down"})
            ffn_norm = PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm2"})
            extra["ffn_after"] = ("norm", PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm2b"}))
        layers.append(LayerSpec(arrangement="sandwich_norm", mixer_norm=PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm1"}),
                                mixer=mixer_spec, ffn_norm=ffn_norm, ffn=ffn, extra=extra,
                                params={"residual_mult": config.residual_mult}))
        order.append(RunEntry(layer=index, reads_cache_of=reads))
    sizes = {"vocab_size": config.vocab, "hidden_size": width}
    return ModelSpec(
        architecture=config.architecture, vocab_size=config.vocab, hidden_size=width, max_positions=MAX_POSITIONS,
        embedding=PartSpec("token_embedding", sizes, {"weight": "embed"}),
        layers=tuple(layers), order=tuple(order),
        final_norm=PartSpec("rms_norm", norm, {"weight": "final.norm"}),
        head=PartSpec("lm_head", {**sizes, "softcap": config.logit_softcap}, {"weight": "head"}))


def init_rules(config: ZabozenConfig):
    """Random weights: norm weights around one; biases, the decays' ``A_log`` and ``dt_bias`` ~ N(0, bias_std); the
    convolutions' taps ~ N(0, conv_std); every matrix ~ N(0, std)."""
    return [
        InitRule(suffix="norm", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm1", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm2", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm1b", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm2b", mean=1.0, std_key="norm_std"),
        InitRule(suffix=".conv", mean=0.0, std_key="conv_std"),
        InitRule(suffix=".A_log", mean=0.0, std_key="bias_std"),
        InitRule(suffix=".dt_bias", mean=0.0, std_key="bias_std"),
        InitRule(suffix=".o.b", mean=0.0, std_key="bias_std"),
        InitRule(suffix=".q.b", mean=0.0, std_key="bias_std"),
        InitRule(suffix=".k.b", mean=0.0, std_key="bias_std"),
        InitRule(suffix=".v.b", mean=0.0, std_key="bias_std"),
        InitRule(suffix="", mean=0.0, std_key="std"),
    ]


register_architecture(Architecture(
    name="Zabozen",
    config_from_dict=ZabozenConfig.from_dict,
    build_spec=build_spec,
    init_rules=init_rules,
))
