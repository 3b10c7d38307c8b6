"""The Gupitar decoder as a ``ModelSpec``.

Token embedding; layers in the pre-norm arrangement with an RMS norm whose weight is stored around zero (the gain is
one plus the weight); per layer either an attention through latents (queries through a normed latent, keys and
values projected up from one cached normed latent a token, a rotated key part shared by all heads, a sliding window,
an output gate) or a recurrent block (a gated branch beside a short causal convolution and a gated linear recurrence);
a dense gated feed-forward, a mixture of experts with a sigmoid router and a gated shared expert, or none; a final
norm and an untied head. A layer may read the cached latents of an earlier layer instead of making its own: its
run entry reads that layer's cache.

Tensor names: ``embed``, ``head``, ``final.norm``; per layer ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``,
``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.router``, ``l<i>.mlp.e<j>.{gate,up,down}``, ``l<i>.mlp.shared.{gate,up,down,sg}``.
"""
from __future__ import annotations

from ..config.gupitar import DenseMlpConfig, GupitarConfig, LatentAttentionConfig, MoeMlpConfig, RglruConfig
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..weights.random_init import InitRule

MAX_POSITIONS = 1 << 20     # the rotation has no longest position; block tables and requests need a bound
DECAY_SCALE = 8.0           # log a = -DECAY_SCALE * r * softplus(lam): fixed by the design


def _feed_forward(mlp, width: int, prefix: str) -> PartSpec:
    if isinstance(mlp, DenseMlpConfig):
        return PartSpec("swiglu", {"hidden_size": width, "intermediate_size": mlp.ff},
                        {"gate_proj.weight": f"{prefix}.mlp.gate", "up_proj.weight": f"{prefix}.mlp.up",
                         "down_proj.weight": f"{prefix}.mlp.down"})
    assert isinstance(mlp, MoeMlpConfig)
    names = {"router": f"{prefix}.mlp.router"}
    for expert in range(mlp.experts):
        for role in ("gate", "up", "down"):
            names[f"expert{expert}.{role}"] = f"{prefix}.mlp.e{expert}.{role}"
    if mlp.shared_ff is not None:
        for role in ("gate", "up", "down"):
            names[f"shared.{role}"] = f"{prefix}.mlp.shared.{role}"
        names["shared.scale"] = f"{prefix}.mlp.shared.sg"
    return PartSpec("routed_experts", {
        "hidden_size": width, "experts": mlp.experts, "top": mlp.top, "expert_size": mlp.expert_ff,
        "shared_size": mlp.shared_ff, "score": "sigmoid", "renormalize": False, "weight_on": "input",
        "shared_scale": "sigmoid" if mlp.shared_ff is not None else None}, names)


def build_spec(config: GupitarConfig) -> ModelSpec:
    width = config.width
    norm = {"size": width, "eps": config.norm_eps, "unit_offset": True}
    # A layer that lends its latents keeps them as long as the widest window among itself and its borrowers.
    kept_window = {}
    for index, layer in enumerate(config.layers):
        if isinstance(layer.mixer, LatentAttentionConfig):
            owner = layer.mixer.kv_from if layer.mixer.kv_from is not None else index
            kept_window[owner] = max(kept_window.get(owner, 0), layer.mixer.window)
    layers, order = [], []
    for index, layer in enumerate(config.layers):
        prefix = f"l{index}"
        mixer = layer.mixer
        reads = None
        if isinstance(mixer, LatentAttentionConfig):
            owns = mixer.kv_from is None
            reads = mixer.kv_from
            roles = ["dq", "uq", "uk", "uv", "g", "o"] + (["dkv"] if owns else [])
            names = {role: f"{prefix}.mix.{role}" for role in roles}
            names["dq_norm"] = f"{prefix}.mix.dq.norm"
            if owns:
                names["dkv_norm"] = f"{prefix}.mix.dkv.norm"
            mixer_spec = PartSpec("latent_attention", {
                "hidden_size": width, "heads": mixer.heads, "dim": mixer.dim, "rot_dim": mixer.rot_dim, "vdim": mixer.vdim,
                "q_rank": mixer.q_rank, "kv_rank": mixer.kv_rank, "scale": mixer.scale, "window": mixer.window,
                "kept_window": kept_window[index if owns else mixer.kv_from], "eps": config.norm_eps, "owns_kv": owns,
                "output_gate": True,
                "position": PartSpec("rope_split_half", {"theta": mixer.rot_base, "head_dim": mixer.rot_dim,
                                                         "rotary_dim": mixer.rot_dims})}, names)
        else:
            assert isinstance(mixer, RglruConfig)
            names = {role: f"{prefix}.mix.{role}" for role in ("y", "x", "conv", "ra", "ri", "lam", "o")}
            names.update({f"{role}_bias": f"{prefix}.mix.{role}.b" for role in ("y", "x", "conv", "ra", "ri")})
            mixer_spec = PartSpec("rglru", {"hidden_size": width, "width": mixer.width, "blocks": mixer.blocks,
                                            "taps": mixer.conv, "decay_scale": DECAY_SCALE}, names)
        ffn = ffn_norm = None
        if layer.mlp is not None:
            ffn = _feed_forward(layer.mlp, width, prefix)
            ffn_norm = PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm2"})
        layers.append(LayerSpec(arrangement="pre_norm", mixer_norm=PartSpec("rms_norm", norm, {"weight": f"{prefix}.norm1"}),
                                mixer=mixer_spec, ffn_norm=ffn_norm, ffn=ffn))
        order.append(RunEntry(layer=index, reads_cache_of=reads))
    sizes = {"vocab_size": config.vocab, "hidden_size": width}
    return ModelSpec(
        architecture=config.architecture, vocab_size=config.vocab, hidden_size=width, max_positions=MAX_POSITIONS,
        embedding=PartSpec("token_embedding", sizes, {"weight": "embed"}),
        layers=tuple(layers), order=tuple(order),
        final_norm=PartSpec("rms_norm", norm, {"weight": "final.norm"}),
        head=PartSpec("lm_head", sizes, {"weight": "head"}))


def init_rules(config: GupitarConfig):
    """Random weights: the layers' norm weights around zero, the latents' norm weights around one, biases and the
    recurrence's ``lam`` ~ N(0, bias_std), every matrix ~ N(0, std)."""
    return [
        InitRule(suffix="final.norm", mean=0.0, std_key="norm_std"),
        InitRule(suffix="norm1", mean=0.0, std_key="norm_std"),
        InitRule(suffix="norm2", mean=0.0, std_key="norm_std"),
        InitRule(suffix=".norm", mean=1.0, std_key="norm_std"),
        InitRule(suffix=".b", mean=0.0, std_key="bias_std"),
        InitRule(suffix=".lam", mean=0.0, std_key="bias_std"),
        InitRule(suffix="", mean=0.0, std_key="std"),
    ]


register_architecture(Architecture(
    name="Gupitar",
    config_from_dict=GupitarConfig.from_dict,
    build_spec=build_spec,
    init_rules=init_rules,
))
