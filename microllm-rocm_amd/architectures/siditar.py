"""The Siditar decoder as a ``ModelSpec``.

Token embedding plus a sinusoidal position vector; layers in the pre-norm arrangement with a layer norm (weight, no
bias), joined to ``streams`` copies of the residual stream by hyper-connections where the configuration names
streams; per layer a ``parallel`` mixer (a softmax attention with a bias by distance bucket, a sink and a query
factor by position, beside a gated linear attention, each times a scale) and, unless the layer has none, a gated
feed-forward with clamped inputs; a final layer norm and an untied head. A range of layers may run several times in
a row with the same weights: every run is a run entry with a cache and state of its own.

Tensor names: ``embed``, ``head``, ``final.norm``; per layer ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.left.*``,
``l<i>.mix.right.*``, ``l<i>.mlp.{gate,up,down}``, ``l<i>.hc1.*`` and ``l<i>.hc2.*`` (``in``, ``out``, ``mix``).
"""
from __future__ import annotations

from ..config.fields import ConfigError
from ..config.registry import Architecture, register_architecture
from ..config.siditar import SiditarConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..weights.random_init import InitRule

MAX_POSITIONS = 1 << 20     # the position vector has no longest position; block tables and requests need a bound


def build_spec(config: SiditarConfig) -> ModelSpec:
    width = config.width
    norm = {"size": width, "eps": config.norm_eps}
    layers = []
    for index, layer in enumerate(config.layers):
        prefix = f"l{index}"
        left, right = layer.mixer.left, layer.mixer.right
        if left.bias_rows is None or right.decay_rank is None:
            raise ConfigError(f"layer {index}: the bias table's rows and the decay's rank are sizes of tensors; read the "
                              "configuration from a model folder, or name bias_rows and decay_rank")
        attention = PartSpec("bucket_bias_attention", {
            "hidden_size": width, "heads": left.heads, "kv_heads": left.kv_heads, "key_dim": left.dim, "value_dim": left.vdim,
            "scale": left.scale, "qk_norm": True, "eps": config.norm_eps, "temp_coef": left.temp_coef,
            "temp_every": left.temp_every, "bias_rows": left.bias_rows, "bias_max": left.bias_max, "sink": True},
            {"q": f"{prefix}.mix.left.q", "k": f"{prefix}.mix.left.k", "v": f"{prefix}.mix.left.v", "o": f"{prefix}.mix.left.o",
             "q_norm": f"{prefix}.mix.left.q.norm", "k_norm": f"{prefix}.mix.left.k.norm", "bias": f"{prefix}.mix.left.rel",
             "sink": f"{prefix}.mix.left.sink"})
        recurrent = PartSpec("gated_linear_attention", {
            "hidden_size": width, "heads": right.heads, "key_dim": right.dim, "value_dim": right.vdim, "tau": right.tau,
            "decay_rank": right.decay_rank, "eps": config.norm_eps, "query_scale": right.dim ** -0.5},
            {"q": f"{prefix}.mix.right.q", "k": f"{prefix}.mix.right.k", "v": f"{prefix}.mix.right.v", "g": f"{prefix}.mix.right.g",
             "o": f"{prefix}.mix.right.o", "norm": f"{prefix}.mix.right.norm", "a1": f"{prefix}.mix.right.a1",
             "a2": f"{prefix}.mix.right.a2", "a2_bias": f"{prefix}.mix.right.a2.b"})
        mixer = PartSpec("parallel", {"members": ((attention, layer.mixer.left_scale), (recurrent, layer.mixer.right_scale))})
        ffn = ffn_norm = None
        if layer.mlp is not None:
            ffn = PartSpec("clamped_glu", {"hidden_size": width, "intermediate_size": layer.mlp.ff, "limit": layer.mlp.limit,
                                           "slope": 1.702},
                           {role: f"{prefix}.mlp.{role}" for role in ("gate", "up", "down")})
            ffn_norm = PartSpec("layer_norm", norm, {"weight": f"{prefix}.norm2"})
        extra = {}
        if config.streams is not None:
            def connection(name: str) -> tuple:
                return ("connection", PartSpec("hyper_connection", {"streams": config.streams},
                                               {key: f"{prefix}.{name}.{key}" for key in ("in", "out", "mix")}))
            extra["mixer_connection"] = connection("hc1")
            if ffn is not None:
                extra["ffn_connection"] = connection("hc2")
        layers.append(LayerSpec(arrangement="hyper_connections" if config.streams is not None else "pre_norm",
                                mixer_norm=PartSpec("layer_norm", norm, {"weight": f"{prefix}.norm1"}), mixer=mixer,
                                ffn_norm=ffn_norm, ffn=ffn, extra=extra))
    sizes = {"vocab_size": config.vocab, "hidden_size": width}
    return ModelSpec(
        architecture=config.architecture, vocab_size=config.vocab, hidden_size=width, max_positions=MAX_POSITIONS,
        embedding=PartSpec("sinusoid_token_embedding", {**sizes, "base": 10000.0}, {"weight": "embed"}),
        layers=tuple(layers), order=tuple(RunEntry(layer=index) for index in config.run_order()),
        final_norm=PartSpec("layer_norm", norm, {"weight": "final.norm"}),
        head=PartSpec("lm_head", sizes, {"weight": "head"}), streams=config.streams)


def init_rules(config: SiditarConfig):
    """Random weights: norm weights 1 (+ N(0, norm_std)); the streams' read and write weights and their mixing matrix
    around an even split and the identity, so that random models stay bounded over many layers; sinks, bias tables
    and every matrix ~ N(0, std)."""
    return [
        InitRule(suffix=".norm", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm1", mean=1.0, std_key="norm_std"),
        InitRule(suffix="norm2", mean=1.0, std_key="norm_std"),
        InitRule(suffix=".in", mean=1.0 / (config.streams or 1), std_key="connection_std"),
        InitRule(suffix=".out", mean=1.0, std_key="connection_std"),
        InitRule(suffix=".mix", mean=1.0 / (config.streams or 1), std_key="connection_std"),
        InitRule(suffix=".rel", mean=0.0, std_key="bias_std"),
        InitRule(suffix=".sink", mean=0.0, std_key="bias_std"),
        InitRule(suffix="", mean=0.0, std_key="std"),
    ]


def complete_config(config: SiditarConfig, shapes) -> SiditarConfig:
    return config.with_tensor_shapes(shapes)


register_architecture(Architecture(
    name="Siditar",
    config_from_dict=SiditarConfig.from_dict,
    build_spec=build_spec,
    init_rules=init_rules,
    complete_config=complete_config,
))
