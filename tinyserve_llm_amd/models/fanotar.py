"""The Fanotar decoder as a ModelSpec. Token rows times a scale pass a norm and start a 32-bit residual
stream; every layer is the sandwich arrangement x <- x + n1b(mixer(n1 x)), x <- x + n2b(ff(n2 x)) with
dynamic-tanh norms n(x) = tanh(alpha x) w + b; the mixer is grouped-query attention without rotation
behind a short convolution on q, k and v (`parts.attention.ConvAttention`), which may read the cache of
an earlier layer instead of keeping its own; the feed-forward is a capped gated unit, dense or as a
mixture of experts with a shared expert, or absent. Checkpoint names: `embed`, `embed.norm[.b|.alpha]`,
`l<i>.norm{1,1b,2,2b}[.b|.alpha]`, `l<i>.mix.{q,k,v}[.conv]`, `l<i>.mix.{q,k}.norm`, `l<i>.mix.{sink,g,o}`,
`l<i>.mlp.{gate,up,down}` or `l<i>.mlp.{router,correction}`, `l<i>.mlp.e<j>.{gate,up,down}`,
`l<i>.mlp.shared.{gate,up,down}`, `final.norm[.b|.alpha]`, `head`."""

from __future__ import annotations

from tinyserve_llm_amd.config.fanotar import FanotarConfig, FanotarExperts, FanotarGatedUnit
from tinyserve_llm_amd.models.registry import Architecture, register_architecture
from tinyserve_llm_amd.models.spec import Destination, LayerRun, LayerSpec, ModelSpec
from tinyserve_llm_amd.parts.base import PartSpec

DISTANCE_SLOPE_EXPONENT = 8.0      # head h of H takes slope 2^(-8 (h + 1) / H) per position of distance
GATE_SLOPE = 1.702                 # of the sigmoid in the gated unit, g sigmoid(1.702 g) (u + 1)
UP_SHIFT = 1.0


def _norm_names(ckpt: dict[str, Destination], src: str, dst: str) -> None:
    ckpt[src] = Destination(f"{dst}weight")
    ckpt[f"{src}.b"] = Destination(f"{dst}bias")
    ckpt[f"{src}.alpha"] = Destination(f"{dst}alpha")


def _unit_names(ckpt: dict[str, Destination], src: str, dst: str, ff: int, index: tuple[int, ...] = ()) -> None:
    """gate and up into the two halves of one fused matrix (of a stack of them, at `index`), down beside it."""
    ckpt[f"{src}.gate"] = Destination(f"{dst}gate_up", 0, ff, index=index)
    ckpt[f"{src}.up"] = Destination(f"{dst}gate_up", ff, ff, index=index)
    ckpt[f"{src}.down"] = Destination(f"{dst}down", index=index)


def fanotar_spec(config: FanotarConfig) -> ModelSpec:
    c = config
    norm = PartSpec("dynamic_tanh", dict(hidden_size=c.width))
    ckpt: dict[str, Destination] = {"embed": Destination("embed.weight"), "head": Destination("head.weight")}
    _norm_names(ckpt, "embed.norm", "embed.norm_")
    _norm_names(ckpt, "final.norm", "final_norm.")
    # a cache is kept for the widest window of the layers that read it (0: for good)
    keep: dict[int, int] = {}
    for i, layer in enumerate(c.layers):
        owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
        w = layer.mixer.window
        keep[owner] = w if owner not in keep else (0 if 0 in (w, keep[owner]) else max(w, keep[owner]))
    layers: list[LayerSpec] = []
    order: list[LayerRun] = []
    for i, layer in enumerate(c.layers):
        src, dst, m = f"l{i}", f"layers.{i}", layer.mixer
        own = m.kv_from is None
        mixer = PartSpec("attention_conv", dict(
            hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
            conv_taps=m.conv, own_kv=own, scale=m.scale, window=m.window, cache_window=keep[i] if own else keep[m.kv_from],
            qk_norm_eps=c.norm_eps, q_temp_coef=m.q_temp_coef, q_temp_every=m.q_temp_every,
            slope_exponent=DISTANCE_SLOPE_EXPONENT, sink=True, gate=True))
        q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
        pieces = [("q", q)] + ([("k", k), ("v", v)] if own else [])
        at = 0
        for name, rows in pieces:
            ckpt[f"{src}.mix.{name}"] = Destination(f"{dst}.mixer.proj", at, rows)
            ckpt[f"{src}.mix.{name}.conv"] = Destination(f"{dst}.mixer.conv", at, rows)
            at += rows
        ckpt[f"{src}.mix.g"] = Destination(f"{dst}.mixer.proj", at, m.heads * m.vdim)
        ckpt[f"{src}.mix.q.norm"] = Destination(f"{dst}.mixer.q_norm")
        if own:
            ckpt[f"{src}.mix.k.norm"] = Destination(f"{dst}.mixer.k_norm")
        ckpt[f"{src}.mix.sink"] = Destination(f"{dst}.mixer.sink")
        ckpt[f"{src}.mix.o"] = Destination(f"{dst}.mixer.o")
        norms = {"norm1": norm, "norm1b": norm}
        unit = dict(slope=GATE_SLOPE, up_shift=UP_SHIFT)
        if layer.mlp is None:
            ff = PartSpec("none")
        elif isinstance(layer.mlp, FanotarGatedUnit):
            ff = PartSpec("capped_glu", dict(hidden_size=c.width, intermediate_size=layer.mlp.ff, limit=layer.mlp.limit, **unit))
            _unit_names(ckpt, f"{src}.mlp", f"{dst}.ff.", layer.mlp.ff)
        else:
            e: FanotarExperts = layer.mlp
            shared = None if e.shared is None else dict(intermediate_size=e.shared.ff, limit=e.shared.limit, **unit)
            ff = PartSpec("routed_experts", dict(
                hidden_size=c.width, num_experts=e.experts, top=e.top, intermediate_size=e.expert.ff, limit=e.expert.limit,
                router_scale=e.scale, normalize=True, correction=True, shared=shared, **unit))
            ckpt[f"{src}.mlp.router"] = Destination(f"{dst}.ff.router")
            ckpt[f"{src}.mlp.correction"] = Destination(f"{dst}.ff.correction")
            for j in range(e.experts):
                _unit_names(ckpt, f"{src}.mlp.e{j}", f"{dst}.ff.", e.expert.ff, index=(j,))
            if e.shared is not None:
                _unit_names(ckpt, f"{src}.mlp.shared", f"{dst}.ff.shared_", e.shared.ff)
        for name in ("norm1", "norm1b") + (("norm2", "norm2b") if layer.mlp is not None else ()):
            _norm_names(ckpt, f"{src}.{name}", f"{dst}.{name}.")
        if layer.mlp is not None:
            norms.update(norm2=norm, norm2b=norm)
        layers.append(LayerSpec(mixer, ff, norms, "sandwich"))
        order.append(LayerRun(i) if own else LayerRun(i, cache=m.kv_from, store=False))
    table = PartSpec("table", dict(vocab_size=c.vocab, hidden_size=c.width, float32_stream=True, scale=c.embedding_scale,
                                   norm=norm, init=(0.0, 1.0 / max(c.embedding_scale, 1e-6))))
    return ModelSpec(
        architecture=c.architecture, vocab_size=c.vocab, hidden_size=c.width, max_position=None, layers=layers, order=order,
        final_norm=norm, tie_word_embeddings=False, residual_dtype="float32", embedding=table, checkpoint=ckpt)


FANOTAR = register_architecture(Architecture(
    name="Fanotar", model_types=("fanotar",), config_from_dict=FanotarConfig.from_dict, build_spec=fanotar_spec,
    config_to_dict=FanotarConfig.to_dict))
