"""The Rugezen decoder as a ModelSpec. Every layer is the parallel arrangement
x <- x + m (mixer(norm1 x) + feed_forward(norm2 x)) on a 32-bit residual stream; the mixer is, layer
by layer, either grouped-query attention (interleaved rotary positions on a leading part of each
head, q, k and value heads divided by their root mean square, capped scores, a softmax with a sink,
value heads of their own size) or a minGRU; the feed-forward is dense with a squared relu and biases,
or absent. A stretch of layers may run several times in a row with the same weights: each pass is a
run of its own in the order, with its own cache or state. Checkpoint names: `embed`, `l<i>.norm1|2`,
`l<i>.mix.{q,k,v,o}` or `l<i>.mix.{z,z.b,x,x.b,g,o}`, `l<i>.mlp.{up,up.b,down,down.b}`, `final.norm`,
`head`."""

from __future__ import annotations

from tinyserve_llm_amd.config.rugezen import RugezenAttention, RugezenConfig
from tinyserve_llm_amd.models.registry import Architecture, register_architecture
from tinyserve_llm_amd.models.spec import Destination, LayerRun, LayerSpec, ModelSpec
from tinyserve_llm_amd.parts.base import PartSpec


def rugezen_spec(config: RugezenConfig) -> ModelSpec:
    c = config
    norm = PartSpec("rmsnorm", dict(hidden_size=c.width, eps=c.norm_eps))
    layers: list[LayerSpec] = []
    encodings: dict[str, PartSpec] = {}
    unused: list[str] = []
    ckpt: dict[str, Destination] = {"embed": Destination("embed.weight"), "final.norm": Destination("final_norm.weight"),
                                    "head": Destination("head.weight")}
    for i, layer in enumerate(c.layers):
        src, dst = f"l{i}", f"layers.{i}"
        ckpt[f"{src}.norm1"] = Destination(f"{dst}.norm1.weight")
        m = layer.mixer
        if isinstance(m, RugezenAttention):
            # one encoding per distinct (dims, base): layers that turn alike share its frequencies
            name = f"rotary_{m.rot_dims}_{m.rot_base!r}"
            encodings.setdefault(name, PartSpec("rotary_frequencies", dict(rotary_dim=m.rot_dims, theta=m.rot_base,
                                                                           interleaved=True)))
            mixer = PartSpec("attention_general", dict(
                hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                position=name if m.rot_dims else None, scale=m.scale, softcap=m.softcap, sink=True,
                qk_norm_eps=c.norm_eps, v_norm_eps=c.norm_eps))
            q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            ckpt[f"{src}.mix.q"] = Destination(f"{dst}.mixer.qkv", 0, q)
            ckpt[f"{src}.mix.k"] = Destination(f"{dst}.mixer.qkv", q, k)
            ckpt[f"{src}.mix.v"] = Destination(f"{dst}.mixer.qkv", q + k, v)
            ckpt[f"{src}.mix.o"] = Destination(f"{dst}.mixer.o")
        else:
            w = m.width
            mixer = PartSpec("mingru", dict(hidden_size=c.width, width=w, bias=True))
            ckpt[f"{src}.mix.z"] = Destination(f"{dst}.mixer.zxg", 0, w)
            ckpt[f"{src}.mix.x"] = Destination(f"{dst}.mixer.zxg", w, w)
            ckpt[f"{src}.mix.g"] = Destination(f"{dst}.mixer.zxg", 2 * w, w)
            ckpt[f"{src}.mix.z.b"] = Destination(f"{dst}.mixer.bias", 0, w)
            ckpt[f"{src}.mix.x.b"] = Destination(f"{dst}.mixer.bias", w, w)
            ckpt[f"{src}.mix.o"] = Destination(f"{dst}.mixer.o")
        norms = {"norm1": norm}
        if layer.ff is None:
            ff = PartSpec("none")
            unused.append(f"{src}.norm2")        # (a checkpoint may carry the norm of the branch that is not there)
        else:
            norms["norm2"] = norm
            ckpt[f"{src}.norm2"] = Destination(f"{dst}.norm2.weight")
            ff = PartSpec("dense_mlp", dict(hidden_size=c.width, intermediate_size=layer.ff, activation="relu2", bias=True))
            ckpt[f"{src}.mlp.up"] = Destination(f"{dst}.ff.up")
            ckpt[f"{src}.mlp.up.b"] = Destination(f"{dst}.ff.up_bias")
            ckpt[f"{src}.mlp.down"] = Destination(f"{dst}.ff.down")
            ckpt[f"{src}.mlp.down.b"] = Destination(f"{dst}.ff.down_bias")
        layers.append(LayerSpec(mixer, ff, norms, "parallel", {"residual_mult": c.residual_mult}))
    return ModelSpec(
        architecture=c.architecture, vocab_size=c.vocab, hidden_size=c.width, max_position=None, layers=layers,
        order=[LayerRun(i) for i in c.run_order()], final_norm=norm, position_encodings=encodings,
        tie_word_embeddings=False, residual_dtype="float32", checkpoint=ckpt, optional=tuple(unused))


RUGEZEN = register_architecture(Architecture(
    name="Rugezen", model_types=("rugezen",), config_from_dict=RugezenConfig.from_dict, build_spec=rugezen_spec,
    config_to_dict=RugezenConfig.to_dict))
