"""Koravik: configuration -> layer plan, and the checkpoint's tensor names.

Pre-norm layers whose parts enter the stream through a sigmoid gate and a common factor; the mixer is a
grouped-query attention whose keys are also its values, whose heads' scores are mixed before the softmax
and whose window keeps the sequence's first tokens; the feed-forward is made of routed experts and a shared
one.  The embedding's rows are normed before they become the stream; a stretch of layers may run several
times in a row, every pass with caches of its own and entering through a matrix that also reads what the
embedding gave; the head is the embedding table.
"""

from atomserve_amd.config.model_config import KoravikConfig
from atomserve_amd.config.registry import Architecture, register_architecture
from atomserve_amd.parts.plan import (
    BlockSpec,
    MixedHeadsAttentionSpec,
    ModelPlan,
    NormSpec,
    RotarySpec,
    RoutedExpertsSpec,
    Run,
)
from atomserve_amd.weights.loader import Stack, Take

MAX_POSITIONS = 1 << 30  # nothing in the design depends on a position's size


def build_plan(c: KoravikConfig) -> ModelPlan:
    def norm():
        return NormSpec("rmsnorm", c.hidden_size, c.norm_eps)

    layers = []
    for layer in c.layers:
        m = layer.mixer
        mixer = MixedHeadsAttentionSpec(
            "mixed_heads_attention", c.hidden_size, m.heads, m.kv_heads, m.dim, m.scale,
            position=RotarySpec("rope_half", m.rot_dims, m.rot_base) if m.rot_dims else None,
            window=m.window, keep_first=m.keep_first, mix_heads=True, values="keys", out_gate=True,
        )  # fmt: skip
        f = layer.mlp
        ffn = None
        if f is not None:
            ffn = RoutedExpertsSpec("routed_experts", c.hidden_size, f.ff, f.experts, f.top, "relu2", "sigmoid",
                                    shared_size=f.shared_ff, out_gate=True)  # fmt: skip
        layers.append(BlockSpec("gated_prenorm", mixer, norm(), ffn, None if ffn is None else norm(),
                                residual_scale=c.residual_mult))  # fmt: skip
    return ModelPlan(
        vocab_size=c.vocab_size,
        hidden_size=c.hidden_size,
        layers=tuple(layers),
        run=tuple(Run(i, reenter=reenter) for i, reenter in c.run_order()),
        final_norm=norm(),
        tied_head=True,
        max_positions=MAX_POSITIONS,
        logit_scale=c.logit_scale,
        embed_norm=norm(),
        reentry=c.reenters,
    )


def checkpoint_map(c: KoravikConfig) -> dict:
    """Plan tensor name -> checkpoint names.  The projections that read a part's input, the part's output gate
    among them, are stacked into one matrix."""
    names = {"embed.weight": "embed", "embed_norm.weight": "embed.norm", "final_norm.weight": "final.norm"}
    if c.reenters:
        names["reentry.weight"] = "loop.in"
    for i, layer in enumerate(c.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"] = src + "norm1"
        mix, to = src + "mix.", dst + "mixer."
        names[to + "in.weight"] = [mix + "q", mix + "k", src + "rg1"]
        names[to + "o.weight"] = mix + "o"
        names[to + "mix"] = mix + "talk"
        names[to + "gate_bias"] = src + "rg1.b"
        f = layer.mlp
        if f is None:
            continue
        names[dst + "ffn_norm.weight"] = src + "norm2"
        mlp, to = src + "mlp.", dst + "ffn."
        names[to + "router.weight"] = mlp + "router"
        for part in ("up", "down"):
            names[to + part + ".weight"] = Stack(tuple(Take(f"{mlp}e{e}.{part}") for e in range(f.experts)), new_axis=True)
        if f.shared_ff:
            names[to + "side.weight"] = [mlp + "shared.up", src + "rg2"]
            names[to + "shared_down.weight"] = mlp + "shared.down"
        else:
            names[to + "side.weight"] = src + "rg2"
        names[to + "gate_bias"] = src + "rg2.b"
    return names


def checkpoint_shapes(c: KoravikConfig) -> dict:
    """Checkpoint name -> (shape, role), in the order in which random weights are drawn."""
    h = c.hidden_size
    shapes = {"embed": ((c.vocab_size, h), "matrix"), "embed.norm": ((h,), "vector")}
    if c.reenters:
        shapes["loop.in"] = ((h, 2 * h), "matrix")
    for i, layer in enumerate(c.layers):
        p, m = f"l{i}.", layer.mixer
        shapes[p + "norm1"] = ((h,), "vector")
        if layer.mlp is not None:
            shapes[p + "norm2"] = ((h,), "vector")
        x = p + "mix."
        shapes[x + "q"] = ((m.heads * m.dim, h), "matrix")
        shapes[x + "k"] = ((m.kv_heads * m.dim, h), "matrix")
        shapes[x + "talk"] = ((m.heads, m.heads), "near_identity")
        shapes[x + "o"] = ((h, m.heads * m.dim), "matrix")
        f = layer.mlp
        if f is not None:
            x = p + "mlp."
            for e in range(f.experts):
                shapes[f"{x}e{e}.up"] = ((f.ff, h), "matrix")
                shapes[f"{x}e{e}.down"] = ((h, f.ff), "matrix")
            shapes[x + "router"] = ((f.experts, h), "matrix")
            if f.shared_ff:
                shapes[x + "shared.up"] = ((f.shared_ff, h), "matrix")
                shapes[x + "shared.down"] = ((h, f.shared_ff), "matrix")
        shapes[p + "rg1"] = ((h, h), "matrix")
        shapes[p + "rg1.b"] = ((h,), "bias")
        if f is not None:
            shapes[p + "rg2"] = ((h, h), "matrix")
            shapes[p + "rg2.b"] = ((h,), "bias")
    shapes["final.norm"] = ((h,), "vector")
    return shapes


KORAVIK = register_architecture(
    Architecture(
        name=KoravikConfig.architecture,
        parse_config=KoravikConfig.from_dict,
        build_plan=build_plan,
        checkpoint_map=checkpoint_map,
        checkpoint_shapes=checkpoint_shapes,
    ),
    replace=True,
)
