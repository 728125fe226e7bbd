"""Dozusun: configuration -> layer plan, and the checkpoint's tensor names.

Every layer adds a mixer and (where it has one) a feed-forward to the stream, both reading the same stream
through an RMS norm each.  The mixer is a gated delta rule ("delta") or a windowed, gated attention side by
side with a gated linear recurrence ("parallel"); the feed-forward is dense or made of experts that a table
names per token id.  A stretch of layers may run several times in a row with the same weights, every pass
with caches and states of its own (the run list names the layer again; a run's caches are its own).
"""

from atomserve_amd.config.model_config import DozusunConfig
from atomserve_amd.config.registry import Architecture, register_architecture
from atomserve_amd.parts.plan import (
    BlockSpec,
    DeltaRuleSpec,
    GatedAttentionSpec,
    GatedMLPSpec,
    LinearRecurrenceSpec,
    ModelPlan,
    NormSpec,
    Run,
    ShortConvSpec,
    SideBySideSpec,
    TableExpertsSpec,
)
from atomserve_amd.weights.loader import Stack, Take

MAX_POSITIONS = 1 << 30  # nothing in the design depends on a position's size


def build_plan(c: DozusunConfig) -> ModelPlan:
    def norm(size):
        return NormSpec("rmsnorm", size, c.norm_eps)

    layers = []
    for layer in c.layers:
        m = layer.mixer
        if layer.type == "delta":
            mixer = DeltaRuleSpec("delta_rule", c.hidden_size, m.heads, m.kv_heads, m.dim, m.vdim, ShortConvSpec(m.conv),
                                  out_norm_eps=c.norm_eps)  # fmt: skip
        else:
            mixer = SideBySideSpec(
                "side_by_side", c.hidden_size,
                left=GatedAttentionSpec(m.heads, m.kv_heads, m.dim, m.vdim, m.scale, norm(m.dim), m.window),
                right=LinearRecurrenceSpec(m.width, m.blocks, ShortConvSpec(m.conv)),
                left_scale=m.left_scale, right_scale=m.right_scale,
            )  # fmt: skip
        f = layer.mlp
        if f is None:
            ffn = None
        elif f.kind == "dense":
            ffn = GatedMLPSpec("gated_mlp", c.hidden_size, f.ff, "silu")
        else:
            ffn = TableExpertsSpec("table_experts", c.hidden_size, f.ff, f.experts, f.top, c.vocab_size, "silu")
        layers.append(BlockSpec("two_norms", mixer, norm(c.hidden_size), ffn, None if ffn is None else norm(c.hidden_size)))
    return ModelPlan(
        vocab_size=c.vocab_size,
        hidden_size=c.hidden_size,
        layers=tuple(layers),
        run=tuple(Run(i) for i in c.run_order()),
        final_norm=norm(c.hidden_size),
        tied_head=False,
        max_positions=MAX_POSITIONS,
    )


def checkpoint_map(c: DozusunConfig) -> dict:
    """Plan tensor name -> checkpoint names.  The projections that read a mixer's input are stacked into one
    matrix, in the order the parts expect their columns."""
    names = {"embed.weight": "embed", "final_norm.weight": "final.norm", "head.weight": "head"}
    for i, layer in enumerate(c.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"] = src + "norm1"
        mix, to = src + "mix.", dst + "mixer."
        if layer.type == "delta":
            names[to + "in.weight"] = [mix + p for p in ("q", "k", "v", "g", "b", "a")]
            names[to + "conv.weight"] = [mix + p + ".conv" for p in ("q", "k", "v")]
            names[to + "a_log"] = mix + "A_log"
            names[to + "dt_bias"] = mix + "dt_bias"
            names[to + "out_norm.weight"] = mix + "norm"
            names[to + "out.weight"] = mix + "o"
        else:
            left, right = mix + "left.", mix + "right."
            names[to + "in.weight"] = [left + "q", left + "k", left + "v", left + "g", right + "y", right + "x"]
            names[to + "out_t.weight"] = [Take(left + "o", transpose=True), Take(right + "o", transpose=True)]
            names[to + "q_norm.weight"] = left + "q.norm"
            names[to + "k_norm.weight"] = left + "k.norm"
            names[to + "y_bias"] = right + "y.b"
            names[to + "x_bias"] = right + "x.b"
            names[to + "conv.weight"] = right + "conv"
            names[to + "conv.bias"] = right + "conv.b"
            names[to + "gate_a.weight"] = right + "ra"
            names[to + "gate_a.bias"] = right + "ra.b"
            names[to + "gate_i.weight"] = right + "ri"
            names[to + "gate_i.bias"] = right + "ri.b"
            names[to + "lam"] = right + "lam"
        f = layer.mlp
        if f is None:
            continue
        names[dst + "ffn_norm.weight"] = src + "norm2"
        mlp, to = src + "mlp.", dst + "ffn."
        if f.kind == "dense":
            names[to + "gate_up.weight"] = [mlp + "gate", mlp + "up"]
            names[to + "down.weight"] = mlp + "down"
        else:
            for part in ("gate", "up", "down"):
                names[to + part + ".weight"] = Stack(tuple(Take(f"{mlp}e{e}.{part}") for e in range(f.experts)), new_axis=True)
            names[to + "table"] = mlp + "table"
    return names


def checkpoint_shapes(c: DozusunConfig) -> dict:
    """Checkpoint name -> (shape, role), in the order in which random weights are drawn."""
    h = c.hidden_size
    shapes = {"embed": ((c.vocab_size, h), "matrix")}
    for i, layer in enumerate(c.layers):
        p, m = f"l{i}.", layer.mixer
        shapes[p + "norm1"] = ((h,), "vector")
        if layer.mlp is not None:
            shapes[p + "norm2"] = ((h,), "vector")
        if layer.type == "delta":
            x = p + "mix."
            for name, rows in (("q", m.kv_heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.heads * m.vdim)):
                shapes[x + name] = ((rows, h), "matrix")
                shapes[x + name + ".conv"] = ((rows, m.conv), "matrix")
            shapes[x + "b"] = ((m.heads, h), "matrix")
            shapes[x + "A_log"] = ((m.heads,), "log_rate")
            shapes[x + "norm"] = ((m.vdim,), "vector")
            shapes[x + "a"] = ((m.heads, h), "matrix")
            shapes[x + "dt_bias"] = ((m.heads,), "bias")
            shapes[x + "g"] = ((m.heads * m.vdim, h), "matrix")
            shapes[x + "o"] = ((h, m.heads * m.vdim), "matrix")
        else:
            x, bw = p + "mix.left.", m.width // m.blocks
            shapes[x + "q"] = ((m.heads * m.dim, h), "matrix")
            shapes[x + "k"] = ((m.kv_heads * m.dim, h), "matrix")
            shapes[x + "v"] = ((m.kv_heads * m.vdim, h), "matrix")
            shapes[x + "q.norm"] = ((m.dim,), "vector")
            shapes[x + "k.norm"] = ((m.dim,), "vector")
            shapes[x + "g"] = ((m.heads * m.vdim, h), "matrix")
            shapes[x + "o"] = ((h, m.heads * m.vdim), "matrix")
            x = p + "mix.right."
            shapes[x + "y"] = ((m.width, h), "matrix")
            shapes[x + "y.b"] = ((m.width,), "bias")
            shapes[x + "x"] = ((m.width, h), "matrix")
            shapes[x + "x.b"] = ((m.width,), "bias")
            shapes[x + "conv"] = ((m.width, m.conv), "matrix")
            shapes[x + "conv.b"] = ((m.width,), "bias")
            shapes[x + "ra"] = ((m.blocks, bw, bw), "matrix")
            shapes[x + "ra.b"] = ((m.blocks, bw), "bias")
            shapes[x + "ri"] = ((m.blocks, bw, bw), "matrix")
            shapes[x + "ri.b"] = ((m.blocks, bw), "bias")
            shapes[x + "lam"] = ((m.width,), "bias")
            shapes[x + "o"] = ((h, m.width), "matrix")
        f = layer.mlp
        if f is None:
            continue
        x = p + "mlp."
        if f.kind == "dense":
            shapes[x + "gate"] = ((f.ff, h), "matrix")
            shapes[x + "up"] = ((f.ff, h), "matrix")
            shapes[x + "down"] = ((h, f.ff), "matrix")
        else:
            for e in range(f.experts):
                shapes[f"{x}e{e}.gate"] = ((f.ff, h), "matrix")
                shapes[f"{x}e{e}.up"] = ((f.ff, h), "matrix")
                shapes[f"{x}e{e}.down"] = ((h, f.ff), "matrix")
            shapes[x + "table"] = ((c.vocab_size, f.top), f"expert_table:{f.experts}")
    shapes["final.norm"] = ((h,), "vector")
    shapes["head"] = ((c.vocab_size, h), "matrix")
    return shapes


DOZUSUN = register_architecture(
    Architecture(
        name=DozusunConfig.architecture,
        parse_config=DozusunConfig.from_dict,
        build_plan=build_plan,
        checkpoint_map=checkpoint_map,
        checkpoint_shapes=checkpoint_shapes,
    ),
    replace=True,
)
