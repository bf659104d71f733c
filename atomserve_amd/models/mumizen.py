"""Mumizen: configuration -> layer plan, and the checkpoint's tensor names.

Pre-norm layers whose norms work in groups, whose mixer reads a token-shifted input and whose result is averaged
with the results of all layers before it.  The mixer is a linear attention with a fixed decay per head (in two
flavours) or a softmax attention through a cached latent, which may be an earlier layer's; the feed-forward is a
gated one with limits, dense or made of routed experts beside a shared one.  A layer that reads an earlier layer's
latent is a run whose cache is that layer's run and that writes nothing.
"""

from atomserve_amd.config.model_config import MumizenConfig
from atomserve_amd.config.registry import Architecture, register_architecture
from atomserve_amd.parts.plan import (
    BlockSpec,
    DecayAttentionSpec,
    GatedMLPSpec,
    GatedRoutedExpertsSpec,
    LatentAttentionSpec,
    ModelPlan,
    NormSpec,
    RotarySpec,
    Run,
    ScaledRotarySpec,
)
from atomserve_amd.weights.loader import Stack, Take

MAX_POSITIONS = 1 << 30  # nothing in the design depends on a position's size


def _mixer_spec(c: MumizenConfig, layer):
    m = layer.mixer
    if layer.type == "lightning":
        return DecayAttentionSpec("decay_attention", c.hidden_size, m.heads, m.dim, m.vdim, tuple(m.decay), activation="silu",
                                  key_scale=1.0, out_norm="all", out_norm_eps=c.norm_eps, gate="sigmoid")  # fmt: skip
    if layer.type == "retention":
        return DecayAttentionSpec("decay_attention", c.hidden_size, m.heads, m.dim, m.vdim, tuple(m.decay), activation=None,
                                  key_scale=m.dim**-0.5, out_norm="heads", out_norm_eps=c.norm_eps, gate="silu")  # fmt: skip
    position = None
    if m.rot_dim:
        if m.scaling:
            position = ScaledRotarySpec("rope_half_scaled", m.rot_dim, m.rot_base, *m.scaling)
        else:
            position = RotarySpec("rope_half", m.rot_dim, m.rot_base)
    return LatentAttentionSpec("latent_attention", c.hidden_size, m.heads, m.dim, m.rot_dim, m.vdim, m.q_rank, m.kv_rank,
                               m.scale, c.norm_eps, position, own_latent=m.kv_from < 0)  # fmt: skip


def build_plan(c: MumizenConfig) -> ModelPlan:
    def norm():
        return NormSpec("grouped_rmsnorm", c.hidden_size, c.norm_eps, c.norm_groups)

    layers, run = [], []
    for i, layer in enumerate(c.layers):
        f = layer.mlp
        if f is None:
            ffn = None
        elif f.kind == "dense":
            ffn = GatedMLPSpec("gated_mlp", c.hidden_size, f.ff, "clamped_swish", f.limit)
        else:
            ffn = GatedRoutedExpertsSpec("gated_routed_experts", c.hidden_size, f.ff, f.experts, f.top, "clamped_swish", f.limit,
                                         score="softmax_of_chosen", router_bias=True, shared_size=f.shared_ff,
                                         shared_limit=f.shared_limit)  # fmt: skip
        layers.append(BlockSpec("depth_prenorm", _mixer_spec(c, layer), norm(), ffn, None if ffn is None else norm(),
                                token_shift=True, depth_index=i, depth_slots=len(c.layers) + 1))  # fmt: skip
        reads = layer.mixer.kv_from if layer.type == "latent_attention" else -1
        run.append(Run(i, cache=reads, writes=False) if reads >= 0 else Run(i))
    return ModelPlan(
        vocab_size=c.vocab_size,
        hidden_size=c.hidden_size,
        layers=tuple(layers),
        run=tuple(run),
        final_norm=norm(),
        tied_head=False,
        max_positions=MAX_POSITIONS,
    )


def checkpoint_map(c: MumizenConfig) -> dict:
    """Plan tensor name -> checkpoint names.  The projections that read a mixer's input are stacked into one matrix,
    in the order the parts expect their columns."""
    names = {"embed.weight": "embed", "final_norm.weight": "final.norm", "head.weight": "head"}
    for i, layer in enumerate(c.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"] = src + "norm1"
        names[dst + "vectors.shift"] = src + "shift"
        names[dst + "vectors.depth"] = src + "dwa"
        mix, to = src + "mix.", dst + "mixer."
        if layer.type == "latent_attention":
            own = layer.mixer.kv_from < 0
            names[to + "in.weight"] = [mix + "dq"] + ([mix + "dkv"] if own else []) + [mix + "g"]
            names[to + "q_norm.weight"] = mix + "dq.norm"
            if own:
                names[to + "kv_norm.weight"] = mix + "dkv.norm"
            for part in ("uq", "uk", "uv", "o"):
                names[to + part + ".weight"] = mix + part
        else:
            names[to + "in.weight"] = [mix + p for p in ("q", "k", "v", "g")]
            names[to + "out.weight"] = mix + "o"
            if layer.type == "lightning":
                names[to + "out_norm.weight"] = mix + "norm"
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
            names[to + "router.weight"] = mlp + "router"
            names[to + "router.bias"] = mlp + "router.b"
            if f.shared_ff:
                names[to + "shared_gate_up.weight"] = [mlp + "shared.gate", mlp + "shared.up"]
                names[to + "shared_down.weight"] = mlp + "shared.down"
    return names


def checkpoint_shapes(c: MumizenConfig) -> dict:
    """Checkpoint name -> (shape, role), in the order in which random weights are drawn."""
    h = c.hidden_size
    shapes = {"embed": ((c.vocab_size, h), "matrix")}
    for i, layer in enumerate(c.layers):
        p, m = f"l{i}.", layer.mixer
        shapes[p + "norm1"] = ((h,), "vector")
        if layer.mlp is not None:
            shapes[p + "norm2"] = ((h,), "vector")
        x = p + "mix."
        if layer.type == "latent_attention":
            shapes[x + "dq"] = ((m.q_rank, h), "matrix")
            shapes[x + "dq.norm"] = ((m.q_rank,), "vector")
            shapes[x + "uq"] = ((m.heads * (m.dim + m.rot_dim), m.q_rank), "matrix")
            if m.kv_from < 0:
                shapes[x + "dkv"] = ((m.kv_rank + m.rot_dim, h), "matrix")
                shapes[x + "dkv.norm"] = ((m.kv_rank,), "vector")
            shapes[x + "uk"] = ((m.heads * m.dim, m.kv_rank), "matrix")
            shapes[x + "uv"] = ((m.heads * m.vdim, m.kv_rank), "matrix")
            shapes[x + "g"] = ((m.heads * m.vdim, h), "matrix")
            shapes[x + "o"] = ((h, m.heads * m.vdim), "matrix")
        else:
            shapes[x + "q"] = ((m.heads * m.dim, h), "matrix")
            shapes[x + "k"] = ((m.heads * m.dim, h), "matrix")
            shapes[x + "v"] = ((m.heads * m.vdim, h), "matrix")
            shapes[x + "g"] = ((m.heads * m.vdim, h), "matrix")
            shapes[x + "o"] = ((h, m.heads * m.vdim), "matrix")
            if layer.type == "lightning":
                shapes[x + "norm"] = ((m.heads * m.vdim,), "vector")
        f = layer.mlp
        if f is not None:
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
                shapes[x + "router"] = ((f.experts, h), "matrix")
                shapes[x + "router.b"] = ((f.experts,), "bias")
                if f.shared_ff:
                    shapes[x + "shared.gate"] = ((f.shared_ff, h), "matrix")
                    shapes[x + "shared.up"] = ((f.shared_ff, h), "matrix")
                    shapes[x + "shared.down"] = ((h, f.shared_ff), "matrix")
        shapes[p + "shift"] = ((h,), "fraction")
        shapes[p + "dwa"] = ((i + 2,), "depth_weights")
    shapes["final.norm"] = ((h,), "vector")
    shapes["head"] = ((c.vocab_size, h), "matrix")
    return shapes


MUMIZEN = register_architecture(
    Architecture(
        name=MumizenConfig.architecture,
        parse_config=MumizenConfig.from_dict,
        build_plan=build_plan,
        checkpoint_map=checkpoint_map,
        checkpoint_shapes=checkpoint_shapes,
    ),
    replace=True,
)
