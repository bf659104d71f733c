"""Natatar: configuration -> layer plan, and the checkpoint's tensor names.

Pre-norm layers over several residual streams (each sublayer reads them as one weighted sum and writes its output
back into all of them through a mixing matrix); norms whose gains are stored around zero.  The mixer is a softmax
attention with biases and a norm over the whole of q and of k whose values may be mixed with those of the first
such layer ("attention"), a rotary, gated attention beside a matrix memory with exponential gates ("parallel"), or
a gated delta rule with a decay per key channel ("channel_delta"); the feed-forward is made of experts chosen by
their softmax scores within the best groups, or absent.  The embedding table, scaled on the way in, is also the head.
"""

from atomserve_amd.config.model_config import ConfigError, NatatarConfig
from atomserve_amd.config.registry import Architecture, register_architecture
from atomserve_amd.parts.plan import (
    BlockSpec,
    ChannelDeltaRuleSpec,
    GatedRoutedExpertsSpec,
    JoinedMixerSpec,
    MatrixMemorySpec,
    ModelPlan,
    NeighbourRotarySpec,
    NormSpec,
    ShortConvSpec,
    SoftmaxCoreSpec,
    sequential_run,
)
from atomserve_amd.weights.loader import Stack, Take

MAX_POSITIONS = 1 << 30  # nothing in the design depends on a position's size
VALUES_KEY = "first_mixed_values"


def _rotation(rot):
    if rot is None:
        return None
    dims, base, scaling = rot
    if scaling:
        return NeighbourRotarySpec("rope_neighbours", dims, base, *scaling)
    return NeighbourRotarySpec("rope_neighbours", dims, base)


def _first_mixing_layer(c: NatatarConfig) -> int:
    for i, layer in enumerate(c.layers):
        if layer.type == "attention" and layer.mixer.v_mix:
            return i
    return -1


def build_plan(c: NatatarConfig) -> ModelPlan:
    def norm(size):
        return NormSpec("rmsnorm", size, c.norm_eps, offset=1.0)

    first_mix = _first_mixing_layer(c)
    layers = []
    for i, layer in enumerate(c.layers):
        m = layer.mixer
        if layer.type == "attention":
            mix = "none" if not m.v_mix else ("first" if i == first_mix else "later")
            core = SoftmaxCoreSpec("softmax_core", m.heads, m.kv_heads, m.dim, m.vdim, m.scale, bias=True,
                                   whole_norm_eps=c.norm_eps, position=_rotation(m.rot), value_mix=mix,
                                   value_mix_key=VALUES_KEY)  # fmt: skip
            mixer = JoinedMixerSpec("joined", c.hidden_size, (core,), (1.0,))
        elif layer.type == "parallel":
            a, r = m.left, m.right
            left = SoftmaxCoreSpec("softmax_core", a.heads, a.kv_heads, a.dim, a.vdim, a.scale, position=_rotation(a.rot),
                                   out_gate=True)  # fmt: skip
            right = MatrixMemorySpec("matrix_memory", r.heads, r.dim, r.vdim, r.gate_cap, c.norm_eps)
            mixer = JoinedMixerSpec("joined", c.hidden_size, (left, right), (m.left_scale, m.right_scale))
        else:
            if m.decay_rank < 1 or m.gate_rank < 1:
                raise ConfigError(f"layers[{i}]: the ranks of the two-step projections are unknown (no checkpoint names "
                                  "them and the configuration has no decay_rank and gate_rank)")  # fmt: skip
            mixer = ChannelDeltaRuleSpec("channel_delta_rule", c.hidden_size, m.heads, m.kv_heads, m.dim, m.vdim,
                                         ShortConvSpec(m.conv), m.decay_rank, m.gate_rank, out_norm_eps=c.norm_eps)  # fmt: skip
        f = layer.mlp
        ffn = None
        if f is not None:
            ffn = GatedRoutedExpertsSpec("gated_routed_experts", c.hidden_size, f.ff, f.experts, f.top, "silu", 0.0,
                                         score="softmax", router_bias=False, groups=f.groups, keep_groups=f.keep,
                                         weight_scale=f.scale)  # fmt: skip
        layers.append(BlockSpec("streams_prenorm", mixer, norm(c.hidden_size), ffn, None if ffn is None else norm(c.hidden_size),
                                residual_scale=c.residual_mult, streams=c.streams, streams_first=i == 0,
                                streams_last=i == len(c.layers) - 1))  # fmt: skip
    return ModelPlan(
        vocab_size=c.vocab_size,
        hidden_size=c.hidden_size,
        layers=tuple(layers),
        run=sequential_run(len(layers)),
        final_norm=norm(c.hidden_size),
        tied_head=True,
        max_positions=MAX_POSITIONS,
        embedding_scale=c.embedding_scale,
    )


def checkpoint_map(c: NatatarConfig) -> dict:
    """Plan tensor name -> checkpoint names.  The projections that read a mixer's input are stacked into one matrix, in
    the order the cores expect their columns; the output projections of a mixer's cores are stacked transposed."""
    names = {"embed.weight": "embed", "final_norm.weight": "final.norm"}
    first_mix = _first_mixing_layer(c)
    for i, layer in enumerate(c.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"] = src + "norm1"
        mix, to = src + "mix.", dst + "mixer."
        if layer.type == "attention":
            names[to + "in.weight"] = [mix + "q", mix + "k", mix + "v"]
            names[to + "out_t.weight"] = Take(mix + "o", transpose=True)
            for p in ("q", "k", "v"):
                names[to + f"c0.{p}_bias"] = mix + p + ".b"
            names[to + "c0.q_norm"] = mix + "q.norm"
            names[to + "c0.k_norm"] = mix + "k.norm"
            if layer.mixer.v_mix and i != first_mix:
                names[to + "c0.value_mix"] = mix + "vmix"
        elif layer.type == "parallel":
            left, right = mix + "left.", mix + "right."
            names[to + "in.weight"] = [left + p for p in ("q", "k", "v", "g")] + [right + p for p in ("q", "k", "v", "g", "i", "f")]
            names[to + "out_t.weight"] = [Take(left + "o", transpose=True), Take(right + "o", transpose=True)]
            names[to + "c1.i_bias"] = right + "i.b"
            names[to + "c1.f_bias"] = right + "f.b"
            names[to + "c1.out_norm"] = right + "norm"
        else:
            names[to + "in.weight"] = [mix + p for p in ("q", "k", "v", "b")]
            names[to + "low.weight"] = [mix + "a1", mix + "g1"]
            names[to + "decay_up.weight"] = mix + "a2"
            names[to + "gate_up.weight"] = mix + "g2"
            names[to + "conv.weight"] = [mix + p + ".conv" for p in ("q", "k", "v")]
            names[to + "a_log"] = mix + "A_log"
            names[to + "dt_bias"] = mix + "dt_bias"
            names[to + "out_norm.weight"] = mix + "norm"
            names[to + "out.weight"] = mix + "o"
        if c.streams:
            for q in (1, 2) if layer.mlp is not None else (1,):
                for p in ("in", "mix", "out"):
                    names[dst + f"streams.hc{q}.{p}"] = src + f"hc{q}.{p}"
        f = layer.mlp
        if f is None:
            continue
        names[dst + "ffn_norm.weight"] = src + "norm2"
        mlp, to = src + "mlp.", dst + "ffn."
        names[to + "router.weight"] = mlp + "router"
        for part in ("gate", "up", "down"):
            names[to + part + ".weight"] = Stack(tuple(Take(f"{mlp}e{e}.{part}") for e in range(f.experts)), new_axis=True)
    return names


def ignored(c: NatatarConfig) -> set:
    """A mixing weight that an attention layer stores and does not use: the first value-mixing layer's own, and that of
    a layer that mixes nothing."""
    first_mix = _first_mixing_layer(c)
    return {f"l{i}.mix.vmix" for i, layer in enumerate(c.layers)
            if layer.type == "attention" and (i == first_mix or not layer.mixer.v_mix)}  # fmt: skip


def checkpoint_shapes(c: NatatarConfig) -> dict:
    """Checkpoint name -> (shape, role), in the order in which random weights are drawn."""
    h = c.hidden_size
    shapes = {"embed": ((c.vocab_size, h), "matrix")}
    for i, layer in enumerate(c.layers):
        p, m = f"l{i}.", layer.mixer
        shapes[p + "norm1"] = ((h,), "bias")
        if layer.mlp is not None:
            shapes[p + "norm2"] = ((h,), "bias")
        x = p + "mix."
        if layer.type == "attention":
            for name, rows in (("q", m.heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.kv_heads * m.vdim)):
                shapes[x + name] = ((rows, h), "matrix")
                shapes[x + name + ".b"] = ((rows,), "bias")
            shapes[x + "q.norm"] = ((m.heads * m.dim,), "vector")
            shapes[x + "k.norm"] = ((m.kv_heads * m.dim,), "vector")
            if m.v_mix:
                shapes[x + "vmix"] = ((), "fraction")
            shapes[x + "o"] = ((h, m.heads * m.vdim), "matrix")
        elif layer.type == "parallel":
            a, r = m.left, m.right
            y = x + "left."
            shapes[y + "q"] = ((a.heads * a.dim, h), "matrix")
            shapes[y + "k"] = ((a.kv_heads * a.dim, h), "matrix")
            shapes[y + "v"] = ((a.kv_heads * a.vdim, h), "matrix")
            shapes[y + "g"] = ((a.heads * a.vdim, h), "matrix")
            shapes[y + "o"] = ((h, a.heads * a.vdim), "matrix")
            y = x + "right."
            shapes[y + "q"] = ((r.heads * r.dim, h), "matrix")
            shapes[y + "k"] = ((r.heads * r.dim, h), "matrix")
            shapes[y + "v"] = ((r.heads * r.vdim, h), "matrix")
            shapes[y + "g"] = ((r.heads * r.vdim, h), "matrix")
            shapes[y + "o"] = ((h, r.heads * r.vdim), "matrix")
            shapes[y + "norm"] = ((r.heads * r.vdim,), "vector")
            shapes[y + "i"] = ((r.heads, h), "matrix")
            shapes[y + "i.b"] = ((r.heads,), "bias")
            shapes[y + "f"] = ((r.heads, h), "matrix")
            shapes[y + "f.b"] = ((r.heads,), "bias")
        else:
            for name, rows in (("q", m.kv_heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.heads * m.vdim)):
                shapes[x + name] = ((rows, h), "matrix")
                shapes[x + name + ".conv"] = ((rows, m.conv), "matrix")
            shapes[x + "b"] = ((m.heads, h), "matrix")
            shapes[x + "A_log"] = ((m.heads,), "log_rate")
            shapes[x + "norm"] = ((m.vdim,), "vector")
            shapes[x + "a1"] = ((m.decay_rank, h), "matrix")
            shapes[x + "a2"] = ((m.heads * m.dim, m.decay_rank), "matrix")
            shapes[x + "dt_bias"] = ((m.heads * m.dim,), "bias")
            shapes[x + "g1"] = ((m.gate_rank, h), "matrix")
            shapes[x + "g2"] = ((m.heads * m.vdim, m.gate_rank), "matrix")
            shapes[x + "o"] = ((h, m.heads * m.vdim), "matrix")
        f = layer.mlp
        if f is not None:
            x = p + "mlp."
            for e in range(f.experts):
                shapes[f"{x}e{e}.gate"] = ((f.ff, h), "matrix")
                shapes[f"{x}e{e}.up"] = ((f.ff, h), "matrix")
                shapes[f"{x}e{e}.down"] = ((h, f.ff), "matrix")
            shapes[x + "router"] = ((f.experts, h), "matrix")
        if c.streams:
            for q in (1, 2) if f is not None else (1,):
                shapes[p + f"hc{q}.in"] = ((c.streams,), "fraction")
                shapes[p + f"hc{q}.out"] = ((c.streams,), "vector")
                shapes[p + f"hc{q}.mix"] = ((c.streams, c.streams), "near_identity")
    shapes["final.norm"] = ((h,), "bias")
    return shapes


NATATAR = register_architecture(
    Architecture(
        name=NatatarConfig.architecture,
        parse_config=NatatarConfig.from_dict,
        build_plan=build_plan,
        checkpoint_map=checkpoint_map,
        checkpoint_shapes=checkpoint_shapes,
        ignored=ignored,
        complete=lambda config, shape_of: config.completed(shape_of),
    ),
    replace=True,
)
