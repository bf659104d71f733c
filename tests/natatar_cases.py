"""Small Natatar configurations for the tests, and random weights under the checkpoint's names.

The configurations differ from one another in every size and option: 0 (plain residual sums), 1, 2 and 4 streams;
attentions with 1 to 4 query heads to a kv head, keys narrower and wider than values, with and without mixed
values (two and three layers that mix, a layer between them that does not); rotations over a whole head and over a
part of it, with and without stretched frequencies; matrix memories with keys narrower and wider than values and
than a lane's slice of the state; delta rules with 1 to 4 value heads to a key head, 1 to 4 taps, ranks of 3 to 9;
experts with one, some and all chosen, in 1 to 4 groups of which some or all are kept, layers without a
feed-forward; every order of the three mixers; sizes that are multiples of nothing."""

import torch


def _attention(heads, kv_heads, dim, vdim, scale, v_mix=False):
    raw = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if v_mix:
        raw["v_mix"] = True
    return raw


def _rot(dims, base, scaling=None):
    raw = {"dims": dims, "base": base}
    if scaling:
        raw["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return raw


def _parallel(left, rot, right, left_scale, right_scale):
    left = dict(left)
    if rot:
        left["rot"] = rot
    heads, dim, vdim, cap = right
    return {"left": left, "right": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "left_scale": left_scale,
            "right_scale": right_scale}  # fmt: skip


def _delta(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "decay_rank": decay_rank,
            "gate_rank": gate_rank}  # fmt: skip


def _moe(ff, experts, top, scale=None, groups=None):
    router = {"experts": experts, "top": top}
    if scale is not None:
        router["scale"] = scale
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


CASES = {
    # two streams; a delta rule first; three attentions, the first and the last of which mix values; a rotation of
    # part of a head with stretched frequencies
    "two_streams": {
        "architecture": "Natatar", "vocab": 200, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 0.6,
        "embedding": {"scale": 4.0}, "streams": 2,
        "layers": [
            {"type": "channel_delta", "mixer": _delta(4, 2, 24, 16, 3, 5, 7), "mlp": _moe(24, 6, 2, 1.5, (3, 2))},
            {"type": "attention", "mixer": _attention(4, 2, 16, 24, 0.3, v_mix=True), "mlp": None},
            {"type": "attention", "mixer": _attention(3, 3, 8, 8, 0.4), "mlp": _moe(16, 4, 1, 0.75, (2, 1))},
            {"type": "parallel", "mixer": _parallel(_attention(2, 1, 32, 16, 0.2), _rot(16, 10000.0, (4.0, 64, 16.0, 2.0)), (3, 8, 24, 10.0), 0.7, 1.2),
             "mlp": _moe(8, 5, 5)},
            {"type": "attention", "mixer": _attention(8, 2, 24, 24, 0.25, v_mix=True), "mlp": _moe(24, 6, 3, 2.0, (2, 2))},
        ],
    },  # fmt: skip
    # no streams, no multiplier, no embedding scale: plain residual sums; sizes that are multiples of nothing; one tap
    "plain_sums": {
        "architecture": "Natatar", "vocab": 203, "width": 88, "norm": {"eps": 1e-6},
        "layers": [
            {"type": "parallel", "mixer": _parallel(_attention(3, 3, 10, 14, 0.3), _rot(10, 500.0), (5, 6, 6, 18.0), 1.0, 0.4), "mlp": _moe(12, 4, 4)},
            {"type": "channel_delta", "mixer": _delta(3, 3, 10, 14, 1, 3, 9), "mlp": None},
            {"type": "attention", "mixer": _attention(2, 1, 12, 20, 0.35), "mlp": _moe(20, 9, 2, 3.0, (3, 1))},
        ],
    },  # fmt: skip
    # one stream (with coefficients of its own); keys wider than a lane's slice of the state in both recurrences;
    # three layers that mix values; a rotation without a scaling over part of a head
    "one_stream": {
        "architecture": "Natatar", "vocab": 128, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 1.25,
        "embedding": {"scale": 0.5}, "streams": 1,
        "layers": [
            {"type": "attention", "mixer": _attention(2, 2, 8, 16, 0.5, v_mix=True), "mlp": _moe(16, 3, 1)},
            {"type": "channel_delta", "mixer": _delta(2, 1, 72, 8, 4, 4, 4), "mlp": _moe(8, 8, 2, 1.0, (4, 2))},
            {"type": "attention", "mixer": _attention(4, 2, 16, 16, 0.2, v_mix=True), "mlp": None},
            {"type": "parallel", "mixer": _parallel(_attention(4, 1, 24, 24, 0.2), _rot(8, 50.0), (1, 80, 8, 5.0), 0.5, 0.5), "mlp": None},
            {"type": "attention", "mixer": _attention(2, 2, 40, 16, 0.15, v_mix=True), "mlp": _moe(24, 2, 2, 0.5)},
        ],
    },  # fmt: skip
    # four streams and heads of the widths the matrix-core kernels take (32, 64, 128); a rotation over a whole head
    "wide_heads": {
        "architecture": "Natatar", "vocab": 320, "width": 128, "norm": {"eps": 1e-5}, "residual_mult": 0.8,
        "embedding": {"scale": 2.0}, "streams": 4,
        "layers": [
            {"type": "parallel", "mixer": _parallel(_attention(4, 2, 64, 64, 0.125), _rot(64, 300000.0, (6.0, 32, 8.0, 1.5)), (2, 64, 32, 12.0), 0.9, 0.6),
             "mlp": _moe(64, 8, 2, 1.25, (4, 3))},
            {"type": "attention", "mixer": _attention(8, 2, 32, 32, 0.18, v_mix=True), "mlp": _moe(32, 4, 2, 1.0, (2, 2))},
            {"type": "channel_delta", "mixer": _delta(2, 2, 128, 64, 2, 8, 8), "mlp": None},
            {"type": "attention", "mixer": _attention(2, 2, 128, 32, 0.09, v_mix=True), "mlp": _moe(48, 6, 3, 0.5, (3, 2))},
        ],
    },  # fmt: skip
}


def random_weights(raw: dict, seed: int, std: float = 0.15) -> dict:
    """Tensors under the checkpoint's names, float32 holding bfloat16 values (exact in both precisions)."""
    g = torch.Generator().manual_seed(seed)
    h, vocab, s = raw["width"], raw["vocab"], raw.get("streams", 0)

    def mat(*shape, s=std):
        return (torch.randn(*shape, generator=g) * s).bfloat16().float()

    def gain(n):
        return (1.0 + torch.randn(n, generator=g) * 0.1).bfloat16().float()

    w = {"embed": mat(vocab, h, s=1.0), "final.norm": mat(h, s=0.1)}
    mixes = 0
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = mat(h, s=0.1)
        x = p + "mix."
        if layer["type"] == "attention":
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for name, rows in (("q", H * D), ("k", G * D), ("v", G * E)):
                w[x + name], w[x + name + ".b"] = mat(rows, h, s=0.3), mat(rows, s=0.3)
            w[x + "q.norm"], w[x + "k.norm"] = gain(H * D) * 2.0, gain(G * D) * 2.0
            if m.get("v_mix"):
                w[x + "vmix"] = torch.tensor(0.2 + 0.15 * mixes).bfloat16().float()
                mixes += 1
            w[x + "o"] = mat(h, H * E)
        elif layer["type"] == "parallel":
            a, r = m["left"], m["right"]
            H, G, D, E = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            y = x + "left."
            w[y + "q"], w[y + "k"], w[y + "v"] = mat(H * D, h, s=0.3), mat(G * D, h, s=0.3), mat(G * E, h, s=0.3)
            w[y + "g"], w[y + "o"] = mat(H * E, h), mat(h, H * E)
            H, D, E = r["heads"], r["dim"], r["vdim"]
            y = x + "right."
            w[y + "q"], w[y + "k"], w[y + "v"] = mat(H * D, h, s=0.3), mat(H * D, h, s=0.3), mat(H * E, h, s=0.3)
            w[y + "g"], w[y + "o"], w[y + "norm"] = mat(H * E, h), mat(h, H * E), gain(H * E)
            w[y + "i"], w[y + "i.b"] = mat(H, h, s=0.3), mat(H, s=0.5)
            w[y + "f"], w[y + "f.b"] = mat(H, h, s=0.3), (2.0 + torch.randn(H, generator=g)).bfloat16().float()
        else:
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for name, rows in (("q", G * D), ("k", G * D), ("v", H * E)):
                w[x + name], w[x + name + ".conv"] = mat(rows, h, s=0.4), mat(rows, m["conv"], s=0.5)
            w[x + "b"], w[x + "A_log"], w[x + "norm"] = mat(H, h, s=0.3), mat(H, s=0.5), gain(E)
            w[x + "a1"], w[x + "a2"] = mat(m["decay_rank"], h, s=0.3), mat(H * D, m["decay_rank"], s=0.5)
            w[x + "dt_bias"] = (torch.randn(H * D, generator=g) - 2.0).bfloat16().float()
            w[x + "g1"], w[x + "g2"] = mat(m["gate_rank"], h, s=0.3), mat(H * E, m["gate_rank"], s=0.5)
            w[x + "o"] = mat(h, H * E)
        mlp = layer["mlp"]
        if mlp is not None:
            w[p + "norm2"] = mat(h, s=0.1)
            x = p + "mlp."
            for e in range(mlp["router"]["experts"]):
                ff = mlp["expert"]["ff"]
                w[f"{x}e{e}.gate"], w[f"{x}e{e}.up"], w[f"{x}e{e}.down"] = mat(ff, h, s=0.3), mat(ff, h, s=0.3), mat(h, ff)
            w[x + "router"] = mat(mlp["router"]["experts"], h, s=0.3)
        for q in (1, 2) if mlp is not None else (1,):
            if s:
                w[p + f"hc{q}.in"] = (torch.rand(s, generator=g) * 0.8 + 0.2).bfloat16().float()
                w[p + f"hc{q}.out"] = gain(s)
                w[p + f"hc{q}.mix"] = (torch.eye(s) + torch.randn(s, s, generator=g) * 0.2).bfloat16().float()
    return w
