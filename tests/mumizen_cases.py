"""Small Mumizen configurations for the tests, and random weights under the checkpoint's names.

The configurations differ from one another in every size and option: norms in 1, 3 and 4 groups; linear attentions
with one head and with several, keys narrower and wider than values, keys wider than a lane's slice of the state;
attentions through a latent with 3 to 18 heads, plain and turned parts of unequal widths, latents of 24 to 128,
rotations with and without stretched frequencies, layers that read the latent of the layer before or of one further
back, two readers of one latent; dense feed-forwards, experts with one, some and all chosen, with and without a shared
expert, and layers without a feed-forward; every order of the three mixers."""

import torch


def _decay(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, scaling=None, kv_from=None):
    raw = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
           "rot": {"dims": rot_dim, "base": base}}  # fmt: skip
    if scaling:
        raw["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if kv_from is not None:
        raw["kv_from"] = kv_from
    return raw


def _dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def _moe(ff, limit, experts, top, shared=None):
    raw = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared:
        raw["shared"] = {"ff": shared[0], "limit": shared[1]}
    return raw


CASES = {
    # a latent first, read again two layers later; keys of 24 over values of 40; three groups
    "latent_first": {
        "architecture": "Mumizen", "vocab": 200, "width": 96, "norm": {"eps": 1e-5, "groups": 3},
        "layers": [
            {"type": "latent_attention", "mixer": _latent(3, 8, 8, 16, 24, 40, 0.3, 10000.0, (4.0, 64, 16.0, 2.0)), "mlp": _moe(24, 2.5, 5, 2, (16, 0.75))},
            {"type": "retention", "mixer": _decay(3, 16, 8, (0.9, 0.99, 0.5)), "mlp": None},
            {"type": "latent_attention", "mixer": _latent(5, 16, 8, 8, 16, 40, 0.2, 10000.0, (4.0, 64, 16.0, 2.0), kv_from=0), "mlp": _dense(40, 1.25)},
            {"type": "lightning", "mixer": _decay(2, 24, 40, (0.97, 0.8)), "mlp": _moe(16, 1.0, 3, 3)},
        ],
    },  # fmt: skip
    # one group; one head whose keys are wider than a lane's slice of the state; 18 heads over one latent; a rotation
    # that is not stretched; one expert chosen
    "wide_keys": {
        "architecture": "Mumizen", "vocab": 128, "width": 64, "norm": {"eps": 1e-6, "groups": 1},
        "layers": [
            {"type": "lightning", "mixer": _decay(1, 72, 32, (0.995,)), "mlp": _dense(48, 3.0)},
            {"type": "retention", "mixer": _decay(4, 8, 24, (1.0, 0.9375, 0.75, 0.25)), "mlp": _moe(8, 0.5, 7, 1, (24, 4.0))},
            {"type": "latent_attention", "mixer": _latent(18, 4, 4, 8, 8, 24, 0.4, 50.0), "mlp": None},
        ],
    },  # fmt: skip
    # latents only: a wide one read by both layers after it, and a second one of another size with its own rotation
    "latents": {
        "architecture": "Mumizen", "vocab": 300, "width": 128, "norm": {"eps": 1e-5, "groups": 4},
        "layers": [
            {"type": "latent_attention", "mixer": _latent(4, 32, 32, 32, 48, 128, 0.125, 300000.0, (16.0, 32, 8.0, 1.0)), "mlp": _dense(64, 0.875)},
            {"type": "latent_attention", "mixer": _latent(8, 8, 32, 24, 32, 128, 0.18, 300000.0, (16.0, 32, 8.0, 1.0), kv_from=0), "mlp": _moe(32, 2.0, 9, 4, (8, 1.5))},
            {"type": "latent_attention", "mixer": _latent(2, 40, 32, 16, 64, 128, 0.11, 300000.0, (16.0, 32, 8.0, 1.0), kv_from=0), "mlp": None},
            {"type": "latent_attention", "mixer": _latent(6, 16, 2, 8, 8, 56, 0.25, 7.0, (2.0, 16, 4.0, 0.5)), "mlp": _dense(24, 6.0)},
        ],
    },  # fmt: skip
    # a latent wider than the paged attention kernels' heads, with a reader; a rotation over few coordinates
    "wide_latent": {
        "architecture": "Mumizen", "vocab": 150, "width": 64, "norm": {"eps": 1e-5, "groups": 2},
        "layers": [
            {"type": "latent_attention", "mixer": _latent(2, 16, 4, 24, 16, 270, 0.06, 300.0, (4.0, 32, 8.0, 1.0)), "mlp": _dense(32, 2.0)},
            {"type": "latent_attention", "mixer": _latent(3, 8, 4, 8, 24, 270, 0.08, 300.0, (4.0, 32, 8.0, 1.0), kv_from=0), "mlp": None},
        ],
    },  # fmt: skip
    # sizes that are multiples of nothing: odd vocabulary, heads of 10 and 14, latents of 20 and 36, inner widths of 20 and 12
    "odd_sizes": {
        "architecture": "Mumizen", "vocab": 203, "width": 88, "norm": {"eps": 1e-6, "groups": 2},
        "layers": [
            {"type": "retention", "mixer": _decay(3, 10, 14, (0.99, 0.9, 0.75)), "mlp": _dense(20, 1.0)},
            {"type": "latent_attention", "mixer": _latent(3, 10, 6, 10, 20, 36, 0.25, 1000.0, (6.0, 32, 24.0, 1.5)), "mlp": _moe(12, 1.75, 6, 3, (20, 2.25))},
            {"type": "lightning", "mixer": _decay(5, 6, 6, (0.55, 0.7, 0.85, 0.95, 0.998)), "mlp": _moe(12, 1.75, 4, 2)},
            {"type": "latent_attention", "mixer": _latent(7, 6, 6, 10, 12, 36, 0.3, 1000.0, (6.0, 32, 24.0, 1.5), kv_from=1), "mlp": _dense(28, 2.0)},
        ],
    },  # fmt: skip
}


def random_weights(raw: dict, seed: int, std: float = 0.15) -> dict:
    """Tensors under the checkpoint's names, float32 holding bfloat16 values (exact in both precisions)."""
    g = torch.Generator().manual_seed(seed)
    h, vocab = raw["width"], raw["vocab"]

    def mat(*shape, s=std):
        return (torch.randn(*shape, generator=g) * s).bfloat16().float()

    def gain(n):
        return (1.0 + torch.randn(n, generator=g) * 0.1).bfloat16().float()

    def ff(prefix, width, inner):
        w[prefix + "gate"], w[prefix + "up"], w[prefix + "down"] = mat(inner, width, s=0.3), mat(inner, width, s=0.3), mat(width, inner)

    w = {"embed": mat(vocab, h, s=1.0), "final.norm": gain(h), "head": mat(vocab, h)}
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = gain(h)
        w[p + "shift"] = torch.rand(h, generator=g).bfloat16().float()
        dwa = torch.randn(i + 2, generator=g) * 0.2
        dwa[-1] += 1.0
        w[p + "dwa"] = dwa.bfloat16().float()
        x = p + "mix."
        if layer["type"] == "latent_attention":
            H, D, R, E = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            w[x + "dq"], w[x + "dq.norm"] = mat(m["q_rank"], h), gain(m["q_rank"])
            w[x + "uq"] = mat(H * (D + R), m["q_rank"], s=0.5)
            if "kv_from" not in m:
                w[x + "dkv"], w[x + "dkv.norm"] = mat(m["kv_rank"] + R, h), gain(m["kv_rank"])
            w[x + "uk"], w[x + "uv"] = mat(H * D, m["kv_rank"], s=0.4), mat(H * E, m["kv_rank"], s=0.2)
            w[x + "g"], w[x + "o"] = mat(H * E, h), mat(h, H * E)
        else:
            H, D, E = m["heads"], m["dim"], m["vdim"]
            w[x + "q"], w[x + "k"], w[x + "v"] = mat(H * D, h, s=0.3), mat(H * D, h, s=0.3), mat(H * E, h, s=0.3)
            w[x + "g"], w[x + "o"] = mat(H * E, h), mat(h, H * E)
            if layer["type"] == "lightning":
                w[x + "norm"] = gain(H * E)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        w[p + "norm2"] = gain(h)
        x = p + "mlp."
        if mlp["kind"] == "dense":
            ff(x, h, mlp["ff"])
        else:
            for e in range(mlp["router"]["experts"]):
                ff(f"{x}e{e}.", h, mlp["expert"]["ff"])
            w[x + "router"], w[x + "router.b"] = mat(mlp["router"]["experts"], h, s=0.3), mat(mlp["router"]["experts"], s=0.5)
            if mlp.get("shared"):
                ff(x + "shared.", h, mlp["shared"]["ff"])
    return w
