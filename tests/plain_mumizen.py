"""Mumizen written plainly: one function per mechanism, a whole sequence at a time, token by token where a
state is carried.  It shares nothing with the package: tensors come as a dict of checkpoint names, the
configuration as the parsed config.json.  `bf16=True` rounds to bfloat16 at the places where an engine that
stores bfloat16 numbers must (the products' inputs and outputs, what a cache holds); how far that moves the
plain model's own logits is the yardstick of the bfloat16 tests.

    layer i:   h = shift(norm1(x));  x += mixer(h);  x += ff(norm2(x));  X_(i+1) = x;  x = sum_j dwa_i[j] X_j
"""

import math

import torch

F = torch.float64


def rnd(t, bf16):
    return t.to(torch.bfloat16).to(t.dtype) if bf16 else t


def linear(w, x, bf16):
    """W x for every row of x, the result rounded as a bfloat16 product's would be."""
    return rnd(rnd(x, bf16) @ w.to(x.dtype).t(), bf16)


def grouped_rms_norm(x, w, eps, groups):
    T, n = x.shape
    parts = x.view(T, groups, n // groups)
    parts = parts / torch.sqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)
    return parts.reshape(T, n) * w.to(x.dtype)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def token_shift(h, mu):
    """h_t + (h_(t-1) - h_t) * mu, zeros before the first token."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (before - h) * mu.to(h.dtype)


def decayed_state_scan(q, k, v, decay):
    """Per head: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  q, k [T, H, D], v [T, H, E] -> [T, H, E]."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[2], dtype=q.dtype)
    lam = torch.tensor(decay, dtype=q.dtype).view(H, 1, 1)
    out = []
    for t in range(T):
        S = lam * S + k[t].unsqueeze(2) * v[t].unsqueeze(1)
        out.append(torch.einsum("hde,hd->he", S, q[t]))
    return torch.stack(out)


def lightning_mixer(h, W, p, m, eps, bf16):
    T = h.shape[0]
    H, D, E = m["heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q = rnd(silu(linear(W[p + "q"], h, bf16)), bf16).view(T, H, D)
    k = rnd(silu(linear(W[p + "k"], h, bf16)), bf16).view(T, H, D)
    v = rnd(silu(linear(W[p + "v"], h, bf16)), bf16).view(T, H, E)
    o = decayed_state_scan(q, k, v, m["decay"]).reshape(T, H * E)
    o = rms(o, eps) * W[p + "norm"].to(h.dtype)
    o = o * torch.sigmoid(linear(W[p + "g"], h, bf16))
    return linear(W[p + "o"], o, bf16)


def retention_mixer(h, W, p, m, eps, bf16):
    T = h.shape[0]
    H, D, E = m["heads"], m["dim"], m["vdim"]
    q = linear(W[p + "q"], h, bf16).view(T, H, D)
    k = rnd(linear(W[p + "k"], h, bf16).view(T, H, D) * D**-0.5, bf16)
    v = linear(W[p + "v"], h, bf16).view(T, H, E)
    o = rms(decayed_state_scan(q, k, v, m["decay"]), eps).reshape(T, H * E)
    o = o * torch.nn.functional.silu(linear(W[p + "g"], h, bf16))
    return linear(W[p + "o"], o, bf16)


def yarn_angles(positions, rot, dtype=F):
    """cos and sin [T, dims/2] of the scaled rotation: frequencies blended between f and f / factor by a ramp over
    the pair index, both tables times 0.1 ln(factor) + 1."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=dtype)
    f = base ** (-2.0 * i / dims)
    scaling = rot.get("scaling")
    mult = 1.0
    if scaling:
        factor, orig = scaling["factor"], scaling["original"]

        def dim_of(turns):
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(dim_of(scaling["fast"])), 0)
        hi = min(math.ceil(dim_of(scaling["slow"])), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        mult = 0.1 * math.log(factor) + 1.0
    a = positions.to(dtype).unsqueeze(1) * f
    return torch.cos(a) * mult, torch.sin(a) * mult


def rotate_half(x, cos, sin):
    """x [T, ..., dims]: pairs (i, i + dims/2) turn by the token's angles."""
    half = x.shape[-1] // 2
    u, v = x[..., :half], x[..., half:]
    while cos.dim() < u.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    return torch.cat([u * cos - v * sin, v * cos + u * sin], dim=-1)


def latent_kv(h, W, p, m, eps, positions, bf16):
    """What a latent-attention layer caches: the normed latent [T, kv_rank] and the turned shared key part [T, rot_dim]."""
    r = m["kv_rank"]
    d = linear(W[p + "dkv"], h, bf16)
    c = rnd(rms(d[:, :r], eps) * W[p + "dkv.norm"].to(h.dtype), bf16)
    cos, sin = yarn_angles(positions, m["rot"], h.dtype)
    return c, rnd(rotate_half(d[:, r:], cos, sin), bf16)


def latent_attention_mixer(h, W, p, m, eps, positions, kv, bf16):
    """kv: (c, k_rot) of this layer or of the layer it reads."""
    T = h.shape[0]
    H, D, R, E = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, k_rot = kv
    cq = rnd(rms(linear(W[p + "dq"], h, bf16), eps) * W[p + "dq.norm"].to(h.dtype), bf16)
    q = linear(W[p + "uq"], cq, bf16).view(T, H, D + R)
    cos, sin = yarn_angles(positions, m["rot"], h.dtype)
    q_rot = rnd(rotate_half(q[:, :, D:], cos, sin), bf16)
    k_plain = linear(W[p + "uk"], c, bf16).view(T, H, D)
    v = linear(W[p + "uv"], c, bf16).view(T, H, E)
    s = torch.einsum("ihd,jhd->hij", q[:, :, :D], k_plain) + torch.einsum("ihr,jr->hij", q_rot, k_rot)
    s = s * m["scale"]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask, float("-inf"))
    w = torch.softmax(s, dim=-1)
    o = rnd(torch.einsum("hij,jhe->ihe", w, v), bf16).reshape(T, H * E)
    o = o * torch.sigmoid(linear(W[p + "g"], h, bf16))
    return linear(W[p + "o"], o, bf16)


def clamped_gate(g, u, limit):
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1)


def gated_ff(h, W, p, limit, bf16):
    y = rnd(clamped_gate(linear(W[p + "gate"], h, bf16), linear(W[p + "up"], h, bf16), limit), bf16)
    return linear(W[p + "down"], y, bf16)


def route(h, W, p, top):
    """(chosen experts [T, top], their weights): the largest logits, softmax over the chosen only."""
    z = h @ W[p + "router"].to(h.dtype).t() + W[p + "router.b"].to(h.dtype)
    best = torch.topk(z, top, dim=-1)
    return best.indices, torch.softmax(best.values, dim=-1), z


def expert_ff(h, W, p, f, bf16):
    chosen, weights, _ = route(rnd(h, bf16), W, p, f["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            out[t] += w * gated_ff(h[t : t + 1], W, f"{p}e{e}.", f["expert"]["limit"], bf16)[0]
    if f.get("shared"):
        out = out + gated_ff(h, W, p + "shared.", f["shared"]["limit"], bf16)
    return rnd(out, bf16)


def forward(config, W, tokens, bf16=False, dtype=F, layers_out=None):
    """Logits [T, vocab] of one sequence from position 0.  layers_out: a list that receives the stream after every layer."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps, groups = config["norm"]["eps"], config["norm"].get("groups", 1)
    T = len(tokens)
    positions = torch.arange(T)
    x = W["embed"][torch.tensor(tokens)]
    streams = [x]
    kept = {}
    for i, layer in enumerate(config["layers"]):
        p, m, f = f"l{i}.", layer["mixer"], layer.get("mlp")
        h = token_shift(grouped_rms_norm(x, W[p + "norm1"], eps, groups), W[p + "shift"])
        if layer["type"] == "lightning":
            y = lightning_mixer(h, W, p + "mix.", m, eps, bf16)
        elif layer["type"] == "retention":
            y = retention_mixer(h, W, p + "mix.", m, eps, bf16)
        elif layer["type"] == "latent_attention":
            if "kv_from" in m:
                kv = kept[m["kv_from"]]
            else:
                kv = kept[i] = latent_kv(h, W, p + "mix.", m, eps, positions, bf16)
            y = latent_attention_mixer(h, W, p + "mix.", m, eps, positions, kv, bf16)
        else:
            raise ValueError(layer["type"])
        x = x + y
        if f is not None:
            h2 = grouped_rms_norm(x, W[p + "norm2"], eps, groups)
            x = x + (gated_ff(h2, W, p + "mlp.", f["limit"], bf16) if f["kind"] == "dense" else expert_ff(h2, W, p + "mlp.", f, bf16))
        streams.append(x)
        x = sum(W[p + "dwa"][j] * streams[j] for j in range(i + 2))
        if layers_out is not None:
            layers_out.append(x)
    return linear(W["head"], grouped_rms_norm(x, W["final.norm"], eps, groups), bf16).to(torch.float32)


def logits(raw, weights, ids, rounded=False):
    """The plain model's logits [T, vocab] of one sequence (float64 inside); rounded: with bfloat16 activations."""
    return forward(raw, weights, list(ids), bf16=rounded)
