"""Natatar written plainly: one function per mechanism, a whole sequence at a time, token by token where a state
is carried.  It shares nothing with the package: tensors come as a dict of checkpoint names, the configuration as
the parsed config.json.  `bf16=True` rounds to bfloat16 at the places where an engine that stores bfloat16 numbers
must (the products' inputs and outputs, what a cache holds); how far that moves the plain model's own logits is the
yardstick of the bfloat16 tests.

    streams x_1 .. x_s, all what the embedding gave; per sublayer (mixer, then feed-forward):
        u = sum_s a[s] x_s;  y = part(norm(u));  x_t <- sum_s M[s, t] x_s + m c[t] y
    at the end x = sum_s x_s, the last norm, the embedding table as the head.
"""

import math

import torch

F = torch.float64


def rnd(t, bf16):
    return t.to(torch.bfloat16).to(t.dtype) if bf16 else t


def linear(w, x, bf16, bias=None):
    """W x (+ b) for every row of x, the result rounded as a bfloat16 product's would be."""
    y = rnd(x, bf16) @ w.to(x.dtype).t()
    if bias is not None:
        y = y + bias.to(x.dtype)
    return rnd(y, bf16)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """The layers' norm: the gain is stored around zero and one is added to it."""
    return rms(x, eps) * (1.0 + w.to(x.dtype))


def plain_norm(x, w, eps):
    return rms(x, eps) * w.to(x.dtype)


# ---- several streams ----------------------------------------------------------------------------------------------
def streams_read(xs, a):
    """xs [s, T, n], a [s] -> sum_s a[s] xs[s]"""
    return torch.einsum("s,stn->tn", a.to(xs.dtype), xs)


def streams_write(xs, M, c, m, y):
    """xs[t] <- sum_s M[s, t] xs[s] + m c[t] y, all streams at once from the old ones."""
    return torch.einsum("sr,stn->rtn", M.to(xs.dtype), xs) + m * c.to(xs.dtype).view(-1, 1, 1) * y.unsqueeze(0)


# ---- softmax attention --------------------------------------------------------------------------------------------
def causal_attention(q, k, v, scale):
    """q [T, H, D], k [T, G, D], v [T, G, E]: head h reads kv head h // (H / G); position i sees j <= i."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].t()) * scale
        s = s.masked_fill(~mask, -math.inf)
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def stretched_frequencies(rot):
    """The frequencies of the pairs of a rotation, stretched for long contexts where rot names a scaling; and the
    factor on cosines and sines."""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor = float(sc["factor"])

    def dim_of(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(sc["fast"])), 0)
    hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_neighbours(x, positions, rot):
    """x [T, heads, D]: of every head's first rot.dims coordinates the pair (2i, 2i + 1) turns by position * f_i."""
    f, mag = stretched_frequencies(rot)
    ang = positions.to(F).unsqueeze(1) * f.unsqueeze(0)  # [T, dims / 2]
    cos, sin = (torch.cos(ang) * mag).to(x.dtype).unsqueeze(1), (torch.sin(ang) * mag).to(x.dtype).unsqueeze(1)
    R = rot["dims"]
    a, b = x[..., 0:R:2], x[..., 1:R:2]
    out = x.clone()
    out[..., 0:R:2] = a * cos - b * sin
    out[..., 1:R:2] = b * cos + a * sin
    return out


def attention_mixer(h, W, p, m, eps, bf16, shared):
    """Biased projections, a norm over the whole of q and of k, no rotation, values mixed with those of the first
    layer that says v_mix (kept in `shared`)."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(W[p + "q"], h, bf16, W[p + "q.b"])
    k = linear(W[p + "k"], h, bf16, W[p + "k.b"])
    v = linear(W[p + "v"], h, bf16, W[p + "v.b"])
    q = rnd(plain_norm(q, W[p + "q.norm"], eps), bf16).view(T, H, D)
    k = rnd(plain_norm(k, W[p + "k.norm"], eps), bf16).view(T, G, D)
    if m.get("v_mix"):
        if "v_first" not in shared:
            shared["v_first"] = v
        else:
            lam = W[p + "vmix"].to(h.dtype)
            v = rnd((1.0 - lam) * v + lam * shared["v_first"], bf16)
    o = rnd(causal_attention(q, k, v.view(T, G, E), m["scale"]), bf16).reshape(T, H * E)
    return linear(W[p + "o"], o, bf16)


def gated_rotary_attention(h, W, p, m, positions, bf16):
    """The left half of the parallel mixer: no biases, neighbouring pairs turned, heads times a sigmoid gate."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(W[p + "q"], h, bf16).view(T, H, D)
    k = linear(W[p + "k"], h, bf16).view(T, G, D)
    v = linear(W[p + "v"], h, bf16).view(T, G, E)
    if m.get("rot"):
        q, k = rnd(rotate_neighbours(q, positions, m["rot"]), bf16), rnd(rotate_neighbours(k, positions, m["rot"]), bf16)
    o = rnd(causal_attention(q, k, v, m["scale"]), bf16).reshape(T, H * E)
    o = o * torch.sigmoid(linear(W[p + "g"], h, bf16))
    return linear(W[p + "o"], o, bf16)


# ---- matrix memory with exponential gates ---------------------------------------------------------------------------
def capped(z, cap):
    return cap * torch.tanh(z / cap)


def matrix_memory_scan(q, k, v, i_log, f_log):
    """Per head: m_t = max(f + m_(t-1), i) with m_0 = 0; S_t = e^(f + m_(t-1) - m_t) S_(t-1) + e^(i - m_t) k v^T, n_t the
    same with k alone; o = S_t^T q / (max(|n_t . q|, e^(-m_t)) + 1e-6).  q, k [T, H, D], v [T, H, E], gates [T, H]."""
    T, H, D = q.shape
    E = v.shape[2]
    S = torch.zeros(H, D, E, dtype=q.dtype)
    n = torch.zeros(H, D, dtype=q.dtype)
    m = torch.zeros(H, dtype=q.dtype)
    out = []
    for t in range(T):
        m_new = torch.maximum(f_log[t] + m, i_log[t])
        keep, take = torch.exp(f_log[t] + m - m_new), torch.exp(i_log[t] - m_new)
        S = keep.view(H, 1, 1) * S + take.view(H, 1, 1) * k[t].unsqueeze(2) * v[t].unsqueeze(1)
        n = keep.view(H, 1) * n + take.view(H, 1) * k[t]
        m = m_new
        num = torch.einsum("hde,hd->he", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out.append(num / den.unsqueeze(1))
    return torch.stack(out)


def matrix_memory_mixer(h, W, p, m, eps, bf16):
    T = h.shape[0]
    H, D, E = m["heads"], m["dim"], m["vdim"]
    cap = float(m["gate_cap"])
    q = linear(W[p + "q"], h, bf16).view(T, H, D) * D**-0.5
    k = linear(W[p + "k"], h, bf16).view(T, H, D)
    v = linear(W[p + "v"], h, bf16).view(T, H, E)
    i_log = capped(linear(W[p + "i"], h, bf16, W[p + "i.b"]), cap)
    f_log = torch.nn.functional.logsigmoid(capped(linear(W[p + "f"], h, bf16, W[p + "f.b"]), cap))
    o = rms(matrix_memory_scan(q, k, v, i_log, f_log), eps).reshape(T, H * E)
    o = o * W[p + "norm"].to(h.dtype) * torch.sigmoid(linear(W[p + "g"], h, bf16))
    return linear(W[p + "o"], o, bf16)


def parallel_mixer(h, W, p, m, positions, eps, bf16):
    left = gated_rotary_attention(h, W, p + "left.", m["left"], positions, bf16)
    right = matrix_memory_mixer(h, W, p + "right.", m["right"], eps, bf16)
    return m["left_scale"] * left + m["right_scale"] * right


# ---- delta rule with a decay per key channel -------------------------------------------------------------------------
def short_conv(x, w):
    """x [T, C], w [C, taps] (the last column is the current token's), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    out = torch.zeros_like(x)
    for i in range(taps):
        out = out + padded[i : i + T] * w[:, i].to(x.dtype)
    return out


def unit(x):
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)


def channel_delta_scan(q, k, v, beta, g):
    """Per head: S <- g * S (g per key channel, on the rows of S); u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    q, k [T, H, D], v [T, H, E], beta [T, H], g [T, H, D]."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[2], dtype=q.dtype)
    out = []
    for t in range(T):
        S = g[t].unsqueeze(2) * S
        u = beta[t].unsqueeze(1) * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
        S = S + k[t].unsqueeze(2) * u.unsqueeze(1)
        out.append(torch.einsum("hde,hd->he", S, q[t]))
    return torch.stack(out)


def channel_delta_mixer(h, W, p, m, eps, bf16):
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu

    def conv_silu(name):
        z = linear(W[p + name], h, bf16)
        if p + name + ".conv" in W:
            z = short_conv(z, W[p + name + ".conv"])
        return rnd(silu(z), bf16)

    q = unit(conv_silu("q").view(T, G, D)) * D**-0.5
    k = unit(conv_silu("k").view(T, G, D))
    v = conv_silu("v").view(T, H, E)
    rep = H // G
    q, k = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(linear(W[p + "b"], h, bf16))
    step = linear(W[p + "a2"], linear(W[p + "a1"], h, bf16), bf16) + W[p + "dt_bias"].to(h.dtype)
    rate = torch.exp(W[p + "A_log"].to(h.dtype)).view(1, H, 1)
    g = torch.exp(-rate * torch.nn.functional.softplus(step).view(T, H, D))
    o = rms(channel_delta_scan(q, k, v, beta, g), eps) * W[p + "norm"].to(h.dtype)
    gate = torch.sigmoid(linear(W[p + "g2"], linear(W[p + "g1"], h, bf16), bf16))
    return linear(W[p + "o"], o.reshape(T, H * E) * gate, bf16)


# ---- experts ------------------------------------------------------------------------------------------------------------
def grouped_choice(scores, top, count, keep):
    """Which `top` experts every row takes: only experts of the `keep` groups (of `count` equal groups of neighbours)
    whose largest score is largest can be chosen.  Of equal scores the lower number comes first."""
    T, n = scores.shape
    allowed = torch.ones(T, n, dtype=torch.bool)
    if count > 1 and keep < count:
        best = scores.view(T, count, n // count).max(dim=-1).values
        order = torch.sort(best, dim=-1, descending=True, stable=True).indices[:, :keep]
        groups = torch.zeros(T, count, dtype=torch.bool)
        groups.scatter_(1, order, True)
        allowed = groups.repeat_interleave(n // count, dim=1)
    masked = scores.masked_fill(~allowed, -math.inf)
    return torch.sort(masked, dim=-1, descending=True, stable=True).indices[:, :top]


def experts(h, W, p, f, bf16):
    r = f["router"]
    n, top = r["experts"], r["top"]
    z = rnd(h, bf16) @ W[p + "router"].to(h.dtype).t()
    s = torch.softmax(z, dim=-1)
    groups = r.get("groups") or {"count": 1, "keep": 1}
    chosen = grouped_choice(s, top, groups["count"], groups["keep"])
    out = torch.zeros_like(h)
    silu = torch.nn.functional.silu
    for e in range(n):
        rows = (chosen == e).any(dim=-1).nonzero().flatten()
        if not rows.numel():
            continue
        x = h[rows]
        a = rnd(silu(linear(W[f"{p}e{e}.gate"], x, bf16)) * linear(W[f"{p}e{e}.up"], x, bf16), bf16)
        y = linear(W[f"{p}e{e}.down"], a, bf16)
        out[rows] += (s[rows, e] * float(r.get("scale", 1.0))).unsqueeze(1) * y
    return out


# ---- the model ------------------------------------------------------------------------------------------------------------
def forward(raw, W, tokens, bf16=False, dtype=F, layers_out=None):
    """Logits [T, vocab] of one sequence from position 0.  layers_out: a list that receives the stream (the sum of
    the streams) after every layer."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps, m = raw["norm"]["eps"], float(raw.get("residual_mult", 1.0))
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    positions = torch.arange(T)
    x = W["embed"][tokens] * float((raw.get("embedding") or {}).get("scale", 1.0))
    s = raw.get("streams")
    xs = x.unsqueeze(0).repeat(s or 1, 1, 1)
    shared = {}
    one = torch.ones(1, dtype=dtype)

    def sublayer(xs, q, p, part):
        if s:
            a, M, c = W[f"{p}hc{q}.in"], W[f"{p}hc{q}.mix"], W[f"{p}hc{q}.out"]
        else:
            a, M, c = one, one.view(1, 1), one
        y = part(offset_norm(streams_read(xs, a), W[f"{p}norm{q}"], eps))
        return streams_write(xs, M, c, m, y)

    for i, layer in enumerate(raw["layers"]):
        p, mix = f"l{i}.", layer["mixer"]
        if layer["type"] == "attention":
            part = lambda h: attention_mixer(h, W, p + "mix.", mix, eps, bf16, shared)  # noqa: E731
        elif layer["type"] == "parallel":
            part = lambda h: parallel_mixer(h, W, p + "mix.", mix, positions, eps, bf16)  # noqa: E731
        elif layer["type"] == "channel_delta":
            part = lambda h: channel_delta_mixer(h, W, p + "mix.", mix, eps, bf16)  # noqa: E731
        else:
            raise ValueError(layer["type"])
        xs = sublayer(xs, 1, p, part)
        f = layer.get("mlp")
        if f is not None:
            xs = sublayer(xs, 2, p, lambda h: experts(h, W, p + "mlp.", f, bf16))
        if layers_out is not None:
            layers_out.append(xs.sum(dim=0))
    x = offset_norm(xs.sum(dim=0), W["final.norm"], eps)
    return rnd(x, bf16) @ W["embed"].t()


def logits(raw, W, ids, rounded=False):
    """Logits [T, vocab] in float32: exact (float64 inside), or with bfloat16 activations."""
    return forward(raw, W, ids, bf16=rounded).float()
