"""Mixers that carry a fixed-size state from token to token: the gated delta rule, and a gated
attention side by side with a gated linear recurrence.

Both ask the cache manager for state slots (`StateCacheRequest`): the recurrent state in fp32 and the
last inputs of their short convolutions; the second also for pages of keys and values.  A request's row
that starts at position 0 starts from zero whatever its slot held; a portion of a prompt goes on from the
state the portion before it left, so prompts may be cut anywhere.  Everything that enters a recurrence
(unit norms, decays, gates, the state) is fp32 in both precisions; the matrix products and what they hand
on are in the compute dtype.

One product makes everything a mixer needs of its input (queries, keys, values, gates, step sizes are rows
of one stacked matrix) and one product takes everything it gives back.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.attention import SHORT_ROW, TILE_Q, attend
from atomserve_amd.parts.base import Mixer, PagedCacheRequest, StateCacheRequest, WeightDecl, register


def _step_rows(step):
    """(tok_row, row_first, row_len, row_start, row_slots) of a step; tok_row None in a decode step, where token t is
    row t (the kernels then take the shorter way of rows of one token)."""
    return (None if step.decode_only else step.tok_row, step.row_first, step.row_len, step.row_start, step.row_slots)


class DeltaRule(Mixer):
    """Per head h (keys and queries of head h // (H / G)), token by token:
        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    with q, k, v = silu(conv(W h)), q and k unit vectors (q also times key_dim^(-1/2)), beta = sigmoid(W_b h),
    g = exp(-exp(A_log) softplus(W_a h + dt_bias)); the output is o / rms(o) * weight * silu(W_g h) through W_o."""

    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"{s.num_heads} value heads do not divide over {s.num_kv_heads} key heads")
        if not 1 <= s.conv.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"a short convolution has 1 to {ops.CONV_MAX_TAPS} taps, not {s.conv.taps}")
        qk, v = s.num_kv_heads * s.key_dim, s.num_heads * s.value_dim
        self.channels = 2 * qk + v  # what passes the convolution: q, k, v
        # columns of the input product's result: q, k, v, output gate, beta, step size
        self.gate_off, self.beta_off, self.step_off = self.channels, self.channels + v, self.channels + v + s.num_heads
        self.in_rows = self.step_off + s.num_heads

    def weight_decls(self) -> dict:
        s = self.spec
        return {
            "in.weight": WeightDecl((self.in_rows, s.hidden_size)),
            "conv.weight": WeightDecl((self.channels, s.conv.taps), role="vector"),
            "a_log": WeightDecl((s.num_heads,), role="vector"),
            "dt_bias": WeightDecl((s.num_heads,), role="vector"),
            "out_norm.weight": WeightDecl((s.value_dim,), role="vector"),
            "out.weight": WeightDecl((s.hidden_size, s.num_heads * s.value_dim)),
        }

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        # what the recurrence reads is fp32 (a bfloat16 checkpoint's values widen exactly)
        for name in ("conv_weight", "a_log", "dt_bias", "out_norm_weight"):
            setattr(self, name, getattr(self, name).float().contiguous())
        self.inp = ops.Streamed(self.in_weight, self.env.stream_copies)
        self.out = ops.Streamed(self.out_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.inp, self.out]

    def cache_request(self):
        s = self.spec
        asked = {"state": StateCacheRequest((s.num_heads, s.key_dim, s.value_dim), torch.float32)}
        if s.conv.taps > 1:
            asked["conv"] = StateCacheRequest((s.conv.taps - 1, self.channels), torch.float32)
        return asked

    def forward(self, h, step, cache):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        H, G = s.num_heads, s.num_kv_heads
        proj = torch.empty((T, self.in_rows), dtype=env.dtype, device=dev)
        ops.gemm(h, self.inp, proj, env.products)
        rows = _step_rows(step)
        state = cache["state"]
        history = cache["conv"].state if "conv" in cache else torch.empty((1, 0, self.channels), dtype=torch.float32, device=dev)
        qkv = torch.empty((T, self.channels), dtype=torch.float32, device=dev)
        ops.short_conv(proj, 0, self.conv_weight, history, rows, qkv, silu=True, writes=state.writes)
        beta = torch.empty((T, H), dtype=torch.float32, device=dev)
        decay = torch.empty((T, H), dtype=torch.float32, device=dev)
        ops.delta_prepare(qkv, G, s.key_dim, H, proj, self.beta_off, self.step_off, self.a_log, self.dt_bias, beta, decay)
        o = torch.empty((T, H, s.value_dim), dtype=torch.float32, device=dev)
        ops.delta_scan(qkv, G, s.key_dim, H, s.value_dim, beta, decay, state.state, rows, o, writes=state.writes)
        act = torch.empty((T, H * s.value_dim), dtype=env.dtype, device=dev)
        ops.delta_finish(o, self.out_norm_weight, s.out_norm_eps, proj, self.gate_off, act)
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.gemm(act, self.out, y, env.products)
        return y


class SideBySide(Mixer):
    """left_scale * attention(h) + right_scale * recurrence(h).

    Left: grouped-query softmax attention over a paged cache, per-head RMS norm of queries and keys, no
    rotation, a window, the concatenated heads times sigmoid(W_g h).  Right: y = gelu(W_y h + b), u =
    conv(W_x h + b) + b_conv, gates r, i from block-diagonal matrices on u, a = exp(-c r softplus(lam)),
    S = a S + sqrt(1 - a^2) i u, output S * y.  The two output projections are one product: its input is
    (left_scale * gated heads, right_scale * S y) side by side, its matrix (W_o left, W_o right) likewise.
    Keys and values of different widths share pages of the wider one (the coordinates a head lacks are zero)."""

    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        a, r = spec.left, spec.right
        if a.num_heads % a.num_kv_heads:
            raise ValueError(f"{a.num_heads} query heads do not divide over {a.num_kv_heads} kv heads")
        if r.width % r.blocks:
            raise ValueError(f"{r.width} channels do not divide into {r.blocks} blocks")
        if not 1 <= r.conv.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"a short convolution has 1 to {ops.CONV_MAX_TAPS} taps, not {r.conv.taps}")
        if a.qk_norm is not None and (a.qk_norm.kind != "rmsnorm" or a.qk_norm.size != a.key_dim):
            raise ValueError("queries and keys are normed per head by an 'rmsnorm' of their width")
        chunk = 4 if env.dtype == torch.float32 else 8
        widest = max(a.key_dim, a.value_dim)
        self.head_width = -(-widest // 32) * 32 if widest > 16 else -(-widest // chunk) * chunk
        if self.head_width > ops.SINGLE_QUERY_MAX_HEAD_DIM:
            raise ValueError(f"heads of {widest} exceed the attention kernels' {ops.SINGLE_QUERY_MAX_HEAD_DIM}")
        H, G = a.num_heads, a.num_kv_heads
        self.q_off, self.k_off = 0, H * a.key_dim
        self.v_off = self.k_off + G * a.key_dim
        self.gate_off = self.v_off + G * a.value_dim
        self.y_off = self.gate_off + H * a.value_dim
        self.x_off = self.y_off + r.width
        self.in_rows = self.x_off + r.width
        self.out_cols = H * a.value_dim + r.width

    def weight_decls(self) -> dict:
        s, a, r = self.spec, self.spec.left, self.spec.right
        bw = r.width // r.blocks
        decls = {
            "in.weight": WeightDecl((self.in_rows, s.hidden_size)),
            "out_t.weight": WeightDecl((self.out_cols, s.hidden_size)),  # (W_o left, W_o right) side by side, transposed
            "y_bias": WeightDecl((r.width,), role="vector"),
            "x_bias": WeightDecl((r.width,), role="vector"),
            "conv.weight": WeightDecl((r.width, r.conv.taps), role="vector"),
            "conv.bias": WeightDecl((r.width,), role="vector"),
            "gate_a.weight": WeightDecl((r.blocks, bw, bw), role="vector"),
            "gate_a.bias": WeightDecl((r.blocks, bw), role="vector"),
            "gate_i.weight": WeightDecl((r.blocks, bw, bw), role="vector"),
            "gate_i.bias": WeightDecl((r.blocks, bw), role="vector"),
            "lam": WeightDecl((r.width,), role="vector"),
        }
        if a.qk_norm is not None:
            decls["q_norm.weight"] = WeightDecl((a.key_dim,), role="vector")
            decls["k_norm.weight"] = WeightDecl((a.key_dim,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        self.q_norm_weight = self.k_norm_weight = None
        super().bind(tensors)
        for name in ("y_bias", "x_bias", "conv_weight", "conv_bias", "gate_a_weight", "gate_a_bias", "gate_i_weight",
                     "gate_i_bias", "lam"):  # fmt: skip
            setattr(self, name, getattr(self, name).float().contiguous())
        self.out_weight = self.out_t_weight.t().contiguous()
        del self.out_t_weight
        self.inp = ops.Streamed(self.in_weight, self.env.stream_copies)
        self.out = ops.Streamed(self.out_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.inp, self.out]

    def cache_request(self):
        a, r = self.spec.left, self.spec.right
        asked = {
            "pages": PagedCacheRequest(a.num_kv_heads, self.head_width, a.window),
            "state": StateCacheRequest((r.width,), torch.float32),
        }
        if r.conv.taps > 1:
            asked["conv"] = StateCacheRequest((r.conv.taps - 1, r.width), torch.float32)
        return asked

    def row_split(self):
        return (SHORT_ROW, TILE_Q)

    def forward(self, h, step, cache):
        s, a, r, env = self.spec, self.spec.left, self.spec.right, self.env
        T, dev = h.shape[0], h.device
        H, G, Dp = a.num_heads, a.num_kv_heads, self.head_width
        proj = torch.empty((T, self.in_rows), dtype=env.dtype, device=dev)
        ops.gemm(h, self.inp, proj, env.products)
        act = torch.empty((T, self.out_cols), dtype=env.dtype, device=dev)
        # left: norm, store, attend, gate
        pages = cache["pages"]
        q = torch.empty((T, H, Dp), dtype=env.dtype, device=dev)
        eps = a.qk_norm.eps if a.qk_norm is not None else 0.0
        ops.head_norm_store(proj, self.q_off, self.k_off, self.v_off, H, G, a.key_dim, a.value_dim, self.q_norm_weight,
                            self.k_norm_weight, eps, pages.slots, q, pages.k_pages, pages.v_pages, store_kv=pages.writes)  # fmt: skip
        heads = torch.empty((T, H, Dp), dtype=env.dtype, device=dev)
        attend(q, heads, step, pages, a.scale, a.window, self.row_split())
        ops.sigmoid_gate_heads(heads, a.value_dim, proj, self.gate_off, s.left_scale, act, 0)
        # right: convolution, gates, scan
        rows = _step_rows(step)
        state = cache["state"]
        history = cache["conv"].state if "conv" in cache else torch.empty((1, 0, r.width), dtype=torch.float32, device=dev)
        u = torch.empty((T, r.width), dtype=torch.float32, device=dev)
        ops.short_conv(proj, self.x_off, self.conv_weight, history, rows, u, in_bias=self.x_bias, bias=self.conv_bias,
                       writes=state.writes)  # fmt: skip
        decay = torch.empty((T, r.width), dtype=torch.float32, device=dev)
        fresh = torch.empty((T, r.width), dtype=torch.float32, device=dev)
        ops.rglru_gates(u, self.gate_a_weight, self.gate_a_bias, self.gate_i_weight, self.gate_i_bias, self.lam,
                        r.decay_scale, decay, fresh)  # fmt: skip
        ops.rglru_scan(decay, fresh, proj, self.y_off, self.y_bias, s.right_scale, state.state, rows, act,
                       H * a.value_dim, writes=state.writes)  # fmt: skip
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.gemm(act, self.out, y, env.products)
        return y


class ChannelDeltaRule(Mixer):
    """The gated delta rule with a decay per head and key channel (`ChannelDeltaRuleSpec`), per head h:
        S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    q, k, v = silu(conv(W h)), q and k unit vectors (q also times key_dim^(-1/2)), beta = sigmoid(W_b h),
    g = exp(-exp(A_log[h]) softplus(W_a2 (W_a1 h) + dt_bias)) laid out heads x key_dim; the output is
    o / rms(o) * weight * sigmoid(W_g2 (W_g1 h)) through W_o.  Three products read: `in` (q, k, v, beta), `low` (the first
    steps W_a1 and W_g1 stacked) and `expand`, which is W_a2 and W_g2 on the diagonal of one matrix, so that the two
    second steps are one product of `low`'s result."""

    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"{s.num_heads} value heads do not divide over {s.num_kv_heads} key heads")
        if not 1 <= s.conv.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"a short convolution has 1 to {ops.CONV_MAX_TAPS} taps, not {s.conv.taps}")
        if s.decay_rank < 1 or s.gate_rank < 1:
            raise ValueError("the two-step projections of the decay and of the output gate have ranks of at least 1")
        qk, v = s.num_kv_heads * s.key_dim, s.num_heads * s.value_dim
        self.channels = 2 * qk + v  # what passes the convolution: q, k, v
        self.beta_off = self.channels
        self.in_rows = self.beta_off + s.num_heads
        self.step_cols = s.num_heads * s.key_dim  # columns of the expanded product: step sizes, then the gate
        self.wide_cols = self.step_cols + v

    def weight_decls(self) -> dict:
        s = self.spec
        return {
            "in.weight": WeightDecl((self.in_rows, s.hidden_size)),
            "low.weight": WeightDecl((s.decay_rank + s.gate_rank, s.hidden_size)),
            "decay_up.weight": WeightDecl((self.step_cols, s.decay_rank)),
            "gate_up.weight": WeightDecl((s.num_heads * s.value_dim, s.gate_rank)),
            "conv.weight": WeightDecl((self.channels, s.conv.taps), role="vector"),
            "a_log": WeightDecl((s.num_heads,), role="vector"),
            "dt_bias": WeightDecl((self.step_cols,), role="vector"),
            "out_norm.weight": WeightDecl((s.value_dim,), role="vector"),
            "out.weight": WeightDecl((s.hidden_size, s.num_heads * s.value_dim)),
        }

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        s = self.spec
        for name in ("conv_weight", "a_log", "dt_bias", "out_norm_weight"):
            setattr(self, name, getattr(self, name).float().contiguous())
        expand = torch.zeros((self.wide_cols, s.decay_rank + s.gate_rank), dtype=self.in_weight.dtype, device=self.in_weight.device)
        expand[: self.step_cols, : s.decay_rank] = self.decay_up_weight
        expand[self.step_cols :, s.decay_rank :] = self.gate_up_weight
        del self.decay_up_weight, self.gate_up_weight
        self.inp = ops.Streamed(self.in_weight, self.env.stream_copies)
        self.low = ops.Streamed(self.low_weight, self.env.stream_copies)
        self.expand = ops.Streamed(expand, self.env.stream_copies)
        self.out = ops.Streamed(self.out_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.inp, self.low, self.expand, self.out]

    def cache_request(self):
        s = self.spec
        asked = {"state": StateCacheRequest((s.num_heads, s.key_dim, s.value_dim), torch.float32)}
        if s.conv.taps > 1:
            asked["conv"] = StateCacheRequest((s.conv.taps - 1, self.channels), torch.float32)
        return asked

    def forward(self, h, step, cache):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        H, G = s.num_heads, s.num_kv_heads
        proj = torch.empty((T, self.in_rows), dtype=env.dtype, device=dev)
        ops.gemm(h, self.inp, proj, env.products)
        low = torch.empty((T, s.decay_rank + s.gate_rank), dtype=env.dtype, device=dev)
        ops.gemm(h, self.low, low, env.products)
        wide = torch.empty((T, self.wide_cols), dtype=env.dtype, device=dev)
        ops.gemm(low, self.expand, wide, env.products)
        rows = _step_rows(step)
        state = cache["state"]
        history = cache["conv"].state if "conv" in cache else torch.empty((1, 0, self.channels), dtype=torch.float32, device=dev)
        qkv = torch.empty((T, self.channels), dtype=torch.float32, device=dev)
        ops.short_conv(proj, 0, self.conv_weight, history, rows, qkv, silu=True, writes=state.writes)
        beta = torch.empty((T, H), dtype=torch.float32, device=dev)
        chan = torch.empty((T, H, s.key_dim), dtype=torch.float32, device=dev)
        ops.delta_prepare_channels(qkv, G, s.key_dim, H, proj, self.beta_off, wide, 0, self.a_log, self.dt_bias, beta, chan)
        o = torch.empty((T, H, s.value_dim), dtype=torch.float32, device=dev)
        ops.delta_scan_channels(qkv, G, s.key_dim, H, s.value_dim, beta, chan, state.state, rows, o, writes=state.writes)
        act = torch.empty((T, H * s.value_dim), dtype=env.dtype, device=dev)
        ops.delta_finish(o, self.out_norm_weight, s.out_norm_eps, wide, self.step_cols, act, gate="sigmoid")
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.gemm(act, self.out, y, env.products)
        return y


register("mixer", "delta_rule", DeltaRule)
register("mixer", "channel_delta_rule", ChannelDeltaRule)
register("mixer", "side_by_side", SideBySide)
