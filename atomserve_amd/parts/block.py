"""Arrangements: how one layer orders its norms, mixer, feed-forward and residual sums.

"prenorm":    x += mixer(norm(x));  x += ffn(norm(x))   (reference atomserve/model.py:378-382)
"two_norms":  x += mixer(norm1(x)) + ffn(norm2(x)), both parts reading the same x through a norm each
"gated_prenorm": x += m g1(h) * mixer(h), h = norm(x);  x += m g2(h) * ffn(h), h = norm(x), with sigmoid gates g
"depth_prenorm": "prenorm" whose mixer may read a token-shifted norm, and whose result may be averaged with the
              results of all layers before it
"streams_prenorm": "prenorm" over several residual streams that a sublayer reads as one weighted sum and writes
              through a mixing matrix

The residual stream `x` is fp32 in both precisions.  A part's output is not added at
once: it travels as the pending `delta` to the next norm, whose kernel adds it into
`x` and normalises in one pass.  With few rows (decoding) both steps move into the matrix
products around them instead: a part's last product adds into `x` and leaves the next norm
pending (`Norm.absorb`), and the next part's first product finishes it (`PendingNorm`).
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import (
    Arrangement,
    DeltaSum,
    GatedDelta,
    Part,
    PendingNorm,
    StateCacheRequest,
    StreamsDelta,
    WeightDecl,
    build,
    register,
)


class PreNormBlock(Arrangement):
    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = build("norm", spec.ffn_norm, env)
        self.ffn = build("feed_forward", spec.ffn, env)

    def parts(self) -> dict:
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def first_norm(self):
        return self.mixer_norm

    def forward(self, x, delta, step, cache, next_norm=None):
        delta = self.apply(self.mixer_norm, self.mixer, self.ffn_norm, x, delta, step, cache)
        return self.apply(self.ffn_norm, self.ffn, next_norm, x, delta, step)

    @staticmethod
    def apply(norm, part, next_norm, x, delta, *args):
        """part(norm(x + delta)): the part's output still to be added, or the PendingNorm of
        `next_norm` if the part added it itself.  `delta` may be the PendingNorm of `norm`."""
        if isinstance(delta, PendingNorm):
            h = delta if part.takes_pending_norm else delta.rows()
        else:
            h = norm.forward(x, delta)
        if part.adds_to_residual:
            return part.forward(h, *args, residual=x, next_norm=next_norm)
        return part.forward(h, *args)


register("arrangement", "prenorm", PreNormBlock)


class TwoNormsBlock(Arrangement):
    """x += mixer(mixer_norm(x)) + ffn(ffn_norm(x)): the two parts read the same stream, each through a norm of
    its own.  Both outputs travel on as one pending `DeltaSum`; the kernel that starts the next layer adds them
    into the stream (in fp32) and takes both of that layer's norms from one root mean square.  A layer without
    a feed-forward (spec.ffn None) is the mixer alone."""

    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = build("norm", spec.ffn_norm, env)
            self.ffn = build("feed_forward", spec.ffn, env)
        self.shared_kernel = self.ffn is not None and hasattr(self.mixer_norm, "with_sibling") and \
            type(self.mixer_norm) is type(self.ffn_norm) and spec.mixer_norm.eps == spec.ffn_norm.eps  # fmt: skip

    def parts(self) -> dict:
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            parts.update(ffn_norm=self.ffn_norm, ffn=self.ffn)
        return parts

    def first_norm(self):
        return None  # nothing is left pending inside a product for this layer: it takes a sum of outputs

    def forward(self, x, delta, step, cache, next_norm=None):
        if isinstance(delta, PendingNorm):
            raise ValueError("a layer of two norms takes pending outputs, not a norm left pending in a product")
        if self.shared_kernel:
            h1, h2 = self.mixer_norm.with_sibling(self.ffn_norm, x, delta)
        else:
            h1 = self.mixer_norm.forward(x, delta)
            h2 = self.ffn_norm.forward(x) if self.ffn is not None else None
        mixed = self.mixer.forward(h1, step, cache)
        if self.ffn is None:
            return mixed
        return DeltaSum((mixed, self.ffn.forward(h2, step)))


register("arrangement", "two_norms", TwoNormsBlock)


class GatedPreNormBlock(Arrangement):
    """x += m * sigmoid(G h + b) * part(h), h = norm(x), for the mixer and then for the feed-forward (spec.ffn
    None: the mixer alone); m = spec.residual_scale.  The gate reads what the part reads, so its logits are rows
    of the part's own input product (parts built with `out_gate` return a `GatedDelta`); the sigmoid, the
    product with the part's output and the sum into the fp32 stream happen in the kernel of the norm that follows."""

    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = build("norm", spec.ffn_norm, env)
            self.ffn = build("feed_forward", spec.ffn, env)
        for name, part in (("mixer", spec.mixer), ("feed-forward", spec.ffn)):
            if part is not None and not getattr(part, "out_gate", False):
                raise ValueError(f"a layer with gated residual sums needs a {name} that computes its output gate (out_gate)")
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and not norm.takes_gated_delta:
                raise ValueError(f"a norm of kind {norm.spec.kind!r} does not add gated outputs into the stream")

    def parts(self) -> dict:
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            parts.update(ffn_norm=self.ffn_norm, ffn=self.ffn)
        return parts

    def first_norm(self):
        return None  # the layer before hands over its output, not a norm left pending in a product

    def forward(self, x, delta, step, cache, next_norm=None):
        if isinstance(delta, (PendingNorm, DeltaSum)):
            raise ValueError("a layer with gated residual sums takes a pending output, gated or plain")
        m = self.spec.residual_scale
        delta = self.mixer.forward(self.mixer_norm.forward(x, delta), step, cache).scaled(m)
        if self.ffn is None:
            return delta
        return self.ffn.forward(self.ffn_norm.forward(x, delta), step).scaled(m)


register("arrangement", "gated_prenorm", GatedPreNormBlock)


class LayerVectors(Part):
    """The small tensors that a layer owns beside its norms and parts: the token shift's weights [hidden] and the
    depth average's [depth_index + 2]; fp32 once bound."""

    capturable = True

    def weight_decls(self) -> dict:
        s, decls = self.spec, {}
        if s.token_shift:
            decls["shift"] = WeightDecl((s.mixer_norm.size,), role="vector")
        if s.depth_slots:
            decls["depth"] = WeightDecl((s.depth_index + 2,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        super().bind({name: t.float().contiguous() for name, t in tensors.items()})


class DepthPreNormBlock(Arrangement):
    """x += mixer(h), h = norm1(x);  x += ffn(norm2(x))  (spec.ffn None: the mixer alone), with two options.

    spec.token_shift: the mixer reads h_t + (h_(t-1) - h_t) * shift instead of h_t, h_(t-1) the normed row of the
    token before (zeros before a sequence's first token).  A request's last normed row waits in a state slot of the
    layer's own for the request's next row, so a prompt may be cut anywhere.

    spec.depth_slots: with X_0 what the embedding gave and X_(i+1) this layer's result (i = spec.depth_index), the
    stream goes on as sum_(j <= i+1) depth[j] X_j.  The X_j of a step are kept in fp32 in the step's shared
    results; the layer leaves the stream complete (nothing pending), so the next layer's norm adds nothing."""

    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = build("norm", spec.ffn_norm, env)
            self.ffn = build("feed_forward", spec.ffn, env)
        self.vectors = LayerVectors(spec, env)
        if spec.token_shift and not hasattr(self.mixer_norm, "forward_shifted"):
            raise ValueError(f"a norm of kind {spec.mixer_norm.kind!r} has no kernel with a token shift")
        if spec.depth_slots and not 0 <= spec.depth_index < spec.depth_slots - 1:
            raise ValueError(f"layer result {spec.depth_index + 1} does not fit {spec.depth_slots} kept results")

    def parts(self) -> dict:
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            parts.update(ffn_norm=self.ffn_norm, ffn=self.ffn)
        if self.vectors.weight_decls():
            parts["vectors"] = self.vectors
        return parts

    def cache_request(self):
        if self.spec.token_shift:
            return {"shift": StateCacheRequest((self.spec.mixer_norm.size,), torch.float32)}
        return None

    def first_norm(self):
        return None  # nothing is left pending inside a product for this layer

    def forward(self, x, delta, step, cache, next_norm=None, own=None):
        if isinstance(delta, (PendingNorm, DeltaSum, GatedDelta)):
            raise ValueError("a layer of this arrangement takes a plain pending output, or none")
        s = self.spec
        if s.depth_slots and s.depth_index == 0:
            if delta is not None:
                raise ValueError("the first of the layers whose results are averaged starts from a complete stream")
            kept = step.shared["depth_results"] = torch.empty((s.depth_slots, *x.shape), dtype=torch.float32, device=x.device)
            kept[0].copy_(x)
        if s.token_shift:
            if delta is not None:  # the shift's kernel reads neighbouring rows of a complete stream
                self.mixer_norm.forward(x, delta)
            kept_rows = own["shift"]
            rows = (None if step.decode_only else step.tok_row, step.row_first, step.row_len, step.row_start, step.row_slots)
            h = self.mixer_norm.forward_shifted(x, self.vectors.shift, rows, kept_rows.state, writes=kept_rows.writes)
        else:
            h = self.mixer_norm.forward(x, delta)
        delta = self.mixer.forward(h, step, cache)
        if self.ffn is not None:
            delta = self.ffn.forward(self.ffn_norm.forward(x, delta), step)
        if not s.depth_slots:
            return delta
        kept = step.shared.get("depth_results")
        if kept is None or kept.shape[0] != s.depth_slots or kept.shape[1:] != x.shape:
            raise ValueError("the layers whose results are averaged run in order, from the first, within one step")
        ops.depth_average(x, delta, kept, self.vectors.depth, s.depth_index + 1)
        return None


register("arrangement", "depth_prenorm", DepthPreNormBlock)


class StreamCoefficients(Part):
    """What the sublayers of a layer over several streams read and write them with: per sublayer q (1: mixer, 2:
    feed-forward) `hc<q>.in` [S], `hc<q>.mix` [S, S] (indexed [from, to]) and `hc<q>.out` [S]; fp32 once bound."""

    capturable = True

    def weight_decls(self) -> dict:
        s, decls = self.spec, {}
        for q in (1, 2) if s.ffn is not None else (1,):
            decls[f"hc{q}.in"] = WeightDecl((s.streams,), role="vector")
            decls[f"hc{q}.mix"] = WeightDecl((s.streams, s.streams), role="vector")
            decls[f"hc{q}.out"] = WeightDecl((s.streams,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        super().bind({name: t.float().contiguous() for name, t in tensors.items()})


class StreamsPreNormBlock(Arrangement):
    """Pre-norm sublayers over S residual streams x_1 .. x_S (fp32 [T, S, hidden], kept in the step's shared results):

        u = sum_s a[s] x_s;  y = part(norm(u));  x_r <- sum_s M[s, r] x_s + m c[r] y      (m = spec.residual_scale)

    with a, M, c of the sublayer's own.  The layer marked `streams_first` makes the streams, all equal to the stream it
    is handed; the one marked `streams_last` leaves their sum as that stream again.  A part's output is not written at
    once: it travels as a pending `StreamsDelta` to the kernel that reads the streams for the next part
    (`ops.streams_step`), which writes, reads and norms in one pass.  spec.streams 0: one stream and a = M = c = 1, the
    plain `x += m y`."""

    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = build("norm", spec.ffn_norm, env)
            self.ffn = build("feed_forward", spec.ffn, env)
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and norm.spec.kind != "rmsnorm":
                raise ValueError(f"the kernel that reads several streams norms by 'rmsnorm', not by {norm.spec.kind!r}")
        if not 0 <= spec.streams <= ops.STREAMS_MAX:
            raise ValueError(f"0 to {ops.STREAMS_MAX} streams, not {spec.streams}")
        self.coefficients = StreamCoefficients(spec, env) if spec.streams else None
        self.ones = None

    def parts(self) -> dict:
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            parts.update(ffn_norm=self.ffn_norm, ffn=self.ffn)
        if self.coefficients is not None:
            parts["streams"] = self.coefficients
        return parts

    def first_norm(self):
        return None  # nothing is left pending inside a product for this layer

    def _coefficients(self, q: int, device):
        """(in, mix, out) of sublayer q."""
        c = self.coefficients
        if c is None:
            if self.ones is None:
                self.ones = torch.ones(1, dtype=torch.float32, device=device)
            return self.ones, None, self.ones
        return getattr(c, f"hc{q}_in"), getattr(c, f"hc{q}_mix"), getattr(c, f"hc{q}_out")

    def forward(self, x, delta, step, cache, next_norm=None):
        s, env = self.spec, self.env
        T, n = x.shape
        first = None
        if s.streams_first:
            if delta is not None:
                raise ValueError("the first of the layers over several streams starts from a complete stream")
            xs = step.shared["streams"] = torch.empty((T, max(s.streams, 1), n), dtype=torch.float32, device=x.device)
            first = x
        else:
            xs = step.shared.get("streams")
            if xs is None or xs.shape != (T, max(s.streams, 1), n) or not isinstance(delta, StreamsDelta):
                raise ValueError("the layers over several streams run in order, from the first, within one step")
        pending = delta
        for q, norm, part in ((1, self.mixer_norm, self.mixer), (2, self.ffn_norm, self.ffn)):
            if part is None:
                continue
            a, mix, c = self._coefficients(q, x.device)
            h = torch.empty((T, n), dtype=env.dtype, device=x.device)
            if pending is None:
                ops.streams_step(xs, first=first, in_c=a, gain=norm.gain_f32, eps=norm.spec.eps, normed=h)
            else:
                ops.streams_step(xs, y=pending.y, mix=pending.mix, out_c=pending.out, mult=pending.mult, in_c=a,
                                 gain=norm.gain_f32, eps=norm.spec.eps, normed=h)  # fmt: skip
            y = part.forward(h, step, cache) if q == 1 else part.forward(h, step)
            if not isinstance(y, torch.Tensor):
                raise ValueError("a part of a layer over several streams returns its output, nothing pending of its own")
            pending = StreamsDelta(y, mix, c, s.residual_scale)
        if not s.streams_last:
            return pending
        ops.streams_step(xs, y=pending.y, mix=pending.mix, out_c=pending.out, mult=pending.mult, total=x)
        return None


register("arrangement", "streams_prenorm", StreamsPreNormBlock)
