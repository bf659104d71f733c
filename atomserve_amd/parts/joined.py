"""A mixer put together from cores that read the same input.

    proj = h @ in^T                      one product makes what every core needs (its columns side by side)
    act[:, core c's columns] = scales[c] * core_c(proj's columns of c)
    y = act @ out^T                      one product takes them all: the weighted sum of the cores is its own sum

A core has no products of its own: it says how many columns of `proj` it reads (`in_rows`) and how many of `act` it
fills (`out_cols`), declares its small tensors, asks for what it keeps between steps, and computes.  One core alone with
the scale 1 is an ordinary mixer.  Cores here: a grouped-query softmax attention with the options a design may combine
(biases, a norm over the whole of q and of k, a rotation, values mixed with an earlier layer's, an output gate), and a
matrix memory with exponential gates.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.attention import SHORT_ROW, TILE_Q, attend
from atomserve_amd.parts.base import Mixer, PagedCacheRequest, StateCacheRequest, WeightDecl, build, register
from atomserve_amd.parts.recurrent import _step_rows


class SoftmaxCore:
    """Causal grouped-query softmax attention over a paged cache.  Columns read: q [H key_dim], k [G key_dim], v [G
    value_dim] and, with spec.out_gate, the gate's logits [H value_dim]; columns filled: the heads [H value_dim].

    A rotation of pairs "half" is applied as it is; one of pairs "neighbours" is applied as "half" after the rows of
    the q and k projections (with their biases and gains) have been brought into the order evens, then odds, within
    every head's turned coordinates: q . k does not see a permutation that both share, and nothing else reads them."""

    capturable = True

    def __init__(self, spec, env):
        self.spec, self.env = spec, env
        s = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"{s.num_heads} query heads do not divide over {s.num_kv_heads} kv heads")
        if s.value_mix not in ("none", "first", "later"):
            raise ValueError(f"values are mixed as 'none', 'first' or 'later', not {s.value_mix!r}")
        chunk = 4 if env.dtype == torch.float32 else 8
        widest = max(s.key_dim, s.value_dim)
        self.head_width = -(-widest // 32) * 32 if widest > 16 else -(-widest // chunk) * chunk
        if self.head_width > ops.SINGLE_QUERY_MAX_HEAD_DIM:
            raise ValueError(f"heads of {widest} exceed the attention kernels' {ops.SINGLE_QUERY_MAX_HEAD_DIM}")
        self.position = build("position", s.position, env) if s.position is not None else None
        pairs = getattr(self.position, "pairs", None)
        if self.position is not None and pairs not in ("half", "neighbours"):
            raise ValueError(f"the kernel turns pairs (i, i + R/2) or neighbours; {s.position.kind!r} declares {pairs!r}")
        if s.position is not None and s.position.rotary_dim > s.key_dim:
            raise ValueError(f"{s.position.rotary_dim} turned coordinates in a head of {s.key_dim}")
        H, G, D, E = s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim
        self.q_off, self.k_off, self.v_off, self.gate_off = 0, H * D, H * D + G * D, H * D + G * D + G * E
        self.in_rows = self.gate_off + (H * E if s.out_gate else 0)
        self.out_cols = H * E
        self.biases = self.gains = None
        self.lam = 0.0

    @property
    def is_capturable(self) -> bool:
        return self.position is None or self.position.capturable

    def weight_decls(self) -> dict:
        s, decls = self.spec, {}
        H, G, D, E = s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim
        if s.bias:
            decls.update({"q_bias": WeightDecl((H * D,), "vector"), "k_bias": WeightDecl((G * D,), "vector"),
                          "v_bias": WeightDecl((G * E,), "vector")})  # fmt: skip
        if s.whole_norm_eps > 0:
            decls.update({"q_norm": WeightDecl((H * D,), "vector"), "k_norm": WeightDecl((G * D,), "vector")})
        if s.value_mix == "later":
            decls["value_mix"] = WeightDecl((), "vector")
        return decls

    def row_order(self):
        """The order into which the rows of this core's share of the input matrix are brought (None: as they are)."""
        s = self.spec
        if self.position is None or self.position.pairs != "neighbours":
            return None
        R, D = s.position.rotary_dim, s.key_dim
        head = list(range(0, R, 2)) + list(range(1, R, 2)) + list(range(R, D))
        order = [h * D + d for h in range(s.num_heads + s.num_kv_heads) for d in head]  # q heads, then k heads
        return torch.tensor(order + list(range(len(order), self.in_rows)), dtype=torch.long)

    def bind(self, tensors: dict) -> None:
        s = self.spec
        f32 = {name: t.float().contiguous() for name, t in tensors.items()}  # exact: what a file holds in 16 bits widens
        order = self.row_order()
        nq = s.num_heads * s.key_dim

        def ordered(t, first):  # a vector over q's (first = 0) or k's (first = nq) rows, in the order of the rows
            if order is None:
                return t
            picked = order[first : first + t.shape[0]].to(t.device) - first
            return t[picked].contiguous()

        if s.bias:
            self.biases = (ordered(f32["q_bias"], 0), ordered(f32["k_bias"], nq), f32["v_bias"])
        if s.whole_norm_eps > 0:
            self.gains = (ordered(f32["q_norm"], 0), ordered(f32["k_norm"], nq))
        if s.value_mix == "later":
            self.lam = float(f32["value_mix"])

    def cache_request(self) -> dict:
        return {"pages": PagedCacheRequest(self.spec.num_kv_heads, self.head_width, 0)}

    def run(self, proj, off, act, out_off, scale, step, cache) -> None:
        s, env = self.spec, self.env
        T, dev = proj.shape[0], proj.device
        H, G, Dp = s.num_heads, s.num_kv_heads, self.head_width
        pages = cache["pages"]
        cos_sin = self.position.prepare(step) if self.position is not None else None
        v_keep, v_mode = None, "none"
        if s.value_mix == "first":
            v_keep = step.shared[("values", s.value_mix_key)] = torch.empty((T, G * s.value_dim), dtype=torch.float32, device=dev)
            v_mode = "keep"
        elif s.value_mix == "later":
            v_keep, v_mode = step.shared.get(("values", s.value_mix_key)), "mix"
            if v_keep is None or v_keep.shape != (T, G * s.value_dim):
                raise ValueError(f"no layer before this one kept values of this shape under {s.value_mix_key!r}")
        q = torch.empty((T, H, Dp), dtype=env.dtype, device=dev)
        ops.whole_norm_store(proj, off + self.q_off, off + self.k_off, off + self.v_off, H, G, s.key_dim, s.value_dim,
                             pages.slots, q, pages.k_pages, pages.v_pages, store_kv=pages.writes, biases=self.biases,
                             gains=self.gains, eps=s.whole_norm_eps, cos_sin=cos_sin, v_keep=v_keep, v_mode=v_mode,
                             lam=self.lam)  # fmt: skip
        if not s.out_gate and scale == 1.0 and Dp == s.value_dim and out_off == 0 and act.shape[1] == self.out_cols:
            # the core alone, its heads as wide as they are laid out: the attention writes the output product's input itself
            attend(q, act.view(T, H, Dp), step, pages, s.scale, 0, (SHORT_ROW, TILE_Q))
            return
        heads = torch.empty((T, H, Dp), dtype=env.dtype, device=dev)
        attend(q, heads, step, pages, s.scale, 0, (SHORT_ROW, TILE_Q))
        ops.sigmoid_gate_heads(heads, s.value_dim, proj if s.out_gate else None, off + self.gate_off, scale, act, out_off)


class MatrixMemoryCore:
    """A matrix memory with exponential gates (`MatrixMemorySpec`).  Columns read: q, k [H key_dim], v [H value_dim], the
    output gate's logits [H value_dim], the input and forget gates' logits [H] each; columns filled: [H value_dim].
    Kept per request, in fp32: the state [H, key_dim, value_dim], the normaliser [H, key_dim], the running maximum [H]."""

    capturable = True
    is_capturable = True
    position = None

    def __init__(self, spec, env):
        self.spec, self.env = spec, env
        s = spec
        if min(s.num_heads, s.key_dim, s.value_dim) < 1 or s.key_dim > ops.MEMORY_MAX_KEY_DIM:
            raise ValueError(f"a matrix memory's sizes are positive, its keys at most {ops.MEMORY_MAX_KEY_DIM} wide")
        if not s.gate_cap > 0:
            raise ValueError("the cap of the gates' logits is positive")
        HD, HE = s.num_heads * s.key_dim, s.num_heads * s.value_dim
        self.q_off, self.k_off, self.v_off, self.gate_off = 0, HD, 2 * HD, 2 * HD + HE
        self.i_off, self.f_off = self.gate_off + HE, self.gate_off + HE + s.num_heads
        self.in_rows = self.f_off + s.num_heads
        self.out_cols = HE

    def weight_decls(self) -> dict:
        s = self.spec
        return {"i_bias": WeightDecl((s.num_heads,), "vector"), "f_bias": WeightDecl((s.num_heads,), "vector"),
                "out_norm": WeightDecl((s.num_heads * s.value_dim,), "vector")}  # fmt: skip

    def row_order(self):
        return None

    def bind(self, tensors: dict) -> None:
        s = self.spec
        self.i_bias, self.f_bias = tensors["i_bias"].float().contiguous(), tensors["f_bias"].float().contiguous()
        self.out_norm = tensors["out_norm"].float().view(s.num_heads, s.value_dim).contiguous()

    def cache_request(self) -> dict:
        s = self.spec
        return {"state": StateCacheRequest((s.num_heads, s.key_dim, s.value_dim), torch.float32),
                "normaliser": StateCacheRequest((s.num_heads, s.key_dim), torch.float32),
                "maximum": StateCacheRequest((s.num_heads,), torch.float32)}  # fmt: skip

    def run(self, proj, off, act, out_off, scale, step, cache) -> None:
        s = self.spec
        T, dev = proj.shape[0], proj.device
        H, D, E = s.num_heads, s.key_dim, s.value_dim
        qkv = torch.empty((T, 2 * H * D + H * E), dtype=torch.float32, device=dev)
        i_log = torch.empty((T, H), dtype=torch.float32, device=dev)
        f_log = torch.empty((T, H), dtype=torch.float32, device=dev)
        ops.memory_prepare(proj, off + self.q_off, off + self.k_off, off + self.v_off, off + self.i_off, off + self.f_off,
                           H, D, E, self.i_bias, self.f_bias, s.gate_cap, qkv, i_log, f_log)  # fmt: skip
        state = cache["state"]
        o = torch.empty((T, H, E), dtype=torch.float32, device=dev)
        ops.memory_scan(qkv, H, D, E, i_log, f_log, state.state, cache["normaliser"].state, cache["maximum"].state,
                        _step_rows(step), o, writes=state.writes)  # fmt: skip
        ops.delta_finish(o, self.out_norm, s.out_norm_eps, proj, off + self.gate_off, act, gate="sigmoid", scale=scale,
                         out_off=out_off)  # fmt: skip


CORES = {"softmax_core": SoftmaxCore, "matrix_memory": MatrixMemoryCore}


class JoinedMixer(Mixer):
    """sum_c scales[c] * core_c(h) through one input and one output product (`JoinedMixerSpec`).  The input matrix is the
    cores' projections stacked along the rows in the cores' order; the output matrix, stored transposed as `out_t` so
    that a checkpoint's per-core matrices stack along its rows, takes the cores' results side by side.  A core's small
    tensors are declared as `c<index>.<name>`, and what it keeps between steps is asked for as `<index>.<name>`."""

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if not spec.cores or len(spec.cores) != len(spec.scales):
            raise ValueError("a joined mixer has at least one core and a scale for each")
        unknown = [c.kind for c in spec.cores if c.kind not in CORES]
        if unknown:
            raise ValueError(f"no core of kind {unknown[0]!r}; there are {sorted(CORES)}")
        self.cores = [CORES[c.kind](c, env) for c in spec.cores]
        self.in_offs, self.out_offs, at_in, at_out = [], [], 0, 0
        for core in self.cores:
            self.in_offs.append(at_in)
            self.out_offs.append(at_out)
            at_in, at_out = at_in + core.in_rows, at_out + core.out_cols
        self.in_rows, self.out_cols = at_in, at_out

    @property
    def capturable(self) -> bool:
        return all(core.is_capturable for core in self.cores)

    def weight_decls(self) -> dict:
        s = self.spec
        decls = {"in.weight": WeightDecl((self.in_rows, s.hidden_size)), "out_t.weight": WeightDecl((self.out_cols, s.hidden_size))}
        for c, core in enumerate(self.cores):
            for name, decl in core.weight_decls().items():
                decls[f"c{c}.{name}"] = decl
        return decls

    def bind(self, tensors: dict) -> None:
        w_in = tensors["in.weight"]
        for c, core in enumerate(self.cores):
            prefix = f"c{c}."
            core.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})
            order = core.row_order()
            if order is not None:
                rows = slice(self.in_offs[c], self.in_offs[c] + core.in_rows)
                w_in[rows] = w_in[rows][order.to(w_in.device)]
        self.in_weight = w_in
        self.out_weight = tensors["out_t.weight"].t().contiguous()
        self.inp = ops.Streamed(self.in_weight, self.env.stream_copies)
        self.out = ops.Streamed(self.out_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.inp, self.out]

    def cache_request(self):
        asked = {}
        for c, core in enumerate(self.cores):
            for name, req in core.cache_request().items():
                asked[f"{c}.{name}"] = req
        return asked

    def row_split(self):
        return (SHORT_ROW, TILE_Q) if any(isinstance(core, SoftmaxCore) for core in self.cores) else None

    def forward(self, h, step, cache):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        proj = torch.empty((T, self.in_rows), dtype=env.dtype, device=dev)
        ops.gemm(h, self.inp, proj, env.products)
        act = torch.empty((T, self.out_cols), dtype=env.dtype, device=dev)
        for c, core in enumerate(self.cores):
            prefix = f"{c}."
            own = {name[len(prefix):]: view for name, view in cache.items() if name.startswith(prefix)}
            core.run(proj, self.in_offs[c], act, self.out_offs[c], float(s.scales[c]), step, own)
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.gemm(act, self.out, y, env.products)
        return y


register("mixer", "joined", JoinedMixer)
