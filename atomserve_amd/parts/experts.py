"""Feed-forward layers made of experts: every token runs through a few of several small gated
feed-forwards, down_e(act(gate_e h) * (up_e h)), and their outputs are added with a weight each.

Which experts a token uses is found on the GPU, so a step never waits for the host and a decode step can
be replayed as a graph.  `TableExperts` reads them from a table indexed by the token's id (no router of
its own: every chosen expert weighs 1 / top); `RoutedExperts` scores every expert with a router matrix and
weighs the chosen by their scores; another way of choosing is another `route`.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import FeedForward, GatedDelta, WeightDecl, register


class TableExperts(FeedForward):
    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if spec.activation != "silu":
            raise ValueError(f"activation {spec.activation!r} has no kernel (only 'silu')")
        if not 1 <= spec.top <= spec.num_experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"{spec.top} of {spec.num_experts} experts (at most {ops.MOE_MAX_EXPERTS}) cannot be chosen")

    def weight_decls(self) -> dict:
        s = self.spec
        return {
            "gate.weight": WeightDecl((s.num_experts, s.intermediate_size, s.hidden_size)),
            "up.weight": WeightDecl((s.num_experts, s.intermediate_size, s.hidden_size)),
            "down.weight": WeightDecl((s.num_experts, s.hidden_size, s.intermediate_size)),
            "table": WeightDecl((s.vocab_size, s.top), role="table_int"),
        }

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        # every expert's gate rows, then its up rows: what the first grouped product reads
        self.gate_up_weight = torch.cat([self.gate_weight, self.up_weight], dim=1).contiguous()
        del self.gate_weight, self.up_weight

    def route(self, step):
        """The step's (token, expert) pairs sorted by expert; every layer with the same table object shares it."""
        key = ("table_experts", self.table.data_ptr())
        found = step.shared.get(key)
        if found is None:
            found = step.shared[key] = ops.moe_route_table(step.token_ids, self.table, self.spec.num_experts)
        return found

    def forward(self, h, step):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        route = self.route(step)
        pairs = T * s.top
        act = torch.empty((pairs, s.intermediate_size), dtype=env.dtype, device=dev)
        ops.moe_gemm(h, self.gate_up_weight, route, act, gated=True, per_token=True)
        if s.top == 1:
            y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
            ops.moe_gemm(act, self.down_weight, route, y, gated=False, per_token=False)
            return y
        each = torch.empty((pairs, s.hidden_size), dtype=torch.float32, device=dev)
        ops.moe_gemm(act, self.down_weight, route, each, gated=False, per_token=False)
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.moe_combine(each, s.top, 1.0 / s.top, y)
        return y


register("feed_forward", "table_experts", TableExperts)


class RoutedExperts(FeedForward):
    """Experts without a gate, chosen by a router:

        s = sigmoid(R h) in fp32; a token's `top` experts are those with the largest s, weighing s / (their sum + 1e-20)
        expert e: down_e(relu(up_e h)^2);  with spec.shared_size one more such expert runs for every token and is added

    The shared expert's up rows and, with spec.out_gate, the logits of the output gate are rows of one matrix."""

    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if spec.activation != "relu2":
            raise ValueError(f"activation {spec.activation!r} has no kernel in experts without a gate (only 'relu2')")
        if spec.score != "sigmoid":
            raise ValueError(f"a router scores by 'sigmoid', not by {spec.score!r}")
        if not 1 <= spec.top <= spec.num_experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"{spec.top} of {spec.num_experts} experts (at most {ops.MOE_MAX_EXPERTS}) cannot be chosen")
        self.side_rows = spec.shared_size + (spec.hidden_size if spec.out_gate else 0)

    def weight_decls(self) -> dict:
        s = self.spec
        decls = {
            "router.weight": WeightDecl((s.num_experts, s.hidden_size)),
            "up.weight": WeightDecl((s.num_experts, s.intermediate_size, s.hidden_size)),
            "down.weight": WeightDecl((s.num_experts, s.hidden_size, s.intermediate_size)),
        }
        if self.side_rows:
            decls["side.weight"] = WeightDecl((self.side_rows, s.hidden_size))
        if s.shared_size:
            decls["shared_down.weight"] = WeightDecl((s.hidden_size, s.shared_size))
        if s.out_gate:
            decls["gate_bias"] = WeightDecl((s.hidden_size,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        self.side = self.shared_down = None
        if self.side_rows:
            self.side = ops.Streamed(self.side_weight, self.env.stream_copies)
        if self.spec.shared_size:
            self.shared_down = ops.Streamed(self.shared_down_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [w for w in (self.side, self.shared_down) if w is not None]

    def forward(self, h, step):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        route = ops.moe_route_sigmoid(h, self.router_weight, s.top)
        pairs = T * s.top
        act = torch.empty((pairs, s.intermediate_size), dtype=env.dtype, device=dev)
        ops.moe_gemm(h, self.up_weight, route, act, gated=False, per_token=True, activation=s.activation)
        each = torch.empty((pairs, s.hidden_size), dtype=torch.float32, device=dev)
        ops.moe_gemm(act, self.down_weight, route, each, gated=False, per_token=False)
        side = shared = None
        if self.side is not None:
            side = torch.empty((T, self.side_rows), dtype=env.dtype, device=dev)
            ops.gemm(h, self.side, side, env.products)
        if s.shared_size:
            a = torch.empty((T, s.shared_size), dtype=env.dtype, device=dev)
            ops.relu2(side, 0, a)
            shared = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
            ops.gemm(a, self.shared_down, shared, env.products)
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.moe_combine(each, s.top, 1.0, y, pair_weight=route.pair_weight, add=shared)
        if s.out_gate:
            return GatedDelta(y, side, s.shared_size, self.gate_bias)
        return y


register("feed_forward", "routed_experts", RoutedExperts)


class GatedRoutedExperts(FeedForward):
    """Gated experts chosen by a router with a bias:

        z = R h + b in fp32; a token's `top` experts are those with the largest z, weighing the softmax over those z alone
        (spec.score "softmax_of_chosen"), or those with the largest softmax(z) among the experts of the best groups, weighing
        that softmax times a factor ("softmax", `GatedRoutedExpertsSpec`)
        expert e: down_e(act(gate_e h, up_e h)), act the gated activation of the spec with its limit
        with spec.shared_size one more such expert (with a limit of its own) runs for every token and is added

    The routed experts run through the grouped products, the shared one through the dense ones."""

    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if spec.activation not in ("silu", "clamped_swish"):
            raise ValueError(f"activation {spec.activation!r} has no kernel in gated experts ('silu' or 'clamped_swish')")
        if spec.activation == "clamped_swish" and not (spec.limit > 0 and (not spec.shared_size or spec.shared_limit > 0)):
            raise ValueError("the activation with limits needs positive limits")
        if spec.score not in ops.ROUTER_SCORES:
            raise ValueError(f"a router scores by one of {sorted(ops.ROUTER_SCORES)}, not by {spec.score!r}")
        if not 1 <= spec.top <= spec.num_experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"{spec.top} of {spec.num_experts} experts (at most {ops.MOE_MAX_EXPERTS}) cannot be chosen")

    def weight_decls(self) -> dict:
        s = self.spec
        decls = {
            "router.weight": WeightDecl((s.num_experts, s.hidden_size)),
            "gate.weight": WeightDecl((s.num_experts, s.intermediate_size, s.hidden_size)),
            "up.weight": WeightDecl((s.num_experts, s.intermediate_size, s.hidden_size)),
            "down.weight": WeightDecl((s.num_experts, s.hidden_size, s.intermediate_size)),
        }
        if s.router_bias:
            decls["router.bias"] = WeightDecl((s.num_experts,), role="vector")
        if s.shared_size:
            decls["shared_gate_up.weight"] = WeightDecl((2 * s.shared_size, s.hidden_size))
            decls["shared_down.weight"] = WeightDecl((s.hidden_size, s.shared_size))
        return decls

    def bind(self, tensors: dict) -> None:
        self.router_bias = None
        super().bind(tensors)
        if self.router_bias is not None:
            self.router_bias = self.router_bias.float().contiguous()
        # every expert's gate rows, then its up rows: what the first grouped product reads
        self.gate_up_weight = torch.cat([self.gate_weight, self.up_weight], dim=1).contiguous()
        del self.gate_weight, self.up_weight
        self.shared_gate_up = self.shared_down = None
        if self.spec.shared_size:
            self.shared_gate_up = ops.Streamed(self.shared_gate_up_weight, self.env.stream_copies)
            self.shared_down = ops.Streamed(self.shared_down_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [w for w in (self.shared_gate_up, self.shared_down) if w is not None]

    def forward(self, h, step):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        clamped = s.activation == "clamped_swish"
        route = ops.moe_route_scores(h, self.router_weight, s.top, s.score, self.router_bias, s.groups, s.keep_groups,
                                     s.weight_scale)  # fmt: skip
        pairs = T * s.top
        act = torch.empty((pairs, s.intermediate_size), dtype=env.dtype, device=dev)
        ops.moe_gemm(h, self.gate_up_weight, route, act, gated=True, per_token=True, limit=s.limit if clamped else 0.0)
        each = torch.empty((pairs, s.hidden_size), dtype=torch.float32, device=dev)
        ops.moe_gemm(act, self.down_weight, route, each, gated=False, per_token=False)
        shared = None
        if s.shared_size:
            a = torch.empty((T, s.shared_size), dtype=env.dtype, device=dev)
            if clamped:
                ops.gemm_clamped_gate(h, self.shared_gate_up, a, s.shared_limit, env.products)
            else:
                ops.gemm_silu_mul(h, self.shared_gate_up, a, env.products)
            shared = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
            ops.gemm(a, self.shared_down, shared, env.products)
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.moe_combine(each, s.top, 1.0, y, pair_weight=route.pair_weight, add=shared)
        return y


register("feed_forward", "gated_routed_experts", GatedRoutedExperts)
