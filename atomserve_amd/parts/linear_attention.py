"""Linear attention with a fixed decay per head: no softmax, no denominator, a state instead of a cache.

    q, k = act(W_q h), act(W_k h) * key_scale   [heads, key_dim];   v = act(W_v h)   [heads, value_dim]
    S_t = decay_h S_(t-1) + k_t v_t^T;   o_t = S_t^T q_t
    out = W_o (norm(o) * gate(W_g h))

`norm` is per head without a gain ("heads") or over the concatenated heads with a gain ("all"); `gate` a sigmoid
or silu.  Two known mixers are instances: one with silu on q, k and v, a norm over all heads and a sigmoid gate,
one without activation, keys times key_dim^(-1/2), a norm per head and a silu gate.

The state [heads, key_dim, value_dim] is fp32 and waits in a slot per request; a row that starts its sequence
starts from zero, a later row goes on where the row before stopped, so a prompt may be cut anywhere.  q, k, v and
the gate are rows of one input matrix.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import Mixer, StateCacheRequest, WeightDecl, register


class DecayAttention(Mixer):
    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if len(s.decay) != s.num_heads:
            raise ValueError(f"{len(s.decay)} decays for {s.num_heads} heads")
        if any(not 0.0 <= float(d) <= 1.0 for d in s.decay):
            raise ValueError("a head's decay lies between 0 and 1")
        if s.activation not in (None, "silu"):
            raise ValueError(f"q, k and v pass no activation or 'silu', not {s.activation!r}")
        if s.out_norm not in ("heads", "all") or s.gate not in ("sigmoid", "silu"):
            raise ValueError(f"out_norm is 'heads' or 'all' and gate 'sigmoid' or 'silu', not {s.out_norm!r}, {s.gate!r}")
        if not 1 <= s.key_dim <= ops.DECAY_SCAN_MAX_DIM:
            raise ValueError(f"keys of {s.key_dim} coordinates exceed the scan's {ops.DECAY_SCAN_MAX_DIM}")
        qk, v = s.num_heads * s.key_dim, s.num_heads * s.value_dim
        self.q_off, self.k_off, self.v_off, self.g_off = 0, qk, 2 * qk, 2 * qk + v
        self.in_rows = 2 * qk + 2 * v
        self.decay = None

    def weight_decls(self) -> dict:
        s = self.spec
        decls = {
            "in.weight": WeightDecl((self.in_rows, s.hidden_size)),
            "out.weight": WeightDecl((s.hidden_size, s.num_heads * s.value_dim)),
        }
        if s.out_norm == "all":
            decls["out_norm.weight"] = WeightDecl((s.num_heads * s.value_dim,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        self.out_norm_weight = None
        super().bind(tensors)
        if self.out_norm_weight is not None:
            self.out_norm_weight = self.out_norm_weight.float().contiguous()
        self.decay = torch.tensor([float(d) for d in self.spec.decay], dtype=torch.float32, device=self.env.device)
        self.inp = ops.Streamed(self.in_weight, self.env.stream_copies)
        self.out = ops.Streamed(self.out_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.inp, self.out]

    def cache_request(self):
        s = self.spec
        return {"state": StateCacheRequest((s.num_heads, s.key_dim, s.value_dim), torch.float32)}

    def forward(self, h, step, cache):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        H, D, E = s.num_heads, s.key_dim, s.value_dim
        proj = torch.empty((T, self.in_rows), dtype=env.dtype, device=dev)
        ops.gemm(h, self.inp, proj, env.products)
        state = cache["state"]
        rows = (None if step.decode_only else step.tok_row, step.row_first, step.row_len, step.row_start, step.row_slots)
        o = torch.empty((T, H, E), dtype=torch.float32, device=dev)
        ops.decay_attention(proj, self.q_off, self.k_off, self.v_off, H, D, E, s.activation, s.key_scale, self.decay,
                            state.state, rows, o, writes=state.writes)  # fmt: skip
        act = torch.empty((T, H * E), dtype=env.dtype, device=dev)
        ops.decay_finish(o.view(T, H * E), H if s.out_norm == "heads" else 1, s.out_norm_eps, self.out_norm_weight, proj,
                         self.g_off, s.gate, act)  # fmt: skip
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.gemm(act, self.out, y, env.products)
        return y


register("mixer", "decay_attention", DecayAttention)
