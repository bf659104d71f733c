"""Causal softmax attention whose keys and values come from one cached latent per token.

    c_q = norm(W_dq h);   q_h = W_uq c_q = [q_h plain (head_dim) | q_h turned (rot_dim)]
    [c raw | k_r raw] = W_dkv h;   c = norm(c raw)  [kv_rank];   k_r turned by the position  [rot_dim], one for all heads
    k_h(j) = U_h c_j,   v_h(j) = V_h c_j;   score_h(i, j) = scale (q_h plain(i) . k_h(j) + q_h turned(i) . k_r(j)),  j <= i
    out = W_o ([softmax_j(score_h) v_h]_h * sigmoid(W_g h))

Only c and k_r are cached: a page holds one kv head whose keys are [c | k_r] and whose values are c.  Because
q_h . (U_h c) = (U_h^T q_h) . c and sum_j p_j V_h c_j = V_h sum_j p_j c_j, the attention itself is the package's paged
attention over that one kv head with queries [U_h^T q_h plain | q_h turned] (all heads one group), and V_h is applied
to what it returns.  A layer without a latent of its own (spec.own_latent False) reads the pages of the run that its
run names as its cache, with its own U, V, queries and everything else.

W_dq, W_dkv (where the layer has one) and W_g are rows of one input matrix.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.attention import SHORT_ROW, TILE_Q, attend
from atomserve_amd.parts.base import Mixer, PagedCacheRequest, WeightDecl, build, register


class LatentAttention(Mixer):
    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if min(s.num_heads, s.head_dim, s.value_dim, s.q_rank, s.kv_rank) < 1 or s.rot_dim < 0 or s.rot_dim % 2:
            raise ValueError("sizes of a latent attention are positive, the turned part even")
        self.position = build("position", s.position, env) if s.position is not None and s.rot_dim else None
        if self.position is not None and getattr(self.position, "pairs", None) != "half":
            raise ValueError(f"the kernels turn the pairs (i, i + R/2) by a table of cosines and sines; "
                             f"{s.position.kind!r} declares {getattr(self.position, 'pairs', None)!r}")  # fmt: skip
        if s.rot_dim and (self.position is None or s.position.rotary_dim != s.rot_dim):
            raise ValueError(f"the turned part has {s.rot_dim} coordinates; its position part must turn exactly those")
        chunk = 4 if env.dtype == torch.float32 else 8
        widest = s.kv_rank + s.rot_dim
        # what the attention kernels take as a head: multiples of 32 on the matrix cores, else of the chunk they load
        self.width = -(-widest // 32) * 32 if widest > 16 else -(-widest // chunk) * chunk
        # a page wider than those kernels' heads goes through a kernel of its own, plain and for any width
        self.wide = self.width > ops.SINGLE_QUERY_MAX_HEAD_DIM
        if self.wide:
            self.width = -(-widest // chunk) * chunk
        if self.width > ops.WIDE_ATTEND_MAX_WIDTH or s.kv_rank > ops.LATENT_MAX_RANK or s.head_dim > ops.LATENT_MAX_HEAD_DIM:
            raise ValueError(f"a latent of {s.kv_rank} and a turned part of {s.rot_dim} exceed the attention kernels' heads "
                             f"of {ops.WIDE_ATTEND_MAX_WIDTH}")  # fmt: skip
        self.dkv_off = s.q_rank
        self.g_off = s.q_rank + (widest if s.own_latent else 0)
        self.in_rows = self.g_off + s.num_heads * s.value_dim

    @property
    def capturable(self) -> bool:
        return self.position is None or self.position.capturable

    def weight_decls(self) -> dict:
        s = self.spec
        decls = {
            "in.weight": WeightDecl((self.in_rows, s.hidden_size)),
            "q_norm.weight": WeightDecl((s.q_rank,), role="vector"),
            "uq.weight": WeightDecl((s.num_heads * (s.head_dim + s.rot_dim), s.q_rank)),
            "uk.weight": WeightDecl((s.num_heads * s.head_dim, s.kv_rank)),
            "uv.weight": WeightDecl((s.num_heads * s.value_dim, s.kv_rank)),
            "o.weight": WeightDecl((s.hidden_size, s.num_heads * s.value_dim)),
        }
        if s.own_latent:
            decls["kv_norm.weight"] = WeightDecl((s.kv_rank,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        self.kv_norm_weight = None
        super().bind(tensors)
        s = self.spec
        self.q_norm_weight = self.q_norm_weight.float().contiguous()
        if self.kv_norm_weight is not None:
            self.kv_norm_weight = self.kv_norm_weight.float().contiguous()
        # every head's value matrix transposed, [heads, kv_rank, value_dim]: lanes that own neighbouring outputs read neighbours
        self.uv_t = self.uv_weight.view(s.num_heads, s.value_dim, s.kv_rank).transpose(1, 2).contiguous()
        # and every head's key matrix transposed, [heads, kv_rank, head_dim]: what prompts multiply with on the matrix cores
        self.uk_t = self.uk_weight.view(s.num_heads, s.head_dim, s.kv_rank).transpose(1, 2).contiguous()
        self.inp = ops.Streamed(self.in_weight, self.env.stream_copies)
        self.uq = ops.Streamed(self.uq_weight, self.env.stream_copies)
        self.o = ops.Streamed(self.o_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.inp, self.uq, self.o]

    def cache_request(self):
        return PagedCacheRequest(1, self.width, 0)

    def row_split(self):
        return None if self.wide else (SHORT_ROW, TILE_Q)

    def forward(self, h, step, cache):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        H, D, R, E = s.num_heads, s.head_dim, s.rot_dim, s.value_dim
        proj = torch.empty((T, self.in_rows), dtype=env.dtype, device=dev)
        ops.gemm(h, self.inp, proj, env.products)
        cos_sin = self.position.prepare(step) if self.position is not None else None
        if s.own_latent and cache.writes:
            ops.latent_kv_store(proj, self.dkv_off, s.kv_rank, R, self.kv_norm_weight, s.norm_eps, cos_sin, cache.slots,
                                cache.k_pages, cache.v_pages)  # fmt: skip
        cq = torch.empty((T, s.q_rank), dtype=env.dtype, device=dev)
        ops.rows_rms_norm(proj, 0, s.q_rank, self.q_norm_weight, s.norm_eps, cq)
        q = torch.empty((T, H * (D + R)), dtype=env.dtype, device=dev)
        ops.gemm(cq, self.uq, q, env.products)
        qa = torch.empty((T, H, self.width), dtype=env.dtype, device=dev)
        ops.latent_q_absorb(q, self.uk_weight, H, D, R, s.kv_rank, cos_sin, qa, uk_t=self.uk_t)
        heads = torch.empty((T, H, self.width), dtype=env.dtype, device=dev)
        if self.wide:
            ops.wide_attend(qa, cache.k_pages, cache.v_pages, step.positions, None if step.decode_only else step.tok_row,
                            cache.block_tables, heads, s.scale, step.max_context)  # fmt: skip
        else:
            attend(qa, heads, step, cache, s.scale, 0, self.row_split())
        act = torch.empty((T, H * E), dtype=env.dtype, device=dev)
        ops.latent_v_expand(heads, self.uv_t, s.kv_rank, proj, self.g_off, act, uv=self.uv_weight)
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.gemm(act, self.o, y, env.products)
        return y


register("mixer", "latent_attention", LatentAttention)
