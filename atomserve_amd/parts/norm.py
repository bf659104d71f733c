"""RMSNorm: weight * x / sqrt(mean(x^2) + eps), accumulated in fp32 and rounded once
(reference atomserve/model.py:125-139).  The residual sum that precedes a norm in a
pre-norm layer is fused into the same kernel: the fp32 residual stream `x` receives
`delta` and the normalised result is written in the compute dtype."""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import DeltaSum, GatedDelta, Norm, PendingNorm, SplitSums, WeightDecl, register


class PendingRMSNorm(PendingNorm):
    """x * gain (rounded to the compute dtype) and the sums of x^2 per 16 columns: a product of
    `scaled` times 1 / rms is the product of the normalised rows."""

    def __init__(self, norm, x, scaled, ssq):
        super().__init__(norm, x)
        self.scaled, self.ssq = scaled, ssq

    def gemm(self, w, out) -> None:
        ops.gemm_scaled(self.scaled, self.ssq, self.norm.spec.eps, w, out)

    def gemm_gated(self, w, out, activation) -> bool:
        if activation != "silu":
            return False
        ops.gemm_scaled(self.scaled, self.ssq, self.norm.spec.eps, w, out, gated=True)
        return True


class RMSNorm(Norm):
    capturable = True
    takes_split_sums = True
    takes_gated_delta = True

    def weight_decls(self) -> dict:
        return {"weight": WeightDecl((self.spec.size,), role="vector")}

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        if self.spec.offset:  # a gain stored around zero: the sum is made once, in 32 bits, and stays so
            self.weight = (self.weight.float() + float(self.spec.offset)).contiguous()
        self.gain_f32 = self.weight.float()  # what the fused product reads (exact: bf16 widens)

    def absorb(self, a, w, x):
        M, N = x.shape
        if not ops.gemm_link_supported(M, N, a.shape[1], self.env.dtype, w):
            return None
        scaled = torch.empty((M, N), dtype=self.env.dtype, device=x.device)
        ssq = torch.empty((M, -(-N // 16)), dtype=torch.float32, device=x.device)
        ops.gemm_link(a, w, x, self.gain_f32, scaled, ssq)
        return PendingRMSNorm(self, x, scaled, ssq)

    def forward(self, x, delta=None, rows=None, update_residual=True) -> torch.Tensor:
        """x: fp32 [T, size] residual stream.  delta: pending sum in the compute dtype (or as the
        partial sums of the product that makes it, `SplitSums`), or None.
        rows: int32 row selection, or None for all rows.  Returns [rows, size], compute dtype."""
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n_out, self.spec.size), dtype=self.env.dtype, device=x.device)
        if isinstance(delta, GatedDelta):
            ops.gated_add_norm(x, delta.y, delta.gate, delta.gate_off, delta.bias, delta.mult, self.weight,
                               self.spec.eps, out, rows=rows, update_x=update_residual)  # fmt: skip
        elif isinstance(delta, DeltaSum):
            self.with_sibling(None, x, delta, rows, update_residual, out)
        elif isinstance(delta, SplitSums):
            ops.rmsnorm(x, self.weight, self.spec.eps, out, rows=rows, update_x=update_residual, split_sums=delta.sums)
        else:
            ops.rmsnorm(x, self.weight, self.spec.eps, out, delta=delta, rows=rows, update_x=update_residual)
        return out


    def stream(self, x) -> torch.Tensor:
        """The norm of the fp32 rows x as a new fp32 tensor: for a norm whose result is itself a residual stream
        (a norm of the embedding), which is never rounded to the compute dtype."""
        out = torch.empty_like(x)
        ops.gated_add_norm(x, None, None, 0, None, 1.0, self.weight, self.spec.eps, out, update_x=False)
        return out

    def with_sibling(self, other, x, delta=None, rows=None, update_residual=True, out=None):
        """This norm and `other` (an RMSNorm of the same size and eps, or None) of the same stream in one
        kernel: x += delta (a tensor, a `DeltaSum` of up to two, or None), the root mean square taken once.
        Returns (this norm's rows, the other's or None)."""
        parts = delta.parts if isinstance(delta, DeltaSum) else (() if delta is None else (delta,))
        if len(parts) > 2 or any(not isinstance(p, torch.Tensor) for p in parts):
            raise ValueError("a norm adds up to two pending outputs (tensors) into the stream")
        if other is not None and (other.spec.size, other.spec.eps) != (self.spec.size, self.spec.eps):
            raise ValueError("two norms of one stream share a kernel only with one size and one eps")
        n_out = x.shape[0] if rows is None else rows.shape[0]
        if out is None:
            out = torch.empty((n_out, self.spec.size), dtype=self.env.dtype, device=x.device)
        out2 = torch.empty_like(out) if other is not None else None
        ops.rmsnorm_multi(x, self.weight, other.weight if other is not None else None, self.spec.eps, out, out2,
                          delta1=parts[0] if parts else None, delta2=parts[1] if len(parts) > 1 else None, rows=rows,
                          update_x=update_residual)  # fmt: skip
        return out, out2


register("norm", "rmsnorm", RMSNorm)


class GroupedRMSNorm(Norm):
    """An RMS norm in groups: the row is cut into spec.groups equal consecutive parts, each divided by its own
    sqrt(mean(part^2) + eps), and the whole multiplied by the gain.  `forward` is the plain norm's (pending residual
    sum, row selection); `forward_shifted` also mixes every token's normed row with the one of the token before."""

    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if spec.groups < 1 or spec.size % spec.groups or spec.groups > ops.NORM_MAX_GROUPS:
            raise ValueError(f"a norm of {spec.size} does not divide into {spec.groups} groups (at most {ops.NORM_MAX_GROUPS})")

    def weight_decls(self) -> dict:
        return {"weight": WeightDecl((self.spec.size,), role="vector")}

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        self.gain_f32 = self.weight.float().contiguous()  # exact: what a file holds in 16 bits widens

    def forward(self, x, delta=None, rows=None, update_residual=True) -> torch.Tensor:
        if delta is not None and not isinstance(delta, torch.Tensor):
            raise ValueError("a grouped norm adds a plain pending output into the stream")
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n_out, self.spec.size), dtype=self.env.dtype, device=x.device)
        ops.group_norm(x, self.gain_f32, self.spec.eps, self.spec.groups, out, delta=delta, rows=rows,
                       update_x=update_residual)  # fmt: skip
        return out

    def forward_shifted(self, x, mu, step_rows, state, writes=True) -> torch.Tensor:
        """norm(x) with a token shift by mu (fp32 [size]): out_t = h_t + (h_(t-1) - h_t) * mu.  state fp32 [slots, size]
        holds every request's last normed row between its rows; step_rows as the kernels of mixers with state take them."""
        out = torch.empty((x.shape[0], self.spec.size), dtype=self.env.dtype, device=x.device)
        ops.group_norm_shift(x, self.gain_f32, mu, self.spec.eps, self.spec.groups, step_rows, state, out, writes=writes)
        return out


register("norm", "grouped_rmsnorm", GroupedRMSNorm)
