"""A decoder assembled from a plan: embedding, the run list over its layers, final
norm and head.  It knows no architecture: which parts a layer has, their sizes and
the order of runs all come from the plan (reference atomserve/model.py:363-412 is
the one hard-wired instance of this loop)."""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import BuildEnv, GatedDelta, WeightDecl, build
from atomserve_amd.parts.plan import ModelPlan


class DecoderModel:
    def __init__(self, plan: ModelPlan, dtype: torch.dtype, device, stream_copies: bool = True):
        """stream_copies: keep the matrices that decode steps stream a second time, in the order their
        kernels read them (`ops.Streamed`): faster decode steps for the weights' bytes again."""
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute dtype must be float32 or bfloat16, got {dtype}")
        self.plan = plan
        self.env = BuildEnv(dtype=dtype, device=torch.device(device), stream_copies=bool(stream_copies),
                            products=ops.ProductChoices())  # fmt: skip
        self.blocks = [build("arrangement", spec, self.env) for spec in plan.layers]
        self.final_norm = build("norm", plan.final_norm, self.env)
        self.embed_norm = build("norm", plan.embed_norm, self.env) if plan.embed_norm is not None else None
        if self.embed_norm is not None and not hasattr(self.embed_norm, "stream"):
            raise ValueError(f"a norm of kind {plan.embed_norm.kind!r} cannot make the embedding's rows the stream")
        if any(r.reenter for r in plan.run) and not plan.reentry:
            raise ValueError("a run re-enters the stream, and the plan names no matrix for it (reentry)")
        for r in plan.run:
            if not 0 <= r.layer < len(self.blocks):
                raise ValueError(f"run list names layer {r.layer}, the plan has {len(self.blocks)}")
        self.embed_weight = None
        self.head_weight = None

    @property
    def capturable(self) -> bool:
        """Whether a decode step may be captured and replayed as a graph: every part says it is."""
        return self.final_norm.capturable and all(self.blocks[r.layer].capturable for r in self.plan.run) and \
            (self.embed_norm is None or self.embed_norm.capturable)  # fmt: skip

    # ---- tensors --------------------------------------------------------------------
    def weight_decls(self) -> dict:
        p = self.plan
        decls = {"embed.weight": WeightDecl((p.vocab_size, p.hidden_size))}
        for i, block in enumerate(self.blocks):
            for part_name, part in block.parts().items():
                for local, decl in part.weight_decls().items():
                    decls[f"layers.{i}.{part_name}.{local}"] = decl
        for local, decl in self.final_norm.weight_decls().items():
            decls[f"final_norm.{local}"] = decl
        if self.embed_norm is not None:
            for local, decl in self.embed_norm.weight_decls().items():
                decls[f"embed_norm.{local}"] = decl
        if p.reentry:
            decls["reentry.weight"] = WeightDecl((p.hidden_size, 2 * p.hidden_size))
        if not p.tied_head:
            decls["head.weight"] = WeightDecl((p.vocab_size, p.hidden_size))
        return decls

    def bind(self, tensors: dict) -> None:
        """Hand every part its tensors, by the names of `weight_decls`."""
        self.embed_weight = tensors["embed.weight"]
        self.head_weight = self.embed_weight if self.plan.tied_head else tensors["head.weight"]
        self.head = ops.Streamed(self.head_weight, self.env.stream_copies)  # the head's product streams it at every decode step
        for i, block in enumerate(self.blocks):
            for part_name, part in block.parts().items():
                prefix = f"layers.{i}.{part_name}."
                part.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})
        self.final_norm.bind({k[len("final_norm."):]: v for k, v in tensors.items() if k.startswith("final_norm.")})
        if self.embed_norm is not None:
            self.embed_norm.bind({k[len("embed_norm."):]: v for k, v in tensors.items() if k.startswith("embed_norm.")})
        self.reentry = ops.Streamed(tensors["reentry.weight"], self.env.stream_copies) if self.plan.reentry else None
        self._tensors = tensors

    @property
    def num_weight_bytes(self) -> int:
        """Bytes of all distinct tensors (a tied head counts once)."""
        seen = {t.data_ptr(): t.numel() * t.element_size() for t in self._tensors.values()}
        return sum(seen.values())

    @property
    def num_stream_copy_bytes(self) -> int:
        """Bytes of the copies in wave order that the parts and the head keep beside the tensors."""
        owned = [self.head] + ([self.reentry] if self.reentry is not None else []) + [w for block in self.blocks for part in block.parts().values() for w in part.streamed()]
        return sum(w.wave_bytes for w in owned)

    # ---- caches ---------------------------------------------------------------------
    def cache_requests(self) -> dict:
        """cache id -> what the mixer writing it asks of the cache manager.  A mixer that keeps several
        things (`Mixer.cache_request` returns a dict) has one entry per name, under the id (cache id, name)."""
        def asked(mixer) -> dict:
            req = mixer.cache_request()
            if req is None:
                return {}
            return dict(req) if isinstance(req, dict) else {None: req}

        def ident(cid, name):
            return cid if name is None else (cid, name)

        requests = {}
        for i, r in enumerate(self.plan.run):
            cid = self.plan.cache_id(i)
            if not r.writes:
                continue
            for name, req in asked(self.blocks[r.layer].parts()["mixer"]).items():
                key = ident(cid, name)
                if key in requests and requests[key] != req:
                    raise ValueError(f"runs sharing cache {cid} ask for different caches")
                requests[key] = req
        for i, r in enumerate(self.plan.run):
            cid = self.plan.cache_id(i)
            for name in asked(self.blocks[r.layer].parts()["mixer"]):
                if ident(cid, name) not in requests:
                    raise ValueError(f"run {i} reads cache {cid}, which no run writes")
        # what a layer keeps beside its mixer belongs to the run, whatever cache the run's mixer reads
        for i, r in enumerate(self.plan.run):
            for name, req in (self.blocks[r.layer].cache_request() or {}).items():
                requests[(self.layer_cache_id(i), name)] = req
        return requests

    @staticmethod
    def layer_cache_id(run_index: int) -> int:
        """The id under which run `run_index` files what its layer keeps itself: apart from every mixer's (those
        are run indices, from 0 up)."""
        return -1 - run_index

    # ---- one pass ---------------------------------------------------------------------
    def row_splits(self) -> tuple:
        """How the mixers want the rows of a step sorted for their kernels: every distinct answer of
        `Mixer.row_split` among the layers (none if no mixer cares); a step is packed once for each."""
        return tuple(sorted({split for block in self.blocks for split in [block.parts()["mixer"].row_split()]
                             if split is not None}))  # fmt: skip

    def forward(self, step, logits: torch.Tensor = None) -> torch.Tensor:
        """Run this step's tokens through every run of the plan; returns fp32 logits
        [len(step.logits_rows), vocab] for the wanted rows (written into `logits` if given)."""
        p, dev = self.plan, self.env.device
        x = torch.empty((step.num_tokens, p.hidden_size), dtype=torch.float32, device=dev)
        ops.embed_gather(self.embed_weight, step.token_ids, x, p.embedding_scale)
        x0 = None
        if self.embed_norm is not None:
            x0 = self.embed_norm.stream(x)  # fp32: the stream starts as the norm's result, unrounded
            # the layers change the stream in place; where runs re-enter with what the embedding gave, that is
            # kept apart (a first run that re-enters replaces the stream before anything has changed it)
            x = self.embed_norm.stream(x) if p.reentry and not p.run[0].reenter else x0
        elif p.reentry:
            x0 = x if p.run[0].reenter else x.clone()
        delta = None
        for i, r in enumerate(p.run):
            if r.reenter:
                x, delta = self._reenter(x, delta, x0), None
            # the norm that the run after this one starts with: this run's last product may add
            # into x and leave that norm pending instead of handing over a delta
            follows = self.blocks[p.run[i + 1].layer].first_norm() if i + 1 < len(p.run) else None
            block = self.blocks[r.layer]
            extra = {}
            kept = block.cache_request()
            if kept:
                extra["own"] = {name: step.cache_view((self.layer_cache_id(i), name), True) for name in kept}
            delta = block.forward(x, delta, step, step.cache_view(p.cache_id(i), r.writes), next_norm=follows, **extra)
        return self._head(x, delta, step, logits)

    def _reenter(self, x, delta, x0):
        """The stream after the pending output `delta` has been added, beside x0, through the re-entry matrix:
        a new fp32 stream W [x ; x0]."""
        T, hidden = x.shape
        join = torch.empty((T, 2 * hidden), dtype=self.env.dtype, device=x.device)
        if isinstance(delta, GatedDelta):
            ops.gated_add_norm(x, delta.y, delta.gate, delta.gate_off, delta.bias, delta.mult, None, 0.0, None,
                               other=x0, join=join)  # fmt: skip
        elif delta is None:
            ops.gated_add_norm(x, None, None, 0, None, 1.0, None, 0.0, None, other=x0, join=join)
        else:
            raise ValueError("a run re-enters the stream after a layer that leaves a gated output, or none")
        out = torch.empty((T, hidden), dtype=torch.float32, device=x.device)
        ops.gemm(join, self.reentry, out, self.env.products)
        return out

    def _head(self, x, delta, step, logits):
        p, dev = self.plan, self.env.device
        n = step.num_logits
        if logits is None:
            logits = torch.empty((n, p.vocab_size), dtype=torch.float32, device=dev)
        elif logits.shape != (n, p.vocab_size) or logits.dtype != torch.float32:
            raise ValueError(f"the logits of this step are float32 {(n, p.vocab_size)}, the buffer is {tuple(logits.shape)}")
        if n:
            hf = self.final_norm.forward(x, delta, rows=step.logits_rows, update_residual=False)
            ops.gemm(hf, self.head, logits, self.env.products)
            if p.logit_scale != 1.0 or p.logit_softcap > 0.0:
                ops.logits_finish(logits, p.logit_scale, p.logit_softcap)
        return logits
