"""A model built from a `ModelSpec`: embedding, runs of layers, final norm, head.

Shape of the forward pass is the reference's engine/model.py:58-86 (embedding ->
every block -> final norm -> gather wanted rows -> output projection), except that
the rows whose logits are wanted are gathered before the final norm, which is
row-wise, so only those rows are normalised and projected.
"""

from __future__ import annotations

import torch

from tokensprint_amd.models.spec import ModelSpec
import tokensprint_amd.parts  # noqa: F401  (registers the built-in parts)
from tokensprint_amd.parts.base import (
    BLOCKS, EMBEDDINGS, HEADS, NORMS, POSITIONS, BuildContext, TensorDecl, build_part,
)


class Model:
    def __init__(self, spec: ModelSpec, ctx: BuildContext) -> None:
        spec.validate()
        if ctx.width != spec.width:
            raise ValueError("build context width differs from the model's")
        self.spec, self.ctx = spec, ctx
        for name, pspec in spec.positions.items():
            ctx.positions[name] = build_part(POSITIONS, pspec, ctx)
        self.embedding = build_part(EMBEDDINGS, spec.embedding, ctx)
        self.blocks = []
        for i, layer in enumerate(spec.layers):
            if layer.block not in BLOCKS:
                raise ValueError(f"unknown block kind '{layer.block}'; registered: {sorted(BLOCKS)}")
            kind = BLOCKS[layer.block]
            unknown = sorted(set(layer.parts) - set(kind.ROLES))
            if unknown:
                raise ValueError(f"layer {i}: a '{layer.block}' block has no parts {unknown}; "
                                 f"its roles are {sorted(kind.ROLES)}")
            # every part from the registry its role names; the block checks what it needs
            built = {role: build_part(kind.ROLES[role][0], pspec, ctx)
                     for role, pspec in layer.parts.items()}
            self.blocks.append(kind(built, ctx))
        self.final_norm = build_part(NORMS, spec.final_norm, ctx)
        self.head = build_part(HEADS, spec.head, ctx)
        self.order = spec.order

    # ------------------------------------------------------------ weights
    def parts(self):
        out = [self.embedding]
        for block in self.blocks:
            out.extend(block.parts())
        out.extend([self.final_norm, self.head])
        out.extend(self.ctx.positions.values())
        return out

    def tensor_decls(self) -> dict[str, TensorDecl]:
        decls: dict[str, TensorDecl] = {}
        for part in self.parts():
            for name, decl in part.tensors().items():
                if name in decls and (decls[name].shape != decl.shape
                                      or decls[name].role != decl.role):
                    raise ValueError(f"tensor {name} declared twice with different shapes")
                # a name needed by any part is not optional
                if name in decls and not decls[name].optional:
                    continue
                decls[name] = decl
        return decls

    def load_tensors(self, tensors: dict[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.load(tensors.get)

    # ------------------------------------------------------------ caches
    def cache_needs(self):
        """Per run: the cache need of its block, or None if the run owns no cache."""
        return [self.blocks[run.layer].cache_need() if run.cache_of is None else None
                for run in self.order]

    # ------------------------------------------------------------ step
    def forward(self, batch, caches) -> torch.Tensor:
        """Run the batch's tokens; logits float32 [len(batch.logit_rows), vocab].

        `caches[r]` is the cache view owned by run r (None if it owns none).
        """
        ops = self.ctx.ops
        resid = self.embedding.forward(batch.token_ids)
        delta = None
        for r, run in enumerate(self.order):
            owner = r if run.cache_of is None else run.cache_of
            # what reads the stream after this run: the next run's block (the final norm
            # and the head take a plain delta)
            next_hint = self.blocks[self.order[r + 1].layer].entry_hint() \
                if r + 1 < len(self.order) else None
            resid, delta = self.blocks[run.layer].forward(
                resid, delta, batch, caches[owner], write_cache=run.cache_of is None,
                next_hint=next_hint)
        if batch.num_logit_rows == 0:
            return torch.empty(0, self.spec.vocab_size, dtype=torch.float32, device=resid.device)
        if batch.all_rows_wanted:
            resid_rows, delta_rows = resid, delta
        else:
            resid_rows = ops.gather_rows(resid, batch.logit_rows)
            delta_rows = None if delta is None else ops.gather_rows(delta, batch.logit_rows)
        return self.head.forward_from_stream(resid_rows, delta_rows, self.final_norm)

    # ------------------------------------------------------------ accounting
    def step_weight_bytes(self) -> int:
        """Bytes of every tensor a step reads whole, each counted once (a tied head and
        the embedding share one table): the weight traffic of a decode step."""
        seen, total = set(), 0
        for part in self.parts():
            for t in part.step_read_tensors():
                if t.data_ptr() not in seen:
                    seen.add(t.data_ptr())
                    total += t.numel() * t.element_size()
        return total

    def all_capturable(self) -> bool:
        return all(part.capturable for part in self.parts())
