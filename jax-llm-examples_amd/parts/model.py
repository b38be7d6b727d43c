"""The generic decoder: embedding, the layers of a plan run in the plan's order,
final norm and output head (``llama4/llama4_jax/model.py:1186-1210``), each a part built from
its :class:`~..config.specs.PartSpec`.  It is built from a :class:`~..config.specs.ModelPlan` alone."""
from __future__ import annotations

import torch

from ..cache.manager import CacheView
from ..config.specs import ModelPlan
from .residual import Residual
from ..config.specs import part
from . import embedding as _ends  # noqa: F401  (registers the built-in embedding and head)
from .base import CacheNeed, ParamSpec, Part, build_embedding, build_head, build_norm
from .block import build_block


class DecoderModel:
    def __init__(self, plan: ModelPlan, dtype: torch.dtype, device) -> None:
        self.plan = plan
        self.dtype = dtype
        self.device = torch.device(device)
        # (a plan that does not describe its two ends gets a plain table and a plain linear head)
        self.embed = build_embedding(plan.embedding or part("token_embedding", vocab_size=plan.vocab_size,
                                                            hidden_size=plan.hidden_size))
        self.blocks = [build_block(spec) for spec in plan.layers]
        self.final_norm = build_norm(plan.final_norm)
        self.lm_head = build_head(plan.head or part("linear_head", vocab_size=plan.vocab_size,
                                                    hidden_size=plan.hidden_size, tied=plan.tie_word_embeddings))
        self._allocated = False

    # ------------------------------------------------------------------ parameters
    def named_parts(self) -> dict[str, Part]:
        out: dict[str, Part] = {"embed": self.embed}
        for i, b in enumerate(self.blocks):
            for name, p in b.parts().items():
                out[f"layers.{i}.{name}"] = p
        out["final_norm"] = self.final_norm
        out["lm_head"] = self.lm_head
        return out

    def param_specs(self) -> dict[str, ParamSpec]:
        return {f"{pn}.{n}": s for pn, p in self.named_parts().items() for n, s in p.param_specs().items()}

    def allocate(self) -> None:
        if not self._allocated:
            for p in self.named_parts().values():
                p.allocate(self.dtype, self.device)
            self._allocated = True

    def named_parameters(self) -> dict[str, torch.Tensor]:
        self.allocate()
        return {f"{pn}.{n}": t for pn, p in self.named_parts().items() for n, t in p.params.items()}

    def finalize(self) -> None:
        for p in self.named_parts().values():
            p.finalize()

    def num_parameters(self) -> int:
        n = 0
        for s in self.param_specs().values():
            k = 1
            for d in s.shape:
                k *= d
            n += k
        return n

    # ------------------------------------------------------------------ cache
    def cache_needs(self) -> dict[int, CacheNeed]:
        needs: dict[int, CacheNeed] = {}
        for e in self.plan.order:
            need = self.blocks[e.layer].mixer.cache_need()
            if e.cache in needs and needs[e.cache] != need:
                raise ValueError(f"runs that share cache {e.cache} need different things: {needs[e.cache]} vs {need}")
            needs[e.cache] = need
        return needs

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, cache) -> torch.Tensor:
        """Runs the step's tokens through every run of the order; returns float32
        logits ``[len(ctx.logits_indices), vocab]``."""
        ops = ctx.ops
        residual = Residual(self.embed.forward(ctx.token_ids, ctx))
        for e in self.plan.order:
            gi = cache.group_of.get(e.cache)
            view = CacheView(cache_id=e.cache, writes=e.writes_cache, group=gi, state=cache.state.get(e.cache))
            if gi is not None:
                g = ctx.groups[gi]
                view.kv = cache.groups[gi].tensors.get(e.cache)
                view.pages = cache.groups[gi].pages.get(e.cache)
                view.block_table = g.block_table
                view.slot_mapping = g.slot_mapping
                view.attn_meta = g
            self.blocks[e.layer].forward(residual, ctx, view)
        if ctx.logits_indices.numel() == 0:
            residual.value(ctx)
            return torch.empty(0, self.plan.vocab_size, dtype=torch.float32, device=ctx.device)
        picked = residual.rows(ctx, ctx.logits_indices)
        h, _ = self.final_norm.forward(picked, ctx)
        return self.lm_head.forward(h, ctx, self.embed)
