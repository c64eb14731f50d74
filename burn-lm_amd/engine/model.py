"""Builds a runnable model from a plan: instantiates the parts by their registered kinds,
collects the tensors they ask for, binds the loaded tensors, and runs a step through the places
of the layer order."""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import registry
from ..models.plan import ModelPlan
from ..parts.base import TensorSpec


class Model:
    def __init__(self, plan: ModelPlan):
        self.plan = plan
        self.positions = {k: registry.part("position", s.kind)(s.params, s.names) for k, s in plan.positions.items()}
        self.embedding = registry.part("embedding", plan.embedding.kind)(plan.embedding.params, plan.embedding.names)
        self.final_norm = registry.part("norm", plan.final_norm.kind)(plan.final_norm.params, plan.final_norm.names)
        self.head = registry.part("head", plan.head.kind)(plan.head.params, plan.head.names)
        self.blocks = []
        for li, lp in enumerate(plan.layers):
            block_cls = registry.part("block", lp.block)
            made = {}
            for role, spec in lp.parts.items():
                family = block_cls.roles.get(role)
                if family is None:
                    raise ValueError(f"layer {li}: the block {lp.block!r} has no role {role!r}; "
                                     f"its roles: {', '.join(block_cls.roles) or 'none'}")
                params = dict(spec.params)
                if family == "mixer" and lp.position is not None:
                    params["position"] = self.positions[lp.position]
                made[role] = registry.part(family, spec.kind)(params, spec.names)
            self.blocks.append(block_cls(made))
        for i, place in enumerate(plan.order):
            if not 0 <= place.layer < len(self.blocks):
                raise ValueError(f"place {i} of the layer order names layer {place.layer}, "
                                 f"but there are {len(self.blocks)} layers")
        self.vocab_size = plan.vocab_size
        self.rt = None

    def all_parts(self):
        """In the order they are bound: the position encodings first, because a mixer consults its
        encoding while it binds its own projections."""
        yield from self.positions.values()
        yield self.embedding
        for b in self.blocks:
            yield from b.parts()
        yield self.final_norm
        yield self.head

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in self.all_parts():
            for name, spec in p.tensor_specs().items():
                if name in specs and specs[name] != spec:
                    raise ValueError(f"tensor {name} is asked for with two shapes: {specs[name].shape} and {spec.shape}")
                specs[name] = spec
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor], rt) -> None:
        self.rt = rt
        for p in self.all_parts():
            p.bind(tensors, rt)

    def cache_needs(self) -> List:
        return [self.blocks[pl.layer].cache_need() for pl in self.plan.order]

    def reads_from(self) -> List:
        return [pl.reads_cache_of for pl in self.plan.order]

    def prepare_positions(self, n_positions: int) -> None:
        for p in self.positions.values():
            p.prepare(n_positions, self.rt)

    def step_costs(self, pasts, news, wanted_rows, cache=None):
        """What one step costs at the least: sequences that hold pasts[i] tokens get news[i] more and
        wanted_rows logits rows are asked for.  -> dict(weight_bytes: every tensor the step uses,
        read once; cache_bytes: the keys and values it reads (given the cache); flops: its matrix
        products and its attention).  The parts answer for themselves, so this holds for any plan."""
        rows = sum(news)
        weight_bytes = self.embedding.step_bytes(rows) + self.final_norm.step_bytes(wanted_rows) + self.head.step_bytes(wanted_rows)
        flops = self.head.step_flops(wanted_rows)
        for place in self.plan.order:
            block = self.blocks[place.layer]
            for part in block.parts():
                weight_bytes += part.step_bytes(rows)
                flops += part.step_flops(rows)
                if hasattr(part, "mixing_flops"):
                    flops += sum(part.mixing_flops(p, n) for p, n in zip(pasts, news))
        cache_bytes = 0
        if cache is not None:
            cache_bytes = sum(cache.bytes_read(p + n) for p, n in zip(pasts, news))
        return dict(weight_bytes=weight_bytes, cache_bytes=cache_bytes, flops=flops)

    def forward(self, step, cache):
        """Logits (float32, [wanted rows, vocab]) of one step, or None when no row is wanted."""
        if step.token_source is None:
            h = self.embedding.forward(step.token_ids)
        else:
            h = self.embedding.forward_from(step.token_ids, *step.token_source)
        delta = None
        for i, place in enumerate(self.plan.order):
            delta = self.blocks[place.layer].forward(h, delta, step, cache.views[i])
        if step.n_wanted == 0:
            return None
        x = self.final_norm.add_norm(h, delta, rows=step.want_rows, write_h=False)
        return self.head.forward(x)
