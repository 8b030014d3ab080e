"""Mixers side by side: several mixers read the same input, each result goes through an RMS norm over the model
width with a plain weight of its own (`<name>.out`), and the mixer's result is `scale` times their sum (one half for
two mixers whose results are averaged).

The mixers are parts like any other (`mixers`: name -> PartSpec, tensors under `<name>.`); what they keep between
steps is put together into one declaration: the pages of the one mixer that keeps pages, and the fixed state of all,
each tensor under `<name>.<tensor>`. Every mixer sees its own tensors under their own names.
"""

from __future__ import annotations

from typing import Dict

from ..config.model_config import PartSpec
from .base import Borrowed, CacheNeeds, FixedState, Mixer, PagedTensors, ParamSpec, TensorDecl, build_part, register_part


class _Own:
    """One mixer's share of the combined view: its state tensors by their own names, the pages as they are."""

    def __init__(self, view, name: str) -> None:
        self._view, self._prefix = view, name + "."
        self.group = view.group

    def __getitem__(self, key: str):
        tensors = self._view.tensors
        return tensors[self._prefix + key] if self._prefix + key in tensors else tensors[key]


class ParallelMixers(Mixer):
    def __init__(self, spec: PartSpec) -> None:
        super().__init__(spec)
        p = spec.params
        self.hidden_size = int(p["hidden_size"])
        self.eps = float(p["eps"])
        self.mixers: Dict[str, Mixer] = {name: build_part("mixer", sub) for name, sub in p["mixers"].items()}
        if not self.mixers:
            raise ValueError("no mixers to put side by side")
        self.scale = float(p.get("scale", 1.0 / len(self.mixers)))
        self.out_weights = {}

    def parts(self):
        for mixer in self.mixers.values():
            yield from mixer.parts()
        yield self

    def param_specs(self):
        return {f"{name}.out": ParamSpec((self.hidden_size,), "ones") for name in self.mixers}

    def load(self, tensors) -> None:
        self.out_weights = {name: tensors[f"{name}.out"].float().contiguous() for name in self.mixers}

    def cache_requirement(self):
        paged, state = None, []
        for name, mixer in self.mixers.items():
            need = mixer.cache_requirement()
            if isinstance(need, CacheNeeds):
                pages, fixed = need.paged, need.state
            elif isinstance(need, FixedState):
                pages, fixed = None, need
            else:
                pages, fixed = need, None
            if pages is not None:
                if paged is not None or not isinstance(pages, (PagedTensors, Borrowed)):
                    raise ValueError("mixers side by side: at most one of them keeps pages")
                paged = pages
            if fixed is not None:
                state.extend(TensorDecl(f"{name}.{t.name}", t.shape, t.dtype) for t in fixed.tensors)
        if paged is None and not state:
            return None
        return CacheNeeds(paged, FixedState(tuple(state)) if state else None)

    def forward(self, ops, x, ctx, cache, writes_cache: bool):
        results = [mixer.forward(ops, x, ctx, _Own(cache, name), writes_cache) for name, mixer in self.mixers.items()]
        return ops.normed_sum(results, [self.out_weights[name] for name in self.mixers], self.eps, self.scale)


register_part("mixer", "parallel_mixers", ParallelMixers)
