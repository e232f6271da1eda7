"""Mixers side by side: every one reads the same rows, and the result is the sum of their
results, each times a constant.

The mixers are named; the tensors, the per-request state and the cache of a member are the
member's own, under its name (``<name>.<tensor>``).  At most one member may keep pages (a run
has one place in one page group); any number may keep state rows.
"""

from __future__ import annotations

import torch
from pydantic import BaseModel, model_validator

from ..config.spec import PartSpec
from ..kernels import ops
from .base import MIXERS, Mixer, RunBinding


class MixerSumParams(BaseModel):
    names: list[str]
    mixers: list[dict]
    """One description a member: ``kind`` and the kind's own parameters."""
    scales: list[float]

    @model_validator(mode="after")
    def _check(self):
        if not self.names or not (len(self.names) == len(self.mixers) == len(self.scales)):
            raise ValueError("a sum of mixers has as many names and scales as members, and at least one")
        if len(set(self.names)) != len(self.names) or any("." in n or not n for n in self.names):
            raise ValueError(f"the members' names {self.names} must differ and hold no dot")
        return self


@MIXERS.register("sum")
class MixerSum(Mixer):
    Params = MixerSumParams

    def __init__(self, params, build):
        super().__init__(params, build)
        self.members = [(name, MIXERS.build(PartSpec(**spec), build), scale)
                        for name, spec, scale in zip(params.names, params.mixers, params.scales)]
        self.graph_safe = all(m.graph_safe for _, m, _ in self.members)
        self._paged = [name for name, m, _ in self.members if m.cache_need() is not None]
        if len(self._paged) > 1:
            raise ValueError(f"only one member of a sum of mixers may keep pages; {self._paged} all do")

    def param_decls(self):
        return {f"{name}.{k}": d for name, m, _ in self.members for k, d in m.param_decls().items()}

    def allocate(self, dtypes):
        out = {}
        for name, m, _ in self.members:
            own = {k[len(name) + 1 :]: v for k, v in dtypes.items() if k.startswith(name + ".")}
            out.update({f"{name}.{k}": t for k, t in m.allocate(own).items()})
        return out

    def finalize(self):
        for _, m, _ in self.members:
            m.finalize()

    def cache_need(self):
        for _, m, _ in self.members:
            need = m.cache_need()
            if need is not None:
                return need
        return None

    def state_need(self):
        return {f"{name}.{k}": need for name, m, _ in self.members for k, need in m.state_need().items()}

    def _member_run(self, run: RunBinding, name: str) -> RunBinding:
        return RunBinding(
            index=run.index, kv=run.kv if name in self._paged else None, appends=run.appends,
            state={k[len(name) + 1 :]: t for k, t in run.state.items() if k.startswith(name + ".")},
        )

    def prepare(self, ctx, run):
        for name, m, _ in self.members:
            m.prepare(ctx, self._member_run(run, name))

    def forward_terms(self, x, ctx, run):
        """The members' results and their constants, for a caller that adds them up itself
        (an arrangement whose next kernel reads the sum anyway)."""
        terms = []
        for name, m, scale in self.members:
            a = m.forward(x, ctx, self._member_run(run, name))
            terms.append((a if a.dtype == torch.float32 else a.float(), scale))
        return terms

    def forward(self, x, ctx, run):
        total = None
        for name, m, scale in self.members:
            a = m.forward(x, ctx, self._member_run(run, name))
            if a.dtype != torch.float32:
                a = a.float()
            total = ops.scale_(a, scale) if total is None else ops.scaled_sum_(total, 1.0, a, scale)
        return total
