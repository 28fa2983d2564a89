"""Several mixers side by side: all read the same input, and their results are added, each times a factor of its own.

Parameters: ``hidden_size`` and ``branches``, a list of ``{"kind", "params", "scale"}``; a branch's tensors lie under
the prefix its own parameters name (``params["prefix"]``) below this part's.  What the branches keep between steps
is kept side by side too: the part's cache spec is the ``CombinedSpec`` of theirs, and every branch is handed its
own view.

A branch says what it computes up to its output projection: ``inner_width``, ``out_weight()`` ([hidden, inner_width])
and ``forward_inner(x, ctx, cache, out)``, which writes its share of one wide row with its factor already in it (its
parameter ``out_scale``).  The output projections of all branches are then ONE product: the wide rows against the
branches' output weights side by side.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

from ..cache.specs import CombinedSpec
from ..weights.store import TensorSpec
from .base import MIXERS, BuildContext, Part, StepContext, StepCost, joined, says
from .linear import Linear


def _branch_params(branch: Dict[str, Any]) -> Dict[str, Any]:
    params = dict(branch["params"])
    params["out_scale"] = float(branch.get("scale", 1.0))
    return params


@MIXERS.register("side_by_side")
class SideBySideMixer(Part):
    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for branch in params["branches"]:
            sub = _branch_params(branch)
            for name, spec in MIXERS.get(branch["kind"]).weight_specs(sub).items():
                out[joined(sub.get("prefix", ""), name)] = spec
        return out

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries: List[Tuple[int, int]], weight_bytes: int,
                  cache_bytes: int) -> StepCost:
        cost = StepCost()
        for branch in params["branches"]:
            cost = cost + MIXERS.get(branch["kind"]).step_cost(_branch_params(branch), entries, weight_bytes, cache_bytes)
        return cost

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.branches = []
        for branch in params["branches"]:
            sub = _branch_params(branch)
            part = MIXERS.get(branch["kind"])(sub, joined(prefix, sub.get("prefix", "")), build)
            for needed in ("inner_width", "out_weight", "forward_inner"):
                if not hasattr(part, needed):
                    raise TypeError(f"mixer '{branch['kind']}' cannot stand side by side with others: it has no '{needed}'")
            self.branches.append(part)
        if not self.branches:
            raise ValueError("side_by_side needs at least one branch")
        # where each branch writes in the wide row (starts kept at multiples of 16 values for the kernels' wide accesses)
        self.starts: List[int] = []
        at = 0
        for part in self.branches:
            self.starts.append(at)
            at += (part.inner_width + 15) // 16 * 16
        self.width = at
        weights = []
        for part, start in zip(self.branches, self.starts):
            w = part.out_weight()
            pad = (part.inner_width + 15) // 16 * 16 - part.inner_width
            weights.append(w if pad == 0 else torch.cat([w, w.new_zeros(w.shape[0], pad)], dim=1))
        dtypes = {w.dtype for w in weights}
        if len(dtypes) != 1:
            weights = [w.to(torch.float32) for w in weights]
        self.out = Linear(torch.cat(weights, dim=1).contiguous(), build.mode)
        self.padded = any((part.inner_width % 16) for part in self.branches)
        self.specs = [part.cache_spec() for part in self.branches]
        self.act_dtype = build.act_dtype

    def records_cleanly(self) -> bool:
        return all(says(part, "records_cleanly") for part in self.branches)

    def cache_spec(self) -> Optional[CombinedSpec]:
        kept = tuple(spec for spec in self.specs if spec is not None)
        return CombinedSpec(kept) if kept else None

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: Any) -> torch.Tensor:
        ws = ctx.workspace
        tokens = x.shape[0]
        wide = ws.buffer("side_by_side.inner", tokens, self.width, self.act_dtype)
        if self.padded:
            wide.zero_()   # (columns between the branches meet zero weights, but must not hold NaN)
        views = iter(cache if cache is not None else ())
        for part, start, spec in zip(self.branches, self.starts, self.specs):
            view = next(views) if spec is not None else None
            part.forward_inner(x, ctx, view, wide[:, start:start + part.inner_width])
        return self.out.forward(wide, ws.buffer("side_by_side.out", tokens, self.hidden, self.act_dtype))
