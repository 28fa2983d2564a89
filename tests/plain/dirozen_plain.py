"""A plain, slow Dirozen decoder: whole sequences, no cache, one function per mechanism, float64 on the CPU.
It shares no code with ``pulse_infer_amd``: it reads a model folder with ``json`` and the ``safetensors`` package
(or takes a dictionary of tensors) and is written from the design's equations.  Tests compare the engine with it.

Notation: x [T, W] the residual stream, n its normed copy, H query heads over G key/value heads of size d,
p the position of a token (from 0 in each sequence).
"""
from __future__ import annotations

import json
import math
import os
from typing import Any, Dict, List, Optional

import torch

DT = torch.float64


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The layer norm: unit_rms(x) * (1 + w), the weight being stored as its distance from one."""
    return unit_rms(x, eps) * (1.0 + w)


def query_temperature(positions: List[int], coef: float, every: int) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1) for every position, [T]."""
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in positions], dtype=DT)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def gated_attention(n: torch.Tensor, wq: torch.Tensor, wk: torch.Tensor, wg: torch.Tensor, wo: torch.Tensor,
                    heads: int, kv_heads: int, dim: int, scale: float, coef: float, every: int, eps: float,
                    positions: Optional[List[int]] = None) -> torch.Tensor:
    """The mixer for one whole sequence, token by token and head by head.

    q = Wq n, k = Wk n, v = k (as projected); q and k each divided by their root mean square over a head; q times
    the temperature of its position; score_ij = (q_i . k_j) * scale for j <= i; softmax over j; head h reads
    key/value head floor(h / (H / G)); its output is multiplied by sigmoid((Wg n)_h); then Wo on all heads."""
    t = n.shape[0]
    positions = list(range(t)) if positions is None else positions
    q = (n @ wq.T).view(t, heads, dim)
    k_raw = (n @ wk.T).view(t, kv_heads, dim)
    v = k_raw
    q = unit_rms(q, eps) * query_temperature(positions, coef, every).view(t, 1, 1)
    k = unit_rms(k_raw, eps)
    gate = torch.sigmoid(n @ wg.T)                       # [T, H]
    share = heads // kv_heads
    out = torch.zeros(t, heads, dim, dtype=DT)
    for h in range(heads):
        g = h // share
        for i in range(t):
            scores = (k[: i + 1, g] @ q[i, h]) * scale    # keys 0..i
            weights = torch.softmax(scores, dim=0)
            out[i, h] = (weights.view(-1, 1) * v[: i + 1, g]).sum(dim=0) * gate[i, h]
    return out.reshape(t, heads * dim) @ wo.T


def dense_ff(n: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """Wdown (silu(Wgate n) * (Wup n))."""
    return (silu(n @ w_gate.T) * (n @ w_up.T)) @ w_down.T


class PlainDirozen:
    def __init__(self, config: Dict[str, Any], tensors: Dict[str, torch.Tensor]):
        self.config = config
        self.w = {name: t.to(DT) for name, t in tensors.items()}
        self.eps = float(config["norm"]["eps"])

    @classmethod
    def from_folder(cls, folder: str) -> "PlainDirozen":
        from safetensors import safe_open

        with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as fh:
            config = json.load(fh)
        tensors = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                tensors[name] = f.get_tensor(name)
        return cls(config, tensors)

    def layer(self, i: int, x: torch.Tensor) -> torch.Tensor:
        """x + (mixer(n) + ff(n)) with n = norm1(x); a layer without a feed-forward adds the mixer alone."""
        entry, w, p = self.config["layers"][i], self.w, f"l{i}."
        assert entry["type"] == "attention"
        m = entry["mixer"]
        n = offset_norm(x, w[p + "norm1"], self.eps)
        update = gated_attention(n, w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.g"], w[p + "mix.o"], m["heads"],
                                 m["kv_heads"], m["dim"], m["scale"], m["q_temp"]["coef"], m["q_temp"]["every"], self.eps)
        if entry["mlp"] is not None:
            assert entry["mlp"]["kind"] == "dense"
            update = update + dense_ff(n, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"])
        return x + update

    def residuals(self, ids: List[int]) -> List[torch.Tensor]:
        """The residual stream after every layer."""
        x = self.w["embed"][torch.tensor(ids, dtype=torch.long)]
        out = []
        for i in range(len(self.config["layers"])):
            x = self.layer(i, x)
            out.append(x)
        return out

    def logits(self, ids: List[int]) -> torch.Tensor:
        x = self.residuals(ids)[-1]
        return offset_norm(x, self.w["final.norm"], self.eps) @ self.w["head"].T

    def greedy(self, prompt: List[int], steps: int) -> List[int]:
        ids, out = list(prompt), []
        for _ in range(steps):
            nxt = int(torch.argmax(self.logits(ids)[-1]))
            out.append(nxt)
            ids.append(nxt)
        return out
