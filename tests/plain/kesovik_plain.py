"""A plain, slow Kesovik decoder: whole sequences, no cache, one function per mechanism, float64 on the CPU.
It shares no code with ``pulse_infer_amd``: it reads a model folder with ``json`` and the ``safetensors`` package
(or takes a dictionary of tensors) and is written from the design's equations.  Tests compare the engine with it.

Notation: x [T, W] the stream, p the position of a token (from 0 in each sequence), W_foo a weight stored [out, in].
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


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def decayed_state_walk(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: List[float],
                       state: Optional[torch.Tensor] = None):
    """Per head h, token by token: S <- decay_h S + k_t v_t^T, o_t = S^T q_t.  q, k [T, H, d], v [T, H, dv];
    returns (o [T, H, dv], the last state [H, d, dv])."""
    t, heads, d = q.shape
    dv = v.shape[2]
    s = torch.zeros(heads, d, dv, dtype=DT) if state is None else state.clone()
    out = torch.zeros(t, heads, dv, dtype=DT)
    for i in range(t):
        for h in range(heads):
            s[h] = decay[h] * s[h] + torch.outer(k[i, h], v[i, h])
            out[i, h] = s[h].T @ q[i, h]
    return out, s


def lightning_mixer(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], eps: float) -> torch.Tensor:
    """q, k, v = silu of their projections; the walk above; the heads together normed with a weight, times
    sigmoid(W_g x), then W_o."""
    t, heads, d, dv = x.shape[0], m["heads"], m["dim"], m["vdim"]
    q = silu(x @ w[p + ".q"].T).view(t, heads, d)
    k = silu(x @ w[p + ".k"].T).view(t, heads, d)
    v = silu(x @ w[p + ".v"].T).view(t, heads, dv)
    o, _ = decayed_state_walk(q, k, v, m["decay"])
    y = unit_rms(o.reshape(t, heads * dv), eps) * w[p + ".norm"] * torch.sigmoid(x @ w[p + ".g"].T)
    return y @ w[p + ".o"].T


def rotate_pairs(x: torch.Tensor, positions: List[int], base: float, dims: int) -> torch.Tensor:
    """Channels (2i, 2i+1), i < dims / 2, of every head turned by p * base^(-2i/dims); x [T, heads, d]."""
    out = x.clone()
    pos = torch.tensor(positions, dtype=DT).view(-1, 1, 1)
    i = torch.arange(dims // 2, dtype=DT)
    angle = pos * (base ** (-2.0 * i / dims)).view(1, 1, -1)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * torch.cos(angle) - v * torch.sin(angle)
    out[..., 1:dims:2] = v * torch.cos(angle) + u * torch.sin(angle)
    return out


def window_scores_softmax(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int,
                          positions: Optional[List[int]] = None) -> torch.Tensor:
    """Grouped softmax attention of a whole sequence: token i sees j with 0 <= i - j < window.
    q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]."""
    t, heads, _ = q.shape
    share = heads // k.shape[1]
    out = torch.zeros(t, heads, v.shape[2], dtype=DT)
    for i in range(t):
        lo = max(0, i - window + 1)
        for h in range(heads):
            g = h // share
            weights = torch.softmax((k[lo:i + 1, g] @ q[i, h]) * scale, dim=0)
            out[i, h] = (weights.view(-1, 1) * v[lo:i + 1, g]).sum(dim=0)
    return out


def window_attention(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Biased projections; q and k each normed over the whole projection (a weight per channel); rotation; windowed
    softmax attention; W_o."""
    t, heads, groups, d, dv = x.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = x @ w[p + ".q"].T + w[p + ".q.b"]
    k = x @ w[p + ".k"].T + w[p + ".k.b"]
    v = x @ w[p + ".v"].T + w[p + ".v.b"]
    q = (unit_rms(q, eps) * w[p + ".q.norm"]).view(t, heads, d)
    k = (unit_rms(k, eps) * w[p + ".k.norm"]).view(t, groups, d)
    positions = list(range(t))
    if m.get("rot") is not None:                  # (a configuration that names no rotation has none)
        q = rotate_pairs(q, positions, m["rot"]["base"], m["rot"]["dims"])
        k = rotate_pairs(k, positions, m["rot"]["base"], m["rot"]["dims"])
    window = m["mask"]["size"] if m.get("mask") is not None else t      # (and one that names no mask sees all before)
    o = window_scores_softmax(q, k, v.view(t, groups, dv), m["scale"], window)
    return o.reshape(t, heads * dv) @ w[p + ".o"].T


def squared_relu_ff(x: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    return (torch.relu(x @ w_up.T) ** 2) @ w_down.T


def gated_expert(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def route(z: torch.Tensor, correction: torch.Tensor, top: int):
    """Softmax scores over all router outputs; the ``top`` largest of score + correction; weights = the chosen scores
    over their sum (+ 1e-20).  Returns (indices [T, top], weights [T, top])."""
    s = torch.softmax(z, dim=-1)
    chosen = torch.topk(s + correction, top, dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(dim=-1, keepdim=True) + 1e-20)


def routed_ff(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any]) -> torch.Tensor:
    """Outputs below router.experts are gated experts, the rest give x itself back; a shared expert is added."""
    experts, top = m["router"]["experts"], m["router"]["top"]
    chosen, weights = route(x @ w[p + ".router"].T, w[p + ".correction"], top)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            if e >= experts:
                out[t] += a * x[t]
            else:
                out[t] += a * gated_expert(x[t], w[f"{p}.e{e}.gate"], w[f"{p}.e{e}.up"], w[f"{p}.e{e}.down"])
    if m.get("shared") is not None:
        out = out + gated_expert(x, w[p + ".shared.gate"], w[p + ".shared.up"], w[p + ".shared.down"])
    return out


class PlainKesovik:
    def __init__(self, config: Dict[str, Any], tensors: Dict[str, torch.Tensor]):
        self.config = config
        self.w = {name: t.to(DT) for name, t in tensors.items()}
        self.eps = float(config["norm"]["eps"])
        self.alpha = float(config.get("postln_alpha", 1.0))

    @classmethod
    def from_folder(cls, folder: str) -> "PlainKesovik":
        from safetensors import safe_open

        with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as fh:
            config = json.load(fh)
        tensors = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                tensors[name] = f.get_tensor(name)
        return cls(config, tensors)

    def mixer(self, i: int, x: torch.Tensor) -> torch.Tensor:
        entry, p = self.config["layers"][i], f"l{i}.mix"
        m = entry["mixer"]
        if entry["type"] == "lightning":
            return lightning_mixer(x, self.w, p, m, self.eps)
        assert entry["type"] == "parallel"
        return (m["left_scale"] * window_attention(x, self.w, p + ".left", m["left"], self.eps)
                + m["right_scale"] * lightning_mixer(x, self.w, p + ".right", m["right"], self.eps))

    def feed_forward(self, i: int, x: torch.Tensor) -> torch.Tensor:
        m, p = self.config["layers"][i]["mlp"], f"l{i}.mlp"
        if m["kind"] == "dense":
            return squared_relu_ff(x, self.w[p + ".up"], self.w[p + ".down"])
        assert m["kind"] == "moe"
        return routed_ff(x, self.w, p, m)

    def layer(self, i: int, x: torch.Tensor) -> torch.Tensor:
        """x <- norm1(alpha x + ls1 * mixer(x)); x <- norm2(alpha x + ls2 * ff(x)); the sublayers read x itself."""
        w, p = self.w, f"l{i}."
        x = unit_rms(self.alpha * x + w[p + "ls1"] * self.mixer(i, x), self.eps) * w[p + "norm1"]
        if self.config["layers"][i]["mlp"] is not None:
            x = unit_rms(self.alpha * x + w[p + "ls2"] * self.feed_forward(i, x), self.eps) * w[p + "norm2"]
        return x

    def router_margins(self, ids: List[int]) -> torch.Tensor:
        """Per position, the smallest distance over the routed layers between the last chosen router output and the
        best one not chosen (score + correction): where it is tiny, an implementation in reduced precision may
        rightly choose otherwise."""
        x = self.w["embed"][torch.tensor(ids, dtype=torch.long)] * float(self.config["embedding"]["scale"])
        least = torch.full((len(ids),), float("inf"), dtype=DT)
        for i, entry in enumerate(self.config["layers"]):
            w, p, m = self.w, f"l{i}.", entry["mlp"]
            x = unit_rms(self.alpha * x + w[p + "ls1"] * self.mixer(i, x), self.eps) * w[p + "norm1"]
            if m is None:
                continue
            if m["kind"] == "moe":
                c = torch.softmax(x @ w[p + "mlp.router"].T, dim=-1) + w[p + "mlp.correction"]
                top = m["router"]["top"]
                if top < c.shape[1]:
                    ranked = torch.sort(c, dim=-1, descending=True).values
                    least = torch.minimum(least, ranked[:, top - 1] - ranked[:, top])
            x = unit_rms(self.alpha * x + w[p + "ls2"] * self.feed_forward(i, x), self.eps) * w[p + "norm2"]
        return least

    def residuals(self, ids: List[int]) -> List[torch.Tensor]:
        """The stream after every layer."""
        x = self.w["embed"][torch.tensor(ids, dtype=torch.long)] * float(self.config["embedding"]["scale"])
        out = []
        for i in range(len(self.config["layers"])):
            x = self.layer(i, x)
            out.append(x)
        return out

    def logits(self, ids: List[int]) -> torch.Tensor:
        x = self.residuals(ids)[-1]
        z = (unit_rms(x, self.eps) * self.w["final.norm"]) @ self.w["head"].T
        cap = float(self.config.get("logit_softcap") or 0.0)
        return cap * torch.tanh(z / cap) if cap else z

    def greedy(self, prompt: List[int], steps: int) -> List[int]:
        ids, out = list(prompt), []
        for _ in range(steps):
            nxt = int(torch.argmax(self.logits(ids)[-1]))
            out.append(nxt)
            ids.append(nxt)
        return out
