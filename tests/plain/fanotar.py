"""A plain, slow implementation of the Fanotar decoder, one function per mechanism, written from
the design's equations with torch on the CPU (64-bit by default). It shares no code with the
engine: it reads config.json and model.safetensors itself. The tests compare the engine with it.

Notation. n(x) = tanh(a x) w + b is the layer norm ("dynamic tanh": a a scalar, w and b vectors).
A layer computes x <- x + n1b(mixer(n1 x)), then x <- x + n2b(ff(n2 x)). The mixer is attention
whose q, k and v rows pass a short causal convolution over time first, with a weighted unit-RMS norm
on q and k heads, a query multiplier that grows with the position, a penalty slope_h (i - j) on the
score of key j for query i, a window, a learned per-head sink in the softmax, and a sigmoid gate on
the heads' output. A layer may read another layer's keys and values instead of making its own. The
feed-forward is a capped gated unit, dense or a mixture of experts with a shared expert.
"""

from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def dynamic_tanh(x: torch.Tensor, alpha: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return torch.tanh(alpha * x) * w + b


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def short_convolution(u: torch.Tensor, w: torch.Tensor, before: torch.Tensor | None = None) -> torch.Tensor:
    """u [n, channels], w [channels, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), with `before`
    ([taps - 1, channels], the rows that came before u; zeros if None) standing in for t < 0."""
    taps = w.shape[1]
    pad = torch.zeros(taps - 1, u.shape[1], dtype=u.dtype) if before is None else before
    full = torch.cat([pad, u])
    y = torch.zeros_like(u)
    for t in range(u.shape[0]):
        for j in range(taps):
            y[t] += w[:, j] * full[t + j]           # full[t + j] is u at time t - taps + 1 + j
    return y


def query_multiplier(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef ln(floor((p + 1) / every) + 1)"""
    return 1.0 + coef * torch.log(torch.floor((positions + 1) / every) + 1.0)


def distance_slopes(heads: int) -> list[float]:
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


def sloped_sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_positions: torch.Tensor, scale: float,
                          slopes: list[float], sinks: torch.Tensor, window: int) -> torch.Tensor:
    """q [n, H, D] at `q_positions` over keys k [m, G, D], values v [m, G, V] at positions 0..m-1.
    s_j = q.k_j scale - slope_h (p - j) for p - window < j <= p; weight_j = exp(s_j) / (exp(sink_h) + sum exp(s))."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        p = int(q_positions[t])
        lo = max(0, p - window + 1) if window else 0
        dist = (p - torch.arange(lo, p + 1)).to(q.dtype)
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:p + 1, g] @ q[t, h]) * scale - slopes[h] * dist
            m = torch.maximum(s.max(), sinks[h])
            e = torch.exp(s - m)
            out[t, h] = (e / (torch.exp(sinks[h] - m) + e.sum())) @ v[lo:p + 1, g]
    return out


def capped_gated_unit(g: torch.Tensor, u: torch.Tensor, limit: float) -> torch.Tensor:
    """min(g, L) sigmoid(1.702 min(g, L)) (clamp(u, -L, L) + 1)"""
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, -limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def route(z: torch.Tensor, correction: torch.Tensor, top: int, scale: float) -> tuple[torch.Tensor, torch.Tensor]:
    """z [n, E] router logits. Returns (chosen [n, top], weights [n, top]): the experts with the largest
    sigmoid(z) + correction, weighted by sigmoid(z) / (sum of the chosen + 1e-20) * scale."""
    s = torch.sigmoid(z)
    chosen = torch.topk(s + correction, top, dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20) * scale


class PlainFanotar:
    def __init__(self, folder: str, dtype: torch.dtype = torch.float64) -> None:
        with open(os.path.join(folder, "config.json")) as f:
            self.cfg = json.load(f)
        self.dtype = dtype
        self.w: dict[str, torch.Tensor] = {}
        with safe_open(os.path.join(folder, "model.safetensors"), "pt", "cpu") as f:
            for name in f.keys():
                self.w[name] = f.get_tensor(name).to(dtype)
        self.eps = self.cfg["norm"]["eps"]

    def norm(self, name: str, x: torch.Tensor) -> torch.Tensor:
        return dynamic_tanh(x, self.w[name + ".alpha"], self.w[name], self.w[name + ".b"])

    def keys_values(self, p: str, m: dict, h: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        n = h.shape[0]
        k = short_convolution(h @ self.w[p + "k"].T, self.w[p + "k.conv"]).view(n, m["kv_heads"], m["dim"])
        v = short_convolution(h @ self.w[p + "v"].T, self.w[p + "v.conv"]).view(n, m["kv_heads"], m["vdim"])
        return unit_rms(k, self.eps) * self.w[p + "k.norm"], v

    def attention(self, p: str, m: dict, h: torch.Tensor, kv: tuple[torch.Tensor, torch.Tensor]) -> torch.Tensor:
        n = h.shape[0]
        pos = torch.arange(n)
        q = short_convolution(h @ self.w[p + "q"].T, self.w[p + "q.conv"]).view(n, m["heads"], m["dim"])
        q = unit_rms(q, self.eps) * self.w[p + "q.norm"]
        if m.get("q_temp"):
            q = q * query_multiplier(pos.to(self.dtype), m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
        o = sloped_sink_attention(q, kv[0], kv[1], pos, m["scale"], distance_slopes(m["heads"]), self.w[p + "sink"],
                                  m["mask"]["size"] if m.get("mask") else 0)
        gate = torch.sigmoid(h @ self.w[p + "g"].T)
        return (o.reshape(n, -1) * gate) @ self.w[p + "o"].T

    def expert(self, p: str, limit: float, h: torch.Tensor) -> torch.Tensor:
        return capped_gated_unit(h @ self.w[p + "gate"].T, h @ self.w[p + "up"].T, limit) @ self.w[p + "down"].T

    def feed_forward(self, p: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
        if mlp["kind"] == "dense":
            return self.expert(p, mlp["limit"], h)
        r = mlp["router"]
        chosen, weights = route(h @ self.w[p + "router"].T, self.w[p + "correction"], r["top"], r["scale"])
        out = torch.zeros_like(h)
        for t in range(h.shape[0]):
            for e, w in zip(chosen[t].tolist(), weights[t]):
                out[t] += w * self.expert(f"{p}e{e}.", mlp["expert"]["limit"], h[t:t + 1])[0]
        if mlp.get("shared"):
            out = out + self.expert(p + "shared.", mlp["shared"]["limit"], h)
        return out

    def streams(self, tokens: list[int]) -> list[torch.Tensor]:
        """The residual stream after every layer."""
        x = self.norm("embed.norm", self.w["embed"][torch.tensor(tokens)] * self.cfg["embedding"]["scale"])
        kept: dict[int, tuple[torch.Tensor, torch.Tensor]] = {}
        out = []
        for i, layer in enumerate(self.cfg["layers"]):
            p, m = f"l{i}.", layer["mixer"]
            h = self.norm(p + "norm1", x)
            if m.get("kv_from") is None:
                kept[i] = self.keys_values(p + "mix.", m, h)
            x = x + self.norm(p + "norm1b", self.attention(p + "mix.", m, h, kept[m["kv_from"] if m.get("kv_from") is not None else i]))
            if layer.get("mlp"):
                x = x + self.norm(p + "norm2b", self.feed_forward(p + "mlp.", layer["mlp"], self.norm(p + "norm2", x)))
            out.append(x)
        return out

    def logits(self, tokens: list[int]) -> torch.Tensor:
        """[len(tokens), vocab]"""
        return self.norm("final.norm", self.streams(tokens)[-1]) @ self.w["head"].T

    def greedy(self, tokens: list[int], n: int) -> list[int]:
        ids, out = list(tokens), []
        for _ in range(n):
            tok = int(self.logits(ids)[-1].argmax())
            out.append(tok)
            ids.append(tok)
        return out
