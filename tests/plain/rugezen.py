"""A plain, slow implementation of the Rugezen decoder, one function per mechanism, written from
the design's equations with torch on the CPU (64-bit by default). It shares no code with the
engine: it reads config.json and model.safetensors itself. The tests compare the engine with it.

Notation: a layer computes x <- x + m (mixer(n1(x)) + ff(n2(x))), n(x) = x / sqrt(mean(x^2) + eps) * w.
"""

from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def weighted_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def turn_pairs(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, interleaved: bool = True) -> torch.Tensor:
    """Rotary positions on the first `dims` dimensions of each head of x [tokens, heads, size]: pair i
    is (2i, 2i+1) if `interleaved`, else (i, i + dims/2); (u, v) -> (u cos a - v sin a, v cos a + u sin a),
    a = position * base^(-2i/dims)."""
    out = x.clone()
    for i in range(dims // 2):
        a = positions.to(x.dtype) * base ** (-2.0 * i / dims)
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        j, k = (2 * i, 2 * i + 1) if interleaved else (i, i + dims // 2)
        u, v = x[..., j], x[..., k]
        out[..., j] = u * c - v * s
        out[..., k] = v * c + u * s
    return out


def sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_positions: torch.Tensor, scale: float,
                   softcap: float = 0.0, sink: bool = True, window: int = 0) -> torch.Tensor:
    """q [n, H, D] at `q_positions` over keys k [m, G, D] and values v [m, G, V] at positions 0..m-1,
    causal: weight_j = exp(s_j) / (sink + sum_visible exp(s)), s = cap(q.k * scale)."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        p = int(q_positions[t])
        lo = max(0, p - window + 1) if window else 0
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:p + 1, g] @ q[t, h]) * scale
            if softcap > 0:
                s = softcap * torch.tanh(s / softcap)
            e = torch.exp(s)
            out[t, h] = (e / ((1.0 if sink else 0.0) + e.sum())) @ v[lo:p + 1, g]
    return out


def mingru_walk(z_in: torch.Tensor, x_in: torch.Tensor, g_in: torch.Tensor, state: torch.Tensor
                ) -> tuple[torch.Tensor, torch.Tensor]:
    """Token by token: z = sigmoid(z_in), c = x_in + 1/2 where x_in >= 0 else sigmoid(x_in),
    S <- (1 - z) S + z c; returns (S_t * silu(g_t) for every t, the last S)."""
    S = state.clone()
    rows = []
    for t in range(z_in.shape[0]):
        z = torch.sigmoid(z_in[t])
        c = torch.where(x_in[t] >= 0, x_in[t] + 0.5, torch.sigmoid(x_in[t]))
        S = (1 - z) * S + z * c
        rows.append(S * g_in[t] * torch.sigmoid(g_in[t]))
    return (torch.stack(rows) if rows else z_in.new_zeros((0, z_in.shape[1]))), S


def squared_relu(z: torch.Tensor) -> torch.Tensor:
    return torch.relu(z) ** 2


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


class PlainRugezen:
    def __init__(self, folder: str, dtype: torch.dtype = torch.float64) -> None:
        with open(os.path.join(folder, "config.json")) as f:
            self.cfg = json.load(f)
        self.dtype = dtype
        self.w: dict[str, torch.Tensor] = {}
        with safe_open(os.path.join(folder, "model.safetensors"), "pt", "cpu") as f:
            for name in f.keys():
                self.w[name] = f.get_tensor(name).to(dtype)
        self.eps = self.cfg["norm"]["eps"]

    def order(self) -> list[int]:
        n, loop = len(self.cfg["layers"]), self.cfg.get("loop")
        if not loop:
            return list(range(n))
        return list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] + list(range(loop["stop"], n))

    def attention(self, p: str, m: dict, h: torch.Tensor) -> torch.Tensor:
        n = h.shape[0]
        q = (h @ self.w[p + "q"].T).view(n, m["heads"], m["dim"])
        k = (h @ self.w[p + "k"].T).view(n, m["kv_heads"], m["dim"])
        v = (h @ self.w[p + "v"].T).view(n, m["kv_heads"], m["vdim"])
        pos = torch.arange(n)
        q = unit_rms(turn_pairs(q, pos, m["rot"]["dims"], m["rot"]["base"]), self.eps)
        k = unit_rms(turn_pairs(k, pos, m["rot"]["dims"], m["rot"]["base"]), self.eps)
        v = unit_rms(v, self.eps)
        o = sink_attention(q, k, v, pos, m["scale"], m["softcap"], sink=True)
        return o.reshape(n, -1) @ self.w[p + "o"].T

    def mingru(self, p: str, m: dict, h: torch.Tensor) -> torch.Tensor:
        z = h @ self.w[p + "z"].T + self.w[p + "z.b"]
        x = h @ self.w[p + "x"].T + self.w[p + "x.b"]
        g = h @ self.w[p + "g"].T
        rows, _ = mingru_walk(z, x, g, torch.zeros(m["width"], dtype=self.dtype))
        return rows @ self.w[p + "o"].T

    def feed_forward(self, p: str, h: torch.Tensor) -> torch.Tensor:
        return squared_relu(h @ self.w[p + "up"].T + self.w[p + "up.b"]) @ self.w[p + "down"].T + self.w[p + "down.b"]

    def streams(self, tokens: list[int]) -> list[torch.Tensor]:
        """The residual stream after every layer run."""
        x = self.w["embed"][torch.tensor(tokens)]
        mult = self.cfg["residual_mult"]
        out = []
        for i in self.order():
            layer, p = self.cfg["layers"][i], f"l{i}."
            h1 = weighted_norm(x, self.w[p + "norm1"], self.eps)
            mixer = self.attention if layer["type"] == "attention" else self.mingru
            add = mixer(p + "mix.", layer["mixer"], h1)
            if layer.get("mlp"):
                add = add + self.feed_forward(p + "mlp.", weighted_norm(x, self.w[p + "norm2"], self.eps))
            x = x + mult * add
            out.append(x)
        return out

    def logits(self, tokens: list[int]) -> torch.Tensor:
        """[len(tokens), vocab]"""
        x = self.streams(tokens)[-1]
        return weighted_norm(x, self.w["final.norm"], self.eps) @ self.w["head"].T

    def greedy(self, tokens: list[int], n: int) -> list[int]:
        ids, out = list(tokens), []
        for _ in range(n):
            tok = int(self.logits(ids)[-1].argmax())
            out.append(tok)
            ids.append(tok)
        return out
