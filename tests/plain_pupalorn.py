"""A plain, slow statement of the Pupalorn design: float32 (or float64), whole
sequences, no cache, one function per mechanism. It shares no code with the
engine: tests hold the engine against it.

Notation: a sequence is a [tokens, width] matrix; positions count from 0; a
linear weight is [out, in] and applied as x @ W.T.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

from plain_tumadra import read_safetensors, rms


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose file keeps w - 1: x / rms(x) * (1 + w)."""
    return rms(x, eps) * (1.0 + w)


def inverse_frequencies(dims: int, base: float, scaling: Optional[dict], dtype=torch.float64) -> torch.Tensor:
    """f_i = base^(-2i/dims) for i < dims/2. With `scaling` (factor, low, high,
    original) a frequency whose wavelength 2 pi / f is longer than original/low
    is divided by factor, one shorter than original/high is kept, and between
    the two it is blended by s = (original / wavelength - low) / (high - low)."""
    i = torch.arange(dims // 2, dtype=dtype)
    f = torch.pow(torch.tensor(base, dtype=dtype), -2.0 * i / dims)
    if scaling is None:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.clone()
    for n in range(f.shape[0]):
        wavelength = 2.0 * math.pi / float(f[n])
        if wavelength < original / high:
            continue
        if wavelength > original / low:
            out[n] = f[n] / factor
        else:
            s = (original / wavelength - low) / (high - low)
            out[n] = (1.0 - s) * f[n] / factor + s * f[n]
    return out


def rotate(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """x [tokens, heads, dim]: the first 2 * len(freq) dimensions of each head
    are rotated, dimension i together with dimension i + len(freq)."""
    half = freq.shape[0]
    if half == 0:
        return x
    angle = (positions.to(x.dtype)[:, None] * freq.to(x.dtype)[None, :])[:, None, :]
    c, s = torch.cos(angle), torch.sin(angle)
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], dim=-1)


def keys_and_values(h, positions, Wk, Wv, k_norm, eps, kv_heads, dim, vdim, freq):
    """What a layer's cache holds: normed, rotated keys [tokens, kv_heads, dim] and values [tokens, kv_heads, vdim]."""
    T = h.shape[0]
    k = (h @ Wk.T).reshape(T, kv_heads, dim)
    k = rotate(rms(k, eps) * k_norm, positions, freq)
    v = (h @ Wv.T).reshape(T, kv_heads, vdim)
    return k, v


def windowed_attention(q, k, v, positions, scale: float, window: Optional[int]) -> torch.Tensor:
    """q [T, H, dim], k [T, G, dim], v [T, G, vdim] -> [T, H * vdim]. Query at
    position i sees the keys at positions j with 0 <= i - j (< window)."""
    T, H, _ = q.shape
    G = k.shape[1]
    per = H // G
    dist = positions[:, None] - positions[None, :]
    seen = dist >= 0
    if window is not None:
        seen = seen & (dist < window)
    out = []
    for hd in range(H):
        g = hd // per
        s = (q[:, hd, :] @ k[:, g, :].T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out.append(torch.softmax(s, dim=-1) @ v[:, g, :])
    return torch.cat(out, dim=-1)


def route(h: torch.Tensor, Wr: torch.Tensor, correction: torch.Tensor, top: int):
    """-> (chosen [T, top] indices, weights [T, top]). Scores are a softmax over
    all router outputs; the choice is by score + correction, the weights are the
    scores themselves, as they are."""
    s = torch.softmax(h @ Wr.T, dim=-1)
    chosen = torch.topk(s + correction, top, dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def expert(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return torch.relu(h @ up.T).square() @ down.T


def mixture(h, Wr, correction, top, ups: List[torch.Tensor], downs: List[torch.Tensor]) -> torch.Tensor:
    """Router outputs past the last real expert pass the input through."""
    chosen, weights = route(h, Wr, correction, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            y = expert(h[t:t + 1], ups[e], downs[e])[0] if e < len(ups) else h[t]
            out[t] += w * y
    return out


class PlainPupalorn:
    def __init__(self, model_dir: str, dtype=torch.float32):
        with open(os.path.join(model_dir, "config.json")) as f:
            self.cfg = json.load(f)
        self.dtype = dtype
        self.w = {k: v.to(dtype) for k, v in read_safetensors(os.path.join(model_dir, "model.safetensors")).items()}

    def _freq(self, mixer) -> torch.Tensor:
        rot = mixer.get("rot")
        if not rot:
            return torch.zeros(0, dtype=self.dtype)
        return inverse_frequencies(rot["dims"], rot["base"], rot.get("scaling")).to(torch.float32).to(self.dtype)

    def forward(self, tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
        """Logits [tokens, vocab]; `layers_out` collects the stream after every layer."""
        cfg, w = self.cfg, self.w
        eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
        T = len(tokens)
        positions = torch.arange(T)
        x = w["embed"][torch.tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
        kept = {}
        for i, layer in enumerate(cfg["layers"]):
            L, mx = f"l{i}", layer["mixer"]
            H, G, dim, vdim = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            freq = self._freq(mx)
            h = offset_norm(x, w[f"{L}.norm1"], eps)
            q = (h @ w[f"{L}.mix.q"].T).reshape(T, H, dim)
            q = rotate(rms(q, eps) * w[f"{L}.mix.q.norm"], positions, freq)
            if mx.get("kv_from") is None:
                kept[i] = keys_and_values(h, positions, w[f"{L}.mix.k"], w[f"{L}.mix.v"], w[f"{L}.mix.k.norm"], eps,
                                          G, dim, vdim, freq)
                k, v = kept[i]
            else:
                k, v = kept[mx["kv_from"]]
            window = (mx.get("mask") or {}).get("size")
            a = windowed_attention(q, k, v, positions, mx["scale"], window) @ w[f"{L}.mix.o"].T
            x = x + m * offset_norm(a, w[f"{L}.norm1b"], eps) * w[f"{L}.ls1"]
            mlp = layer.get("mlp")
            if mlp is not None:
                h = offset_norm(x, w[f"{L}.norm2"], eps)
                r = mlp["router"]
                ups = [w[f"{L}.mlp.e{e}.up"] for e in range(r["experts"])]
                downs = [w[f"{L}.mlp.e{e}.down"] for e in range(r["experts"])]
                f = mixture(h, w[f"{L}.mlp.router"], w[f"{L}.mlp.correction"], r["top"], ups, downs)
                x = x + m * offset_norm(f, w[f"{L}.norm2b"], eps) * w[f"{L}.ls2"]
            if layers_out is not None:
                layers_out.append(x.clone())
        return offset_norm(x, w["final.norm"], eps) @ w["head"].T

    def logits(self, tokens: List[int], order=None) -> torch.Tensor:
        return self.forward(list(tokens)).to(torch.float32)

    def greedy(self, prompt: List[int], n: int) -> List[int]:
        tokens, out = list(prompt), []
        for _ in range(n):
            out.append(int(self.forward(tokens)[-1].argmax()))
            tokens.append(out[-1])
        return out
