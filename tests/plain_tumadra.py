"""A plain, slow statement of the Tumadra design: float32 (or float64), whole
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


def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    """Reads a safetensors file with nothing but the file format: eight bytes
    of header length, a JSON header, raw little-endian data."""
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16, "I32": torch.int32,
             "I64": torch.int64}
    with open(path, "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        t = torch.frombuffer(bytearray(data[lo:hi]), dtype=kinds[meta["dtype"]])
        out[name] = t.reshape(meta["shape"]).clone()
    return out


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by sqrt(mean(x^2) + eps) along the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def sinusoid(positions: torch.Tensor, width: int, dtype=torch.float32) -> torch.Tensor:
    """Entry 2i is sin(p * 10000^(-2i/width)), entry 2i+1 the cosine of the same angle."""
    i = torch.arange((width + 1) // 2, dtype=dtype)
    inv = torch.pow(torch.tensor(10000.0, dtype=dtype), -2.0 * i / width)
    angle = positions.to(dtype)[:, None] * inv[None, :]
    out = torch.zeros(positions.shape[0], 2 * inv.shape[0], dtype=dtype)
    out[:, 0::2] = torch.sin(angle)
    out[:, 1::2] = torch.cos(angle)
    return out[:, :width]


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """The vector in `groups` equal consecutive parts, each divided by its own
    root mean square, the whole times w."""
    T, E = x.shape
    parts = x.reshape(T, groups, E // groups)
    return rms(parts, eps).reshape(T, E) * w


def token_shift(h: torch.Tensor, mix: torch.Tensor) -> torch.Tensor:
    """h_t + (h_{t-1} - h_t) * mix, with h_{-1} = 0; h_{t-1} is the unshifted one."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (before - h) * mix


def query_temperature(positions: torch.Tensor, coef: float, every: int, dtype=torch.float32) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * torch.log(torch.floor((positions + 1) / every).to(dtype) + 1.0)


def differential_core(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_pos: torch.Tensor, scale: float,
                      lam: float, diff: float, eps: float) -> torch.Tensor:
    """q [Tq, H, 2, D] at positions q_pos, k [Tk, G, 2, D] and v [Tk, G, V] at positions 0..Tk-1:
    per head a1 - lam a2 over the keys j <= q_pos, divided by its root mean square, times 1 - diff.
    Returns [Tq, H * V]."""
    Tq, H = q.shape[0], q.shape[1]
    Tk, G = k.shape[0], k.shape[1]
    seen = torch.arange(Tk)[None, :] <= q_pos[:, None]
    heads = []
    for head in range(H):
        g = head // (H // G)
        maps = []
        for m in range(2):
            s = (q[:, head, m] @ k[:, g, m].T) * scale
            s = s.masked_fill(~seen, float("-inf"))
            maps.append(torch.softmax(s, dim=-1) @ v[:, g])
        heads.append(rms(maps[0] - lam * maps[1], eps) * (1.0 - diff))
    return torch.cat(heads, dim=-1)


def differential_lambda(p: Dict[str, torch.Tensor], diff: float) -> float:
    return float(torch.exp((p["lq1"] * p["lk1"]).sum()) - torch.exp((p["lq2"] * p["lk2"]).sum()) + diff)


def differential_attention(h: torch.Tensor, p: Dict[str, torch.Tensor], c: dict, eps: float) -> torch.Tensor:
    """Two softmax maps per head over shared values, a1 - lambda a2, unit-RMS
    per head times (1 - diff), a sigmoid gate, the output projection."""
    T = h.shape[0]
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = (h @ p["q"].T + p["q.b"]).reshape(T, H, 2, D)
    k = (h @ p["k"].T + p["k.b"]).reshape(T, G, 2, D)
    v = (h @ p["v"].T + p["v.b"]).reshape(T, G, V)
    pos = torch.arange(T)
    if c.get("q_temp"):
        q = q * query_temperature(pos, c["q_temp"]["coef"], c["q_temp"]["every"], h.dtype)[:, None, None, None]
    o = differential_core(q, k, v, pos, c["scale"], differential_lambda(p, c["diff"]), c["diff"], eps)
    return (o * torch.sigmoid(h @ p["g"].T)) @ p["o"].T


def causal_conv(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """out[t, c] = b[c] + sum_j w[c, j] x[t - (taps - 1) + j, c], zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    out = b.expand(T, C).clone()
    for j in range(taps):
        out = out + padded[j:j + T] * w[:, j]
    return out


def scan(dt: torch.Tensor, x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, A: torch.Tensor, D: torch.Tensor,
         S: Optional[torch.Tensor] = None) -> torch.Tensor:
    """S <- exp(dt A) S + dt x B; y = S C + D x, token by token from S = 0 (or the given S, updated in place)."""
    T, inner = x.shape
    if S is None:
        S = torch.zeros(inner, A.shape[1], dtype=x.dtype)
    ys = []
    for t in range(T):
        S.copy_(torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :])
        ys.append(S @ C[t] + D * x[t])
    return torch.stack(ys)


def mamba1(h: torch.Tensor, p: Dict[str, torch.Tensor], c: dict) -> torch.Tensor:
    """Selective scan: in -> (x, z); x through a causal per-channel conv and
    silu; (dt, B, C) from x; S <- exp(dt A) S + dt x B; y = S C + D x; y silu(z); out."""
    inner, N, R = c["inner"], c["state"], c["dt_rank"]
    xz = h @ p["in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = torch.nn.functional.silu(causal_conv(x, p["conv"], p["conv.b"]))
    low = x @ p["x"].T
    dt = torch.nn.functional.softplus(low[:, :R] @ p["dt"].T + p["dt.b"])
    y = scan(dt, x, low[:, R:R + N], low[:, R + N:R + 2 * N], -torch.exp(p["A_log"]), p["D"])
    return (y * torch.nn.functional.silu(z)) @ p["o"].T


def poly_norm_ffn(n: torch.Tensor, p: Dict[str, torch.Tensor], eps: float) -> torch.Tensor:
    """down( a N(z) + b N(z^2) + c N(z^3) + e ), z = up n, N = unit RMS over the hidden width."""
    z = n @ p["up"].T
    a, b, c, e = [float(v) for v in p["act"]]
    act = a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z * z * z, eps) + e
    return act @ p["down"].T


def run_order(config: dict) -> List[int]:
    """Layers start..stop-1 run `times` times in a row, the rest once."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    inside = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + inside * loop["times"] + list(range(loop["stop"], n))


class PlainTumadra:
    def __init__(self, model_dir: str, dtype=torch.float32):
        with open(os.path.join(model_dir, "config.json")) as f:
            self.config = json.load(f)
        raw = read_safetensors(os.path.join(model_dir, "model.safetensors"))
        self.t = {k: v.to(dtype) for k, v in raw.items()}
        self.dtype = dtype
        self.eps = float(self.config["norm"]["eps"])
        self.groups = int(self.config["norm"].get("groups", 1))

    def _sub(self, prefix: str) -> Dict[str, torch.Tensor]:
        return {k[len(prefix):]: v for k, v in self.t.items() if k.startswith(prefix)}

    def layer(self, i: int, x: torch.Tensor) -> torch.Tensor:
        c = self.config["layers"][i]
        t = self.t
        h = token_shift(group_norm(x, t[f"l{i}.norm1"], self.groups, self.eps), t[f"l{i}.shift"])
        if c["type"] == "attention":
            x = x + differential_attention(h, self._sub(f"l{i}.mix."), c["mixer"], self.eps)
        elif c["type"] == "mamba1":
            x = x + mamba1(h, self._sub(f"l{i}.mix."), c["mixer"])
        else:
            raise ValueError(c["type"])
        if c.get("mlp") is not None:
            n = group_norm(x, t[f"l{i}.norm2"], self.groups, self.eps)
            x = x + poly_norm_ffn(n, self._sub(f"l{i}.mlp."), self.eps)
        return x

    def streams(self, tokens: List[int]) -> List[torch.Tensor]:
        """The residual stream after every layer run."""
        ids = torch.tensor(tokens, dtype=torch.long)
        width = self.config["width"]
        x = self.t["embed"][ids] + sinusoid(torch.arange(len(tokens)), width, self.dtype)
        out = []
        for i in run_order(self.config):
            x = self.layer(i, x)
            out.append(x)
        return out

    def logits(self, tokens: List[int]) -> torch.Tensor:
        x = self.streams(tokens)[-1]
        n = group_norm(x, self.t["final.norm"], self.groups, self.eps)
        return (n @ self.t["head"].T).to(torch.float32)

    def greedy(self, prompt: List[int], n: int) -> List[int]:
        seq = list(prompt)
        for _ in range(n):
            seq.append(int(torch.argmax(self.logits(seq)[-1])))
        return seq[len(prompt):]
