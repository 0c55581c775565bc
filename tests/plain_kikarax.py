"""A plain, slow Kikarax in float64 on the CPU: one function per mechanism, written from the equations, whole
sequences at a time.  It shares no code with the package; the tests compare the engine with it.

Notation: T tokens, h a sublayer's input [T, width]; weights are [out, in] and applied as x @ W.T.
``w`` maps tensor names to float64 tensors, ``pre`` is a layer's prefix ("l3.").
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch

F = torch.float64


def to64(tensors: Mapping[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(F) if v.is_floating_point() else v) for k, v in tensors.items()}


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


# ------------------------------------------------------------------------------ embedding

def bigram_rows(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the pair table for every token: a hash of (token before, token); the sequence's first token has
    the row behind the hashed ones."""
    return [buckets if t == 0 else (tokens[t - 1] * mul_prev + tokens[t] * mul_cur) % buckets for t in range(len(tokens))]


def embed(cfg: Mapping, w: Mapping[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    e = cfg["embedding"]
    x = w["embed"][tokens] * float(e["scale"])
    bg = e.get("bigram")
    if bg:
        x = x + w["bigram"][bigram_rows(tokens, int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"]))]
    return x + w["pos"][:len(tokens)]


# ------------------------------------------------------------------------------ attention

def visible(T: int, chunk: Optional[int]) -> torch.Tensor:
    """[T, T] mask: query i sees key j <= i; with chunks of ``chunk`` positions counted from 0 only keys of its own chunk."""
    i = torch.arange(T).unsqueeze(1)
    j = torch.arange(T).unsqueeze(0)
    m = j <= i
    if chunk:
        m = m & (i // chunk == j // chunk)
    return m


def soft_cap(s: torch.Tensor, cap: Optional[float]) -> torch.Tensor:
    return s if not cap else cap * torch.tanh(s / cap)


def mix_values(v: torch.Tensor, v_first: Optional[torch.Tensor], lam: torch.Tensor) -> torch.Tensor:
    return v if v_first is None else (1.0 - lam) * v + lam * v_first


def attention(m: Mapping, w: Mapping[str, torch.Tensor], pre: str, h: torch.Tensor, eps: float, shared: dict) -> torch.Tensor:
    """``shared``: what layers hand to later ones within a pass (the first value-mixing layer's values)."""
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms_norm(h @ w[pre + "mix.q"].T, w[pre + "mix.q.norm"], eps)          # over all heads at once
    k = rms_norm(h @ w[pre + "mix.k"].T, w[pre + "mix.k.norm"], eps)
    v = h @ w[pre + "mix.v"].T
    if m.get("v_mix"):
        if "v_first" in shared:
            v = mix_values(v, shared["v_first"], w[pre + "mix.vmix"])
        else:
            shared["v_first"] = v
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, V)
    mask = visible(T, (m.get("mask") or {}).get("size"))
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        g = head // (H // G)
        s = soft_cap((q[:, head] @ k[:, g].T) * float(m["scale"]), m.get("softcap"))
        s = s.masked_fill(~mask, -math.inf)
        out[:, head] = torch.softmax(s, -1) @ v[:, g]
    gate = torch.sigmoid(h @ w[pre + "mix.g"].T)
    return (out.reshape(T, H * V) * gate) @ w[pre + "mix.o"].T


# ------------------------------------------------------------------------------ feed-forwards

def dense_ff(p: Mapping, w: Mapping[str, torch.Tensor], pre: str, h: torch.Tensor) -> torch.Tensor:
    lim = float(p["limit"])
    g = torch.clamp(h @ w[pre + "gate"].T, max=lim)
    u = torch.clamp(h @ w[pre + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def silu_expert(w: Mapping[str, torch.Tensor], pre: str, h: torch.Tensor) -> torch.Tensor:
    g = h @ w[pre + "gate"].T
    return (g * torch.sigmoid(g) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(z: torch.Tensor, top: int, scale: float):
    """(indices [T, top], weights [T, top]) of the ``top`` largest softmax scores, scaled and not renormalized."""
    s = torch.softmax(z, -1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val * scale


def moe_ff(p: Mapping, w: Mapping[str, torch.Tensor], pre: str, h: torch.Tensor) -> torch.Tensor:
    r = p["router"]
    idx, wt = route(h @ w[pre + "router"].T, int(r["top"]), float(r.get("scale", 1.0)))
    y = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            y[t] += wt[t, j] * silu_expert(w, f"{pre}e{int(idx[t, j])}.", h[t:t + 1])[0]
    if p.get("shared"):
        y = y + torch.sigmoid(h @ w[pre + "shared.sg"].T) * silu_expert(w, pre + "shared.", h)
    return y


# ------------------------------------------------------------------------------ the model

def forward(cfg: Mapping, w: Mapping[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from its first token on."""
    eps = float(cfg["norm"]["eps"])
    x = embed(cfg, w, list(tokens))
    shared: dict = {}
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        if layer["type"] != "attention":
            raise ValueError(layer["type"])
        x = x + attention(layer["mixer"], w, pre, rms_norm(x, w[pre + "norm1"], eps), eps, shared)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, w[pre + "norm2"], eps)
            x = x + (dense_ff(mlp, w, pre + "mlp.", h) if mlp["kind"] == "dense" else moe_ff(mlp, w, pre + "mlp.", h))
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms_norm(x, w["final.norm"], eps) @ w["embed"].T) * float(cfg["logit_scale"])


def generate_greedy(cfg: Mapping, w: Mapping[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    """``n`` tokens, each the largest logit of the whole sequence so far run from its first token."""
    toks, out = list(prompt), []
    for _ in range(n):
        t = int(torch.argmax(forward(cfg, w, toks)[-1]))
        toks.append(t)
        out.append(t)
    return out


def logits_error(got, want, quantile: float = 1.0) -> float:
    """Per row: the root mean square of the difference (its mean taken off) over that of the wanted row (its mean taken
    off); the given quantile over the rows."""
    g, r = torch.as_tensor(got, dtype=F), torch.as_tensor(want, dtype=F)
    d = g - r
    d = d - d.mean(-1, keepdim=True)
    c = r - r.mean(-1, keepdim=True)
    err = torch.sqrt((d * d).mean(-1)) / torch.sqrt((c * c).mean(-1)).clamp_min(1e-30)
    if not torch.isfinite(g).all():
        return math.inf
    return float(torch.quantile(err, quantile))
