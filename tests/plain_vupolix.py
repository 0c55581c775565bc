"""A plain, slow Vupolix in float64 on the CPU: one function per mechanism, written from the
equations, whole sequences at a time, with explicit loops over tokens where a mechanism is
recurrent.  It shares no code with the package; the tests compare the engine with it.

Notation: T tokens, h a sublayer's input [T, width]; weights are [out, in] and applied as x @ W.T.
``w`` maps tensor names to float64 tensors, ``pre`` is a prefix of tensor names ("l3.mix.").
``rnd`` rounds what the engine's bfloat16 mode hands to a matrix product or to the cache (identity: nothing is rounded).
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch

F = torch.float64


def identity(x):
    return x


def round_bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float32).to(torch.bfloat16).to(F)


def to64(tensors: Mapping[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(F) if v.is_floating_point() else v) for k, v in tensors.items()}


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms_unit(x, eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


# ----------------------------------------------------------------------------- wkv

def shifted(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """h_t + (h_(t-1) - h_t) * mu, zeros before the first token."""
    before = torch.cat([torch.zeros(1, h.shape[1], dtype=h.dtype), h[:-1]], 0)
    return h + (before - h) * mu


def wkv_decay(mix_w, w1, w2, w0):
    """exp(-exp(W2 tanh(W1 x) + w0)), one number per head and key channel."""
    return torch.exp(-torch.exp(torch.tanh(mix_w @ w1.T) @ w2.T + w0))


def wkv_recurrence(r, k, v, decay, bonus) -> torch.Tensor:
    """r, k, v, decay [T, heads, dim], bonus [heads, dim].  The token's own k v^T is read through the bonus and joins the
    state, undecayed, afterwards; what was there before is decayed channel by channel."""
    T, H, D = r.shape
    out = torch.zeros(T, H, D, dtype=F)
    for hd in range(H):
        S = torch.zeros(D, D, dtype=F)                     # [key channel, value channel]
        for t in range(T):
            kv = torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = (S + bonus[hd][:, None] * kv).T @ r[t, hd]
            S = decay[t, hd][:, None] * S + kv
    return out


def wkv_mixer(h, w, pre, mixer, eps, rnd=identity):
    H, D = int(mixer["heads"]), int(mixer["dim"])
    T = h.shape[0]
    mix = {s: rnd(shifted(h, w[pre + "mu." + s])) for s in "rkvgw"}
    r = (mix["r"] @ w[pre + "r"].T).view(T, H, D)
    k = (mix["k"] @ w[pre + "k"].T).view(T, H, D)
    v = (mix["v"] @ w[pre + "v"].T).view(T, H, D)
    gate = silu(mix["g"] @ w[pre + "g"].T)
    decay = wkv_decay(mix["w"], w[pre + "w1"], w[pre + "w2"], w[pre + "w0"]).view(T, H, D)
    o = wkv_recurrence(r, k, v, decay, w[pre + "u"].view(H, D))
    o = rms_unit(o, eps).reshape(T, H * D) * w[pre + "norm"] * gate
    return rnd(o) @ w[pre + "o"].T


# ----------------------------------------------------------------------------- rotation

def rotary_frequencies(rot: Mapping):
    """(frequencies [dims/2], factor on cosines and sines).  f_i = base^(-2i/dims); with ``scaling`` the frequencies
    whose index lies beyond a ramp are divided by ``factor``, those inside it are blended."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def index_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(index_of(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return torch.tensor(out, dtype=F), 0.1 * math.log(factor) + 1.0


def rotate_halves(x: torch.Tensor, pos0: int, rot: Mapping) -> torch.Tensor:
    """x [T, heads, dim]: element i < dims/2 of every head is paired with element i + dims/2."""
    T = x.shape[0]
    dims = int(rot["dims"])
    half = dims // 2
    f, mag = rotary_frequencies(rot)
    ang = torch.arange(pos0, pos0 + T, dtype=F)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


# ----------------------------------------------------------------------------- the two side-by-side mixers

def window_sink_attention(q, k, v, scale, window, sink) -> torch.Tensor:
    """q [T, H, D], k, v [T, G, D]; query i sees keys j with 0 <= i - j < window; the softmax's denominator also holds
    exp(sink) per head."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, hd]) * scale
            m = max(float(s.max()), float(sink[hd]))
            e = torch.exp(s - m)
            out[i, hd] = (e[:, None] * v[lo:i + 1, g]).sum(0) / (e.sum() + math.exp(float(sink[hd]) - m))
    return out


def left_mixer(h, w, pre, mixer, pos0=0, rnd=identity):
    H, G, D = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"])
    T = h.shape[0]
    q = (h @ w[pre + "q"].T).view(T, H, D)
    k = (h @ w[pre + "k"].T).view(T, G, D)
    v = k                                               # the values are the keys as projected
    q, k = rotate_halves(q, pos0, mixer["rot"]), rotate_halves(k, pos0, mixer["rot"])
    o = window_sink_attention(rnd(q), rnd(k), rnd(v), float(mixer["scale"]), int(mixer["mask"]["size"]), w[pre + "sink"])
    o = o * torch.sigmoid(h @ w[pre + "g"].T)[:, :, None]
    return rnd(o.reshape(T, -1)) @ w[pre + "o"].T


def retention(q, k, v, decay) -> torch.Tensor:
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T, H, D = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for hd in range(H):
        S = torch.zeros(D, v.shape[2], dtype=F)
        for t in range(T):
            S = float(decay[hd]) * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    return out


def right_mixer(h, w, pre, mixer, eps, pos0=0, rnd=identity):
    H, D, V = int(mixer["heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = rotate_halves((h @ w[pre + "q"].T).view(T, H, D), pos0, mixer["rot"])
    k = rotate_halves((h @ w[pre + "k"].T).view(T, H, D), pos0, mixer["rot"]) * D ** -0.5
    v = (h @ w[pre + "v"].T).view(T, H, V)
    o = rms_unit(retention(q, k, v, mixer["decay"]), eps).reshape(T, H * V) * silu(h @ w[pre + "g"].T)
    return rnd(o) @ w[pre + "o"].T


def parallel_mixer(h, w, pre, mixer, eps, rnd=identity):
    left = left_mixer(h, w, pre + "left.", mixer["left"], rnd=rnd)
    right = right_mixer(h, w, pre + "right.", mixer["right"], eps, rnd=rnd)
    return 0.5 * (rms_norm(left, w[pre + "left.out"], eps) + rms_norm(right, w[pre + "right.out"], eps))


# ----------------------------------------------------------------------------- feed-forward

def route(z: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int):
    """z [experts] -> (chosen experts, their weights).  Scores sigmoid(z); the choice is made on scores + correction among
    the experts of the ``keep`` groups whose two best choice scores add up highest; the weights are the scores themselves."""
    s = torch.sigmoid(z)
    choice = s + correction
    E = z.numel()
    size = E // groups
    if groups > 1:
        gs = [choice[g * size:(g + 1) * size].topk(min(2, size)).values.sum() for g in range(groups)]
        kept = sorted(range(groups), key=lambda g: (-float(gs[g]), g))[:keep]
        masked = torch.full_like(choice, -math.inf)
        for g in kept:
            masked[g * size:(g + 1) * size] = choice[g * size:(g + 1) * size]
        choice = masked
    ids = sorted(range(E), key=lambda e: (-float(choice[e]), e))[:top]
    return ids, [s[e] for e in ids]


def gated_unit(h, w, pre, rnd=identity):
    a = silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)
    return rnd(a) @ w[pre + "down"].T


def moe(h, w, pre, mlp, rnd=identity):
    ro = mlp["router"]
    groups = ro.get("groups") or {"count": 1, "keep": 1}
    out = torch.zeros_like(h)
    z = h @ w[pre + "router"].T
    for t in range(h.shape[0]):
        ids, wts = route(z[t], w[pre + "correction"], int(ro["top"]), int(groups["count"]), int(groups["keep"]))
        for e, s in zip(ids, wts):
            out[t] += s * gated_unit(h[t:t + 1], w, f"{pre}e{e}.", rnd)[0]
    if mlp.get("shared"):
        out = out + gated_unit(h, w, pre + "shared.", rnd)
    return out


# ----------------------------------------------------------------------------- the model

def layer_runs(cfg) -> List[tuple]:
    """(layer, whether the embedding output is added in front of it) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for p in range(times):
        runs += [(i, p > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, w, tokens, rnd=identity, stream_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from its first token.  ``stream_out``: receives the stream after every layer run."""
    eps, m = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    e = rms_norm(w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)], w["embed.norm"], eps)
    x = e.clone()
    for i, add in layer_runs(cfg):
        L, pre = cfg["layers"][i], f"l{i}."
        if add:
            x = x + e
        h = rnd(rms_norm(x, w[pre + "norm1"], eps))
        if L["type"] == "wkv":
            y = wkv_mixer(h, w, pre + "mix.", L["mixer"], eps, rnd)
        else:
            y = parallel_mixer(h, w, pre + "mix.", L["mixer"], eps, rnd)
        x = x + m * rms_norm(y, w[pre + "norm1b"], eps)
        if L.get("mlp") is not None:
            h = rnd(rms_norm(x, w[pre + "norm2"], eps))
            x = x + m * rms_norm(moe(h, w, pre + "mlp.", L["mlp"], rnd), w[pre + "norm2b"], eps)
        if stream_out is not None:
            stream_out.append(x.clone())
    return (rnd(rms_norm(x, w["final.norm"], eps)) @ w["head"].T) * float(cfg["logit_scale"])


def generate_greedy(cfg, w, prompt, new_tokens: int) -> List[int]:
    """The whole sequence recomputed for every new token; the largest logit wins, the lower index among equals."""
    toks, out = list(prompt), []
    for _ in range(new_tokens):
        nxt = int(torch.argmax(forward(cfg, w, toks)[-1]))
        toks.append(nxt)
        out.append(nxt)
    return out


def logits_error(got, want, quantile: float = 1.0) -> float:
    """Per row: the root mean square of the difference (its mean taken off) over that of the wanted row (its mean taken
    off); the given quantile over the rows."""
    g, r = torch.as_tensor(got, dtype=F), torch.as_tensor(want, dtype=F)
    if not torch.isfinite(g).all():
        return math.inf
    d = g - r
    d = d - d.mean(-1, keepdim=True)
    c = r - r.mean(-1, keepdim=True)
    err = torch.sqrt((d * d).mean(-1)) / torch.sqrt((c * c).mean(-1)).clamp_min(1e-30)
    return float(torch.quantile(err, quantile))
