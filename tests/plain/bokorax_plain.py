"""Plain implementation of the Bokorax decoder: float64, whole sequences, no cache, one function per mechanism.

It shares no code with the package: it reads the ``config.json`` dictionary and the stored tensors by their names.
For tokens ``t_0 .. t_{n-1}`` at places ``0 .. n-1`` (``rms(y) = y / sqrt(mean(y^2) + eps)``):

* ``x = embed[t_p] * embedding.scale``
* a layer: ``x <- x + rms(mixer(x)) (1 + norm1)``, then ``x <- x + rms(ff(x)) (1 + norm2)``: the sublayers read the
  stream itself, the norm stands behind them
* mixer ``attention``: grouped heads whose values are the keys as projected; queries and keys normalised over their
  whole projection, partly rotated, a sliding window, an ordinary softmax
* mixer ``attention_2``: grouped heads, queries and keys normalised head by head, rotated with stretched
  frequencies, capped scores, every ``j <= i`` seen, a valueless term per head in the softmax, a gate of one number per
  head; such a layer may read the keys and values of an earlier one
* mixer ``wkv``: a token-shifted linear recurrence with a decay per channel that depends on the input
* ``ff``: routed experts with identity experts, groups of experts, a shared expert behind a gate
* logits ``head @ (rms(x) (1 + final.norm)) * logit_scale``.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64


def rms(y: torch.Tensor, eps: float) -> torch.Tensor:
    return y / torch.sqrt((y * y).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The norm of a layer: the weight is stored around zero."""
    return rms(y, eps) * (1.0 + w)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ---------------------------------------------------------------------------------------------- rotation
def frequencies(rot: dict) -> List[float]:
    """``f_i = base ** (-2 i / dims)``, every one divided by ``scaling.factor`` where ``rot`` has a scaling."""
    dims, base = int(rot["dims"]), float(rot["base"])
    factor = float(rot["scaling"]["factor"]) if rot.get("scaling") else 1.0
    return [base ** (-2.0 * i / dims) / factor for i in range(dims // 2)]


def rotate_halves(x: torch.Tensor, places: Sequence[int], freqs: Sequence[float]) -> torch.Tensor:
    """``x`` ``[n, heads, d]``: channels ``i`` and ``i + len(freqs)`` of every head turn by ``place * freqs[i]``; channels
    behind ``2 len(freqs)`` stay."""
    out = x.clone()
    half = len(freqs)
    p = torch.tensor(list(places), dtype=F64)[:, None]
    for i, f in enumerate(freqs):
        c, s = torch.cos(p * f), torch.sin(p * f)
        u, v = x[:, :, i], x[:, :, i + half]
        out[:, :, i] = u * c - v * s
        out[:, :, i + half] = v * c + u * s
    return out


# ---------------------------------------------------------------------------------------------- softmax attention
def window_mask(n: int, size: Optional[int]) -> torch.Tensor:
    """``seen[i, j]``: ``0 <= i - j`` and, with a window, ``i - j < size``."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if size is not None:
        seen = seen & (i - j < size)
    return seen


def softmax_weights(scores: torch.Tensor, seen: torch.Tensor, sink: Optional[float] = None) -> torch.Tensor:
    """``scores`` ``[nq, nk]``: ``exp(s_j) / (sum over seen j of exp(s_j) [+ exp(sink)])``, 0 for unseen ``j``."""
    s = scores.masked_fill(~seen, -math.inf)
    top = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        top = torch.clamp(top, min=float(sink))
    e = torch.exp(s - top)
    total = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(torch.tensor(float(sink), dtype=F64) - top)
    return e / total


def grouped_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, seen: torch.Tensor,
                      softcap: Optional[float] = None, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``q`` ``[n, H, d]``, ``k`` ``[n, G, d]``, ``v`` ``[n, G, dv]``; query head ``h`` reads kv head ``h // (H / G)``.
    Returns ``[n, H, dv]``."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap is not None:
            s = softcap * torch.tanh(s / softcap)
        w = softmax_weights(s, seen, None if sinks is None else float(sinks[h]))
        out[:, h] = w @ v[:, g]
    return out


def attention_keys_as_values(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Mixer ``attention``: returns ``[n, width]``."""
    n = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = h @ w[p + "q"].T
    k = h @ w[p + "k"].T
    v = k.reshape(n, G, d)                                   # as projected: before norm and rotation
    q = (rms(q, eps) * w[p + "q.norm"]).reshape(n, H, d)     # one root mean square over the whole projection
    k = (rms(k, eps) * w[p + "k.norm"]).reshape(n, G, d)
    freqs = frequencies(m["rot"])
    q, k = rotate_halves(q, range(n), freqs), rotate_halves(k, range(n), freqs)
    mask = m.get("mask")
    o = grouped_attention(q, k, v, float(m["scale"]), window_mask(n, int(mask["size"]) if mask else None))
    return o.reshape(n, -1) @ w[p + "o"].T


def attention_2_keys_values(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float):
    """Keys (normalised head by head, rotated) and values of an ``attention_2`` layer with projections of its own."""
    n = h.shape[0]
    G, d, dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    k = (h @ w[p + "k"].T).reshape(n, G, d)
    k = rms(k, eps) * w[p + "k.norm"]
    k = rotate_halves(k, range(n), frequencies(m["rot"]))
    v = (h @ w[p + "v"].T).reshape(n, G, dv)
    return k, v


def attention_2(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Mixer ``attention_2`` over the given keys and values (its own, or those of the layer ``kv_from`` names)."""
    n = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    q = (h @ w[p + "q"].T).reshape(n, H, d)
    q = rms(q, eps) * w[p + "q.norm"]
    q = rotate_halves(q, range(n), frequencies(m["rot"]))
    cap = m.get("softcap")
    o = grouped_attention(q, k, v, float(m["scale"]), window_mask(n, None), None if cap is None else float(cap), w[p + "sink"])
    o = o * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]      # one number per head
    return o.reshape(n, -1) @ w[p + "o"].T


# ---------------------------------------------------------------------------------------------- wkv
def token_shift(h: torch.Tensor, mu: torch.Tensor, before: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h + (h' - h) * mu`` with ``h'`` the row before (``before`` for the first, zeros if there is none)."""
    first = torch.zeros(1, h.shape[1], dtype=F64) if before is None else before.reshape(1, -1)
    prev = torch.cat([first, h[:-1]], dim=0)
    return h + (prev - h) * mu


def wkv_recurrence(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, u: torch.Tensor,
                   state: Optional[torch.Tensor] = None):
    """One head, token by token: ``o_t = (S + diag(u) k_t v_t^T)^T r_t``, then ``S <- diag(decay_t) S + k_t v_t^T``.
    ``r, k, decay`` ``[n, d]``, ``v`` ``[n, dv]``, ``u`` ``[d]``. Returns ``(o [n, dv], S [d, dv])``."""
    n, d = k.shape
    S = torch.zeros(d, v.shape[1], dtype=F64) if state is None else state.clone()
    out = torch.zeros(n, v.shape[1], dtype=F64)
    for t in range(n):
        kv = k[t][:, None] * v[t][None, :]
        out[t] = (S + u[:, None] * kv).T @ r[t]
        S = decay[t][:, None] * S + kv
    return out, S


def wkv(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Mixer ``wkv``: returns ``[n, width]``."""
    n = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    mixes = {s: token_shift(h, w[p + "mu." + s]) for s in "rkvgw"}
    r = (mixes["r"] @ w[p + "r"].T).reshape(n, H, d)
    k = (mixes["k"] @ w[p + "k"].T).reshape(n, H, d)
    v = (mixes["v"] @ w[p + "v"].T).reshape(n, H, d)
    gate = silu(mixes["g"] @ w[p + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mixes["w"] @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).reshape(n, H, d)
    heads = []
    for a in range(H):
        o, _ = wkv_recurrence(r[:, a], k[:, a], v[:, a], decay[:, a], w[p + "u"][a])
        heads.append(rms(o, eps))
    o = torch.cat(heads, dim=-1) * w[p + "norm"] * gate
    return o @ w[p + "o"].T


# ---------------------------------------------------------------------------------------------- experts
def route(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, r: dict):
    """Per token the chosen experts (identity experts count from ``experts`` on) and their weights:
    ``(chosen [n, top], weights [n, top])``."""
    n_all = router.shape[0]
    top, scale = int(r["top"]), float(r.get("scale", 1.0))
    groups = r.get("groups")
    s = torch.softmax(h @ router.T, dim=-1)
    choice = s + correction
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        per = n_all // count
        best = choice.reshape(-1, count, per).max(dim=-1).values
        kept = torch.topk(best, keep, dim=-1).indices
        allowed = torch.zeros(h.shape[0], count, dtype=torch.bool)
        allowed.scatter_(1, kept, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), -math.inf)
    chosen = torch.topk(choice, top, dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(dim=-1, keepdim=True) + 1e-20) * scale


def expert(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def routed_experts(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    n_experts = int(r["experts"])
    chosen, weights = route(h, w[p + "router"], w[p + "correction"], r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            # the router's last outputs are identity experts: the input itself
            out[t] += a * (expert(h[t:t + 1], w, f"{p}e{e}.")[0] if e < n_experts else h[t])
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ w[p + "shared.sg"].T) * expert(h, w, p + "shared.")
    return out


# ---------------------------------------------------------------------------------------------- the model
def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits ``[n, vocab]`` of a whole sequence; ``streams`` (a list) receives the stream after every layer."""
    w = {name: t.to(F64) for name, t in weights.items()}
    eps = float(config["norm"]["eps"])
    x = w["embed"][list(tokens)] * float(config.get("embedding", {}).get("scale", 1.0))
    kept = {}
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        if layer["type"] == "attention":
            y = attention_keys_as_values(x, w, p + "mix.", m, eps)
        elif layer["type"] == "attention_2":
            source = m.get("kv_from")
            if source is None:
                kept[i] = attention_2_keys_values(x, w, p + "mix.", m, eps)
            y = attention_2(x, w, p + "mix.", m, eps, *kept[i if source is None else int(source)])
        elif layer["type"] == "wkv":
            y = wkv(x, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_one_plus(y, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + norm_one_plus(routed_experts(x, w, p + "mlp.", layer["mlp"]), w[p + "norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    return (norm_one_plus(x, w["final.norm"], eps) @ w["head"].T) * float(config.get("logit_scale", 1.0))
