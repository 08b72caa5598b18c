"""Plain implementation of the Letevik decoder: float64, whole sequences, no cache, one function per mechanism.

It shares no code with the package: it reads the ``config.json`` dictionary and the stored tensors by their names.
For tokens ``t_0 .. t_{n-1}`` at places ``0 .. n-1`` (``rms(x) = x / sqrt(mean(x^2) + eps)``):

* ``x_p = embed[t_p] + bigram[r_p]`` with ``r_0 = buckets`` and ``r_p = (t_{p-1} mul_prev + t_p mul_cur) mod buckets``
* the layers ``loop.start .. loop.stop - 1`` run ``loop.times`` times in a row; each pass begins with ``x <- x + loop.step[pass]``
* a layer: ``x <- x + mixer(rms(x) norm1)``, then ``x <- x + ff(rms(x) norm2)`` where the layer has a feed-forward
* mixer ``attention``: two softmax maps per head over the same values, combined as ``a1 - lambda a2``; short causal
  convolutions on q, k, v; interleaved rotation; a window that also keeps the first keys
* mixer ``latent_attention``: queries, keys and values through low-rank latents, one rotated key part shared by the heads,
  a per-head term without a value in the softmax's denominator, an output gate
* ``ff``: ``down(g sigmoid(1.702 g) (u + 1))`` with ``g = min(gate h, limit)``, ``u = clamp(up h, -limit, limit)``
* logits ``embed @ (rms(x) final.norm)``.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64
SIGMOID_SLOPE = 1.702


def rms_norm(x: torch.Tensor, gain: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if gain is None else y * gain


# ---------------------------------------------------------------------------------------------- embedding
def bigram_rows(tokens: Sequence[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the bigram table per place: the last row for the first token, else a hash of the pair."""
    rows = []
    for p, t in enumerate(tokens):
        rows.append(buckets if p == 0 else (int(tokens[p - 1]) * mul_prev + int(t) * mul_cur) % buckets)
    return rows


def embed(tokens: Sequence[int], w: Dict[str, torch.Tensor], config: dict) -> torch.Tensor:
    x = w["embed"][list(tokens)]
    bigram = (config.get("embedding") or {}).get("bigram")
    if bigram:
        x = x + w["bigram"][bigram_rows(tokens, bigram["buckets"], bigram["mul_prev"], bigram["mul_cur"])]
    return x


# ---------------------------------------------------------------------------------------------- pieces of the mixers
def short_convolution(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """``u`` ``[n, channels]``, ``taps`` ``[channels, K]``: ``y_t = sum_j taps[:, j] u_(t - K + 1 + j)``, zeros before place 0."""
    n, K = u.shape[0], taps.shape[1]
    y = torch.zeros_like(u)
    for j in range(K):
        shift = K - 1 - j
        if shift < n:
            y[shift:] += taps[:, j] * u[:n - shift]
    return y


def rotate_interleaved(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """``x`` ``[n, ..., d]``, place = index along axis 0: channels ``2 i`` and ``2 i + 1`` turn by ``place * base^(-2 i / dims)``."""
    out = x.clone()
    place = torch.arange(x.shape[0], dtype=F64).reshape([-1] + [1] * (x.dim() - 2))
    for i in range(dims // 2):
        a = place * float(base) ** (-2.0 * i / dims)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * torch.cos(a) - v * torch.sin(a)
        out[..., 2 * i + 1] = v * torch.cos(a) + u * torch.sin(a)
    return out


def rotate_halves(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """As above with channel ``i`` paired with channel ``i + dims / 2``."""
    out = x.clone()
    half = dims // 2
    place = torch.arange(x.shape[0], dtype=F64).reshape([-1] + [1] * (x.dim() - 2))
    for i in range(half):
        a = place * float(base) ** (-2.0 * i / dims)
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * torch.cos(a) - v * torch.sin(a)
        out[..., i + half] = v * torch.cos(a) + u * torch.sin(a)
    return out


def visible(n: int, window: Optional[int] = None, keep_first: int = 0) -> torch.Tensor:
    """bool ``[n, n]``: query ``i`` sees key ``j <= i`` that is either within the last ``window`` places or among the first
    ``keep_first``."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if window is not None:
        seen &= (i - j < window) | (j < keep_first)
    return seen


def softmax_weights(scores: torch.Tensor, seen: torch.Tensor, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``scores`` ``[H, n, n]``; ``sink`` ``[H]``: one more term ``exp(sink_h)`` in every denominator of head ``h``."""
    scores = scores.masked_fill(~seen, float("-inf"))
    top = scores.max(dim=-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink[:, None, None])
    e = torch.exp(scores - top)
    total = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink[:, None, None] - top)
    return e / total


# ---------------------------------------------------------------------------------------------- mixers
def differential_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    if m.get("conv"):
        q, k, v = (short_convolution(t, w[p + name + ".conv"]) for t, name in ((q, "q"), (k, "k"), (v, "v")))
    q = q.reshape(n, H, 2, d)
    k = k.reshape(n, G, 2, d)
    v = v.reshape(n, G, dv)
    rot = m.get("rot")
    if rot:
        q, k = rotate_interleaved(q, rot["dims"], rot["base"]), rotate_interleaved(k, rot["dims"], rot["base"])
    mask = m.get("mask") or {}
    seen = visible(n, mask.get("size"), mask.get("keep_first", 0))
    group = H // G
    diff = float(m["diff"])
    lam = torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + diff
    out = torch.zeros(n, H, dv, dtype=F64)
    for head in range(H):
        g = head // group
        maps = []
        for which in range(2):
            scores = (q[:, head, which] @ k[:, g, which].T) * float(m["scale"])
            maps.append(softmax_weights(scores[None], seen)[0] @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, head] = rms_norm(o, None, eps) * (1.0 - diff)
    return out.reshape(n, H * dv) @ w[p + "o"].T


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, d, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(n, H, d + dr)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    k_rot = down[:, rank:]
    k_plain = (c @ w[p + "uk"].T).reshape(n, H, d)
    v = (c @ w[p + "uv"].T).reshape(n, H, dv)
    rot = m["rot"]
    q_rot = rotate_halves(q[:, :, d:], rot["dims"], rot["base"])
    k_rot = rotate_halves(k_rot, rot["dims"], rot["base"])
    scores = (torch.einsum("ihd,jhd->hij", q[:, :, :d], k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * float(m["scale"])
    weights = softmax_weights(scores, visible(n), w[p + "sink"])
    heads = torch.einsum("hij,jhd->ihd", weights, v).reshape(n, H * dv)
    heads = heads * torch.sigmoid(h @ w[p + "g"].T)
    return heads @ w[p + "o"].T


def feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    limit = float(mlp["limit"])
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(SIGMOID_SLOPE * g) * (u + 1.0)) @ w[p + "down"].T


# ---------------------------------------------------------------------------------------------- the model
def layer_order(config: dict) -> List[tuple]:
    """``(layer, pass or None)`` per run of a layer; ``pass`` is given at the first layer of a pass of the loop."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(start)]
    for t in range(times):
        order += [(i, t if i == start else None) for i in range(start, stop)]
    return order + [(i, None) for i in range(stop, n)]


def forward(tokens: Sequence[int], w: Dict[str, torch.Tensor], config: dict, streams: Optional[list] = None) -> torch.Tensor:
    """Logits ``[n, vocab]`` of the whole sequence; ``streams`` (a list) gets the residual stream after every run of a layer."""
    w = {name: t.to(F64) for name, t in w.items()}
    eps = float(config["norm"]["eps"])
    x = embed(tokens, w, config)
    for index, begins_pass in layer_order(config):
        layer = config["layers"][index]
        p = f"l{index}."
        if begins_pass is not None:
            x = x + w["loop.step"][begins_pass]
        h = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            x = x + differential_attention(h, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "latent_attention":
            x = x + latent_attention(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            x = x + feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"])
        if streams is not None:
            streams.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T
