"""A plain, slow Kuponex in float64 on the CPU: one function per mechanism, written from the
equations, whole sequences at a time with explicit loops over tokens where a mechanism is
recurrent.  It shares no code with the package; the tests compare the engine with it.

Notation: T tokens, h the mixer's input [T, width]; weights are [out, in] and applied as x @ W.T.
``w`` maps tensor names to float64 tensors, ``pre`` is a layer's prefix ("l3.").
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch

F = torch.float64


def identity(x):
    return x


def round_bf16(x: torch.Tensor) -> torch.Tensor:
    """Round to the nearest bfloat16 (ties to even) and come back: the places where the engine's bfloat16 mode hands a
    value to a matrix product or to the cache."""
    return x.to(torch.float32).to(torch.bfloat16).to(F)


def to64(tensors: Mapping[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: v.to(F) for k, v in tensors.items()}


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over the root of (its mean square + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, weight, eps):
    return rms_unit(x, eps) * (1.0 + weight)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def token_shift(h: torch.Tensor, mix: torch.Tensor) -> torch.Tensor:
    """h_t + (h_{t-1} - h_t) * mix, with zeros before the first token."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mix


def dense_ff(h, w, pre, rnd=identity):
    return rnd(gelu_tanh(h @ w[pre + "mlp.gate"].T) * (h @ w[pre + "mlp.up"].T)) @ w[pre + "mlp.down"].T


def mlstm_mixer(h, w, pre, m, eps, rnd=identity):
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    T = h.shape[0]
    q = (h @ w[pre + "mix.q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[pre + "mix.k"].T).view(T, H, D)
    v = (h @ w[pre + "mix.v"].T).view(T, H, V)
    gi = cap * torch.tanh((h @ w[pre + "mix.i"].T + w[pre + "mix.i.b"]) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w[pre + "mix.f"].T + w[pre + "mix.f.b"]) / cap))
    S = torch.zeros(H, D, V, dtype=F)
    n = torch.zeros(H, D, dtype=F)
    mx = torch.zeros(H, dtype=F)
    out = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        m_new = torch.maximum(gf[t] + mx, gi[t])
        a = torch.exp(gf[t] + mx - m_new)
        b = torch.exp(gi[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    o = rms_unit(out, eps).reshape(T, H * V) * w[pre + "mix.norm"]
    o = o * torch.sigmoid(h @ w[pre + "mix.g"].T)
    return rnd(o) @ w[pre + "mix.o"].T


def gla_mixer(h, w, pre, m, eps, rnd=identity):
    H, D, V, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    T = h.shape[0]
    q = (h @ w[pre + "mix.q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[pre + "mix.k"].T).view(T, H, D)
    v = (h @ w[pre + "mix.v"].T).view(T, H, V)
    z = (h @ w[pre + "mix.a1"].T) @ w[pre + "mix.a2"].T + w[pre + "mix.a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / tau).view(T, H, D)
    S = torch.zeros(H, D, V, dtype=F)
    out = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = (rms_unit(out, eps) * w[pre + "mix.norm"]).reshape(T, H * V)
    o = o * torch.nn.functional.silu(h @ w[pre + "mix.g"].T)
    return rnd(o) @ w[pre + "mix.o"].T


def rotate_half(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, ..., n]: the first ``dims`` elements of the last axis are rotated, pairs (i, i + dims/2)."""
    half = dims // 2
    f = base ** (-2.0 * torch.arange(half, dtype=F) / dims)
    a = positions.to(F)[:, None] * f[None, :]
    while a.dim() < x.dim():
        a = a.unsqueeze(1)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a), x[..., dims:]], -1)


def latent_attention_mixer(h, w, pre, m, eps, rnd=identity):
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims, scale = float(m["rot"]["base"]), int(m["rot"]["dims"]), float(m["scale"])
    T = h.shape[0]
    pos = torch.arange(T)
    q = (h @ w[pre + "mix.q"].T).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_half(q[..., D:], pos, base, dims)
    dkv = h @ w[pre + "mix.dkv"].T
    c = rnd(rms_unit(dkv[:, :C], eps) * w[pre + "mix.dkv.norm"])          # what the cache holds
    k_rot = rnd(rotate_half(dkv[:, C:], pos, base, dims))                  # one for all heads
    k_plain = (c @ w[pre + "mix.uk"].T).view(T, H, D)
    val = (c @ w[pre + "mix.uv"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=F)
    sink = w[pre + "mix.sink"]
    for t in range(T):
        s = (torch.einsum("hd,jhd->hj", q_plain[t], k_plain[:t + 1]) + q_rot[t] @ k_rot[:t + 1].T) * scale
        top = torch.maximum(s.max(-1).values, sink)
        e = torch.exp(s - top[:, None])
        den = e.sum(-1) + torch.exp(sink - top)
        out[t] = torch.einsum("hj,jhv->hv", e / den[:, None], val[:t + 1])
    return rnd(out.reshape(T, H * V)) @ w[pre + "mix.o"].T


MIXERS = {"mlstm": mlstm_mixer, "gla": gla_mixer, "latent_attention": latent_attention_mixer}


def layer(x, w, i, spec, eps, rnd=identity):
    pre = f"l{i}."
    h = rnd(token_shift(norm_around_zero(x, w[pre + "norm1"], eps), w[pre + "shift"]))
    y = MIXERS[spec["type"]](h, w, pre, spec["mixer"], eps, rnd)
    if spec.get("mlp") is not None:
        y = y + dense_ff(rnd(norm_around_zero(x, w[pre + "norm2"], eps)), w, pre, rnd)
    return x + y


def forward(config: Mapping, w: Mapping[str, torch.Tensor], tokens: List[int], keep_layers: Optional[list] = None,
            rnd=identity) -> torch.Tensor:
    """Logits [T, vocab] of one sequence (float64).  ``rnd`` = round_bf16 rounds where the engine's bfloat16 mode does:
    the inputs of the projections, the feed-forward's gated unit, what the mixers hand to their output projection,
    what the cache holds; every sum, state, gate, score and norm stays exact."""
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, spec in enumerate(config["layers"]):
        x = layer(x, w, i, spec, eps, rnd)
        if keep_layers is not None:
            keep_layers.append(x.clone())
    return rnd(norm_around_zero(x, w["final.norm"], eps)) @ w["head"].T


def generate_greedy(config: Mapping, w: Mapping[str, torch.Tensor], prompt: List[int], new_tokens: int) -> List[int]:
    """Greedy continuation, the whole sequence recomputed for every token (the first maximum wins)."""
    toks, out = list(prompt), []
    for _ in range(new_tokens):
        nxt = int(torch.argmax(forward(config, w, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out


def logits_error(got, want, quantile: float = 1.0) -> float:
    """A row's error: the root mean square of the difference (its mean taken off) over that of the wanted row; the
    largest over the rows, or the given quantile of them."""
    import numpy as np
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    ref = want - want.mean(-1, keepdims=True)
    return float(np.quantile(np.sqrt((d * d).mean(-1)) / np.sqrt((ref * ref).mean(-1)), quantile))
