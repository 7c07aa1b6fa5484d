"""A plain, slow Sepedra in float64 on the CPU: one function per mechanism, written from the
equations, whole sequences at a time, with explicit loops over tokens where a mechanism is
recurrent.  It shares no code with the package; the tests compare the engine with it.

Notation: T tokens, h a sublayer's input [T, width]; weights are [out, in] and applied as x @ W.T.
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
    """To the nearest bfloat16 and back: the places where the engine's bfloat16 mode hands a value to a matrix
    product or to the cache."""
    return x.to(torch.float32).to(torch.bfloat16).to(F)


def to64(tensors: Mapping[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(F) if v.is_floating_point() else v) for k, v in tensors.items()}


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms_unit(x, eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(u: torch.Tensor, taps_w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y_t = sum_j w[:, j] * u_(t - taps + 1 + j) per channel, zeros before the first token.  u [T, C], taps_w [C, taps]."""
    T, C = u.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + T] * taps_w[:, j]
    return y if bias is None else y + bias


def rotary_frequencies(rot: Mapping) -> torch.Tensor:
    """f_i = base^(-2i/dims), then stretched band by band: wavelengths under original/high stay, those over
    original/low are divided by factor, those between are blended linearly in original/wavelength."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    sc = rot.get("scaling")
    if not sc:
        return f
    factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = f.clone()
    for i in range(f.numel()):
        wl = 2.0 * math.pi / float(f[i])
        if wl < orig / high:
            continue
        if wl > orig / low:
            out[i] = f[i] / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[i] = (1.0 - s) * f[i] / factor + s * f[i]
    return out


def rotate_pairs(x: torch.Tensor, pos0: int, rot: Mapping) -> torch.Tensor:
    """x [T, heads, dim]: elements (2i, 2i+1), i < dims/2, of every head turned by the angle position * f_i."""
    T = x.shape[0]
    dims = int(rot["dims"])
    f = rotary_frequencies(rot)
    ang = torch.arange(pos0, pos0 + T, dtype=F)[:, None] * f[None, :]            # [T, dims/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def attention_keys_values(h, w, pre, m, eps, rnd=identity):
    """A layer's keys (convolved, rotated, unit-normed) [T, G, dim] and values (convolved) [T, G, vdim]."""
    T = h.shape[0]
    G, D, V = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    k = causal_conv(h @ w[pre + "mix.k"].T, w[pre + "mix.k.conv"]).view(T, G, D)
    v = causal_conv(h @ w[pre + "mix.v"].T, w[pre + "mix.v.conv"]).view(T, G, V)
    k = rms_unit(rotate_pairs(k, 0, m["rot"]), eps)
    return rnd(k), rnd(v)


def attention_mixer(h, w, pre, m, eps, keys, values, rnd=identity):
    """Queries of this layer against ``keys`` / ``values`` (its own or another layer's); softmax with a sink of score 0
    in the denominator; sigmoid output gate; output projection."""
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = causal_conv(h @ w[pre + "mix.q"].T, w[pre + "mix.q.conv"]).view(T, H, D)
    q = rnd(rms_unit(rotate_pairs(q, 0, m["rot"]), eps))
    scale = float(m["scale"])
    out = torch.zeros(T, H, V, dtype=F)
    per = H // G
    for hd in range(H):
        g = hd // per
        s = (q[:, hd] @ keys[:, g].T) * scale                       # [T, T]
        mask = torch.ones(T, T, dtype=torch.bool).tril()
        s = s.masked_fill(~mask, -math.inf)
        mx = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
        e = torch.exp(s - mx)
        p = e / (torch.exp(-mx) + e.sum(-1, keepdim=True))
        out[:, hd] = p @ values[:, g]
    gate = torch.sigmoid(h @ w[pre + "mix.g"].T)
    return rnd(out.reshape(T, H * V) * gate) @ w[pre + "mix.o"].T


def rglru_mixer(h, w, pre, m, rnd=identity):
    T = h.shape[0]
    R, B = int(m["width"]), int(m["blocks"])
    y = gelu_tanh(h @ w[pre + "mix.y"].T + w[pre + "mix.y.b"])
    u = causal_conv(h @ w[pre + "mix.x"].T + w[pre + "mix.x.b"], w[pre + "mix.conv"], w[pre + "mix.conv.b"])
    bs = R // B
    ub = u.view(T, B, bs)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[pre + "mix.ra"]) + w[pre + "mix.ra.b"]).reshape(T, R)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[pre + "mix.ri"]) + w[pre + "mix.ri.b"]).reshape(T, R)
    log_a = -8.0 * r * torch.nn.functional.softplus(w[pre + "mix.lam"])
    a = torch.exp(log_a)
    S = torch.zeros(R, dtype=F)
    out = torch.zeros(T, R, dtype=F)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return rnd(out * y) @ w[pre + "mix.o"].T


def route(h, w, pre, mlp):
    """Chosen experts [T, top] and their weights: softmax over all experts; a group's score is its best expert's; only
    experts of the ``keep`` best groups can be chosen; the weights are the scores as they are."""
    r = mlp["router"]
    E, top = int(r["experts"]), int(r["top"])
    groups = r.get("groups") or {"count": 1, "keep": 1}
    count, keep = int(groups["count"]), int(groups["keep"])
    s = torch.softmax(h @ w[pre + "mlp.router"].T, -1)
    T = h.shape[0]
    gs = s.view(T, count, E // count).max(-1).values
    best = torch.topk(gs, keep, dim=-1).indices
    allowed = torch.zeros(T, count, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    allowed = allowed[:, :, None].expand(T, count, E // count).reshape(T, E)
    masked = torch.where(allowed, s, torch.full_like(s, -1.0))
    idx = torch.topk(masked, top, dim=-1).indices
    return idx, torch.gather(s, 1, idx)


def expert(h, w, name, limit, rnd=identity):
    g = torch.clamp(h @ w[name + ".gate"].T, max=limit)
    u = torch.clamp(h @ w[name + ".up"].T, min=-limit, max=limit)
    return rnd(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[name + ".down"].T


def moe_ff(h, w, pre, mlp, rnd=identity):
    idx, wt = route(h, w, pre, mlp)
    limit = float(mlp["expert"]["limit"])
    out = torch.zeros(h.shape[0], w[pre + "mlp.e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            out[t] += wt[t, j] * expert(h[t:t + 1], w, f"{pre}mlp.e{e}", limit, rnd)[0]
    return out


def forward(cfg: Mapping, w: Mapping[str, torch.Tensor], tokens, rnd=identity, layers_out: Optional[List] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  ``layers_out``: receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    kv: Dict[int, tuple] = {}
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        m = layer["mixer"]
        h = rnd(x)
        if layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = attention_keys_values(h, w, pre, m, eps, rnd)
                src = i
            y = attention_mixer(h, w, pre, m, eps, kv[src][0], kv[src][1], rnd)
        elif layer["type"] == "rglru":
            y = rglru_mixer(h, w, pre, m, rnd)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, w[pre + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + rms_norm(moe_ff(rnd(x), w, pre, layer["mlp"], rnd), w[pre + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    cap = float(cfg["logit_softcap"])
    logits = rnd(rms_norm(x, w["final.norm"], eps)) @ w["head"].T
    return cap * torch.tanh(logits / cap)


def generate_greedy(cfg: Mapping, w: Mapping[str, torch.Tensor], prompt, n: int) -> List[int]:
    """n tokens by the first maximum of the last position's logits, the whole sequence recomputed for every token."""
    toks = list(prompt)
    out: List[int] = []
    for _ in range(n):
        nxt = int(torch.argmax(forward(cfg, w, toks)[-1]))
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
