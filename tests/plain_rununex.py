"""The Rununex decoder in plain, slow PyTorch on the CPU: one function per mechanism, written from the
design's equations, sharing no code with the engine.  Everything is computed in the dtype of the tensors
it is given (the tests hand it float64 or float32 copies of the weights); a whole sequence at a time,
token by token where a recurrence asks for it.

Notation: h [T, width] is a mixer's or feed-forward's input for the T tokens of one sequence, positions
0 .. T - 1; ``w`` maps tensor names to tensors; ``p`` is the prefix of the part's tensors.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch
import torch.nn.functional as F


def layer_norm(x, weight, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal_conv(u, taps, bias=None):
    """u [T, C], taps [C, K]: y_t = sum_j taps[:, j] u_(t - K + 1 + j), zeros before the start."""
    T, C = u.shape
    K = taps.shape[1]
    padded = torch.cat([u.new_zeros((K - 1, C)), u], dim=0)
    y = u.new_zeros((T, C))
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j]
    return y if bias is None else y + bias


def chunk_mask(T, size):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def scaled_frequencies(dims, base, scaling, dtype=torch.float64):
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    if scaling:
        factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
        original = float(scaling["original"])
        out = []
        for fi in f.tolist():
            wavelength = 2.0 * math.pi / fi
            if wavelength < original / high:
                out.append(fi)
            elif wavelength > original / low:
                out.append(fi / factor)
            else:
                s = (original / wavelength - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=torch.float64)
    return f.to(dtype)


def rotate_interleaved(x, positions, freqs):
    """x [T, n, d]: entry 2i is paired with entry 2i + 1 over the first 2 len(freqs) entries."""
    rot = 2 * freqs.shape[0]
    angle = positions.to(freqs.dtype)[:, None] * freqs[None, :]
    cos, sin = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    a, b = x[..., 0:rot:2], x[..., 1:rot:2]
    out = x.clone()
    out[..., 0:rot:2] = a * cos - b * sin
    out[..., 1:rot:2] = b * cos + a * sin
    return out


def differential_attention(h, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    if m.get("conv"):
        q, k, v = (causal_conv(u, w[p + name + ".conv"]) for u, name in ((q, "q"), (k, "k"), (v, "v")))
    q = q.view(T, H * 2, d)
    k = k.view(T, G * 2, d)
    v = v.view(T, G, dv)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        freqs = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"), torch.float64)
        positions = torch.arange(T)
        q = rotate_interleaved(q, positions, freqs)
        k = rotate_interleaved(k, positions, freqs)
    mask = chunk_mask(T, m["mask"]["size"]) if m.get("mask") else chunk_mask(T, T)
    lam = (torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum())
           + m["diff"])
    heads = []
    for head in range(H):
        g = head // (H // G)
        maps = []
        for which in range(2):
            s = (q[:, 2 * head + which] @ k[:, 2 * g + which].T) * m["scale"]
            s = s.masked_fill(~mask, float("-inf"))
            maps.append(torch.softmax(s, dim=-1) @ v[:, g])
        o = maps[0] - lam * maps[1]
        heads.append(unit_rms(o, eps) * (1.0 - m["diff"]))
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


def biased_sink_attention(h, w, p: str, m: dict, eps: float):
    """The parallel mixer's left half."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ w[p + "q"].T).view(T, H, d), eps)
    k = unit_rms((h @ w[p + "k"].T).view(T, G, d), eps)
    v = (h @ w[p + "v"].T).view(T, G, dv)
    mask = chunk_mask(T, m["mask"]["size"]) if m.get("mask") else chunk_mask(T, T)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    distance = (i - j).clamp(min=0).to(h.dtype)
    heads = []
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        s = s - w[p + "r1"][head] * torch.log1p(w[p + "r2"][head] * distance)
        s = s.masked_fill(~mask, float("-inf"))
        # the sink: one more term in the denominator, without a value
        top = torch.maximum(s.max(dim=-1, keepdim=True).values, w[p + "sink"][head])
        e = torch.exp(s - top)
        weights = e / (e.sum(-1, keepdim=True) + torch.exp(w[p + "sink"][head] - top))
        heads.append(weights @ v[:, g])
    y = torch.cat(heads, dim=-1) * torch.sigmoid(h @ w[p + "g"].T)
    return y @ w[p + "o"].T


def mamba2(h, w, p: str, m: dict, eps: float):
    """The parallel mixer's right half."""
    T = h.shape[0]
    nh, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = nh * dv
    zxbcdt = h @ w[p + "in"].T
    z = zxbcdt[:, :inner]
    xbc = zxbcdt[:, inner:2 * inner + 2 * G * N]
    dt = zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc = F.silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(T, nh, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = F.softplus(dt + w[p + "dt_bias"])
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * dt)        # [T, nh]
    S = h.new_zeros((nh, N, dv))
    y = h.new_zeros((T, nh, dv))
    for t in range(T):
        for head in range(nh):
            g = head // (nh // G)
            S[head] = decay[t, head] * S[head] + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S[head].T @ C[t, g] + w[p + "D"][head] * x[t, head]
    y = y.reshape(T, inner) * F.silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


def parallel_mixer(h, w, p: str, m: dict, eps: float):
    left = biased_sink_attention(h, w, p + "left.", m["left"], eps)
    right = mamba2(h, w, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def gated_expert(h, w, p: str):
    return (F.silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def routed_experts(h, w, p: str, mlp: dict):
    """Sigmoid scores, the ``top`` largest chosen, each chosen expert fed its score times h."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    scores = torch.sigmoid(h.to(torch.float32) @ w[p + "router"].to(torch.float32).T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = torch.topk(scores[t], top).indices.tolist()
        for e in chosen:
            out[t] = out[t] + gated_expert((scores[t, e].to(h.dtype) * h[t])[None], w, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_expert(h, w, p + "shared.")
    return out


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], keep_layers: bool = False):
    """Logits [T, vocab] of one sequence; with ``keep_layers`` also the stream after every layer."""
    eps = cfg["norm"]["eps"]
    mult = cfg.get("residual_mult", 1.0)
    x = w["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = layer_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            x = x + mult * differential_attention(h, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            x = x + mult * parallel_mixer(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp"):
            h = layer_norm(x, w[p + "norm2"], eps)
            x = x + mult * routed_experts(h, w, p + "mlp.", layer["mlp"])
        after.append(x)
    logits = layer_norm(x, w["final.norm"], eps) @ w["head"].T * cfg.get("logit_scale", 1.0)
    return (logits, after) if keep_layers else logits
