"""A plain, slow implementation of the Povatar decoder on the CPU, one function per mechanism.

It shares no code with the engine: torch on the CPU in float64 (or any type that is asked for), token by token
where the design is recurrent, every key of a sequence where it attends.  The tests hold the engine's logits
against it.  ``config`` is the dictionary of config.json, ``w`` maps tensor names to torch tensors.

The design: x = embed[token] * embedding.scale; every layer is x <- x + mixer(norm1(x)) + moe(norm2(x)) with both
branches reading the same x; the mixer is the mean of two mixers' outputs, each RMS-normed over the width with a
weight of its own: softmax attention (grouped heads, partly rotated with stretched frequencies, visible keys limited
to the query's own block of positions, one more term of 1 in the softmax's denominator) and a selective state-space
recurrence with a scalar decay per head; then the model's norm and the vocabulary projection.
"""
from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def weighted_norm(x, weight, eps):
    return rms(x, eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def embed(tokens, table, scale, dtype):
    return table[torch.as_tensor(tokens, dtype=torch.long)].to(dtype) * scale


# ------------------------------------------------------------------------------------------- rotation
def rotation_frequencies(rot, dtype=torch.float64):
    """Frequencies of the dims/2 pairs and the factor on cosine and sine.  Without 'scaling': base^(-2i/dims) and 1.
    With it, slow pairs (long wavelengths) are divided by 'factor', fast ones stay, a linear ramp between them."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    s = rot.get("scaling")
    if not s:
        return f.to(dtype), 1.0

    def turn_dim(turns):          # the pair whose wavelength makes `turns` turns over the original length
        return dims * math.log(s["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(turn_dim(s["fast"])), 0)
    hi = min(math.ceil(turn_dim(s["slow"])), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    f = f / s["factor"] * ramp + f * (1 - ramp)
    return f.to(dtype), 0.1 * math.log(s["factor"]) + 1.0


def rotate(x, positions, rot):
    """x [T, heads, d]: the first dims entries of every head in pairs (i, i + dims/2), the rest unchanged."""
    dims = rot["dims"]
    half = dims // 2
    f, mag = rotation_frequencies(rot, x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]
    cos, sin = (torch.cos(a) * mag)[:, None, :], (torch.sin(a) * mag)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], -1)


# ------------------------------------------------------------------------------------------ attention
def block_visible(i, j, size):
    """Whether the query at position i sees the key at position j: not later, and in the same block of `size`."""
    return j <= i and (size <= 0 or i // size == j // size)


def block_attention(h, w, pre, m):
    """h [T, width] (positions 0..T-1) -> [T, width].  p_j = exp(s_j) / (1 + sum over visible keys of exp(s))."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ w[pre + "q"].to(h.dtype).T).view(T, H, d)
    k = (h @ w[pre + "k"].to(h.dtype).T).view(T, G, d)
    v = (h @ w[pre + "v"].to(h.dtype).T).view(T, G, dv)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    size = (m.get("mask") or {}).get("size", 0)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        see = torch.tensor([[block_visible(i, j, size) for j in range(T)] for i in range(T)])
        # exp(s) / (1 + sum exp(s)), with everything divided by exp(top), top the row's largest visible score or 0
        top = torch.where(see, s, torch.zeros_like(s)).amax(-1, keepdim=True).clamp(min=0.0)
        e = torch.where(see, torch.exp(s - top), torch.zeros_like(s))
        out[:, head] = (e / (torch.exp(-top) + e.sum(-1, keepdim=True))) @ v[:, g]
    return out.reshape(T, H * dv) @ w[pre + "o"].to(h.dtype).T


# ---------------------------------------------------------------------------------------- state space
def causal_conv(x, taps, bias):
    """x [T, C], taps [C, K] with the last column for the current token; zeros before the sequence starts."""
    T, _ = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, x.shape[1], dtype=x.dtype), x], 0)
    out = bias[None, :].expand(T, -1).clone()
    for j in range(K):
        out = out + padded[j:j + T] * taps[:, j][None, :]
    return out


def group_norm_gate(y, z, weight, parts, eps):
    """(y * silu(z)), each of `parts` equal parts of a row divided by its own root mean square, times weight."""
    T, n = y.shape
    g = (y * silu(z)).view(T, parts, n // parts)
    return rms(g, eps).reshape(T, n) * weight


def state_space(h, w, pre, m, eps):
    """h [T, width] -> [T, width].  Per head, S (N x P) <- exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x."""
    T = h.shape[0]
    Hn, P, N, G, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = Hn * P
    proj = h @ w[pre + "in"].to(h.dtype).T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[pre + "conv"].to(h.dtype), w[pre + "conv.b"].to(h.dtype)))
    x = xbc[:, :inner].view(T, Hn, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[pre + "dt_bias"].to(h.dtype))
    A = -torch.exp(w[pre + "A_log"].to(h.dtype))
    D = w[pre + "D"].to(h.dtype)
    y = torch.zeros(T, Hn, P, dtype=h.dtype)
    S = torch.zeros(Hn, N, P, dtype=h.dtype)
    for t in range(T):
        for head in range(Hn):
            g = head // (Hn // G)
            S[head] = torch.exp(A[head] * dt[t, head]) * S[head] + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S[head].T @ C[t, g] + D[head] * x[t, head]
    y = group_norm_gate(y.reshape(T, inner), z, w[pre + "norm"].to(h.dtype), parts, eps)
    return y @ w[pre + "o"].to(h.dtype).T


def pair_mixer(h, w, pre, m, eps):
    left = weighted_norm(block_attention(h, w, pre + "left.", m["left"]), w[pre + "left.out"].to(h.dtype), eps)
    right = weighted_norm(state_space(h, w, pre + "right.", m["right"], eps), w[pre + "right.out"].to(h.dtype), eps)
    return 0.5 * (left + right)


# -------------------------------------------------------------------------------------- feed-forward
def route(h, router, top):
    """Softmax over all experts, the `top` largest, their scores divided by their sum.  -> (indices, weights) [T, top]."""
    s = torch.softmax(h @ router.to(h.dtype).T, -1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val / (val.sum(-1, keepdim=True) + 1e-20)


def experts(h, w, pre, mlp):
    T = h.shape[0]
    idx, wt = route(h, w[pre + "router"], mlp["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(T):
        for e, c in zip(idx[t].tolist(), wt[t]):
            up = torch.relu(w[f"{pre}e{e}.up"].to(h.dtype) @ h[t]) ** 2
            out[t] += c * (w[f"{pre}e{e}.down"].to(h.dtype) @ up)
    return out


# --------------------------------------------------------------------------------------------- model
def layer(x, w, i, spec, eps):
    p = f"l{i}."
    if spec["type"] != "parallel":
        raise ValueError(spec["type"])
    add = pair_mixer(weighted_norm(x, w[p + "norm1"].to(x.dtype), eps), w, p + "mix.", spec["mixer"], eps)
    if spec.get("mlp"):
        add = add + experts(weighted_norm(x, w[p + "norm2"].to(x.dtype), eps), w, p + "mlp.", spec["mlp"])
    return x + add


def forward(config, w, tokens, dtype=torch.float64, states=None):
    """Logits [T, vocab] of one sequence from its first token.  states: a list that gets the stream after every layer."""
    eps = config["norm"]["eps"]
    x = embed(tokens, w["embed"], config["embedding"]["scale"], dtype)
    for i, spec in enumerate(config["layers"]):
        x = layer(x, w, i, spec, eps)
        if states is not None:
            states.append(x.clone())
    return weighted_norm(x, w["final.norm"].to(dtype), eps) @ w["head"].to(dtype).T
