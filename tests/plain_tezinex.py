"""A plain, slow implementation of the Tezinex decoder on the CPU, one function per mechanism.

It shares no code with the engine: torch on the CPU in float64 (or any type that is asked for), token by token
where the design is recurrent, every key of a sequence where it attends.  The tests hold the engine's logits
against it.  ``config`` is the dictionary of config.json, ``w`` maps tensor names to torch tensors.

Notation: x[t] is the residual stream at token t of one sequence, p its position from 0.
"""
from __future__ import annotations

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def unit_offset_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * (1 + weight): the weight is stored around zero."""
    return rms(x, eps) * (1.0 + weight)


def sinusoid(positions, width, dtype):
    """Entry 2i is sin(p * 10000^(-2i / width)), entry 2i + 1 the cosine of the same angle."""
    i = torch.arange(width // 2, dtype=dtype)
    angle = positions.to(dtype)[:, None] * torch.pow(torch.tensor(10000.0, dtype=dtype), -2.0 * i / width)[None, :]
    out = torch.zeros(len(positions), width, dtype=dtype)
    out[:, 0::2] = torch.sin(angle)
    out[:, 1::2] = torch.cos(angle)
    return out


def embed(tokens, table, dtype):
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    return table[tokens].to(dtype) + sinusoid(torch.arange(len(tokens)), table.shape[1], dtype)


def silu(z):
    return z * torch.sigmoid(z)


def causal_conv(x, taps):
    """x [T, C], taps [C, K] with the last column for the current token; zeros before the sequence starts."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], 0)
    out = torch.zeros_like(x)
    for j in range(K):
        out += padded[j:j + T] * taps[:, j][None, :]
    return out


def visible(i, j, size, keep_first):
    """Whether the query at position i sees the key at position j."""
    return j <= i and (i - j < size or j < keep_first)


def attention(h, w, pre, m, keys_values=None):
    """Softmax attention with biases, capped scores, a window that keeps the first tokens, and a sink per head.
    h [T, width]; returns (output [T, width], (k, v)).  With ``keys_values`` the layer uses those and projects none."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).view(T, H, d)
    if keys_values is None:
        k = (h @ w[pre + "k"].T + w[pre + "k.b"]).view(T, G, d)
        v = (h @ w[pre + "v"].T + w[pre + "v.b"]).view(T, G, dv)
    else:
        k, v = keys_values
    cap, size, keep = m["softcap"], m["mask"]["size"], m["mask"]["keep_first"]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        s = cap * torch.tanh(s / cap)
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j, size, keep)]
            e = torch.exp(s[i, js] - s[i, js].max())
            sink = torch.exp(w[pre + "sink"][head] - s[i, js].max())
            out[i, head] = (e[:, None] * v[js, g]).sum(0) / (e.sum() + sink)
    return out.reshape(T, H * dv) @ w[pre + "o"].T, (k, v)


def channel_delta(h, w, pre, m, eps):
    """The gated delta rule with one decay per head and key channel, token by token from a zero state."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(causal_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[pre + "b"].T)                                        # [T, H]
    a = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]
    decay = torch.exp(-torch.exp(w[pre + "A_log"])[None, :, None] * torch.nn.functional.softplus(a).view(T, H, d))
    gate = torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(T):
            S = decay[t, head][:, None] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, head] = S.T @ q[t, g]
    out = rms(out, eps) * w[pre + "norm"][None, None, :] * gate
    return out.reshape(T, H * dv) @ w[pre + "o"].T


def dense_ff(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def forward(config, w, tokens, dtype=torch.float64, streams=None):
    """Logits [T, vocab] of one sequence.  ``streams``, a list, receives what every layer passes on."""
    w = {n: (t.to(dtype) if t.is_floating_point() else t) for n, t in w.items()}
    eps, mult = config["norm"]["eps"], config["residual_mult"]
    x = embed(tokens, w["embed"], dtype)
    results = [x]
    kept = {}
    for i, layer in enumerate(config["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        h = unit_offset_norm(x, w[pre + "norm1"], eps)
        if layer["type"] == "attention":
            src = m.get("kv_from")
            y, kept[i] = attention(h, w, pre + "mix.", m, kept[src] if src is not None else None)
        elif layer["type"] == "channel_delta":
            y = channel_delta(h, w, pre + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + mult * unit_offset_norm(y, w[pre + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = unit_offset_norm(x, w[pre + "norm2"], eps)
            x = x + mult * unit_offset_norm(dense_ff(h, w, pre + "mlp."), w[pre + "norm2b"], eps)
        results.append(x)
        x = sum(w[pre + "dwa"][j] * results[j] for j in range(i + 2))
        if streams is not None:
            streams.append(x)
    x = unit_offset_norm(x, w["final.norm"], eps)
    logits = x @ w["embed"].T
    cap = config["logit_softcap"]
    return cap * torch.tanh(logits / cap)
