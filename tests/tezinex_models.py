"""Small Tezinex models for the tests: configurations that differ from each other in every size and option, and
random weights for them, written as a model folder (config.json, model.safetensors in bfloat16)."""
from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def attention_layer(heads, kv_heads, dim, vdim, size, keep_first, scale=None, softcap=20.0, kv_from=None, ff=None):
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "mask": {"size": size, "keep_first": keep_first},
             "scale": scale if scale is not None else dim ** -0.5, "softcap": softcap}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta_layer(heads, kv_heads, dim, vdim, conv, ff=None):
    return {"type": "channel_delta", "mixer": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "conv": conv},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=64, vocab=97, residual_mult=0.6, eps=1e-5, logit_softcap=12.0):
    return {"architecture": "Tezinex", "layers": layers, "logit_softcap": logit_softcap, "norm": {"eps": eps}, "residual_mult": residual_mult,
            "vocab": vocab, "width": width}


# Attention first, two windows (two cache groups), grouped heads in both mixers, key and value sizes that differ and
# are no multiples of 16, a layer that reads another's keys past a layer in between, a feed-forward on a delta layer,
# convolutions of two and five taps.
MIXED = config([
    attention_layer(4, 2, 24, 40, size=19, keep_first=5, ff=80),
    delta_layer(4, 2, 16, 24, conv=2, ff=48),
    attention_layer(2, 2, 32, 32, size=33, keep_first=0, softcap=8.0),
    attention_layer(4, 2, 24, 40, size=19, keep_first=5, kv_from=0),
    delta_layer(3, 3, 40, 8, conv=5),
], width=64, vocab=97)
# Delta layers only; wide key size (several lanes a column), one head.
DELTAS = config([delta_layer(1, 1, 96, 48, conv=3), delta_layer(2, 1, 8, 72, conv=4, ff=40)], width=48, vocab=61, residual_mult=1.0,
                logit_softcap=26.0)
# One attention layer alone, all q heads on one kv head, the head size of the kernels' widest tiles.
ATTENTION = config([attention_layer(4, 1, 128, 128, size=40, keep_first=3, ff=None)], width=96, vocab=130, residual_mult=0.9)

RANKS = {"MIXED": (5, 12), "DELTAS": (8, 3), "ATTENTION": (4, 4)}     # ranks of the decay and gate projections


def random_weights(cfg, seed, decay_rank=5, gate_rank=12):
    g = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0):
        return torch.randn(*shape, generator=g) * std

    def uniform(*shape, lo=-1.0, hi=1.0):
        return torch.rand(*shape, generator=g) * (hi - lo) + lo

    W = cfg["width"]
    w = {"embed": normal(cfg["vocab"], W, std=1.0), "final.norm": uniform(W, lo=-0.3, hi=0.3)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        w[p + "norm1"] = uniform(W, lo=-0.3, hi=0.3)
        w[p + "norm1b"] = uniform(W, lo=-0.3, hi=0.3)
        w[p + "dwa"] = uniform(i + 2, lo=0.1, hi=0.9)
        if layer["type"] == "attention":
            w[p + "mix.q"] = normal(H * d, W, std=2.0 * W ** -0.5)
            w[p + "mix.q.b"] = normal(H * d, std=0.3)
            if "kv_from" not in m:
                w[p + "mix.k"] = normal(G * d, W, std=2.0 * W ** -0.5)
                w[p + "mix.k.b"] = normal(G * d, std=0.3)
                w[p + "mix.v"] = normal(G * dv, W, std=W ** -0.5)
                w[p + "mix.v.b"] = normal(G * dv, std=0.3)
            w[p + "mix.sink"] = uniform(H, lo=-2.0, hi=3.0)
            w[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
        else:
            K = m["conv"]
            for n, rows in (("q", G * d), ("k", G * d), ("v", H * dv)):
                w[p + f"mix.{n}"] = normal(rows, W, std=2.0 * W ** -0.5)
                w[p + f"mix.{n}.conv"] = normal(rows, K, std=0.6)
            w[p + "mix.b"] = normal(H, W, std=W ** -0.5)
            w[p + "mix.A_log"] = uniform(H, lo=-2.0, hi=0.5)
            w[p + "mix.norm"] = uniform(dv, lo=0.5, hi=1.5)
            w[p + "mix.a1"] = normal(decay_rank, W, std=W ** -0.5)
            w[p + "mix.a2"] = normal(H * d, decay_rank, std=decay_rank ** -0.5)
            w[p + "mix.dt_bias"] = uniform(H * d, lo=-3.0, hi=1.0)
            w[p + "mix.g1"] = normal(gate_rank, W, std=W ** -0.5)
            w[p + "mix.g2"] = normal(H * dv, gate_rank, std=gate_rank ** -0.5)
            w[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
        if layer["mlp"]:
            F = layer["mlp"]["ff"]
            w[p + "norm2"] = uniform(W, lo=-0.3, hi=0.3)
            w[p + "norm2b"] = uniform(W, lo=-0.3, hi=0.3)
            w[p + "mlp.gate"] = normal(F, W, std=W ** -0.5)
            w[p + "mlp.up"] = normal(F, W, std=W ** -0.5)
            w[p + "mlp.down"] = normal(W, F, std=F ** -0.5)
    # What the file stores is what both sides compute with.
    return {n: t.to(torch.bfloat16).contiguous() for n, t in w.items()}


def write_model(folder, cfg, weights):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file(weights, str(folder / "model.safetensors"))
    return folder
