"""Small Povatar models for the tests: configurations that differ from each other in every size and option, and random
weights for them, written as a model folder (config.json, model.safetensors in bfloat16)."""
from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def left(heads, kv_heads, dim, vdim, size, rot_dims, base=10000.0, scaling=None, scale=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    return {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "mask": {"size": size}, "rot": rot,
            "scale": scale if scale is not None else dim ** -0.5}


def right(heads, vdim, state, groups, norm_groups, conv):
    return {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups, "state": state, "vdim": vdim}


def moe(experts, top, ff):
    return {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top}}


def layer(left_half, right_half, mlp):
    return {"type": "parallel", "mixer": {"left": left_half, "right": right_half}, "mlp": mlp}


def config(layers, width=64, vocab=97, embed_scale=4.0, eps=1e-5):
    return {"architecture": "Povatar", "embedding": {"scale": embed_scale}, "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


STRETCH = {"factor": 4.0, "fast": 16.0, "original": 64, "slow": 2.0}
# Layers that differ from each other: grouped and ungrouped heads, key and value sizes that differ and are no multiples of
# 16, a rotation of part of a head and of all of it, with and without the stretch, blocks of positions that end inside
# pages, one and several groups of the recurrence, a layer without a feed-forward, one expert of one, all experts chosen.
MIXED = config([
    layer(left(4, 2, 24, 40, size=19, rot_dims=8, scaling=STRETCH), right(4, 12, 16, 2, 2, conv=3), moe(6, 2, 24)),
    layer(left(2, 2, 32, 32, size=33, rot_dims=32, base=500.0), right(3, 8, 5, 1, 1, conv=2), None),
    layer(left(4, 1, 16, 16, size=7, rot_dims=4, scaling={"factor": 2.0, "fast": 4.0, "original": 16, "slow": 1.0}, scale=0.4),
          right(2, 40, 24, 2, 4, conv=4), moe(3, 3, 40)),
    layer(left(2, 1, 48, 16, size=64, rot_dims=16), right(6, 4, 8, 3, 3, conv=1), moe(1, 1, 16)),
], width=64, vocab=97)
# One layer with the head size of the kernels' widest tiles and a state as wide as a wave.
WIDE = config([layer(left(4, 2, 128, 128, size=150, rot_dims=64, scaling={"factor": 6.0, "fast": 20.0, "original": 256, "slow": 1.5}),
                     right(2, 64, 64, 1, 2, conv=4), moe(8, 2, 72))], width=96, vocab=130, embed_scale=9.0)
CONFIGS = {"MIXED": MIXED, "WIDE": WIDE}


def random_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0):
        return torch.randn(*shape, generator=g) * std

    def uniform(*shape, lo=-1.0, hi=1.0):
        return torch.rand(*shape, generator=g) * (hi - lo) + lo

    W = cfg["width"]
    w = {"embed": normal(cfg["vocab"], W, std=1.0 / cfg["embedding"]["scale"]), "final.norm": uniform(W, lo=0.7, hi=1.3),
         "head": normal(cfg["vocab"], W, std=W ** -0.5)}
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        a, b = spec["mixer"]["left"], spec["mixer"]["right"]
        w[p + "norm1"] = uniform(W, lo=0.7, hi=1.3)
        w[p + "norm2"] = uniform(W, lo=0.7, hi=1.3)
        H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        w[p + "mix.left.q"] = normal(H * d, W, std=2.0 * W ** -0.5)
        w[p + "mix.left.k"] = normal(G * d, W, std=2.0 * W ** -0.5)
        w[p + "mix.left.v"] = normal(G * dv, W, std=W ** -0.5)
        w[p + "mix.left.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
        w[p + "mix.left.out"] = uniform(W, lo=0.5, hi=1.5)
        Hn, P, N, Gn, K = b["heads"], b["vdim"], b["state"], b["groups"], b["conv"]
        inner, C = Hn * P, Hn * P + 2 * Gn * N
        w[p + "mix.right.in"] = normal(2 * inner + 2 * Gn * N + Hn, W, std=W ** -0.5)
        w[p + "mix.right.conv"] = normal(C, K, std=0.6)
        w[p + "mix.right.conv.b"] = normal(C, std=0.2)
        w[p + "mix.right.dt_bias"] = uniform(Hn, lo=-3.0, hi=0.5)
        w[p + "mix.right.A_log"] = uniform(Hn, lo=-2.0, hi=1.0)
        w[p + "mix.right.D"] = uniform(Hn, lo=0.5, hi=1.5)
        w[p + "mix.right.norm"] = uniform(inner, lo=0.5, hi=1.5)
        w[p + "mix.right.o"] = normal(W, inner, std=inner ** -0.5)
        w[p + "mix.right.out"] = uniform(W, lo=0.5, hi=1.5)
        if spec["mlp"]:
            E, F = spec["mlp"]["router"]["experts"], spec["mlp"]["expert"]["ff"]
            w[p + "mlp.router"] = normal(E, W, std=2.0 * W ** -0.5)
            for e in range(E):
                w[p + f"mlp.e{e}.up"] = normal(F, W, std=W ** -0.5)
                w[p + f"mlp.e{e}.down"] = normal(W, F, std=F ** -0.5)
    # What the file stores is what both sides compute with.
    return {n: t.to(torch.bfloat16).contiguous() for n, t in w.items()}


def write_model(folder, cfg, weights):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file(weights, str(folder / "model.safetensors"))
    return folder
