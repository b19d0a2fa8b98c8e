"""The Povatar architecture on the CPU: what the native library makes of its config.json, the rule for the stretched
rotation frequencies, and the plain implementation's own pieces against torch's routines and equations written out."""
import json
import math
import subprocess

import numpy as np
import pytest
import torch

import plain_povatar as plain
from povatar_models import MIXED, STRETCH, config, layer, left, moe, random_weights, right, write_model
from vosti_amd.cache.host import rotary_stretched_frequencies
from vosti_amd.config import ConfigError, config_from_dict
from vosti_amd.kernels import build


def test_description_of_a_configuration():
    c = config_from_dict(MIXED)
    assert c.architecture == "Povatar" and c.vocab == 97 and c.width == 64 and c.layers == 4 and c.embedding_scale == 4.0
    spec = c.model_spec()
    assert [l.block for l in spec.layers] == ["parallel_sum"] * 4
    assert [l.mixer.kind for l in spec.layers] == ["pair_mean"] * 4
    assert [l.feed_forward.kind for l in spec.layers] == ["routed_experts", "none", "routed_experts", "routed_experts"]
    assert [(e.layer, e.cache_from) for e in spec.schedule] == [(0, None), (1, None), (2, None), (3, None)]
    assert spec.embedding.kind == "token_embedding_scaled" and spec.embedding.params["scale"] == 4.0
    assert spec.final_norm.params == {"size": 64, "eps": 1e-5}
    assert spec.names["head.weight"] == "head" and spec.names["embedding.weight"] == "embed"
    f = spec.layers[2].feed_forward.params
    assert (f["experts"], f["top"], f["intermediate_size"], f["weight_eps"]) == (3, 3, 40, 1e-20)
    assert spec.layers[0].names["feed_forward.experts.5.down_proj.weight"] == "l0.mlp.e5.down"
    assert spec.layers[0].names["mixer.right.conv.bias"] == "l0.mix.right.conv.b" and spec.layers[0].names["mixer.left_out"] == "l0.mix.left.out"
    assert "norms.ffn_in.weight" not in spec.layers[1].names and spec.layers[0].names["norms.ffn_in.weight"] == "l0.norm2"


def test_the_halves_of_a_mixer_in_the_library_s_own_words():
    """The description as the library writes it: the halves are parts below the pair, the rotation a part below the attention."""
    from vosti_amd.config.registry import describe
    m = describe(MIXED)["layers"][0]["mixer"]
    a, b = m["parts"]["left_mixer"], m["parts"]["right_mixer"]
    assert a["kind"] == "attention" and b["kind"] == "state_space"
    n = a["numbers"]
    assert (n["num_heads"], n["num_kv_heads"], n["head_dim"], n["value_dim"], n["block"], n["sink"], n["exact_weights"]) == (4, 2, 24, 40, 19, 2, 1)
    r = a["parts"]["position"]
    assert r["kind"] == "rotary_stretched" and (r["numbers"]["rotary_dim"], r["numbers"]["factor"], r["numbers"]["original"]) == (8, 4, 64)
    n = b["numbers"]
    assert (n["num_heads"], n["value_dim"], n["state_dim"], n["groups"], n["norm_groups"], n["conv_taps"]) == (4, 12, 16, 2, 2, 3)
    plain_rot = describe(MIXED)["layers"][1]["mixer"]["parts"]["left_mixer"]["parts"]["position"]["numbers"]
    assert "factor" not in plain_rot and plain_rot["theta"] == 500.0


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][1].update(type="serial"), "unknown mixer type"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][0]["mixer"]["left"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(groups=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(norm_groups=5), "norm_groups"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "moe"),
    (lambda c: c.pop("embedding"), "embedding"),
])
def test_configuration_errors_name_the_key(change, text):
    cfg = json.loads(json.dumps(MIXED))
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(cfg)


def test_tensor_names_are_the_files(tmp_path):
    """The program's own description of a model folder lists exactly the tensors that such a file holds (a layer without
    a feed-forward has no use for its second norm; a file may hold it all the same)."""
    w = random_weights(MIXED, 1)
    folder = write_model(tmp_path / "m", MIXED, w)
    program = str(build.ensure("engine", verbose=False))
    r = subprocess.run([program, "--kind", "describe", "--model-path", str(folder)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    got = json.loads(r.stdout)
    assert got["architecture"] == "Povatar"
    assert got["tensor_names"] == sorted(n for n in w if n != "l1.norm2")


@pytest.mark.parametrize("rot", [
    {"base": 10000.0, "dims": 8, "scaling": STRETCH},
    {"base": 50000.0, "dims": 64, "scaling": {"factor": 6.0, "fast": 24.0, "original": 4096, "slow": 1.5}},
    {"base": 300.0, "dims": 6, "scaling": {"factor": 2.0, "fast": 4.0, "original": 16, "slow": 1.0}},
    {"base": 500.0, "dims": 32},
])
def test_stretched_frequencies_are_the_formula(rot):
    s = rot.get("scaling") or {}
    got, mag = rotary_stretched_frequencies(rot["base"], rot["dims"], s.get("factor", 0.0), s.get("original", 1.0), s.get("fast", 1.0), s.get("slow", 1.0))
    want, want_mag = plain.rotation_frequencies(rot)
    assert np.allclose(got, want.numpy(), rtol=2e-7, atol=0) and abs(mag - want_mag) < 1e-6
    if s:      # the fastest pair is untouched, the slowest divided by the factor, and nothing in between leaves that range
        plainf = np.array([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)])
        assert np.all(got <= plainf * (1 + 1e-6)) and np.all(got >= plainf / s["factor"] * (1 - 1e-6))
        assert mag == pytest.approx(0.1 * math.log(s["factor"]) + 1.0)


def test_rotation_keeps_what_it_does_not_turn_and_turns_pairs_half_apart():
    x = torch.randn(5, 2, 12, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    rot = {"base": 100.0, "dims": 4}
    y = plain.rotate(x, torch.arange(5), rot)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.equal(y[0], x[0])
    a = 3 * 100.0 ** (-2 * 1 / 4)                                # position 3, pair 1: elements 1 and 3
    assert torch.allclose(y[3, :, 1], x[3, :, 1] * math.cos(a) - x[3, :, 3] * math.sin(a))
    assert torch.allclose(y[3, :, 3], x[3, :, 3] * math.cos(a) + x[3, :, 1] * math.sin(a))


def test_visibility_in_blocks():
    seen = [[plain.block_visible(i, j, 4) for j in range(10)] for i in range(10)]
    assert seen[3] == [True] * 4 + [False] * 6 and seen[4] == [False] * 4 + [True] + [False] * 5
    assert seen[9] == [False] * 8 + [True, True] and seen[0] == [True] + [False] * 9


def test_attention_weights_leave_room_for_the_constant():
    """One head, two tokens, written out: p = exp(s) / (1 + sum exp(s))."""
    m = left(1, 1, 4, 4, size=8, rot_dims=2, scale=0.5)
    m.pop("rot")
    g = torch.Generator().manual_seed(2)
    w = {"q": torch.randn(4, 6, generator=g, dtype=torch.float64), "k": torch.randn(4, 6, generator=g, dtype=torch.float64),
         "v": torch.randn(4, 6, generator=g, dtype=torch.float64), "o": torch.eye(4, dtype=torch.float64)}
    h = torch.randn(2, 6, generator=g, dtype=torch.float64)
    got = plain.block_attention(h, w, "", m)
    q, k, v = h @ w["q"].T, h @ w["k"].T, h @ w["v"].T
    e00 = math.exp(float(q[0] @ k[0]) * 0.5)
    e10, e11 = math.exp(float(q[1] @ k[0]) * 0.5), math.exp(float(q[1] @ k[1]) * 0.5)
    assert torch.allclose(got[0], e00 / (1 + e00) * v[0]) and torch.allclose(got[1], (e10 * v[0] + e11 * v[1]) / (1 + e10 + e11))


def test_convolution_against_torch():
    g = torch.Generator().manual_seed(0)
    x, taps, bias = (torch.randn(*s, generator=g, dtype=torch.float64) for s in ((11, 6), (6, 4), (6,)))
    ref = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), taps[:, None, :], bias=bias, groups=6)[0].T
    assert torch.allclose(plain.causal_conv(x, taps, bias), ref, atol=1e-12)


def test_recurrence_as_a_sum_over_the_past():
    """y_t = sum over s <= t of exp(A (dt_(s+1) + ... + dt_t)) dt_s (C_t . B_s) x_s + D x_t, for one head without convolution taps."""
    cfg = config([layer(left(1, 1, 8, 8, size=4, rot_dims=2), right(1, 3, 4, 1, 1, conv=1), None)], width=8, vocab=10)
    w = {n: t.double() for n, t in random_weights(cfg, 2).items()}
    h = torch.randn(5, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    p, m = "l0.mix.right.", cfg["layers"][0]["mixer"]["right"]
    got = plain.state_space(h, w, p, m, 1e-5)
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :3], plain.silu(proj[:, 3:14] * w[p + "conv"][:, 0] + w[p + "conv.b"]), torch.nn.functional.softplus(proj[:, 14] + w[p + "dt_bias"][0])
    x, B, C = xbc[:, :3], xbc[:, 3:7], xbc[:, 7:11]
    A = -torch.exp(w[p + "A_log"][0])
    y = torch.zeros(5, 3, dtype=torch.float64)
    for t in range(5):
        for s in range(t + 1):
            y[t] += torch.exp(A * dt[s + 1:t + 1].sum()) * dt[s] * (C[t] @ B[s]) * x[s]
        y[t] += w[p + "D"][0] * x[t]
    gated = y * plain.silu(z)
    gated = gated / torch.sqrt((gated * gated).mean(-1, keepdim=True) + 1e-5) * w[p + "norm"]
    assert torch.allclose(got, gated @ w[p + "o"].T, atol=1e-10)


def test_gated_norm_takes_each_part_by_itself():
    y, z, wt = torch.tensor([[3.0, 4.0, 0.0, 10.0]], dtype=torch.float64), torch.full((1, 4), 50.0, dtype=torch.float64), torch.ones(4, dtype=torch.float64)
    out = plain.group_norm_gate(y, z, wt, 2, 0.0)      # silu(50) = 50: the gate multiplies before the norm, which divides it out
    assert torch.allclose(out, torch.tensor([[3.0, 4.0, 0.0, 10.0]], dtype=torch.float64) / torch.tensor([12.5 ** 0.5, 12.5 ** 0.5, 50 ** 0.5, 50 ** 0.5], dtype=torch.float64))


def test_routing_weights_sum_to_one_over_the_chosen():
    g = torch.Generator().manual_seed(3)
    h, router = torch.randn(9, 6, generator=g, dtype=torch.float64), torch.randn(5, 6, generator=g, dtype=torch.float64)
    idx, wt = plain.route(h, router, 2)
    s = torch.softmax(h @ router.T, -1)
    for t in range(9):
        order = sorted(range(5), key=lambda e: -float(s[t, e]))[:2]
        assert idx[t].tolist() == order
        assert torch.allclose(wt[t], s[t, order] / s[t, order].sum())
    idx, wt = plain.route(h, router, 5)
    assert torch.allclose(wt, s.gather(1, idx))                 # all chosen: the scores themselves


def test_experts_written_out():
    cfg = config([layer(left(1, 1, 8, 8, size=4, rot_dims=2), right(1, 4, 4, 1, 1, conv=1), moe(3, 1, 5))], width=8, vocab=10)
    w = {n: t.double() for n, t in random_weights(cfg, 4).items()}
    h = torch.randn(4, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(5))
    got = plain.experts(h, w, "l0.mlp.", cfg["layers"][0]["mlp"])
    for t in range(4):
        e = int((h[t] @ w["l0.mlp.router"].T).argmax())
        assert torch.allclose(got[t], w[f"l0.mlp.e{e}.down"] @ torch.relu(w[f"l0.mlp.e{e}.up"] @ h[t]) ** 2)
