"""The Tezinex architecture on the CPU: what the native library makes of its config.json, the cache manager's groups
that keep a request's first keys, and the plain implementation's own pieces against torch's routines."""
import json
import subprocess

import pytest
import torch

import plain_tezinex as plain
from tezinex_models import MIXED, RANKS, attention_layer, config, delta_layer, random_weights, write_model
from vosti_amd.cache.manager import CacheError, CacheManager, GroupSpec
from vosti_amd.config import ConfigError, config_from_dict
from vosti_amd.kernels import build


def test_description_of_a_configuration():
    c = config_from_dict(MIXED)
    assert c.architecture == "Tezinex" and c.vocab == 97 and c.width == 64 and c.layers == 5
    spec = c.model_spec()
    assert [l.mixer.kind for l in spec.layers] == ["attention", "channel_delta", "attention", "attention", "channel_delta"]
    assert [l.feed_forward.kind for l in spec.layers] == ["swiglu", "swiglu", "none", "none", "none"]
    assert [(e.layer, e.cache_from) for e in spec.schedule] == [(0, None), (1, None), (2, None), (3, 0), (4, None)]
    a = spec.layers[0].mixer.params
    assert (a["num_heads"], a["num_kv_heads"], a["head_dim"], a["value_dim"], a["window"], a["keep_first"]) == (4, 2, 24, 40, 19, 5)
    assert a["softcap"] == 20.0 and a["scale"] == 24 ** -0.5 and a["own_kv"] == 1 and spec.layers[3].mixer.params["own_kv"] == 0
    d = spec.layers[4].mixer.params
    assert (d["num_heads"], d["num_kv_heads"], d["key_dim"], d["value_dim"], d["conv_taps"]) == (3, 3, 40, 8, 5)
    assert spec.embedding.kind == "token_embedding_sinusoid" and spec.head.params["softcap"] == 12.0
    assert spec.final_norm.params == {"size": 64, "eps": 1e-5, "offset": 1}
    assert spec.names["head.weight"] == spec.names["embedding.weight"] == "embed"
    assert "mixer.k_proj.weight" not in spec.layers[3].names and spec.layers[3].names["mixer.q_proj.bias"] == "l3.mix.q.b"


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][0]["mixer"].update(kv_from=0), "kv_from"),
    (lambda c: c["layers"][1].update(type="convolution"), "unknown mixer type"),
    (lambda c: c.update(width=63), "even"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].pop("mask"), "mask"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "dense"),
    (lambda c: c.pop("residual_mult"), "residual_mult"),
])
def test_configuration_errors_name_the_key(change, text):
    cfg = json.loads(json.dumps(MIXED))
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(cfg)


def test_tensor_names_are_the_files(tmp_path):
    """The program's own description of a model folder lists exactly the tensors that such a file holds."""
    folder = write_model(tmp_path / "m", MIXED, random_weights(MIXED, 1, *RANKS["MIXED"]))
    program = str(build.ensure("engine", verbose=False))
    r = subprocess.run([program, "--kind", "describe", "--model-path", str(folder)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    got = json.loads(r.stdout)
    assert got["architecture"] == "Tezinex"
    assert got["tensor_names"] == sorted(random_weights(MIXED, 1))


def test_kept_first_pages_are_never_given_back():
    m = CacheManager(4, [GroupSpec(0, 32), GroupSpec(6, 32, keep_first=5), GroupSpec(6, 32)], 2, False)
    m.add_request(1)
    for step in range(10):
        m.extend(1, list(range(5)))
        m.commit(1)
        assert m.check() == ""
    n = m.num_logical_pages(1, 0)
    assert n == 13                                              # 50 tokens in pages of 4
    assert len(set(m.block_table_row(1, 0, n).tolist())) == n
    # The next query stands at 50 and sees keys from 45 on: logical pages 11 and 12, and with kept keys pages 0 and 1.
    assert m.free_pages(2) == 32 - 2 and m.free_pages(1) == 32 - 4
    assert len(set(m.slots(1, 1, 0, 8).tolist())) == 8 and min(m.slots(1, 1, 0, 8).tolist()) >= 0      # the kept pages are still there
    assert len(set(m.slots(1, 1, 44, 6).tolist())) == 6
    with pytest.raises(CacheError):
        m.slots(1, 1, 8, 1)                                      # a page between the kept ones and the window is gone
    with pytest.raises(CacheError):
        m.slots(1, 2, 0, 1)                                      # and without kept keys the first page too
    m.finish(1)
    assert [m.free_pages(g) for g in range(3)] == [32, 32, 32] and m.check() == ""


def test_visibility():
    size, keep = 5, 2
    seen = [[plain.visible(i, j, size, keep) for j in range(10)] for i in range(10)]
    assert seen[9] == [True, True, False, False, False, True, True, True, True, True]
    assert seen[4] == [True] * 5 + [False] * 5 and seen[0] == [True] + [False] * 9
    assert seen[6][2] is True and seen[7][2] is False          # i - j < size, so 6 - 2 = 4 is inside and 7 - 2 = 5 is not


def test_convolution_and_positions_against_torch():
    g = torch.Generator().manual_seed(0)
    x, taps = torch.randn(11, 6, generator=g, dtype=torch.float64), torch.randn(6, 4, generator=g, dtype=torch.float64)
    ref = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), taps[:, None, :], groups=6)[0].T
    assert torch.allclose(plain.causal_conv(x, taps), ref, atol=1e-12)
    s = plain.sinusoid(torch.arange(7), 8, torch.float64)
    assert s[0].tolist() == [0.0, 1.0] * 4
    assert abs(s[5, 2] - torch.sin(torch.tensor(5 * 10000 ** (-2 / 8), dtype=torch.float64))) < 1e-12
    assert abs(s[5, 3] - torch.cos(torch.tensor(5 * 10000 ** (-2 / 8), dtype=torch.float64))) < 1e-12


def test_recurrence_written_out_for_two_tokens():
    """The delta rule of the plain implementation against its equations expanded by hand for one head."""
    cfg = config([delta_layer(1, 1, 4, 3, conv=1)], width=8, vocab=10)
    w = {n: t.double() for n, t in random_weights(cfg, 2, 2, 2).items()}
    h = torch.randn(2, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    got = plain.channel_delta(h, w, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    p = "l0.mix."
    q = plain.silu((h @ w[p + "q"].T) * w[p + "q.conv"][:, 0]); k = plain.silu((h @ w[p + "k"].T) * w[p + "k.conv"][:, 0])
    v = plain.silu((h @ w[p + "v"].T) * w[p + "v.conv"][:, 0])
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) / 2.0
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)[:, 0]
    g = torch.exp(-torch.exp(w[p + "A_log"][0]) * torch.log1p(torch.exp((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"])))
    S1 = torch.outer(k[0], beta[0] * v[0])
    o0 = S1.T @ q[0]
    S1d = g[1][:, None] * S1
    S2 = S1d + torch.outer(k[1], beta[1] * (v[1] - S1d.T @ k[1]))
    o = torch.stack([o0, S2.T @ q[1]])
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5) * w[p + "norm"] * torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T)
    assert torch.allclose(got, o @ w[p + "o"].T, atol=1e-10)
