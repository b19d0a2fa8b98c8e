"""The Tezinex decoder through the native engine against the plain implementation (tests/plain_tezinex.py).

Every test builds its own small model.  The engine is driven through its step function (given tokens in, logits out:
what bin/trace_run drives) and through its scheduler (``generate``).  In float32 the engine must agree with the plain
float64 implementation to a few units of 32-bit rounding; in bfloat16 to what rounding the matrix products to 16 bits
costs.  Two cuttings of the same tokens through the engine must agree far closer than either does with the plain
implementation: nothing may depend on portions, batches, pages or slots."""
import numpy as np
import pytest
import torch

import plain_tezinex as plain
from tezinex_models import ATTENTION, DELTAS, MIXED, RANKS, attention_layer, config, delta_layer, random_weights, write_model

pytestmark = pytest.mark.gpu

CONFIGS = {"MIXED": MIXED, "DELTAS": DELTAS, "ATTENTION": ATTENTION}
TOLERANCE = {"float32": 2e-4, "bfloat16": 6e-2}      # of the logits' root mean square
SAME = {"float32": 2e-5, "bfloat16": 2e-5}           # two cuttings of the same tokens through the engine


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for seed, (name, cfg) in enumerate(CONFIGS.items()):
        w = random_weights(cfg, 10 + seed, *RANKS[name])
        out[name] = (write_model(tmp_path_factory.mktemp(name), cfg, w), cfg, w)
    return out


def engine(folder, dtype, num_pages=24, page_size=16, max_num_seqs=4, **kw):
    from vosti_amd.engine.native import NativeEngine
    return NativeEngine(folder, dtype=dtype, num_pages=num_pages, page_size=page_size, max_num_seqs=max_num_seqs,
                        enable_prefix_cache=False, graphs=kw.pop("graphs", False), **kw)


def tokens_for(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_cut(eng, rid, tokens, cuts, finish=True):
    """All logits of one request fed in portions of the given sizes."""
    rows, at = [], 0
    for c in cuts:
        rows.append(eng.trace_step([(rid, tokens[at:at + c], list(range(c)))]))
        at += c
    assert at == len(tokens)
    if finish:
        eng.trace_finish(rid)
    return np.concatenate(rows, 0)


def deviation(got, want):
    """Largest row deviation as a fraction of the logits' root mean square."""
    want = np.asarray(want, dtype=np.float64)
    return float(np.sqrt(((got - want) ** 2).mean(-1)).max() / np.sqrt((want ** 2).mean()))


def plain_logits(cfg, w, tokens):
    return plain.forward(cfg, w, tokens, torch.float64).numpy()


# ------------------------------------------------------------------------------------------ each mechanism alone
ALONE = {
    "attention": config([attention_layer(4, 2, 16, 16, size=12, keep_first=2)], width=32, vocab=50),
    "attention_no_keep_wide_values": config([attention_layer(2, 1, 8, 48, size=7, keep_first=0, softcap=5.0)], width=32, vocab=50),
    "attention_all_visible": config([attention_layer(2, 2, 32, 16, size=500, keep_first=0)], width=32, vocab=50),
    "delta": config([delta_layer(2, 1, 16, 8, conv=3)], width=32, vocab=50),
    "delta_one_tap": config([delta_layer(2, 2, 24, 24, conv=1)], width=32, vocab=50),
    "feed_forward": config([delta_layer(1, 1, 8, 8, conv=2, ff=56)], width=32, vocab=50, residual_mult=1.3),
    "sizes_that_need_padding": config([delta_layer(3, 1, 10, 5, conv=3, ff=20), attention_layer(3, 3, 6, 10, size=8, keep_first=1, ff=12)], width=24, vocab=33),
    "shared_keys_seen_further_back": config([attention_layer(2, 2, 16, 16, size=5, keep_first=0), delta_layer(1, 1, 8, 8, conv=2),
                                             attention_layer(2, 2, 16, 16, size=23, keep_first=4, kv_from=0)], width=32, vocab=50),
    "shared_keys": config([attention_layer(2, 1, 16, 32, size=9, keep_first=1), attention_layer(2, 1, 16, 32, size=9, keep_first=1, kv_from=0)],
                          width=32, vocab=50),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ALONE))
def test_each_mechanism_alone(tmp_path, name, dtype):
    cfg = ALONE[name]
    w = random_weights(cfg, 3, decay_rank=3, gate_rank=9)
    folder = write_model(tmp_path / name, cfg, w)
    tokens = tokens_for(cfg, 45, 1)
    want = plain_logits(cfg, w, tokens)
    eng = engine(folder, dtype)
    assert deviation(run_cut(eng, 0, tokens, [45]), want) < TOLERANCE[dtype]
    assert deviation(run_cut(eng, 1, tokens, [9, 2, 17] + [1] * 17), want) < TOLERANCE[dtype]


def test_the_residual_stream_and_the_depth_average_are_32_bit(tmp_path):
    """Many layers with small updates: a stream rounded to 16 bits between layers would lose them."""
    layers = [delta_layer(1, 1, 8, 8, conv=2) for _ in range(12)]
    cfg = config(layers, width=32, vocab=40, residual_mult=0.02, logit_softcap=50.0)
    w = random_weights(cfg, 5, 2, 2)
    folder = write_model(tmp_path / "deep", cfg, w)
    tokens = tokens_for(cfg, 20, 2)
    got = run_cut(engine(folder, "bfloat16"), 0, tokens, [20])
    assert deviation(got, plain_logits(cfg, w, tokens)) < 1.5e-2


# ----------------------------------------------------------------------------- cuttings, batches, pages and slots
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_portions_and_decoding_agree(models, name, dtype):
    folder, cfg, w = models[name]
    n = 150
    tokens = tokens_for(cfg, n, 7)
    want = plain_logits(cfg, w, tokens)
    eng = engine(folder, dtype)
    whole = run_cut(eng, 0, tokens, [n])
    assert deviation(whole, want) < TOLERANCE[dtype]
    # The first tokens of a sequence on their own rows.
    assert deviation(whole[:4], want[:4]) < TOLERANCE[dtype]
    cuttings = {
        "token by token": [1] * n,
        "portions down to two tokens": [2, 3, 16, 2, 1, 31, 2, 33, 5, 1, 1, 2, 17, 32, 2],
        "a prompt and then decoding": [n - 60] + [1] * 60,
        "portions that end on page borders": [16, 48, 64, 22],
    }
    for what, cuts in cuttings.items():
        got = run_cut(eng, 1, tokens, cuts)
        assert deviation(got, whole) < SAME[dtype], what


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("head", [64, 128, 256])
def test_head_sizes_and_pages_of_the_kernels_that_share_tiles(tmp_path, head, dtype):
    """Head sizes 64, 128 and 256 with pages of 64: prompt rows go through the kernel that passes key tiles through LDS,
    decoded rows through the one that keeps the next tile in flight; windows and kept keys that end inside tiles,
    several prompt items, a prompt after cached keys."""
    cfg = config([attention_layer(4, 2, head, head, size=150, keep_first=70, softcap=15.0, ff=64),
                  attention_layer(4, 2, head, head, size=150, keep_first=70, softcap=15.0, kv_from=0)], width=64, vocab=90)
    w = random_weights(cfg, 31)
    folder = write_model(tmp_path / f"h{head}", cfg, w)
    n = 420
    tokens = tokens_for(cfg, n, 14)
    want = plain_logits(cfg, w, tokens)
    eng = engine(folder, dtype, num_pages=16, page_size=64)
    whole = run_cut(eng, 0, tokens, [n])
    assert deviation(whole, want) < TOLERANCE[dtype]
    for cuts in ([200, 150, 70], [n - 30] + [1] * 30, [64, 64, 129, 100, 63]):
        assert deviation(run_cut(eng, 1, tokens, cuts), whole) < SAME[dtype], cuts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch_equal_each_alone(models, dtype):
    folder, cfg, w = models["MIXED"]
    lengths = [70, 9, 41, 120]
    prompts = [tokens_for(cfg, n, 20 + i) for i, n in enumerate(lengths)]
    eng = engine(folder, dtype, num_pages=40)
    alone = [run_cut(eng, 10 + i, p, [len(p)]) for i, p in enumerate(prompts)]
    # Portions of some beside single tokens of others; a request is left out of a step and goes on later.
    schedule = [
        [(0, 30), (1, 2), (3, 64)],
        [(0, 1), (1, 1), (2, 20), (3, 3)],
        [(0, 1), (1, 1), (2, 1)],
        [(0, 38), (1, 5), (2, 20), (3, 53)],
    ]
    fed = [0] * 4
    got = [[] for _ in prompts]
    for step in schedule:
        entries = [(i, prompts[i][fed[i]:fed[i] + c], list(range(c))) for i, c in step]
        out = eng.trace_step(entries)
        at = 0
        for i, c in step:
            got[i].append(out[at:at + c])
            at += c
            fed[i] += c
    assert fed == lengths
    for i in range(4):
        assert deviation(np.concatenate(got[i], 0), alone[i]) < SAME[dtype], i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_and_slots_that_are_used_again(models, dtype):
    """A pool that holds one request at a time: every request gets the pages and the state slot that the one before
    it gave back, with the other's keys and states still in them."""
    folder, cfg, w = models["MIXED"]
    prompts = [tokens_for(cfg, n, 40 + i) for i, n in enumerate([90, 96, 33, 90])]
    fresh = [run_cut(engine(folder, dtype, num_pages=6, max_num_seqs=1), 0, p, [len(p)]) for p in prompts]
    eng = engine(folder, dtype, num_pages=6, max_num_seqs=1)
    for i, p in enumerate(prompts):
        got = run_cut(eng, i, p, [len(p) - 7, 3, 1, 1, 2])
        assert deviation(got, fresh[i]) < SAME[dtype], i
        assert eng.cache_check() == ""


def test_long_decoding_past_every_window(models):
    folder, cfg, w = models["MIXED"]
    n = 260
    tokens = tokens_for(cfg, n, 9)
    got = run_cut(engine(folder, "float32", num_pages=20), 0, tokens, [4] + [1] * (n - 4))
    assert deviation(got, plain_logits(cfg, w, tokens)) < TOLERANCE["float32"]


# ------------------------------------------------------------------------------ one key that stands out
def marked_attention_model(size, keep_first):
    """One attention layer in which a query token finds one key token wherever it stands.  The query and key
    projections are one matrix that reads the first half of the width, where both tokens carry the same large vector;
    the key projection also reads one more entry that only the key token has, along the query's own direction, so that
    the key token's score beats the query token's score with itself; the values read the second half, where the two
    tokens differ.  So whether that one key is visible moves the logits by far more than any tolerance."""
    W, d, vocab = 32, 16, 30
    cfg = config([attention_layer(1, 1, d, d, size=size, keep_first=keep_first, scale=0.25, softcap=50.0)], width=W, vocab=vocab,
                 residual_mult=6.0, logit_softcap=28.0)
    w = {n: t.float() for n, t in random_weights(cfg, 11).items()}
    g = torch.Generator().manual_seed(4)
    half, extra = W // 2, W - 1
    proj = torch.zeros(d, W)
    proj[:, :half] = torch.randn(d, half, generator=g) * 0.5
    mark = torch.randn(half, generator=g) * 3.0
    towards = proj[:, :half] @ mark
    w["l0.mix.q"], w["l0.mix.k"] = proj.clone(), proj.clone()
    w["l0.mix.k"][:, extra] = 3.0 * towards / towards.norm()
    w["l0.mix.q.b"].zero_(), w["l0.mix.k.b"].zero_()
    v = torch.zeros(d, W)
    v[:, half:] = torch.randn(d, W - half, generator=g)
    w["l0.mix.v"] = v
    w["l0.norm1"].zero_()
    w["l0.mix.sink"].fill_(-5.0)
    emb = torch.randn(vocab, W, generator=g) * 0.3
    emb[:, extra] = 0.0
    QUERY, KEY = 1, 2
    emb[QUERY, :half] = mark
    emb[KEY, :half] = mark
    emb[KEY, half:] = torch.randn(W - half, generator=g) * 1.5
    emb[KEY, extra] = 3.0
    w["embed"] = emb
    return cfg, {n: t.to(torch.bfloat16).contiguous() for n, t in w.items()}, QUERY, KEY


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_every_edge_in_prompts_and_in_decoding(tmp_path, dtype):
    size, keep = 37, 6
    cfg, w, QUERY, KEY = marked_attention_model(size, keep)
    folder = write_model(tmp_path / "marked", cfg, w)
    n = 200
    q_at = n - 1
    # (place of the key, visible): the window's edges, the kept keys' edge, far away, page borders (pages of 16).
    cases = [(q_at - size + 1, True), (q_at - size, False), (keep - 1, True), (keep, False), (0, True), (100, False),
             (q_at - 1, True), (175, True), (176, True), (q_at - size + 1 - 16, False), (15, False), (16, False)]
    base = [t if t not in (QUERY, KEY) else 3 for t in tokens_for(cfg, n, 8)]
    base[q_at] = QUERY
    without = plain_logits(cfg, w, base)[q_at]
    eng = engine(folder, dtype, num_pages=30)
    for place, seen in cases:
        tokens = list(base)
        tokens[place] = KEY
        want = plain_logits(cfg, w, tokens)[q_at]
        moved = float(np.sqrt(((want - without) ** 2).mean()) / np.sqrt((want ** 2).mean()))
        assert (moved > 0.08) == seen and (seen or moved < 1e-3), (place, moved)       # the plain implementation itself: the key matters iff visible
        for what, cuts in (("prompt", [n]), ("decoded", [n - 50] + [1] * 50), ("portions", [place + 1, n - place - 3, 2] if place + 4 < n else [n])):
            got = run_cut(eng, 0, tokens, cuts)[q_at]
            assert deviation(got[None], want[None]) < min(TOLERANCE[dtype], 0.02), (place, what)      # a quarter of what the key moves


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(tmp_path, dtype):
    """A kept first key seen from 700 tokens away, over pages that the window has long given back."""
    size, keep = 24, 4
    cfg, w, QUERY, KEY = marked_attention_model(size, keep)
    folder = write_model(tmp_path / "far", cfg, w)
    n = 720
    tokens = [t if t not in (QUERY, KEY) else 3 for t in tokens_for(cfg, n, 12)]
    tokens[2] = KEY
    tokens[-1] = QUERY
    want = plain_logits(cfg, w, tokens)[-1]
    without = list(tokens)
    without[2] = 3
    assert deviation(plain_logits(cfg, w, without)[-1][None], want[None]) > 0.08
    eng = engine(folder, dtype, num_pages=12, page_size=16)      # 192 keys: fewer than the request has tokens
    for cuts in ([100] * 7 + [19, 1], [90] * 7 + [70] + [1] * 20):
        got = run_cut(eng, 0, tokens, cuts)[-1]
        assert deviation(got[None], want[None]) < min(TOLERANCE[dtype], 0.02), cuts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_sink_that_takes_most_of_one_head(tmp_path, dtype):
    """Two heads, one with a sink far above its scores and one with a sink far below: a sink left out, scaled or
    capped would change how much each head contributes (the norm after the mixer hides a common factor, not this)."""
    cfg = config([attention_layer(2, 1, 16, 16, size=30, keep_first=2, softcap=4.0)], width=32, vocab=50, residual_mult=3.0)
    w = dict(random_weights(cfg, 21))
    w["l0.mix.sink"] = torch.tensor([9.0, -9.0]).to(torch.bfloat16)       # above the cap of 4: capping the sink would show
    folder = write_model(tmp_path / "sink", cfg, w)
    tokens = tokens_for(cfg, 70, 5)
    want = plain_logits(cfg, w, tokens)
    other = dict(w)
    other["l0.mix.sink"] = torch.tensor([4.0, -9.0]).to(torch.bfloat16)
    assert deviation(plain_logits(cfg, other, tokens), want) > 0.3
    eng = engine(folder, dtype)
    for cuts in ([70], [40] + [1] * 30):
        assert deviation(run_cut(eng, 0, tokens, cuts), want) < TOLERANCE[dtype], cuts


def test_a_lost_state_or_convolution_tail_would_show(models):
    """The delta layers alone: cutting between any two tokens must change nothing, so the state and the last inputs of
    the convolutions are carried; the plain implementation, given only the tokens after a cut, differs widely."""
    folder, cfg, w = models["DELTAS"]
    tokens = tokens_for(cfg, 40, 3)
    want = plain_logits(cfg, w, tokens)
    assert deviation(plain_logits(cfg, w, tokens[20:]), want[20:]) > 0.05
    eng = engine(folder, "float32")
    for cut in (1, 2, 3, 4, 20, 38, 39):
        got = run_cut(eng, 0, tokens, [cut, 40 - cut])
        assert deviation(got, want) < TOLERANCE["float32"], cut


# ------------------------------------------------------------------------ the engine's own entry point and scheduler
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_scheduler(models, graphs):
    from vosti_amd.sampling import SamplingParams
    folder, cfg, w = models["MIXED"]
    prompts = [tokens_for(cfg, n, 60 + i) for i, n in enumerate([23, 5, 48])]
    steps = 14
    eng = engine(folder, "float32", num_pages=30, graphs=graphs, max_num_batched_tokens=32)
    outs = eng.generate(prompts, SamplingParams(max_tokens=steps, ignore_eos=True))
    for p, out in zip(prompts, outs):
        assert len(out) == steps
        seq = list(p)
        for tok in out:
            logits = plain_logits(cfg, w, seq)[-1]
            best = int(logits.argmax())
            if tok != best:      # only a tie within rounding may be broken the other way
                assert logits[best] - logits[tok] < 1e-3 * np.abs(logits).max(), (len(seq), tok, best)
            seq.append(tok)


def test_create_engine_and_the_launcher_find_the_architecture(models):
    from vosti_amd.engine import create_engine
    from vosti_amd.engine.native import NativeEngine, native_support
    from vosti_amd.sampling import SamplingParams
    folder, cfg, w = models["DELTAS"]
    assert native_support(folder) == (True, "")
    eng = create_engine(str(folder), dtype="bfloat16", num_pages=8, max_num_seqs=2, graphs=True)
    assert isinstance(eng, NativeEngine)
    outs = eng.generate([tokens_for(cfg, 12, 1), tokens_for(cfg, 3, 2)], SamplingParams(max_tokens=20, temperature=0.7, seed=3, ignore_eos=True))
    assert [len(o) for o in outs] == [20, 20] and all(0 <= t < cfg["vocab"] for o in outs for t in o)
