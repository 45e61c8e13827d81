"""Dumazen on the GPU against its plain implementation (``tests/plain/dumazen_plain.py``): each mechanism alone, whole
prompts against portions and token-by-token decoding, unequal requests in one batch against each alone, pages and state
slots that are used again, keys at page borders and at both sides of a window's edge, tokens far back in every recurrent
state, the first tokens, long decoding through recorded steps, sizes that are no multiples of anything, and greedy
generation through the entry point and its scheduler."""
import numpy as np
import pytest
import torch

from tests.dumazen_util import (ALL_SMALL, SMALL_A, SMALL_B, SMALL_C, WAVES, check_rows, config, expected, gated_delta, layer,
                                make_folder, mamba2, parallel, plain_logits, plain_of, retention, rot, tokens_of,
                                window_attention)
from tests.plain import dumazen_plain as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {s["name"]: make_folder(s, tmp_path_factory.mktemp(f"dz{s['name']}")) for s in ALL_SMALL}


def entry(rid, tokens, want=None):
    from jax_vllm_amd.engine.entries import StepEntry

    return StepEntry(rid, tokens, range(len(tokens)) if want is None else want)


def make_core(folder, dtype, page_size, pages=64, seqs=4, graphs=False):
    from jax_vllm_amd.config import EngineConfig
    from jax_vllm_amd.engine.core import EngineCore
    from jax_vllm_amd.weights import load_model

    model, _ = load_model(folder, dtype, "cuda")
    cfg = EngineConfig(dtype=dtype, block_size=page_size, num_blocks=pages + 1, max_num_seqs=seqs,
                       max_model_len=pages * page_size, max_num_batched_tokens=4096, enable_prefix_cache=False,
                       use_hip_graphs=graphs)
    return EngineCore(model, cfg)


def run_cut(core, rid, tokens, cuts):
    """The request's logits at every position, its tokens fed in portions of the given sizes."""
    core.start_request(rid)
    out, at = [], 0
    for n in cuts:
        out.append(core.run([entry(rid, tokens[at:at + n])]).cpu().numpy())
        at += n
    assert at == len(tokens)
    core.finish_request(rid)
    return np.concatenate(out)


# ------------------------------------------------------------------ each mechanism alone
QUIET = gated_delta(1, 1, 4, 4, conv=2)            # the smallest partner for a window attention under test
ALONE = {
    "retention": layer(retention(3, 12, 20, (0.3, 0.9, 0.9995), rot(8, 50.0))),
    "retention_plain": layer(retention(2, 6, 4, (1.0, 0.0))),
    "state_space": layer(mamba2(4, 6, 10, groups=2, norm_groups=2, conv=3)),
    "state_space_wide": layer(mamba2(3, 20, 40, groups=1, norm_groups=3, conv=5)),
    "window_attention": layer(parallel(window_attention(4, 2, 12, 20, window=13, scale=1.5, rot_=rot(8, 100.0, WAVES)), QUIET, 1.0, 0.05)),
    "attention_no_window_no_rotation": layer(parallel(window_attention(2, 2, 20, 12), QUIET, 1.0, 0.05)),
    "gated_delta": layer(parallel(window_attention(1, 1, 4, 4, window=1), gated_delta(4, 2, 12, 20, conv=3), 0.05, 1.0)),
    "feed_forward": layer(retention(1, 4, 4, (0.5,)), 72),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", sorted(ALONE))
def test_one_layer_of_each_mechanism(tmp_path, dtype, which):
    """A model of one layer (a mixer without a feed-forward; a mixer beside the smallest partner with a small scale; the
    smallest mixer under the feed-forward): a prompt of 70 tokens whole, and again in portions down to two tokens and
    single ones."""
    small = dict(name=which, seed=11, std=0.3, norm_std=0.2, config=config(40, 61, [ALONE[which]], mult=0.9))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 70, 1)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 8)
    check_rows(dtype, run_cut(core, "whole", toks, [70]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [2, 3, 1, 17, 2, 31, 1, 1, 2, 10]), want, "portions")


# ------------------------------------------------------------------ portions, decoding, first tokens
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("small", ALL_SMALL, ids=[s["name"] for s in ALL_SMALL])
def test_whole_prompt_portions_and_decoding_agree(folders, dtype, small):
    cfg, w = plain_of(folders[small["name"]])
    toks = tokens_of(cfg, 75, 2)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folders[small["name"]], dtype, small["page_size"])
    check_rows(dtype, run_cut(core, "whole", toks, [75]), want, "whole")
    check_rows(dtype, run_cut(core, "single", toks, [1] * 75), want, "token by token")
    check_rows(dtype, run_cut(core, "twos", toks, [2] * 37 + [1]), want, "portions of two")
    check_rows(dtype, run_cut(core, "mixed", toks, [7, 9, 16, 1, 1, 33, 8]), want, "portions of several sizes")
    check_rows(dtype, run_cut(core, "prompt+decode", toks, [40] + [1] * 35), want, "prompt, then decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("small", ALL_SMALL, ids=[s["name"] for s in ALL_SMALL])
def test_first_tokens_of_a_sequence(folders, dtype, small):
    """The convolutions see zeros before the first token, the states start at zero, the window holds fewer keys than
    its size: prompts of one to five tokens in every cut."""
    cfg, w = plain_of(folders[small["name"]])
    toks = [5, 1, 9, 2, 7]
    want = expected(cfg, w, toks, dtype)
    core = make_core(folders[small["name"]], dtype, small["page_size"])
    for rid, cuts in (("one", [1, 1, 1, 1, 1]), ("two", [1, 2, 2]), ("three", [3, 2]), ("whole", [5])):
        check_rows(dtype, run_cut(core, rid, toks, cuts), want, rid)
    check_rows(dtype, run_cut(core, "alone", toks[:1], [1]), expected(cfg, w, toks[:1], dtype), "a prompt of one token")


# ------------------------------------------------------------------ windows and page borders
@pytest.mark.parametrize("dtype", DTYPES)
def test_keys_at_both_sides_of_a_window_and_at_page_borders(tmp_path, dtype):
    """One window-attention layer (its partner scaled away) whose scores are so flat that every key in the window
    counts: a window of 11 over pages of 8.  One key too many or too few moves every row by far more than the tolerance
    (checked on the plain implementation).  Prompt portions end and begin at page borders, one before and one after
    them, and decoding carries the window over two further pages."""
    def cfg_with(window):
        return config(32, 50, [layer(parallel(window_attention(2, 1, 16, 24, window=window, scale=0.05, rot_=rot(8, 100.0)), QUIET, 1.0, 0.001))])

    small = dict(name="w", seed=21, std=0.2, norm_std=0.1, config=cfg_with(11))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 60, 3)
    want = expected(cfg, w, toks, dtype)
    plain = plain_logits(cfg, w, toks)
    for other in (10, 12):      # the oracle itself must tell the window from its neighbours, else this test shows nothing
        far = np.abs(plain_logits(cfg_with(other), w, toks)[15:] - plain[15:]).max(axis=-1)
        assert np.median(far) > 0.05 * np.abs(plain).max() and far.min() > 0.002 * np.abs(plain).max()
    core = make_core(folder, dtype, 8, pages=12)
    check_rows(dtype, run_cut(core, "whole", toks, [60]), want, "whole")
    check_rows(dtype, run_cut(core, "borders", toks, [8, 7, 1, 9, 15, 1, 1, 2, 16]), want, "cut at page borders")
    check_rows(dtype, run_cut(core, "decode", toks, [23] + [1] * 37), want, "decoding over the window's edge")
    assert core.cache.num_free_pages(0) == 12       # every page came back


@pytest.mark.parametrize("dtype", DTYPES)
def test_one_far_key_among_hundreds_without_a_window(tmp_path, dtype):
    """Attention over every earlier key with scores sharp enough that single keys carry a row, as often as not far ones:
    rows beyond position 200 change by much when the plain implementation is kept from seeing keys more than 150 back.
    300 tokens over 19 pages: whole, in portions around page borders, and with the last 40 decoded one by one."""
    def cfg_with(window):
        return config(32, 50, [layer(parallel(window_attention(2, 2, 16, 8, window=window, scale=3.0, rot_=rot(16, 1e4)), QUIET, 1.0, 0.001))])

    small = dict(name="far", seed=23, std=0.3, norm_std=0.1, config=cfg_with(None))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 300, 12)
    want = expected(cfg, w, toks, dtype)
    plain = plain_logits(cfg, w, toks)
    near = plain_logits(cfg_with(150), w, toks)
    assert np.median(np.abs(near[200:] - plain[200:]).max(axis=-1)) > 0.01 * np.abs(plain).max()
    core = make_core(folder, dtype, 16, pages=20)
    check_rows(dtype, run_cut(core, "whole", toks, [300]), want, "whole")
    check_rows(dtype, run_cut(core, "portions", toks, [64, 63, 1, 17, 47, 2, 66] + [1] * 40), want, "portions and decoding")


FAR_STATES = {
    # a decay of 1 in one head: the first token's share of the state does not fade
    "retention": (layer(retention(2, 16, 16, (1.0, 0.9999), rot(16, 1e4))), {}),
    # decay rates of e^-12: exp(-rate * dt) stays 1 to six digits over 330 tokens
    "state_space": (layer(mamba2(2, 16, 16, conv=4)), {"l0.mix.A_log": -12.0}),
    "gated_delta": (layer(parallel(window_attention(1, 1, 4, 4, window=2), gated_delta(2, 2, 16, 16), 0.001, 1.0)),
                    {"l0.mix.right.A_log": -12.0}),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", sorted(FAR_STATES))
def test_a_far_token_stays_in_the_state(tmp_path, dtype, which):
    """One recurrent layer that hardly forgets: logits 330 tokens later still depend on the first token, through portions
    and decoding; a state that is lost, zeroed at a portion's start or decayed once too often shows."""
    lay, patch = FAR_STATES[which]
    small = dict(name="f", seed=22, std=0.4, norm_std=0.1, config=config(32, 50, [lay]))
    folder = make_folder(small, tmp_path, patch)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 330, 4)
    want = expected(cfg, w, toks, dtype)
    plain = plain_logits(cfg, w, toks)
    other = plain_logits(cfg, w, [(toks[0] + 1) % 50] + toks[1:])
    assert np.abs(other[-1] - plain[-1]).max() > 1e-3 * np.abs(plain).max()       # the first token is still seen at the end
    core = make_core(folder, dtype, 16, pages=24)
    check_rows(dtype, run_cut(core, "whole", toks, [330]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [100, 2, 31, 64, 33, 70] + [1] * 30), want, "portions and decoding")


# ------------------------------------------------------------------ batches, pages and slots used again
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("small", [SMALL_A, SMALL_B], ids=["A", "B"])
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(folders, dtype, small):
    """Seven requests of 1 to 90 tokens through two state slots and a small pool of pages, portions of some beside single
    tokens of others; each request's logits equal the plain implementation's of it alone."""
    cfg, w = plain_of(folders[small["name"]])
    ps = small["page_size"]
    lengths = [33, 1, 90, 17, 64, 5, 48]
    reqs = {f"r{i}": tokens_of(cfg, n, 10 + i) for i, n in enumerate(lengths)}
    want = {r: expected(cfg, w, t, dtype) for r, t in reqs.items()}
    core = make_core(folders[small["name"]], dtype, ps, pages=max(14, 2 * (-(-90 // ps)) + 2), seqs=2)
    got = {r: [] for r in reqs}
    at = {r: 0 for r in reqs}
    waiting, live = list(reqs), []
    rng = np.random.default_rng(5)
    slots_seen = []
    while waiting or live:
        while waiting and len(live) < 2:
            r = waiting.pop(0)
            core.start_request(r)
            slots_seen.append(core.cache.slot(r))
            live.append(r)
        entries = []
        for r in live:
            left = len(reqs[r]) - at[r]
            n = 1 if (at[r] > 0 and rng.integers(2)) else int(min(left, rng.choice([1, 2, 3, 8, 21])))
            entries.append(entry(r, reqs[r][at[r]:at[r] + n]))
            at[r] += n
        logits = core.run(entries).cpu().numpy()
        k = 0
        for e in entries:
            got[e.request_id].append(logits[k:k + len(e.tokens)])
            k += len(e.tokens)
        for r in list(live):
            if at[r] == len(reqs[r]):
                core.finish_request(r)
                live.remove(r)
        core.cache.check_invariants()
    assert sorted(set(slots_seen)) == [0, 1] and len(slots_seen) == 7         # slots were used again
    if dtype == "float32":
        for r in reqs:
            check_rows(dtype, np.concatenate(got[r]), want[r], r)
    else:       # few rows a request: the shares of rows that rounding moves far are judged over all of them
        check_rows(dtype, np.concatenate([x for r in reqs for x in got[r]]),
                   tuple(np.concatenate([want[r][k] for r in reqs]) for k in (0, 1)), "all requests")


# ------------------------------------------------------------------ long decoding, recorded steps
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "recorded"])
def test_long_decoding(folders, dtype, graphs):
    """260 decoded tokens behind a prompt of 9: far beyond the window, over many pages, with pages of the window given
    back on the way; with recorded steps two requests decode side by side (the shorter one leaves a padded row)."""
    cfg, w = plain_of(folders["A"])
    a, b = tokens_of(cfg, 269, 6), tokens_of(cfg, 150, 7)
    want_a, want_b = expected(cfg, w, a, dtype), expected(cfg, w, b, dtype)
    core = make_core(folders["A"], dtype, SMALL_A["page_size"], pages=40, graphs=graphs)
    core.start_request("a")
    core.start_request("b")
    got_a = [core.run([entry("a", a[:9])]).cpu().numpy()]
    got_b = [core.run([entry("b", b[:30])]).cpu().numpy()]
    for i in range(9, 269):
        es = [entry("a", a[i:i + 1])]
        j = 30 + i - 9
        if j < 150:
            es.append(entry("b", b[j:j + 1]))
        out = core.run(es).cpu().numpy()
        got_a.append(out[:1])
        if j < 150:
            got_b.append(out[1:2])
    check_rows(dtype, np.concatenate(got_a), want_a, "a")
    check_rows(dtype, np.concatenate(got_b), want_b, "b")
    if graphs:
        assert core.graph_replays > 200


# ------------------------------------------------------------------ the entry point
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_entry_point(folders, dtype):
    """Four prompts through ``LLM.generate`` with two slots, a small token budget (prompts are cut) and few pages: in
    float32 every token is the plain implementation's argmax; in bfloat16 each token is within a margin of the plain
    maximum given what came before."""
    from jax_vllm_amd import LLM, SamplingParams

    cfg, w = plain_of(folders["C"])
    prompts = [tokens_of(cfg, n, 30 + n) for n in (3, 41, 18, 70)]
    llm = LLM(folders["C"], dtype=dtype, block_size=SMALL_C["page_size"], max_num_seqs=2, max_model_len=128,
              max_num_batched_tokens=24, num_blocks=9)
    assert llm.prewarm() > 0.0            # records the decode steps of both batch sizes; leaves no trace in the state slots
    got = llm.generate(prompts, SamplingParams(max_new_tokens=12))
    assert [len(g) for g in got] == [12] * 4
    assert llm.stats.graph_replays > 0
    for p, g in zip(prompts, got):
        seq = list(p)
        for i, t in enumerate(g):
            logits = P.forward(w, cfg, seq)[-1]
            if dtype == "float32":
                assert int(torch.argmax(logits)) == t, f"token {i}: engine {t}, plain {int(torch.argmax(logits))}"
            else:
                assert float(logits.max() - logits[t]) <= 0.06 * float(logits.abs().max()), f"token {i} is far below the maximum"
            seq.append(t)


def test_command_line_runs_the_design(folders, capsys):
    from jax_vllm_amd.engine.cli import main

    cfg, w = plain_of(folders["B"])
    prompt = tokens_of(cfg, 12, 40)
    code = main(["--model-path", str(folders["B"]), "--dtype", "fp32", "--block-size", "16", "--max-model-len", "64",
                 "--max-prefill-len", "32", "--max-new-tokens", "5", "--no-prewarm", "--prompt-ids",
                 " ".join(map(str, prompt))])
    assert code == 0
    got = [int(t) for t in capsys.readouterr().out.split()]
    seq = list(prompt)
    for t in got:
        assert int(torch.argmax(P.forward(w, cfg, seq)[-1])) == t
        seq.append(t)
    assert len(got) == 5


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_with_four_slots_and_a_pool_for_the_live_requests_only(folders, dtype, tmp_path):
    """``bin/trace_run`` on a mixed schedule: nine requests of 20 to 150 tokens, at most four live, portions of some
    beside single tokens of others, some sitting a step out; the pool holds what the live requests hold at the peak, so
    pages and slots are used again; then one request whole, one with its tail decoded, one in portions down to two."""
    from tests.replay_util import Trace, compare, mixed, portions, run_trace, tail_one_by_one, whole

    cfg, w = plain_of(folders["A"])
    rng = np.random.default_rng(17)
    reqs = {f"q{i}": tokens_of(cfg, n, 50 + i) for i, n in enumerate((150, 20, 77, 64, 33, 129, 48, 90, 65))}
    trace = Trace()
    peak = mixed(trace, reqs, rng)
    whole(trace, "q0#w", reqs["q0"])
    tail_one_by_one(trace, "q2#t", reqs["q2"], tail=40)
    portions(trace, "q5#p", reqs["q5"], (2, 31, 3, 17))
    got = run_trace(folders["A"], dtype, trace, max(peak, 192), tmp_path / "out", block_size=SMALL_A["page_size"])
    want = {r: expected(cfg, w, t, dtype) for r, t in reqs.items()}
    rows_got, rows_plain, rows_rounded = [], [], []

    def collect(name, pos, got_row, want_row):
        rows_got.append(got_row)
        if dtype == "float32":
            rows_plain.append(want_row)
        else:
            rows_plain.append(want_row[0][pos])
            rows_rounded.append(want_row[1][pos])

    if dtype == "float32":
        n = compare(trace, got, want, collect)
        check_rows(dtype, np.stack(rows_got), np.stack(rows_plain), "trace")
    else:
        n = compare(trace, got, {r: _Both(v) for r, v in want.items()}, collect)
        check_rows(dtype, np.stack(rows_got), (np.stack(rows_plain), np.stack(rows_rounded)), "trace")
    assert n == sum(len(t) for t in reqs.values()) + 150 + 41 + 129


class _Both:
    """(plain logits, plain logits with rounded products) of a request, indexed by position as one."""

    def __init__(self, pair):
        self.pair = pair

    def __getitem__(self, pos):
        return self.pair


# ------------------------------------------------------------------ sizes that are no multiples of anything
@pytest.mark.parametrize("dtype", DTYPES)
def test_odd_sizes_and_heads_beyond_the_matrix_core_kernels(tmp_path, dtype):
    """A width that is no multiple of 4, a value size of 260 (above the matrix-core attention kernels: the float kernel
    runs in bfloat16 too), key sizes of 6 and 10, a state of 5 x 3, seven taps, feed-forwards of odd sizes."""
    small = dict(name="odd", seed=31, std=0.25, norm_std=0.2, config=config(50, 61, [
        layer(parallel(window_attention(2, 1, 10, 260, window=40, rot_=rot(6)), gated_delta(3, 3, 6, 5, conv=7), 0.5, 2.0), 21),
        layer(mamba2(5, 3, 5, groups=5, norm_groups=1, conv=2), 13),
        layer(retention(2, 6, 10, (0.8, 0.99), rot(2, 10.0))),
    ]))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 70, 8)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 16)
    check_rows(dtype, run_cut(core, "whole", toks, [70]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [33, 2, 1, 17, 1, 1, 15]), want, "portions")


@pytest.mark.parametrize("dtype", DTYPES)
def test_wider_layers_and_a_prompt_of_many_chunks(tmp_path, dtype):
    """Six layers at a width of 256 with heads of 32 to 64 (the sizes at which the matrix-core attention kernels, the
    chunked recurrences and the streaming products all run), the mixers in another order, a window of 100 inside a
    prompt of 420 tokens: whole, in portions that end inside chunks, pages and the window, and with a decoded tail."""
    small = dict(name="wide", seed=41, std=0.08, norm_std=0.1, config=config(256, 500, [
        layer(parallel(window_attention(6, 3, 32, 64, window=100, scale=0.2, rot_=rot(16, 5e4, dict(WAVES, original=256, factor=8.0))),
                       gated_delta(4, 2, 48, 32, conv=4), 0.6, 0.9), 320),
        layer(mamba2(8, 32, 64, groups=2, norm_groups=2, conv=3)),
        layer(retention(4, 64, 48, (0.97, 0.99, 0.999, 0.9999), rot(32, 1e6)), 192),
        layer(mamba2(8, 32, 64, groups=1, norm_groups=1, conv=4)),
        layer(parallel(window_attention(4, 4, 64, 32, window=37, rot_=rot(64, 1e4)), gated_delta(2, 2, 64, 64, conv=2), 1.1, 0.4)),
        layer(retention(2, 32, 128, (0.9, 0.995))),
    ], mult=0.7))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 420, 9)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 16, pages=40)
    whole, cut = run_cut(core, "whole", toks, [420]), run_cut(core, "cut", toks, [100, 31, 2, 64, 33, 7, 129, 14] + [1] * 40)
    if dtype == "bfloat16":
        check_rows(dtype, whole, want, "whole")
        check_rows(dtype, cut, want, "portions and decoding")
        return
    # six layers deep a few positions are badly conditioned (a small sublayer output in front of its norm): the plain
    # implementation in float32 is itself off there, so a row may be off by three times that on top of the usual bound
    own = np.abs(P.forward(P.read_weights(folder, torch.float32), cfg, toks).numpy().astype(np.float64) - want).max(axis=-1)
    scale = float(np.abs(want).max())
    for what, got in (("whole", whole), ("portions and decoding", cut)):
        err = np.abs(got.astype(np.float64) - want).max(axis=-1)
        worst = int((err - 3 * own).argmax())
        assert (err <= 3e-5 * scale + 1e-5 + 3 * own).all(), f"{what}: row {worst} is off by {err[worst]}, plain float32 by {own[worst]}"
        assert np.median(err) <= 1e-5 * scale, f"{what}: median error {np.median(err)}"


# ------------------------------------------------------------------ kernels alone
def _recurrence_reference(q, k, v, g, wgt, skip, state, lens, slots, heads, qk_heads, delta):
    n = v.shape[0]
    out = torch.zeros(n, heads, v.shape[-1], dtype=torch.float64)
    t = 0
    for ln, s in zip(lens, slots):
        for _ in range(ln):
            for h in range(heads):
                hk = h // (heads // qk_heads)
                S = state[s, h] * g[t, h]
                u = wgt[t, h] * (v[t, h] - S.T @ k[t, hk]) if delta else wgt[t, h] * v[t, h]
                S = S + torch.outer(k[t, hk], u)
                state[s, h] = S
                out[t, h] = S.T @ q[t, hk] + skip[h] * v[t, h]
            t += 1
    return out


@pytest.mark.parametrize("delta", [False, True], ids=["plain", "delta"])
@pytest.mark.parametrize("heads,qk_heads,dim,vdim", [(2, 2, 16, 16), (4, 2, 40, 72), (1, 1, 128, 130), (6, 2, 200, 24), (2, 1, 18, 7)])
def test_recurrence_kernel(delta, heads, qk_heads, dim, vdim):
    """The recurrence against float64: three requests of 1, 45 and 100 tokens with states that do not start at zero, in
    slots that are not in order, q and k shared by groups of heads and read from wider rows; decays per token and per
    head alone; the state after the step is compared as well, and the other slots are left alone."""
    from jax_vllm_amd.ops import kernels as K

    gen = torch.Generator().manual_seed(dim + vdim + delta)
    lens, slots = [1, 45, 100], [2, 0, 3]
    n = sum(lens)
    wide = torch.randn(n, 2 * qk_heads * dim + 3, generator=gen) * (0.3 if delta else 0.7)
    q, k = wide[:, :qk_heads * dim], wide[:, qk_heads * dim + 3:]
    if delta:       # keys of at most unit length, as the delta rule is used
        k.copy_((k.view(n, qk_heads, dim) / k.view(n, qk_heads, dim).norm(dim=-1, keepdim=True).clamp_min(1.0)).view(n, -1))
    v = torch.randn(n, heads * vdim, generator=gen) * 0.7
    g = torch.rand(n, heads, generator=gen) * 0.5 + 0.5
    wgt = torch.rand(n, heads, generator=gen)
    skip = torch.randn(heads, generator=gen)
    state0 = torch.randn(5, heads, dim, vdim, generator=gen) * 0.5
    cu = torch.tensor([0, 1, 46, 146], dtype=torch.int32, device="cuda")
    sl = torch.tensor(slots, dtype=torch.int32, device="cuda")
    for per_token, with_w, with_skip in ((True, True, True), (False, False, False)):
        gg = g if per_token else g[:1].expand(n, heads).contiguous()
        want_state = state0.double().clone()
        want = _recurrence_reference(q.double().view(n, qk_heads, dim), k.double().view(n, qk_heads, dim), v.double().view(n, heads, vdim),
                                     gg.double(), wgt.double() if with_w else torch.ones(n, heads, dtype=torch.float64),
                                     skip.double() if with_skip else torch.zeros(heads, dtype=torch.float64), want_state, lens, slots,
                                     heads, qk_heads, delta)
        state = state0.cuda().clone()
        wc = wide.cuda()
        out = K.recurrence_steps(wc[:, :qk_heads * dim], wc[:, qk_heads * dim + 3:], v.cuda(), (gg if per_token else gg[0]).contiguous().cuda(),
                                 state, sl, cu, heads, qk_heads, dim, vdim, write=wgt.cuda() if with_w else None,
                                 skip=skip.cuda() if with_skip else None, delta=delta)
        scale = float(want.abs().max())
        assert float((out.cpu().double().view(n, heads, vdim) - want).abs().max()) <= 3e-5 * scale, f"per_token={per_token}"
        assert float((state.cpu().double() - want_state).abs().max()) <= 3e-5 * float(want_state.abs().max())
        assert torch.equal(state[1].cpu(), state0[1]) and torch.equal(state[4].cpu(), state0[4])    # other slots untouched
        if K.recurrence_chunks_possible(dim, delta):       # the same by chunks of tokens side by side
            state = state0.cuda().clone()
            out = K.recurrence_steps(wc[:, :qk_heads * dim], wc[:, qk_heads * dim + 3:], v.cuda(), (gg if per_token else gg[0]).contiguous().cuda(),
                                     state, sl, cu, heads, qk_heads, dim, vdim, write=wgt.cuda() if with_w else None,
                                     skip=skip.cuda() if with_skip and not delta else None, delta=delta,
                                     chunk_plan=K.recurrence_chunk_plan(lens, "cuda"))
            if delta and with_skip:
                out = out + (skip.cuda()[None, :, None] * v.cuda().view(n, heads, vdim)).view(n, -1)
            assert float((out.cpu().double().view(n, heads, vdim) - want).abs().max()) <= 3e-5 * scale, f"chunks, per_token={per_token}"
            assert float((state.cpu().double() - want_state).abs().max()) <= 3e-5 * float(want_state.abs().max())
            assert torch.equal(state[1].cpu(), state0[1]) and torch.equal(state[4].cpu(), state0[4])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("taps,channels", [(4, 70), (2, 300), (8, 5), (1, 12)])
def test_short_convolution_with_state(dtype, taps, channels):
    """Requests of 1, 2, 3, 70 and 200 tokens in one launch, their earlier inputs in state rows that are not in order:
    outputs and the state the step leaves, against the sum written out; a second step continues from that state."""
    from jax_vllm_amd.ops import kernels as K

    gen = torch.Generator().manual_seed(taps * 100 + channels)
    lens, slots = [1, 2, 3, 70, 200], [4, 1, 0, 5, 2]
    n, off = sum(lens), 3
    w, b = torch.randn(channels, taps, generator=gen), torch.randn(channels, generator=gen)
    state0 = torch.randn(7, taps - 1, channels, generator=gen).to(dtype).float()
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device="cuda")
    sl = torch.tensor(slots, dtype=torch.int32, device="cuda")
    state = state0.cuda().clone()
    history = {s: state0[s].double() for s in slots}
    for step in range(2):
        proj = torch.randn(n, channels + 7, generator=gen).to(dtype)
        want, t = torch.zeros(n, channels, dtype=torch.float64), 0
        for ln, s in zip(lens, slots):
            x = torch.cat([history[s], proj[t:t + ln, off:off + channels].double()])
            for i in range(ln):
                want[t + i] = (x[i:i + taps] * w.double().T).sum(0) + b.double()
            history[s] = x[x.shape[0] - (taps - 1):]
            t += ln
        want = torch.nn.functional.silu(want)
        out = K.short_conv(proj.cuda(), off, channels, w.cuda(), b.cuda(), state, sl, cu, max(lens))
        assert float((out.cpu().double() - want).abs().max()) <= 1e-5 * max(1.0, float(want.abs().max())), f"step {step}"
        for s in slots:
            assert torch.equal(state[s].cpu().double(), history[s]), f"state of slot {s} after step {step}"
        assert torch.equal(state[3].cpu(), state0[3]) and torch.equal(state[6].cpu(), state0[6])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_gates_heads_and_norms_around_the_recurrence(dtype):
    """The small kernels against their formulas in float64: decays and write strengths, heads rotated and scaled as
    float, unit vectors per head in place on the leading heads of wider rows, the norm in groups with its gate before
    or behind it and a weight that repeats."""
    from jax_vllm_amd.ops import kernels as K

    gen = torch.Generator().manual_seed(5)
    n, heads, d = 37, 3, 10
    proj = (torch.randn(n, 80, generator=gen) * 2).to(dtype)
    bias, a_log = torch.randn(heads, generator=gen), torch.randn(heads, generator=gen) - 1
    raw = proj.double()
    dt = torch.nn.functional.softplus(raw[:, 5:5 + heads] + bias.double(), threshold=1e9)
    for beta_off in (None, 20):
        g, wg = K.recurrence_gates(proj.cuda(), 5, bias.cuda(), a_log.cuda(), heads, beta_off=beta_off)
        assert float((g.cpu().double() - torch.exp(-torch.exp(a_log.double()) * dt)).abs().max()) < 1e-6
        want_w = dt if beta_off is None else torch.sigmoid(raw[:, 20:20 + heads])
        assert float((wg.cpu().double() - want_w).abs().max()) < 1e-5
    pos = torch.arange(100, 100 + n, dtype=torch.int32)
    r = rot(6, 50.0)
    table = K.rope_table(pos.cuda(), P.rotary_frequencies(r).float().cuda())
    got = K.heads_to_f32(proj.cuda(), 7, heads, d, 6, table, scale=0.3).cpu().double().view(n, heads, d)
    want = P.rotate(raw[:, 7:7 + heads * d].view(n, heads, d).transpose(0, 1), pos, r).transpose(0, 1) * 0.3
    assert float((got - want).abs().max()) < 1e-4 * float(want.abs().max())
    both = K.qkv_to_f32(proj.cuda(), heads, d, 4, 6, table, k_scale=0.3).cpu().double()      # q, k and v of one mixer in one launch
    wq = P.rotate(raw[:, :heads * d].view(n, heads, d).transpose(0, 1), pos, r).transpose(0, 1).reshape(n, -1)
    wk = P.rotate(raw[:, heads * d:2 * heads * d].view(n, heads, d).transpose(0, 1), pos, r).transpose(0, 1).reshape(n, -1) * 0.3
    wantb = torch.cat([wq, wk, raw[:, 2 * heads * d:2 * heads * d + heads * 4]], dim=1)
    assert both.shape == wantb.shape and float((both - wantb).abs().max()) < 1e-4 * float(wantb.abs().max())
    x = torch.randn(n, 5 * d + 3, generator=gen)
    y = x.cuda().clone()
    K.head_unit_norm(y, 4, d, 1e-6, scale=2.0, first_heads=1, first_scale=0.5)
    xv = x.double()[:, :4 * d].view(n, 4, d)
    wantu = xv / torch.sqrt((xv * xv).sum(-1, keepdim=True) + 1e-6) * torch.tensor([0.5, 2.0, 2.0, 2.0], dtype=torch.float64)[None, :, None]
    assert float((y.cpu().double()[:, :4 * d].view(n, 4, d) - wantu).abs().max()) < 1e-6
    assert torch.equal(y.cpu()[:, 4 * d:], x[:, 4 * d:])
    wide = (torch.randn(n, 610, generator=gen) * 2).to(dtype)
    for width, weight_len, cases in ((24, 8, ((8, False, "silu", True), (12, True, "silu", False), (24, False, "sigmoid", True), (4, True, "sigmoid", True))),
                                     (600, 300, ((300, True, "silu", True), (600, False, "silu", False)))):      # wide groups take a block each
        o = torch.randn(n, width, generator=gen)
        weight = 1 + 0.3 * torch.randn(weight_len, generator=gen)
        src = proj if width == 24 else wide
        gate = src[:, 10:10 + width]
        for group, first, act, weighted in cases:
            a = torch.nn.functional.silu(gate.double()) if act == "silu" else torch.sigmoid(gate.double())
            z = o.double() * a if first else o.double()
            z = (z.view(n, -1, group) / torch.sqrt((z.view(n, -1, group) ** 2).mean(-1, keepdim=True) + 1e-3)).view(n, width)
            if weighted:
                z = z * weight.double().repeat(width // weight_len)
            z = (z if first else z * a) * 0.7
            got = K.group_gated_norm(o.cuda(), src.cuda()[:, 10:10 + width], weight.cuda() if weighted else None, group, 1e-3, act,
                                     gate_first=first, out_scale=0.7)
            tol = 1e-5 if dtype == torch.float32 else 1e-2
            assert float((got.cpu().double() - z).abs().max()) <= tol * max(1.0, float(z.abs().max())), (group, first, act)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_attention_input_with_heads_of_two_sizes(dtype):
    """Bias, the norm over the whole projection, partial rotation, scaled values and zero padding, into q rows and pages
    of both layouts; tokens without a slot store nothing; the pad of the pages stays zero."""
    from jax_vllm_amd.ops import kernels as K

    gen = torch.Generator().manual_seed(9)
    n, nq, nkv, dk, dv, ps, pages = 21, 4, 2, 12, 20, 8, 6
    dp = K.padded_head_dim(dk, dv)
    assert dp == 32
    width = (nq + nkv) * dk + nkv * dv
    qkv = torch.randn(n, width, generator=gen).to(dtype)
    bias = torch.randn(width, generator=gen)
    qw, kw = 1 + 0.2 * torch.randn(nq * dk, generator=gen), 1 + 0.2 * torch.randn(nkv * dk, generator=gen)
    pos = torch.arange(3, 3 + n, dtype=torch.int32)
    r = rot(8, 30.0)
    table = K.rope_table(pos.cuda(), P.rotary_frequencies(r).float().cuda())
    slots = torch.randperm(pages * ps - ps, generator=gen)[:n].to(torch.int32) + ps
    slots[4] = -1
    kp = torch.zeros(pages, nkv, ps, dp, dtype=dtype, device="cuda")
    vp = torch.zeros(pages, nkv, dp, ps, dtype=dtype, device="cuda")
    q = K.attn_prepare_wide(qkv.cuda(), bias.cuda(), qw.cuda(), kw.cuda(), 1e-4, table, 8, slots.cuda(), kp, vp, ps, nq, nkv, dk, dv, dp, v_scale=0.6)
    x = qkv.double() + bias.double()
    xq, xk, xv = x[:, :nq * dk], x[:, nq * dk:(nq + nkv) * dk], x[:, (nq + nkv) * dk:]
    wq = (P.rms(xq, 1e-4) * qw.double()).view(n, nq, dk).transpose(0, 1)
    wk = (P.rms(xk, 1e-4) * kw.double()).view(n, nkv, dk).transpose(0, 1)
    wq, wk = P.rotate(wq, pos, r).transpose(0, 1), P.rotate(wk, pos, r).transpose(0, 1)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    got_q = q.cpu().double().view(n, nq, dp)
    assert float((got_q[..., :dk] - wq).abs().max()) <= tol * float(wq.abs().max()) and float(got_q[..., dk:].abs().max()) == 0.0
    kc, vc = kp.cpu().double(), vp.cpu().double()
    seen = torch.zeros(pages, ps, dtype=torch.bool)
    for t in range(n):
        s = int(slots[t])
        if s < 0:
            continue
        pg, at = s // ps, s % ps
        seen[pg, at] = True
        assert float((kc[pg, :, at, :dk] - wk[t]).abs().max()) <= tol * float(wk.abs().max())
        assert float((vc[pg, :, :dv, at] - 0.6 * xv[t].view(nkv, dv)).abs().max()) <= tol * float(xv.abs().max())
    assert float(kc[..., dk:].abs().max()) == 0.0 and float(vc[:, :, dv:, :].abs().max()) == 0.0
    assert float(kc.transpose(1, 2)[~seen].abs().max()) == 0.0          # slots of no token hold nothing


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_bias_with_activation_stream_in_the_activation_type_and_weighed_sums(dtype):
    from jax_vllm_amd.ops import kernels as K

    gen = torch.Generator().manual_seed(2)
    y0, b = (torch.randn(9, 50, generator=gen) * 2).to(dtype), torch.randn(50, generator=gen)
    z = y0.double() + b.double()
    wants = {"gelu": 0.5 * z * (1 + torch.erf(z / 2 ** 0.5)), "gelu_tanh": torch.nn.functional.gelu(z, approximate="tanh"),
             "silu": torch.nn.functional.silu(z), None: z}
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for act, want in wants.items():
        y = y0.cuda().clone()
        K.bias_act(y, b.cuda(), act)
        assert float((y.cpu().double() - want).abs().max()) <= tol * float(want.abs().max()), act
    # the kernel that adds a sublayer's normed output to the stream hands the stream on without a norm where no weight is given
    h0, yy, wb = torch.randn(9, 52, generator=gen), torch.randn(9, 52, generator=gen).to(dtype), 1 + 0.3 * torch.randn(52, generator=gen)
    want_h = h0.double() + P.rms(yy.double(), 1e-3) * wb.double()
    h, out = h0.cuda().clone(), torch.empty(9, 52, dtype=dtype, device="cuda")
    K.postnorm_add_rmsnorm(h, yy.cuda(), None, wb.cuda(), 1e-3, None, out)
    assert float((h.cpu().double() - want_h).abs().max()) <= 1e-5
    assert float((out.cpu().double() - want_h).abs().max()) <= tol * float(want_h.abs().max())
    # a bias that the sublayer's output still owes is added before its norm, in rows of any width
    for width in (52, 50):
        bb = torch.randn(width, generator=gen)
        want_b = h0[:, :width].double() + P.rms(yy[:, :width].double() + bb.double(), 1e-3) * wb[:width].double()
        h = h0[:, :width].contiguous().cuda()
        K.postnorm_add_rmsnorm(h, yy[:, :width].contiguous().cuda(), None, wb[:width].contiguous().cuda(), 1e-3, None, None, bias=bb.cuda())
        assert float((h.cpu().double() - want_b).abs().max()) <= 1e-5, width
    parts = torch.randn(3, 9, 52, generator=gen)
    acc = torch.empty(9, 52, dtype=torch.float32, device="cuda")
    K.scaled_sum(acc, (yy.cuda(), parts.cuda()), 0.6)
    assert float((acc.cpu().double() - 0.6 * (yy.double() + parts.double().sum(0))).abs().max()) <= 1e-5
    K.scaled_sum(acc, yy.cuda(), -2.0)
    assert float((acc.cpu().double() + 2.0 * yy.double()).abs().max()) <= 1e-5
