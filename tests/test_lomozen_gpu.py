"""Lomozen on the GPU against its plain implementation (``tests/plain/lomozen_plain.py``): each mechanism
alone, whole prompts against portions and token-by-token decoding, unequal requests in one batch against
each alone, pages and state slots that are used again, keys at page borders and at both sides of a
window's edge, the first tokens, long decoding through recorded steps, sizes that are no multiples of
anything, and greedy generation through the entry point and its scheduler."""
import numpy as np
import pytest
import torch

from tests.lomozen_util import (ALL_SMALL, SMALL_A, SMALL_B, SMALL_C, YARN, check_rows, config, latent, layer, lightning,
                                expected, make_folder, moe, plain_logits, plain_of)
from tests.plain import lomozen_plain as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {s["name"]: make_folder(s, tmp_path_factory.mktemp(f"lz{s['name']}")) for s in ALL_SMALL}


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


def tokens_of(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], size=n).tolist()


# ------------------------------------------------------------------ each mechanism alone
ALONE = {
    "latent": layer(latent(3, 16, 8, 12, 24, 40, window=13, scale=2.0, scaling=YARN)),
    "latent_plain_rotation_no_window": layer(latent(2, 16, 16, 8, 16, 24, dims=6, base=100.0)),
    "lightning": layer(lightning(3, 12, 20, (0.3, 0.9, 0.9995))),
    "experts_top1": layer(lightning(1, 8, 8, (0.5,)), moe(7, 1, 24)),
    "experts_top3_shared": layer(lightning(1, 8, 8, (0.5,)), moe(7, 3, 24, 40)),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", sorted(ALONE))
def test_one_layer_of_each_mechanism(tmp_path, dtype, which):
    """A model of one layer (a mixer without a feed-forward, or the smallest mixer under the feed-forward
    in question): a prompt of 70 tokens whole, and again in portions down to two tokens and single ones."""
    small = dict(name=which, seed=11, std=0.3, norm_std=0.2, config=config(40, 61, [ALONE[which]]))
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
    cfg, w = plain_of(folders[small["name"]])
    toks = [5, 1, 9, 2, 7]
    want = expected(cfg, w, toks, dtype)
    core = make_core(folders[small["name"]], dtype, small["page_size"])
    for rid, cuts in (("one", [1, 1, 1, 1, 1]), ("two", [1, 2, 2]), ("whole", [5])):
        check_rows(dtype, run_cut(core, rid, toks, cuts), want, rid)
    check_rows(dtype, run_cut(core, "alone", toks[:1], [1]), expected(cfg, w, toks[:1], dtype), "a prompt of one token")


# ------------------------------------------------------------------ windows and page borders
@pytest.mark.parametrize("dtype", DTYPES)
def test_keys_at_both_sides_of_a_window_and_at_page_borders(tmp_path, dtype):
    """One latent-attention layer whose scores are so flat that every key in the window counts: a window of 11
    over pages of 8.  The logits at every position depend on exactly the keys i-10..i: one key too many
    or too few moves every row by far more than the tolerance (checked on the plain implementation).  Prompt portions end and begin at page borders, one before and one
    after them, and decoding carries the window over two further pages."""
    small = dict(name="w", seed=21, std=0.2, norm_std=0.1,
                 config=config(32, 50, [layer(latent(2, 16, 8, 16, 24, 24, window=11, scale=0.3))]))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 60, 3)
    want = expected(cfg, w, toks, dtype)
    # the oracle itself must tell the window from its neighbours, else this test shows nothing
    plain = plain_logits(cfg, w, toks)
    for other in (10, 12):
        c2 = config(32, 50, [layer(latent(2, 16, 8, 16, 24, 24, window=other, scale=0.3))])
        far = np.abs(plain_logits(c2, w, toks)[15:] - plain[15:]).max(axis=-1)
        assert np.median(far) > 0.05 * np.abs(plain).max() and far.min() > 0.002 * np.abs(plain).max()
    core = make_core(folder, dtype, 8, pages=12)
    check_rows(dtype, run_cut(core, "whole", toks, [60]), want, "whole")
    check_rows(dtype, run_cut(core, "borders", toks, [8, 7, 1, 9, 15, 1, 1, 2, 16]), want, "cut at page borders")
    check_rows(dtype, run_cut(core, "decode", toks, [23] + [1] * 37), want, "decoding over the window's edge")
    assert core.cache.num_free_pages(0) == 12       # every page came back


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_token_stays_in_the_lightning_state(tmp_path, dtype):
    """One lightning layer with a decay of 1 in one head and 0.9999 in the other: the first token's share of
    the state does not fade, so logits 300 tokens later still depend on it, through portions and decoding;
    a state that is lost or zeroed at a portion's start shows."""
    small = dict(name="f", seed=22, std=0.4, norm_std=0.1,
                 config=config(32, 50, [layer(lightning(2, 16, 16, (1.0, 0.9999)))]))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 330, 4)
    want = expected(cfg, w, toks, dtype)
    plain = plain_logits(cfg, w, toks)
    other = plain_logits(cfg, w, [(toks[0] + 1) % 50] + toks[1:])
    assert np.abs(other[-1] - plain[-1]).max() > 1e-3 * np.abs(plain).max()       # the first token is still seen at the end
    core = make_core(folder, dtype, 16, pages=4)
    check_rows(dtype, run_cut(core, "whole", toks, [330]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [100, 2, 31, 64, 33, 70] + [1] * 30), want, "portions and decoding")


# ------------------------------------------------------------------ batches, pages and slots used again
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("small", [SMALL_A, SMALL_B], ids=["A", "B"])
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(folders, dtype, small):
    """Seven requests of 1 to 90 tokens through two state slots and a pool of 14 pages, portions of some
    beside single tokens of others; each request's logits equal the plain implementation's of it alone."""
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
    """260 decoded tokens behind a prompt of 9: far beyond every window, over many pages, with pages of
    the window given back on the way; with recorded steps two requests decode side by side."""
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
    """Four prompts through ``LLM.generate`` with two slots, a small token budget (prompts are cut) and few
    pages: in float32 every token is the plain implementation's argmax; in bfloat16 each token is within a
    margin of the plain maximum given what came before."""
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


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("heads,dim,vdim", [(2, 16, 16), (3, 40, 72), (1, 128, 130), (2, 200, 24), (2, 18, 7)])
def test_lightning_kernels_token_by_token_and_by_chunks(dtype, heads, dim, vdim):
    """Both kernels against the recurrence in float64, three requests of 1, 45 and 100 tokens with states that
    do not start at zero, in slots that are not in order; the state after the step is compared as well."""
    from jax_vllm_amd.ops import kernels as K

    g = torch.Generator().manual_seed(dim + vdim)
    lens, slots = [1, 45, 100], [2, 0, 3]
    n = sum(lens)
    ld = 2 * heads * dim + heads * vdim + 5
    proj = (torch.randn(n, ld, generator=g) * 0.7).to(dtype)
    state0 = torch.randn(5, heads, dim, vdim, generator=g) * 0.5
    decay = torch.tensor([0.0, 0.93, 0.9999][:heads] if heads <= 3 else [0.9] * heads)
    act = torch.nn.functional.silu(proj.double())
    q = act[:, 5:5 + heads * dim].view(n, heads, dim)
    k = act[:, 5 + heads * dim:5 + 2 * heads * dim].view(n, heads, dim)
    v = act[:, 5 + 2 * heads * dim:].view(n, heads, vdim)
    want, want_state, t = torch.zeros(n, heads, vdim, dtype=torch.float64), state0.double().clone(), 0
    for ln, s in zip(lens, slots):
        for _ in range(ln):
            want_state[s] = decay.double()[:, None, None] * want_state[s] + k[t][:, :, None] * v[t][:, None, :]
            want[t] = torch.einsum("hde,hd->he", want_state[s], q[t])
            t += 1
    cu = torch.tensor([0, 1, 46, 146], dtype=torch.int32, device="cuda")
    for chunks in (False, True):
        if chunks and not K.lightning_chunks_possible(dim):
            continue
        state = state0.cuda().clone()
        out = K.lightning_attention(proj.cuda(), 5, 5 + heads * dim, 5 + 2 * heads * dim, state,
                                    torch.tensor(slots, dtype=torch.int32, device="cuda"), cu, decay.cuda(), heads, dim,
                                    vdim, K.lightning_chunk_plan(lens, "cuda") if chunks else None)
        scale = float(want.abs().max())
        assert float((out.cpu().double().view(n, heads, vdim) - want).abs().max()) <= 2e-5 * scale, f"chunks={chunks}"
        assert float((state.cpu().double() - want_state).abs().max()) <= 2e-5 * float(want_state.abs().max())
        assert torch.equal(state[1].cpu(), state0[1]) and torch.equal(state[4].cpu(), state0[4])    # other slots untouched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("n,experts,top,hidden,ff", [(1, 4, 1, 32, 24), (7, 5, 5, 40, 72), (300, 7, 3, 96, 136),
                                                     (130, 3, 2, 200, 88), (9, 6, 2, 36, 20)])
def test_routed_expert_kernels(dtype, n, experts, top, hidden, ff):
    """Choice, grouping and the grouped products against a loop over tokens in float64; 300 tokens over 7
    experts fill several row tiles per expert.  The router rows are made so that no choice is close."""
    from jax_vllm_amd.ops import kernels as K

    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, hidden, generator=g).to(dtype)
    wr = torch.randn(experts, hidden, generator=g).to(dtype)
    wg, wu = (torch.randn(experts, ff, hidden, generator=g) * hidden ** -0.5).to(dtype), (torch.randn(experts, ff, hidden, generator=g) * hidden ** -0.5).to(dtype)
    wd = (torch.randn(experts, hidden, ff, generator=g) * ff ** -0.5).to(dtype)
    z = x.double() @ wr.double().T
    srt = torch.sort(z, dim=-1, descending=True).values
    clear = torch.ones(n, dtype=torch.bool) if top == experts else (srt[:, top - 1] - srt[:, top]) > 1e-3
    logits = torch.empty(n, experts, dtype=torch.float32, device="cuda")
    tile_rows = 128 if (n >= 100 and K.moe_matrix_cores_possible(dtype, hidden, ff)) else None
    plan = K.moe_route(None, top, x=x.cuda(), w_router=wr.cuda(), logits_out=logits, tile_rows=tile_rows)
    assert float((logits.cpu().double() - z).abs().max()) <= 1e-5 * float(z.abs().max())
    ids = plan.ids.cpu().view(n, top).long()
    want_ids = torch.topk(z, top, dim=-1).indices
    assert torch.equal(torch.sort(ids[clear], dim=-1).values, torch.sort(want_ids[clear], dim=-1).values)
    order, offsets = plan.order.cpu().long(), plan.offsets.cpu().long()
    assert sorted(order.tolist()) == list(range(n * top)) and int(offsets[-1]) == n * top
    for e in range(experts):
        assert (plan.ids.cpu()[order[offsets[e]:offsets[e + 1]]] == e).all()
    again = K.moe_route(logits, top)                       # the choice from given logits is the same choice
    assert torch.equal(again.ids, plan.ids) and torch.equal(again.weights, plan.weights)
    forms = [None, False] if K.moe_matrix_cores_possible(dtype, hidden, ff) and not tile_rows else [None]     # matrix cores and float FMA
    for on_input, form in [(a, b) for a in (True, False) for b in forms]:
        out = torch.full((top, n, hidden), float("nan"), dtype=torch.float32, device="cuda")
        K.moe_experts(x.cuda(), plan, wg.cuda(), wu.cuda(), wd.cuda(), "silu", out, weight_on_input=on_input,
                      matrix_cores=form)
        want = torch.zeros(top, n, hidden, dtype=torch.float64)
        for t in range(n):
            for kk in range(top):
                e = int(ids[t, kk])
                s = torch.sigmoid(z[t, e])
                u = x[t].double() * (s if on_input else 1.0)
                y = wd[e].double() @ (torch.nn.functional.silu(wg[e].double() @ u) * (wu[e].double() @ u))
                want[kk, t] = y if on_input else y * s
        tol = 2e-5 if dtype == torch.float32 else 2e-2          # bfloat16: the rounding of the inner activations
        assert float((out.cpu().double() - want).abs().max()) <= tol * float(want.abs().max()), f"on_input={on_input} form={form}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_norm_of_a_sublayer_output_joined_to_the_stream(dtype):
    """h += norm(y + parts; wb), then norm(h; w): all rows, and chosen rows with h left alone."""
    from jax_vllm_amd.ops import kernels as K

    g = torch.Generator().manual_seed(0)
    n, hidden = 9, 100
    h0 = torch.randn(n, hidden, generator=g)
    y = torch.randn(n, hidden, generator=g).to(dtype)
    parts = torch.randn(3, n, hidden, generator=g)
    wb, w = 1 + 0.3 * torch.randn(hidden, generator=g), 1 + 0.3 * torch.randn(hidden, generator=g)

    def norm(v, weight, eps):
        return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight

    for use_y, use_parts in ((True, False), (False, True), (True, True)):
        v = (y.double() if use_y else 0) + (parts.double().sum(0) if use_parts else 0)
        want_h = h0.double() + norm(v, wb.double(), 1e-3)
        want = norm(want_h, w.double(), 1e-5)
        h = h0.cuda().clone()
        out = torch.empty(n, hidden, dtype=dtype, device="cuda")
        K.postnorm_add_rmsnorm(h, y.cuda() if use_y else None, parts.cuda() if use_parts else None, wb.cuda(), 1e-3,
                               w.cuda(), out, out_eps=1e-5)
        assert float((h.cpu().double() - want_h).abs().max()) <= 1e-5
        assert float((out.cpu().double() - want).abs().max()) <= (1e-5 if dtype == torch.float32 else 2e-2)
        rows = torch.tensor([7, 0, 3], dtype=torch.int32, device="cuda")
        h = h0.cuda().clone()
        out = torch.empty(3, hidden, dtype=dtype, device="cuda")
        K.postnorm_add_rmsnorm(h, y.cuda() if use_y else None, parts.cuda() if use_parts else None, wb.cuda(), 1e-3,
                               w.cuda(), out, rows, out_eps=1e-5)
        assert torch.equal(h.cpu(), h0)
        assert float((out.cpu().double() - want[[7, 0, 3]]).abs().max()) <= (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("n,heads,N,K", [(1, 3, 24, 16), (9, 2, 40, 72), (70, 5, 20, 24), (200, 2, 100, 136), (5, 4, 7, 10)])
def test_one_matrix_per_head(dtype, n, heads, N, K):
    """Every form of the per-head product (few rows, tiles, matrix cores) against float64, with heads that sit at
    strides wider than their sizes, with and without the sigmoid gate."""
    from jax_vllm_amd.ops import kernels as K_

    g = torch.Generator().manual_seed(n + N)
    xs, ys = K + 8, N + 3
    x = torch.randn(n, heads * xs, generator=g).to(dtype)
    w = (torch.randn(heads, N, K, generator=g) * K ** -0.5).to(dtype)
    gate = torch.randn(n, heads * N + 5, generator=g).to(dtype)
    want = torch.einsum("hnk,thk->thn", w.double(), x.double().view(n, heads, xs)[..., :K])
    forms = [None, False] if dtype == torch.bfloat16 and K % 8 == 0 else [None]
    for gated, form in [(a, b) for a in (False, True) for b in forms]:
        y = torch.zeros(n, heads * ys, dtype=dtype, device="cuda")
        gv = gate.cuda()[:, 5:] if gated else None
        K_.head_linear(y, ys, x.cuda(), xs, w.cuda(), gate=gv, matrix_cores=form)
        ref = want * torch.sigmoid(gate.double()[:, 5:].view(n, heads, N)) if gated else want
        got = y.cpu().double().view(n, heads, ys)
        tol = 1e-5 if dtype == torch.float32 else 1e-2
        assert float((got[..., :N] - ref).abs().max()) <= tol * max(1.0, float(ref.abs().max())), f"gated={gated} form={form}"
        assert float(got[..., N:].abs().max()) == 0.0           # nothing is written between the heads


@pytest.mark.parametrize("dtype", DTYPES)
def test_odd_width_and_a_cached_vector_above_256(tmp_path, dtype):
    """A width that is no multiple of 4 (no kernel may take its 16-byte path), a cached vector of 288 elements
    (beyond the matrix-core attention kernels: the float kernel runs in bfloat16 too), expert sizes that are no
    multiples of 8 (float-FMA expert products in bfloat16), under a lightning layer with a key size of 6."""
    small = dict(name="odd", seed=31, std=0.25, norm_std=0.2, config=config(50, 61, [
        layer(latent(2, 16, 32, 8, 256, 24, window=40), moe(3, 2, 20, 12)),
        layer(lightning(2, 6, 10, (0.8, 0.99)), moe(4, 1, 12)),
    ]))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 70, 8)
    want = expected(cfg, w, toks, dtype)
    core = make_core(folder, dtype, 16)
    check_rows(dtype, run_cut(core, "whole", toks, [70]), want, "whole")
    check_rows(dtype, run_cut(core, "cut", toks, [33, 2, 1, 17, 1, 1, 15]), want, "portions")


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys_without_a_window(tmp_path, dtype):
    """Latent attention over every earlier key, scores sharp enough that one key among hundreds carries a row, as
    often as not a far one: rows beyond position 200 change by much when the plain implementation is kept from
    seeing keys more than 150 back.  300 tokens over 19 pages: whole, in portions that end at and around page
    borders, and with the last 40 decoded one by one."""
    mixer = dict(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, q_rank=24, scale=1.0)
    small = dict(name="far", seed=23, std=0.3, norm_std=0.1, config=config(32, 50, [layer(latent(window=None, **mixer))]))
    folder = make_folder(small, tmp_path)
    cfg, w = plain_of(folder)
    toks = tokens_of(cfg, 300, 12)
    want = expected(cfg, w, toks, dtype)
    plain = plain_logits(cfg, w, toks)
    near = plain_logits(config(32, 50, [layer(latent(window=150, **mixer))]), w, toks)
    assert np.median(np.abs(near[200:] - plain[200:]).max(axis=-1)) > 0.01 * np.abs(plain).max()
    core = make_core(folder, dtype, 16, pages=20)
    check_rows(dtype, run_cut(core, "whole", toks, [300]), want, "whole")
    check_rows(dtype, run_cut(core, "portions", toks, [64, 63, 1, 17, 47, 2, 66] + [1] * 40), want, "portions and decoding")
