"""Lomozen on the host: its configuration reader, the tensors its ``ModelSpec`` asks for, a random model
folder written and read back, the memory plan (pages for latent attention, state for lightning), and the
two identities of the plain implementation that the kernels rely on."""
import copy
import math

import pytest
import torch

from tests.lomozen_util import ALL_SMALL, SMALL_A, SMALL_B, YARN, config, latent, layer, lightning, moe
from tests.plain import lomozen_plain as P


def spec_of(cfg_dict):
    from jax_vllm_amd.config.registry import resolve
    from jax_vllm_amd.parts.model import DecoderModel

    arch, cfg, _ = resolve(cfg_dict)
    return arch, cfg, DecoderModel(arch.build_spec(cfg))


def expected_tensors(c):
    """Names and shapes from the configuration alone, written out independently of the product."""
    w = c["width"]
    out = {"embed": (c["vocab"], w), "head": (c["vocab"], w), "final.norm": (w,)}
    for i, l in enumerate(c["layers"]):
        p, m = f"l{i}.", l["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (w,)
        if l["type"] == "lightning":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * d, w), p + "mix.k": (H * d, w), p + "mix.v": (H * dv, w), p + "mix.g": (H * dv, w),
                        p + "mix.o": (w, H * dv), p + "mix.norm": (H * dv,)})
        else:
            H, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            out.update({p + "mix.dq": (m["q_rank"], w), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (H * (d + r), m["q_rank"]),
                        p + "mix.dkv": (m["kv_rank"] + r, w), p + "mix.dkv.norm": (m["kv_rank"],),
                        p + "mix.uk": (H * d, m["kv_rank"]), p + "mix.uv": (H * dv, m["kv_rank"]),
                        p + "mix.g": (H * dv, w), p + "mix.o": (w, H * dv)})
        f = l.get("mlp")
        if f:
            out[p + "norm2"] = out[p + "norm2b"] = (w,)
            out[p + "mlp.router"] = (f["router"]["experts"], w)
            names = [f"e{e}" for e in range(f["router"]["experts"])] + (["shared"] if f.get("shared") else [])
            for nme in names:
                ff = f["shared"]["ff"] if nme == "shared" else f["expert"]["ff"]
                out.update({f"{p}mlp.{nme}.gate": (ff, w), f"{p}mlp.{nme}.up": (ff, w), f"{p}mlp.{nme}.down": (w, ff)})
    return out


@pytest.mark.parametrize("small", ALL_SMALL, ids=[s["name"] for s in ALL_SMALL])
def test_tensors_and_memory_plan_follow_the_configuration(small):
    _, cfg, model = spec_of(small["config"])
    got = {k: tuple(v.shape) for k, v in model.tensor_specs().items()}
    assert got == expected_tensors(small["config"])
    assert all(v.role == "vector" for k, v in model.tensor_specs().items() if "norm" in k)
    for run, l in zip(model.memory_plan(), small["config"]["layers"]):
        m = l["mixer"]
        if l["type"] == "lightning":
            assert run.cache is None and run.state.shape == (m["heads"], m["dim"], m["vdim"]) and run.state.dtype == "float32"
        else:
            assert run.state is None and run.cache.window == (m.get("mask") or {}).get("size")
            assert [t.token_shape for t in run.cache.tensors] == [(1, m["kv_rank"] + m["rot_dim"])] * 2


def test_bad_configurations_are_refused_with_the_key_named():
    from jax_vllm_amd.config import ConfigError

    good = SMALL_A["config"]
    spec_of(good)

    def broken(path, value):
        c = copy.deepcopy(good)
        at = c
        for k in path[:-1]:
            at = at[k]
        if value is KeyError:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        return c

    cases = [
        (("vocab",), 0, "vocab"), (("width",), KeyError, "width"), (("norm",), KeyError, "norm"),
        (("layers",), [], "layers"), (("layers", 0, "type"), "conv", "type"),
        (("layers", 0, "mixer", "decay"), [0.5], "decay"), (("layers", 0, "mixer", "decay"), [0.5, 0.5, 1.5], "decay"),
        (("layers", 1, "mixer", "kv_rank"), KeyError, "kv_rank"), (("layers", 1, "mixer", "rot", "dims"), 10, "dims"),
        (("layers", 1, "mixer", "rot", "dims"), 3, "dims"), (("layers", 1, "mixer", "scale"), 0.0, "scale"),
        (("layers", 1, "mixer", "mask", "size"), -4, "size"), (("layers", 1, "mixer", "rot", "scaling", "factor"), KeyError, "factor"),
        (("layers", 0, "mlp", "router", "top"), 7, "top"), (("layers", 0, "mlp", "kind"), "dense", "kind"),
        (("layers", 0, "mlp", "expert"), KeyError, "expert"),
    ]
    for path, value, word in cases:
        with pytest.raises(ConfigError, match=word):
            spec_of(broken(path, value))
    with pytest.raises(ConfigError, match="unsupported architecture"):
        spec_of(dict(good, architecture="Nobody"))


def test_random_model_folder_round_trip(tmp_path):
    """``write_random_model`` writes what the plain reader and the loader's shape check both accept."""
    from jax_vllm_amd import write_random_model
    from jax_vllm_amd.weights.loader import check_against_specs
    from jax_vllm_amd.weights.safetensors_io import open_shards

    folder = write_random_model(tmp_path, SMALL_B["config"], seed=1, std=0.1, norm_std=0.1)
    cfg, w = P.read_config(folder), P.read_weights(folder)
    assert {k: tuple(v.shape) for k, v in w.items()} == expected_tensors(SMALL_B["config"])
    assert abs(float(w["l0.norm1"].mean()) - 1.0) < 0.2 and abs(float(w["l0.mix.dq"].mean())) < 0.05
    logits = P.forward(w, cfg, [1, 2, 3, 4])
    assert logits.shape == (4, SMALL_B["config"]["vocab"]) and torch.isfinite(logits).all()
    _, _, model = spec_of(SMALL_B["config"])
    shard = next(iter(open_shards(folder)))
    assert check_against_specs(folder, model.tensor_specs(), set(), shard.entries) == []


def test_rescaled_frequencies_of_the_rotary_part_equal_the_plain_ones():
    from jax_vllm_amd.parts.rotary import RotaryEncoding

    for dims, base, sc in ((8, 10000.0, YARN), (16, 500000.0, dict(YARN, factor=2.0, original=2048, fast=32.0)), (6, 100.0, None)):
        part = RotaryEncoding(head_dim=dims + 2, theta=base, rotary_dim=dims, rescale=sc)
        f, amp = P.rotary_frequencies({"dims": dims, "base": base, "scaling": sc})
        assert torch.allclose(part.inverse_frequencies().double(), f, rtol=1e-6, atol=0)
        assert part.amplitude == pytest.approx(amp)
        if sc:     # the fastest pair keeps its frequency, the slowest is slowed down by the factor
            plain = base ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)
            assert f[0] == plain[0] and float(f[-1]) == pytest.approx(float(plain[-1]) / sc["factor"])


def test_latent_attention_equals_attention_over_the_cached_vector():
    """What the product computes (one shared key/value vector [c | k_rot] per token, queries W_uk^T q, values
    through W_uv afterwards) is the plain formula (per-head keys and values made from c)."""
    torch.manual_seed(0)
    m = latent(3, 8, 4, 6, 10, 12, window=5, scale=0.9, scaling=YARN)["mixer"]
    H, d, r, dv, kr, n, w_ = 3, 8, 4, 6, 10, 17, 20
    w = {"dq": torch.randn(12, w_), "dq.norm": torch.rand(12) + 0.5, "uq": torch.randn(H * (d + r), 12), "dkv": torch.randn(kr + r, w_),
         "dkv.norm": torch.rand(kr) + 0.5, "uk": torch.randn(H * d, kr), "uv": torch.randn(H * dv, kr), "g": torch.randn(H * dv, w_),
         "o": torch.randn(w_, H * dv)}
    w = {"x." + k: v.double() for k, v in w.items()}
    h = torch.randn(n, w_).double()
    want = P.latent_attention(w, "x.", m, h, 1e-5)
    pos = torch.arange(n)
    cq = P.rms_norm(h @ w["x.dq"].T, w["x.dq.norm"], 1e-5)
    q = (cq @ w["x.uq"].T).view(n, H, d + r)
    dkv = h @ w["x.dkv"].T
    e = torch.cat([P.rms_norm(dkv[:, :kr], w["x.dkv.norm"], 1e-5), P.rotate(dkv[:, kr:], pos, m["rot"])], dim=-1)     # cached
    qe = torch.cat([torch.einsum("hdk,nhd->nhk", w["x.uk"].view(H, d, kr), q[..., :d]),
                    P.rotate(q[..., d:].transpose(0, 1), pos, m["rot"]).transpose(0, 1)], dim=-1)
    s = torch.einsum("nhe,je->hnj", qe, e) * m["scale"]
    i, j = pos[:, None], pos[None, :]
    s = s.masked_fill(~((j <= i) & (i - j < 5)), float("-inf"))
    o = torch.einsum("hnj,je->nhe", torch.softmax(s, -1), e)[..., :kr]
    o = torch.einsum("hvk,nhk->nhv", w["x.uv"].view(H, dv, kr), o).reshape(n, H * dv)
    got = (o * torch.sigmoid(h @ w["x.g"].T)) @ w["x.o"].T
    assert torch.allclose(got, want, rtol=1e-9, atol=1e-9)


def test_lightning_by_chunks_equals_the_recurrence():
    """The chunked form of the kernel for prompts: within a chunk of n tokens after state S,
    o_i = decay^(i+1) S^T q_i + sum_{j<=i} decay^(i-j) (q_i . k_j) v_j and S' = decay^n S + sum_j decay^(n-1-j) k_j v_j^T."""
    torch.manual_seed(1)
    n, d, dv, lam = 23, 5, 7, 0.8
    q, k, v = torch.randn(n, d).double(), torch.randn(n, d).double(), torch.randn(n, dv).double()
    S = torch.randn(d, dv).double()
    want, T = [], S.clone()
    for t in range(n):
        T = lam * T + k[t][:, None] * v[t][None, :]
        want.append(T.T @ q[t])
    got, U = [], S.clone()
    for b0 in range(0, n, 8):
        m = min(8, n - b0)
        qq, kk, vv = q[b0:b0 + m], k[b0:b0 + m], v[b0:b0 + m]
        for i in range(m):
            o = lam ** (i + 1) * (U.T @ qq[i])
            for j in range(i + 1):
                o = o + lam ** (i - j) * (qq[i] @ kk[j]) * vv[j]
            got.append(o)
        U = lam ** m * U + sum(lam ** (m - 1 - j) * kk[j][:, None] * vv[j][None, :] for j in range(m))
    assert torch.allclose(torch.stack(got), torch.stack(want), rtol=1e-10, atol=1e-10) and torch.allclose(U, T, rtol=1e-10, atol=1e-10)


def test_state_only_model_needs_no_pages():
    """A model of lightning layers alone has no page group at all: the cache manager hands out slots only."""
    from jax_vllm_amd.cache.manager import CacheManager
    from jax_vllm_amd.cache.storage import group_keys_of, has_state

    _, _, model = spec_of(config(32, 40, [layer(lightning(2, 8, 8, (0.5, 0.9)), moe(3, 1, 16)), layer(lightning(1, 8, 8, (1.0,)))]))
    plan = model.memory_plan()
    assert group_keys_of(plan) == [] and has_state(plan)
    cm = CacheManager([], 16, 8, 2, True, True)
    assert not cm.prefix_cache
    cm.start("a")
    cm.reserve("a", 100)
    assert cm.groups == [] and cm.pages_needed("a", 1000) == []
    cm.commit("a", list(range(100)))
    assert cm.context_len("a") == 100
    cm.finish("a")
    cm.check_invariants()
