"""Dumazen on the host: its configuration reader, the tensors its ``ModelSpec`` asks for, a random model folder
written and read back, the memory plan (pages for the window attention, several state tensors for the recurrent
mixers), the frequency rule of its rotation, and the plain implementation's own consistency."""
import copy

import pytest
import torch

from tests.dumazen_util import ALL_SMALL, SMALL_A, SMALL_B, WAVES, config, layer, mamba2, retention, rot
from tests.plain import dumazen_plain as P


def spec_of(cfg_dict):
    from jax_vllm_amd.config.registry import resolve
    from jax_vllm_amd.parts.model import DecoderModel

    arch, cfg, _ = resolve(cfg_dict)
    return arch, cfg, DecoderModel(arch.build_spec(cfg))


def expected_tensors(c):
    """Names and shapes from the configuration alone, written out independently of the product."""
    w = c["width"]
    out = {"embed": (c["vocab"], w), "final.norm": (w,)}
    for i, l in enumerate(c["layers"]):
        p, m = f"l{i}.", l["mixer"]
        out[p + "norm1"] = (w,)
        if l["type"] == "retention":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * d, w), p + "mix.k": (H * d, w), p + "mix.v": (H * dv, w), p + "mix.g": (H * dv, w),
                        p + "mix.o": (w, H * dv)})
        elif l["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            out.update({p + "mix.in": (2 * inner + 2 * gn + m["heads"], w), p + "mix.conv": (inner + 2 * gn, m["conv"]),
                        p + "mix.conv.b": (inner + 2 * gn,), p + "mix.dt_bias": (m["heads"],), p + "mix.A_log": (m["heads"],),
                        p + "mix.D": (m["heads"],), p + "mix.norm": (inner,), p + "mix.o": (w, inner)})
        else:
            a, b = m["left"], m["right"]
            q = p + "mix.left."
            out.update({q + "q": (a["heads"] * a["dim"], w), q + "q.b": (a["heads"] * a["dim"],),
                        q + "k": (a["kv_heads"] * a["dim"], w), q + "k.b": (a["kv_heads"] * a["dim"],),
                        q + "v": (a["kv_heads"] * a["vdim"], w), q + "v.b": (a["kv_heads"] * a["vdim"],),
                        q + "q.norm": (a["heads"] * a["dim"],), q + "k.norm": (a["kv_heads"] * a["dim"],),
                        q + "o": (w, a["heads"] * a["vdim"])})
            q = p + "mix.right."
            qk, inner = b["kv_heads"] * b["dim"], b["heads"] * b["vdim"]
            out.update({q + "q": (qk, w), q + "k": (qk, w), q + "v": (inner, w), q + "q.conv": (qk, b["conv"]),
                        q + "k.conv": (qk, b["conv"]), q + "v.conv": (inner, b["conv"]), q + "b": (b["heads"], w),
                        q + "a": (b["heads"], w), q + "A_log": (b["heads"],), q + "dt_bias": (b["heads"],),
                        q + "norm": (b["vdim"],), q + "g": (inner, w), q + "o": (w, inner)})
        f = l.get("mlp")
        if f:
            out[p + "norm2"] = (w,)
            out.update({p + "mlp.up": (f["ff"], w), p + "mlp.up.b": (f["ff"],), p + "mlp.down": (w, f["ff"]),
                        p + "mlp.down.b": (w,)})
    return out


@pytest.mark.parametrize("small", ALL_SMALL, ids=[s["name"] for s in ALL_SMALL])
def test_tensors_and_memory_plan_follow_the_configuration(small):
    from jax_vllm_amd.parts.spec import state_specs_of

    _, cfg, model = spec_of(small["config"])
    got = {k: tuple(v.shape) for k, v in model.tensor_specs().items()}
    assert got == expected_tensors(small["config"])
    assert model.spec.tie_head_to_embedding
    for run, l in zip(model.memory_plan(), small["config"]["layers"]):
        m = l["mixer"]
        states = {s.name: s for s in state_specs_of(run.state)}
        assert all(s.dtype == "float32" for s in states.values())
        if l["type"] == "retention":
            assert run.cache is None and {k: v.shape for k, v in states.items()} == {"S": (m["heads"], m["dim"], m["vdim"])}
        elif l["type"] == "mamba2":
            channels = m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]
            assert run.cache is None
            assert {k: v.shape for k, v in states.items()} == {"S": (m["heads"], m["state"], m["vdim"]), "conv": (m["conv"] - 1, channels)}
        else:
            a, b = m["left"], m["right"]
            assert run.cache.window == (a.get("mask") or {}).get("size")
            padded = -(-max(a["dim"], a["vdim"]) // 16) * 16
            assert [t.token_shape for t in run.cache.tensors] == [(a["kv_heads"], padded)] * 2
            channels = 2 * b["kv_heads"] * b["dim"] + b["heads"] * b["vdim"]
            assert {k: v.shape for k, v in states.items()} == {"right.S": (b["heads"], b["dim"], b["vdim"]),
                                                               "right.conv": (b["conv"] - 1, channels)}
    assert model.replayable()


def test_configuration_errors_name_the_place():
    from jax_vllm_amd.config.errors import ConfigError
    from jax_vllm_amd.config.registry import resolve

    def broken(change):
        c = copy.deepcopy(SMALL_A["config"])
        change(c)
        with pytest.raises(ConfigError) as e:
            resolve(c)
        return str(e.value)

    assert "layers[0].mixer.decay" in broken(lambda c: c["layers"][0]["mixer"]["decay"].pop())
    assert "layers[1].mixer" in broken(lambda c: c["layers"][1]["mixer"].update(groups=3))
    assert "norm groups" in broken(lambda c: c["layers"][1]["mixer"].update(norm_groups=5))
    assert "layers[2].mixer.left" in broken(lambda c: c["layers"][2]["mixer"]["left"].update(kv_heads=3))
    assert "layers[2].mixer.left.rot.dims" in broken(lambda c: c["layers"][2]["mixer"]["left"]["rot"].update(dims=14))
    assert "layers[2].mixer.right" in broken(lambda c: c["layers"][2]["mixer"]["right"].update(kv_heads=3))
    assert "residual_mult" in broken(lambda c: c.pop("residual_mult"))
    assert "layers[3].type" in broken(lambda c: c["layers"][3].update(type="attention"))
    assert "layers[0].mlp.kind" in broken(lambda c: c["layers"][0]["mlp"].update(kind="moe"))


def test_random_folder_is_read_back_and_its_norm_weights_lie_around_zero(tmp_path):
    from jax_vllm_amd import write_random_model
    from jax_vllm_amd.weights.safetensors_io import open_shards

    folder = write_random_model(tmp_path, SMALL_B["config"], seed=1, std=0.1, norm_std=0.05)
    w = P.read_weights(folder)
    assert {k: tuple(v.shape) for k, v in w.items()} == expected_tensors(SMALL_B["config"])
    assert abs(float(w["l1.norm1"].mean())) < 0.05 and abs(float(w["final.norm"].mean())) < 0.05      # 1 + weight multiplies
    assert float(w["l2.mix.A_log"].mean()) < -1.0                                                          # slow decays
    shard = next(iter(open_shards(folder)))
    assert set(shard.entries) == set(w)
    shard.close()


def test_frequencies_of_the_rotation_part_follow_the_wavelength_rule():
    from jax_vllm_amd.parts.rotary import RotaryEncoding

    for dims, base, sc in ((8, 500.0, WAVES), (32, 1e6, dict(WAVES, factor=1.5)), (48, 250000.0, dict(WAVES, original=2048, factor=8.0)),
                           (6, 100.0, None)):
        part = RotaryEncoding(dims + 4, base, dims, by_wavelength=sc)
        want = P.rotary_frequencies(rot(dims, base, sc))
        got = part.inverse_frequencies().double()
        assert got.shape == (dims // 2,) and float(((got - want) / want).abs().max()) < 3e-7
    # all three branches occur in the first case: kept, slowed down, blended
    f = 500.0 ** (-2.0 * torch.arange(4, dtype=torch.float64) / 8)
    ratio = P.rotary_frequencies(rot(8, 500.0, WAVES)) / f
    assert float(ratio[0]) == 1.0 and abs(float(ratio[-1]) - 0.25) < 1e-12 and any(0.26 < float(r) < 0.99 for r in ratio)


def test_plain_mixers_do_not_look_ahead_and_carry_their_state():
    """The oracle's own sanity: logits at a position do not change when tokens are appended, and a retention head with
    decay 0 sees the current token only."""
    small = dict(SMALL_A, config=config(24, 40, [layer(retention(2, 4, 6, (0.0, 1.0), rot(4))), layer(mamba2(2, 4, 6, conv=3), 16)]))
    torch.manual_seed(0)
    _, _, model = spec_of(small["config"])
    w = {k: torch.randn(v.shape, dtype=torch.float64) * 0.3 for k, v in model.tensor_specs().items()}
    toks = list(range(1, 20))
    full = P.forward(w, small["config"], toks)
    assert torch.allclose(P.forward(w, small["config"], toks[:11]), full[:11], atol=1e-12)
    m = small["config"]["layers"][0]["mixer"]
    h = torch.randn(5, 24, dtype=torch.float64)
    one = dict(m, heads=1, decay=[0.0])
    w1 = {"q": w["l0.mix.q"][:4], "k": w["l0.mix.k"][:4], "v": w["l0.mix.v"][:6], "g": w["l0.mix.g"][:6], "o": w["l0.mix.o"][:, :6]}
    a = P.retention(w1, "", one, h, 1e-5)
    b = torch.cat([P.retention(w1, "", one, h[i:i + 1], 1e-5) for i in range(5)])
    # with decay 0 only the rotation's relative angle (zero for a token and itself) is left of the position
    assert torch.allclose(a, b, atol=1e-10)
