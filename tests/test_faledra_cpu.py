"""Faledra without a GPU: the plain implementation's mechanisms pinned on small
cases worked out by hand, the typed configuration, the model's structure (tensor
names, running order, cache buffers and states) and the random-weights folder."""
import json
import math
import os

import pytest
import torch

from faledra_util import CONFIGS, config, gru, latent, write_model
from plain import faledra_plain as FP


# ------------------------------------------------------------- plain mechanisms
def test_rms_norm_has_eps_under_the_root():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    got = FP.rms_norm(x, torch.tensor([2.0, 0.5], dtype=torch.float64), 0.5)
    want = x / math.sqrt(12.5 + 0.5) * torch.tensor([2.0, 0.5])
    assert torch.allclose(got, want, atol=1e-15)


def test_short_conv_taps_and_start():
    h = torch.tensor([[1.0], [10.0], [100.0], [1000.0]], dtype=torch.float64)
    w = torch.tensor([[2.0, 3.0, 5.0]], dtype=torch.float64)          # the last tap is the token itself
    out = FP.short_conv(h, w)
    assert out[:, 0].tolist() == [5.0, 3.0 + 50.0, 2.0 + 30.0 + 500.0, 20.0 + 300.0 + 5000.0]
    one = FP.short_conv(h, torch.tensor([[7.0]], dtype=torch.float64))
    assert one[:, 0].tolist() == [7.0, 70.0, 700.0, 7000.0]


def test_xielu_branches_and_continuity():
    p, q = torch.tensor(0.3, dtype=torch.float64), torch.tensor(-0.7, dtype=torch.float64)
    sp = lambda v: math.log1p(math.exp(v))
    z = torch.tensor([2.0, -1.5, 0.0], dtype=torch.float64)
    got = FP.xielu(z, p, q)
    assert got[0].item() == pytest.approx(sp(0.3) * 4.0 + 1.0)
    assert got[1].item() == pytest.approx((0.5 + sp(-0.7)) * (math.exp(-1.5) - 1.0 + 1.5) - 0.75)
    assert got[2].item() == 0.0
    eps = torch.tensor([1e-9, -1e-9], dtype=torch.float64)
    lo = FP.xielu(eps, p, q)
    assert abs(lo[0].item() - lo[1].item()) < 2e-9                    # value and slope 1/2 on both sides of 0


def test_gelu_tanh_formula():
    z = torch.tensor([0.7], dtype=torch.float64)
    want = 0.5 * 0.7 * (1 + math.tanh(math.sqrt(2 / math.pi) * (0.7 + 0.044715 * 0.7 ** 3)))
    assert FP.gelu_tanh(z).item() == pytest.approx(want)


def test_rotation_turns_neighbouring_pairs_and_leaves_the_rest():
    v = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 9.0, 8.0]]], dtype=torch.float64).repeat(3, 1, 1)
    out = FP.rotate_pairs(v, torch.tensor([0, 1, 5]), base=100.0, dims=4)
    assert torch.equal(out[0], v[0])                                   # position 0: no turn
    a0, a1 = 1.0, 100.0 ** (-2.0 / 4)                                  # f_0 = 1, f_1 = base^(-2/dims)
    assert out[1, 0, 0].item() == pytest.approx(math.cos(a0)) and out[1, 0, 1].item() == pytest.approx(math.sin(a0))
    assert out[1, 0, 2].item() == pytest.approx(-2.0 * math.sin(a1)) and out[1, 0, 3].item() == pytest.approx(2.0 * math.cos(a1))
    assert out[2, 0, 2].item() == pytest.approx(-2.0 * math.sin(5 * a1))
    assert out[:, 0, 4:].tolist() == [[9.0, 8.0]] * 3                  # beyond dims: unchanged
    # the score of a rotated query and key depends on the distance alone
    q = torch.randn(1, 1, 4, dtype=torch.float64)
    k = torch.randn(1, 1, 4, dtype=torch.float64)
    s = lambda i, j: (FP.rotate_pairs(q, torch.tensor([i]), 50.0, 4) * FP.rotate_pairs(k, torch.tensor([j]), 50.0, 4)).sum()
    assert s(7, 3).item() == pytest.approx(s(104, 100).item())


def test_sink_counts_once_without_value_or_scale():
    q = torch.zeros(2, 1, 2, dtype=torch.float64)                      # all scores 0
    k = torch.zeros(2, 1, 2, dtype=torch.float64)
    v = torch.tensor([[[1.0]], [[3.0]]], dtype=torch.float64)
    out = FP.sink_softmax_attention(q, k, v, torch.tensor([math.log(2.0)], dtype=torch.float64), scale=5.0)
    assert out[0, 0, 0].item() == pytest.approx(1.0 / (1.0 + 2.0))     # one key of weight 1, sink of weight 2
    assert out[1, 0, 0].item() == pytest.approx((1.0 + 3.0) / (2.0 + 2.0))
    far = FP.sink_softmax_attention(q, k, v, torch.tensor([-1e9], dtype=torch.float64), scale=5.0)
    assert far[1, 0, 0].item() == pytest.approx(2.0)                   # no sink: the plain causal mean


def test_mingru_recurrence_by_hand():
    w = {"z": torch.tensor([[1.0]]), "z.b": torch.tensor([0.0]), "x": torch.tensor([[1.0]]), "x.b": torch.tensor([0.5]),
         "g": torch.tensor([[1.0]]), "o": torch.tensor([[2.0]])}
    w = {k: v.double() for k, v in w.items()}
    h = torch.tensor([[1.0], [-2.0]], dtype=torch.float64)
    sig = lambda a: 1 / (1 + math.exp(-a))
    z1, c1 = sig(1.0), 1.5 + 0.5                                       # u = 1.5 >= 0: u + 1/2
    s1 = z1 * c1
    z2, c2 = sig(-2.0), sig(-1.5)                                      # u = -1.5 < 0: sigmoid(u)
    s2 = (1 - z2) * s1 + z2 * c2
    out = FP.mingru(h, w)
    assert out[0, 0].item() == pytest.approx(2.0 * s1 * (1.0 * sig(1.0)))
    assert out[1, 0].item() == pytest.approx(2.0 * s2 * (-2.0 * sig(-2.0)))


def test_layer_order_of_a_loop():
    assert FP.layer_order(3, None) == [(0, None, False), (1, None, False), (2, None, False)]
    got = FP.layer_order(5, dict(start=1, stop=3, times=2))
    assert [(i, t) for i, t, _ in got] == [(0, None), (1, 0), (2, 0), (1, 1), (2, 1), (3, None), (4, None)]
    assert [first for _, _, first in got] == [False, True, False, True, False, False, False]


# ------------------------------------------------------------------ configuration
def test_config_round_trip_and_errors():
    from lyapunov_engine_amd.config import ConfigError, FaledraConfig
    from lyapunov_engine_amd.config.registry import architecture_of

    for name, raw in CONFIGS.items():
        assert architecture_of(raw).name == "Faledra"
        cfg = FaledraConfig.from_dict(raw)
        assert FaledraConfig.from_dict(cfg.to_dict()) == cfg
        assert cfg.vocab == raw["vocab"] and cfg.width == raw["width"] and len(cfg.layers) == len(raw["layers"])
    with pytest.raises(ConfigError, match="lacks"):
        FaledraConfig.from_dict({k: v for k, v in CONFIGS["A"].items() if k != "residual_mult"})
    bad = json.loads(json.dumps(CONFIGS["A"]))
    bad["layers"][1]["mixer"].pop("kv_rank")
    with pytest.raises(ConfigError, match="kv_rank"):
        FaledraConfig.from_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["A"]))
    bad["layers"][0]["type"] = "something_else"
    with pytest.raises(ConfigError, match="not implemented"):
        FaledraConfig.from_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["A"]))
    bad["loop"]["stop"] = 9
    with pytest.raises(ConfigError, match="loop"):
        FaledraConfig.from_dict(bad)


def test_structure_of_the_built_model():
    from lyapunov_engine_amd.config import FaledraConfig
    from lyapunov_engine_amd.models.decoder import build_model
    from lyapunov_engine_amd.models.faledra import faledra_spec

    model = build_model(faledra_spec(FaledraConfig.from_dict(CONFIGS["A"])))
    names = model.expected_tensors()
    assert names["embed"][0] == (203, 72) and names["head"][0] == (203, 72) and names["final.norm"][0] == (72,)
    assert names["loop.step"][0] == (3, 72)
    assert names["l1.mix.dkv"][0] == (40 + 8, 72) and names["l1.mix.uq"][0] == (3 * 32, 36)
    assert names["l1.mix.uk"][0] == (3 * 24, 40) and names["l1.mix.uv"][0] == (3 * 20, 40) and names["l1.mix.o"][0] == (72, 60)
    assert names["l0.mix.z.b"][0] == (40,) and names["l0.canon1"][0] == (72, 4) and names["l0.mlp.act"][0] == (2,)
    assert "l2.norm2" not in names and "l2.mlp.up" not in names            # a layer without feed-forward
    assert model.ignorable("l2.norm2b") and not model.ignorable("l1.norm2b")
    # layers 1 and 2 run three times: 1 + 3 * 2 + 1 calls, a cache buffer each, the pass's vector at its first layer
    sched = model.schedule
    assert [c.layer for c in sched] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [c.cache for c in sched] == list(range(8))
    assert [c.shift for c in sched] == [None, 0, None, 1, None, 2, None, None]
    layout = model.cache_layout()
    assert len(layout.groups) == 2                                        # two shapes of latent: two pools
    assert sorted(layout.states) == [0, 7]                                # the recurrences' states
    assert sorted(k[0] for k in layout.part_states) == list(range(8))     # a filter's memory for every call
    assert all(s.shape == (3, 72) for s in layout.part_states.values())
    # one tap: a filter without memory; no loop: no shift
    model = build_model(faledra_spec(FaledraConfig.from_dict(CONFIGS["B"])))
    assert model.cache_layout().part_states == {} and model.stream_shift is None
    assert "loop.step" not in model.expected_tensors() and model.expected_tensors()["l0.canon1"][0] == (64, 1)


def test_model_folder_is_read_back_tensor_by_tensor(tmp_path):
    from lyapunov_engine_amd.weights.loader import FolderSource, WeightError, check_tensors
    from lyapunov_engine_amd.config.registry import load_config
    from lyapunov_engine_amd.models.decoder import build_model

    folder = write_model(str(tmp_path / "m"), CONFIGS["C"], seed=1, dtype="bfloat16")
    arch, cfg = load_config(folder)
    model = build_model(arch.to_spec(cfg))
    check_tensors(model, FolderSource(folder).shapes())
    cfg2, tensors = FP.load_folder(folder)
    assert set(tensors) == set(model.expected_tensors())
    shapes = dict(FolderSource(folder).shapes())
    shapes.pop("l0.mix.sink")
    shapes["l1.mix.z"] = (5, 5)
    with pytest.raises(WeightError) as e:
        check_tensors(model, shapes)
    assert "l0.mix.sink" in str(e.value) and "l1.mix.z" in str(e.value)


def test_random_weights_mode_writes_a_faledra_folder(tmp_path):
    from lyapunov_engine_amd.weights import write_random_model

    folder = write_random_model(dict(CONFIGS["B"]), str(tmp_path / "r"), seed=3, dtype="float32")
    cfg, tensors = FP.load_folder(folder)
    assert cfg["architecture"] == "Faledra" and tensors["l1.mix.uv"].shape == (48, 48)
    logits = FP.forward([1, 2, 3], tensors, cfg)
    assert logits.shape == (3, 150) and torch.isfinite(logits).all()
