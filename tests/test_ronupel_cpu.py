"""Ronupel without a GPU: the plain implementation's mechanisms pinned on small
cases worked out by hand, the typed configuration, the model's structure (tensor
names, running order, cache buffers and groups), the cache manager's kept first
pages and the position table with divided frequencies."""
import math

import pytest
import torch

from plain import ronupel_plain as RP
from ronupel_util import CONFIGS, attn, config, moe, write_model

F64 = torch.float64


# ------------------------------------------------------------- plain mechanisms
def test_rms_norm_has_eps_under_the_root():
    x = torch.tensor([[3.0, 4.0]], dtype=F64)
    got = RP.rms_norm(x, torch.tensor([2.0, 0.5], dtype=F64), 0.5)
    assert torch.allclose(got, x / math.sqrt(12.5 + 0.5) * torch.tensor([2.0, 0.5]), atol=1e-15)


def test_who_sees_whom():
    pos = torch.arange(12)
    m = RP.visible(pos, pos, size=3, keep_first=2)
    assert m[0].tolist() == [True] + [False] * 11
    # position 7: itself and the two before it, and the sequence's first two
    assert [j for j in range(12) if m[7, j]] == [0, 1, 5, 6, 7]
    assert [j for j in range(12) if m[3, j]] == [0, 1, 2, 3]            # the window and the kept tokens overlap
    assert [j for j in range(12) if RP.visible(pos, pos, 3, 0)[7, j]] == [5, 6, 7]
    assert [j for j in range(12) if RP.visible(pos, pos, 1, 0)[7, j]] == [7]
    assert not RP.visible(pos, pos, 100, 100).triu(1).any()               # never the future


def test_sink_counts_once_without_value_or_scale():
    scores = torch.zeros(1, 3, dtype=F64)
    mask = torch.tensor([[True, True, False]])
    p = RP.sink_softmax(scores, mask, torch.tensor(0.0, dtype=F64))
    assert p[0].tolist() == pytest.approx([1 / 3, 1 / 3, 0.0])           # two keys and the sink share the weight
    p = RP.sink_softmax(scores, mask, torch.tensor(math.log(2.0), dtype=F64))
    assert p[0].tolist() == pytest.approx([0.25, 0.25, 0.0])
    p = RP.sink_softmax(scores + 500.0, mask, torch.tensor(-1e9, dtype=F64))
    assert p[0].tolist() == pytest.approx([0.5, 0.5, 0.0])


def test_rotation_turns_neighbouring_pairs_slowly_and_leaves_the_rest():
    v = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 9.0, 8.0]]], dtype=F64).repeat(3, 1, 1)
    out = RP.rotate_neighbours(v, torch.tensor([0, 1, 6]), base=100.0, dims=4, factor=2.0)
    assert torch.equal(out[0], v[0])
    a0, a1 = 1.0 / 2.0, 100.0 ** (-2.0 / 4) / 2.0
    assert out[1, 0, 0].item() == pytest.approx(math.cos(a0)) and out[1, 0, 1].item() == pytest.approx(math.sin(a0))
    assert out[1, 0, 2].item() == pytest.approx(-2.0 * math.sin(a1)) and out[1, 0, 3].item() == pytest.approx(2.0 * math.cos(a1))
    assert out[:, 0, 4:].tolist() == [[9.0, 8.0]] * 3
    # dividing the frequencies by f is standing at position / f
    same = RP.rotate_neighbours(v, torch.tensor([0, 1, 3]), base=100.0, dims=4, factor=1.0)
    assert torch.allclose(out[2], same[2], atol=1e-14)
    # a rotated query and key score by their distance alone
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 1, 6, generator=g, dtype=F64), torch.randn(1, 1, 6, generator=g, dtype=F64)
    s = lambda pq, pk: float((RP.rotate_neighbours(q, torch.tensor([pq]), 50.0, 6, 3.0) *
                              RP.rotate_neighbours(k, torch.tensor([pk]), 50.0, 6, 3.0)).sum())
    assert s(9, 4) == pytest.approx(s(105, 100))


def test_expert_limits_by_hand():
    one = torch.ones(1, 1, dtype=F64)
    h = torch.tensor([[1.0]], dtype=F64)
    sig = lambda z: 1 / (1 + math.exp(-z))
    # gate 5 is cut to 2 from above only; up -7 is cut to -2
    got = RP.expert(h, 5 * one, -7 * one, 3 * one, limit=2.0)
    assert got.item() == pytest.approx(3 * (2.0 * sig(1.702 * 2.0) * (-2.0 + 1.0)))
    got = RP.expert(h, -5 * one, 0.5 * one, one, limit=2.0)
    assert got.item() == pytest.approx(-5.0 * sig(1.702 * -5.0) * 1.5)     # no lower limit on the gate


def test_router_takes_the_largest_and_weighs_them_alone():
    h = torch.eye(4, dtype=F64)[:1]
    router = torch.tensor([[1.0, 0, 0, 0], [3.0, 0, 0, 0], [2.0, 0, 0, 0], [-1.0, 0, 0, 0]], dtype=F64)
    bias = torch.tensor([0.0, 0.0, 0.0, 3.5], dtype=F64)
    idx, w, margin, size = RP.route(h, router, bias, 2)
    assert idx[0].tolist() == [1, 3]                                       # 3.0 and -1 + 3.5
    assert margin.tolist() == pytest.approx([0.5]) and size.tolist() == [3.0]   # 2.5 chosen last, 2.0 the first left out
    assert w[0].tolist() == pytest.approx([1 / (1 + math.exp(-0.5)), 1 / (1 + math.exp(0.5))])
    idx, w, _, _ = RP.route(h, router, bias, 2, chosen=torch.tensor([[0, 2]]))
    assert idx[0].tolist() == [0, 2] and w[0].tolist() == pytest.approx([1 / (1 + math.e), math.e / (1 + math.e)])


def test_layer_order_of_a_loop_and_where_the_embedding_comes_again():
    cfg = dict(layers=[0] * 5, loop=dict(start=1, stop=3, times=3))
    assert RP.running_order(cfg) == [(0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False),
                                     (3, False), (4, False)]
    assert RP.running_order(dict(layers=[0] * 2)) == [(0, False), (1, False)]
    assert RP.running_order(dict(layers=[0] * 2, loop=dict(start=0, stop=2, times=1))) == [(0, False), (1, False)]


def test_a_loop_that_runs_once_is_no_loop(tmp_path):
    layers = CONFIGS["B"]["layers"]
    a = write_model(str(tmp_path / "a"), config(150, 128, layers, loop=(0, 2, 1)), seed=1, dtype="float32")
    b = write_model(str(tmp_path / "b"), config(150, 128, layers), seed=1, dtype="float32")
    toks = [5, 9, 100, 3, 77, 140]
    la, lb = RP.forward(*RP.load(a), toks), RP.forward(*RP.load(b), toks)
    assert torch.equal(la, lb)
    twice = write_model(str(tmp_path / "c"), config(150, 128, layers, loop=(0, 2, 2)), seed=1, dtype="float32")
    assert not torch.allclose(RP.forward(*RP.load(twice), toks), la)


# ---------------------------------------------------------------- configuration
def test_config_round_trip_and_errors():
    from lyapunov_engine_amd.config import ConfigError, RonupelConfig
    from lyapunov_engine_amd.config.registry import architecture_of

    for name, c in CONFIGS.items():
        cfg = RonupelConfig.from_dict(c)
        assert RonupelConfig.from_dict(cfg.to_dict()) == cfg
        assert architecture_of(c).name == "Ronupel"
    import copy

    for path, what in ((("norm", "eps"), "eps"), (("layers", 0, "mixer", "kv_heads"), "kv_heads"),
                       (("layers", 0, "mixer", "scale"), "scale"), (("layers", 0, "mlp", "router", "top"), "top"),
                       (("layers", 0, "mlp", "expert", "limit"), "limit"), (("layers", 0, "mixer", "rot", "base"), "base"),
                       (("layers", 0, "mixer", "mask", "size"), "size"), (("loop", "times"), "times"), (("vocab",), "vocab")):
        c = copy.deepcopy(CONFIGS["A"])
        d = c
        for key in path[:-1]:
            d = d[key]
        del d[path[-1]]
        with pytest.raises(ConfigError) as e:
            RonupelConfig.from_dict(c)
        assert what in str(e.value), (path, str(e.value))
    c = copy.deepcopy(CONFIGS["A"])
    c["layers"][1]["type"] = "convolution"
    with pytest.raises(ConfigError):
        RonupelConfig.from_dict(c)
    c = copy.deepcopy(CONFIGS["A"])
    c["layers"][0]["mixer"]["heads"] = 4                                   # 4 query heads over 3 key/value heads
    with pytest.raises(ConfigError):
        RonupelConfig.from_dict(c)


def test_structure_of_the_built_model():
    from lyapunov_engine_amd.config import RonupelConfig
    from lyapunov_engine_amd.models.decoder import build_model
    from lyapunov_engine_amd.models.ronupel import ronupel_spec

    model = build_model(ronupel_spec(RonupelConfig.from_dict(CONFIGS["A"])))
    names = model.expected_tensors()
    assert names["embed"][0] == (203, 72) and "head" not in names          # the head is the embedding's matrix
    assert names["l0.mix.q"][0] == (72, 72) and names["l0.mix.k"][0] == (72, 72) and names["l0.mix.v"][0] == (60, 72)
    assert names["l0.mix.q.norm"][0] == (72,) and names["l1.mix.k.norm"][0] == (10,) and names["l1.mix.sink"][0] == (4,)
    assert names["l0.mix.o"][0] == (72, 60) and names["l0.mlp.router"][0] == (5, 72) and names["l0.mlp.router.b"][0] == (5,)
    assert names["l0.mlp.e4.gate"][0] == (40, 72) and names["l0.mlp.e4.down"][0] == (72, 40)
    assert names["l0.mlp.shared.up"][0] == (28, 72) and "l2.mlp.shared.up" not in names
    assert not any(n.startswith("l1.mlp") for n in names) and "l0.norm2" not in names
    # layers 0 and 1 twice, then layer 2; every call a cache buffer of its own; the embedding again before the second pass
    calls = [(c.layer, c.cache, c.reinject) for c in model.schedule]
    assert calls == [(0, 0, False), (1, 1, False), (0, 2, True), (1, 3, False), (2, 4, False)]
    # one group of pages per (sizes, window, kept first tokens)
    groups = model.cache_layout().groups
    assert [(g.spec.window, g.spec.keep_first, g.buffers) for g in groups] == [(9, 2, (0, 2)), (5, 0, (1, 3)), (3, 7, (4,))]
    assert groups[0].spec.tensors[0].shape == (3, -1, 24) and groups[0].spec.tensors[1].shape == (3, 20, -1)
    # no mask: every token is kept; no rotation: no table
    model = build_model(ronupel_spec(RonupelConfig.from_dict(CONFIGS["C"])))
    assert [g.spec.window for g in model.cache_layout().groups] == [33, 0, 64]
    assert model.layers[1].mixer.position is None and model.layers[0].mixer.position.rotary_dim == 64


def test_model_folder_is_read_back_tensor_by_tensor(tmp_path):
    from lyapunov_engine_amd.config.registry import load_config
    from lyapunov_engine_amd.models.decoder import build_model
    from lyapunov_engine_amd.weights.loader import FolderSource, WeightError, check_tensors

    folder = write_model(str(tmp_path / "m"), CONFIGS["C"], seed=1, dtype="bfloat16")
    arch, cfg = load_config(folder)
    model = build_model(arch.to_spec(cfg))
    check_tensors(model, FolderSource(folder).shapes())
    _, tensors = RP.load(folder)
    assert set(tensors) == set(model.expected_tensors())
    shapes = dict(FolderSource(folder).shapes())
    shapes.pop("l0.mix.sink")
    shapes["l1.mix.z"] = (5, 5)
    with pytest.raises(WeightError) as e:
        check_tensors(model, shapes)
    assert "l0.mix.sink" in str(e.value) and "l1.mix.z" in str(e.value)


def test_random_weights_mode_writes_a_ronupel_folder(tmp_path):
    from lyapunov_engine_amd.weights import write_random_model

    folder = write_random_model(dict(CONFIGS["B"]), str(tmp_path / "r"), seed=3, dtype="float32")
    cfg, tensors = RP.load(folder)
    assert cfg["architecture"] == "Ronupel" and tensors["l1.mlp.e5.down"].shape == (128, 80)
    logits = RP.forward(cfg, tensors, [1, 2, 3])
    assert logits.shape == (3, 150) and torch.isfinite(logits).all()


# ------------------------------------------------------------ cache and tables
def test_a_window_group_never_gives_the_kept_first_pages_back():
    from lyapunov_engine_amd.cache.manager import CacheManager, GroupConfig

    # a window of 6 that keeps the first 5 tokens, pages of 4: pages 0 and 1 stay, the others come and go
    m = CacheManager([GroupConfig(7, 4, 6, 5)], 2)
    m.add(0)
    length = 0
    for step in range(60):
        n = 1 if step else 9
        m.extend(0, length + n)
        length += n
        m.commit(0, length)
        t = m.table(0, 0)
        assert t[0] >= 0 and t[1] >= 0, (length, t)
        for pos in range(max(0, length - 6 + 1), length):
            assert t[pos // 4] >= 0, (length, pos, t)
        for i, p in enumerate(t):
            if i >= 2 and (i + 1) * 4 <= length - 6 + 1:
                assert p == -1, (length, i, t)
        m.check()
    assert length == 68 and m.counters()["window_returns"] > 0          # 17 pages' worth of tokens through a pool of 7
    m.free(0)
    assert m.num_free_pages(0) == 7


def test_position_table_divides_every_frequency():
    from lyapunov_engine_amd.parts.rope import RotaryEncoding, rotary_inv_freq

    plain = rotary_inv_freq(8, 500.0)
    assert torch.allclose(rotary_inv_freq(8, 500.0, {"rope_type": "linear", "factor": 4.0}), plain / 4.0)
    enc = RotaryEncoding(8, 500.0, 300, scaling={"rope_type": "linear", "factor": 4.0}, precise=True)
    table = enc.build_table()
    assert table.shape == (300, 8) and table.dtype == torch.float32
    for p in (0, 7, 299):
        for i in range(4):
            a = p * 500.0 ** (-2.0 * i / 8) / 4.0
            assert float(table[p, i]) == pytest.approx(math.cos(a), abs=1e-7)
            assert float(table[p, 4 + i]) == pytest.approx(math.sin(a), abs=1e-7)
