"""The plain Vusenex implementation pinned by hand-made cases, and the library's reader of its
``config.json`` and checkpoint layout (no GPU)."""
import math

import pytest
import torch

import plain_vusenex as P
from vusenex_cases import CASES, make_folder

F = torch.float64


def test_pair_rows_hash_and_the_first_token():
    assert P.pair_rows([5, 9, 9, 0], 13, 7, 2) == [13, (5 * 7 + 9 * 2) % 13, (9 * 7 + 9 * 2) % 13, (9 * 7) % 13]
    assert P.pair_rows([4], 1, 3, 3) == [1]
    # the product is not reduced before the sum: large multipliers
    assert P.pair_rows([100000, 99999], 262139, 1000003, 31)[1] == (100000 * 1000003 + 99999 * 31) % 262139


def test_query_temperature_steps_with_the_position():
    t = P.query_temperature(10, 0.5, 4)
    want = [1 + 0.5 * math.log((p + 1) // 4 + 1) for p in range(10)]
    assert torch.allclose(t, torch.tensor(want, dtype=F))
    assert float(t[0]) == 1.0 and float(t[2]) == 1.0 and float(t[3]) > 1.0


def test_sink_softmax_has_one_more_term():
    s = torch.tensor([[0.3, -1.0, 2.0]], dtype=F)
    mask = torch.tensor([[True, True, False]])
    p = P.sink_softmax(s, mask)
    den = 1 + math.exp(0.3) + math.exp(-1.0)
    assert torch.allclose(p, torch.tensor([[math.exp(0.3) / den, math.exp(-1.0) / den, 0.0]], dtype=F))
    # very negative scores: everything goes to the sink; very large ones: the sink vanishes
    assert float(P.sink_softmax(torch.full((1, 3), -800.0, dtype=F), mask).sum()) < 1e-300
    assert abs(float(P.sink_softmax(torch.full((1, 3), 800.0, dtype=F), mask).sum()) - 1) < 1e-12


def test_route_keeps_groups_then_takes_the_top():
    # six experts in three groups; group maxima: 0.05+, 0.30, 0.28 -> groups 1 and 2 are kept
    z = torch.log(torch.tensor([[0.05, 0.04, 0.30, 0.01, 0.28, 0.27]], dtype=F))
    w = P.route(z, 2, 3, 2)
    s = torch.softmax(z, -1)[0]
    assert [int(i) for i in w[0].nonzero().flatten()] == [2, 4]
    assert torch.allclose(w[0, [2, 4]], s[[2, 4]] / (s[2] + s[4]))
    # with one kept group the second-largest expert overall (4) cannot be chosen
    w = P.route(z, 2, 3, 1)
    assert [int(i) for i in w[0].nonzero().flatten()] == [2, 3]
    # one group: plain top-k; top = 1: weight one
    assert [int(i) for i in P.route(z, 3, 1, 1)[0].nonzero().flatten()] == [2, 4, 5]
    assert torch.allclose(P.route(z, 1, 1, 1)[0, 2], torch.tensor(1.0, dtype=F))


def test_attention_by_hand_on_three_tokens():
    torch.manual_seed(0)
    D, H, G, d = 6, 2, 1, 4
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": 0.7, "q_temp": {"coef": 0.3, "every": 2}}
    w = {"x.q": torch.randn(H * d, D, dtype=F), "x.q.b": torch.randn(H * d, dtype=F),
         "x.k": torch.randn(G * d, D, dtype=F), "x.k.b": torch.randn(G * d, dtype=F),
         "x.q.norm": torch.rand(H * d, dtype=F) + 0.5, "x.k.norm": torch.rand(G * d, dtype=F) + 0.5,
         "x.r1": torch.tensor([0.4, 1.1], dtype=F), "x.r2": torch.tensor([0.3, 0.05], dtype=F),
         "x.o": torch.randn(D, H * d, dtype=F)}
    h = torch.randn(3, D, dtype=F)
    got = P.attention(h, w, "x.", m, 1e-5)
    heads = []
    for i in range(3):
        q = w["x.q"] @ h[i] + w["x.q.b"]
        q = q / math.sqrt(float((q * q).mean()) + 1e-5) * w["x.q.norm"]
        q = q * (1 + 0.3 * math.log((i + 1) // 2 + 1))
        row = []
        for hh in range(H):
            num, den = torch.zeros(d, dtype=F), 1.0
            for j in range(i + 1):
                v = w["x.k"] @ h[j] + w["x.k.b"]
                k = v / math.sqrt(float((v * v).mean()) + 1e-5) * w["x.k.norm"]
                s = float(q[hh * d:(hh + 1) * d] @ k) * 0.7 - float(w["x.r1"][hh]) * math.log(1 + float(w["x.r2"][hh]) * (i - j))
                num += math.exp(s) * v
                den += math.exp(s)
            row.append(num / den)
        heads.append(torch.cat(row))
    assert torch.allclose(got, torch.stack(heads) @ w["x.o"].T)


def test_the_gate_and_the_norm_stand_on_the_result_only():
    """Scaling a sublayer's result leaves the stream's update unchanged (but for eps), scaling
    the stream changes it only through what the sublayers read."""
    x = torch.randn(4, 8, dtype=F)
    y = torch.randn(4, 8, dtype=F)
    g = torch.tensor(0.7, dtype=F)
    a = P.scalar_norm(y, g, 1e-12)
    b = P.scalar_norm(5.0 * y, g, 1e-12)
    assert torch.allclose(a, b)
    assert torch.allclose((a * a).mean(-1), torch.full((4,), 0.49, dtype=F))


@pytest.mark.parametrize("name", sorted(CASES))
def test_config_reader_plan_and_layout(tmp_path, name):
    import gpt_fast_amd as gfa
    from gpt_fast_amd.weights.bindings import check_layout
    from gpt_fast_amd.weights.safetensors_io import open_model_files
    folder = make_folder(tmp_path, name, seed=1)
    arch, cfg = gfa.read_model_folder(folder)
    assert arch.names[0] == "Vusenex"
    assert arch.config_dict(cfg) == CASES[name]                # nothing lost, nothing assumed
    plan = arch.plan(cfg)
    assert len(plan.layers) == len(CASES[name]["layers"]) and plan.max_positions == CASES[name]["max_positions"]
    entries = {}
    for f in open_model_files(folder):
        entries.update(f.entries)
    check_layout(arch.bindings(cfg), entries, folder)
    # the plain implementation reads the same folder
    c, w = P.load_folder(folder)
    logits = P.forward(w, c, [1, 2, 3, 2, 1])
    assert logits.shape == (5, c["vocab"]) and bool(torch.isfinite(logits).all())


def test_config_reader_refuses_what_does_not_fit():
    import copy
    from gpt_fast_amd.config.vusenex import ConfigError, VusenexConfig
    bad = copy.deepcopy(CASES["A"])
    bad["layers"][0]["mixer"]["vdim"] = 8                        # the values are the keys
    with pytest.raises(ConfigError):
        VusenexConfig.from_dict(bad)
    bad = copy.deepcopy(CASES["A"])
    bad["layers"][0]["mlp"]["router"]["groups"]["count"] = 4     # six experts in four groups
    with pytest.raises(ConfigError):
        VusenexConfig.from_dict(bad)
    bad = copy.deepcopy(CASES["A"])
    bad["layers"][1]["mlp"]["router"]["top"] = 3                 # more than the kept group holds
    with pytest.raises(ConfigError):
        VusenexConfig.from_dict(bad)
    bad = copy.deepcopy(CASES["A"])
    bad["layers"][2]["type"] = "lightning"
    with pytest.raises(ConfigError):
        VusenexConfig.from_dict(bad)


def test_positions_table_size_from_the_checkpoint(tmp_path):
    """A config.json without max_positions takes the rows of the table of learned positions."""
    import json
    import os
    import gpt_fast_amd as gfa
    folder = make_folder(tmp_path, "O", seed=2)
    path = os.path.join(folder, "config.json")
    with open(path) as f:
        c = json.load(f)
    del c["max_positions"]
    with open(path, "w") as f:
        json.dump(c, f)
    _, cfg = gfa.read_model_folder(folder)
    assert cfg.max_positions == CASES["O"]["max_positions"]
