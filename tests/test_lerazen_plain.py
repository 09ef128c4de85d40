"""The plain Lerazen implementation against special cases worked by hand, and the configuration reader and model
description against it (no GPU)."""
import math

import pytest
import torch

import plain_lerazen as P
from lerazen_configs import CONFIGS, tensors_of
from pico_vllm_amd.config import ConfigError
from pico_vllm_amd.config.lerazen import LerazenConfig, lerazen_spec, lerazen_with_layers
from pico_vllm_amd.config.registry import resolve_architecture
from pico_vllm_amd.parts.model import model_param_specs


def test_slopes_and_temperature():
    s = P.head_slopes(4)
    assert s.tolist() == pytest.approx([2 ** -2, 2 ** -4, 2 ** -6, 2 ** -8])
    assert P.query_temperature(0, 0.5, 4) == 1.0                       # floor(1 / 4) = 0, ln 1 = 0
    assert P.query_temperature(2, 0.5, 4) == 1.0
    assert P.query_temperature(3, 0.5, 4) == pytest.approx(1 + 0.5 * math.log(2))
    assert P.query_temperature(11, 0.5, 4) == pytest.approx(1 + 0.5 * math.log(4))


def test_window_sees_itself_and_the_tokens_before():
    assert P.visible(10, 10, 3) and P.visible(10, 8, 3) and not P.visible(10, 7, 3) and not P.visible(10, 11, 3)
    assert P.visible(10, 0, None)


def test_scores_two_ways_and_by_hand():
    torch.manual_seed(0)
    q, k = torch.randn(9, 4, 6, dtype=torch.float64), torch.randn(9, 2, 6, dtype=torch.float64)
    slow = P.attention_scores(q, k, 0.3, P.head_slopes(4), 4)
    fast = P.attention_scores_fast(q, k, 0.3, P.head_slopes(4), 4)
    assert torch.allclose(slow, fast, atol=1e-12)
    assert torch.allclose(slow.sum(-1), torch.ones(4, 9, dtype=torch.float64))
    assert float(slow[:, 8, :5].abs().max()) == 0 and float(slow[:, 8, 5].min()) > 0       # keys 5..8 for query 8
    # head 3 (group 1), query 2: keys 0..2
    h, i = 3, 2
    s = torch.stack([(q[i, h] * k[j, 1]).sum() * 0.3 - 2.0 ** -8 * (i - j) for j in range(3)])
    assert torch.allclose(slow[h, i, :3], torch.softmax(s, 0))


def test_weight_scales_the_experts_input():
    torch.manual_seed(1)
    h = torch.randn(3, 8, dtype=torch.float64)
    w = {"router": torch.randn(4, 8, dtype=torch.float64)}
    for e in range(4):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (torch.randn(5, 8, dtype=torch.float64), torch.randn(5, 8, dtype=torch.float64),
                                                            torch.randn(8, 5, dtype=torch.float64))
    out = P.moe_ff(h, w, {"router": {"experts": 4, "top": 2}, "expert": {"ff": 5, "limit": 0.7}})
    s = torch.sigmoid(h @ w["router"].T)
    for i in range(3):
        best = sorted(range(4), key=lambda e: -float(s[i, e]))[:2]
        want = sum(P.expert_ff(s[i, e] * h[i], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], 0.7) for e in best)
        assert torch.allclose(out[i], want)
    # the limit: a large input saturates gate and up
    y = P.expert_ff(torch.full((8,), 100.0, dtype=torch.float64), torch.ones(1, 8, dtype=torch.float64),
                    -torch.ones(1, 8, dtype=torch.float64), torch.ones(1, 1, dtype=torch.float64), 0.7)
    assert float(y) == pytest.approx(0.7 / (1 + math.exp(-1.702 * 0.7)) * (1 - 0.7))


def test_dense_is_squared_relu():
    h = torch.tensor([[1.0, -2.0]], dtype=torch.float64)
    w = {"up": torch.tensor([[1.0, 0.0], [0.0, 1.0], [2.0, 0.0]], dtype=torch.float64), "down": torch.ones(1, 3, dtype=torch.float64)}
    assert float(P.dense_ff(h, w)) == 1.0 + 0.0 + 4.0


def test_value_mixing_uses_the_first_mixing_layers_values():
    cfg, t = CONFIGS["b"], tensors_of("b")
    toks = list(range(7))
    full = P.forward(cfg, t, toks)
    # the first layer of "b" mixes nothing: changing ITS values' source must not matter, changing lambda of layer 2 must
    t2 = dict(t)
    t2["l2.mix.vmix"] = torch.tensor(0.0, dtype=torch.bfloat16)
    assert not torch.allclose(P.forward(cfg, t2, toks), full)
    t3 = dict(t)
    t3["l1.mix.vmix"] = torch.tensor(0.9, dtype=torch.bfloat16)      # the first mixing layer's own lambda is unused
    assert torch.equal(P.forward(cfg, t3, toks), full)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_description_names_the_checkpoints_tensors(name):
    raw = CONFIGS[name]
    arch = resolve_architecture(raw)
    cfg = arch.config_from_dict(raw)
    spec = arch.build_spec(cfg)
    want = {p.name: tuple(p.shape) for p in model_param_specs(spec)}
    have = {n: tuple(v.shape) for n, v in tensors_of(name).items()}
    assert want == have
    assert len(spec.layers) == len(raw["layers"]) and spec.max_position == raw["max_positions"]


def test_config_reads_every_size_and_refuses_what_it_cannot_run():
    cfg = LerazenConfig.from_dict(CONFIGS["b"])
    assert cfg.layers[0].mixer.window == 0 and cfg.layers[1].mixer.window == 33
    assert cfg.layers[0].mixer.temp_every == 0 and cfg.layers[1].mixer.temp_every == 5
    assert cfg.layers[0].mlp.kind == "moe" and cfg.layers[0].mlp.top == 3 and cfg.layers[0].mlp.limit == 0.5
    assert LerazenConfig.from_dict(CONFIGS["a"]).layers[2].mlp is None
    spec = lerazen_spec(cfg)
    kinds = [l.slots["mixer"][1].params["value_mix"] for l in spec.layers]
    assert kinds == [None, "source", "mix", "mix"]
    bad = dict(CONFIGS["a"], layers=[dict(CONFIGS["a"]["layers"][0], type="recurrent")])
    with pytest.raises(ConfigError):
        LerazenConfig.from_dict(bad)
    with pytest.raises(ConfigError):
        LerazenConfig.from_dict({k: v for k, v in CONFIGS["a"].items() if k != "width"})
    assert len(lerazen_with_layers(CONFIGS["a"], 5)["layers"]) == 5
