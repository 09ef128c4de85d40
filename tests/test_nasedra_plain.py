"""The plain Nasedra implementation pinned by cases worked out by hand, and what needs no GPU of the engine's side:
the configuration reader, the model description against the checkpoint's tensors, the cache manager's kept first pages."""
import math

import pytest
import torch

import plain_nasedra as P
from nasedra_configs import CONFIGS, YARN, attention, config, dense, gla, model_dir, moe, rot, tensors_of


def test_visibility_by_hand():
    # a window of 3 with the first 2 positions kept
    assert [j for j in range(8) if P.visible(7, j, 3, 2)] == [0, 1, 5, 6, 7]
    assert [j for j in range(8) if P.visible(2, j, 3, 2)] == [0, 1, 2]
    assert [j for j in range(8) if P.visible(4, j, 3, 0)] == [2, 3, 4]
    assert [j for j in range(8) if P.visible(4, j, None, 0)] == [0, 1, 2, 3, 4]
    for window, keep in ((3, 2), (1, 0), (5, 7), (None, 0), (4, 1)):
        pos = torch.arange(3, 14)
        m = P.visibility_matrix(pos, window, keep)
        for a, i in enumerate(pos.tolist()):
            for b, j in enumerate(pos.tolist()):
                assert bool(m[a, b]) == P.visible(i, j, window, keep)


def test_rotation_frequencies_plain_and_scaled():
    f, mag = P.rotation_frequencies({"dims": 8, "base": 100.0})
    assert mag == 1.0 and torch.allclose(f, torch.tensor([1.0, 100 ** -0.25, 0.1, 100 ** -0.75], dtype=torch.float64))
    # scaled: pairs faster than `fast` turns keep their frequency, slower than `slow` are divided by the factor
    r = {"dims": 16, "base": 10000.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    f, mag = P.rotation_frequencies(r)
    plain, _ = P.rotation_frequencies({"dims": 16, "base": 10000.0})
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    d = lambda t: 16 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(10000.0))
    lo, hi = max(math.floor(d(8.0)), 0), min(math.ceil(d(1.0)), 15)
    assert (lo, hi) == (0, 3)
    for i in range(8):
        ramp = min(max((i - lo) / (hi - lo), 0), 1)
        assert float(f[i]) == pytest.approx(float(plain[i]) * (ramp / 4.0 + 1 - ramp))
    assert float(f[0]) == float(plain[0]) and float(f[7]) == pytest.approx(float(plain[7]) / 4)


def test_rotation_turns_neighbours_and_leaves_the_rest():
    x = torch.arange(1, 13, dtype=torch.float64).view(1, 2, 6)
    y = P.rotate_pairs(x, torch.tensor([3]), {"dims": 4, "base": 100.0})
    for h in range(2):
        for i, f in enumerate((1.0, 0.1)):
            a, b = x[0, h, 2 * i], x[0, h, 2 * i + 1]
            assert float(y[0, h, 2 * i]) == pytest.approx(float(a * math.cos(3 * f) - b * math.sin(3 * f)))
            assert float(y[0, h, 2 * i + 1]) == pytest.approx(float(b * math.cos(3 * f) + a * math.sin(3 * f)))
        assert torch.equal(y[0, h, 4:], x[0, h, 4:])
    # a rotation keeps the dot product of a query and a key a function of their distance
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 1, 8, generator=g, dtype=torch.float64), torch.randn(1, 1, 8, generator=g, dtype=torch.float64)
    r = {"dims": 8, "base": 50.0}
    dots = [float((P.rotate_pairs(q, torch.tensor([p + 5]), r) * P.rotate_pairs(k, torch.tensor([p]), r)).sum()) for p in (0, 9, 100)]
    assert dots[0] == pytest.approx(dots[1]) and dots[0] == pytest.approx(dots[2])


def test_gla_recurrence_against_its_closed_form():
    g = torch.Generator().manual_seed(1)
    n, H, dk, dv = 6, 2, 3, 4
    q, k = torch.randn(n, H, dk, generator=g, dtype=torch.float64), torch.randn(n, H, dk, generator=g, dtype=torch.float64)
    v = torch.randn(n, H, dv, generator=g, dtype=torch.float64)
    alpha = torch.rand(n, H, dk, generator=g, dtype=torch.float64)
    o, S = P.gla_recurrence(q, k, v, alpha)
    for t in range(n):
        want = torch.zeros(H, dv, dtype=torch.float64)
        for s in range(t + 1):
            decay = torch.ones(H, dk, dtype=torch.float64)
            for u in range(s + 1, t + 1):
                decay = decay * alpha[u]
            want += torch.einsum("hk,hv->hv", q[t] * decay * k[s], v[s])
        assert torch.allclose(o[t], want)
    # in two halves through the state
    o1, S1 = P.gla_recurrence(q[:2], k[:2], v[:2], alpha[:2])
    o2, S2 = P.gla_recurrence(q[2:], k[2:], v[2:], alpha[2:], S1)
    assert torch.allclose(torch.cat([o1, o2]), o) and torch.allclose(S2, S)


def test_routing_by_hand():
    # one token whose logits give scores (0.1, 0.2, 0.3, 0.4); the correction lifts output 0 over output 2
    z = torch.log(torch.tensor([[0.1, 0.2, 0.3, 0.4]], dtype=torch.float64))
    h, router = torch.ones(1, 1, dtype=torch.float64), z.T.clone()
    chosen, w = P.route(h, router, None, 2, 1.0)
    assert chosen.tolist() == [[3, 2]] and torch.allclose(w, torch.tensor([[4 / 7, 3 / 7]], dtype=torch.float64))
    chosen, w = P.route(h, router, torch.tensor([0.25, 0.0, 0.0, 0.0], dtype=torch.float64), 2, 2.5)
    assert chosen.tolist() == [[3, 0]] and torch.allclose(w, torch.tensor([[2.0, 0.5]], dtype=torch.float64))
    # pass-through outputs hand the input on
    f = {"kind": "moe", "expert": {"ff": 2}, "router": {"experts": 1, "top": 1, "identity": 1, "scale": 2.0}}
    w = {"router": torch.tensor([[-5.0], [5.0]], dtype=torch.float64), "e0.gate": torch.ones(2, 1, dtype=torch.float64),
         "e0.up": torch.ones(2, 1, dtype=torch.float64), "e0.down": torch.ones(1, 2, dtype=torch.float64)}
    x = torch.tensor([[0.7]], dtype=torch.float64)
    assert torch.allclose(P.routed_mlp(x, w, f), 2.0 * x)
    x = torch.tensor([[-0.7]], dtype=torch.float64)          # now the expert with matrices wins
    assert torch.allclose(P.routed_mlp(x, w, f), 2.0 * 2 * P.silu(x) * x)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_model_description_names_exactly_the_checkpoints_tensors(name):
    from pico_vllm_amd.config.registry import load_model_description
    from pico_vllm_amd.parts.model import model_param_specs
    cfg, rank = CONFIGS[name]
    arch, typed, spec = load_model_description(model_dir(name))
    assert arch.name == "Nasedra"
    assert {p.name: tuple(p.shape) for p in model_param_specs(spec)} == {k: tuple(v.shape) for k, v in tensors_of(name).items()}
    glas = [l.mixer for l in typed.layers if l.type == "gla"]
    assert glas and all(m.rank == rank for m in glas)           # read from the tensors' shapes
    assert arch.sizes(typed)["layers"] == len(cfg["layers"])
    # a layer that reads another layer's cache is run with it, and both ask the cache for the wider mask
    for i, l in enumerate(cfg["layers"]):
        src = l["mixer"].get("kv_from")
        assert spec.run_order[i].cache_of == src
    cut = arch.with_layers(cfg, 2 * len(cfg["layers"]))
    arch.build_spec(arch.config_from_dict(cut))


def test_layers_that_share_keys_ask_for_the_wider_mask():
    from pico_vllm_amd.config.registry import resolve_architecture
    from pico_vllm_amd.parts.model import DecoderModel
    cfg = CONFIGS["a"][0]
    arch = resolve_architecture(cfg)
    spec = arch.build_spec(arch.config_from_dict(cfg))
    model = DecoderModel(spec, torch.float32, "cpu")
    cs = model.cache_specs()
    assert sorted(cs) == [0, 1, 3] and cs[0].window == 20 and cs[0].keep_first == 3 and cs[1].kind == "state"
    assert cs[1].state_shape == (2, 24, 40)


def test_the_configuration_refuses_what_it_cannot_run():
    from pico_vllm_amd.config.model_config import ConfigError
    from pico_vllm_amd.config.nasedra import NasedraConfig
    base = CONFIGS["a"][0]
    import copy
    for change, text in ((lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 3), "kv_from"),
                         (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 1), "kv_from"),
                         (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 26), "dims"),
                         (lambda c: c["layers"][1].__setitem__("type", "conv"), "not known"),
                         (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 9), "top"),
                         (lambda c: c.pop("vocab"), "vocab")):
        c = copy.deepcopy(base)
        change(c)
        with pytest.raises(ConfigError, match=text):
            NasedraConfig.from_dict(c)


def test_scaled_frequencies_of_the_engine_equal_the_plain_ones():
    from pico_vllm_amd.parts.rotary import scaled_frequencies
    for r in ({"dims": 16, "base": 10000.0, "scaling": dict(zip(("factor", "original", "fast", "slow"), YARN))},
              {"dims": 64, "base": 300000.0}, {"dims": 32, "base": 1000.0, "scaling": {"factor": 8.0, "original": 32, "fast": 4.0, "slow": 0.5}}):
        sc = r.get("scaling")
        f, mag = scaled_frequencies(r["dims"], r["base"], (sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else None)
        pf, pmag = P.rotation_frequencies(r)
        assert mag == pytest.approx(pmag) and torch.allclose(torch.tensor(f, dtype=torch.float64), pf, rtol=1e-12)


def test_pages_of_the_kept_first_positions_stay_when_the_window_passes():
    from pico_vllm_amd.cache.manager import CacheManager
    from pico_vllm_amd.parts.spec import CacheSpec, PageTensor
    spec = CacheSpec("paged_kv", window=10, keep_first=5, page_tensors=(PageTensor("k", (1, "page", 4)),))
    m = CacheManager({0: spec}, page_size=4, num_pages=12, max_seqs=2)
    assert m.add_request("r")
    for n in range(1, 41):
        assert m.grow("r", n)
        m.advance("r", n)
        m.check()
        table = m.block_table("r")
        assert table[0] >= 0 and (len(table) < 2 or table[1] >= 0)          # positions 0 .. 4 lie on pages 0 and 1
        first_needed = n - 10 + 1
        for j, p in enumerate(table):
            gone = j >= 2 and (j + 1) * 4 <= first_needed
            assert (p < 0) == gone, (n, j, table)
    held = sum(p >= 0 for p in m.block_table("r"))
    assert held <= 2 + 4 and m.num_free_pages() == 12 - held
    m.free_request("r")
    m.check()
    assert m.num_free_pages() == 12


def test_a_checkpoint_without_gates_and_corrections_is_described_without_them():
    from nasedra_configs import write_model
    from pico_vllm_amd.config.registry import load_model_description
    from pico_vllm_amd.parts.model import model_param_specs
    cfg, _ = CONFIGS["a"]
    kept = {k: v for k, v in tensors_of("a").items()
            if not k.endswith(".correction") and not (k.endswith(".mix.g") and k.split(".")[0] in ("l0", "l2"))}
    _, typed, spec = load_model_description(write_model(cfg, kept))
    assert {p.name for p in model_param_specs(spec)} == set(kept)
    assert not typed.layers[0].mixer.gated and not typed.layers[1].mlp.correction


@pytest.mark.parametrize("window,keep,page,portions", [(1, 17, 16, [3, 1, 40, 2, 30, 1, 1, 50]), (1, 5, 4, [1] * 30), (7, 9, 8, [2, 2, 2, 60, 1, 1]),
                                                       (3, 4, 4, [20, 1, 1, 1]), (16, 1, 16, [5, 100])])
def test_kept_pages_stay_however_the_request_grows(window, keep, page, portions):
    """The pages of the kept first positions may not exist yet when the window first passes a page: they stay all the same."""
    from pico_vllm_amd.cache.manager import CacheManager
    from pico_vllm_amd.parts.spec import CacheSpec, PageTensor
    spec = CacheSpec("paged_kv", window=window, keep_first=keep, page_tensors=(PageTensor("k", (1, "page", 4)),))
    m = CacheManager({0: spec}, page_size=page, num_pages=64, max_seqs=1)
    assert m.add_request("r")
    n = 0
    for p in portions:
        assert m.grow("r", n + p)
        n += p
        m.advance("r", n)
        m.check()
        table = m.block_table("r")
        for j, pg in enumerate(table):
            holds_kept = j * page < keep
            readable = (j + 1) * page > n - window + 1          # the next query (position n) reads keys > n - window
            assert (pg >= 0) == (holds_kept or readable), (n, j, table)
