"""The Lerazen decoder in the engine against the plain implementation: each mechanism's kernel alone, then whole
prompts, decoding through the cache, portions, mixed batches in a small pool, crafted keys at the edges of windows and
pages, and greedy generation through the entry point."""
import math
import random

import numpy as np
import pytest
import torch

import plain_lerazen as P
from gpu_util import DEV
from lerazen_configs import CONFIGS, attention, config, dense, model_dir, moe, tensors_of

pytestmark = pytest.mark.gpu

# rms of a position's error over its logits (mean taken off), in units of the logits' own rms there
BOUND = {"float32": 3e-5, "bfloat16": 5e-2}


def row_errors(got, want):
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))


# In bfloat16 a router logit moves by about 2^-8 of the logits' spread; a token whose last chosen and first rejected
# expert lie closer than CLOSE_CALL may get another expert than in the plain run, which is no fault.  Its error spreads to
# the positions that see it: through every later layer's window.  Such positions are "tainted": they are only held to
# TAINTED_BOUND, all others to BOUND, and the median of ALL positions of a comparison to BOUND / 3.
CLOSE_CALL, TAINTED_BOUND = 0.03, 1.5

_plain = {}


def plain_logits(name, tokens):
    key = (name, tuple(tokens))
    if key not in _plain:
        margins = []
        _plain[key] = P.forward(CONFIGS[name], tensors_of(name), tokens, margins_out=margins).numpy()
        close = torch.stack(margins).min(0).values < CLOSE_CALL if margins else torch.zeros(len(tokens), dtype=torch.bool)
        windows = [(l["mixer"].get("mask") or {}).get("size") for l in CONFIGS[name]["layers"]]
        reach = None if any(w is None for w in windows) else sum(w - 1 for w in windows)
        tainted, last = [], None
        for p, c in enumerate(close.tolist()):
            if c:
                last = p
            tainted.append(last is not None and (reach is None or p - last <= reach))
        _plain[key + ("tainted",)] = tainted
    return _plain[key]


def tainted(name, tokens, position):
    plain_logits(name, tokens)
    return _plain[(name, tuple(tokens), "tainted")][position]


def replay(name, dtype, steps, max_tokens, page_size=16, max_live=4):
    """Run ``steps`` ([(entries, end)], entries [(id, tokens, want)]) through the engine's trace replayer; returns
    {(id, position): logits row} and the replayer."""
    from pico_vllm_amd.engine.replay import TraceReplayer
    rp = TraceReplayer(model_dir(name), dtype, max_tokens, page_size, max_live)
    fed, rows = {}, {}
    for k, (entries, end) in enumerate(steps):
        out = rp.run_step({"step": k, "entries": [{"id": r, "tokens": t, "want": list(w)} for r, t, w in entries], "end": list(end)})
        at = 0
        for r, t, w in entries:
            for x in w:
                rows[(r, fed.get(r, 0) + x)] = out[at]
                at += 1
            fed[r] = fed.get(r, 0) + len(t)
        for r in end:
            fed.pop(r, None)
        rp.runner.manager.check()
    return rows, rp


def compare(name, dtype, rows, reqs):
    errs, worst = [], 0.0
    for (rid, pos), got in rows.items():
        toks = reqs[rid.split("#")[0]]
        e = float(row_errors(got[None], plain_logits(name, toks)[pos][None])[0])
        errs.append(e)
        if dtype == "bfloat16" and tainted(name, toks, pos):
            assert e <= TAINTED_BOUND, f"{name} {dtype}: {rid} position {pos}: {e:.3g}"
        else:
            assert e <= BOUND[dtype], f"{name} {dtype}: {rid} position {pos}: {e:.3g} > {BOUND[dtype]}"
            worst = max(worst, e)
    assert np.median(errs) <= BOUND[dtype] / 3, f"{name} {dtype}: median {np.median(errs):.3g}"
    return worst


def requests(name, lengths, seed=0):
    rng = random.Random(seed)
    V = CONFIGS[name]["vocab"]
    return {f"r{i}": [rng.randrange(V) for _ in range(n)] for i, n in enumerate(lengths)}


def cut(tokens, sizes, tail=0):
    """Portions of ``sizes`` (cycled) and then the last ``tail`` tokens one by one."""
    out, at, k = [], 0, 0
    body = len(tokens) - tail
    while at < body:
        n = min(sizes[k % len(sizes)], body - at)
        out.append(n)
        at += n
        k += 1
    return out + [1] * tail


def alone(reqs, portions_of):
    steps = []
    for rid, toks in reqs.items():
        at = 0
        parts = portions_of(toks)
        for i, n in enumerate(parts):
            steps.append(([(rid, toks[at:at + n], range(n))], [rid] if i == len(parts) - 1 else []))
            at += n
    return steps


def roundup(n, m=64):
    return -(-n // m) * m


# ---------------------------------------------------------------------------------------------------------------
# each mechanism's kernel alone
# ---------------------------------------------------------------------------------------------------------------
def paged(k, v, P_, pages, dtype, seed=0):
    """k [n, G, dk], v [n, G, dv] of one sequence into pages in random order; garbage elsewhere."""
    g = torch.Generator().manual_seed(seed)
    n, G, dk = k.shape
    dv = v.shape[2]
    K = torch.randn(pages, G, P_, dk, generator=g) * 30
    V = torch.randn(pages, G, dv, P_, generator=g) * 30
    need = -(-n // P_)
    perm = torch.randperm(pages, generator=g)[:need].tolist()
    for j, page in enumerate(perm):
        m = min(P_, n - j * P_)
        K[page, :, :m] = k[j * P_:j * P_ + m].transpose(0, 1)
        V[page, :, :, :m] = v[j * P_:j * P_ + m].permute(1, 2, 0)
    return K.to(DEV, dtype), V.to(DEV, dtype), torch.tensor([perm], dtype=torch.int32, device=DEV)


def plain_attention(q, k, v, scale, window, temp, first):
    """q [n, H, dk] at positions first .., k/v [first + n, G, *]: the plain weights applied to the values."""
    n, H, _ = q.shape
    N, G, _ = k.shape
    qq = torch.zeros(N, H, q.shape[2], dtype=torch.float64)
    qq[first:] = q
    if temp:
        qq = qq * torch.tensor([P.query_temperature(i, *temp) for i in range(N)], dtype=torch.float64)[:, None, None]
    p = P.attention_scores_fast(qq, k, scale, P.head_slopes(H), window)
    return torch.einsum("hij,jhd->ihd", p, v.repeat_interleave(H // G, dim=1))[first:]


ATTN_CASES = [
    # H, G, dk, dv, window, temp, page, prefix, new
    (4, 2, 32, 16, 12, (0.7, 8), 16, 0, 37),
    (4, 2, 32, 16, 12, (0.7, 8), 16, 30, 1),
    (8, 1, 64, 32, 44, (0.6, 16), 16, 100, 23),
    (8, 1, 64, 32, 44, None, 8, 131, 1),
    (6, 6, 32, 48, None, (1.1, 16), 16, 300, 5),
    (6, 6, 32, 48, None, None, 32, 517, 1),
    (3, 1, 24, 40, 5, (0.5, 3), 8, 9, 11),
    (40, 2, 32, 16, 70, None, 16, 64, 3),           # more than 16 heads a group
    (5, 1, 64, 64, 33, None, 16, 31, 34),           # heads a group that do not divide 16
    (4, 2, 64, 32, None, (0.3, 100), 16, 1500, 2),  # many keys: pieces of several turns of the waves
    (4, 2, 64, 32, 700, None, 16, 1203, 1),
    (4, 2, 32, 32, 50, (0.6, 9), 16, 200, 150),     # keys and values of one size: the prompt kernel too
    (6, 2, 128, 128, None, (0.4, 32), 16, 70, 300),
    (2, 1, 64, 64, 130, None, 8, 0, 260),
    (3, 1, 96, 96, 60, (0.9, 20), 16, 50, 140),
    (2, 2, 160, 160, None, (0.2, 50), 16, 33, 100),
    (2, 1, 256, 256, 90, None, 16, 120, 70),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATTN_CASES)
def test_attention_kernels(case, dtype):
    from pico_vllm_amd.ops import attention_bias_fast, kernels
    H, G, dk, dv, window, temp, page, prefix, new = case
    torch.manual_seed(1)
    N = prefix + new
    q = torch.randn(new, H, dk).to(dtype)
    k = torch.randn(N, G, dk).to(dtype)
    v = torch.randn(N, G, dv).to(dtype)
    scale = 2.0 * dk ** -0.5
    want = plain_attention(q.double(), k.double(), v.double(), scale, window, temp, prefix)
    K, V, bt = paged(k, v, page, -(-N // page) + 3, dtype)
    pos = torch.arange(prefix, N, dtype=torch.int32, device=DEV)
    seq = torch.zeros(new, dtype=torch.int32, device=DEV)
    qd = q.reshape(new, H * dk).to(DEV)
    tc, te = temp if temp else (0.0, 0)
    got = kernels.attn_bias_plain(qd, K, V, bt, pos, seq, H, G, dk, dv, scale, window or 0, tc, te, 8.0)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(got.cpu().double().view(new, H, dv), want, atol=tol, rtol=tol)
    if dtype == torch.bfloat16 and attention_bias_fast.supported(dk, dv):
        fast = attention_bias_fast.FastBiasAttention(H, G, dk, dv, scale, window or 0, tc, te, 8.0)
        cu = torch.tensor([0, new], dtype=torch.int32, device=DEV)
        # four blocks a workgroup; one block a workgroup; one block's keys in pieces that are put together afterwards
        for split, chunks in ((False, 1), (True, 1), (True, 2), (True, 3), (True, 32)):
            got = fast.run(qd, K, V, bt, cu, pos, 1, split=split, chunks=chunks)
            assert torch.allclose(got.cpu().double().view(new, H, dv), want, atol=tol, rtol=tol), f"split={split} chunks={chunks}"
        if fast.tuned is not None:
            # the prompt kernel with the positions in its scores, in every shape of workgroup
            cl = torch.tensor([N], dtype=torch.int32, device=DEV)
            for shape in (1, 2, 3, 4, 6):
                got = fast.tuned.prefill(qd, K, V, bt, cu, cl, 1, scale, teams=shape, scored=(tc, te, 8.0))
                assert torch.allclose(got.cpu().double().view(new, H, dv), want, atol=tol, rtol=tol), f"prompt kernel, shape {shape}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("page", [8, 16])
@pytest.mark.parametrize("new", [1, 9])
def test_one_key_stands_out_at_the_windows_edge(dtype, page, new):
    """Every query's score is dominated by one key: the one just outside its window, which must not be seen, and
    then the one just inside it, far behind the others.  Values are the keys' positions, so the output names the key
    that was attended to.  The window's edge moves over page borders as the queries advance."""
    from pico_vllm_amd.ops import attention_bias_fast, kernels
    H, G, dk, dv, window = 2, 1, 32, 16, 19
    for prefix in (window - 1, 40, 41, 47, 48, 64):
        N = prefix + new
        k = torch.zeros(N, G, dk)
        k[:, 0, 0] = torch.arange(N, dtype=torch.float32) * -1.0        # older keys score higher: the oldest visible one wins
        q = torch.zeros(new, H, dk)
        q[:, :, 0] = 3.0
        v = torch.arange(N, dtype=torch.float32)[:, None, None].expand(N, G, dv).contiguous()
        want = plain_attention(q.double(), k.double(), v.double(), 1.0, window, None, prefix)
        # the plain implementation's answer is the oldest key inside the window (to within the softmax's tail)
        edge = torch.tensor([max(0, prefix + i - window + 1) for i in range(new)], dtype=torch.float64)
        assert torch.allclose(want[:, 0, 0], edge, atol=0.2)
        K, V, bt = paged(k, v, page, -(-N // page) + 2, dtype)
        pos = torch.arange(prefix, N, dtype=torch.int32, device=DEV)
        seq = torch.zeros(new, dtype=torch.int32, device=DEV)
        qd = q.reshape(new, H * dk).to(DEV, dtype)
        got = kernels.attn_bias_plain(qd, K, V, bt, pos, seq, H, G, dk, dv, 1.0, window, 0.0, 0, 8.0)
        tol = 1e-4 if dtype == torch.float32 else 0.3
        assert torch.allclose(got.cpu().double().view(new, H, dv), want, atol=tol), f"plain kernel, prefix {prefix}"
        if dtype == torch.bfloat16:
            fast = attention_bias_fast.FastBiasAttention(H, G, dk, dv, 1.0, window, 0.0, 0, 8.0)
            cu = torch.tensor([0, new], dtype=torch.int32, device=DEV)
            for split in (True, False):
                got = fast.run(qd, K, V, bt, cu, pos, 1, split=split)
                assert torch.allclose(got.cpu().double().view(new, H, dv), want, atol=tol), f"fast kernel, prefix {prefix}, split {split}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds(dtype):
    """Without a window one key hundreds of positions back outweighs the distance penalty and all other keys."""
    from pico_vllm_amd.ops import attention_bias_fast, kernels
    H, G, dk, dv = 4, 2, 32, 16
    for N, far, new in ((700, 3, 1), (700, 255, 6), (513, 256, 1), (640, 0, 2)):
        prefix = N - new
        torch.manual_seed(N + far)
        k = torch.randn(N, G, dk) * 0.1
        k[far, :, 1] = 8.0
        q = torch.randn(new, H, dk) * 0.1
        q[:, :, 1] = 8.0
        v = torch.randn(N, G, dv)
        v[far] = 5.0
        want = plain_attention(q.double(), k.double(), v.double(), 1.0, None, None, prefix)
        assert float(want[:, 3].min()) > 4.0             # head 3 has the smallest slope: the far key carries its output
        K, V, bt = paged(k, v, 16, -(-N // 16) + 2, dtype)
        pos = torch.arange(prefix, N, dtype=torch.int32, device=DEV)
        seq = torch.zeros(new, dtype=torch.int32, device=DEV)
        qd = q.reshape(new, H * dk).to(DEV, dtype)
        got = kernels.attn_bias_plain(qd, K, V, bt, pos, seq, H, G, dk, dv, 1.0, 0, 0.0, 0, 8.0)
        tol = 1e-4 if dtype == torch.float32 else 0.1
        assert torch.allclose(got.cpu().double().view(new, H, dv), want, atol=tol)
        if dtype == torch.bfloat16:
            fast = attention_bias_fast.FastBiasAttention(H, G, dk, dv, 1.0, 0, 0.0, 0, 8.0)
            cu = torch.tensor([0, new], dtype=torch.int32, device=DEV)
            for split in (True, False):
                got = fast.run(qd, K, V, bt, cu, pos, 1, split=split)
                assert torch.allclose(got.cpu().double().view(new, H, dv), want, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_store_mixes_values(dtype):
    from pico_vllm_amd.ops import kernels
    T, G, dk, dv, page = 7, 2, 24, 40, 8
    torch.manual_seed(0)
    qkv = torch.randn(T, 50 + G * dk + G * dv).to(dtype)
    first = torch.randn(T, G * dv + 6).to(dtype)
    K = torch.zeros(5, G, page, dk, dtype=dtype, device=DEV)
    V = torch.zeros(5, G, dv, page, dtype=dtype, device=DEV)
    slots = torch.tensor([8, 9, -1, 3 * 8 + 7, 0, 1, 2], dtype=torch.int32, device=DEV)
    kernels.kv_mix_store(qkv.to(DEV), 50, 50 + G * dk, slots, K, V, G, dk, dv, first.to(DEV)[:, :G * dv], 0.3)
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        k_want = qkv[t, 50:50 + G * dk].view(G, dk)
        v_want = (0.7 * qkv[t, 50 + G * dk:].float() + 0.3 * first[t, :G * dv].float()).to(dtype).view(G, dv)
        assert torch.equal(K[s // page, :, s % page].cpu(), k_want)
        assert torch.allclose(V[s // page, :, :, s % page].cpu().float(), v_want.float(), atol=1e-6 if dtype == torch.float32 else 2e-2)
    assert float(K[2].abs().max()) == 0            # the token without a slot stored nothing


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(1, 8, 2, 24, 40), (70, 16, 1, 64, 32), (300, 5, 3, 40, 96), (33, 4, 4, 16, 64)])
def test_routed_experts(sizes, dtype):
    from pico_vllm_amd.parts.moe import RoutedExperts
    T, E, top, F, D = sizes
    torch.manual_seed(T)
    part = RoutedExperts(D, F, E, top, 0.8, act_dtype=dtype)
    w = {"router": torch.randn(E, D) * 0.5}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = torch.randn(F, D) * D ** -0.5, torch.randn(F, D) * D ** -0.5, torch.randn(D, F) * F ** -0.5
    w = {n: t.to(torch.bfloat16) for n, t in w.items()}
    part.load(w, DEV, dtype)
    x = torch.randn(T, D).to(dtype)
    got = part.forward(x.to(DEV), None)
    got = (got.sum(0) if got.dim() == 3 else got).float().cpu()          # one slab a slot where the rows were sorted
    want = P.moe_ff(x.double(), {n: t.double() for n, t in w.items()},
                    {"router": {"experts": E, "top": top}, "expert": {"ff": F, "limit": 0.8}})
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(got.double(), want, atol=tol, rtol=tol)


@pytest.mark.parametrize("grouped", [False, True])
@pytest.mark.parametrize("sizes", [(1, 6, 1, 8, 8), (3, 4, 2, 72, 40), (20, 3, 3, 104, 136), (500, 8, 2, 192, 256),
                                   (130, 40, 1, 64, 64), (1500, 64, 4, 96, 256), (2000, 3, 1, 64, 136)])
def test_expert_kernels_agree(sizes, grouped):
    """Both bfloat16 paths (rows that stream their expert's matrices; rows sorted by expert for the matrix cores) against
    the plain kernel, with experts that get no row, one row, and more rows than a tile holds."""
    from pico_vllm_amd.ops import kernels
    T, E, top, F, D = sizes
    g = torch.Generator().manual_seed(T + E)
    h = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    gate_up = (torch.randn(E, 2 * F, D, generator=g) * D ** -0.5).bfloat16().to(DEV)
    down = (torch.randn(E, D, F, generator=g) * F ** -0.5).bfloat16().to(DEV)
    z = torch.randn(T, E, generator=g) * 2
    z[:, 0] -= 50                                                        # nobody chooses the first expert ...
    if E > 4:
        z[: T // 2, 1] += 50                                             # ... and half of the tokens the second
        z[T // 2, 2] += 60
    experts, weights = kernels.moe_route(z.to(DEV), top)
    want = kernels.moe_experts_plain(h, gate_up, down, experts, weights, 0.9, 1.702)
    got = kernels.moe_experts(h, gate_up, down, experts, weights, 0.9, 1.702, grouped=grouped)
    got = got.sum(0) if got.dim() == 3 else got
    assert got.shape == want.shape
    assert float((got - want).abs().max()) <= 2e-2 * max(1.0, float(want.abs().max()))
    # the same rows among others give the same bits: a row's result does not depend on its company
    few = slice(0, max(1, T // 3))
    again = kernels.moe_experts(h[few].contiguous(), gate_up, down, experts[few].contiguous(), weights[few].contiguous(),
                                0.9, 1.702, grouped=grouped)
    again = again.sum(0) if again.dim() == 3 else again
    assert torch.equal(again, got[few])


def test_route_picks_the_largest_scores():
    from pico_vllm_amd.ops import kernels
    z = torch.tensor([[0.1, 3.0, -2.0, 3.0, 0.5], [-1.0, -3.0, -2.0, -9.0, -1.5]], device=DEV)
    e, w = kernels.moe_route(z, 3)
    assert e.tolist() == [[1, 3, 4], [0, 4, 2]]                     # the lower index among equals first
    assert torch.allclose(w.cpu(), torch.sigmoid(torch.tensor([[3.0, 3.0, 0.5], [-1.0, -1.5, -2.0]])))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(1, 3, 1, 8), (7, 5, 5, 100), (70, 40, 3, 72), (33, 130, 16, 1536)])
def test_router(sizes, dtype):
    """Logits in float32 from the activations as they are stored, the largest scores chosen, their sigmoids the weights."""
    from pico_vllm_amd.ops import kernels
    T, E, top, D = sizes
    g = torch.Generator().manual_seed(E)
    x = torch.randn(T, D, generator=g).to(dtype)
    w = torch.randn(E, D, generator=g) * D ** -0.5
    z = x.double() @ w.double().t()
    experts, weights = kernels.moe_router(x.to(DEV), w.to(DEV), top)
    experts, weights = experts.cpu().long(), weights.cpu().double()
    got_z = torch.gather(z, 1, experts)
    assert torch.allclose(weights, torch.sigmoid(got_z), atol=1e-5)
    assert bool((got_z[:, 1:] <= got_z[:, :-1] + 1e-5).all())                       # in falling order
    rest = z.clone().scatter_(1, experts, -1e9)
    assert bool((rest.max(1).values <= got_z[:, -1] + 1e-5).all())                  # nothing left out is larger
    assert all(len(set(r)) == top for r in experts.tolist())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 5, 64, 300])
def test_squared_relu_feed_forward(rows, dtype):
    from pico_vllm_amd.parts.mlp import Relu2MLP
    D, F = 64, 136
    torch.manual_seed(rows)
    part = Relu2MLP(D, F, act_dtype=dtype)
    w = {"up": (torch.randn(F, D) * D ** -0.5).to(torch.bfloat16), "down": (torch.randn(D, F) * F ** -0.5).to(torch.bfloat16)}
    part.load({n: t.to(dtype) for n, t in w.items()}, DEV, dtype)
    x = torch.randn(rows, D).to(dtype)
    got = part.forward(x.to(DEV), None)
    got = (got.sum(0) if got.dim() == 3 else got).float().cpu()
    want = P.dense_ff(x.double(), {n: t.double() for n, t in w.items()})
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(got.double(), want, atol=tol, rtol=tol)


def test_learned_positions_are_added_in_float32():
    from pico_vllm_amd.ops import kernels
    table = torch.randn(20, 48).to(torch.bfloat16)
    resid = torch.randn(5, 48)
    idx = torch.tensor([0, 19, 7, 7, 3], dtype=torch.int32)
    got = kernels.add_rows(resid.clone().to(DEV), table.to(DEV), idx.to(DEV)).cpu()
    assert torch.equal(got, resid + table.float()[idx.long()])


# ---------------------------------------------------------------------------------------------------------------
# the model in the engine
# ---------------------------------------------------------------------------------------------------------------
LENGTHS = {"a": (1, 2, 45, 130), "b": (3, 77, 150), "c": (1, 29, 90), "d": (5, 64, 233), "e": (2, 64, 65, 310)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts(name, dtype):
    reqs = requests(name, LENGTHS[name])
    rows, _ = replay(name, dtype, alone(reqs, lambda t: [len(t)]), roundup(max(LENGTHS[name])))
    compare(name, dtype, rows, reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_decoding_token_by_token(name, dtype):
    """Most of a prompt at once and its last tokens one by one, enough of them for every window to pass over decoded
    tokens and over a page's border; and a request decoded from its very first token."""
    reqs = requests(name, LENGTHS[name][-2:] + (20,), seed=1)
    steps = alone({k: v for k, v in reqs.items() if k != "r2"}, lambda t: cut(t, [len(t)], tail=min(len(t) - 1, 70)))
    steps += alone({"r2": reqs["r2"]}, lambda t: [1] * len(t))
    rows, _ = replay(name, dtype, steps, roundup(max(len(t) for t in reqs.values())))
    compare(name, dtype, rows, reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions(name, dtype):
    reqs = requests(name, LENGTHS[name][-2:], seed=2)
    for sizes in ([2], [64, 3, 2, 17], [5, 1, 31]):
        rows, _ = replay(name, dtype, alone(reqs, lambda t: cut(t, sizes, tail=3)), roundup(max(len(t) for t in reqs.values())))
        compare(name, dtype, rows, reqs)


def mixed_steps(reqs, seed, max_live, sizes=(1, 2, 3, 16, 29, 64)):
    """Random steps with up to ``max_live`` live requests: portions of some beside single tokens of others, some
    requests left out of a step; a request that ended may come again under another name."""
    rng = random.Random(seed)
    waiting = list(reqs) + [r + "#2" for r in list(reqs)[:2]]
    rng.shuffle(waiting)
    live, steps, peak = {}, [], 0
    while waiting or live:
        while waiting and len(live) < max_live and rng.random() < 0.7:
            live[waiting.pop()] = 0
        if not live:
            continue
        entries, end = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.25:
                continue                                   # left out of this step
            toks = reqs[rid.split("#")[0]]
            at = live[rid]
            n = min(rng.choice(sizes), len(toks) - at)
            entries.append((rid, toks[at:at + n], range(n)))
            live[rid] = at + n
        peak = max(peak, sum(roundup(n) for n in live.values()))
        for rid in list(live):
            if live[rid] == len(reqs[rid.split("#")[0]]):
                end.append(rid)
                del live[rid]
        if entries:
            rng.shuffle(entries)
            steps.append((entries, end))
        elif end:
            steps[-1][1].extend(end)
    return steps, peak


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_mixed_batches_in_a_small_pool(name, dtype):
    """Unequal requests together against each alone (the plain implementation); the pool holds just what is live, so
    pages and slots are used again."""
    reqs = requests(name, LENGTHS[name] + (40, 101), seed=3)
    steps, peak = mixed_steps(reqs, seed=sum(map(ord, name)), max_live=3)
    rows, rp = replay(name, dtype, steps, peak, max_live=3)
    compare(name, dtype, rows, reqs)
    pools = [g.pool for g in rp.runner.manager.groups]
    assert all(p.reuse_count > 0 for p in pools), "no page was used again"
    assert all(p.num_free == p.num_pages for p in pools), "pages were lost"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batch_equals_each_alone(dtype):
    """The same positions computed in a batch of unequal requests and alone agree to rounding (bitwise in float32,
    where every sum has an order of its own)."""
    name = "d"
    reqs = requests(name, (50, 9, 120), seed=4)
    together = [([(r, t[:len(t) - 2], range(len(t) - 2)) for r, t in reqs.items()], []),
                ([(r, t[-2:-1], [0]) for r, t in reqs.items()], []), ([(r, t[-1:], [0]) for r, t in reqs.items()], list(reqs))]
    a, _ = replay(name, dtype, together, sum(roundup(len(t)) for t in reqs.values()))
    b, _ = replay(name, dtype, alone(reqs, lambda t: cut(t, [len(t)], tail=2)), 192)
    for key in a:
        if dtype == "float32":
            assert np.array_equal(a[key], b[key]), key
        elif not tainted(name, reqs[key[0]], key[1]):
            assert float(row_errors(a[key][None], b[key][None])[0]) <= BOUND[dtype]
    compare(name, dtype, a, reqs)


def draw_config(seed):
    """A configuration drawn at random: sizes, head counts, windows, constants and the order of layers all differ from
    the hand-picked ones, and include the values that make mechanisms vanish (a window of 1, one expert, one head)."""
    rng = random.Random(1000 + seed)
    width = rng.choice([24, 40, 64, 72, 90, 96, 100, 128])           # also widths that are no multiple of 8, or of 4
    kv_heads, vdim = rng.choice([1, 2, 3]), rng.choice([8, 16, 24, 32, 48, 64])      # the same in all layers that mix values
    layers = []
    for _ in range(rng.randint(1, 5)):
        per = rng.choice([1, 2, 4, 6])
        dim = rng.choice([8, 16, 24, 32, 64, 96])
        m = attention(kv_heads * per, kv_heads, dim, vdim, window=rng.choice([None, 1, 2, 7, 16, 17, 40, 100]),
                      temp=rng.choice([None, (0.9, 1), (0.3, 7), (1.5, 64)]), v_mix=rng.random() < 0.7,
                      scale=rng.choice([None, 0.31, 2.0 * dim ** -0.5]))
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "moe":
            E = rng.choice([1, 2, 5, 8, 16])
            f = moe(E, rng.randint(1, min(E, 4)), rng.choice([8, 12, 16, 40, 64]), rng.choice([0.5, 1.0, 7.0]))
        else:
            f = dense(rng.choice([8, 56, 128])) if kind == "dense" else None
        layers.append((m, f))
    return config(rng.choice([50, 131, 256]), width, layers, max_positions=rng.choice([256, 300]), eps=rng.choice([1e-5, 1e-6, 1e-3]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(seed, dtype):
    name = f"drawn{seed}"
    CONFIGS[name] = draw_config(seed)
    reqs = requests(name, (1, 2, 19, 66, 150, 37), seed=seed)
    steps, peak = mixed_steps(reqs, seed=seed, max_live=4, sizes=(1, 1, 2, 5, 16, 33, 64))
    rows, rp = replay(name, dtype, steps, peak, page_size=(8, 16, 32)[seed % 3], max_live=4)
    compare(name, dtype, rows, reqs)
    assert all(g.pool.num_free == g.pool.num_pages for g in rp.runner.manager.groups), "pages were lost"


def test_long_decoding_float32():
    name = "a"
    reqs = requests(name, (260,), seed=5)
    rows, _ = replay(name, "float32", alone(reqs, lambda t: cut(t, [4], tail=250)), 320)
    compare(name, "float32", rows, reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(dtype, graphs):
    """LLM.generate (scheduler, cache manager, sampler; recorded steps or not) against the plain argmax loop."""
    from pico_vllm_amd.engine.llm import LLM
    from pico_vllm_amd.sampling.params import SamplingParams
    name = "d"
    reqs = requests(name, (3, 41, 70, 12, 25), seed=6)
    new = 24
    llm = LLM(model=model_dir(name), dtype=dtype, max_seq_len=256, max_num_seqs=3, max_num_batched_tokens=64,
              num_gpu_blocks=40, use_cuda_graph=graphs)
    outs = llm.generate(list(reqs.values()), SamplingParams(max_new_tokens=new, ignore_eos=True))
    for toks, o in zip(reqs.values(), outs):
        assert len(o.token_ids) == new
        seq = list(toks)
        for tok in o.token_ids:
            lg = torch.from_numpy(plain_logits(name, seq)[-1])
            best = int(lg.argmax())
            if tok != best and not (dtype == "bfloat16" and tainted(name, seq, len(seq) - 1)):
                # two logits within rounding of each other may swap; then go on from the engine's token
                gap = float(lg[best] - lg[tok]) / float(lg.std())
                assert gap < (1e-4 if dtype == "float32" else 0.1), f"token {tok} instead of {best}, gap {gap}"
            seq.append(tok)
    llm.engine.runner.manager.check()


def test_command_line_generates_from_a_model_folder(capsys):
    """python -m pico_vllm_amd.run on a Lerazen folder: the architecture is found from config.json, sampling with a
    temperature and a seed gives the same tokens twice."""
    from pico_vllm_amd import run
    common = ["--model", model_dir("e"), "--prompt-ids", "5,17,3", "--prompt-ids", "9", "--max-new-tokens", "6", "--ignore-eos",
              "--num-gpu-blocks", "16", "--max-seq-len", "64"]
    assert run.main(common + ["--dtype", "float32"]) == 0
    lines = [l for l in capsys.readouterr().out.splitlines() if l.startswith("[")]
    assert len(lines) == 2 and all(len(l.split(")")[1].split()) == 6 for l in lines)
    seq = [5, 17, 3]
    for tok in map(int, lines[0].split(")")[1].split()):
        lg = plain_logits("e", seq)[-1]
        assert lg[tok] >= lg.max() - 1e-4 * lg.std()          # the plain argmax (or its equal within rounding)
        seq.append(tok)
    runs = []
    for _ in range(2):
        assert run.main(common + ["--dtype", "bfloat16", "--temperature", "0.9", "--top-p", "0.8", "--seed", "7"]) == 0
        runs.append([l for l in capsys.readouterr().out.splitlines() if l.startswith("[")])
    assert runs[0] == runs[1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_replay_program_in_a_subprocess(dtype):
    import json
    import os
    import subprocess
    import tempfile
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    name = "c"
    reqs = requests(name, (30, 9, 75), seed=8)
    steps, peak = mixed_steps(reqs, seed=5, max_live=2)
    lines = [json.dumps({"step": k, "entries": [{"id": r, "tokens": t, "want": list(w)} for r, t, w in entries], "end": list(end)})
             for k, (entries, end) in enumerate(steps)]
    with tempfile.TemporaryDirectory() as out:
        r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_dir(name), "--dtype", dtype, "--out", out,
                            "--max-tokens", str(peak)], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.split("\n") if l.startswith("done")] == [f"done {k}" for k in range(len(steps))]
        rows, fed = {}, {}
        for k, (entries, end) in enumerate(steps):
            wanted = sum(len(w) for _, _, w in entries)
            a = np.fromfile(os.path.join(out, f"{k}.f32"), dtype="<f4").reshape(wanted, -1)
            at = 0
            for rid, t, w in entries:
                for x in w:
                    rows[(rid, fed.get(rid, 0) + x)] = a[at]
                    at += 1
                fed[rid] = fed.get(rid, 0) + len(t)
            for rid in end:
                fed.pop(rid, None)
    compare(name, dtype, rows, reqs)


@pytest.mark.parametrize("rows", [1, 5, 33, 64, 300])
@pytest.mark.parametrize("sizes", [(96, 64), (1536, 1536), (200, 72)])
def test_projection_adds_into_the_stream(rows, sizes):
    """resid += x W^T + b: as the epilogue of the weight-streaming kernel for few rows, product and sum otherwise."""
    from pico_vllm_amd.ops.linear import Linear
    N, K = sizes
    g = torch.Generator().manual_seed(rows + N)
    w = (torch.randn(N, K, generator=g) * K ** -0.5).bfloat16()
    b = torch.randn(N, generator=g) * 0.1
    x = torch.randn(rows, K, generator=g).bfloat16()
    resid = torch.randn(rows, N, generator=g) * 3
    lin = Linear(w.to(DEV), b.to(DEV))
    got = resid.clone().to(DEV)
    assert lin.add_into(x.to(DEV), got) is got
    want = resid.double() + x.double() @ w.double().t() + b.double()
    assert torch.allclose(got.cpu().double(), want, atol=2e-2, rtol=2e-2)
    # few rows: only the product's own float32 rounding stands between the two
    if rows <= 64:
        assert float((got.cpu().double() - want).abs().max()) < 1e-4 * max(1.0, float(want.abs().max()))
