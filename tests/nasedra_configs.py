"""Small Nasedra configurations for the tests, and model folders made from them with random weights."""
import functools
import json
import os
import tempfile

import plain_nasedra as P


def rot(dims, base=10000.0, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def attention(heads, kv_heads, dim, vdim, window=None, keep_first=None, softcap=None, rotation=None, scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 0.9 * dim ** -0.5}
    if window is not None:
        m["mask"] = {"size": window}
        if keep_first is not None:
            m["mask"]["keep_first"] = keep_first
    if softcap is not None:
        m["softcap"] = softcap
    if rotation is not None:
        m["rot"] = rotation
    if kv_from is not None:
        m["kv_from"] = kv_from
    return ("attention", m)


def gla(heads, dim, vdim, tau):
    return ("gla", {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau})


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=None, scale=None, shared=None):
    r = {"experts": experts, "top": top}
    if identity is not None:
        r["identity"] = identity
    if scale is not None:
        r["scale"] = scale
    f = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared is not None:
        f["shared"] = {"ff": shared}
    return f


def config(vocab, width, layers, eps=1e-5, embed_scale=None):
    c = {"architecture": "Nasedra", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "layers": [{"type": t, "mixer": m, "mlp": f} for (t, m), f in layers]}
    if embed_scale is not None:
        c["embedding"] = {"scale": embed_scale}
    return c


YARN = (4.0, 64, 8.0, 1.0)

# name -> (config, inner size of the decay's matrices)
CONFIGS = {
    # sizes that are no multiples of 16 (the plain kernels in both precisions): a window shorter than a page with three
    # kept positions, part of the head rotated with scaled frequencies, a layer that reads the first layer's keys and
    # values through another mask, experts with two pass-through outputs and a shared expert
    "a": (config(97, 72, [
        (attention(3, 1, 24, 40, 12, 3, 30.0, rot(16, 10000.0, YARN)), dense(100)),
        (gla(2, 24, 40, 4.0), moe(5, 2, 32, identity=2, scale=1.25, shared=48)),
        (attention(3, 1, 24, 40, 20, 1, 30.0, rot(16, 10000.0, YARN), kv_from=0), dense(100)),
        (gla(2, 24, 40, 4.0), dense(64))], embed_scale=3.0), 5),
    # sizes the matrix-core kernels take: a window that spans pages with kept positions, a recurrent layer first, several
    # kv heads, the whole head rotated without scaling, three of seven router outputs, no cap on one layer, layers that
    # differ in their heads
    "b": (config(256, 128, [
        (gla(4, 64, 64, 12.0), moe(6, 3, 64, identity=1)),
        (attention(8, 2, 64, 32, 44, 5, None, rot(64, 300000.0)), dense(256)),
        (attention(4, 4, 32, 64, 100, 20, 15.0, rot(32, 1000.0, (8.0, 32, 4.0, 0.5))), moe(4, 1, 32, identity=2, scale=0.7, shared=64)),
        (attention(8, 2, 64, 32, 17, 0, 8.0, rot(64, 300000.0), kv_from=1), None)], eps=1e-6), 16),
    # no mask at all, as many kv heads as heads, no rotation on one layer, a recurrent layer whose key channels fill three
    # waves and whose values two workgroups, one expert a token, no embedding multiplier, a layer without feed-forward
    "c": (config(130, 96, [
        (attention(6, 6, 32, 48, None, None, 20.0, rot(8, 100.0)), moe(3, 1, 40)),
        (gla(1, 80, 100, 1.0), None),
        (attention(2, 1, 64, 16, 33, 2, None, None, scale=0.2), dense(64)),
        (gla(3, 16, 8, 30.0), moe(8, 4, 24, identity=3, scale=2.0, shared=16))]), 3),
    # a width that is no multiple of 8, a vocabulary that is odd, two heads on two kv heads, a window of one page with
    # more kept positions than a page holds, every router output chosen
    "d": (config(51, 44, [
        (gla(2, 12, 20, 2.0), dense(36)),
        (attention(2, 2, 12, 20, 16, 18, 25.0, rot(6, 200.0, (2.0, 16, 4.0, 1.0)), scale=0.31), moe(2, 3, 20, identity=1, scale=1.2, shared=12)),
        (attention(2, 2, 12, 20, 7, 0, None, rot(6, 200.0, (2.0, 16, 4.0, 1.0)), kv_from=1), dense(28))], eps=1e-6, embed_scale=2.5), 4),
}


@functools.lru_cache(maxsize=None)
def tensors_of(name, seed=0):
    cfg, rank = CONFIGS[name]
    return P.random_model(cfg, seed, rank=rank)


_dirs = {}


def write_model(cfg, tensors, prefix="nasedra_"):
    from pico_vllm_amd.weights.safetensors_io import write_safetensors
    d = tempfile.mkdtemp(prefix=prefix)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(d, "model.safetensors"), [(n, tuple(v.shape), v.dtype) for n, v in tensors.items()],
                      lambda n: tensors[n])
    return d


def model_dir(name, seed=0):
    """A folder with config.json and model.safetensors of configuration ``name``; made once a process."""
    key = (name, seed)
    if key not in _dirs:
        _dirs[key] = write_model(CONFIGS[name][0], tensors_of(name, seed), f"nasedra_{name}_")
    return _dirs[key]
