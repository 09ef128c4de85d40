"""Small Lerazen configurations for the tests, and model folders made from them with random weights."""
import functools
import json
import os
import tempfile

import torch

import plain_lerazen as P


def attention(heads, kv_heads, dim, vdim, window=None, temp=None, v_mix=False, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
         "v_mix": v_mix}
    if window is not None:
        m["mask"] = {"size": window}
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def config(vocab, width, layers, max_positions=512, eps=1e-5):
    return {"architecture": "Lerazen", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": eps},
            "layers": [{"type": "attention", "mixer": m, "mlp": f} for m, f in layers]}


CONFIGS = {
    # every layer mixes values, a window shorter than a page, a temperature that changes every 8 positions,
    # a dense, a routed (two of eight) and a missing feed-forward
    "a": config(97, 64, [(attention(4, 2, 32, 16, 12, (0.7, 8), True), dense(80)),
                         (attention(4, 2, 32, 16, 12, (0.7, 8), True), moe(8, 2, 48, 1.5)),
                         (attention(4, 2, 32, 16, 12, (0.7, 8), True), None)]),
    # as many kv heads as heads, values larger than keys, a layer without window and temperature, value mixing that
    # starts at the second layer, three of five experts, windows that differ between layers
    "b": config(130, 96, [(attention(6, 6, 16, 32, None, None, False), moe(5, 3, 40, 0.5)),
                          (attention(6, 6, 16, 32, 33, (0.3, 5), True), dense(64)),
                          (attention(6, 6, 16, 32, 17, None, True), moe(5, 1, 40, 2.0)),
                          (attention(6, 6, 16, 32, None, (1.1, 16), True), dense(64))], eps=1e-6),
    # sizes that are no multiples of 16, one kv head, a window of 5, pages larger than the window
    "c": config(61, 72, [(attention(3, 1, 24, 40, 5, (0.5, 3), True), dense(100)),
                         (attention(3, 1, 24, 40, 64, (0.5, 3), True), moe(3, 2, 24, 1.0))]),
    # sizes the matrix-core kernels take (multiples of 32), a window that spans pages, many heads a group
    "d": config(256, 128, [(attention(8, 1, 64, 32, 44, (0.6, 16), True), dense(256)),
                           (attention(8, 1, 64, 32, 44, (0.6, 16), True), moe(12, 2, 64, 1.0)),
                           (attention(8, 2, 32, 64, 100, None, False), moe(4, 4, 32, 3.0))], max_positions=1024),
    # keys and values of one size in steps of 32 (prompt steps take another kernel), windowed and not, with and without
    # a temperature
    "e": config(200, 96, [(attention(6, 2, 32, 32, 24, (0.8, 10), True), dense(96)),
                          (attention(6, 2, 32, 32, None, None, True), moe(6, 2, 32, 1.5)),
                          (attention(4, 4, 64, 64, 70, (0.5, 64), False), None)], max_positions=600),
}


@functools.lru_cache(maxsize=None)
def tensors_of(name, seed=0):
    return P.random_model(CONFIGS[name], seed)


_dirs = {}


def model_dir(name, seed=0):
    """A folder with config.json and model.safetensors of configuration ``name``; made once a process."""
    from pico_vllm_amd.weights.safetensors_io import write_safetensors
    key = (name, seed)
    if key not in _dirs:
        d = tempfile.mkdtemp(prefix=f"lerazen_{name}_")
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump(CONFIGS[name], f)
        t = tensors_of(name, seed)
        write_safetensors(os.path.join(d, "model.safetensors"), [(n, tuple(v.shape), v.dtype) for n, v in t.items()],
                          lambda n: t[n])
        _dirs[key] = d
    return _dirs[key]
