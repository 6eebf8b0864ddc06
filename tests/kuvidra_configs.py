"""Small Kuvidra configurations for the tests, and their random weights.

They differ from one another in every size and option, layer by layer: head counts, key and value
sizes that differ, latents narrower and wider than a wave, ranks that are no multiple of 8, one and
several experts per token (also all of them), experts with and without a shared one, layers without
a feed-forward, a looped stretch that starts at the first layer or later and runs one, two or three
times, with an mLSTM layer inside and outside it, and a model without a loop at all."""
import json

import numpy as np
import torch

from flambeau_amd.weights import SafetensorsFile, write_random_model, write_safetensors


def _att(heads, dim, vdim, q_rank, kv_rank, scale):
    return {"type": "latent_attention", "mixer": dict(heads=heads, dim=dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale)}


def _rec(heads, dim, vdim, cap):
    return {"type": "mlstm", "mixer": dict(heads=heads, dim=dim, vdim=vdim, gate_cap=cap)}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def _model(vocab, width, eps, layers, loop=None):
    cfg = {"architecture": "Kuvidra", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": [dict(l, mlp=m) for l, m in layers]}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


CONFIGS = {
    # a loop from the second layer on, three passes, an mLSTM layer inside it; values wider than 64
    "P": dict(config=_model(97, 48, 1e-5, [
        (_att(3, 8, 12, 20, 24, 1.1), _dense(40)),
        (_rec(2, 12, 20, 8.0), _moe(5, 2, 16, 24)),
        (_att(2, 16, 8, 12, 40, 0.8), _moe(3, 3, 8, None)),
        (_rec(1, 20, 70, 15.0), None),
        (_att(5, 8, 8, 8, 70, 0.6), _dense(24)),
    ], loop=(1, 3, 3)), seed=3, std=0.16, page_size=8),
    # no loop; a width and ranks that are no multiples of 8; one expert of two
    "Q": dict(config=_model(61, 36, 3e-4, [
        (_rec(3, 4, 6, 5.0), _dense(20)),
        (_att(4, 6, 10, 7, 9, 1.5), _moe(2, 1, 12, 10)),
        (_att(1, 24, 24, 16, 130, 0.4), None),
    ]), seed=11, std=0.2, page_size=16),
    # the whole model is the loop, once over; a single layer of each kind
    "R": dict(config=_model(130, 64, 1e-6, [
        (_att(4, 16, 16, 32, 32, 0.9), _moe(6, 4, 24, 40)),
        (_rec(4, 16, 16, 10.0), _dense(96)),
    ], loop=(0, 2, 1)), seed=21, std=0.12, page_size=16),
    # sizes in steps of 32 and 16, which in bfloat16 run on the matrix cores: more heads than a tile of 16, pages of 16 and 32
    "S": dict(config=_model(150, 64, 1e-5, [
        (_att(20, 32, 16, 48, 64, 0.5), _moe(4, 2, 32, 32)),
        (_rec(2, 32, 32, 10.0), _dense(64)),
        (_att(4, 64, 48, 32, 96, 0.3), None),
    ], loop=(0, 1, 2)), seed=31, std=0.15, page_size=16),
    # attention layers only: no mixer advances a state, so steps of single tokens replay captured graphs
    "T": dict(config=_model(90, 64, 1e-5, [
        (_att(4, 32, 16, 16, 32, 0.6), _moe(3, 1, 32, 16)),
        (_att(3, 8, 24, 12, 20, 0.9), _dense(48)),
    ], loop=(1, 2, 2)), seed=41, std=0.15, page_size=16),
}

STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def write_model(name, out_dir, store="float32", sharpen=1.0, forget_bias=None):
    """The folder of a configuration.  ``sharpen`` scales every attention layer's query expansion, so
    that softmax is peaked and a single key, near or far, carries the output; ``forget_bias`` replaces
    the forget gates' biases (a large one keeps old tokens in the memory for hundreds of steps)."""
    c = CONFIGS[name]
    d = write_random_model(c["config"], out_dir, seed=c["seed"], std=c["std"], gain_std=0.1, store_dtype=STORE[store])
    (d / "config.json").write_text(json.dumps(c["config"], indent=1))       # exactly the keys the design has
    if sharpen != 1.0 or forget_bias is not None:
        f = SafetensorsFile(d / "model.safetensors")
        tensors = {}
        for n in f.names():
            t = f.read(n)
            if n.endswith(".mix.uq"):
                t = (t.float() * sharpen).to(t.dtype)
            if forget_bias is not None and n.endswith(".mix.f.b"):
                t = torch.full_like(t, forget_bias)
            tensors[n] = t
        f.close()
        write_safetensors(d / "model.safetensors", tensors)
    return d


def read_model(model_dir):
    """``(config dictionary, {name: float64 array})`` as the plain implementation takes them."""
    cfg = json.loads((model_dir / "config.json").read_text())
    f = SafetensorsFile(model_dir / "model.safetensors")
    tensors = {n: f.read(n).to(torch.float64).numpy() for n in f.names()}
    f.close()
    return cfg, tensors
