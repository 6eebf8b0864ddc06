"""Small Bugidra configurations for the tests, and their random weights.

They differ from one another in every size and option, layer by layer: the order of the three kinds of
layers, head counts and groupings (also one key/value head, and as many as query heads), key and value
sizes that differ either way and are no multiples of 8, rotations over all and over a part of a head,
with and without the stretched ladder, caps, one, two and three layers that blend their values and
layers that do not, convolutions of one to four taps, decays near and far from one, layers without a
feed-forward, widths and vocabularies that are no multiples of 8."""
import json

import torch

from flambeau_amd.weights import SafetensorsFile, write_random_model, write_safetensors


def rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def att(heads, kv_heads, dim, vdim, scale, r=None, softcap=None, v_mix=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if r is not None:
        m["rot"] = r
    if softcap is not None:
        m["softcap"] = softcap
    if v_mix is not None:
        m["v_mix"] = v_mix
    return {"type": "attention", "mixer": m}


def par(left, right):
    return {"type": "parallel", "mixer": {"left": left["mixer"], "right": right}}


def ret(heads, dim, vdim, decay, r=None):
    m = dict(heads=heads, dim=dim, vdim=vdim, decay=decay)
    if r is not None:
        m["rot"] = r
    return m


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def model(vocab, width, eps, scale, layers):
    return {"architecture": "Bugidra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": [dict(l, mlp=m) for l, m in layers]}


CONFIGS = {
    # every kind of layer; three blending layers; fewer query/key heads than heads in the delta rule; values wider than keys
    "A": dict(config=model(97, 48, 1e-5, 5.5, [
        (att(4, 2, 16, 24, 0.3, rot(10000.0, 8), softcap=20.0, v_mix=True), dense(40)),
        (delta(4, 2, 12, 20, 4), dense(56)),
        (par(att(6, 3, 16, 8, 0.25, rot(5000.0, 16, (4.0, 64, 16.0, 2.0))), ret(3, 8, 12, [0.9, 0.97, 0.995], rot(100000.0, 8))), None),
        (att(2, 2, 24, 24, 0.2, rot(300.0, 24), softcap=5.0, v_mix=True), dense(24)),
        (att(8, 2, 8, 24, 0.4, None, v_mix=True), dense(32)),
    ]), seed=3, std=0.16, page_size=8),
    # starts with the pair side by side; a width and sizes that are no multiples of 8; one tap, two taps; no blending
    "B": dict(config=model(61, 36, 3e-4, 1.0, [
        (par(att(3, 1, 12, 20, 0.3, rot(777.0, 6)), ret(2, 20, 6, [0.5, 0.999])), dense(20)),
        (delta(3, 3, 6, 10, 1), None),
        (att(5, 5, 10, 6, 0.35, rot(50.0, 10)), dense(28)),
        (delta(2, 1, 20, 36, 2), dense(16)),
    ]), seed=11, std=0.2, page_size=16),
    # sizes in steps of 16 and 32, which in bfloat16 run on the matrix cores; more than 16 query heads per key/value head
    "C": dict(config=model(150, 64, 1e-5, 8.0, [
        (delta(4, 4, 32, 32, 3), dense(64)),
        (att(20, 1, 32, 32, 0.18, rot(10000.0, 16), softcap=30.0, v_mix=True), dense(96)),
        (par(att(4, 2, 64, 32, 0.12, rot(20000.0, 64, (8.0, 128, 4.0, 0.5))), ret(2, 64, 48, [0.99, 0.9999], rot(1e6, 32))), dense(64)),
        (att(20, 1, 32, 32, 0.18, rot(10000.0, 16), v_mix=True), None),
    ]), seed=21, std=0.12, page_size=16),
    # attention layers only: no mixer advances a state, so steps of single tokens replay captured graphs
    "D": dict(config=model(90, 40, 1e-6, 3.0, [
        (att(4, 2, 16, 16, 0.3, rot(1000.0, 16), softcap=10.0), dense(48)),
        (att(3, 3, 8, 12, 0.5, rot(99.0, 4), v_mix=True), dense(24)),
    ]), seed=41, std=0.15, page_size=16),
}

STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def sharpened(config, factor):
    """The configuration with every softmax mixer's score scale multiplied (queries and keys are normed, so
    scaling a projection would change nothing): softmax becomes peaked and single keys carry the output."""
    cfg = json.loads(json.dumps(config))
    for layer in cfg["layers"]:
        m = layer["mixer"]
        for part in ([m] if layer["type"] == "attention" else [m["left"]] if layer["type"] == "parallel" else []):
            part["scale"] *= factor
    return cfg


def write_model(name, out_dir, store="float32", sharpen=1.0, remember=False):
    """The folder of a configuration.  ``sharpen``: see ``sharpened``; ``remember`` makes the recurrent
    memories long (decays of the delta rule next to one: A_log far below zero; retention's decays of
    0.9999 and more)."""
    c = CONFIGS[name]
    config = sharpened(c["config"], sharpen) if sharpen != 1.0 else json.loads(json.dumps(c["config"]))
    if remember:
        for layer in config["layers"]:
            if layer["type"] == "parallel":
                right = layer["mixer"]["right"]
                right["decay"] = [1.0 - 1e-4 / (i + 1) for i in range(right["heads"])]
    d = write_random_model(config, out_dir, seed=c["seed"], std=c["std"], gain_std=0.1, store_dtype=STORE[store])
    (d / "config.json").write_text(json.dumps(config, indent=1))       # exactly the keys the design has
    if remember:
        f = SafetensorsFile(d / "model.safetensors")
        tensors = {}
        for n in f.names():
            t = f.read(n)
            if n.endswith(".A_log"):
                t = torch.full_like(t, -7.0)
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
