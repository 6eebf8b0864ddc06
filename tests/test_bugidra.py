"""Bugidra without a GPU: its configuration, its description as parts, its tensor names, random weights
as a folder, and the plain implementation's own invariants."""
import json

import numpy as np
import pytest
import torch

import plain_bugidra as pb
from bugidra_configs import CONFIGS, read_model, rot, write_model


def _spec(name):
    from flambeau_amd.registry import config_from_dict
    arch, cfg = config_from_dict(CONFIGS[name]["config"], "test")
    return arch, cfg, arch.build_spec(cfg)


def test_the_architecture_is_found_by_its_name():
    from flambeau_amd.registry import known_architectures
    assert {"Bugidra", "Kuvidra", "MistralForCausalLM"} <= set(known_architectures())
    arch, cfg, spec = _spec("A")
    assert arch.name == "Bugidra" and cfg.width == 48 and cfg.vocab_size == 97 and not spec.tied_head
    assert spec.embedding.kind == "scaled_token_embedding" and spec.embedding.params["scale"] == 5.5


def test_every_size_comes_from_the_file():
    _, cfg, _ = _spec("A")
    l0, l1, l2, l3, l4 = cfg.layers
    m = l0.mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.softcap, m.v_mix, m.rot.base, m.rot.dims) == (4, 2, 16, 24, 0.3, 20.0, True, 10000.0, 8)
    d = l1.mixer
    assert (l1.type, d.heads, d.kv_heads, d.dim, d.vdim, d.conv, l1.mlp.ff) == ("delta", 4, 2, 12, 20, 4, 56)
    s = l2.mixer.left.rot.scaling
    assert (s.factor, s.original, s.fast, s.slow) == (4.0, 64, 16.0, 2.0) and l2.mlp is None
    assert l2.mixer.right.decay == (0.9, 0.97, 0.995) and l2.mixer.right.rot.dims == 8
    assert l4.mixer.rot is None and l4.mixer.softcap is None and cfg.eps == 1e-5
    assert _spec("B")[1].embedding_scale == 1.0 and _spec("B")[1].layers[0].mixer.right.rot is None


@pytest.mark.parametrize("damage,text", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda c: c["layers"][0].update(type="conv"), "conv"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "moe"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "dims"),
    (lambda c: c["layers"][2]["mixer"]["right"].update(decay=[0.5, 0.5]), "decay"),
    (lambda c: c["layers"][1]["mixer"].update(conv=0), "conv"),
    (lambda c: c["layers"][0]["mixer"].update(softcap=-1.0), "softcap"),
    (lambda c: c["layers"][0]["mixer"].update(v_mix="yes"), "v_mix"),
    (lambda c: c["layers"][2]["mixer"]["left"]["rot"]["scaling"].pop("fast"), "fast"),
])
def test_a_bad_file_is_refused_with_the_key_s_name(damage, text):
    from flambeau_amd.config import ConfigError
    from flambeau_amd.registry import config_from_dict
    raw = json.loads(json.dumps(CONFIGS["A"]["config"]))
    damage(raw)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(raw, "test")


def test_parts_caches_and_names():
    """Which part every layer becomes, what it keeps per request, and under which names its tensors lie."""
    from flambeau_amd.models.decoder import DecoderModel
    from flambeau_amd.parts import JoinedCacheSpec, PagedKVSpec, StateSpec
    _, cfg, spec = _spec("A")
    model = DecoderModel(spec, rt=None)
    specs, shares = model.cache_entries()
    assert shares == [None] * 5
    assert specs[0] == PagedKVSpec(2, 24, 0) and specs[3] == PagedKVSpec(2, 24, 0) and specs[4] == PagedKVSpec(2, 24, 0)
    # the delta rule: a memory per head and the last three inputs of the convolution's channels
    assert specs[1] == StateSpec((4 * 12 * 20 + 3 * (2 * 2 * 12 + 4 * 20),), torch.float32)
    assert isinstance(specs[2], JoinedCacheSpec) and specs[2].paged == PagedKVSpec(3, 16, 0)
    assert specs[2].states == (None, StateSpec((3 * 8 * 12,), torch.float32))
    roles = [b.mixer.value_mix for b in model.blocks if hasattr(b.mixer, "value_mix")]
    assert roles == ["source", "blend", "blend"]
    assert model.blocks[2].ffn is None and "ffn_norm.weight" not in model.blocks[2].tensors()
    kinds = [c.__name__ for c in model.mixers_by_class()]
    assert kinds == ["NormedGQAAttention", "GatedDelta", "Retention"]              # the members of the pair, not the pair
    names = set(model.manifest())
    for n in ("embed", "head", "final.norm", "final.norm.alpha", "final.norm.b", "l0.norm1.alpha", "l0.mix.q.norm", "l0.mix.vmix",
              "l0.mix.g", "l1.mix.q.conv", "l1.mix.A_log", "l1.mix.dt_bias", "l1.mix.norm", "l1.mix.b", "l1.mix.a", "l2.mix.left.q",
              "l2.mix.left.out", "l2.mix.right.g", "l2.mix.right.out", "l3.mlp.gate", "l4.mix.vmix"):
        assert n in names, n
    assert "l2.norm2" not in names and "l2.mix.left.g" not in names
    man = model.manifest()
    assert man["l1.mix.q.conv"][2].shape == (2 * 12, 4) and man["l0.mix.vmix"][2].shape == () and man["l1.mix.norm"][2].shape == (20,)
    # a model of attention alone keeps no state, one blending layer alone is a source nobody reads
    d = DecoderModel(_spec("D")[2], rt=None)
    assert [b.mixer.value_mix for b in d.blocks] == [None, "source"]


def test_random_weights_as_a_folder(tmp_path):
    from flambeau_amd.models.decoder import DecoderModel
    from flambeau_amd.weights.loader import SafetensorsDir, check_against_manifest
    for name in CONFIGS:
        d = write_model(name, tmp_path / name, "bfloat16")
        src = SafetensorsDir(d)
        assert check_against_manifest(DecoderModel(_spec(name)[2], rt=None).manifest(), src) == []
        src.close()
        cfg, t = read_model(d)
        logits = pb.forward(cfg, t, [1, 2, 3, 4, 5])
        assert logits.shape == (5, cfg["vocab"]) and np.isfinite(logits).all() and np.abs(logits).max() > 0.05


def test_the_plain_implementation_is_causal_and_its_layers_matter(tmp_path):
    d = write_model("A", tmp_path / "A", "float32")
    cfg, t = read_model(d)
    toks = list(np.random.default_rng(1).integers(0, 97, 40))
    a, layers = pb.forward(cfg, t, toks, return_layers=True)
    b = pb.forward(cfg, t, toks[:25])
    assert np.allclose(a[:25], b, atol=1e-12)
    other = list(toks)
    other[0] = (other[0] + 1) % 97
    assert np.abs(pb.forward(cfg, t, other)[-1] - a[-1]).max() > 1e-6
    assert len(layers) == 5 and all(np.abs(layers[i + 1] - layers[i]).max() > 1e-3 for i in range(4))
    # every constant of a mixer changes the result
    for path, value in (("layers.0.mixer.softcap", 2.0), ("layers.0.mixer.scale", 0.6), ("layers.2.mixer.right.decay", [0.5, 0.5, 0.5]),
                        ("layers.2.mixer.left.rot.scaling.factor", 8.0), ("layers.3.mixer.rot.base", 30.0), ("embedding.scale", 2.0),
                        ("layers.0.mixer.v_mix", False)):
        c = json.loads(json.dumps(cfg))
        at = c
        keys = path.split(".")
        for k in keys[:-1]:
            at = at[int(k)] if k.isdigit() else at[k]
        at[keys[-1]] = value
        assert np.abs(pb.forward(c, t, toks)[-1] - a[-1]).max() > 1e-5, path


def test_the_recurrences_written_out_by_hand():
    """Two tokens of the delta rule and of retention against the sums written out."""
    rng = np.random.default_rng(0)
    W, D, Dv = 5, 3, 2
    h = rng.normal(size=(2, W))
    t = {"m." + k: rng.normal(size=s) for k, s in dict(q=(D, W), k=(D, W), v=(Dv, W), b=(1, W), a=(1, W), g=(Dv, W), o=(W, Dv)).items()}
    t.update({"m.q.conv": rng.normal(size=(D, 2)), "m.k.conv": rng.normal(size=(D, 2)), "m.v.conv": rng.normal(size=(Dv, 2)),
              "m.A_log": np.array([0.3]), "m.dt_bias": np.array([-0.2]), "m.norm": rng.normal(size=Dv)})
    got = pb.gated_delta(h, t, "m.", dict(heads=1, kv_heads=1, dim=D, vdim=Dv, conv=2), 1e-5)

    def conv(name):
        x = h @ t["m." + name].T
        w = t[f"m.{name}.conv"]
        return pb.silu(np.stack([x[0] * w[:, 1], x[1] * w[:, 1] + x[0] * w[:, 0]]))
    q, k, v = conv("q"), conv("k"), conv("v")
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) / np.sqrt(D)
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = 1 / (1 + np.exp(-(h @ t["m.b"].T)[:, 0]))
    g = np.exp(-np.exp(0.3) * np.log1p(np.exp((h @ t["m.a"].T)[:, 0] - 0.2)))
    S1 = np.outer(k[0], beta[0] * v[0])
    o1 = S1.T @ q[0]
    S2 = g[1] * S1
    S2 = S2 + np.outer(k[1], beta[1] * (v[1] - S2.T @ k[1]))
    o = np.stack([o1, S2.T @ q[1]])
    o = o / np.sqrt((o * o).mean(-1, keepdims=True) + 1e-5) * t["m.norm"] * pb.silu(h @ t["m.g"].T)
    assert np.allclose(got, o @ t["m.o"].T)
    # retention without rotation: o_1 = (decay k_0 v_0^T + k_1 v_1^T)^T q_1
    r = {"m." + k_: rng.normal(size=s) for k_, s in dict(q=(D, W), k=(D, W), v=(Dv, W), g=(Dv, W), o=(W, Dv)).items()}
    got = pb.retention(h, r, "m.", dict(heads=1, dim=D, vdim=Dv, decay=[0.75]), 1e-5)
    q, k, v = h @ r["m.q"].T, h @ r["m.k"].T / np.sqrt(D), h @ r["m.v"].T
    o = np.stack([np.outer(k[0], v[0]).T @ q[0], (0.75 * np.outer(k[0], v[0]) + np.outer(k[1], v[1])).T @ q[1]])
    o = o / np.sqrt((o * o).mean(-1, keepdims=True) + 1e-5) * pb.silu(h @ r["m.g"].T)
    assert np.allclose(got, o @ r["m.o"].T)


def test_rotations_written_out():
    x = np.arange(1.0, 9.0).reshape(1, 1, 8)
    r = rot(100.0, 4)
    a = 3 * np.array([1.0, 100.0 ** -0.5])
    half = pb.rotate(x, [3], r, "half")[0, 0]
    assert np.allclose(half[:4], [1 * np.cos(a[0]) - 3 * np.sin(a[0]), 2 * np.cos(a[1]) - 4 * np.sin(a[1]),
                                  3 * np.cos(a[0]) + 1 * np.sin(a[0]), 4 * np.cos(a[1]) + 2 * np.sin(a[1])])
    inter = pb.rotate(x, [3], r, "interleaved")[0, 0]
    assert np.allclose(inter[:4], [1 * np.cos(a[0]) - 2 * np.sin(a[0]), 2 * np.cos(a[0]) + 1 * np.sin(a[0]),
                                   3 * np.cos(a[1]) - 4 * np.sin(a[1]), 4 * np.cos(a[1]) + 3 * np.sin(a[1])])
    assert np.array_equal(half[4:], x[0, 0, 4:]) and np.array_equal(inter[4:], x[0, 0, 4:])


def test_a_stretched_ladder_on_either_rotation():
    """The frequencies' stretch is a key of a rotation, whichever mixer has it: the interleaved rotation of an
    attention layer and the retention's take it like the pair's left side."""
    from flambeau_amd.registry import config_from_dict
    raw = json.loads(json.dumps(CONFIGS["A"]["config"]))
    raw["layers"][0]["mixer"]["rot"]["scaling"] = {"factor": 2.0, "original": 32, "fast": 8.0, "slow": 1.0}
    raw["layers"][2]["mixer"]["right"]["rot"]["scaling"] = {"factor": 3.0, "original": 16, "fast": 4.0, "slow": 0.5}
    arch, cfg = config_from_dict(raw, "test")
    spec = arch.build_spec(cfg)
    first = spec.layers[0].block.params["mixer"].params["position"]
    assert first.kind == "rope_blended" and first.params["layout"] == "interleaved" and first.params["factor"] == 2.0
    right = spec.layers[2].block.params["mixer"].params["right"].params["position"]
    assert right.kind == "rope_blended" and right.params["layout"] == "half" and right.params["original"] == 16
    plain = spec.layers[3].block.params["mixer"].params["position"]
    assert plain.kind == "rope_interleaved" and plain.params["rotated_dims"] == 24
