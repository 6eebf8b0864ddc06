"""Kuvidra without a GPU: its configuration, its description as parts, its tensor names, random
weights as a folder, and the plain implementation's own invariants."""
import json

import numpy as np
import pytest
import torch

import plain_kuvidra as pk
from kuvidra_configs import CONFIGS, read_model, write_model


def _spec(name):
    from flambeau_amd.registry import config_from_dict
    arch, cfg = config_from_dict(CONFIGS[name]["config"], "test")
    return arch, cfg, arch.build_spec(cfg)


def test_the_architecture_is_found_by_its_name():
    from flambeau_amd.registry import known_architectures
    assert "Kuvidra" in known_architectures() and "MistralForCausalLM" in known_architectures()
    arch, cfg, spec = _spec("P")
    assert arch.name == "Kuvidra" and cfg.width == 48 and cfg.vocab_size == 97 and spec.tied_head


def test_every_size_comes_from_the_file():
    _, cfg, _ = _spec("P")
    l0, l1, l2, l3, _ = cfg.layers
    assert (l0.mixer.heads, l0.mixer.dim, l0.mixer.vdim, l0.mixer.q_rank, l0.mixer.kv_rank, l0.mixer.scale) == (3, 8, 12, 20, 24, 1.1)
    assert (l1.type, l1.mixer.gate_cap, l1.mlp.experts, l1.mlp.top, l1.mlp.expert_ff, l1.mlp.shared_ff) == ("mlstm", 8.0, 5, 2, 16, 24)
    assert l2.mlp.shared_ff is None and l3.mlp is None and l0.mlp.ff == 40
    assert (cfg.loop.start, cfg.loop.stop, cfg.loop.times) == (1, 3, 3) and cfg.eps == 1e-5
    assert _spec("Q")[1].loop is None


@pytest.mark.parametrize("damage,text", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0].update(type="conv"), "conv"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][1]["mlp"].update(kind="glu"), "glu"),
    (lambda c: c["loop"].update(stop=9), "stretch"),
    (lambda c: c["layers"][1]["mixer"].update(gate_cap=0), "gate_cap"),
    (lambda c: c["layers"][0]["mixer"].update(heads=2.5), "heads"),
])
def test_a_bad_file_is_refused_with_the_key_s_name(damage, text):
    from flambeau_amd.config import ConfigError
    from flambeau_amd.registry import config_from_dict
    raw = json.loads(json.dumps(CONFIGS["P"]["config"]))
    damage(raw)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(raw, "test")


def test_run_order_and_caches():
    """The looped stretch runs ``times`` times behind a re-entry each; every run has a cache of its own
    kind; the plain implementation walks the same order."""
    from flambeau_amd.models.decoder import DecoderModel
    from flambeau_amd.parts import PagedRowSpec, StateSpec
    _, cfg, spec = _spec("P")
    model = DecoderModel(spec, rt=None)
    re = len(cfg.layers)
    assert [e.layer for e in spec.run_order] == [0, re, 1, 2, re, 1, 2, re, 1, 2, 3, 4]
    assert [model._visits[i] for i, e in enumerate(spec.run_order) if e.layer == re] == [0, 1, 2]
    assert [l for l, _, _ in pk.run_order(CONFIGS["P"]["config"])] == [e.layer for e in spec.run_order if e.layer != re]
    specs, shares = model.cache_entries()
    assert shares == [None] * len(specs)
    kinds = [type(s).__name__ if s is not None else None for s in specs]
    assert kinds == ["PagedRowSpec", None, "StateSpec", "PagedRowSpec", None, "StateSpec", "PagedRowSpec", None, "StateSpec",
                     "PagedRowSpec", "StateSpec", "PagedRowSpec"]
    assert specs[0] == PagedRowSpec(24) and specs[3] == PagedRowSpec(40) and isinstance(specs[10], StateSpec)
    assert spec.keeps_embedding and not _spec("Q")[2].keeps_embedding
    assert [e.layer for e in _spec("R")[2].run_order] == [2, 0, 1]


def test_tensor_names_and_random_weights_round_trip(tmp_path):
    from flambeau_amd.models.decoder import DecoderModel
    _, _, spec = _spec("P")
    names = set(DecoderModel(spec, rt=None).manifest())
    assert {"embed", "final.norm", "loop.in", "loop.step", "l0.norm1", "l0.mix.dq", "l0.mix.dq.norm", "l0.mix.uk", "l0.mix.g",
            "l0.mlp.up", "l1.mix.i.b", "l1.mix.f", "l1.mix.norm", "l1.mlp.router", "l1.mlp.e4.down", "l1.mlp.shared.sg",
            "l2.mlp.e2.gate"} <= names
    assert "l2.mlp.shared.sg" not in names and not any(n.startswith("l3.mlp") for n in names)
    d = write_model("P", tmp_path / "m", "bfloat16")
    cfg, t = read_model(d)
    assert set(t) == names and cfg == CONFIGS["P"]["config"]
    assert t["loop.step"].shape == (3, 48) and t["l1.mlp.shared.sg"].shape == (1, 48) and t["l3.mix.v"].shape == (70, 48)
    logits = pk.forward(cfg, t, [5, 1, 96, 0])
    assert logits.shape == (4, 97) and np.isfinite(logits).all()


def test_plain_implementation_is_causal_and_cut_free():
    """A later token changes nothing earlier, and the mLSTM walk gives the same numbers whether the
    state is carried by hand or the sequence is run whole."""
    rng = np.random.default_rng(0)
    W, T = 24, 9
    mixer = dict(heads=2, dim=4, vdim=6, gate_cap=7.0)
    t = {"m.q": rng.normal(size=(8, W)), "m.k": rng.normal(size=(8, W)), "m.v": rng.normal(size=(12, W)),
         "m.g": rng.normal(size=(12, W)), "m.o": rng.normal(size=(W, 12)), "m.norm": rng.normal(size=12),
         "m.i": rng.normal(size=(2, W)), "m.i.b": rng.normal(size=2), "m.f": rng.normal(size=(2, W)), "m.f.b": rng.normal(size=2)}
    h = rng.normal(size=(T, W))
    whole = pk.mlstm(h, t, "m.", mixer, 1e-5)
    assert np.allclose(pk.mlstm(h[:5], t, "m.", mixer, 1e-5), whole[:5], atol=1e-12)
    att = dict(heads=2, dim=4, vdim=3, q_rank=5, kv_rank=6, scale=0.7)
    a = {"a.dq": rng.normal(size=(5, W)), "a.dq.norm": rng.normal(size=5), "a.uq": rng.normal(size=(8, 5)),
         "a.dkv": rng.normal(size=(6, W)), "a.dkv.norm": rng.normal(size=6), "a.uk": rng.normal(size=(8, 6)),
         "a.uv": rng.normal(size=(6, 6)), "a.g": rng.normal(size=(2, W)), "a.o": rng.normal(size=(W, 6))}
    full = pk.latent_attention(h, a, "a.", att, 1e-5)
    assert np.allclose(pk.latent_attention(h[:4], a, "a.", att, 1e-5), full[:4], atol=1e-12)
    # the first token sees itself alone: softmax of one score is 1 whatever the score
    c = pk.rms_norm(h[:1] @ a["a.dkv"].T, a["a.dkv.norm"], 1e-5)
    v = (c @ a["a.uv"].T).reshape(1, 2, 3) * pk.sigmoid(h[:1] @ a["a.g"].T)[:, :, None]
    assert np.allclose(full[0], v.reshape(1, 6) @ a["a.o"].T)


def test_routed_experts_plain():
    """top = experts with every score taken as it is equals the sum over all experts; the weight
    multiplies the input, which is not the same as multiplying the output."""
    rng = np.random.default_rng(1)
    W, F, E = 10, 6, 3
    t = {"f.router": rng.normal(size=(E, W))}
    for e in range(E):
        t.update({f"f.e{e}.gate": rng.normal(size=(F, W)), f"f.e{e}.up": rng.normal(size=(F, W)), f"f.e{e}.down": rng.normal(size=(W, F))})
    h = rng.normal(size=(4, W))
    s = pk.sigmoid(h @ t["f.router"].T)
    allof = pk.moe_ff(h, t, "f.", {"router": {"experts": E, "top": E}})
    want = sum(pk.gated_expert(s[:, e:e + 1] * h, t, f"f.e{e}.") for e in range(E))
    assert np.allclose(allof, want)
    on_output = sum(s[:, e:e + 1] * pk.gated_expert(h, t, f"f.e{e}.") for e in range(E))
    assert np.abs(on_output - want).max() > 1e-3
    one = pk.moe_ff(h, t, "f.", {"router": {"experts": E, "top": 1}})
    best = s.argmax(axis=1)
    assert np.allclose(one[2], pk.gated_expert(s[2, best[2]] * h[2:3], t, f"f.e{best[2]}.")[0])


def test_work_lists_of_the_attention_kernels():
    """The blocks of the kernel that shares its keys cover every (token, group of 16 heads) once, hold at most four
    waves and never cross a request; the number of parts the keys are dealt into is a power of two that follows
    the rows and the longest context."""
    from flambeau_amd.kernels.latent_attention import key_splits, shared_tiles
    from flambeau_amd.parts import HostBatch
    batch = HostBatch([0, 7, 8, 21], [7, 1, 13, 2], [0, 99, 5, 0], [0, 1, 2, 3], 23, 0)
    for groups in (1, 2, 3, 4, 5, 9):
        tiles = shared_tiles(batch, groups)
        seen = set()
        for t0, nt, g0, ng in tiles.tolist():
            assert 1 <= nt * ng <= 4
            owner = [s for s, (q0, ql) in enumerate(zip(batch.q_starts, batch.q_lens)) if q0 <= t0 < q0 + ql]
            assert len(owner) == 1 and t0 + nt <= batch.q_starts[owner[0]] + batch.q_lens[owner[0]]
            for t in range(t0, t0 + nt):
                for g in range(g0, g0 + ng):
                    assert (t, g) not in seen
                    seen.add((t, g))
        assert seen == {(t, g) for t in range(23) for g in range(groups)}
    one = HostBatch([0], [1], [4000], [0], 1, 0)
    assert key_splits(one, 32) == 32 and key_splits(one, 8) == 32          # 4,001 keys: 62 chunks, the next power of two below
    assert key_splits(HostBatch([0], [1], [100], [0], 1, 0), 8) == 1
    assert key_splits(HostBatch([0], [2048], [0], [0], 2048, 0), 32) == 1
    many = HostBatch(list(range(64)), [1] * 64, [3000] * 64, list(range(64)), 64, 0)
    assert key_splits(many, 32) == 8
