"""Bugidra on the GPU against the plain implementation: every mechanism alone, the layers one by one,
and whole models in every cutting (whole prompts, single tokens, portions down to two tokens, mixed
batches over a small poisoned pool whose pages and slots are used again), in 32-bit and in bfloat16,
at sizes of the tests' own."""
import json

import numpy as np
import pytest
import torch

import plain_bugidra as pb
import replay_helpers as rh
from bugidra_configs import CONFIGS, read_model, rot, sharpened, write_model
from test_kuvidra_gpu import close, make_rt, make_step

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("bugidra")
    out = {}
    for name in CONFIGS:
        for store in DTYPES:
            out[(name, store)] = write_model(name, base / f"{name}-{store}", store)
    for store in DTYPES:          # (weights are stored in the dtype they are run in: the plain side reads the same numbers)
        out[("sharp", store)] = write_model("A", base / f"A-sharp-{store}", store, sharpen=8.0)
        out[("memory", store)] = write_model("A", base / f"A-memory-{store}", store, remember=True)
    return out


_refs = {}


def reference(d, reqs):
    out = {}
    cfg = t = None
    for rid, toks in reqs.items():
        key = (str(d), tuple(toks))
        if key not in _refs:
            if cfg is None:
                cfg, t = read_model(d)
            _refs[key] = pb.forward(cfg, t, toks)
        out[rid] = _refs[key]
    return out


def runner_for(d, dtype, n_pages, page_size, max_tokens=512, slots=4, poison=True, **kw):
    from flambeau_amd.engine import ModelRunner, load_model
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=max_tokens)
    runner = ModelRunner(model, n_pages=n_pages, page_size=page_size, max_slots=slots, max_seq_len=max_tokens, **kw)
    if poison:
        runner.storage.fill(float("nan"))
    return runner


# ---------------------------------------------------------------- each mechanism alone
# local tensor names of the parts -> the design's names (what the plain functions read)
RENAMES = [("q_norm.weight", "q.norm"), ("k_norm.weight", "k.norm"), ("value_mix.weight", "vmix"), ("q_conv.weight", "q.conv"),
           ("k_conv.weight", "k.conv"), ("v_conv.weight", "v.conv"), ("left_out.weight", "left.out"), ("right_out.weight", "right.out"),
           ("norm.weight", "norm"), (".weight", ""), (".bias", ".b")]


def plain_name(name):
    for a, b in RENAMES:
        if name.endswith(a):
            return name[:len(name) - len(a)] + b
    return name


def bound_part(registry, spec, dtype, rt, seed, scale=0.3, prefix="m.", fix=None):
    """A part with random weights (rounded to the compute dtype) and the same numbers for the plain side."""
    part = registry.create(spec)
    g = torch.Generator().manual_seed(seed)
    w, plain = {}, {}
    for k, ts in part.tensors().items():
        v = torch.randn(tuple(ts.shape), generator=g) * scale
        if ts.role == "vector32" and (k.endswith("norm.weight") or k.endswith("out.weight")):
            v = 1 + v
        if k.endswith("value_mix.weight"):
            v = v.abs().clamp(0.1, 0.9)
        if fix and k in fix:
            v = fix[k](v)
        v = v.to(TORCH[dtype])
        w[k] = rt.to_device(v, ts.role)
        plain[plain_name(prefix + k)] = v.double().numpy()
    part.bind(w, rt)
    return part, plain


def run_mixer(mixer, rt, x, cuts, page_size=8, n_pages=40, before=None):
    """The mixer over ``x`` cut into steps, one request in slot 2 over shuffled pages; ``before(step)`` runs
    ahead of every step (what an earlier layer would have left)."""
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.parts import Product
    store = CacheStorage([mixer.cache_spec()], [None], rt.device, rt.dtype, n_pages=n_pages, page_size=page_size, max_slots=3)
    for p in store.pools:
        p.fill_(float("nan"))
    for st in store.states.values():
        st[:2] = float("nan")                                 # other requests' records
    members = getattr(mixer, "mixers", lambda: [mixer])()
    got, at = [], 0
    for k in cuts:
        step = make_step([(at, k)], page_size, n_pages, slots=[2], seed=1)
        if not store.pools:
            step.block_tables = []
        for m in members:
            if hasattr(m, "step_metadata_for"):                # the work lists the step function would upload
                step.extra.update({name: torch.tensor(arr, dtype=torch.int32, device=DEV)
                                   for name, arr in type(m).step_metadata_for(step.host, [m]).items()})
        if before is not None:
            before(step, at, k)
        r = mixer.forward(x[at:at + k].to(DEV).contiguous(), step, store.entries[0])
        r = r.compute(rt) if isinstance(r, Product) else r
        got.append(r.double().cpu().numpy())
        at += k
    return np.concatenate(got)


CUTS = ([90], [40, 5, 1, 1, 2, 20, 2, 6, 1, 12], [1] * 20 + [70])
TOL = {"float32": 3e-5, "bfloat16": 3e-2}


def _x(n, W, dtype, seed):
    return torch.randn(n, W, generator=torch.Generator().manual_seed(seed)).to(TORCH[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
def test_dynamic_tanh_and_scaled_embedding(dtype):
    from flambeau_amd.parts import EMBEDDINGS, NORMS, PartSpec
    rt = make_rt(dtype)
    W, n = 52, 37
    norm, plain = bound_part(NORMS, PartSpec("dynamic_tanh", dict(hidden_size=W)), dtype, rt, seed=1, prefix="n.")
    x = torch.randn(n, W, generator=torch.Generator().manual_seed(2)) * 3
    d = torch.randn(n, W, generator=torch.Generator().manual_seed(3))
    out = torch.empty(n, W, dtype=TORCH[dtype], device=DEV)
    xs = x.to(DEV).contiguous()
    norm.forward(xs, out, delta=d.to(DEV), store_sum=True)
    want = pb.dynamic_tanh((x + d).double().numpy(), plain, "n")
    assert np.abs(out.double().cpu().numpy() - want).max() < (2e-6 if dtype == "float32" else 1e-2) * np.abs(want).max()
    assert torch.equal(xs.cpu(), x + d)                         # the sum went back into the stream
    rows = torch.tensor([5, 0, 36], dtype=torch.int32, device=DEV)
    picked = torch.empty(3, W, dtype=TORCH[dtype], device=DEV)
    norm.forward(xs, picked, rows=rows)
    assert torch.equal(picked, out[rows.long()])
    emb = EMBEDDINGS.create(PartSpec("scaled_token_embedding", dict(vocab_size=11, hidden_size=W, scale=7.25)))
    table = torch.randn(11, W, generator=torch.Generator().manual_seed(4)).to(TORCH[dtype])
    emb.bind({"weight": table.to(DEV)}, rt)
    toks = torch.tensor([3, 10, 0, 3], dtype=torch.int32, device=DEV)
    got = emb.forward(toks, torch.empty(4, W, dtype=torch.float32, device=DEV))
    assert torch.equal(got.cpu(), table[toks.cpu().long()].float() * 7.25)


@pytest.mark.parametrize("n,K,H", [(1, 256, 128), (8, 512, 192), (16, 64, 4096), (40, 256, 128), (100, 256, 128), (300, 1024, 512), (700, 128, 96), (512, 512, 2048)])
def test_a_product_that_norms_in_its_epilogue(n, K, H):
    """The product that adds to the stream and applies Dynamic Tanh before it stores (few rows: the skinny
    kernel, many: the tiled one) against product, addition and norm apart."""
    from flambeau_amd.kernels import ops, tuned
    from flambeau_amd.parts import NORMS, PartSpec, Product, ResidualStream
    rt = make_rt("bfloat16", max_tokens=1024)
    norm, plain = bound_part(NORMS, PartSpec("dynamic_tanh", dict(hidden_size=H)), "bfloat16", rt, seed=n, prefix="n.")
    gen = torch.Generator().manual_seed(K)
    x = (torch.randn(n, K, generator=gen) * 0.5).to(torch.bfloat16).to(DEV)
    w = (torch.randn(H, K, generator=gen) * 0.1).to(torch.bfloat16).to(DEV)
    resid0 = torch.randn(n, H, generator=gen).to(DEV)
    weight = rt.prepare_weight(w)
    resid = resid0.clone()
    fused = tuned.gemm_add_dyt(rt, x, weight, resid, norm.alpha, norm.weight, norm.bias)
    want_resid = resid0.double() + x.double() @ w.double().T
    if fused is None:
        # a shape whose K the tiled product splits, or rows between the two kernels: product and norm run apart
        assert 16 < n <= 64 or tuned.gemm_tiled_splits(n, H, K) > 1
        stream = ResidualStream(resid0.clone(), rt)
        stream.push(Product(x, weight))
        fused, resid = stream.normed(norm, lazy=True), stream.resid
    assert (resid.double() - want_resid).abs().max().item() < 2e-4 * want_resid.abs().max().item()
    want = pb.dynamic_tanh(want_resid.cpu().numpy(), plain, "n")
    assert np.abs(fused.double().cpu().numpy() - want).max() < 1e-2 * np.abs(want).max()
    # and through the stream, as a block does it
    stream = ResidualStream(resid0.clone(), rt)
    stream.push(Product(x, weight))
    via = stream.normed(norm, lazy=True).clone()
    assert stream.pending is None and torch.equal(via, fused) and torch.equal(stream.resid, resid)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W,F", [(40, 24), (36, 50), (64, 128)])
def test_gated_feed_forward(dtype, W, F):
    from flambeau_amd.parts import FEED_FORWARDS, PartSpec, Product
    rt = make_rt(dtype)
    part, plain = bound_part(FEED_FORWARDS, PartSpec("gated_mlp", dict(hidden_size=W, intermediate_size=F, activation="gelu_tanh")),
                             dtype, rt, seed=F)
    x = _x(70, W, dtype, 5) * 2
    got = part.forward(x.to(DEV), None)
    got = got.compute(rt) if isinstance(got, Product) else got
    want = pb.feed_forward(x.double().numpy(), plain, "m.")
    assert np.abs(got.double().cpu().numpy() - want).max() < TOL[dtype] * np.abs(want).max()


ATT_SHAPES = [
    # H, G, D, Dv, rotated dims, cap
    (4, 2, 16, 24, 8, 20.0), (3, 3, 10, 6, 10, None), (20, 1, 32, 32, 16, 3.0), (2, 1, 72, 40, 0, None), (8, 4, 64, 48, 64, 50.0),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,rd,cap", ATT_SHAPES)
def test_gated_attention_alone(dtype, H, G, D, Dv, rd, cap):
    """Norm over the whole projection, interleaved rotation, capped scores, blended values, sigmoid gate:
    as the layer whose values are the source and as a layer that blends with them."""
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps, scale = 40, 90, 2e-5, 0.9
    position = PartSpec("rope_interleaved", dict(head_dim=D, theta=500.0, rotated_dims=rd)) if rd else PartSpec("none", {})
    common = dict(hidden_size=W, n_heads=H, n_kv_heads=G, head_dim=D, value_dim=Dv, scale=scale, position=position,
                  qk_norm="projection", eps=eps, softcap=cap, gate="sigmoid", value_mix_key="vm")
    x = _x(n, W, dtype, 5)
    cfg = dict(heads=H, kv_heads=G, dim=D, vdim=Dv, scale=scale, softcap=cap, v_mix=True)
    if rd:
        cfg["rot"] = rot(500.0, rd)
    first = torch.randn(n, G * Dv, generator=torch.Generator().manual_seed(9))
    for role in ("source", "blend"):
        mixer, plain = bound_part(MIXERS, PartSpec("normed_gqa_attention", dict(common, value_mix=role)), dtype, rt, seed=H + D)
        shared = {} if role == "source" else {"v_first": first.double().numpy().reshape(n, G, Dv)}
        want = pb.attention_mixer(x.double().numpy(), plain, "m.", cfg, eps, shared)

        def before(step, at, k):
            if role == "blend":
                step.scratch["vm"] = first[at:at + k].to(DEV).contiguous()
        for cuts in CUTS:
            got = run_mixer(mixer, rt, x, cuts, before=before)
            assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), (role, cuts)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,rd,scaling", [(6, 3, 16, 8, 16, (4.0, 64, 16.0, 2.0)), (3, 1, 12, 20, 6, None),
                                                  (8, 4, 64, 48, 64, (2.0, 32, 8.0, 1.0)), (4, 4, 32, 32, 32, (16.0, 20, 3.0, 0.2))])
def test_rotated_attention_alone(dtype, H, G, D, Dv, rd, scaling):
    """Split-half rotation with the stretched ladder, every head of q and k divided by its root mean square."""
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps, scale = 40, 90, 1e-5, 0.8
    if scaling:
        position = PartSpec("rope_blended", dict(head_dim=D, theta=3000.0, rotated_dims=rd, factor=scaling[0], original=scaling[1],
                                                 fast=scaling[2], slow=scaling[3]))
    else:
        position = PartSpec("rope_neox", dict(head_dim=D, theta=3000.0, rotated_dims=rd))
    mixer, plain = bound_part(MIXERS, PartSpec("normed_gqa_attention", dict(
        hidden_size=W, n_heads=H, n_kv_heads=G, head_dim=D, value_dim=Dv, scale=scale, position=position, qk_norm="head", eps=eps)),
        dtype, rt, seed=D)
    x = _x(n, W, dtype, 6)
    want = pb.rotated_attention(x.double().numpy(), plain, "m.", dict(heads=H, kv_heads=G, dim=D, vdim=Dv, scale=scale,
                                                                      rot=rot(3000.0, rd, scaling)), eps)
    for cuts in CUTS:
        got = run_mixer(mixer, rt, x, cuts)
        assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), cuts


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,Dv,window", [(16, 24, 13), (64, 64, 70), (32, 16, 64), (24, 8, 1)])
def test_attention_with_a_window(dtype, D, Dv, window):
    """``window`` keys, the query's own included (no model of the package sets it for this mixer yet), with the
    stretched ladder in the interleaved layout: against the formula written out, whole and in portions that
    cross the window's edge and the kernels' chunks of 64 keys."""
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps, H, G, scale, cap = 40, 150, 1e-5, 4, 2, 0.7, 8.0
    scaling = (4.0, 32, 8.0, 1.0)
    position = PartSpec("rope_blended", dict(head_dim=D, theta=900.0, rotated_dims=8, factor=scaling[0], original=scaling[1],
                                             fast=scaling[2], slow=scaling[3], layout="interleaved"))
    mixer, plain = bound_part(MIXERS, PartSpec("normed_gqa_attention", dict(
        hidden_size=W, n_heads=H, n_kv_heads=G, head_dim=D, value_dim=Dv, scale=scale, position=position, qk_norm="projection",
        eps=eps, softcap=cap, gate="silu", window=window)), dtype, rt, seed=D)
    assert mixer.cache_spec().window == window
    x = _x(n, W, dtype, 8)
    h = x.double().numpy()
    r = rot(900.0, 8, scaling)
    q = pb.rotate(pb.rms_norm(h @ plain["m.q"].T, plain["m.q.norm"], eps).reshape(n, H, D), np.arange(n), r, "interleaved")
    k = pb.rotate(pb.rms_norm(h @ plain["m.k"].T, plain["m.k.norm"], eps).reshape(n, G, D), np.arange(n), r, "interleaved")
    v = (h @ plain["m.v"].T).reshape(n, G, Dv)
    want = np.zeros((n, H, Dv))
    for i in range(n):
        lo = max(0, i - window + 1)
        for a in range(H):
            s = cap * np.tanh(k[lo:i + 1, a // (H // G)] @ q[i, a] * scale / cap)
            p = np.exp(s - s.max())
            want[i, a] = (p / p.sum()) @ v[lo:i + 1, a // (H // G)]
    want = (want.reshape(n, H * Dv) * pb.silu(h @ plain["m.g"].T)) @ plain["m.o"].T
    for cuts in ([150], [60, 4, 1, 1, 70, 2, 12], [1] * 30 + [120]):
        got = run_mixer(mixer, rt, x, cuts, n_pages=60)
        assert np.abs(got - want).max() < TOL[dtype] * np.abs(want).max(), cuts


def test_the_stretched_ladder_written_out():
    """The frequencies of one small case by hand: dims 8, base 16, original 16, factor 4, fast 2, slow 0.5."""
    import math
    from flambeau_amd.parts.rope import blended_frequencies
    f, mag = blended_frequencies(8, 16.0, 4.0, 16, 2.0, 0.5)
    turn = lambda n: 8 * math.log(16 / (2 * math.pi * n)) / (2 * math.log(16.0))
    lo, hi = max(math.floor(turn(2.0)), 0), min(math.ceil(turn(0.5)), 7)
    assert (lo, hi) == (0, 3)
    plain = [16.0 ** (-2 * i / 8) for i in range(4)]
    assert np.allclose(f, [plain[0], plain[1] * (2 / 3 + 1 / 12), plain[2] * (1 / 3 + 1 / 6), plain[3] / 4])
    assert mag == 0.1 * math.log(4.0) + 1
    g, _ = pb.rotary_frequencies(rot(16.0, 8, (4.0, 16, 2.0, 0.5)))
    assert np.allclose(f, g)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv,rd,decay", [(3, 8, 12, 8, [0.9, 0.97, 0.995]), (2, 20, 6, 0, [0.5, 0.999]), (1, 100, 33, 64, [0.99]),
                                             (2, 64, 48, 32, [1.0, 0.25])])
def test_retention_alone(dtype, H, D, Dv, rd, decay):
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps = 40, 90, 1e-5
    position = PartSpec("rope_neox", dict(head_dim=D, theta=1e4, rotated_dims=rd)) if rd else PartSpec("none", {})
    mixer, plain = bound_part(MIXERS, PartSpec("retention", dict(hidden_size=W, n_heads=H, head_dim=D, value_dim=Dv, decay=decay,
                                                                  position=position, eps=eps)), dtype, rt, seed=D)
    x = _x(n, W, dtype, 7)
    cfg = dict(heads=H, dim=D, vdim=Dv, decay=decay)
    if rd:
        cfg["rot"] = rot(1e4, rd)
    want = pb.retention(x.double().numpy(), plain, "m.", cfg, eps)
    results = [run_mixer(mixer, rt, x, cuts) for cuts in CUTS]
    for got in results:
        assert np.abs(got - want).max() < (3e-5 if dtype == "float32" else 4e-2) * np.abs(want).max()
    if dtype == "float32":                                   # the walk is the recurrence: no bit depends on the cutting
        assert np.array_equal(results[0], results[1]) and np.array_equal(results[0], results[2])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,taps", [(4, 2, 12, 20, 4), (3, 3, 6, 10, 1), (2, 1, 20, 36, 2), (4, 4, 64, 32, 3), (1, 1, 130, 17, 5)])
def test_gated_delta_rule_alone(dtype, H, G, D, Dv, taps):
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps = 40, 90, 1e-5
    fix = {"A_log": lambda v: v * 3 - 1.0, "dt_bias": lambda v: v * 3}
    mixer, plain = bound_part(MIXERS, PartSpec("gated_delta", dict(hidden_size=W, n_heads=H, n_qk_heads=G, head_dim=D, value_dim=Dv,
                                                                    conv_taps=taps, eps=eps)), dtype, rt, seed=D, fix=fix)
    x = _x(n, W, dtype, 8)
    want = pb.gated_delta(x.double().numpy(), plain, "m.", dict(heads=H, kv_heads=G, dim=D, vdim=Dv, conv=taps), eps)
    results = [run_mixer(mixer, rt, x, cuts) for cuts in CUTS]
    for got in results:
        assert np.abs(got - want).max() < (5e-5 if dtype == "float32" else 5e-2) * np.abs(want).max()
    if dtype == "float32":
        assert np.array_equal(results[0], results[1]) and np.array_equal(results[0], results[2])


@pytest.mark.parametrize("dtype", DTYPES)
def test_two_mixers_side_by_side(dtype):
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps = 40, 90, 1e-4
    left = dict(heads=6, kv_heads=3, dim=16, vdim=8, scale=0.5, rot=rot(5000.0, 16, (4.0, 64, 16.0, 2.0)))
    right = dict(heads=3, dim=8, vdim=12, decay=[0.9, 0.97, 0.995], rot=rot(1e5, 8))
    spec = PartSpec("side_by_side", dict(hidden_size=W, eps=eps, left=PartSpec("normed_gqa_attention", dict(
        hidden_size=W, n_heads=6, n_kv_heads=3, head_dim=16, value_dim=8, scale=0.5, qk_norm="head", eps=eps,
        position=PartSpec("rope_blended", dict(head_dim=16, theta=5000.0, rotated_dims=16, factor=4.0, original=64, fast=16.0, slow=2.0)))),
        right=PartSpec("retention", dict(hidden_size=W, n_heads=3, head_dim=8, value_dim=12, decay=right["decay"], eps=eps,
                                         position=PartSpec("rope_neox", dict(head_dim=8, theta=1e5, rotated_dims=8))))))
    mixer, plain = bound_part(MIXERS, spec, dtype, rt, seed=3)
    x = _x(n, W, dtype, 9)
    want = pb.side_by_side(x.double().numpy(), plain, "m.", dict(left=left, right=right), eps)
    for cuts in CUTS:
        got = run_mixer(mixer, rt, x, cuts)
        assert np.abs(got - want).max() < (3e-5 if dtype == "float32" else 4e-2) * np.abs(want).max(), cuts


def test_capped_scores_in_every_attention_kernel():
    """The cap against the formula written out, with scores far beyond it: the plain kernel in both dtypes,
    the single-row kernel and the tiled kernel of the matrix cores (rows of short and of long portions)."""
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.kernels import ops, tuned
    from flambeau_amd.parts import PagedKVSpec
    H, G, D, ps, n_pages, cap, scale = 8, 2, 64, 16, 40, 4.0, 0.5
    seqs = [(0, 150), (100, 1), (37, 5), (60, 70)]
    step = make_step(seqs, ps, n_pages)
    n = step.n_tokens
    gen = torch.Generator().manual_seed(3)
    store = CacheStorage([PagedKVSpec(G, D)], [None], torch.device(DEV), torch.bfloat16, n_pages=n_pages, page_size=ps, max_slots=4)
    pool = store.pools[0]
    pool.copy_(torch.randn(pool.shape, generator=gen).to(torch.bfloat16))
    q = torch.randn(n, H * D, generator=gen).to(torch.bfloat16).to(DEV)
    cache = store.entries[0].kv
    table = step.block_tables[0].cpu().numpy()
    want = np.zeros((n, H, D))
    kv = pool[0].double().cpu().numpy()                        # [pages, 2, G, ps, D]: keys row by row, values transposed
    at = 0
    for s, (st, ql) in enumerate(seqs):
        for i in range(ql):
            p = st + i
            keys = np.stack([kv[table[s, t // ps], 0, :, t % ps] for t in range(p + 1)])                       # [p + 1, G, D]
            vals = np.stack([kv[table[s, t // ps], 1].reshape(G, D, ps)[:, :, t % ps] for t in range(p + 1)])
            for h in range(H):
                sc = keys[:, h // (H // G)] @ q[at + i].double().cpu().numpy().reshape(H, D)[h] * scale
                sc = cap * np.tanh(sc / cap)
                w = np.exp(sc - sc.max())
                want[at + i, h] = (w / w.sum()) @ vals[:, h // (H // G)]
        at += ql
    want = want.reshape(n, H * D)
    out = torch.empty_like(q)
    ops.attn_plain(q, out, cache, step.positions, step.tok_seq, step.block_tables[0], H, scale, 0, softcap=cap)
    assert np.abs(out.double().cpu().numpy() - want).max() < 2e-2
    uncapped = torch.empty_like(q)
    ops.attn_plain(q, uncapped, cache, step.positions, step.tok_seq, step.block_tables[0], H, scale, 0)
    assert np.abs(uncapped.double().cpu().numpy() - want).max() > 0.2          # the cap matters here
    rt = make_rt("bfloat16")
    meta = tuned.attention_metadata(step.host, [(tuned.decode_blocks_per_row(H, G), 0)])
    step.extra.update({k: torch.tensor(v, dtype=torch.int32, device=DEV) for k, v in meta.items()})
    fast = torch.full_like(q, float("nan"))
    tuned.attention(rt, q, fast, cache, step, step.block_tables[0], H, scale, 0, softcap=cap)
    assert np.abs(fast.double().cpu().numpy() - want).max() < 2e-2


# ---------------------------------------------------------------- the layers one by one
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_stream_after_every_layer(dirs, name, dtype):
    from flambeau_amd.engine import StepEntry
    d = dirs[(name, dtype)]
    runner = runner_for(d, dtype, n_pages=16, page_size=CONFIGS[name]["page_size"], step_programs=False, decode_graphs=False)
    seen = []
    for b in runner.model.blocks:
        def wrapped(stream, step, cache, fwd=b.forward):
            fwd(stream, step, cache)
            seen.append(stream.flush().double().cpu().numpy())
        b.forward = wrapped
    toks = rh.make_requests(CONFIGS[name]["config"]["vocab"], [37], seed=1)["r0"]
    assert runner.begin("a")
    runner.step([StepEntry("a", toks, [0])])
    cfg, t = read_model(d)
    _, want = pb.forward(cfg, t, toks, return_layers=True)
    assert len(seen) == len(want)
    for i, (g, w) in enumerate(zip(seen, want)):
        assert np.abs(g - w).max() < (2e-5 if dtype == "float32" else 1e-1) * np.abs(w).max(), f"layer {i}"


# ---------------------------------------------------------------- whole models in every cutting
LENGTHS = {"A": [40, 70, 97, 1, 33, 64, 2, 90, 55, 128, 21], "B": [97, 1, 150, 64, 31, 2, 120, 17, 65],
           "C": [150, 64, 3, 65, 1, 200, 31, 90], "D": [40, 100, 7, 64, 130, 2, 55]}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_every_cutting(dirs, name, dtype):
    d = dirs[(name, dtype)]
    ps = CONFIGS[name]["page_size"]
    reqs = rh.make_requests(CONFIGS[name]["config"]["vocab"], LENGTHS[name], seed=5)
    ref = reference(d, reqs)
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs)), ("portions", rh.trace_portions(reqs)),
                        ("mixed", rh.trace_mixed(reqs, seed=13))]:
        peak = rh.peak_tokens(steps)
        runner = runner_for(d, dtype, n_pages=peak // ps, page_size=ps, max_tokens=max(peak, 256), slots=4)
        got = rh.run_in_process(runner, steps)
        pools = runner.manager.pools
        assert sum(p.n_acquired for p in pools) > sum(p.n_pages for p in pools), mode       # pages were used again
        assert not runner.manager.live and runner.manager.n_free_slots == 4
        close(got, ref, dtype, f"{name} {mode}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_single_tokens_replay_graphs_where_no_state_is_advanced(dirs, dtype):
    """A model of attention layers alone captures its decode steps (padded to a bucket: rows without pages
    ride along); one with a recurrent layer never does.  Both give the plain logits."""
    from flambeau_amd.engine import StepEntry
    d = dirs[("D", dtype)]
    reqs = rh.make_requests(90, [20, 33, 5], seed=12)
    ref = reference(d, reqs)
    runner = runner_for(d, dtype, n_pages=24, page_size=16, max_tokens=256)
    assert runner.decode_graphs
    assert not runner_for(dirs[("A", dtype)], dtype, n_pages=24, page_size=8).decode_graphs
    got = {}
    for rid, toks in reqs.items():
        assert runner.begin(rid)
        runner.step([StepEntry(rid, toks[:3], [])])
    for i in range(3, 33):
        live = [rid for rid, toks in reqs.items() if i < len(toks)]
        rows = runner.step([StepEntry(rid, [reqs[rid][i]], [0]) for rid in live]).cpu().double().numpy()
        for rid, row in zip(live, rows):
            got[(rid, i)] = row
    assert runner._graphs
    close(got, ref, dtype, "graphs")


def test_a_batch_equals_each_request_alone(dirs):
    """Unequal requests in one step against each alone: in 32-bit not a bit differs, whatever the
    neighbours, pages and slots are."""
    from flambeau_amd.engine import StepEntry
    d = dirs[("A", "float32")]
    reqs = rh.make_requests(97, [50, 3, 1, 77], seed=9)
    alone = {}
    for rid, toks in reqs.items():
        r = runner_for(d, "float32", n_pages=32, page_size=8)
        assert r.begin(rid)
        alone[rid] = r.step([StepEntry(rid, toks, list(range(len(toks))))]).cpu().numpy().copy()
    r = runner_for(d, "float32", n_pages=32, page_size=8)
    for rid in ("x", "y"):                  # two requests come and go first: other slots, other pages, states that are not zero
        assert r.begin(rid)
        r.step([StepEntry(rid, [1, 2, 3, 4, 5, 6, 7, 8, 9], [])])
    r.end("x"); r.end("y")
    for rid in reversed(list(reqs)):
        assert r.begin(rid)
    both = r.step([StepEntry(rid, toks, list(range(len(toks)))) for rid, toks in reqs.items()]).cpu().numpy()
    at = 0
    for rid, toks in reqs.items():
        assert np.array_equal(both[at:at + len(toks)], alone[rid]), rid
        at += len(toks)


@pytest.mark.parametrize("dtype", DTYPES)
def test_peaked_attention_over_far_keys_and_page_borders(dirs, dtype):
    """Score scales eight times as large: softmax puts nearly all weight on single keys, hundreds of tokens
    back or next to a page's edge alike, so one key lost or one too many shows in the logits."""
    d = dirs[("sharp", dtype)]
    reqs = rh.make_requests(97, [260, 131], seed=2)
    ref = reference(d, reqs)
    blunt = reference(dirs[("A", dtype)], reqs)
    assert np.abs(ref["r0"] - blunt["r0"]).max() > 0.1 * np.abs(ref["r0"]).max()
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=40)),
                        ("portions", rh.trace_portions(reqs, sizes=(7, 2, 8, 9, 16, 1, 15, 33, 3)))]:
        runner = runner_for(d, dtype, n_pages=48, page_size=8)
        close(rh.run_in_process(runner, steps), ref, dtype, f"sharp {mode}", bf16=8e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_memory_and_long_decoding(dirs, dtype):
    """Decays next to one: the first tokens stay in the matrix memories for hundreds of steps (the plain
    logits at the end change when the first token does), through 230 single-token steps."""
    d = dirs[("memory", dtype)]
    toks = rh.make_requests(97, [240], seed=4)["r0"]
    reqs = {"r0": toks}
    ref = reference(d, reqs)
    other = reference(d, {"r0": [(toks[0] + 1) % 97] + toks[1:]})
    assert np.abs(ref["r0"][-1] - other["r0"][-1]).max() > 1e-3 * np.abs(ref["r0"]).max()
    runner = runner_for(d, dtype, n_pages=32, page_size=8)
    close(rh.run_in_process(runner, rh.trace_tail(reqs, tail=230)), ref, dtype, "memory")


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens(dirs, dtype):
    """Requests of one and two tokens (fewer than the convolution has taps), alone, side by side, and
    continued one token at a time."""
    d = dirs[("A", dtype)]
    reqs = rh.make_requests(97, [1, 2, 1, 3], seed=7)
    ref = reference(d, reqs)
    steps = [dict(entries=[dict(id=rid, tokens=toks[:1], want=[0]) for rid, toks in reqs.items()], end=["r0", "r2"]),
             dict(entries=[dict(id="r1", tokens=reqs["r1"][1:], want=[0]), dict(id="r3", tokens=reqs["r3"][1:2], want=[0])], end=["r1"]),
             dict(entries=[dict(id="r3", tokens=reqs["r3"][2:], want=[0])], end=["r3"])]
    close(rh.run_in_process(runner_for(d, dtype, n_pages=8, page_size=8), steps), ref, dtype, "first tokens")


def test_a_slot_that_is_used_again_starts_from_zero(dirs):
    """One state slot: every request inherits the slot of the one before, whose memories and kept
    convolution inputs are not zero, and still gives the plain logits."""
    d = dirs[("B", "float32")]
    reqs = rh.make_requests(61, [30, 9, 1, 44], seed=8)
    ref = reference(d, reqs)
    runner = runner_for(d, "float32", n_pages=8, page_size=16, slots=1)
    close(rh.run_in_process(runner, rh.trace_portions(reqs, sizes=(5, 2, 11))), ref, "float32", "one slot")


# ---------------------------------------------------------------- through the entry points
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(dirs, dtype):
    """``generate``: scheduler, portions, batching, device sampler.  Every token is the plain
    implementation's argmax (or within rounding of it)."""
    from flambeau_amd import generate
    d = dirs[("A", dtype)]
    cfg, t = read_model(d)
    prompts = [p for p in rh.make_requests(97, [7, 19, 1, 30, 12], seed=3).values()]
    outs = generate(str(d), prompts, max_new_tokens=10, dtype=dtype, page_size=8, inflight_slots=3, prefill_chunk_tokens=16)
    turned = 0
    for prompt, out in zip(prompts, outs):
        assert len(out) == 10
        toks = list(prompt)
        for tok in out:
            logits = pb.forward(cfg, t, toks)[-1]
            best = int(np.argmax(logits))
            if not (tok == best or logits[best] - logits[tok] < (1e-4 if dtype == "float32" else 3e-2) * np.abs(logits).max()):
                turned += 1
            toks.append(tok)
    assert turned <= (0 if dtype == "float32" else 2), turned


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_as_a_program(dirs, tmp_path, dtype):
    d = dirs[("C", dtype)]
    reqs = rh.make_requests(150, [40, 70, 97, 33, 64, 12, 90, 55], seed=6)
    ref = reference(d, reqs)
    steps = rh.trace_mixed(reqs, seed=3)
    stats = {}
    got = rh.run_program(d, dtype, steps, tmp_path / "o", rh.peak_tokens(steps), 150, extra=("--poison-cache",), stats=stats)
    assert stats["handed_out"] > stats["pool"]
    close(got, ref, dtype, "trace_run")


def test_the_command_line_serves_it(tmp_path):
    """``random-weights`` -> ``inspect`` -> ``infer --json`` on a Bugidra configuration, greedy in 32-bit with so
    few slots and pages that requests wait and are pre-empted (a pre-empted request starts again from a
    zeroed state): exactly the plain implementation's tokens."""
    import subprocess
    import sys
    cfg = CONFIGS["A"]["config"]
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    d = tmp_path / "model"

    def cli(*args):
        r = subprocess.run([sys.executable, "-m", "flambeau_amd", *map(str, args)], capture_output=True, text=True, timeout=600, cwd=str(rh.ROOT))
        assert r.returncode == 0, f"{args}\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
        return r
    cli("random-weights", "--config", tmp_path / "config.json", "--out", d, "--seed", 5, "--std", 0.16, "--gain-std", 0.1, "--dtype", "float32")
    seen = cli("inspect", d).stdout
    assert "architecture: Bugidra" in seen and "tensors fit the model" in seen and "l2.mix.right.out" in seen
    prompts = list(rh.make_requests(97, [3, 30, 17], seed=6).values())
    flags = []
    for p in prompts:
        flags += ["--prompt", ",".join(map(str, p))]
    out = json.loads(cli("infer", "--model", d, *flags, "--max-tokens", 18, "--dtype", "float32", "--json", "--inflight-slots", 2,
                         "--paged-kv", 5, "--page-size", 16, "--prefill-chunk-tokens", 16, "--max-queue-depth", 4).stdout)
    conf, t = read_model(d)
    for p, o in zip(prompts, out["outputs"]):
        toks = list(p)
        for tok in o:
            logits = pb.forward(conf, t, toks)[-1]
            best = int(np.argmax(logits))
            assert tok == best or logits[best] - logits[tok] < 1e-4 * np.abs(logits).max()
            toks.append(tok)
        assert len(o) == 18
