"""Kuvidra on the GPU against the plain implementation: every mechanism alone, the layers one by
one, and whole models in every cutting (whole prompts, single tokens, portions down to two tokens,
mixed batches over a small poisoned pool whose pages and slots are used again), in 32-bit and in
bfloat16, at sizes of the tests' own."""
import numpy as np
import pytest
import torch

import plain_kuvidra as pk
import replay_helpers as rh
from kuvidra_configs import CONFIGS, read_model, write_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("kuvidra")
    out = {}
    for name in CONFIGS:
        for store in DTYPES:
            out[(name, store)] = write_model(name, base / f"{name}-{store}", store)
    for store in DTYPES:          # (weights are stored in the dtype they are run in: the plain side reads the same numbers)
        out[("sharp", store)] = write_model("P", base / f"P-sharp-{store}", store, sharpen=6.0)
        out[("memory", store)] = write_model("P", base / f"P-memory-{store}", store, forget_bias=7.0)
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
            _refs[key] = pk.forward(cfg, t, toks)
        out[rid] = _refs[key]
    return out


def runner_for(d, dtype, n_pages, page_size, max_tokens=512, slots=4, poison=True, **kw):
    from flambeau_amd.engine import ModelRunner, load_model
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=max_tokens)
    runner = ModelRunner(model, n_pages=n_pages, page_size=page_size, max_slots=slots, max_seq_len=max_tokens, **kw)
    if poison:
        runner.storage.fill(float("nan"))
    return runner


def close(got, ref, dtype, what, f32=3e-4, bf16=4e-2):
    """Every wanted row against the plain one: the largest difference relative to the largest logit.
    In 32-bit every row must agree.  In bfloat16 the rounding of a layer's input now and then turns a
    close call (which expert scores highest, which of two keys a peaked softmax takes) the other way,
    and such a row is far off without any fault: there the typical row must agree closely and at most
    a fifth of the rows may be beyond the bound (a lost key, a stale page or a wrong state moves most rows,
    and shows in the 32-bit run of the same trace)."""
    scale = max(float(np.abs(r).max()) for r in ref.values())
    tol = (f32 if dtype == "float32" else bf16) * scale
    errs = {k: float(np.abs(row - ref[k[0]][k[1]]).max()) for k, row in sorted(got.items())}
    bad = [(rid, p, e) for (rid, p), e in errs.items() if not e <= tol]
    assert got, what
    if dtype == "float32":
        assert not bad, f"{what} [{dtype}]: {len(bad)} of {len(got)} rows off by more than {tol:.3g}; first {bad[:3]}"
    else:
        assert np.isfinite(list(errs.values())).all(), what
        assert np.median(list(errs.values())) <= tol / 3 and len(bad) <= 0.2 * len(got), \
            f"{what} [{dtype}]: {len(bad)} of {len(got)} rows off by more than {tol:.3g}, median {np.median(list(errs.values())):.3g}"


# ---------------------------------------------------------------- each mechanism alone
def make_rt(dtype, max_tokens=256):
    from flambeau_amd.engine import Runtime
    return Runtime(DEV, TORCH[dtype], max_tokens, True)


def make_step(seqs, page_size, n_pages, slots=None, seed=0):
    """A StepState for requests ``seqs`` = (start position, tokens), pages handed out in a shuffled order."""
    from flambeau_amd.parts import HostBatch, StepState
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    q_starts, q_lens, starts, pos, tok_seq = [], [], [], [], []
    width = max(-(-(st + q) // page_size) for st, q in seqs) + 1
    table = np.full((len(seqs), width), -1, dtype=np.int32)
    at = 0
    for s, (st, q) in enumerate(seqs):
        nb = -(-(st + q) // page_size)
        table[s, :nb] = [perm.pop() for _ in range(nb)]
        q_starts.append(at); q_lens.append(q); starts.append(st)
        pos += range(st, st + q); tok_seq += [s] * q
        at += q
    slots = list(slots if slots is not None else range(len(seqs)))
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)
    return StepState(n_tokens=at, n_seqs=len(seqs), tokens=i32([0] * at), positions=i32(pos), tok_seq=i32(tok_seq),
                     seq_slots=i32(slots), seq_q_start=i32(q_starts), seq_q_len=i32(q_lens),
                     seq_ctx_len=i32([st + q for st, q in seqs]), block_tables=[i32(table)], logit_rows=i32([]),
                     host=HostBatch(q_starts, q_lens, starts, slots, at, 0))


def bound_part(registry, spec, dtype, rt, seed, scale=0.3, prefix="m."):
    """A part with random weights (rounded to the compute dtype) and the same numbers for the plain side,
    under the design's tensor names."""
    part = registry.create(spec)
    g = torch.Generator().manual_seed(seed)
    w, plain = {}, {}
    for k, ts in part.tensors().items():
        v = torch.randn(*ts.shape, generator=g) * scale
        if ts.role == "vector32" and not k.endswith("bias"):
            v = 1 + v
        v = v.to(TORCH[dtype])
        w[k] = rt.to_device(v, ts.role)
        name = k.replace("_norm.weight", ".norm").replace(".weight", "").replace(".bias", ".b")
        plain[prefix + name] = v.double().numpy()
    part.bind(w, rt)
    return part, plain


def run_mixer(mixer, rt, x, cuts, page_size=8, n_pages=40):
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.parts import Product
    store = CacheStorage([mixer.cache_spec()], [None], rt.device, rt.dtype, n_pages=n_pages, page_size=page_size, max_slots=3)
    for p in store.pools:
        p.fill_(float("nan"))
    got, at = [], 0
    for k in cuts:
        step = make_step([(at, k)], page_size, n_pages, slots=[2], seed=1)
        if hasattr(mixer, "step_metadata_for"):                # the work lists the step function would upload
            step.extra.update({name: torch.tensor(arr, dtype=torch.int32, device=DEV)
                               for name, arr in type(mixer).step_metadata_for(step.host, [mixer]).items()})
        r = mixer.forward(x[at:at + k].to(DEV).contiguous(), step, store.entries[0])
        r = r.compute(rt) if isinstance(r, Product) else r
        got.append(r.double().cpu().numpy())
        at += k
    return np.concatenate(got)


CUTS = ([90], [40, 5, 1, 1, 2, 20, 2, 6, 1, 12], [1] * 20 + [70])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv,Rq,R,scale", [(3, 8, 12, 20, 24, 0.9), (1, 40, 5, 9, 150, 0.3), (6, 4, 4, 4, 64, 2.0),
                                               # sizes that the matrix-core kernels take, all three or some of them
                                               (20, 32, 48, 24, 96, 0.7), (4, 64, 16, 40, 160, 0.04), (16, 8, 32, 8, 32, 1.0),
                                               (2, 96, 12, 16, 512, 0.2)])
def test_latent_attention_alone(dtype, H, D, Dv, Rq, R, scale):
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps = 40, 90, 2e-5
    mixer, plain = bound_part(MIXERS, PartSpec("latent_attention", dict(hidden_size=W, n_heads=H, head_dim=D, value_dim=Dv, q_rank=Rq,
                                                                         kv_rank=R, scale=scale, eps=eps)), dtype, rt, seed=H)
    x = (torch.randn(n, W, generator=torch.Generator().manual_seed(5))).to(TORCH[dtype])
    want = pk.latent_attention(x.double().numpy(), plain, "m.", dict(heads=H, dim=D, vdim=Dv, scale=scale), eps)
    for cuts in CUTS:
        got = run_mixer(mixer, rt, x, cuts)
        assert np.abs(got - want).max() < (3e-5 if dtype == "float32" else 3e-2) * np.abs(want).max(), cuts


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv,cap", [(2, 12, 20, 8.0), (1, 20, 70, 15.0), (3, 4, 6, 2.0), (1, 100, 33, 30.0), (1, 300, 17, 12.0)])
def test_mlstm_alone(dtype, H, D, Dv, cap):
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps = 40, 90, 1e-5
    mixer, plain = bound_part(MIXERS, PartSpec("mlstm", dict(hidden_size=W, n_heads=H, head_dim=D, value_dim=Dv, gate_cap=cap, eps=eps)),
                              dtype, rt, seed=D)
    x = (torch.randn(n, W, generator=torch.Generator().manual_seed(6))).to(TORCH[dtype])
    want = pk.mlstm(x.double().numpy(), plain, "m.", dict(heads=H, dim=D, vdim=Dv, gate_cap=cap), eps)
    results = [run_mixer(mixer, rt, x, cuts) for cuts in CUTS]
    for got, cuts in zip(results, CUTS):
        assert np.abs(got - want).max() < (5e-5 if dtype == "float32" else 4e-2) * np.abs(want).max(), cuts
    if dtype == "float32":
        # the walk is the same however the tokens are cut: not a bit differs
        assert all(np.array_equal(results[0], r) for r in results[1:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 7, 150])
@pytest.mark.parametrize("W", [40, 64])          # 64: in bfloat16 the experts' products run on the matrix cores
def test_feed_forwards_alone(dtype, n, W):
    from flambeau_amd.parts import FEED_FORWARDS, PartSpec, Product
    rt = make_rt(dtype)
    x = (torch.randn(n, W, generator=torch.Generator().manual_seed(n))).to(TORCH[dtype])
    xs = x.double().numpy()
    tol = 3e-5 if dtype == "float32" else 3e-2

    def run(part):
        r = part.forward(x.to(DEV), None)
        return (r.compute(rt) if isinstance(r, Product) else r).double().cpu().numpy()
    for act, fn in (("gelu", pk.gelu_erf), ("gelu_tanh", pk.gelu_tanh), ("silu", pk.silu)):
        part, plain = bound_part(FEED_FORWARDS, PartSpec("mlp", dict(hidden_size=W, intermediate_size=56, activation=act)), dtype, rt, seed=1)
        want = fn(xs @ plain["m.up"].T) @ plain["m.down"].T
        assert np.abs(run(part) - want).max() < tol * np.abs(want).max(), act
    for E, top, shared in ((5, 2, 24), (3, 3, None), (7, 1, 8), (70, 4, None)):
        spec = dict(hidden_size=W, n_experts=E, top=top, expert_size=16 if W == 40 else 32, shared_size=shared)
        part, plain = bound_part(FEED_FORWARDS, PartSpec("routed_experts", spec), dtype, rt, seed=E, scale=0.4)
        mlp = {"router": {"experts": E, "top": top}, "shared": {"ff": shared} if shared else None}
        want = pk.moe_ff(xs, plain, "m.", mlp)
        assert np.abs(run(part) - want).max() < tol * np.abs(want).max(), (E, top, shared)
        # the weight on the expert's output instead, and the chosen weights renormalised
        other, plain = bound_part(FEED_FORWARDS, PartSpec("routed_experts", dict(spec, weight_on="output", renormalise=True)), dtype, rt, seed=E, scale=0.4)
        s = pk.sigmoid(xs @ plain["m.router"].T)
        want = np.zeros((n, W))
        for i in range(n):
            chosen = sorted(range(E), key=lambda e: (-s[i, e], e))[:top]
            for e in chosen:
                want[i] += s[i, e] / s[i, chosen].sum() * pk.gated_expert(xs[i:i + 1], plain, f"m.e{e}.")[0]
        if shared:
            want += pk.sigmoid(xs @ plain["m.shared.sg"].T) * pk.gated_expert(xs, plain, "m.shared.")
        assert np.abs(run(other) - want).max() < tol * np.abs(want).max(), ("output", E, top)


# ---------------------------------------------------------------- the layers one by one
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_stream_after_every_layer(dirs, name, dtype):
    from flambeau_amd.engine import StepEntry
    d = dirs[(name, dtype)]
    runner = runner_for(d, dtype, n_pages=16, page_size=CONFIGS[name]["page_size"], step_programs=False)
    seen = []
    for b in runner.model.blocks:
        if b.mixers():
            def wrapped(stream, step, cache, fwd=b.forward):
                fwd(stream, step, cache)
                seen.append(stream.flush().double().cpu().numpy())
            b.forward = wrapped
    toks = rh.make_requests(CONFIGS[name]["config"]["vocab"], [37], seed=1)["r0"]
    assert runner.begin("a")
    runner.step([StepEntry("a", toks, [0])])
    cfg, t = read_model(d)
    _, want = pk.forward(cfg, t, toks, return_layers=True)
    assert len(seen) == len(want)
    for i, (g, w) in enumerate(zip(seen, want)):
        # (bfloat16: the unit norm behind the matrix memory magnifies the rounding of its input where a head's output is small)
            assert np.abs(g - w).max() < (2e-5 if dtype == "float32" else 1e-1) * np.abs(w).max(), f"layer run {i}"


# ---------------------------------------------------------------- whole models in every cutting
LENGTHS = {"P": [40, 70, 97, 1, 33, 64, 2, 90, 55, 128, 21], "Q": [97, 1, 150, 64, 31, 2, 120, 17, 65],
           "R": [33, 80, 5, 129, 64, 16, 100], "S": [150, 64, 3, 65, 1, 200, 31, 90],
           "T": [40, 100, 7, 64, 130, 2, 55]}


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
    ride along); one with an mLSTM layer never does.  Both give the plain logits."""
    from flambeau_amd.engine import StepEntry
    d = dirs[("T", dtype)]
    reqs = rh.make_requests(90, [20, 33, 5], seed=12)
    ref = reference(d, reqs)
    runner = runner_for(d, dtype, n_pages=24, page_size=16, max_tokens=256)
    assert runner.decode_graphs
    assert not runner_for(dirs[("P", dtype)], dtype, n_pages=24, page_size=8).decode_graphs
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
    d = dirs[("P", "float32")]
    reqs = rh.make_requests(97, [50, 3, 1, 77], seed=9)
    alone = {}
    for rid, toks in reqs.items():
        r = runner_for(d, "float32", n_pages=32, page_size=8)
        assert r.begin(rid)
        alone[rid] = r.step([StepEntry(rid, toks, list(range(len(toks))))]).cpu().numpy().copy()
    r = runner_for(d, "float32", n_pages=32, page_size=8)
    for rid in ("x", "y", *reqs):           # two requests come and go first: other slots, other pages
        if rid in ("x", "y"):
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
    """Queries six times as large: softmax puts nearly all weight on single keys, hundreds of tokens
    back or next to a page's edge alike, so one key lost or one too many shows in the logits."""
    d = dirs[("sharp", dtype)]
    reqs = rh.make_requests(97, [260, 131], seed=2)
    ref = reference(d, reqs)
    blunt = reference(dirs[("P", dtype)], reqs)
    assert np.abs(ref["r0"] - blunt["r0"]).max() > 0.2 * np.abs(ref["r0"]).max()
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=40)),
                        ("portions", rh.trace_portions(reqs, sizes=(7, 2, 8, 9, 16, 1, 15, 33, 3)))]:
        runner = runner_for(d, dtype, n_pages=48, page_size=8)
        close(rh.run_in_process(runner, steps), ref, dtype, f"sharp {mode}", bf16=8e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_memory_and_long_decoding(dirs, dtype):
    """Forget gates near one: the first tokens stay in the matrix memory for hundreds of steps (the
    plain logits at the end change when the first token does), through 230 single-token steps."""
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
    """Requests of one and two tokens, alone, side by side, and continued one token at a time."""
    d = dirs[("Q", dtype)]
    reqs = rh.make_requests(61, [1, 2, 1, 3], seed=7)
    ref = reference(d, reqs)
    steps = [dict(entries=[dict(id=rid, tokens=toks[:1], want=[0]) for rid, toks in reqs.items()], end=["r0", "r2"]),
             dict(entries=[dict(id="r1", tokens=reqs["r1"][1:], want=[0]), dict(id="r3", tokens=reqs["r3"][1:2], want=[0])], end=["r1"]),
             dict(entries=[dict(id="r3", tokens=reqs["r3"][2:], want=[0])], end=["r3"])]
    close(rh.run_in_process(runner_for(d, dtype, n_pages=8, page_size=16), steps), ref, dtype, "first tokens")


# ---------------------------------------------------------------- through the entry points
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(dirs, dtype):
    """``generate``: scheduler, portions, batching, device sampler.  Every token is the plain
    implementation's argmax (or within rounding of it)."""
    from flambeau_amd import generate
    d = dirs[("P", dtype)]
    cfg, t = read_model(d)
    prompts = [p for p in rh.make_requests(97, [7, 19, 1, 30, 12], seed=3).values()]
    outs = generate(str(d), prompts, max_new_tokens=10, dtype=dtype, page_size=8, inflight_slots=3, prefill_chunk_tokens=16)
    turned = 0
    for prompt, out in zip(prompts, outs):
        assert len(out) == 10
        toks = list(prompt)
        for i, tok in enumerate(out):
            logits = pk.forward(cfg, t, toks)[-1]
            best = int(np.argmax(logits))
            if not (tok == best or logits[best] - logits[tok] < (1e-4 if dtype == "float32" else 3e-2) * np.abs(logits).max()):
                turned += 1
            toks.append(tok)
    # (bfloat16: a close call of a router may fall the other way; every later token is judged from the engine's own prefix)
    assert turned <= (0 if dtype == "float32" else 3), turned


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_as_a_program(dirs, tmp_path, dtype):
    d = dirs[("R", dtype)]
    reqs = rh.make_requests(130, [40, 70, 97, 33, 64, 12, 90, 55], seed=6)
    ref = reference(d, reqs)
    steps = rh.trace_mixed(reqs, seed=3)
    stats = {}
    got = rh.run_program(d, dtype, steps, tmp_path / "o", rh.peak_tokens(steps), 130, extra=("--poison-cache",), stats=stats)
    assert stats["handed_out"] > stats["pool"]
    close(got, ref, dtype, "trace_run")


@pytest.mark.parametrize("H,R", [(20, 96), (5, 512), (33, 160), (16, 32)])
@pytest.mark.parametrize("splits", [2, 8, 64])
def test_keys_dealt_out_to_several_waves(splits, H, R):
    """The matrix-core attention kernel with every token's keys in several parts (what a decode step behind
    a long context does) against the same kernel in one part, rows of unequal contexts side by side, some
    shorter than the number of parts."""
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.kernels import latent_attention as la
    from flambeau_amd.parts import PagedRowSpec
    ps, n_pages = 16, 80
    store = CacheStorage([PagedRowSpec(R)], [None], torch.device(DEV), torch.bfloat16, n_pages=n_pages, page_size=ps, max_slots=4)
    pool = store.pools[0]                       # [entries, pages, 2, page, R]: rows, and the same rows transposed
    pool[:, :, 0].normal_(0.0, 1.0)
    pool[:, :, 1] = pool[:, :, 0].transpose(-1, -2).reshape(pool[:, :, 1].shape)
    seqs = [(700, 1), (0, 1), (130, 3), (63, 2)]
    step = make_step(seqs, ps, n_pages)
    n = step.n_tokens
    qa = (torch.randn(n, H * R, generator=torch.Generator().manual_seed(1)) * 0.3).to(torch.bfloat16).to(DEV)
    cache = store.entries[0].kv
    one = torch.empty(n, H * R, dtype=torch.float32, device=DEV)
    la.latent_attention_mfma(qa, one, cache, step.positions, step.tok_seq, step.block_tables[0], H, 0.5)
    rows = n * -(-H // 16) * splits * 16
    part_o = torch.full((rows, R), float("nan"), dtype=torch.float32, device=DEV)
    part_ml = torch.full((rows, 2), float("nan"), dtype=torch.float32, device=DEV)
    many = torch.empty_like(one)
    la.latent_attention_mfma(qa, many, cache, step.positions, step.tok_seq, step.block_tables[0], H, 0.5, 0, splits, part_o, part_ml)
    assert torch.isfinite(many).all()
    assert (many - one).abs().max().item() < 2e-3 * one.abs().max().item()
    # the form in which four waves share a (token, 16 heads, part of the keys), in parts and whole
    for k in (splits, 1):
        dealt = torch.full_like(one, float("nan"))
        la.latent_attention_mfma(qa, dealt, cache, step.positions, step.tok_seq, step.block_tables[0], H, 0.5, 0, k, part_o, part_ml, dealt=True)
        assert torch.isfinite(dealt).all() and (dealt - one).abs().max().item() < 2e-3 * one.abs().max().item(), k
    # and both against the float kernel
    plain = torch.empty_like(one)
    from flambeau_amd.kernels import ops
    ops.latent_attention(qa.float(), plain, cache, step.positions, step.tok_seq, step.block_tables[0], H, 0.5)
    assert (one - plain).abs().max().item() < 2e-2 * plain.abs().max().item()


@pytest.mark.parametrize("H,R,ps", [(20, 96, 16), (32, 64, 32), (7, 512, 16), (40, 32, 16), (70, 160, 64)])
def test_blocks_that_share_their_keys(H, R, ps):
    """The matrix-core kernel whose four waves read every chunk of keys from LDS against the one whose waves
    fetch for themselves: portions of unequal requests (some start mid-context, one is a single token, one
    crosses several chunks), with one, two, three and more groups of 16 heads."""
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.kernels import latent_attention as la
    from flambeau_amd.parts import PagedRowSpec
    n_pages = 64
    store = CacheStorage([PagedRowSpec(R)], [None], torch.device(DEV), torch.bfloat16, n_pages=n_pages, page_size=ps, max_slots=4)
    pool = store.pools[0]
    pool[:, :, 0].normal_(0.0, 1.0)
    pool[:, :, 1] = pool[:, :, 0].transpose(-1, -2).reshape(pool[:, :, 1].shape)
    seqs = [(0, 150), (300, 7), (63, 1), (120, 70)]
    step = make_step(seqs, ps, n_pages)
    n = step.n_tokens
    qa = (torch.randn(n, H * R, generator=torch.Generator().manual_seed(2)) * 0.4).to(torch.bfloat16).to(DEV)
    cache = store.entries[0].kv
    # rows beyond each request's newest token are poisoned: the kernels may load them but must not use them
    for s, (st, q) in enumerate(seqs):
        last = st + q
        page = int(step.block_tables[0][s, last // ps]) if last % ps else -1
        if page >= 0:
            pool[0, page, 0, last % ps:] = float("nan")
            pool[0, page, 1].view(R, ps)[:, last % ps:] = float("nan")
    alone = torch.empty(n, H * R, dtype=torch.float32, device=DEV)
    la.latent_attention_mfma(qa, alone, cache, step.positions, step.tok_seq, step.block_tables[0], H, 0.3)
    tiles = torch.tensor(la.shared_tiles(step.host, -(-H // 16)), dtype=torch.int32, device=DEV)
    shared = torch.full_like(alone, float("nan"))
    la.latent_attention_shared(qa, shared, cache, step.positions, step.tok_seq, step.block_tables[0], H, 0.3, 0, tiles)
    assert torch.isfinite(alone).all() and torch.isfinite(shared).all()
    # (the two kernels round their weights against different bases: the shared one follows the maximum lazily)
    assert (shared - alone).abs().max().item() < 5e-3 * alone.abs().max().item()


def test_the_command_line_serves_it(tmp_path):
    """``random-weights`` -> ``inspect`` -> ``infer --json`` on a Kuvidra configuration, greedy in 32-bit with so
    few slots and pages that requests wait and are pre-empted (a pre-empted request starts again from a
    zeroed state): exactly the plain implementation's tokens."""
    import json
    import subprocess
    import sys
    cfg = CONFIGS["P"]["config"]
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    d = tmp_path / "model"

    def cli(*args):
        r = subprocess.run([sys.executable, "-m", "flambeau_amd", *map(str, args)], capture_output=True, text=True, timeout=600, cwd=str(rh.ROOT))
        assert r.returncode == 0, f"{args}\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
        return r
    cli("random-weights", "--config", tmp_path / "config.json", "--out", d, "--seed", 5, "--std", 0.16, "--gain-std", 0.1, "--dtype", "float32")
    seen = cli("inspect", d).stdout
    assert "architecture: Kuvidra" in seen and "tensors fit the model" in seen and "l1.mlp.shared.sg" in seen
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
            logits = pk.forward(conf, t, toks)[-1]
            best = int(np.argmax(logits))
            assert tok == best or logits[best] - logits[tok] < 1e-4 * np.abs(logits).max()
            toks.append(tok)
        assert len(o) == 18


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("R,window", [(24, 13), (64, 70), (96, 64), (32, 1)])
def test_latent_attention_with_a_window(dtype, R, window):
    """``window`` keys, the query's own included (no model of the package sets it yet): the mixer against the
    formula written out, whole and in portions that cross the window's edge and the kernels' chunks of 64 keys;
    pages that the window has passed are poisoned as a manager that returns them would leave them."""
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype)
    W, n, eps, H, D, Dv, Rq = 40, 150, 1e-5, 5, 32, 16, 16
    mixer, plain = bound_part(MIXERS, PartSpec("latent_attention", dict(hidden_size=W, n_heads=H, head_dim=D, value_dim=Dv, q_rank=Rq,
                                                                         kv_rank=R, scale=0.2, eps=eps, window=window)), dtype, rt, seed=R)
    assert mixer.cache_spec().window == window
    x = (torch.randn(n, W, generator=torch.Generator().manual_seed(8))).to(TORCH[dtype])
    h = x.double().numpy()
    cq = pk.rms_norm(h @ plain["m.dq"].T, plain["m.dq.norm"], eps)
    q = (cq @ plain["m.uq"].T).reshape(n, H, D)
    c = pk.rms_norm(h @ plain["m.dkv"].T, plain["m.dkv.norm"], eps)
    k, v = (c @ plain["m.uk"].T).reshape(n, H, D), (c @ plain["m.uv"].T).reshape(n, H, Dv)
    want = np.zeros((n, H, Dv))
    for i in range(n):
        lo = max(0, i - window + 1)
        s = np.einsum("hd,jhd->hj", q[i], k[lo:i + 1]) * 0.2
        p = np.exp(s - s.max(axis=1, keepdims=True))
        want[i] = np.einsum("hj,jhv->hv", p / p.sum(axis=1, keepdims=True), v[lo:i + 1])
    want = (want * pk.sigmoid(h @ plain["m.g"].T)[:, :, None]).reshape(n, H * Dv) @ plain["m.o"].T
    for cuts in ([n], [60, 5, 1, 1, 2, 30, 2, 6, 1, 42], [1] * 90 + [60]):
        got = run_mixer(mixer, rt, x, cuts)
        assert np.abs(got - want).max() < (3e-5 if dtype == "float32" else 3e-2) * np.abs(want).max(), cuts
