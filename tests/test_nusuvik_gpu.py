"""The Nusuvik decoder on the GPU against the plain implementation (tests/plain_nusuvik.py): every mechanism alone at
the level of its kernels, then whole models of four tiny configurations through the engine's step function (whole
prompts, tails decoded one by one, portions down to two tokens, mixed batches with pages and slots used again), every
layer run against the plain stream, a standout key far away and at page borders, the previous token across steps and
slots, long decoding through recorded steps, and greedy generation through the entry point and the scheduler."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
import nusuvik_cases as cases
import plain_nusuvik as plain
import schedules

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": 2e-5, "bfloat16": 3e-2}
LENGTHS = [5, 17, 33, 70, 150, 41, 64, 2, 1]
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def row_errs(got, ref):
    return np.abs(got.astype(np.float64) - ref).max(axis=-1) / np.abs(ref).max()


def check_rows(out, ref, dt, what):
    """float32: every row within the limit.  bfloat16: nine rows in ten (a router's choice between two experts whose
    choice values differ by less than the rounding may fall the other way, and moves that token's rows)."""
    e = np.concatenate([row_errs(out[r], ref[r]) for r in ref])
    worst, q90 = float(e.max()), float(np.quantile(e, 0.9))
    print(f"[observed] {what} {dt}: worst {worst:.3e}, nine in ten below {q90:.3e}")
    assert (worst if dt == "float32" else q90) < TOL[dt], (what, dt, worst, q90)
    assert np.isfinite(e).all()


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (cfg, page, seed) in cases.CASES.items():
        w = cases.draw_weights(cfg, seed)
        for dt in ("float32", "bfloat16"):
            d = cases.write_model(tmp_path_factory.mktemp(f"n{name}{dt}"), cfg, w, DT[dt])
            reqs = helpers.random_requests(cfg["vocab"], LENGTHS, seed + 10)
            wd = cases.stored(w, DT[dt])
            out[(name, dt)] = (d, reqs, {r: plain.forward(t, wd, cfg) for r, t in reqs.items()})
    return out


def _engine(d, dt, page, max_tokens, **kw):
    from litinfer_amd.engine import Engine
    return Engine.from_dir(d, dtype=dt, device=DEV, page_size=page, max_tokens=max_tokens, max_seqs=4,
                           page_order_seed=5, **kw)


def _rows(eng, rid, toks, cuts):
    from litinfer_amd.engine import StepEntry
    return np.concatenate([eng.step([StepEntry(rid, toks[a:b], list(range(b - a)))]).float().cpu().numpy()
                           for a, b in zip(cuts, cuts[1:]) if b > a])


# ------------------------------------------------------------------------------------------ whole models
@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(cases.CASES))
@pytest.mark.parametrize("kind", ["whole", "tail", "chunks", "mixed"])
def test_schedules_match_the_plain_implementation(models, name, dt, kind):
    cfg, page, _ = cases.CASES[name]
    d, reqs, ref = models[(name, dt)]
    steps = getattr(schedules, kind)(reqs)
    eng = _engine(d, dt, page, schedules.max_live_tokens(reqs, steps, page if kind == "mixed" else 64))
    out = schedules.run(eng, reqs, steps)
    eng.cache.check_invariants()
    assert all(f == g.pool.capacity for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
    assert eng.cache.free_slots() == 4
    if kind == "mixed":
        assert all(g.pool.total_allocations > g.pool.capacity for g in eng.cache.groups), "no page was used again"
    check_rows(out, ref, dt, f"{name} {kind}")


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Sizes, order of layers, loop, routers and constants drawn from a seed: a mixed schedule on few pages, both dtypes."""
    cfg = cases.random_config(seed)
    w32 = cases.draw_weights(cfg, 100 + seed)
    reqs = helpers.random_requests(cfg["vocab"], [3, 40, 18, 75, 1, 29], 200 + seed)
    page = (4, 8, 16, 32)[seed % 4]
    for dt in ("float32", "bfloat16"):
        d = cases.write_model(tmp_path / dt, cfg, w32, DT[dt])
        w = cases.stored(w32, DT[dt])
        ref = {r: plain.forward(t, w, cfg) for r, t in reqs.items()}
        steps = schedules.mixed(reqs, seed=seed)
        eng = _engine(d, dt, page, schedules.max_live_tokens(reqs, steps, page))
        out = schedules.run(eng, reqs, steps)
        eng.cache.check_invariants()
        check_rows(out, ref, dt, f"random configuration {seed}")


@pytest.mark.parametrize("name", list(cases.CASES))
def test_float32_logits_do_not_depend_on_the_schedule(models, name):
    cfg, page, _ = cases.CASES[name]
    d, reqs, _ = models[(name, "float32")]
    outs = {}
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        outs[kind] = schedules.run(_engine(d, "float32", page, schedules.max_live_tokens(reqs, steps)), reqs, steps)
    for kind in ("tail", "chunks", "mixed"):
        for r in reqs:
            assert schedules.rel_err(outs[kind][r], outs["whole"][r].astype(np.float64)) < 2e-5, (kind, r)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(cases.CASES))
def test_every_layer_run_against_the_plain_stream(models, name, dt):
    from litinfer_amd.engine import StepEntry
    cfg, page, seed = cases.CASES[name]
    d, reqs, _ = models[(name, dt)]
    w = cases.stored(cases.draw_weights(cfg, seed), DT[dt])
    toks = reqs["r3"]
    streams, taps = [], []
    plain.forward(toks, w, cfg, streams)
    eng = _engine(d, dt, page, 256)
    eng.model.tap = lambda i, x: taps.append(x.detach().cpu().numpy().copy())
    eng.step([StepEntry("a", toks, [0])])
    assert len(taps) == len(streams) == len(plain.layer_runs(cfg))
    for i, (got, ref) in enumerate(zip(taps, streams)):
        e = np.abs(got - ref).max(axis=-1) / np.abs(ref).max()
        assert (e.max() if dt == "float32" else np.quantile(e, 0.9)) < TOL[dt], (i, e.max())


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_long_decoding_through_recorded_steps(models, dt):
    from litinfer_amd.engine import StepEntry
    cfg, page, seed = cases.CASES["A"]
    d, _, _ = models[("A", dt)]
    w = cases.stored(cases.draw_weights(cfg, seed), DT[dt])
    toks = np.random.default_rng(3).integers(0, cfg["vocab"], 170).tolist()
    ref = plain.forward(toks, w, cfg)
    eng = _engine(d, dt, page, 256)
    rows = [eng.step([StepEntry("a", toks[:20], list(range(20)))]).float().cpu().numpy()]
    rows += [eng.step([StepEntry("a", [toks[i]], [0])]).float().cpu().numpy().copy() for i in range(20, 170)]
    assert eng.graph_replays > 100
    check_rows({"a": np.concatenate(rows)}, {"a": ref}, dt, "150 tokens decoded")


def test_a_slot_that_is_used_again_forgets_the_last_token(models):
    """Requests follow each other on the same slots; a request's first token takes the pair table's last row whatever
    the slot's last request ended with, and a request that sits out steps keeps its own last token."""
    from litinfer_amd.engine import StepEntry
    cfg, page, _ = cases.CASES["B"]
    d, reqs, ref = models[("B", "float32")]
    eng = _engine(d, "float32", page, 1024)
    for rnd in range(3):
        for r in ("r0", "r1", "r2", "r5", "r7"):
            toks = reqs[r]
            out = _rows(eng, r, toks, [0, 1, len(toks)] if len(toks) > 1 else [0, 1])
            eng.finish(r)
            assert schedules.rel_err(out, ref[r]) < 2e-5, (rnd, r)
    # two requests take turns, one token a step each: every one continues from its own last token
    a, b = reqs["r1"], reqs["r2"]
    got = {"a": [], "b": []}
    for i in range(12):
        got["a"].append(eng.step([StepEntry("a", [a[i]], [0])]).float().cpu().numpy().copy())
        got["b"].append(eng.step([StepEntry("b", [b[i]], [0])]).float().cpu().numpy().copy())
    assert schedules.rel_err(np.concatenate(got["a"]), ref["r1"][:12]) < 2e-5
    assert schedules.rel_err(np.concatenate(got["b"]), ref["r2"][:12]) < 2e-5


def test_tokens_that_the_device_chose_count_as_previous_tokens(models):
    """A token that enters a step from the feedback buffer (the host does not know it) is the next token's predecessor."""
    from litinfer_amd.engine import StepEntry
    cfg, page, _ = cases.CASES["A"]
    d, reqs, ref = models[("A", "float32")]
    toks = reqs["r2"]
    eng = _engine(d, "float32", page, 256)
    eng.feedback[:len(toks)] = torch.tensor(toks, dtype=torch.int32, device=DEV)
    rows = [eng.step([StepEntry("a", [0] * 7, list(range(7)), take=list(range(7)))]).float().cpu().numpy()]
    rows += [eng.step([StepEntry("a", [0], [0], take=[i])]).float().cpu().numpy().copy() for i in range(7, 12)]
    rows += [eng.step([StepEntry("a", toks[12:], list(range(len(toks) - 12)))]).float().cpu().numpy()]
    assert schedules.rel_err(np.concatenate(rows), ref["r2"]) < 2e-5


def test_greedy_generation_through_the_entry_point(models):
    from litinfer_amd import models as entry
    cfg, page, seed = cases.CASES["A"]
    d, reqs, _ = models[("A", "float32")]
    w = cases.stored(cases.draw_weights(cfg, seed), torch.float32)
    lm = entry.load(d, dtype="float32", device=DEV, page_size=page, max_tokens=512, max_seqs=4)
    prompt = reqs["r1"]
    new = list(lm.generate(prompt, max_new_tokens=12, top_k=1, top_p=1.0, temperature=1.0))
    assert len(new) == 12
    seq = list(prompt)
    for t in new:
        logits = plain.forward(seq, w, cfg)[-1]
        top = np.argsort(logits)[::-1]
        assert t == top[0] or logits[top[0]] - logits[t] < 1e-4 * np.abs(logits).max(), (len(seq), t, top[:3])
        seq.append(int(t))


def test_several_requests_through_the_scheduler(models):
    """Continuous batching of five prompts on four state slots (tokens are fed back on the device, the scheduler
    looks ahead): each request's greedy tokens are those of the request alone."""
    from litinfer_amd import models as entry
    cfg, page, seed = cases.CASES["C"]
    d, reqs, _ = models[("C", "float32")]
    lm = entry.load(d, dtype="float32", device=DEV, page_size=page, max_tokens=1024, max_seqs=4)
    prompts = [reqs[r] for r in ("r0", "r1", "r2", "r5", "r7")]
    alone = [list(lm.generate(p, max_new_tokens=8)) for p in prompts]
    lm.engine_start()
    ids = [lm.engine_add_request(p, 8) for p in prompts]
    while lm.engine_has_unfinished():
        lm.engine_step()
    got = {i: list(lm.engine_get_output(i)) for i in ids}
    assert [got[i] for i in ids] == alone


# ------------------------------------------------------------------------------------------- a standout key
def _standout_model(tmp, dt):
    """One attention layer (and a second layer behind it) whose weights make ONE key win: token A's key scores e^14
    with token B's query in every head, through the unrotated parts, and A's value is large.  Whether B sees A decides
    B's logits."""
    heads, dn, dr, dv, rank, q_rank, scale = 2, 16, 8, 16, 32, 24, 0.25
    cfg = {"architecture": "Nusuvik", "vocab": 64, "width": 64, "norm": {"eps": 1e-6},
           "embedding": {"bigram": {"buckets": 11, "mul_prev": 3, "mul_cur": 2}},
           "layers": [cases.latent_layer(heads, dn, dr, dv, rank, q_rank, scale, None),
                      cases.latent_layer(3, 8, 4, 8, 12, 10, 0.3, cases.dense(48))]}
    w = cases.draw_weights(cfg, 5)
    A, B = 63, 62
    w["embed"][:, :2] = 0.0
    w["embed"][A] = 0.0
    w["embed"][B] = 0.0
    w["embed"][A, 0] = w["embed"][B, 1] = 24.0
    w["bigram"] *= 0.05
    w["bigram"][:, :2] = 0.0
    w["l0.norm1"][:] = 1.0
    w["l0.norm1.b"][:] = 0.0
    w["l0.mix.dkv.norm"][:] = 1.0
    w["l0.mix.dq.norm"][:] = 1.0
    rng = np.random.default_rng(1)
    unit = lambda n: (lambda v: v / np.linalg.norm(v))(rng.normal(size=n))
    dk, dq = unit(rank), unit(q_rank)
    w["l0.mix.dkv"][:rank, 0] += 3.0 * dk                              # A's latent points along dk, B's query latent along dq
    w["l0.mix.dq"][:, 1] += 3.0 * dq
    a = math.sqrt(14.0 / (scale * math.sqrt(rank * q_rank)))
    for h in range(heads):
        p = unit(dn)
        w["l0.mix.uk"][h * dn:(h + 1) * dn] += a * np.outer(p, dk)
        w["l0.mix.uq"][h * (dn + dr):h * (dn + dr) + dn] += a * np.outer(p, dq)
        w["l0.mix.uv"][h * dv:(h + 1) * dv] += 3.0 * np.outer(rng.normal(size=dv), dk) / math.sqrt(rank)
    d = cases.write_model(tmp, cfg, w, DT[dt])
    return cfg, cases.stored(w, DT[dt]), d, A, B


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(tmp_path, dt):
    from litinfer_amd.engine import StepEntry
    cfg, w, d, A, B = _standout_model(tmp_path / "m", dt)
    rng = np.random.default_rng(4)
    toks = rng.integers(0, 60, 420).tolist()
    toks[3], toks[400] = A, B
    ref = plain.forward(toks, w, cfg)
    other = list(toks)
    other[3] = 5
    assert np.abs(plain.forward(other, w, cfg)[400] - ref[400]).max() > 0.1 * np.abs(ref[400]).max()
    for cuts in ([0, 420], [0, 390, 420], [0, 2, 5, 399, 401, 420]):
        out = _rows(_engine(d, dt, 16, 512), "a", toks, cuts)
        assert schedules.rel_err(out[395:], ref[395:]) < TOL[dt], cuts
    eng = _engine(d, dt, 16, 512)
    eng.step([StepEntry("a", toks[:398], [])])
    out = np.concatenate([eng.step([StepEntry("a", [toks[i]], [0])]).float().cpu().numpy().copy() for i in range(398, 404)])
    assert schedules.rel_err(out, ref[398:404]) < TOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("how", ["prompt", "portions", "decoded"])
def test_a_key_at_page_borders_at_the_query_and_behind_it(tmp_path, dt, how):
    """The key at the last and the first row of a page and at position 0; the query right behind the key, many pages
    later, and BEFORE it (the key must not be seen: the rows then equal those of a sequence without it)."""
    from litinfer_amd.engine import StepEntry
    cfg, w, d, A, B = _standout_model(tmp_path / "m", dt)
    rng = np.random.default_rng(3)
    page, moved = 8, []
    for pa, pb in ((0, 70), (7, 8), (8, 71), (15, 16), (16, 95), (31, 33), (40, 39)):
        toks = rng.integers(0, 60, max(pa, pb) + 4).tolist()
        toks[pa], toks[pb] = A, B
        ref = plain.forward(toks, w, cfg)
        without = list(toks)
        without[pa] = 7
        moved.append(np.abs(plain.forward(without, w, cfg)[pb] - ref[pb]).max() / np.abs(ref[pb]).max())
        eng = _engine(d, dt, page, 128)
        n = len(toks)
        if how == "prompt":
            out = _rows(eng, "a", toks, [0, n])
        elif how == "portions":                                  # a cut between the two, one right at the later one, portions of two
            lo, hi = min(pa, pb), max(pa, pb)
            out = _rows(eng, "a", toks, sorted({0, lo + 1, hi, hi + 2, n}))
        else:
            head = min(pa, pb) + 1
            rows = [eng.step([StepEntry("a", toks[:head], list(range(head)))]).float().cpu().numpy()]
            rows += [eng.step([StepEntry("a", [toks[i]], [0])]).float().cpu().numpy().copy() for i in range(head, n)]
            out = np.concatenate(rows)
        assert schedules.rel_err(out, ref) < TOL[dt], (pa, pb)
    # the test has teeth: the key, where it is seen, moves the query's logits by far more than the tolerance
    assert min(moved[:-1]) > 0.1 and moved[-1] == 0.0


# ------------------------------------------------------------------------------------------ mechanisms alone
def _ctx(q_lens, slots, positions):
    q_len = np.asarray(q_lens, dtype=np.int32)
    q_start = np.concatenate([[0], np.cumsum(q_len)[:-1]]).astype(np.int32)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(DEV)
    return SimpleNamespace(seg_of_token=dev(np.repeat(np.arange(len(q_len)), q_len)), q_start=dev(q_start), q_len=dev(q_len),
                           state_slots=dev(slots), positions=dev(positions))


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("V,H,buckets,mp,mc", [(50, 24, 7, 3, 5), (300, 130, 1021, 1000003, 77), (9, 8, 1, 1, 1), (40, 512, 64, 0, 1)])
def test_pair_embedding_across_steps_and_slots(dt, V, H, buckets, mp, mc):
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(V)
    table = torch.tensor(rng.normal(size=(V, H)), dtype=torch.float32).to(DT[dt])
    pair = torch.tensor(rng.normal(size=(buckets + 1, H)), dtype=torch.float32).to(DT[dt])
    seqs = {0: rng.integers(0, V, 40).tolist(), 2: rng.integers(0, V, 33).tolist(), 3: rng.integers(0, V, 3).tolist()}
    cfg = {"embedding": {"bigram": {"buckets": buckets, "mul_prev": mp, "mul_cur": mc}}}
    W = {"embed": table.double().numpy(), "bigram": pair.double().numpy()}
    ref = {s: plain.embed(t, W, cfg) for s, t in seqs.items()}
    last = torch.full((5,), 12345, dtype=torch.int32, device=DEV)            # what earlier requests left in the slots
    at = {s: 0 for s in seqs}
    for step in ([(0, 1), (2, 5)], [(2, 1), (0, 2)], [(0, 1)], [(3, 3), (0, 20), (2, 2)], [(2, 25), (0, 16)]):
        ids = np.concatenate([seqs[s][at[s]:at[s] + n] for s, n in step]).astype(np.int32)
        pos = np.concatenate([np.arange(at[s], at[s] + n) for s, n in step])
        c = _ctx([n for _, n in step], [s for s, _ in step], pos)
        out = torch.empty(len(ids), H, device=DEV)
        ops.pair_embedding(torch.from_numpy(ids).to(DEV), table.to(DEV), pair.to(DEV), out, c.positions, c.seg_of_token, c.q_start,
                           c.q_len, c.state_slots, last, buckets, mp, mc)
        o = 0
        for s, n in step:
            np.testing.assert_allclose(out[o:o + n].cpu().numpy(), ref[s][at[s]:at[s] + n], rtol=1e-6, atol=1e-6)
            at[s] += n
            o += n
            assert int(last[s]) == seqs[s][at[s] - 1]
    assert int(last[1]) == 12345 and int(last[4]) == 12345


def test_layer_norm_gelu_rows_side_by_side_and_gated_products():
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(0)
    f32 = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    for T, H in ((5, 96), (300, 320), (3, 4100), (2, 7), (70, 5000)):
        x, w, b = rng.normal(2.0, 3.0, (T, H)), rng.normal(1, 0.2, H), rng.normal(0, 0.3, H)
        ref = plain.layer_norm(x, w, b, 1e-5)
        for dt, tol in ((torch.float32, 2e-5), (torch.bfloat16, 1e-2)):
            out = torch.empty(T, H, dtype=dt, device=DEV)
            ops.layernorm(f32(x), f32(w), f32(b), 1e-5, out)
            assert np.abs(out.float().cpu().numpy() - ref).max() < tol * np.abs(ref).max(), (T, H)
    z = np.linspace(-9, 9, 1001)
    out = torch.empty(1001, device=DEV)
    ops.gelu_tanh(f32(z), out)
    assert np.abs(out.cpu().numpy() - plain.gelu_tanh(z)).max() < 2e-6
    a, b = rng.normal(size=(9, 37)), rng.normal(size=(9, 37))
    both = torch.empty(9, 74, device=DEV)
    ops.concat_rows(f32(a), f32(b), both)
    assert np.allclose(both.cpu().numpy(), np.concatenate([a, b], axis=1).astype(np.float32))
    # per-head products with a sigmoid gate a head, on both paths (few tokens and odd sizes; the matrix cores)
    for T, nh, n_out, n_in, dt in ((5, 3, 20, 24, torch.float32), (70, 4, 64, 32, torch.bfloat16), (3, 2, 7, 40, torch.bfloat16)):
        m = torch.tensor(rng.normal(size=(nh, n_out, n_in)), dtype=torch.float32).to(dt)
        x = torch.tensor(rng.normal(size=(T, nh * n_in)), dtype=torch.float32).to(dt)
        wide = f32(rng.normal(size=(T, nh + 9)))
        g = wide[:, 4:4 + nh]
        out = torch.empty(T, nh * n_out, dtype=dt, device=DEV)
        ops.headwise_linear(x.to(DEV), nh * n_in, n_in, m.to(DEV), out, nh * n_out, n_out, T, gate=g)
        ref = np.einsum("hjk,thk->thj", m.double().numpy(), x.double().numpy().reshape(T, nh, n_in))
        ref = ref * plain.sigmoid(g.double().cpu().numpy())[:, :, None]
        assert np.abs(out.float().cpu().numpy().reshape(T, nh, n_out) - ref).max() < (1e-5 if dt is torch.float32 else 2e-2) * np.abs(ref).max()


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("T,nh,n_out,n_in,tail,mdt", [(5, 3, 40, 24, 8, torch.float32), (70, 4, 64, 32, 64, torch.bfloat16),
                                                      (33, 2, 20, 48, 2, torch.bfloat16), (200, 8, 192, 64, 32, torch.bfloat16)])
def test_per_head_product_that_rotates_the_columns_behind_its_inputs(split, T, nh, n_out, n_in, tail, mdt):
    """Queries into the latent space: a head's plain columns are multiplied, its rotated columns behind them are
    rotated and written behind the outputs, on both paths of the kernel."""
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(T)
    f32 = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    m = torch.tensor(rng.normal(size=(nh, n_out, n_in)), dtype=torch.float32).to(mdt)
    x = rng.normal(size=(T, nh, n_in + tail))
    pos = rng.integers(0, 900, T)
    ang = pos[:, None] * np.array([70.0 ** (-2.0 * i / tail) for i in range(tail // 2)])
    out = torch.full((T, nh, n_out + tail), 7.0, device=DEV)
    ops.headwise_linear(f32(x.reshape(T, -1)), nh * (n_in + tail), n_in + tail, m.to(DEV), out, nh * (n_out + tail), n_out + tail, T,
                        rotate_tail=(tail, f32(np.cos(ang)), f32(np.sin(ang)), split))
    got = out.cpu().numpy()
    ref = np.einsum("hjk,thk->thj", m.double().numpy(), x[:, :, :n_in])
    assert np.abs(got[:, :, :n_out] - ref).max() < (1e-5 if mdt is torch.float32 else 2e-2) * np.abs(ref).max()
    for h in range(nh):
        r = x[:, h, n_in:]
        if split:
            want = plain.rotate_half(r, pos, 70.0, tail)
        else:
            want = np.empty_like(r)
            want[:, 0::2] = r[:, 0::2] * np.cos(ang) - r[:, 1::2] * np.sin(ang)
            want[:, 1::2] = r[:, 1::2] * np.cos(ang) + r[:, 0::2] * np.sin(ang)
        assert np.abs(got[:, h, n_out:] - want).max() < 2e-5 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,dn,dr,rank,q_rank", [(3, 24, 8, 40, 56), (1, 48, 16, 64, 32), (4, 32, 64, 64, 96), (5, 8, 24, 8, 16)])
def test_norms_rotation_and_page_write_of_the_latent_mixer(dt, nh, dn, dr, rank, q_rank):
    """The kernel between the projections and the attention, in the three calls the mixer makes of it: the latents'
    norms with the shared key part rotated into the page; the queries' rotated parts; and both at once."""
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(nh + rank)
    T, page, eps, base = 21, 8, 1e-5, 300.0
    f32 = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    pos = rng.integers(0, 500, T)
    freq = np.array([base ** (-2.0 * i / dr) for i in range(dr // 2)])
    ang = pos[:, None].astype(np.float64) * freq
    cos, sin = f32(np.cos(ang)), f32(np.sin(ang))
    packed = rng.normal(size=(T, q_rank + rank + dr + 3))
    q = rng.normal(size=(T, nh * (dn + dr)))
    wc, wq = rng.normal(1, 0.1, rank), rng.normal(1, 0.1, q_rank)
    slots = rng.permutation(4 * page)[:T].astype(np.int32)
    cache = torch.zeros(4, 1, page, rank + dr, dtype=DT[dt], device=DEV)
    cq = torch.empty(T, q_rank, dtype=DT[dt], device=DEV)
    pd = f32(packed)
    down = pd[:, q_rank:q_rank + rank + dr]
    ops.latent_norm_pairs_store(None, 0, dn, dr, rank, f32(wc), eps, cos, sin, torch.from_numpy(slots).to(DEV), cache, None,
                                down=down, half_split=True, q_latent=pd[:, :q_rank], wq=f32(wq), cq=cq)
    qfull = torch.zeros(T, nh, rank + dr, device=DEV)
    ops.latent_norm_pairs_store(f32(q), nh, dn, dr, rank, f32(wc), eps, cos, sin, None, None, qfull, down=down, half_split=True)
    tol = 1e-5 if dt == "float32" else 1e-2
    ref_cq = plain.rms(packed[:, :q_rank], eps) * wq
    assert np.abs(cq.float().cpu().numpy() - ref_cq).max() < tol * np.abs(ref_cq).max()
    ref_row = np.concatenate([plain.rms(packed[:, q_rank:q_rank + rank], eps) * wc,
                              plain.rotate_half(packed[:, q_rank + rank:q_rank + rank + dr], pos, base, dr)], axis=1)
    got = cache.float().cpu().numpy().reshape(4 * page, rank + dr)[slots]
    assert np.abs(got - ref_row).max() < tol * np.abs(ref_row).max()
    untouched = np.setdiff1d(np.arange(4 * page), slots)
    assert not cache.float().cpu().numpy().reshape(4 * page, rank + dr)[untouched].any()
    for h in range(nh):
        ref_q = plain.rotate_half(q[:, h * (dn + dr) + dn:(h + 1) * (dn + dr)], pos, base, dr)
        assert np.abs(qfull[:, h, rank:].cpu().numpy() - ref_q).max() < 2e-5 * np.abs(ref_q).max()
    # the form with the queries in front of the latent in one row, neighbouring pairs: what the other design calls
    qd = np.concatenate([q, packed[:, q_rank:q_rank + rank + dr]], axis=1)
    cache2 = torch.zeros_like(cache)
    qfull2 = torch.zeros_like(qfull)
    ops.latent_norm_pairs_store(f32(qd), nh, dn, dr, rank, f32(wc), eps, cos, sin, torch.from_numpy(slots).to(DEV), cache2, qfull2)
    kr = packed[:, q_rank + rank:q_rank + rank + dr]
    pairs = np.empty_like(kr)
    pairs[:, 0::2] = kr[:, 0::2] * np.cos(ang) - kr[:, 1::2] * np.sin(ang)
    pairs[:, 1::2] = kr[:, 1::2] * np.cos(ang) + kr[:, 0::2] * np.sin(ang)
    got2 = cache2.float().cpu().numpy().reshape(4 * page, rank + dr)[slots]
    assert np.abs(got2[:, rank:] - pairs).max() < tol * np.abs(pairs).max() and np.abs(got2[:, :rank] - ref_row[:, :rank]).max() < tol * 4


@pytest.mark.parametrize("E,top,groups,keep", [(6, 2, 3, 2), (12, 3, 4, 2), (8, 2, 4, 1), (4, 2, 4, 2), (5, 5, 1, 1), (64, 6, 8, 3), (4, 1, 1, 1)])
def test_sigmoid_router_with_groups(E, top, groups, keep):
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(E + top)
    T, K = 150, 40
    x = rng.normal(size=(T, K))
    wr = rng.normal(0, 3 / math.sqrt(K), (E, K))
    corr = rng.normal(0, 0.4, E) - 0.5                                  # negative choice values are common
    r = {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}
    picks, weights = plain.route(x, {"router": wr, "correction": corr}, "", r)
    f32 = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    idx = torch.empty(T, top, dtype=torch.int32, device=DEV)
    wt = torch.empty(T, top, device=DEV)
    ops.moe_route(f32(x), f32(wr), None, None, idx, wt, None, scores="sigmoid", correction=f32(corr), groups=groups, keep_groups=keep)
    assert idx.cpu().tolist() == picks
    assert np.abs(wt.cpu().numpy() - np.array(weights)).max() < 1e-5
    assert np.allclose(wt.cpu().numpy().sum(axis=1), 1.0, atol=1e-5)


def test_equal_choice_values_take_the_lower_expert_and_the_lower_group():
    from litinfer_amd.kernels import ops
    x = torch.ones(2, 32, device=DEV)
    router = torch.zeros(8, 32, device=DEV)
    idx = torch.empty(2, 3, dtype=torch.int32, device=DEV)
    wt = torch.empty(2, 3, device=DEV)
    ops.moe_route(x, router, None, None, idx, wt, None, scores="sigmoid", correction=torch.zeros(8, device=DEV), groups=4, keep_groups=2)
    assert idx.cpu().tolist() == [[0, 1, 2]] * 2 and np.allclose(wt.cpu().numpy(), 1 / 3, atol=1e-6)
    # experts outside the kept groups are out whatever their value: every choice value is negative here
    corr = torch.tensor([-3.0, -3.0, -1.0, -9.0, -2.0, -2.0, -4.0, -4.0], device=DEV)
    i2 = torch.empty(2, 2, dtype=torch.int32, device=DEV)
    w2 = torch.empty(2, 2, device=DEV)
    ops.moe_route(x, router, None, None, i2, w2, None, scores="sigmoid", correction=corr, groups=4, keep_groups=1)
    assert i2.cpu().tolist() == [[4, 5]] * 2                            # group sums -5, -9, -3, -7


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,K,E,top,ff,groups,keep", [(1, 96, 6, 2, 40, 3, 2), (70, 128, 8, 2, 64, 4, 2), (300, 64, 3, 3, 48, 1, 1),
                                                      (9, 128, 4, 1, 72, 2, 1), (2200, 256, 4, 2, 160, 1, 1), (600, 128, 8, 2, 96, 2, 1)])
def test_routed_feed_forward_with_gated_experts(dt, T, K, E, top, ff, groups, keep):
    """The part itself (router, plan, products by tile, activation, weighted sum) against the plain one, on tokens
    whose choice of experts and of groups is no close call for the rounding of the engine's dtype."""
    from litinfer_amd.config.spec import PartSpec
    from litinfer_amd.engine.workspace import Workspace
    from litinfer_amd.parts.base import Runtime, build_part
    from litinfer_amd.parts.stream import ResidualStream
    rng = np.random.default_rng(T + E)
    tdt = DT[dt]
    rnd = lambda a: torch.tensor(a, dtype=torch.float32).to(tdt)
    w = {"router": rng.normal(0, 3 / math.sqrt(K), (E, K)), "correction": rng.normal(0, 0.3, E)}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"] = rng.normal(0, 1 / math.sqrt(K), (ff, K)), rng.normal(0, 1 / math.sqrt(K), (ff, K))
        w[f"e{e}.down"] = rng.normal(0, 1 / math.sqrt(ff), (K, ff))
    wt = {n: rnd(a) for n, a in w.items()}
    w64 = {n: a.double().numpy() for n, a in wt.items()}
    mlp = {"router": {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}}
    # tokens whose choice is clear: moving every choice value by the dtype's rounding changes nothing
    cand = rnd(rng.normal(size=(6 * T + 40, K)))
    c64 = cand.double().numpy()
    margin = 1e-4 if dt == "float32" else 2e-2
    nudge = np.random.default_rng(1).uniform(-margin, margin, (3, E))
    base_picks = plain.route(c64, w64, "", mlp["router"])[0]
    ok = np.ones(len(cand), bool)
    for n in nudge:
        moved = plain.route(c64, {"router": w64["router"], "correction": w64["correction"] + n}, "", mlp["router"])[0]
        ok &= np.array([sorted(a) == sorted(b) for a, b in zip(base_picks, moved)])
    assert ok.sum() >= T
    h = cand[np.nonzero(ok)[0][:T]]
    part = build_part("feed_forward", PartSpec("routed_mlp", "", {"hidden_size": K, "experts": E, "top": top, "intermediate_size": ff,
                                                                   "activation": "swiglu", "scores": "sigmoid", "correction": True,
                                                                   "router_bias": False, "groups": groups, "keep_groups": keep}),
                      Runtime(torch.device(DEV), tdt))
    part.load_params(lambda n: wt[n])
    x0 = rng.normal(size=(T, K))
    x = torch.tensor(x0, dtype=torch.float32, device=DEV)
    ws = Workspace(DEV)
    part.forward(h.to(DEV), ResidualStream(x, ws), SimpleNamespace(ws=ws))
    ref = plain.moe_mlp(h.double().numpy(), w64, "", mlp)
    e = np.abs(x.cpu().numpy() - x0 - ref).max(axis=1) / np.abs(ref).max()
    print(f"[observed] routed feed-forward {dt} {T, K, E, top, ff, groups, keep}: worst {e.max():.3e}")
    assert (e.max() if dt == "float32" else np.quantile(e, 0.95)) < (1e-5 if dt == "float32" else 2e-2)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_dense_feed_forward_with_biases(dt):
    from litinfer_amd.config.spec import PartSpec
    from litinfer_amd.engine.workspace import Workspace
    from litinfer_amd.parts.base import Runtime, build_part
    from litinfer_amd.parts.stream import ResidualStream
    rng = np.random.default_rng(2)
    for T, K, ff in ((3, 96, 120), (150, 128, 200), (40, 72, 36)):
        w = {"up": rng.normal(0, 1 / math.sqrt(K), (ff, K)), "up.b": rng.normal(0, 0.5, ff),
             "down": rng.normal(0, 1 / math.sqrt(ff), (K, ff)), "down.b": rng.normal(0, 0.5, K)}
        wt = {n: torch.tensor(a, dtype=torch.float32).to(DT[dt]) for n, a in w.items()}
        part = build_part("feed_forward", PartSpec("gelu_mlp", "", {"hidden_size": K, "intermediate_size": ff}), Runtime(torch.device(DEV), DT[dt]))
        part.load_params(lambda n: wt[n])
        h = torch.tensor(rng.normal(size=(T, K)), dtype=torch.float32).to(DT[dt])
        x0 = rng.normal(size=(T, K))
        x = torch.tensor(x0, dtype=torch.float32, device=DEV)
        ws = Workspace(DEV)
        part.forward(h.to(DEV), ResidualStream(x, ws), SimpleNamespace(ws=ws))
        ref = plain.dense_mlp(h.double().numpy(), {n: a.double().numpy() for n, a in wt.items()}, "")
        assert np.abs(x.cpu().numpy() - x0 - ref).max() < (1e-5 if dt == "float32" else 2e-2) * np.abs(ref).max()


# ------------------------------------------------------------------------------- as a user runs it, in a subprocess
def test_generate_through_the_command_line(models):
    from test_cli import cli, last_json
    cfg, page, seed = cases.CASES["D"]
    d, reqs, _ = models[("D", "float32")]
    w = cases.stored(cases.draw_weights(cfg, seed), torch.float32)
    prompt = reqs["r1"]
    out = last_json(cli("generate", "--model", d, "--test", "--max_steps", 10, "--dtype", "float32", "--page-size", page,
                        "--chunk-size", 6, "--prompt-ids", ",".join(map(str, prompt))).stdout)
    assert len(out["tokens"]) == 10
    seq = list(prompt)
    for t in out["tokens"]:
        logits = plain.forward(seq, w, cfg)[-1]
        assert logits.max() - logits[t] < 1e-4 * np.abs(logits).max(), (len(seq), t)
        seq.append(int(t))


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_trace_replay_in_a_subprocess(models, tmp_path, dt):
    from test_trace_run_gpu import replay
    d, reqs, ref = models[("C", dt)]
    some = {r: reqs[r] for r in ("r0", "r1", "r3", "r5", "r7", "r8")}
    for kind in ("chunks", "mixed"):
        steps = getattr(schedules, kind)(some)
        out = replay(d, dt, some, steps, tmp_path / f"out_{kind}", schedules.max_live_tokens(some, steps))
        check_rows(out, {r: ref[r] for r in some}, dt, f"replay {kind}")
