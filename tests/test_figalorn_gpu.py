"""The Figalorn decoder through the engine against the plain implementation (tests/plain/figalorn_plain.py):
whole prompts, decoding token by token, portions down to two tokens, unequal requests side by side with
pages and slots that come round again, long decoding past windows, chunks and pages, generation through
the engine's own entry point, the trace replay program, and each mechanism alone with inputs made so
that a fault shows (a mutated plain implementation must differ by far more than the tolerance)."""
import copy

import pytest
import torch

import axon_amd
from axon_amd.config.base import PartSpec
from axon_amd.config.figalorn import FigalornConfig
from axon_amd.engine import StepEntry
from axon_amd.parts import CacheBinding, build_part
from axon_amd.weights import WeightStore
from figalorn_models import MODELS, config, diff, draw_weights, keyed, layer, make
from gpu_helpers import DTYPES, DictSource, PartHarness
from helpers import TraceBuilder, engine_for, run_trace, tolerance
from plain import figalorn_plain as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = make(str(tmp_path_factory.mktemp("figalorn_" + name)), name)
        return made[name]
    return get


@pytest.fixture(scope="module")
def plain_logits(folders):
    kept = {}

    def get(name, seq):
        key = (name, tuple(seq))
        if key not in kept:
            cfg, W = P.load_plain(folders(name))
            kept[key] = P.forward(cfg, W, seq).float()
        return kept[key]
    return get


def sequences(name, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, MODELS[name]["cfg"]["vocab"], (n,), generator=g).tolist() for n in lengths]


def assert_close(got, ref, dtype, what):
    err = (got - ref).abs().max(dim=-1).values
    limit = tolerance(dtype, ref) * (1.0 if dtype == "float32" else 2.0)
    assert float(err.max()) <= limit, f"{what}: {float(err.max())} > {limit} at row {int(err.argmax())}"


def run_schedule(eng, seqs, schedule):
    """schedule: steps of [(request, tokens)]; every position's logits are asked for.  A request
    ends with its last token.  Returns {request: [len, vocab]}."""
    at = {r: 0 for r in seqs}
    got = {r: [] for r in seqs}
    for step in schedule:
        entries, ends = [], []
        for rid, n in step:
            toks = seqs[rid][at[rid]:at[rid] + n]
            entries.append(StepEntry(rid, toks, list(range(len(toks)))))
            at[rid] += len(toks)
            if at[rid] == len(seqs[rid]):
                ends.append(rid)
        out = eng.step(entries, ends).cpu()
        row = 0
        for e in entries:
            got[e.id].append(out[row:row + len(e.tokens)].clone())
            row += len(e.tokens)
    assert all(at[r] == len(seqs[r]) for r in seqs)
    return {r: torch.cat(v) for r, v in got.items()}


def pages_for(name, tokens):
    return -(-tokens // MODELS[name]["page"]) + 2


# --------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MODELS))
def test_whole_prompts_and_decoding_token_by_token(folders, plain_logits, name, dtype):
    n = 150
    (seq,) = sequences(name, [n], seed=1)
    ref = plain_logits(name, seq)
    eng = engine_for(folders(name), dtype, MODELS[name]["page"], pages_for(name, n), max_seqs=2, max_seq_len=256)
    whole = run_schedule(eng, {"a": seq}, [[("a", n)]])["a"]
    assert_close(whole, ref, dtype, "whole prompt")
    # from the first token on, one token a step: the first tokens of a sequence, every window's, chunk's and page's edge
    single = run_schedule(eng, {"b": seq}, [[("b", 1)] for _ in range(n)])["b"]
    assert_close(single, ref, dtype, "token by token")
    both = run_schedule(eng, {"c": seq}, [[("c", n - 90)]] + [[("c", 1)] for _ in range(90)])["c"]
    assert_close(both, ref, dtype, "prompt then decoding")
    if dtype == "float32":
        assert float((single - whole).abs().max()) <= 2 * tolerance(dtype, ref)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MODELS))
def test_portions_of_many_sizes_down_to_two_tokens(folders, plain_logits, name, dtype):
    n = 200
    (seq,) = sequences(name, [n], seed=2)
    ref = plain_logits(name, seq)
    eng = engine_for(folders(name), dtype, MODELS[name]["page"], pages_for(name, n), max_seqs=2, max_seq_len=256)
    for cuts in ([2, 2, 3, 1, 2, 7, 1, 1, 5, 64, 2], [63, 2, 1, 64, 9], [8, 8, 1, 16, 2], [17, 16, 15, 33]):
        sched, left, i = [], n, 0
        while left:
            take = min(cuts[i % len(cuts)], left)
            sched.append([("a", take)])
            left -= take
            i += 1
        got = run_schedule(eng, {"a": seq}, sched)["a"]
        assert_close(got, ref, dtype, f"portions {cuts}")
    eng.cache.check()


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MODELS))
def test_unequal_requests_side_by_side_with_pages_and_slots_used_again(folders, plain_logits, name, dtype, graphs):
    lengths = [57, 5, 140, 33, 1, 76]
    seqs = dict(enumerate(sequences(name, lengths, seed=3)))
    refs = {r: plain_logits(name, s) for r, s in seqs.items()}
    page = MODELS[name]["page"]
    # three slots and a pool for the three longest live at once: later requests get the pages and slots of finished ones
    eng = engine_for(folders(name), dtype, page, 3 * (-(-140 // page)) + 1, max_seqs=3, max_seq_len=192, shuffle_pages_seed=5,
                     use_graphs=graphs)
    cuts = {0: [9, 1, 1, 2, 30, 1], 1: [2, 1, 1, 1], 2: [1, 40, 1, 1, 3, 64, 1], 3: [33], 4: [1], 5: [2, 1, 50, 1, 1, 1]}
    at = {r: 0 for r in seqs}
    waiting, live, sched, turn = [0, 1, 2, 3, 4, 5], [], [], 0
    while waiting or live:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        step = []
        for r in list(live):
            if (turn + r) % 4 == 3 and len(live) > 1:
                continue                                  # left out of this step, goes on later
            n = min(cuts[r][(turn // 2) % len(cuts[r])], lengths[r] - at[r])
            step.append((r, n))
            at[r] += n
            if at[r] == lengths[r]:
                live.remove(r)
        if step:
            sched.append(step)
        turn += 1
    got = run_schedule(eng, seqs, sched)
    for r in seqs:
        assert_close(got[r], refs[r], dtype, f"request {r} in the mixed schedule")
    eng.cache.check()
    assert not eng.live
    for g in range(len(eng.cache.groups)):
        assert eng.cache.free_pages(g) == eng.cache.groups[g].n_pages
    if dtype == "float32":
        alone = run_schedule(eng, {2: seqs[2]}, [[(2, lengths[2])]])[2]
        assert float((alone - got[2]).abs().max()) <= 2 * tolerance(dtype, refs[2])


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("A", "bfloat16")])
def test_long_decoding_far_past_windows_chunks_and_pages(folders, plain_logits, name, dtype):
    n = 330
    (seq,) = sequences(name, [n], seed=4)
    ref = plain_logits(name, seq)
    eng = engine_for(folders(name), dtype, MODELS[name]["page"], pages_for(name, n), max_seqs=1, max_seq_len=384)
    got = run_schedule(eng, {"a": seq}, [[("a", 3)]] + [[("a", 1)] for _ in range(n - 3)])["a"]
    assert_close(got, ref, dtype, "long decoding")


@pytest.mark.parametrize("name", sorted(MODELS))
def test_greedy_generation_through_the_entry_point(folders, name):
    cfg, W = P.load_plain(folders(name))
    prompts = sequences(name, [11, 3, 30], seed=6)
    want = [P.greedy_generate(cfg, W, p, 10) for p in prompts]
    page = MODELS[name]["page"]
    llm = axon_amd.load(folders(name), dtype="float32", page_size=page, num_pages=24, max_seqs=3, max_seq_len=128)
    assert llm.generate(prompts, max_new_tokens=10) == want                       # decoding steps replay graphs
    assert llm.engine.graphs_ok and all(c for c, _, _ in llm.engine._segments)
    assert llm.generate(prompts[:1], max_new_tokens=10) == want[:1]               # alone, in a slot used before
    eager = axon_amd.load(folders(name), dtype="float32", page_size=page, num_pages=24, max_seqs=3, max_seq_len=128,
                          use_graphs=False)
    assert eager.generate(prompts, max_new_tokens=10) == want
    half = axon_amd.load(folders(name), dtype="bfloat16", page_size=page, num_pages=24, max_seqs=3, max_seq_len=128)
    for p, o in zip(prompts, half.generate(prompts, max_new_tokens=10)):
        logits = P.forward(cfg, W, p + o).float()
        for i, tok in enumerate(o):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= 20 * tolerance("bfloat16", logits)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_replay_program_runs_the_design(folders, plain_logits, tmp_path, dtype):
    name = "A"
    seqs = sequences(name, [90, 17, 130], seed=7)
    refs = [plain_logits(name, s) for s in seqs]
    tb = TraceBuilder()
    tb.step([("a", seqs[0][:70], [0, 69]), ("b", seqs[1][:2], [1])])
    tb.step([("a", seqs[0][70:71], [0]), ("b", seqs[1][2:], [0, 14]), ("c", seqs[2][:7], [])], end=["b"])
    tb.step([("a", seqs[0][71:], [18]), ("c", seqs[2][7:], [0, 122])], end=["a", "c"])
    rows = tb.collect(run_trace(folders(name), dtype, tb.steps, str(tmp_path), max_tokens=384))
    for (rid, pos), row in rows.items():
        ref = refs["abc".index(rid)]
        assert float((torch.from_numpy(row) - ref[pos]).abs().max()) <= 3 * tolerance(dtype, ref)


def test_the_command_line_generates_with_the_design(folders):
    import os
    import subprocess
    import sys
    from helpers import ROOT
    name = "A"
    cfg, W = P.load_plain(folders(name))
    p, q = sequences(name, [9, 14], seed=9)
    axon = [sys.executable, os.path.join(ROOT, "bin", "axon")]
    ids = lambda seq: " ".join(map(str, seq))
    r = subprocess.run(axon + ["gen", folders(name), ids(p), ids(q), "-n", "8", "--dtype", "float32", "--page-size", "64"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [[int(t) for t in line.split()] for line in r.stdout.splitlines()] == [
        P.greedy_generate(cfg, W, p, 8), P.greedy_generate(cfg, W, q, 8)]
    r = subprocess.run(axon + ["logits", folders(name), ids(p), "-k", "3", "--dtype", "float32"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr
    top = torch.topk(P.forward(cfg, W, p)[-1].float(), 3)
    lines = [l.split() for l in r.stdout.splitlines() if "logit" in l]
    assert [int(l[0]) for l in lines] == top.indices.tolist()


# --------------------------------------------------------------------------- the mixers alone
def rows_in(T, width, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(T, width, generator=g)
    return h.to(torch.bfloat16).float() if dtype == "bfloat16" else h


def part_tol(dtype, ref):
    return (3e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))


def run_mixer(part, harness, h, cuts, width):
    """What the mixer adds to a residual stream of zeros for rows h, fed in portions of the given sizes."""
    outs, at = [], 0
    for n in cuts:
        ctx = harness.ctx([0] * n)
        x = h[at:at + n].to(harness.rt.dtype).cuda()
        out = torch.zeros((n, width), dtype=torch.float32, device="cuda")
        part.forward(ctx, CacheBinding(group=0, index=0, writes=True), x, out)
        outs.append(out.cpu())
        at += n
    assert at == h.shape[0]
    return torch.cat(outs)


def check_mixer(entry, width, page, dtype, T, seed=21, sharp=1.0):
    """One mixer alone, whole and in portions cut just before, at and behind its mask's edges, against the plain
    function; then the plain function with the mask one position off either way, which must differ by far more."""
    cfg = config(width, 16, [layer(entry, None)])
    W = {k: v for k, v in draw_weights(cfg, seed).items() if k.startswith("l0.")}
    m = copy.deepcopy(cfg["layers"][0]["mixer"])
    m["scale"] *= sharp
    cfg["layers"][0]["mixer"] = m
    spec = FigalornConfig(cfg).layers[0]["mixer"]
    part = build_part("mixer", spec, "l0.")
    size = m["mask"]["size"]
    h = rows_in(T, width, seed + 1, dtype)
    Wd = {k: v.double() for k, v in W.items()}
    plain = P.MIXERS[entry["type"]]
    eps = cfg["norm"]["eps"]
    ref = plain(h.double(), Wd, "l0.mix.", m, eps).float()
    first = max(size - 3, 2)
    for cuts in ([T], [first] + [1] * 8 + [T - first - 8], [2, 1, 1, 3] + [1] * 30 + [64, 2, T - 103], [16, 17, 15, T - 48]):
        hs = PartHarness(dtype, part.cache_spec(), page_size=page, n_pages=-(-T // page) + 3, max_seq_len=1024)
        part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
        got = run_mixer(part, hs, h, cuts, width)
        assert float((got - ref).abs().max()) <= part_tol(dtype, ref), cuts
    wrongs = [size - 1, size + 1] if size > 1 else [size + 1]
    for wrong in wrongs + ([T // 2] if size > T // 2 + 1 else []):
        off = copy.deepcopy(m)
        off["mask"]["size"] = wrong
        assert float((plain(h.double(), Wd, "l0.mix.", off, eps).float() - ref).abs().max()) > 20 * part_tol("float32", ref), wrong


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("entry,width,page", [
    (keyed(heads=4, kv_heads=2, dim=16, window=24, rot_dims=8), 64, 64),          # the matrix cores' smallest tile
    (keyed(heads=6, kv_heads=2, dim=80, window=64, rot_dims=80, softcap=3.0), 48, 64),     # a window of exactly a page
    (keyed(heads=2, kv_heads=1, dim=144, window=65, rot_dims=2), 64, 128),        # the largest tile, a page and one
    (keyed(heads=3, kv_heads=3, dim=12, window=1, rot_dims=4), 40, 8),            # any sizes; a token sees itself alone
    (keyed(heads=5, kv_heads=1, dim=20, window=130, rot_dims=20, scaling=None, softcap=0.0), 40, 16)])
def test_windowed_attention_whose_values_are_its_keys(entry, width, page, dtype):
    check_mixer(entry, width, page, dtype, T=max(2 * entry["mixer"]["mask"]["size"] + 70, 200))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("entry,width,page", [
    (diff(heads=4, kv_heads=2, dim=8, vdim=32, chunk=40, rot_dims=4), 64, 64),
    (diff(heads=2, kv_heads=2, dim=40, vdim=144, chunk=64, rot_dims=12, d=0.0), 64, 64),     # chunks of exactly a page
    (diff(heads=20, kv_heads=1, dim=16, vdim=16, chunk=129, rot_dims=16, scaling=None), 96, 128),
    (diff(heads=3, kv_heads=1, dim=6, vdim=10, chunk=7, rot_dims=6, d=0.5), 40, 8),
    (diff(heads=1, kv_heads=1, dim=10, vdim=4, chunk=1, rot_dims=2), 24, 4),                 # every token a chunk of its own
    (diff(heads=2, kv_heads=1, dim=8, vdim=320, chunk=30, rot_dims=4), 32, 16)])             # values wider than the matrix cores' tiles
def test_differential_attention_in_chunks(entry, width, page, dtype):
    check_mixer(entry, width, page, dtype, T=max(2 * entry["mixer"]["mask"]["size"] + 70, 200))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("entry", [keyed(heads=4, kv_heads=1, dim=32, window=700, rot_dims=16),
                                   diff(heads=2, kv_heads=1, dim=16, vdim=32, chunk=800, rot_dims=8)])
def test_keys_hundreds_of_positions_back_are_seen(entry, dtype):
    """900 positions in pages of 64 under a window of 700 and chunks of 800, with scores sharp enough that single keys
    decide rows: a mask of half the size (far keys left out) changes the result by far more than the tolerance."""
    check_mixer(entry, 64, 64, dtype, T=900, sharp=2.0 if dtype == "float32" else 1.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_rewrite_of_the_stream_at_the_start_of_a_pass(dtype):
    hs = PartHarness(dtype)
    width, T = 72, 19
    g = torch.Generator().manual_seed(3)
    W = {"loop.in": (torch.randn(width, 2 * width, generator=g) / width ** 0.5).to(torch.bfloat16).float()}
    part = build_part("stream", PartSpec("embedding_mix", {"hidden_size": width, "tensor": "loop.in"}))
    part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
    x, x0 = rows_in(T, width, 4, dtype), rows_in(T, width, 5, dtype)
    ref = (torch.cat([x, x0], dim=-1).double() @ W["loop.in"].double().T).float()
    got, kept = x.cuda(), x0.cuda()
    part.forward(hs.ctx([0] * T), got, kept)
    assert float((got.cpu() - ref).abs().max()) <= part_tol(dtype, ref) / 3
    assert torch.equal(kept.cpu(), x0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_feed_forward_with_the_exact_gelu(dtype):
    hs = PartHarness(dtype)
    width, ff, T = 56, 88, 33
    g = torch.Generator().manual_seed(9)
    W = {"mlp.up": (torch.randn(ff, width, generator=g) * 3 / width ** 0.5).to(torch.bfloat16).float(),
         "mlp.down": (torch.randn(width, ff, generator=g) / ff ** 0.5).to(torch.bfloat16).float()}
    part = build_part("feed_forward", PartSpec("dense_mlp", {"hidden_size": width, "ff": ff, "activation": "gelu_erf"}))
    part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
    h = rows_in(T, width, 10, dtype)
    ref = P.feed_forward(h.double(), {k: v.double() for k, v in W.items()}, "mlp.").float()
    out = torch.zeros((T, width), dtype=torch.float32, device="cuda")
    part.forward(hs.ctx([0] * T), h.to(hs.rt.dtype).cuda(), out)
    assert float((out.cpu() - ref).abs().max()) <= part_tol(dtype, ref)
    # the tanh form is another function (by little: the two differ by 5e-4 at most): in 32 bits it does not pass
    z = h.double() @ W["mlp.up"].double().T
    tanh_form = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
    other = float(((tanh_form @ W["mlp.down"].double().T).float() - ref).abs().max())
    assert other > 2 * part_tol("float32", ref)
    if dtype == "float32":
        assert float((out.cpu() - ref).abs().max()) <= other / 10


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_norm_whose_gain_is_stored_around_zero(dtype):
    hs = PartHarness(dtype)
    width, T = 100, 9
    g = torch.Generator().manual_seed(2)
    w = (torch.randn(width, generator=g) * 0.01).to(torch.bfloat16).float()      # 1 + w needs more digits than bfloat16 has
    part = build_part("norm", PartSpec("rmsnorm", {"size": width, "eps": 1e-5, "tensor": "n", "offset": 1.0}))
    part.load(WeightStore(DictSource({"n": w.to(torch.bfloat16)}), hs.rt.device, hs.rt.dtype), hs.rt)
    x = torch.randn(T, width, generator=g) * 5
    ref = P.norm(x.double(), w.double(), 1e-5).float()
    got = part.forward(hs.ctx([0] * T), x.cuda()).float().cpu()
    assert float((got - ref).abs().max()) <= (1e-5 if dtype == "float32" else 2e-2) * float(ref.abs().max())
