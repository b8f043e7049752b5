"""The Pikesun decoder through the engine against the plain implementation (tests/plain/pikesun_plain.py):
whole prompts, decoding token by token, portions down to two tokens, unequal requests side by side with
pages and state slots that come round again, long decoding past windows and pages, generation through
the engine's own entry point, the trace replay program, and every mechanism alone with inputs made
so that a fault shows (a mutated plain implementation must differ by far more than the tolerance)."""
import os

import pytest
import torch

import axon_amd
from axon_amd.config.base import PartSpec
from axon_amd.engine import StepEntry
from axon_amd.parts import CacheBinding, CacheSpec, build_part
from axon_amd.weights import WeightStore
from gpu_helpers import DTYPES, DictSource, PartHarness
from helpers import TraceBuilder, engine_for, run_trace, tolerance
from pikesun_models import MODELS, make
from plain import pikesun_plain as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            made[name] = make(str(tmp_path_factory.mktemp("pikesun_" + name)), name)
        return made[name]
    return get


@pytest.fixture(scope="module")
def plain_logits(folders):
    """The plain implementation's logits of a model's test sequences, worked out once."""
    kept = {}

    def get(name, seq):
        key = (name, tuple(seq))
        if key not in kept:
            cfg, W = P.load_plain(folders(name))
            kept[key] = P.forward_logits(cfg, W, seq).float()
        return kept[key]
    return get


def sequences(name, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, MODELS[name]["cfg"]["vocab"], (n,), generator=g).tolist() for n in lengths]


def assert_close(got, ref, dtype, what, routed=True):
    """Rows of logits against the plain implementation's.  float32: every row.  bfloat16: a router's
    close call may go the other way in 16 bits, and with one expert a token that is another expert:
    one row in twenty may miss (never by much)."""
    err = (got - ref).abs().max(dim=-1).values
    # 16 bits: norms on the sublayers' outputs pass every rounding on at full size; rows of these models
    # are off by up to 1.1 % of the logits' range where the pre-norm models' are by 0.3 %
    limit = tolerance(dtype, ref) * (1.0 if dtype == "float32" else 3.0)
    if dtype == "float32" or not routed:
        assert float(err.max()) <= limit, f"{what}: {float(err.max())} > {limit} at row {int(err.argmax())}"
    else:
        assert int((err > limit).sum()) <= max(2, len(err) // 20), f"{what}: {int((err > limit).sum())} rows of {len(err)} beyond {limit}"
        assert float(err.max()) <= 7 * limit, f"{what}: row {int(err.argmax())} is off by {float(err.max())}"


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
    n = 200 if name == "Q" else 70
    (seq,) = sequences(name, [n], seed=1)
    ref = plain_logits(name, seq)
    eng = engine_for(folders(name), dtype, MODELS[name]["page"], pages_for(name, n), max_seqs=2, max_seq_len=256)
    whole = run_schedule(eng, {"a": seq}, [[("a", n)]])["a"]
    assert_close(whole, ref, dtype, "whole prompt")
    # from the first token on, one token a step: the first tokens of a sequence, every window's and page's edge
    single = run_schedule(eng, {"b": seq}, [[("b", 1)] for _ in range(n)])["b"]
    assert_close(single, ref, dtype, "token by token")
    # most of it at once, the rest decoded
    both = run_schedule(eng, {"c": seq}, [[("c", n - 45)]] + [[("c", 1)] for _ in range(45)])["c"]
    assert_close(both, ref, dtype, "prompt then decoding")
    if dtype == "float32":
        assert float((single - whole).abs().max()) <= 2 * tolerance(dtype, ref)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MODELS))
def test_portions_of_many_sizes_down_to_two_tokens(folders, plain_logits, name, dtype):
    n = 230 if name == "Q" else 90
    (seq,) = sequences(name, [n], seed=2)
    ref = plain_logits(name, seq)
    eng = engine_for(folders(name), dtype, MODELS[name]["page"], pages_for(name, n), max_seqs=2, max_seq_len=256)
    for cuts in ([2, 2, 3, 1, 2, 7, 1, 1, 5, 64, 2], [63, 2, 1, 64, 9], [8, 8, 1, 16, 2]):
        sched, left, i = [], n, 0
        while left:
            take = min(cuts[i % len(cuts)], left)
            sched.append([("a", take)])
            left -= take
            i += 1
        got = run_schedule(eng, {"a": seq}, sched)["a"]
        assert_close(got, ref, dtype, f"portions {cuts}")
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MODELS))
def test_unequal_requests_side_by_side_with_pages_and_slots_used_again(folders, plain_logits, name, dtype):
    lengths = [57, 5, 120, 33, 1, 76]
    seqs = dict(enumerate(sequences(name, lengths, seed=3)))
    refs = {r: plain_logits(name, s) for r, s in seqs.items()}
    page = MODELS[name]["page"]
    # three slots and a pool for the three longest live at once: later requests get the pages and
    # the slots (with their state rows) of finished ones
    eng = engine_for(folders(name), dtype, page, 3 * (-(-120 // page)) + 1, max_seqs=3, max_seq_len=128, shuffle_pages_seed=5)
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
        # each request alone gives the same rows as side by side, to rounding
        alone = run_schedule(eng, {2: seqs[2]}, [[(2, lengths[2])]])[2]
        assert float((alone - got[2]).abs().max()) <= 2 * tolerance(dtype, refs[2])


@pytest.mark.parametrize("name", ["P", "R"])
def test_long_decoding_far_past_windows_and_pages(folders, plain_logits, name):
    n = 250
    (seq,) = sequences(name, [n], seed=4)
    ref = plain_logits(name, seq)
    eng = engine_for(folders(name), "float32", MODELS[name]["page"], pages_for(name, n), max_seqs=1, max_seq_len=256)
    got = run_schedule(eng, {"a": seq}, [[("a", 3)]] + [[("a", 1)] for _ in range(n - 3)])["a"]
    assert_close(got, ref, "float32", "long decoding")


@pytest.mark.parametrize("name", sorted(MODELS))
def test_greedy_generation_through_the_entry_point(folders, name):
    cfg, W = P.load_plain(folders(name))
    prompts = sequences(name, [11, 3, 30], seed=6)
    want = [P.greedy_generate(cfg, W, p, 10) for p in prompts]
    llm = axon_amd.load(folders(name), dtype="float32", page_size=MODELS[name]["page"], num_pages=24, max_seqs=3, max_seq_len=128)
    assert llm.generate(prompts, max_new_tokens=10) == want                       # decoding steps replay graphs
    assert llm.engine.graphs_ok and all(c for c, _, _ in llm.engine._segments)
    assert llm.generate(prompts[:1], max_new_tokens=10) == want[:1]               # alone, in a slot used before
    eager = axon_amd.load(folders(name), dtype="float32", page_size=MODELS[name]["page"], num_pages=24, max_seqs=3,
                          max_seq_len=128, use_graphs=False)
    assert eager.generate(prompts, max_new_tokens=10) == want
    half = axon_amd.load(folders(name), dtype="bfloat16", page_size=MODELS[name]["page"], num_pages=24, max_seqs=3, max_seq_len=128)
    for p, o in zip(prompts, half.generate(prompts, max_new_tokens=10)):
        logits = P.forward_logits(cfg, W, p + o).float()
        for i, tok in enumerate(o):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= 20 * tolerance("bfloat16", logits)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_replay_program_runs_the_design(folders, plain_logits, tmp_path, dtype):
    name = "P"
    seqs = sequences(name, [40, 17, 64], seed=7)
    refs = [plain_logits(name, s) for s in seqs]
    tb = TraceBuilder()
    tb.step([("a", seqs[0][:30], [0, 29]), ("b", seqs[1][:2], [1])])
    tb.step([("a", seqs[0][30:31], [0]), ("b", seqs[1][2:], [0, 14]), ("c", seqs[2][:7], [])], end=["b"])
    tb.step([("a", seqs[0][31:], [8]), ("c", seqs[2][7:], [0, 56])], end=["a", "c"])
    rows = tb.collect(run_trace(folders(name), dtype, tb.steps, str(tmp_path), max_tokens=192))
    for (rid, pos), row in rows.items():
        ref = refs["abc".index(rid)]
        assert float((torch.from_numpy(row) - ref[pos]).abs().max()) <= 3 * tolerance(dtype, ref)


# --------------------------------------------------------------------------- the mechanisms alone
def weights_of_layer(name, layer):
    from pikesun_models import draw_weights
    m = MODELS[name]
    W = draw_weights(m["cfg"], m["seed"])
    return m["cfg"], {k: v for k, v in W.items() if k.startswith(f"l{layer}.")}


def rows_in(T, width, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(T, width, generator=g)
    return h.to(torch.bfloat16).float() if dtype == "bfloat16" else h


def part_tol(dtype, ref):
    return (3e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))


def run_mixer(part, harness, h, cuts, width):
    """The mixer's 32-bit output for rows h, fed in portions of the given sizes."""
    outs, at = [], 0
    for n in cuts:
        ctx = harness.ctx([0] * n)
        x = h[at:at + n].to(harness.rt.dtype).cuda()
        out = torch.full((n, width), float("nan"), dtype=torch.float32, device="cuda")
        part.forward(ctx, CacheBinding(group=0, index=0, writes=True, state_index=0), x, out, accumulate=False)
        outs.append(out.cpu())
        at += n
    assert at == h.shape[0]
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layer", [("P", 1), ("Q", 0), ("Q", 2), ("R", 0)])
def test_the_recurrence_carries_its_state_across_portions(name, layer, dtype):
    cfg, W = weights_of_layer(name, layer)
    c = cfg["layers"][layer]["mixer"]
    prefix = f"l{layer}."
    part = build_part("mixer", PartSpec("gated_recurrence", {"hidden_size": cfg["width"], **c}), prefix)
    T = 150
    h = rows_in(T, cfg["width"], 11, dtype)
    Wd = {k: v.double() for k, v in W.items()}
    ref = P.gated_recurrence(Wd, prefix + "mix.", c, h.double()).float()
    for cuts in ([T], [1] * 12 + [2, 1, 3, 2, 64, 1, 1, 64], [2] * 75):
        hs = PartHarness(dtype, CacheSpec(entries=1, heads=1, head_dim=8), state_elems=[part.state_spec().elems])
        part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
        got = run_mixer(part, hs, h, cuts, cfg["width"])
        assert float((got - ref).abs().max()) <= part_tol(dtype, ref), cuts
    # what the test would catch: a state that is lost at a portion's start, inputs of the convolution forgotten
    lost = torch.cat([P.gated_recurrence(Wd, prefix + "mix.", c, h[:70].double()), P.gated_recurrence(Wd, prefix + "mix.", c, h[70:].double())]).float()
    assert float((lost - ref)[70:].abs().max()) > 20 * part_tol("float32", ref)
    # the memory is long: the first token still moves the last row
    other = h.clone()
    other[0] += 3.0
    moved = P.gated_recurrence(Wd, prefix + "mix.", c, other.double()).float()
    assert float((moved - ref)[-1].abs().max()) > part_tol("float32", ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layer,page", [("P", 0, 8), ("Q", 1, 64), ("Q", 3, 16), ("R", 1, 4), ("R", 2, 32)])
def test_latent_attention_at_every_edge_of_its_window(name, layer, page, dtype):
    cfg, W = weights_of_layer(name, layer)
    check_latent_attention(cfg, W, layer, page, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,rot,vdim,rank,window,page", [(16, 16, 32, 16, 32, 100, 64), (32, 8, 32, 24, 96, 70, 128),
                                                                 (16, 32, 64, 8, 256, 130, 64), (16, 16, 32, 16, 32, 0, 64)])
def test_latent_attention_with_heads_in_sixteens(heads, dim, rot, vdim, rank, window, page, dtype):
    """Sizes that the matrix-core form takes in 16 bits (heads in sixteens, latents in sixteens, key rows
    in chunks of 32, pages of 64 or 128): its three sizes of register tile."""
    from pikesun_models import att, config, draw_weights, layer
    cfg = config(64, 16, [layer(att(heads, dim, rot, vdim, rank, 24, window), None)])
    W = {k: v for k, v in draw_weights(cfg, 31).items() if k.startswith("l0.")}
    # few tokens over a window: a token's blocks of positions side by side and folded; many tokens: a wave walks them
    check_latent_attention(cfg, W, 0, page, dtype, T=600 if heads == 32 else 330)


def check_latent_attention(cfg, W, layer, page, dtype, T=None):
    c = dict(cfg["layers"][layer]["mixer"])
    prefix = f"l{layer}."
    window = c["mask"]["size"] if c.get("mask") else 0
    sharp = 3.0 if dtype == "float32" else 1.0        # 16 bits of cache cannot carry weights that sharp
    spec = PartSpec("latent_attention", {
        "hidden_size": cfg["width"], "heads": c["heads"], "dim": c["dim"], "rot_dim": c["rot_dim"], "vdim": c["vdim"],
        "kv_rank": c["kv_rank"], "q_rank": c["q_rank"], "scale": c["scale"] * sharp, "window": window, "eps": cfg["norm"]["eps"],
        "position": PartSpec("rope", {"head_dim": c["rot_dim"], "rotary_dim": c["rot"]["dims"], "theta": c["rot"]["base"]})})
    c["scale"] *= sharp               # sharp weights: the key that wins decides the row, wherever it lies
    part = build_part("mixer", spec, prefix)
    T = T or max(2 * window + 70, 200)
    h = rows_in(T, cfg["width"], 13, dtype)
    Wd = {k: v.double() for k, v in W.items()}
    ref = P.latent_attention(Wd, prefix + "mix.", c, h.double(), cfg["norm"]["eps"]).float()
    first = max(window - 3, 2)
    for cuts in ([T], [first] + [1] * 8 + [T - first - 8], [2, 1, 1, 3] + [1] * 30 + [64, 2, T - 103]):
        hs = PartHarness(dtype, part.cache_spec(), page_size=page, n_pages=-(-T // page) + 3, max_seq_len=1024)
        part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
        got = run_mixer(part, hs, h, cuts, cfg["width"])
        assert float((got - ref).abs().max()) <= part_tol(dtype, ref), cuts
    # what the test would catch: a window one position off, either way; a far key left out
    for wrong in ([window - 1, window + 1] if window else [T // 2]):
        off = P.latent_attention(Wd, prefix + "mix.", c, h.double(), cfg["norm"]["eps"], window_override=wrong).float()
        assert float((off - ref).abs().max()) > 20 * part_tol("float32", ref), wrong


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_key_hundreds_of_positions_back_decides_a_row(dtype):
    """A window of 700 over 900 positions in pages of 64, with weights set by hand: the latent's
    first half is what keys and queries compare, its second half what values carry.  Positions 150,
    200 and 880 share the first half (a loud match) and differ in the second; every other key is
    faint.  Row 880 is then the mean of the values at 200 and 880: 200 is just inside the window
    (680 back), 150 outside (730 back)."""
    width, H, half = 64, 2, 16
    eye = torch.eye(half)
    W = {"l0.mix.dkv": torch.eye(2 * half, width), "l0.mix.dkv.norm": torch.ones(2 * half),
         "l0.mix.dq": torch.eye(half, width), "l0.mix.dq.norm": torch.ones(half),
         "l0.mix.uq": torch.cat([eye] * H), "l0.mix.uk": torch.cat([torch.cat([eye, 0 * eye], 1)] * H),
         "l0.mix.uv": torch.cat([torch.cat([0 * eye, eye], 1)] * H), "l0.mix.g": torch.zeros(H * half, width),
         "l0.mix.o": torch.randn(width, H * half, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).float()}
    c = {"heads": H, "dim": half, "rot_dim": 0, "vdim": half, "kv_rank": 2 * half, "q_rank": half, "scale": 1.0, "mask": {"size": 700}}
    part = build_part("mixer", PartSpec("latent_attention", {
        "hidden_size": width, "heads": H, "dim": half, "rot_dim": 0, "vdim": half, "kv_rank": 2 * half, "q_rank": half,
        "scale": 1.0, "window": 700, "eps": 1e-6, "position": None}), "l0.")
    T = 900
    h = rows_in(T, width, 17, dtype)
    h[:, :half] *= 0.1                                   # faint keys
    h[150, :half] = h[200, :half] = h[880, :half] = rows_in(1, half, 18, dtype)[0]
    Wd = {k: v.double() for k, v in W.items()}
    ref = P.latent_attention(Wd, "l0.mix.", c, h.double(), 1e-6).float()
    outside_seen = P.latent_attention(Wd, "l0.mix.", c, h.double(), 1e-6, window_override=740).float()
    inside_lost = P.latent_attention(Wd, "l0.mix.", c, h.double(), 1e-6, window_override=600).float()
    assert float((outside_seen - ref)[880].abs().max()) > 0.05 * float(ref.abs().max())
    assert float((inside_lost - ref)[880].abs().max()) > 0.05 * float(ref.abs().max())
    for cuts in ([T], [870] + [1] * 30):
        hs = PartHarness(dtype, part.cache_spec(), page_size=64, n_pages=16, max_seq_len=1024)
        part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
        got = run_mixer(part, hs, h, cuts, width)
        assert float((got - ref).abs().max()) <= part_tol(dtype, ref), cuts


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layer", [("P", 0), ("Q", 1), ("Q", 2), ("R", 2), ("P", 1), ("Q", 3)])
def test_feed_forwards_alone(name, layer, dtype):
    from axon_amd.config import config_from_dict
    cfg, W = weights_of_layer(name, layer)
    mlp = cfg["layers"][layer]["mlp"]
    prefix = f"l{layer}."
    spec = config_from_dict(cfg).layers[layer]["mlp"]
    part = build_part("feed_forward", spec, prefix)
    hs = PartHarness(dtype, CacheSpec(entries=1, heads=1, head_dim=8), page_size=64, n_pages=16, max_seq_len=1024)
    part.load(WeightStore(DictSource(W), hs.rt.device, hs.rt.dtype), hs.rt)
    Wd = {k: v.double() for k, v in W.items()}
    for T in (1, 5, 70, 400):            # 400 rows: experts with many rows each run one by one through the large products
        h = rows_in(T, cfg["width"], 19 + T, dtype) * 1.5
        ref = P.feed_forward(Wd, prefix + "mlp.", mlp, h.double()).float()
        ctx = hs.ctx([0] * T)
        out = torch.full((T, cfg["width"]), float("nan"), dtype=torch.float32, device="cuda")
        part.forward(ctx, h.to(hs.rt.dtype).cuda(), out, accumulate=False)
        err = (out.cpu() - ref).abs().max(dim=-1).values
        if mlp["kind"] == "moe" and mlp["router"]["top"] < mlp["router"]["experts"]:
            # a row whose last chosen expert and first left out are a close call may go either way: not this test's matter
            z = (h.double() @ Wd[prefix + "mlp.router"].T).sort(dim=-1, descending=True).values
            top = mlp["router"]["top"]
            err = err[(z[:, top - 1] - z[:, top]) > 0.05]
        assert float(err.max()) <= part_tol(dtype, ref), (T, int(err.argmax()))
        again = torch.ones((T, cfg["width"]), dtype=torch.float32, device="cuda")
        part.forward(ctx, h.to(hs.rt.dtype).cuda(), again)               # added into rows that hold something
        assert float((again.cpu() - 1.0 - out.cpu()).abs().max()) <= 1e-5 * max(1.0, float(ref.abs().max()))
    if mlp["kind"] == "moe":
        # the clamps are met, and the ranking matters: the plain run with one expert fewer differs
        h = rows_in(70, cfg["width"], 89, dtype) * 1.5
        ref = P.feed_forward(Wd, prefix + "mlp.", mlp, h.double()).float()
        g = h.double() @ Wd[prefix + "mlp.e0.gate"].T
        assert float(g.max()) > mlp["expert"]["limit"] and float(g.min()) < -mlp["expert"]["limit"]
        if mlp["router"]["top"] > 1:
            fewer = dict(mlp, router=dict(mlp["router"], top=mlp["router"]["top"] - 1))
            assert float((P.feed_forward(Wd, prefix + "mlp.", fewer, h.double()).float() - ref).abs().max()) > 20 * part_tol("float32", ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_grouped_products_block_diagonal_and_routed(dtype):
    from axon_amd.kernels import kernels
    k = kernels(dtype)
    td = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    g = torch.Generator().manual_seed(1)
    for (M, G, N, K, x32) in [(37, 3, 20, 24, True), (70, 2, 64, 64, True), (5, 4, 48, 96, False), (33, 1, 130, 32, False)]:
        x = torch.randn(M, G * K + 8, generator=g)
        x = (x if x32 and dtype == "float32" else x.to(torch.bfloat16).float())
        w = (torch.randn(G, N, K, generator=g) * 0.3).to(torch.bfloat16).float()
        bias = torch.randn(G, N, generator=g)
        gate = torch.randn(M, G * N, generator=g)
        ref = torch.stack([x[:, i * K:(i + 1) * K].double() @ w[i].double().T + bias[i].double() for i in range(G)], 1).reshape(M, G * N)
        ref = (ref * torch.sigmoid(gate.double())).float()
        xd = x.cuda() if x32 else x.to(td).cuda()
        out = torch.zeros(M, G * N, dtype=torch.float32, device="cuda")
        k.grouped_gemm(xd, w.to(td).cuda(), out, x_group_stride=K, out_group_stride=N, bias=bias.cuda(), gate=gate.cuda())
        assert float((out.cpu() - ref).abs().max()) <= part_tol(dtype, ref), (M, G, N, K)
        # a row's bits do not depend on the rows beside it
        alone = torch.zeros(1, G * N, dtype=torch.float32, device="cuda")
        k.grouped_gemm(xd[M - 1:], w.to(td).cuda(), alone, x_group_stride=K, out_group_stride=N, bias=bias.cuda(), gate=gate[M - 1:].cuda())
        assert torch.equal(alone[0], out[M - 1])
    # routed, with the gated epilogue: rows meet the matrix their tile names
    T, E, top, F, K = 45, 5, 2, 24, 64
    h = torch.randn(T, K, generator=g).to(torch.bfloat16).float()
    w = (torch.randn(E, 2 * F, K, generator=g) * 0.4).to(torch.bfloat16).float()
    logits = torch.randn(T, E, generator=g)
    chosen = torch.zeros(T, top, dtype=torch.int32, device="cuda")
    weights = torch.zeros(T, top, dtype=torch.float32, device="cuda")
    k.route_topk(logits.cuda(), top, chosen, weights)
    val, idx = torch.topk(logits, top, dim=-1)
    assert torch.equal(chosen.cpu().long(), idx)
    assert float((weights.cpu() - torch.softmax(val, -1)).abs().max()) < 1e-6
    for n_e, n_top, rows_ in ((200, 7, 33), (64, 64, 3), (1100, 3, 9)):          # a wave a token; every expert; a thread a token
        z = torch.randn(rows_, n_e, generator=g)
        c2, w2 = torch.zeros(rows_, n_top, dtype=torch.int32, device="cuda"), torch.zeros(rows_, n_top, dtype=torch.float32, device="cuda")
        k.route_topk(z.cuda(), n_top, c2, w2)
        v2, i2 = torch.topk(z, n_top, dim=-1)
        assert torch.equal(c2.cpu().long(), i2) and float((w2.cpu() - torch.softmax(v2, -1)).abs().max()) < 1e-6
    tie = torch.zeros(2, 70)
    tie[:, [3, 9, 68]] = 1.0
    c2, w2 = torch.zeros(2, 2, dtype=torch.int32, device="cuda"), torch.zeros(2, 2, dtype=torch.float32, device="cuda")
    k.route_topk(tie.cuda(), 2, c2, w2)
    assert c2.tolist() == [[3, 9], [3, 9]] and w2.tolist() == [[0.5, 0.5], [0.5, 0.5]]      # of equal logits the lower expert
    P_ = T * top
    pairs, tokens = torch.zeros(P_, dtype=torch.int32, device="cuda"), torch.zeros(P_, dtype=torch.int32, device="cuda")
    max_tiles = k.route_max_tiles(P_, E)
    tiles, n_tiles = torch.zeros(3 * max_tiles, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    k.route_sort(chosen, E, pairs, tokens, tiles, n_tiles)
    assert sorted(pairs.tolist()) == list(range(P_)) and tokens.tolist() == [p // top for p in pairs.tolist()]
    listed = tiles.view(-1, 3)[:int(n_tiles)].tolist()
    assert sum(c for _, _, c in listed) == P_ and all(1 <= c <= 16 for _, _, c in listed)
    for e, first, count in listed:
        assert all(int(chosen.view(-1)[p]) == e for p in pairs[first:first + count].tolist())
    act = torch.zeros(P_, F, dtype=td, device="cuda")
    k.grouped_gemm(h.to(td).cuda(), w.to(td).cuda(), act, x_group_stride=0, out_group_stride=0, glu=(1.2, 1.702),
                   routed=(tiles, n_tiles, max_tiles, tokens, pairs), rows=P_)
    # the same rows listed in tiles of 64 (many rows a group): the same bits; and what else the listing offers
    wide_tiles, n_wide = torch.zeros(3 * k.route_max_tiles(P_, E, 64), dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
    pairs64, tokens64 = torch.zeros_like(pairs), torch.zeros_like(tokens)
    place_of, first_of = torch.zeros(P_, dtype=torch.int32, device="cuda"), torch.zeros(E + 1, dtype=torch.int32, device="cuda")
    k.route_sort(chosen, E, pairs64, tokens64, wide_tiles, n_wide, place_of, first_of, tile_rows=64)
    assert int(n_wide) <= E and pairs64[place_of.long()].tolist() == list(range(P_))
    assert first_of.tolist() == [0] + torch.bincount(idx.view(-1), minlength=E).cumsum(0).tolist()
    act64 = torch.zeros(P_, F, dtype=td, device="cuda")
    k.grouped_gemm(h.to(td).cuda(), w.to(td).cuda(), act64, x_group_stride=0, out_group_stride=0, glu=(1.2, 1.702),
                   routed=(wide_tiles, n_wide, k.route_max_tiles(P_, E, 64), tokens64, pairs64, 64), rows=P_)
    assert torch.equal(act64, act)
    gathered = k.gather_rows(h.to(td).cuda(), tokens64, torch.zeros(P_, K, dtype=td, device="cuda"))
    assert torch.equal(gathered.cpu(), h.to(td)[tokens64.cpu().long()])
    rows32 = torch.randn(P_, 8, generator=g).cuda()
    y_a, y_b = torch.zeros(T, 8, device="cuda"), torch.zeros(T, 8, device="cuda")
    k.route_combine(rows32, weights, y_a)
    k.route_combine(rows32[pairs64.long()].contiguous(), weights, y_b, place_of=place_of)
    assert torch.equal(y_a, y_b)
    assert float((y_a.cpu() - (rows32.cpu().view(T, top, 8) * weights.cpu()[:, :, None]).sum(1)).abs().max()) < 1e-5
    for p in range(P_):
        e = int(idx.view(-1)[p])
        z = h[p // top].double() @ w[e].double().T
        gt, up = torch.clamp(z[:F], max=1.2), torch.clamp(z[F:], -1.2, 1.2)
        want = (gt * torch.sigmoid(1.702 * gt) * (up + 1)).float()
        assert float((act[p].float().cpu() - want).abs().max()) <= part_tol(dtype, want), p


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_block_with_norms_on_the_sublayers_outputs(dtype):
    from axon_amd.kernels import kernels
    k = kernels(dtype)
    g = torch.Generator().manual_seed(2)
    for T, width in ((1, 48), (9, 250)):
        y, x, gain = torch.randn(T, width, generator=g) * 3, torch.randn(T, width, generator=g), 1 + 0.1 * torch.randn(width, generator=g)
        ref = x.double() + 0.7 * P.rms(y.double(), gain.double(), 1e-5)
        xd = x.clone().cuda()
        rounded = torch.zeros(T, width, dtype=k.dtype, device="cuda")
        k.norm_add(y.cuda(), gain.cuda(), 1e-5, 0.7, xd, rounded)
        assert float((xd.cpu() - ref.float()).abs().max()) <= 1e-5
        assert torch.equal(rounded.cpu(), xd.cpu().to(k.dtype))
