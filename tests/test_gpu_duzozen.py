"""Duzozen on the GPU against the plain implementation: each mechanism's kernel alone, then whole models under
every way of cutting the work, in float32 (tight) and bfloat16, and greedy generation through the engine."""

import math

import pytest
import torch

import plain_duzozen as plain
import trace_helpers as th
from duzozen_fixtures import BLOCK_SIZE, CONFIGS, load_plain, write_model

pytestmark = pytest.mark.gpu
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32) * scale


def close(got, want, rel, what=""):
    got, want = got.detach().cpu().to(F64), want.detach().cpu().to(F64)
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= rel, f"{what}: relative error {err:.3e} > {rel:.0e}"


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


class Scratch:
    def __init__(self):
        self.memory = {}

    def __call__(self, name, shape, dtype):
        key = (name, tuple(shape), dtype)
        if key not in self.memory:
            self.memory[key] = torch.zeros(tuple(shape), dtype=dtype, device="cuda")
        return self.memory[key]


# ------------------------------------------------------------------------------------------- kernels alone
def test_gelu_kernel_is_the_exact_form():
    from tie_amd import kernels

    x = torch.cat([rnd(1000, seed=1, scale=3.0), torch.tensor([0.0, -0.0, 8.0, -8.0, 1e-4])]).cuda()
    out = torch.empty_like(x)
    kernels.gelu(x, out)
    close(out, plain.gelu_erf(x.cpu()), 1e-6, "gelu")
    half = torch.empty(x.shape, dtype=torch.bfloat16, device="cuda")
    kernels.gelu(x, half)
    close(half, plain.gelu_erf(x.cpu()), 5e-3, "gelu to bfloat16")


@pytest.mark.parametrize("planes", [0, 1, 3])
@pytest.mark.parametrize("n", [24, 96, 1024, 2500, 9000])
def test_a_result_is_normed_added_and_the_stream_normed_again(planes, n):
    from tie_amd import kernels

    T, eps_a, eps_b = 5, 1e-5, 1e-3
    y = rnd(max(planes, 1), T, n, seed=3, scale=2.0)
    x = rnd(T, n, seed=4)
    wa, wb = 1 + 0.3 * rnd(n, seed=5), 1 + 0.3 * rnd(n, seed=6)
    total = y.sum(0).to(F64) if planes else y[0].to(F64)
    x_want = x.to(F64) + plain.rms_norm(total, wa, eps_a)
    for with_next in (False, True):
        xg = x.clone().cuda()
        out = torch.empty(T, n, device="cuda") if with_next else None
        kernels.norm_add_norm((y if planes else y[0]).cuda().contiguous(), wa.cuda(), eps_a, xg,
                              wb.cuda() if with_next else None, eps_b, out)
        close(xg, x_want, 1e-6, f"stream, {planes} planes")
        if with_next:
            close(out, plain.rms_norm(x_want, wb, eps_b), 1e-6, "the next norm")


@pytest.mark.parametrize("E,groups,keep,top", [(8, 4, 2, 3), (16, 4, 3, 4), (5, 1, 1, 1), (6, 6, 2, 2), (64, 8, 3, 6),
                                               (1, 1, 1, 1), (12, 3, 3, 12)])
def test_the_routers_choice(E, groups, keep, top):
    from tie_amd import kernels

    T = 40
    logits = rnd(T, E, seed=E + top, scale=2.0)
    correction = rnd(E, seed=7, scale=0.3) - 0.5            # mostly negative choice scores
    router = {"experts": E, "identity": 0, "top": top, "groups": {"count": groups, "keep": keep}}
    # the plain router takes rows and a matrix: rows = the logits themselves, matrix = identity
    chosen, weights = plain.route(logits.to(F64), torch.eye(E, dtype=F64), correction, router)
    ids = torch.empty(T, top, dtype=torch.int32, device="cuda")
    w = torch.empty(T, top, device="cuda")
    kernels.moe_route(logits.cuda(), correction.cuda(), groups, keep, top, ids, w)
    assert ids.cpu().tolist() == chosen.tolist()
    close(w, weights, 1e-6, "routing weights")
    kernels.moe_route(logits.cuda(), None, groups, keep, top, ids, w)
    chosen, weights = plain.route(logits.to(F64), torch.eye(E, dtype=F64), torch.zeros(E, dtype=F64), router)
    assert ids.cpu().tolist() == chosen.tolist()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,real,identity,top,K,F_", [(1, 4, 0, 2, 32, 16), (7, 6, 2, 3, 64, 24), (150, 5, 3, 2, 96, 48),
                                                     (33, 3, 1, 4, 40, 20), (300, 12, 4, 4, 128, 64), (500, 3, 0, 2, 72, 136),
                                                     (40, 2, 2, 3, 200, 100), (260, 4, 0, 1, 64, 40)])
def test_experts_over_rows_sorted_on_the_device(dtype, T, real, identity, top, K, F_):
    from tie_amd import kernels

    E = real + identity
    h = rnd(T, K, seed=11).to(dtype)
    gate, up = rnd(real, F_, K, seed=12, scale=0.2).to(dtype), rnd(real, F_, K, seed=13, scale=0.2).to(dtype)
    down = rnd(real, K, F_, seed=14, scale=0.2).to(dtype)
    g = torch.Generator().manual_seed(15)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    weights = torch.rand(T, top, generator=g)
    want = torch.zeros(T, K, dtype=F64)
    names = {}
    for e in range(real):
        names.update({f"e{e}.gate": gate[e], f"e{e}.up": up[e], f"e{e}.down": down[e]})
    for t in range(T):
        for k in range(top):
            e = int(ids[t, k])
            row = h[t:t + 1].to(F64)
            want[t] += float(weights[t, k]) * (plain.expert(row, names, f"e{e}.")[0] if e < real else row[0])
    scratch = Scratch()
    tile_rows = kernels.moe_tile_rows(dtype, dtype, K, F_, T * top, real)
    if dtype == torch.bfloat16:          # the matrix-core kernels, in both tile sizes, unless a size is in no step of 8
        slots = T * top
        assert tile_rows == (32 if F_ % 8 else (128 if slots >= 96 * real else (64 if slots >= 48 * real else 16)))
    rows = kernels.moe_align(ids.cuda(), real, tile_rows, scratch)
    offsets = rows.offsets.cpu().tolist()
    counts = [int((ids == e).sum()) for e in range(real)]
    assert [b - a for a, b in zip(offsets, offsets[1:])] == counts
    where = rows.where.cpu()
    assert ((where < 0) == (ids >= real)).all()
    placed = sorted(where[where >= 0].tolist())
    assert placed == list(range(sum(counts)))                 # every real slot has a place of its own
    act = torch.zeros(T * top, F_, dtype=dtype, device="cuda")
    kernels.moe_gate_up(h.cuda(), gate.cuda(), up.cuda(), rows, act)
    parts = torch.zeros(T * top, K, device="cuda")
    kernels.moe_down(act, down.cuda(), rows, parts)
    routed = kernels.RoutedParts(parts, rows.where, weights.cuda(), h.cuda())
    out = torch.full((T, K), float("nan"), device="cuda")
    kernels.moe_combine(routed, out)
    tolerance = 1e-5 if dtype == torch.float32 else 2e-2
    close(out, want, tolerance, "experts, combined")
    # the same parts through the norm that places a result in the stream
    x = rnd(T, K, seed=16).cuda()
    w_post = (1 + 0.2 * rnd(K, seed=17))
    x_want = x.cpu().to(F64) + plain.rms_norm(want, w_post, 1e-5)
    kernels.norm_add_norm(routed, w_post.cuda(), 1e-5, x)
    close(x, x_want, tolerance, "experts, normed into the stream")


def attention_case(H, G, D, bs, lens_new, lens_ctx, seed, dtype, window, softcap, scale, spike=None):
    """Sequences in scattered pages; returns what the kernels take and the plain result for the new rows."""
    g = torch.Generator().manual_seed(seed)
    S = len(lens_ctx)
    MB = max(math.ceil(c / bs) for c in lens_ctx) + 1
    NB = sum(math.ceil(c / bs) for c in lens_ctx) + 3
    pages = torch.randperm(NB, generator=g).tolist()
    kc = torch.full((NB, G, bs, D), 1e30, dtype=dtype)
    vc = torch.full((NB, G, D, bs), 1e30, dtype=dtype)
    tables = torch.zeros(S, MB, dtype=torch.int32)
    q_rows, want_rows, seq_of_row, query_start = [], [], [], [0]
    for s in range(S):
        ctx, n_new = lens_ctx[s], lens_new[s]
        q, k, v = (torch.randn(ctx, heads, D, generator=g) for heads in (H, G, G))
        if spike is not None:                 # one key stands out for the last query, far beyond what the cap leaves
            j = spike(ctx)
            k[j] = 0
            k[j, :, 0] = 40.0
            q[ctx - 1] = 0
            q[ctx - 1, :, 0] = 4.0
            v[j] = 7.0
        q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
        table = [pages.pop() for _ in range(math.ceil(ctx / bs))]
        tables[s, :len(table)] = torch.tensor(table, dtype=torch.int32)
        for j in range(ctx):
            kc[table[j // bs], :, j % bs] = k[j]
            vc[table[j // bs], :, :, j % bs] = v[j]
        full = plain.attention(q, k, v, scale, softcap, window)
        q_rows.append(q[ctx - n_new:].reshape(n_new, H * D))
        want_rows.append(full[ctx - n_new:].reshape(n_new, H * D))
        seq_of_row += [s] * n_new
        query_start.append(query_start[-1] + n_new)

    class Batch:
        all_decode = all(n == 1 for n in lens_new)
        num_seqs, plan_context, memo = S, 1024, {}
        host_new_tokens, host_context_lens = list(lens_new), list(lens_ctx)

    Batch.query_start, Batch.context_lens, Batch.seq_of_row = i32(query_start), i32(lens_ctx), i32(seq_of_row)

    class Step:
        block_tables = tables.cuda()
        key_shares = None

    return dict(q=torch.cat(q_rows).cuda().contiguous(), kc=kc.cuda(), vc=vc.cuda(), want=torch.cat(want_rows),
                batch=Batch, step=Step)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,bs", [(4, 2, 16, 4), (3, 3, 48, 16), (6, 1, 32, 16), (2, 2, 24, 8)])
@pytest.mark.parametrize("kind", ["mixed", "decode"])
def test_capped_scores_in_every_attention_kernel(dtype, H, G, D, bs, kind):
    """A cap small enough to bend most scores, a window, prompt portions and single rows: the float32 kernel, and in
    bfloat16 the matrix-core kernels for prompts and for decoded tokens (head sizes in steps of 16) or the generic one."""
    from tie_amd import kernels

    lens_ctx = [13, 29, 40, 300, 1] if kind == "mixed" else [1, 40, 300, 77, 16]
    lens_new = [13, 5, 1, 1, 1] if kind == "mixed" else [1] * 5
    scale, softcap, window = 0.9, 1.5, 21
    case = attention_case(H, G, D, bs, lens_new, lens_ctx, 3, dtype, window, softcap, scale)
    out = torch.full_like(case["q"], float("nan"))
    kernels.paged_attention(case["q"], case["kc"], case["vc"], out, case["step"], case["batch"], H, scale, window,
                            Scratch(), softcap=softcap)
    close(out, case["want"], 1e-5 if dtype == torch.float32 else 1.5e-2, f"capped attention {kind}")
    uncapped = attention_case(H, G, D, bs, lens_new, lens_ctx, 3, dtype, window, None, scale)
    assert float((uncapped["want"] - case["want"]).abs().max()) > 0.05       # the cap matters in this case


@pytest.mark.parametrize("nsplit", [1, 3])
@pytest.mark.parametrize("H,G,D,bs", [(3, 3, 48, 16), (8, 2, 128, 16), (2, 1, 256, 32), (4, 4, 64, 4)])
def test_capped_scores_in_the_decode_kernel_at_every_depth(H, G, D, bs, nsplit):
    """The decode kernel's variants (page lookups per lane; two to four tiles of keys in registers) with a cap: each
    against the plain formula, and all the same bits."""
    from tie_amd import kernels

    lens_ctx = [1, 40, 300, 777, 16, 129]
    scale, softcap, window = 0.8, 2.5, 500
    case = attention_case(H, G, D, bs, [1] * len(lens_ctx), lens_ctx, 13, torch.bfloat16, window, softcap, scale)
    S = len(lens_ctx)
    part_o = torch.empty(S * H * nsplit * D, device="cuda")
    part_ml = torch.empty(S * H * nsplit * 2, device="cuda")
    results = []
    for depth in (1, 2, 3, 4):
        if depth > 1 and bs < 16:
            continue
        out = torch.full_like(case["q"], float("nan"))
        kernels.attention_decode_bf16(case["q"], case["kc"], case["vc"], out, case["batch"].query_start,
                                      case["batch"].context_lens, case["step"].block_tables, S, H, scale, window, nsplit,
                                      part_o if nsplit > 1 else None, part_ml if nsplit > 1 else None, depth=depth,
                                      softcap=softcap)
        close(out, case["want"], 1.5e-2, f"capped decode, depth {depth}")
        results.append(out)
    for other in results[1:]:
        assert torch.equal(results[0], other)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("where", ["first", "page_edge", "far", "window_first", "before_window"])
def test_one_key_far_away_under_a_cap(dtype, where):
    """One key's score towers over the others even after the cap; inside the window its value must come out, one
    position before the window it must not."""
    from tie_amd import kernels

    H, G, D, bs, scale, softcap = 4, 2, 32, 16, 0.5, 15.0
    window = None if where in ("first", "page_edge", "far") else 300
    spike = {"first": lambda c: 0, "page_edge": lambda c: 16 * 3 - 1, "far": lambda c: c - 259,
             "window_first": lambda c: c - 300, "before_window": lambda c: c - 301}[where]
    for lens_new in ([1, 7], [1, 1]):
        case = attention_case(H, G, D, bs, lens_new, [700, 523], 5, dtype, window, softcap, scale, spike=spike)
        out = torch.full_like(case["q"], float("nan"))
        kernels.paged_attention(case["q"], case["kc"], case["vc"], out, case["step"], case["batch"], H, scale, window,
                                Scratch(), softcap=softcap)
        close(out, case["want"], 1e-5 if dtype == torch.float32 else 1.5e-2, f"spike at {where}")
        last_of_first = lens_new[0] - 1
        if where == "before_window":
            assert float(out[last_of_first].float().abs().max()) < 3.0
        else:
            assert float(out[last_of_first].float().min()) > 6.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv,bs,T", [(4, 2, 32, 32, 16, 70), (2, 1, 48, 32, 8, 9), (3, 3, 64, 64, 16, 33)])
def test_values_are_kept_and_blended_on_their_way_into_the_cache(dtype, H, G, D, Dv, bs, T):
    from tie_amd import kernels

    width = (H + 2 * G) * D
    lam = 0.37
    for planes in (1, 2):
        qkv = rnd(planes, T, width, seed=21)
        on_gpu = qkv.cuda().contiguous()
        total = qkv.sum(0)
        v = total[:, (H + G) * D:].view(T, G, D)
        slots = torch.randperm(T + 5)[:T].to(torch.int32)
        NB = (T + 5 + bs - 1) // bs
        kept = torch.zeros(T, G * Dv, device="cuda")
        q = torch.empty(T, H * D, dtype=dtype, device="cuda")

        def run(mix):
            kc = torch.zeros(NB, G, bs, D, dtype=dtype, device="cuda")
            vc = torch.zeros(NB, G, D, bs, dtype=dtype, device="cuda")
            kernels.qk_norm_rope_kv_write(on_gpu[0], q, None, None, 0.0, None, i32(list(range(T))), slots.cuda(), kc, vc,
                                          H, G, D, bs, planes=planes, plane_stride=T * width, value_mix=mix)
            return torch.stack([vc[int(s) // bs, :, :, int(s) % bs] for s in slots]).float().cpu()

        tolerance = 1e-6 if dtype == torch.float32 else 8e-3
        first = run(("keep", kept))
        close(first, v, tolerance, "the keeper caches its own values")
        close(kept.view(T, G, Dv), v[:, :, :Dv], 1e-6, "and keeps them in float32")
        kept.copy_(rnd(T, G * Dv, seed=22).cuda())
        blended = run(("blend", kept, torch.tensor([lam], device="cuda")))
        want = v.clone().to(F64)
        want[:, :, :Dv] = plain.mix_values(v[:, :, :Dv], kept.view(T, G, Dv).cpu(), lam)
        close(blended, want, tolerance, "blended values")


# ------------------------------------------------------------------------------------------- whole models
LENGTHS = {"P": [1, 2, 9, 23, 40, 64, 90, 37], "Q": [5, 17, 33, 70, 128], "R": [1, 3, 30, 77, 18]}
TOLERANCE = {"float32": 2e-5, "bfloat16": 3e-2}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            folder = tmp_path_factory.mktemp(f"duzozen_{name}_{dtype}")
            out[name, dtype] = write_model(folder, config, seed=31 + len(out), dtype=dtype,
                                           decisive_router=dtype == "bfloat16")
    return out


def reference(folder, config, requests, streams=None):
    weights = load_plain(folder)
    out = {}
    for rid, toks in requests.items():
        after = [] if streams is not None else None
        out[rid] = plain.forward(config, weights, toks, after).float()
        if streams is not None:
            streams[rid] = after
    return out


def check(got, want, tolerance, label):
    worst = 0.0
    for rid, ref in want.items():
        rows = got[rid]
        assert sorted(rows) == list(range(ref.shape[0])), f"{label}: request {rid} misses positions"
        mine = torch.stack([rows[p] for p in range(ref.shape[0])])
        assert torch.isfinite(mine).all(), f"{label}: request {rid} has non-finite logits"
        err = (mine - ref).abs().amax(dim=1) / ref.abs().max()
        bad = int(torch.argmax((err > tolerance).float())) if bool((err > tolerance).any()) else -1
        assert bad < 0, (f"{label}: request {rid} first differs at position {bad} "
                         f"(relative error {float(err[bad]):.3e}, allowed {tolerance:.0e})")
        worst = max(worst, float(err.max()))
    print(f"[observed] {label}: {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_every_way_of_cutting_the_work(folders, name, dtype):
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders[name, dtype], CONFIGS[name]
    requests = th.make_requests(config["vocab"], LENGTHS[name], seed=5)
    want = reference(folder, config, requests)
    bs = BLOCK_SIZE[name]
    biggest = max(th.round64(len(t)) for t in requests.values())

    def replayer(max_tokens):
        return TraceReplayer.from_folder(folder, dtype, max_tokens, block_size=bs)

    first = replayer(biggest)
    results = {"whole": th.collect(first, th.whole(requests)),
               "prefill+decode": th.collect(replayer(biggest), th.prefill_then_decode(requests, tail=40)),
               "portions": th.collect(replayer(biggest), th.portions(requests)),
               "token by token": th.collect(replayer(biggest), th.portions(requests, sizes=(1,)))}
    if name == "Q":              # six routed layers alike: the later ones ran from an earlier one's launch list
        assert first.model.layers_replayed > 0
    steps, peak = th.mixed(requests, max_live=4, seed=3)
    assert max(len(s["entries"]) for s in steps) >= 3
    rep = replayer(peak)
    results["mixed"] = th.collect(rep, steps)
    assert rep.cache.all_free()                                   # every page came back
    for label, got in results.items():
        check(got, want, TOLERANCE[dtype], f"{name}/{dtype}/{label}")
    if dtype == "float32":       # the ways of cutting agree with each other beyond what they owe the plain one
        for label in ("prefill+decode", "portions", "token by token", "mixed"):
            for rid in requests:
                a = torch.stack([results["whole"][rid][p] for p in range(len(requests[rid]))])
                b = torch.stack([results[label][rid][p] for p in range(len(requests[rid]))])
                assert float((a - b).abs().max() / a.abs().max()) < 1e-5, f"{name}: whole vs {label}, request {rid}"


@pytest.mark.parametrize("name", ["P", "Q"])
def test_the_stream_after_every_layer(folders, name):
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders[name, "float32"], CONFIGS[name]
    requests = th.make_requests(config["vocab"], [29], seed=8)
    streams = {}
    reference(folder, config, requests, streams)
    rep = TraceReplayer.from_folder(folder, "float32", 64, block_size=BLOCK_SIZE[name])
    seen = []
    rep.model.layer_hook = lambda index, x: seen.append(x.detach().double().cpu().clone())
    th.collect(rep, th.whole(requests))
    assert len(seen) == len(config["layers"])
    for i, (mine, ref) in enumerate(zip(seen, streams["r0"])):
        close(mine, ref, 1e-5, f"{name}: stream after layer {i}")


def test_long_decoding_through_windows_with_pages_given_back_and_used_again(folders):
    """Two requests decode 150 tokens each in a pool that holds them only because the windows' pages go back;
    a third then runs in the pages they left."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders["Q", "float32"], CONFIGS["Q"]
    requests = th.make_requests(config["vocab"], [170, 165, 60], seed=9)
    want = reference(folder, config, requests)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": requests[r][:20 - i], "want": list(range(20 - i))}
                                    for i, r in enumerate(("r0", "r1"))], "end": []}]
    at = {"r0": 20, "r1": 19}
    while at:
        entries = [{"id": r, "tokens": [requests[r][p]], "want": [0]} for r, p in at.items()]
        at = {r: p + 1 for r, p in at.items()}
        ended = [r for r, p in at.items() if p == len(requests[r])]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        for r in ended:
            del at[r]
    steps.append({"step": len(steps), "entries": [{"id": "r2", "tokens": requests["r2"], "want": list(range(60))}],
                  "end": ["r2"]})
    rep = TraceReplayer.from_folder(folder, "float32", 128, block_size=16)       # 8 pages: far fewer than 335 tokens
    got = th.collect(rep, steps)
    assert rep.cache.all_free()
    check(got, want, TOLERANCE["float32"], "long decoding")


@pytest.mark.parametrize("name", ["P", "Q"])
def test_decode_steps_replayed_from_recordings_give_the_eager_logits(folders, name):
    """bfloat16 decode-only steps are recorded into HIP graphs and replayed; every replay against the eager engine."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders[name, "bfloat16"], CONFIGS[name]
    requests = th.make_requests(config["vocab"], [50, 41, 47], seed=10)
    steps, peak = th.mixed(requests, max_live=3, seed=4, tail=30)
    eager = TraceReplayer.from_folder(folder, "bfloat16", peak, block_size=BLOCK_SIZE[name], use_graphs=False)
    recorded = TraceReplayer.from_folder(folder, "bfloat16", peak, block_size=BLOCK_SIZE[name])
    assert recorded.runner.use_graphs
    a, b = th.collect(eager, steps), th.collect(recorded, steps)
    assert recorded.runner.graph_replays > 10
    for rid, toks in requests.items():
        for p in range(len(toks)):
            assert torch.equal(a[rid][p], b[rid][p]), f"request {rid}, position {p}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    """The engine's own entry point and scheduler: several requests at once, prompts in portions, a small pool."""
    import tie_amd

    folder, config = folders[name, dtype], CONFIGS[name]
    weights = load_plain(folder)
    prompts = list(th.make_requests(config["vocab"], [7, 19, 3, 30], seed=12).values())
    new = 10
    engine = tie_amd.create_engine(folder, dtype=dtype, kv_blocks=64, block_size=BLOCK_SIZE[name], max_seqs=3,
                                   max_tokens_per_step=16, prefill_chunk=8)
    ids = [engine.add_request(p, tie_amd.SamplingParams(max_tokens=new)) for p in prompts]
    while engine.has_work():
        engine.step()
    for sid, prompt in zip(ids, prompts):
        generated = list(engine.sequence(sid).generated)
        assert len(generated) == new
        tokens = list(prompt)
        for i, token in enumerate(generated):       # every generated token is the plain model's best, or ties it
            logits = plain.forward(config, weights, tokens)[-1]
            best = float(logits.max())
            margin = 1e-4 if dtype == "float32" else 0.05 * float(logits.abs().max())
            assert float(logits[token]) >= best - margin, f"request {sid}: token {i} is not the plain model's choice"
            tokens.append(token)


def test_the_command_line_generates_the_plain_models_tokens(folders):
    import subprocess
    import sys

    from conftest import ROOT

    folder, config = folders["P", "float32"], CONFIGS["P"]
    weights = load_plain(folder)
    prompt = list(th.make_requests(config["vocab"], [11], seed=14).values())[0]
    tokens = list(prompt)
    for _ in range(6):
        tokens.append(int(plain.forward(config, weights, tokens)[-1].argmax()))
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "tie"), "generate", "-m", folder, "-p",
                           ",".join(map(str, prompt)), "--temp", "0", "--max-tokens", "6", "--dtype", "float32",
                           "--kv-mem", "16M"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == tokens[len(prompt):]
