"""Topapel on the GPU against the plain implementation: each mechanism's kernel alone, then whole models under
every way of cutting the work, in float32 (tight) and bfloat16, and greedy generation through the engine."""

import math

import pytest
import torch

import plain_topapel as plain
import trace_helpers as th
from topapel_fixtures import BLOCK_SIZE, CONFIGS, load_plain, write_model

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
@pytest.mark.parametrize("n", [7, 40, 300, 2048, 2500, 9000])
def test_polynorm_kernel(n):
    from tie_amd import kernels

    z = rnd(5, n, seed=n, scale=1.7).cuda()
    coeff = torch.tensor([0.7, -0.4, 0.25, 0.1])
    want = plain.polynorm(z.cpu(), coeff, 1e-5)
    out = torch.empty_like(z)
    kernels.poly_norm(z, coeff.cuda(), 1e-5, out)
    close(out, want, 2e-6, "polynorm")
    half = torch.empty(z.shape, dtype=torch.bfloat16, device="cuda")
    kernels.poly_norm(z, coeff.cuda(), 1e-5, half)
    close(half, want, 5e-3, "polynorm to bfloat16")


def test_scaled_embedding_and_capped_logits():
    from tie_amd import kernels

    table = rnd(50, 24, seed=1).to(torch.bfloat16).cuda()
    ids = i32([3, 49, 0, 3])
    out = torch.empty(4, 24, device="cuda")
    kernels.embed(table, ids, out, 12.0)
    assert torch.equal(out.cpu(), table.float().cpu()[[3, 49, 0, 3]] * 12.0)
    x = rnd(3, 100, seed=2, scale=40.0).cuda()
    want = 20.0 * torch.tanh(x.cpu().to(F64) * 0.5 / 20.0)
    kernels.scale_softcap(x, 0.5, 20.0)
    close(x, want, 1e-6, "capped logits")
    y = rnd(2, 10, seed=3).cuda()
    want = y.cpu() * 3.0
    kernels.scale_softcap(y, 3.0, None)
    assert torch.equal(y.cpu(), want)


@pytest.mark.parametrize("H,d,e", [(2, 8, 24), (3, 20, 12), (1, 64, 32), (3, 64, 64), (5, 12, 40), (2, 128, 128), (1, 200, 16),
                                   (1, 300, 70), (1, 512, 8)])
def test_decayed_linear_attention_kernel_carries_its_state(H, d, e):
    """Three sequences in one step and then further portions, single tokens among them, in other slots' company:
    every output against the plain scan of the whole sequence; the state of a slot that sat a step out is untouched."""
    from tie_amd import kernels

    lengths = [37, 5, 64]
    decay = torch.tensor([0.999, 0.5, 1.0, 0.9, 0.2][:H])
    width = H * (2 * d + e) + H * e
    proj = {s: rnd(n, width, seed=10 * s + d) for s, n in enumerate(lengths)}
    want = {}
    for s, n in enumerate(lengths):
        p = proj[s].to(F64)
        q, k = plain.silu(p[:, :H * d]).view(n, H, d), plain.silu(p[:, H * d:2 * H * d]).view(n, H, d)
        v = plain.silu(p[:, 2 * H * d:2 * H * d + H * e]).view(n, H, e)
        want[s] = torch.cat([plain.decayed_linear_attention(q[:, h], k[:, h], v[:, h], float(decay[h]))
                             for h in range(H)], dim=1)
    state = torch.zeros(6, H, d, e, device="cuda")
    slots = {0: 4, 1: 1, 2: 2}
    state[3].fill_(7.0)                                      # a neighbour's state must stay what it is
    done = {s: 0 for s in slots}
    got = {s: [] for s in slots}
    plan = [{0: 20, 1: 5, 2: 1}, {2: 1, 0: 1}, {0: 16, 2: 62}]
    for step in plan:
        rows = torch.cat([proj[s][done[s]:done[s] + n] for s, n in step.items()]).cuda().contiguous()
        starts = [0]
        for n in step.values():
            starts.append(starts[-1] + n)
        out = torch.full((rows.shape[0], H * e), float("nan"), device="cuda")
        kernels.decay_attention_scan(rows, out, state, i32(starts), i32([slots[s] for s in step]), decay.cuda(),
                                     len(step), H, d, e)
        for j, (s, n) in enumerate(step.items()):
            got[s].append(out[starts[j]:starts[j + 1]].cpu())
            done[s] += n
    for s in slots:
        assert done[s] == lengths[s]
        close(torch.cat(got[s]), want[s], 2e-5, f"sequence {s}")
    assert bool((state[3] == 7.0).all()) and bool((state[0] == 0).all())


@pytest.mark.parametrize("H,d,e", [(2, 8, 24), (3, 64, 64), (1, 200, 16), (2, 128, 100), (1, 384, 40)])
def test_long_portions_run_the_linear_attention_chunk_beside_chunk(H, d, e):
    """A step of two long portions and a single token, after a step that left states behind: the three launches over
    chunks give what one token after the other gives, outputs and the states they leave."""
    from tie_amd import kernels

    decay = torch.tensor([0.999, 0.5, 1.0][:H]).cuda()
    first, second = [20, 3, 9], [300, 1, 131]
    width = H * (2 * d + e)
    results = []
    for chunked in (False, True):
        state = torch.zeros(5, H, d, e, device="cuda")
        slots = i32([2, 0, 4])
        outs = []
        for n, lengths in enumerate((first, second)):
            rows = rnd(sum(lengths), width, seed=50 + n).cuda()
            starts = [0]
            for c in lengths:
                starts.append(starts[-1] + c)

            class Batch:
                host_new_tokens, memo = lengths, {}

            chunks = kernels.scan_chunks(Batch, "cuda", rows=37) if chunked and n == 1 else None
            assert chunks is None or chunks.count == 9 + 1 + 4
            out = torch.full((rows.shape[0], H * e), float("nan"), device="cuda")
            kernels.decay_attention_scan(rows, out, state, i32(starts), slots, decay, 3, H, d, e, chunks=chunks,
                                         scratch=Scratch())
            outs.append(out)
        results.append((torch.cat(outs), state))
    close(results[1][0], results[0][0], 1e-5, "outputs")
    close(results[1][1], results[0][1], 1e-5, "states")


def test_long_portions_run_the_gated_recurrence_chunk_beside_chunk():
    from tie_amd import kernels

    n = 100
    results = []
    for chunked in (False, True):
        state = torch.zeros(5, n, device="cuda")
        outs = []
        for step, lengths in enumerate(([20, 3, 9], [300, 1, 131])):
            rows = rnd(sum(lengths), 3 * n, seed=60 + step, scale=2.0).cuda()
            starts = [0]
            for c in lengths:
                starts.append(starts[-1] + c)

            class Batch:
                host_new_tokens, memo = lengths, {}

            chunks = kernels.scan_chunks(Batch, "cuda", rows=37) if chunked and step == 1 else None
            out = torch.full((rows.shape[0], n), float("nan"), device="cuda")
            kernels.min_gru_scan(rows, out, state, i32(starts), i32([2, 0, 4]), 3, n, chunks=chunks, scratch=Scratch())
            outs.append(out)
        results.append((torch.cat(outs), state))
    close(results[1][0], results[0][0], 1e-5, "outputs")
    close(results[1][1], results[0][1], 1e-5, "states")


def test_gated_norm_of_the_heads():
    from tie_amd import kernels

    T, n = 6, 72
    o, w = rnd(T, n, seed=1, scale=3.0), 1 + 0.2 * rnd(n, seed=2)
    wide = rnd(T, 200, seed=3)                                # the gate is a view into wider rows
    want = plain.norm_plain(o, w, 1e-5) * plain.sigmoid(wide[:, 128:])
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 5e-3)):
        out = torch.empty(T, n, dtype=dtype, device="cuda")
        kernels.gated_rms_norm(o.cuda(), w.cuda(), 1e-5, wide.cuda()[:, 128:], out)
        close(out, want, tol, "gated norm")


@pytest.mark.parametrize("n", [7, 40, 200, 1000])
def test_minimal_gated_recurrence_kernel_carries_its_state(n):
    from tie_amd import kernels

    lengths = [45, 3]
    proj = {s: rnd(L, 3 * n, seed=s + n, scale=2.0) for s, L in enumerate(lengths)}
    bias = rnd(3 * n, seed=99)
    want = {}
    for s in proj:
        p = proj[s].to(F64) + bias.to(F64)
        S = plain.mingru_scan(plain.sigmoid(p[:, :n]), plain.mingru_candidate(p[:, n:2 * n]))
        want[s] = S * plain.silu(p[:, 2 * n:])
    state = torch.zeros(4, n, device="cuda")
    slots, done, got = {0: 3, 1: 0}, {0: 0, 1: 0}, {0: [], 1: []}
    for step in ({0: 30, 1: 2}, {0: 1}, {1: 1, 0: 14}):
        rows = torch.cat([proj[s][done[s]:done[s] + c] for s, c in step.items()]).cuda().contiguous()
        starts = [0]
        for c in step.values():
            starts.append(starts[-1] + c)
        out = torch.full((rows.shape[0], n), float("nan"), device="cuda")
        kernels.min_gru_scan(rows, out, state, i32(starts), i32([slots[s] for s in step]), len(step), n,
                             bias=bias.cuda())
        for j, (s, c) in enumerate(step.items()):
            got[s].append(out[starts[j]:starts[j + 1]].cpu())
            done[s] += c
    for s in slots:
        close(torch.cat(got[s]), want[s], 2e-6, f"sequence {s}")


def plain_attention(q, k, v, scale, chunk, sinks):
    """q ``[T, H, D]``, k and v ``[T, G, D]`` of one whole sequence; returns ``[T, H, D]``."""
    T, H, _ = q.shape
    G = k.shape[1]
    allowed = plain.chunk_mask(T, chunk)
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = scale * (q[:, h].to(F64) @ k[:, g].to(F64).T)
        out[:, h] = plain.softmax_with_sink(s, allowed, float(sinks[h]) if sinks is not None else -1e300) @ v[:, g].to(F64)
    return out


def attention_case(H, G, D, bs, lens_new, lens_ctx, seed, dtype, chunk, sinks, scale, spike=None):
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
        if spike is not None:                 # one key stands out for the last query; its value is unmistakable
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
        full = plain_attention(q, k, v, scale, chunk, sinks)
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
@pytest.mark.parametrize("H,G,D,bs", [(4, 2, 16, 4), (6, 1, 48, 16), (2, 2, 64, 16), (6, 2, 96, 16), (2, 2, 24, 8),
                                      (4, 1, 128, 32)])
@pytest.mark.parametrize("chunk", [None, 1, 7, 64, 100, 1000])
@pytest.mark.parametrize("kind", ["mixed", "decode"])
def test_chunks_and_sinks_in_every_attention_kernel(dtype, H, G, D, bs, chunk, kind):
    """Prompt portions and single rows over chunks that end anywhere: the float32 kernel, and in bfloat16 the
    matrix-core kernels for prompts and for decoded tokens (head sizes in steps of 16) or the generic one. Without
    sinks and chunks the same call is the attention the other designs use."""
    from tie_amd import kernels

    lens_ctx = [13, 150, 40, 300, 1, 101] if kind == "mixed" else [1, 40, 300, 77, 16, 100, 101, 201]
    lens_new = [13, 70, 1, 1, 1, 2] if kind == "mixed" else [1] * len(lens_ctx)
    scale = 0.5
    sinks = torch.tensor([0.5, -1.0, 3.0, 0.0, 6.0, -4.0, 1.0, 2.0][:H])
    case = attention_case(H, G, D, bs, lens_new, lens_ctx, 3, dtype, chunk, sinks, scale)
    out = torch.full_like(case["q"], float("nan"))
    kernels.paged_attention(case["q"], case["kc"], case["vc"], out, case["step"], case["batch"], H, scale, None,
                            Scratch(), chunk=chunk, sinks=sinks.cuda())
    close(out, case["want"], 1e-5 if dtype == torch.float32 else 1.5e-2, f"attention {kind}, chunk {chunk}")
    plain_case = attention_case(H, G, D, bs, lens_new, lens_ctx, 3, dtype, chunk, None, scale)
    assert float((plain_case["want"] - case["want"]).abs().max()) > 0.05         # the sinks matter in this case
    out = torch.full_like(case["q"], float("nan"))
    kernels.paged_attention(case["q"], case["kc"], case["vc"], out, case["step"], case["batch"], H, scale, None,
                            Scratch(), chunk=chunk)
    close(out, plain_case["want"], 1e-5 if dtype == torch.float32 else 1.5e-2, f"attention {kind} without sinks")


@pytest.mark.parametrize("nsplit", [1, 3, 8])
@pytest.mark.parametrize("H,G,D,bs", [(3, 3, 48, 16), (8, 2, 128, 16), (4, 4, 64, 4), (6, 2, 96, 16)])
def test_chunks_and_sinks_in_the_decode_kernel_at_every_depth(H, G, D, bs, nsplit):
    """The decode kernel's variants with the keys of a chunk cut into shares (the merge adds the sink): each against
    the plain formula, and all the same bits."""
    from tie_amd import kernels

    lens_ctx = [1, 40, 300, 777, 16, 129, 512, 513]
    scale, chunk = 0.4, 256
    sinks = torch.tensor([0.5, -1.0, 3.0, 0.0, 6.0, -4.0, 1.0, 2.0][:H])
    case = attention_case(H, G, D, bs, [1] * len(lens_ctx), lens_ctx, 13, torch.bfloat16, chunk, sinks, scale)
    S = len(lens_ctx)
    part_o = torch.empty(S * H * nsplit * D, device="cuda")
    part_ml = torch.empty(S * H * nsplit * 2, device="cuda")
    results = []
    for depth in (1, 2, 3, 4):
        if depth > 1 and bs < 16:
            continue
        out = torch.full_like(case["q"], float("nan"))
        kernels.attention_decode_bf16(case["q"], case["kc"], case["vc"], out, case["batch"].query_start,
                                      case["batch"].context_lens, case["step"].block_tables, S, H, scale, None, nsplit,
                                      part_o if nsplit > 1 else None, part_ml if nsplit > 1 else None, depth=depth,
                                      chunk=chunk, sinks=sinks.cuda())
        close(out, case["want"], 1.5e-2, f"decode, depth {depth}, {nsplit} shares")
        results.append(out)
    for other in results[1:]:
        assert torch.equal(results[0], other)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("where", ["first", "page_edge", "far", "chunk_first", "before_chunk", "own_chunk_only"])
def test_one_key_that_towers(dtype, where):
    """One key's score towers over the others: where the last query's chunk holds it, its value must come out; one
    position before the chunk's first it must not. Without chunks a key hundreds of positions back is found."""
    from tie_amd import kernels

    H, G, D, bs, scale = 4, 2, 32, 16, 0.5
    chunk = None if where in ("first", "page_edge", "far") else 300
    # the last query sits at c - 1, in the chunk that starts at (c - 1) - (c - 1) % 300
    first = lambda c: (c - 1) - (c - 1) % 300      # noqa: E731
    spike = {"first": lambda c: 0, "page_edge": lambda c: 16 * 3 - 1, "far": lambda c: c - 459,
             "chunk_first": first, "before_chunk": lambda c: first(c) - 1, "own_chunk_only": lambda c: 5}[where]
    sinks = torch.tensor([0.0, 1.0, -1.0, 2.0])
    for lens_new in ([1, 7], [1, 1], [64, 130]):
        case = attention_case(H, G, D, bs, lens_new, [700, 923], 5, dtype, chunk, sinks, scale, spike=spike)
        out = torch.full_like(case["q"], float("nan"))
        kernels.paged_attention(case["q"], case["kc"], case["vc"], out, case["step"], case["batch"], H, scale, None,
                                Scratch(), chunk=chunk, sinks=sinks.cuda())
        close(out, case["want"], 1e-5 if dtype == torch.float32 else 1.5e-2, f"towering key {where}")
        last = out[lens_new[0] - 1].float().cpu()         # the first sequence's last query
        if where in ("before_chunk", "own_chunk_only"):
            assert float(last.abs().max()) < 5.0
        else:
            assert float((last - 7.0).abs().max()) < 0.1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D,rot", [(16, 8), (32, 32), (96, 48), (40, 10), (64, 64), (128, 32)])
def test_keys_cached_as_values_before_norm_and_rotation(dtype, D, rot):
    """The cache-write kernel with rows ``[q | k]``: queries and keys normed and partly rotated, the keys as they
    were projected cached as values; one plane of sums and three."""
    from tie_amd import kernels

    T, H, G, bs, eps = 37, 4, 2, 16, 1e-5
    qk = rnd(T, (H + G) * D, seed=D)
    qw, kw = 1 + 0.2 * rnd(D, seed=1), 1 + 0.2 * rnd(D, seed=2)
    positions = torch.arange(100, 100 + T)
    inv_freq = (300.0 ** (-2.0 * torch.arange(rot // 2, dtype=F64) / rot) / 2.0).float()
    q = plain.norm_plain(qk[:, :H * D].view(T, H, D), qw, eps)
    k = plain.norm_plain(qk[:, H * D:].view(T, G, D), kw, eps)
    q_want = plain.rotate_partial(q, positions, rot, 300.0, 2.0)
    k_want = plain.rotate_partial(k, positions, rot, 300.0, 2.0)
    slots = torch.randperm(4 * bs)[:T].to(torch.int32)
    cache_dtype = dtype
    tol = 2e-5 if dtype == torch.float32 else 8e-3
    for planes in (1, 3):
        rows = (qk / planes).repeat(planes, 1, 1).cuda().contiguous() if planes > 1 else qk.cuda()
        kc = torch.zeros(4, G, bs, D, dtype=cache_dtype, device="cuda")
        vc = torch.zeros(4, G, D, bs, dtype=cache_dtype, device="cuda")
        q_out = torch.empty(T, H * D, dtype=dtype, device="cuda")
        kernels.qk_norm_rope_kv_write(rows[0] if planes > 1 else rows, q_out, qw.cuda(), kw.cuda(), eps, inv_freq.cuda(),
                                      positions.to(torch.int32).cuda(), slots.cuda(), kc, vc, H, G, D, bs,
                                      planes=planes, plane_stride=T * (H + G) * D, rotary_dim=rot,
                                      values_are_keys=True)
        close(q_out.view(T, H, D), q_want, tol, "queries")
        page, off = (slots // bs).long(), (slots % bs).long()
        close(kc.cpu()[page, :, off], k_want, tol, "cached keys")
        close(vc.cpu()[page, :, :, off], qk[:, H * D:].view(T, G, D), tol, "cached values are the projected keys")


# ------------------------------------------------------------------------------------------- whole models
LENGTHS = {"A": [1, 2, 9, 23, 40, 64, 90, 37], "B": [5, 17, 33, 70, 128], "C": [1, 3, 30, 77, 18, 300],
           "D": [4, 150, 31, 2, 66], "E": [3, 70, 25, 49]}
TOLERANCE = {"float32": 2e-5, "bfloat16": 3e-2}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            folder = tmp_path_factory.mktemp(f"topapel_{name}_{dtype}")
            out[name, dtype] = write_model(folder, config, seed=41 + len(out), dtype=dtype)
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
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_every_way_of_cutting_the_work(folders, name, dtype):
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders[name, dtype], CONFIGS[name]
    requests = th.make_requests(config["vocab"], LENGTHS[name], seed=5)
    want = reference(folder, config, requests)
    bs = BLOCK_SIZE[name]
    biggest = max(th.round64(len(t)) for t in requests.values())

    def replayer(max_tokens):
        return TraceReplayer.from_folder(folder, dtype, max_tokens, block_size=bs)

    results = {"whole": th.collect(replayer(biggest), th.whole(requests)),
               "prefill+decode": th.collect(replayer(biggest), th.prefill_then_decode(requests, tail=40)),
               "portions": th.collect(replayer(biggest), th.portions(requests)),
               "token by token": th.collect(replayer(biggest), th.portions(requests, sizes=(1,)))}
    steps, peak = th.mixed(requests, max_live=4, seed=3)
    assert max(len(s["entries"]) for s in steps) >= 3
    rep = replayer(peak)
    results["mixed"] = th.collect(rep, steps)
    assert rep.cache.all_free()                                   # every page and every state slot came back
    for label, got in results.items():
        check(got, want, TOLERANCE[dtype], f"{name}/{dtype}/{label}")
    if dtype == "float32":       # the ways of cutting agree with each other beyond what they owe the plain one
        for label in ("prefill+decode", "portions", "token by token", "mixed"):
            for rid in requests:
                a = torch.stack([results["whole"][rid][p] for p in range(len(requests[rid]))])
                b = torch.stack([results[label][rid][p] for p in range(len(requests[rid]))])
                assert float((a - b).abs().max() / a.abs().max()) < 1e-5, f"{name}: whole vs {label}, request {rid}"


def random_config(rng):
    """A Topapel of random layers and sizes: odd widths, head sizes in and out of the matrix kernels' steps, up to 40
    query heads on a key/value head, chunks from one position to longer than any request, decays of 0 and 1."""
    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["lightning", "attention", "mingru"])
        if kind == "lightning":
            H = rng.randint(1, 5)
            mixer = {"heads": H, "dim": rng.choice([4, 12, 16, 32, 64, 128, 200]), "vdim": rng.choice([4, 20, 32, 64, 100]),
                     "decay": [rng.choice([0.0, 0.3, 0.9, 0.999, 1.0, rng.random()]) for _ in range(H)]}
        elif kind == "attention":
            G = rng.choice([1, 2, 3])
            dim = rng.choice([8, 16, 24, 40, 48, 64, 80, 112, 128])
            mixer = {"heads": G * rng.choice([1, 2, 5, 20]), "kv_heads": G, "dim": dim, "vdim": dim,
                     "scale": rng.choice([dim ** -0.5, 0.05, 0.3])}
            if rng.random() < 0.8:
                mixer["mask"] = {"size": rng.choice([1, 2, 17, 32, 50, 64, 300])}
            if rng.random() < 0.85:
                mixer["rot"] = {"dims": rng.choice([d for d in (2, 8, dim // 4 * 2, dim) if 0 < d <= dim]),
                                "base": rng.choice([10.0, 1e4, 5e5])}
                if rng.random() < 0.7:
                    mixer["rot"]["scaling"] = {"factor": rng.choice([0.5, 1.0, 2.0, 8.0])}
        else:
            mixer = {"width": rng.choice([1, 5, 33, 64, 200])}
        mlp = {"kind": "dense", "ff": rng.choice([4, 9, 100, 256])} if rng.random() < 0.6 else None
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    config = {"architecture": "Topapel", "vocab": rng.choice([17, 100, 301]), "width": rng.choice([32, 72, 100, 128]),
              "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "layers": layers}
    if rng.random() < 0.7:
        config["embedding"] = {"scale": rng.choice([0.5, 8.0])}
    if rng.random() < 0.7:
        config["logit_scale"] = rng.choice([0.1, 3.0])
    if rng.random() < 0.7:
        config["logit_softcap"] = rng.choice([5.0, 40.0])
    return config


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations_under_every_way_of_cutting(tmp_path, seed):
    """Float32 at the tight bound; bfloat16 (recorded decode steps included) at a bound that only a wrong mechanism
    exceeds: random weights this wide make some of these models amplify rounding."""
    import random

    from tie_amd.engine.replay import TraceReplayer

    rng = random.Random(1000 + seed)
    config = random_config(rng)
    bs = rng.choice([4, 8, 16, 32])
    lengths = [rng.choice([1, 2, 7, 33, 64, 65, 150]) for _ in range(rng.randint(2, 5))]
    for dtype, tolerance in (("float32", 5e-5), ("bfloat16", 0.15)):
        folder = write_model(tmp_path / dtype, config, seed, dtype)
        requests = th.make_requests(config["vocab"], lengths, seed=seed)
        want = reference(folder, config, requests)
        biggest = max(th.round64(len(t)) for t in requests.values())
        steps, peak = th.mixed(requests, max_live=4, seed=seed)
        for label, trace, room in (("whole", th.whole(requests), biggest),
                                   ("prefill+decode", th.prefill_then_decode(requests, tail=20), biggest),
                                   ("portions", th.portions(requests), biggest), ("mixed", steps, peak)):
            rep = TraceReplayer.from_folder(folder, dtype, room, block_size=bs)
            check(th.collect(rep, trace), want, tolerance, f"seed {seed}/{dtype}/{label}")
            assert rep.cache.all_free()


@pytest.mark.parametrize("name", ["A", "B", "C"])
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


def test_a_state_slot_used_again_starts_from_zero(folders):
    """Six requests through four slots: a request that takes a slot another has left must not see what it left."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders["A", "float32"], CONFIGS["A"]
    requests = th.make_requests(config["vocab"], [30, 8, 21, 5, 17, 26], seed=21)
    want = reference(folder, config, requests)
    steps, peak = th.mixed(requests, max_live=4, seed=6, tail=4)
    rep = TraceReplayer.from_folder(folder, "float32", peak, block_size=4, state_slots=4)
    got = th.collect(rep, steps)
    assert rep.cache.all_free()
    check(got, want, TOLERANCE["float32"], "slots used again")
    from tie_amd.errors import CapacityError
    rep = TraceReplayer.from_folder(folder, "float32", 512, block_size=4, state_slots=2)
    with pytest.raises(CapacityError):
        th.collect(rep, [{"step": 0, "entries": [{"id": r, "tokens": requests[r], "want": []} for r in ("r0", "r1", "r2")],
                          "end": []}])


def test_long_decoding_through_chunks_with_pages_given_back_and_used_again(folders):
    """Two requests decode 150 tokens each in a pool that holds them only because the pages of chunks left behind go
    back; a third then runs in the pages they left. Every attention layer of B has chunks."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders["B", "float32"], CONFIGS["B"]
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
    rep = TraceReplayer.from_folder(folder, "float32", 192, block_size=16)       # 12 pages: far fewer than 335 tokens
    got = th.collect(rep, steps)
    assert rep.cache.all_free()
    check(got, want, TOLERANCE["float32"], "long decoding")


@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_decode_steps_replayed_from_recordings_give_the_eager_logits(folders, name):
    """bfloat16 decode-only steps are recorded into HIP graphs and replayed; every replay against the eager engine.
    (E: what a recording launches must not point into memory that lives only as long as the recorded step.)"""
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
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    """The engine's own entry point and scheduler: several requests at once, prompts in portions, a pool so small
    that requests are put back and computed again (their state slots cleared and taken anew)."""
    import tie_amd

    folder, config = folders[name, dtype], CONFIGS[name]
    weights = load_plain(folder)
    prompts = list(th.make_requests(config["vocab"], [7, 19, 3, 30], seed=12).values())
    new = 10
    pages = 64 if name == "A" else 6             # B: 96 positions for requests that need 40, 29, 17 and 13 together
    engine = tie_amd.create_engine(folder, dtype=dtype, kv_blocks=pages, block_size=BLOCK_SIZE[name], max_seqs=3,
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

    folder, config = folders["A", "float32"], CONFIGS["A"]
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
