"""The Fekorax design in the engine against the plain implementation (`plain_fekorax.py`): each kernel alone, then whole models of
three small configurations under every way of cutting the work into steps, and generation through the entry point and the
scheduler.  In float32 the engine's logits must not depend on the cutting at all (equal bits); in bfloat16 they must lie as close
to the exact model as rounding alone explains."""
import math

import pytest
import torch

from fekorax_folders import CONFIGS, PAGE_SIZE, write_model
from model_folders import assert_within_bfloat16_noise, relative_error
from plain_fekorax import (PlainFekorax, gelu_tanh, matrix_memory, scaled_frequencies, sink_attention, to_bfloat16_and_back,
                           turn_first_channels, unit_rms, visible)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = torch.float64


def _prompt(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("fekorax")
    out = {}
    for name, cfg in CONFIGS.items():
        write_model(root / name, cfg, seed=11 + len(name) + ord(name))
        out[name] = root / name
    return out


_plain_cache = {}


def plain_logits(folders, name, tokens, rounded=False, dtype=torch.float64):
    key = (name, tuple(tokens), rounded, dtype)
    if key not in _plain_cache:
        model = PlainFekorax(folders[name], dtype=dtype, store=to_bfloat16_and_back if rounded else None)
        _plain_cache[key] = model.logits(tokens)
    return _plain_cache[key]


def make_runner(folders, name, dtype, **kw):
    from geneinfer_amd.engine import Runner, load_model
    model = load_model(folders[name], dtype, DEV)
    kw.setdefault("page_size", PAGE_SIZE[name])
    kw.setdefault("max_tokens", 1024)
    kw.setdefault("max_requests", 4)
    return Runner(model, **kw)


def feed(runner, request, tokens, cuts):
    """The request's tokens in portions of the sizes in `cuts` (the rest one by one); logits of every position, on the host."""
    from geneinfer_amd.engine import StepEntry
    rows, at = [], 0
    sizes = list(cuts) + [1] * (len(tokens) - sum(cuts))
    for n in sizes:
        rows.append(runner.step([StepEntry(request, tokens[at:at + n], tuple(range(n)))]).cpu())
        at += n
    return torch.cat(rows)


def check_against_plain(folders, name, dtype, tokens, got, what):
    exact = plain_logits(folders, name, tokens)
    if dtype == "float32":            # as close to the 64-bit model as 32-bit arithmetic explains: within 4 times what the plain model loses in 32-bit
        single = plain_logits(folders, name, tokens, dtype=torch.float32)
        noise = max(relative_error(single[p], exact[p]) for p in range(len(tokens)))
        err = max(relative_error(got[p], exact[p]) for p in range(len(tokens)))
        assert err < 4 * noise + 1e-5, f"{what}: float32 logits differ from the plain implementation by {err:.2e} (the plain model in 32-bit: {noise:.2e})"
    else:
        rounded = plain_logits(folders, name, tokens, rounded=True)
        assert_within_bfloat16_noise({p: got[p] for p in range(len(tokens))}, lambda p: exact[p], lambda p: rounded[p], what)


# =============================================================================================== kernels alone
def test_the_library_and_the_planner_agree_on_the_state_size():
    from geneinfer_amd.kernels import ops
    for h, dk, dv in ((1, 1, 1), (3, 20, 72), (6, 48, 64), (2, 255, 129)):
        assert ops.lib().gi_mlstm_state_floats(h, dk, dv) == ops.mlstm_state_floats(h, dk, dv)


def test_segments_are_found_on_the_device():
    from geneinfer_amd.kernels import ops
    from geneinfer_amd.parts import StepContext
    lens, slots, pos0 = [3, 1, 70, 1, 1, 130], [2, 0, 5, 9, 9, 1], [4, 0, 64, 0, 0, 7]       # (two rows of one slot at position 0: two runs)
    slot = torch.tensor([s for s, n in zip(slots, lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    pos = torch.tensor([p + i for p, n in zip(pos0, lens) for i in range(n)], dtype=torch.int32, device=DEV)
    ctx = StepContext(n_rows=sum(lens), dtype=torch.float32, device=torch.device(DEV), tokens=slot, row_pos=pos, row_slot=slot, seg_slot=slots,
                      seg_start=[], seg_len=lens, seg_pos0=pos0)
    start, length = ops.segments(ctx)
    assert length.tolist() == lens and start.tolist() == [0, 3, 4, 74, 75, 76]


@pytest.mark.parametrize("heads, dk, dv", [(2, 20, 72), (3, 64, 64), (1, 130, 40), (2, 7, 200), (1, 100, 50), (1, 300, 10)])
def test_matrix_memory_kernel(heads, dk, dv):
    """Two requests of unequal length in one step; then the longer one again in three steps from a fresh slot: the state carries."""
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(dk)
    lens, cols = [37, 150], 2 * heads * dk + heads * dv + 2 * heads
    T = sum(lens)
    proj = torch.randn(T, cols, generator=g)
    proj[:, -2 * heads:] *= 4.0                                         # gates that move
    i_b, f_b, cap = torch.randn(heads, generator=g), torch.randn(heads, generator=g) + 2.0, 5.0
    off = (0, heads * dk, 2 * heads * dk, 2 * heads * dk + heads * dv, 2 * heads * dk + heads * dv + heads)

    def plain(rows):
        x = rows.double()
        q = x[:, off[0]:off[1]].view(-1, heads, dk) * dk ** -0.5
        k, v = x[:, off[1]:off[2]].view(-1, heads, dk), x[:, off[2]:off[3]].view(-1, heads, dv)
        li = cap * torch.tanh((x[:, off[3]:off[4]] + i_b.double()) / cap)
        lf = torch.nn.functional.logsigmoid(cap * torch.tanh((x[:, off[4]:] + f_b.double()) / cap))
        return matrix_memory(q, k, v, li, lf).reshape(-1, heads * dv)

    want = torch.cat([plain(proj[:lens[0]]), plain(proj[lens[0]:])])
    state = torch.zeros(4, ops.mlstm_state_floats(heads, dk, dv), device=DEV)
    dev = lambda t, dt=None: t.to(DEV) if dt is None else t.to(DEV, dt)

    def run(rows, seg_lens, slots):
        starts = [sum(seg_lens[:i]) for i in range(len(seg_lens))]
        out, den = torch.empty(rows.shape[0], heads * dv, device=DEV), torch.empty(rows.shape[0], heads, device=DEV)
        row_slot = torch.tensor([s for s, n in zip(slots, seg_lens) for _ in range(n)], dtype=torch.int32, device=DEV)
        ops.mlstm_scan(dev(rows), off, dev(i_b), dev(f_b), cap, dk ** -0.5, torch.tensor(starts, dtype=torch.int32, device=DEV),
                       torch.tensor(seg_lens, dtype=torch.int32, device=DEV), row_slot, state, out, den, heads, dk, dv)
        return (out.view(-1, heads, dv) / den[:, :, None]).reshape(-1, heads * dv).cpu().double()       # (the kernel leaves the division to its reader)

    got = run(proj, lens, [2, 0])
    assert relative_error(got, want) < 2e-5
    pieces = [run(proj[lens[0] + a:lens[0] + b], [b - a], [3]) for a, b in ((0, 2), (2, 67), (67, 150))]
    assert torch.equal(torch.cat(pieces), got[lens[0]:])               # the same bits however the rows were cut


def _attend(T, heads, kv, dk, dv, rot, chunk, window, sinks, q_scale=None, k_scale=None, gate=True, page=4, dtype=torch.float32, seed=0):
    """One request of T tokens through norm_rope_store and the attention kernel, on shuffled pages; and the plain result."""
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(seed)
    q, k, v = torch.randn(T, heads * dk, generator=g), torch.randn(T, kv * dk, generator=g), torch.randn(T, kv * dv, generator=g)
    if q_scale is not None:
        q, k = q * q_scale[:, None], k * k_scale[:, None]
    qn, kn = 1 + 0.1 * torch.randn(dk, generator=g), 1 + 0.1 * torch.randn(dk, generator=g)
    gates = torch.randn(T, heads, generator=g) if gate else None
    n_pages = -(-T // page)
    order = torch.randperm(n_pages + 3, generator=g)[:n_pages].to(torch.int32)
    table = torch.full((2, n_pages + 2), -1, dtype=torch.int32)
    table[1, :n_pages] = order
    cache = torch.zeros(n_pages + 3, kv * page * (dk + dv), dtype=dtype, device=DEV)
    pos, slot = torch.arange(T, dtype=torch.int32, device=DEV), torch.ones(T, dtype=torch.int32, device=DEV)
    freqs = scaled_frequencies(rot, 40.0) if rot else None
    cos = sin = None
    if rot:
        cos, sin = torch.empty(T, rot // 2, device=DEV), torch.empty(T, rot // 2, device=DEV)
        ops.rope_cos_sin(pos, torch.tensor(freqs, dtype=torch.float64, device=DEV), cos, sin)
    q_ready = torch.empty(T, heads * dk, dtype=dtype, device=DEV)
    eps = 1e-5
    ops.norm_rope_store(q.to(DEV), k.to(DEV), v.to(DEV), qn.to(DEV), kn.to(DEV), eps, cos, sin, rot, pos, slot, table.to(DEV), q_ready, cache, page, heads, kv, dk, dv)
    out = torch.empty(T, heads * dv, dtype=dtype, device=DEV)
    ops.attention_exact(q_ready, cache, out, pos, slot, table.to(DEV), heads, kv, dk, window, 0.3, page_size=page, value_dim=dv, chunk=chunk,
                        sinks=None if sinks is None else sinks.to(DEV), gate=None if gates is None else gates.to(DEV))
    store = to_bfloat16_and_back if dtype == torch.bfloat16 else (lambda x: x)
    P = torch.arange(T)
    qq = unit_rms(q.double().view(T, heads, dk), eps) * qn.double()
    kk = unit_rms(k.double().view(T, kv, dk), eps) * kn.double()
    if rot:
        qq, kk = turn_first_channels(qq, P, rot, freqs), turn_first_channels(kk, P, rot, freqs)
    mask = visible(P, P, chunk)
    if window:
        mask = mask & (P[None, :] > P[:, None] - window)
    want = sink_attention(store(qq), store(kk), store(v.double().view(T, kv, dv)), mask, 0.3, sinks.double() if sinks is not None else torch.full((heads,), -1e30, dtype=D))
    if gates is not None:
        want = want * torch.sigmoid(gates.double())[:, :, None]
    return out.float().cpu().double().view(T, heads, dv), want, v.double().view(T, kv, dv)


@pytest.mark.parametrize("heads, kv, dk, dv, rot, chunk, window", [(4, 2, 32, 16, 8, 24, None), (3, 3, 16, 48, 16, 7, None), (2, 1, 24, 24, 0, None, None),
                                                                   (6, 2, 80, 130, 30, 50, 33), (1, 1, 2, 1, 2, 1, None)])
def test_head_norm_partial_rotation_store_and_attention(heads, kv, dk, dv, rot, chunk, window):
    sinks = torch.randn(heads, generator=torch.Generator().manual_seed(1))
    got, want, _ = _attend(103, heads, kv, dk, dv, rot, chunk, window, sinks)
    assert relative_error(got, want) < 2e-5
    got, want, _ = _attend(103, heads, kv, dk, dv, rot, chunk, window, None, gate=False)
    assert relative_error(got, want) < 2e-5
    got, want, _ = _attend(70, heads, kv, dk, dv, rot, chunk, window, sinks, dtype=torch.bfloat16)
    assert relative_error(got, want) < 2e-2


def test_keys_at_the_edges_of_chunks_and_pages_stand_out():
    """One key's score is made to tower over the others' (its norm weight is bypassed by scaling query and key alike: the norm
    divides the scale out, so the towering comes from equal directions).  The query at p then returns that key's value if and
    only if the key is visible: just inside the chunk, not just outside it, far back across many pages, at a page's first and
    last place; and with a sink that towers higher still, next to nothing."""
    from geneinfer_amd.kernels import ops
    T, heads, kv, dk, dv, chunk, page = 200, 2, 1, 16, 8, 48, 4
    g = torch.Generator().manual_seed(9)
    direction = torch.randn(dk, generator=g)

    def run(p, j, sink=-30.0):
        q, k = 0.01 * torch.randn(T, heads * dk, generator=g), 0.01 * torch.randn(T, kv * dk, generator=g)
        q[p] = direction.repeat(heads) * 5
        k[j] = direction * 5
        v = torch.randn(T, kv * dv, generator=g)
        table = torch.arange(T // page, dtype=torch.int32).flip(0).reshape(1, -1).contiguous().to(DEV)
        cache = torch.zeros(T // page, kv * page * (dk + dv), device=DEV)
        pos, slot = torch.arange(T, dtype=torch.int32, device=DEV), torch.zeros(T, dtype=torch.int32, device=DEV)
        q_ready, out = torch.empty(T, heads * dk, device=DEV), torch.empty(T, heads * dv, device=DEV)
        ones = torch.ones(dk, device=DEV)
        ops.norm_rope_store(q.to(DEV), k.to(DEV), v.to(DEV), ones, ones, 1e-6, None, None, 0, pos, slot, table, q_ready, cache, page, heads, kv, dk, dv)
        ops.attention_exact(q_ready, cache, out, pos, slot, table, heads, kv, dk, None, 8.0, page_size=page, value_dim=dv, chunk=chunk,
                            sinks=torch.full((heads,), sink, device=DEV))
        return out.cpu()[p].view(heads, dv), v[j]

    # after the head norm every row has unit root mean square: the towering score is 8 * dk = 128, the others' 128 * the cosine between
    # two random directions of 16 channels (seldom above 0.8)
    for p, j, seen in ((48, 48, True), (49, 48, True), (95, 48, True), (95, 47, False), (96, 95, False), (96, 96, True), (143, 96, True),
                       (191, 144, True), (191, 143, False), (47, 0, True), (51, 48, True), (52, 51, True), (3, 0, True)):
        out, value = run(p, j)
        close = bool((out - value).abs().max() < 1e-3)
        assert close == seen, f"query {p}, key {j}: {'not ' if seen else ''}seen"
    out, _ = run(95, 48, sink=300.0)
    assert out.abs().max() < 1e-30


def test_small_kernels():
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    x, y, w = torch.randn(5, 70, generator=g), torch.randn(5, 70, generator=g), 1 + 0.1 * torch.randn(70, generator=g)
    got = ops.rmsnorm_add(y.to(DEV), w.to(DEV), 1e-5, x.clone().to(DEV)).cpu()
    assert relative_error(got, x.double() + unit_rms(y.double(), 1e-5) * w.double()) < 1e-6
    w2 = 1 + 0.1 * torch.randn(70, generator=g)
    for out_dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 5e-3)):
        xs = x.clone().to(DEV)
        nxt = ops.rmsnorm_add_norm(y.to(DEV), w.to(DEV), 1e-5, xs, w2.to(DEV), 1e-4, torch.empty(5, 70, dtype=out_dtype, device=DEV)).float().cpu()
        summed = x.double() + unit_rms(y.double(), 1e-5) * w.double()
        assert relative_error(xs.cpu(), summed) < 1e-6 and relative_error(nxt, unit_rms(summed, 1e-4) * w2.double()) < tol
    gu = 3 * torch.randn(7, 2 * 33, generator=g)
    for name, act in (("gelu_tanh", gelu_tanh), ("silu", torch.nn.functional.silu)):
        out = ops.act_mul(gu.to(DEV), torch.empty(7, 33, device=DEV), name).cpu()
        assert relative_error(out, act(gu[:, :33].double()) * gu[:, 33:].double()) < 1e-6
    o, gate, nw = torch.randn(6, 3 * 40, generator=g), torch.randn(6, 3 * 40, generator=g), 1 + 0.1 * torch.randn(3 * 40, generator=g)
    out = ops.head_norm_gate(o.to(DEV), gate.to(DEV), nw.to(DEV), 1e-5, torch.empty(6, 120, device=DEV), 3, 40).cpu()
    want = unit_rms(o.double().view(6, 3, 40), 1e-5).reshape(6, 120) * nw.double() * torch.sigmoid(gate.double())
    assert relative_error(out, want) < 1e-6


# ================================================================================================= whole models
LENGTHS = {"A": 90, "B": 75, "C": 150, "D": 70}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_prompts_decoding_and_portions_agree_with_the_plain_model(folders, name, dtype):
    cfg = CONFIGS[name]
    tokens = _prompt(cfg, LENGTHS[name], 3)
    runner = make_runner(folders, name, dtype)
    n = len(tokens)
    cuttings = {"whole": [n], "token by token after a prompt": [n - 40], "portions": [2, 5, 2, 17, 1, 30, 3, 2], "single tokens from the first": []}
    results = {}
    for what, cuts in cuttings.items():
        runner.open(what)
        results[what] = feed(runner, what, tokens, cuts)
        runner.close(what)
        check_against_plain(folders, name, dtype, tokens, results[what], f"{name} {dtype} {what}")
    if dtype == "float32":                                    # nothing depends on the cutting: the same bits
        for what in cuttings:
            assert torch.equal(results[what], results["whole"]), f"{name}: '{what}' differs from the whole prompt in float32"
    runner.cache.check_consistency()
    assert all(free == g.pool.n_pages for free, g in zip(runner.cache.free_pages(), runner.cache.groups))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_unequal_requests_side_by_side_on_pages_and_slots_used_again(folders, name, dtype):
    """Four requests of unequal lengths in steps that mix portions with single tokens, in a pool that holds less than the sum of
    what they need in all: requests end, their pages and slots go to the next.  Every request's logits equal what it gets alone."""
    from geneinfer_amd.engine import StepEntry
    cfg = CONFIGS[name]
    lengths = [61, 9, 34, 50, 27, 1, 44]
    prompts = [_prompt(cfg, n, 20 + i) for i, n in enumerate(lengths)]
    page = PAGE_SIZE[name]
    runner = make_runner(folders, name, dtype, max_tokens=4 * (-(-61 // page) * page), max_requests=4)
    alone = []
    for i, p in enumerate(prompts):
        runner.open(("alone", i))
        alone.append(feed(runner, ("alone", i), p, [len(p)]))
        runner.close(("alone", i))
        check_against_plain(folders, name, dtype, p, alone[-1], f"{name} {dtype} request {i} alone")
    portion = [7, 2, 1, 5, 3, 1, 4]                           # request i advances by so many tokens a step
    fed, got, waiting, live = [0] * len(prompts), [[] for _ in prompts], list(range(len(prompts))), []
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
            runner.open(live[-1])
        entries = []
        for i in live:
            n = min(portion[i], len(prompts[i]) - fed[i])
            entries.append(StepEntry(i, prompts[i][fed[i]:fed[i] + n], tuple(range(n))))
        rows = runner.step(entries).cpu()
        at = 0
        for i, e in zip(list(live), entries):
            got[i].append(rows[at:at + len(e.tokens)])
            at += len(e.tokens)
            fed[i] += len(e.tokens)
            if fed[i] == len(prompts[i]):
                runner.close(i)
                live.remove(i)
        runner.cache.check_consistency()
    for i, p in enumerate(prompts):
        mixed = torch.cat(got[i])
        if dtype == "float32":
            assert torch.equal(mixed, alone[i]), f"{name}: request {i} in a batch differs from itself alone"
        else:
            check_against_plain(folders, name, dtype, p, mixed, f"{name} bfloat16 request {i} in mixed batches")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_across_chunks_through_captured_steps(folders, dtype):
    cfg = CONFIGS["A"]
    tokens = _prompt(cfg, 260, 8)
    runner = make_runner(folders, "A", dtype)
    runner.open("r")
    got = feed(runner, "r", tokens, [10])                     # 250 single tokens over ten chunks of 24
    assert runner.steps_replayed > 200
    check_against_plain(folders, "A", dtype, tokens, got, f"A {dtype} long decoding")
    slot = runner.cache.slot("r")
    held = runner.cache.groups[0].held_pages(slot)
    assert len(held) <= -(-24 // PAGE_SIZE["A"]) + 1          # the pages of chunks gone by went back to the pool
    runner.close("r")


def test_greedy_generation_through_the_entry_point_and_the_scheduler(folders):
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig
    cfg = CONFIGS["B"]
    plain = PlainFekorax(folders["B"])
    prompts = [_prompt(cfg, n, 40 + n) for n in (5, 23, 12)]
    want = [plain.greedy(p, 8) for p in prompts]
    llm = gi.LLM(str(folders["B"]), dtype="float32", page_size=8, max_tokens=256, max_running=2)
    assert type(llm.model.config).__name__ == "FekoraxConfig"
    for p, w in zip(prompts, want):
        out = llm.generate(p, steps=len(p) + 7, temperature=0.0)
        assert out.generated_tokens == w
    eng = llm.engine(EngineConfig(max_running=2, step_rows=16, prefill_chunk=6))
    from geneinfer_amd.engine import EngineRequest
    from geneinfer_amd.sampling import SamplerConfig
    ids = [eng.submit(EngineRequest(p, len(p) + 7, SamplerConfig(0.0))) for p in prompts]
    eng.run_until_idle()
    assert [eng.result(i).generated_tokens for i in ids] == want


@pytest.mark.parametrize("hd, heads, kv, chunk", [(64, 4, 2, 64), (64, 6, 1, 80), (128, 4, 4, 200), (32, 2, 1, 48), (64, 32, 8, 1000), (64, 2, 1, 2000)])
def test_matrix_core_attention_with_chunks_sinks_and_gates(hd, heads, kv, chunk):
    """The bfloat16 kernels on the matrix cores against the 32-bit-arithmetic kernel on the same pages and queries: a long
    portion on top of a past (tiles, pairs of tiles, keys shared out), short portions and single rows of other requests."""
    from geneinfer_amd.kernels import ops
    from geneinfer_amd.parts import StepContext
    g = torch.Generator().manual_seed(hd + chunk)
    page, scale = 16, 0.7 * hd ** -0.5
    lens, pos0 = [300, 1, 40, 1, 700], [150, 333, 90, 0, 0]
    n_slots, width = len(lens), -(-1100 // page)
    table = torch.randperm(n_slots * width, generator=g).to(torch.int32).view(n_slots, width)
    cache = (torch.randn(n_slots * width, 2, kv, page, hd, generator=g)).to(torch.bfloat16).to(DEV)
    T = sum(lens)
    starts = [sum(lens[:i]) for i in range(n_slots)]
    q = torch.randn(T, heads * hd, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.tensor([p + i for p, n in zip(pos0, lens) for i in range(n)], dtype=torch.int32, device=DEV)
    slot = torch.tensor([s for s, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    sinks = (2 * torch.randn(heads, generator=g)).to(DEV)
    gate = torch.randn(T, heads + 3, generator=g).to(DEV)[:, :heads]
    ctx = StepContext(n_rows=T, dtype=torch.bfloat16, device=torch.device(DEV), tokens=slot, row_pos=pos, row_slot=slot, seg_slot=list(range(n_slots)),
                      seg_start=starts, seg_len=lens, seg_pos0=pos0)
    for extras in (dict(chunk=chunk, sinks=sinks, gate=gate), dict(chunk=chunk), dict(sinks=sinks), dict(gate=gate)):
        fast = ops.attention_general(q, cache, torch.empty_like(q), ctx, table.to(DEV), heads, kv, hd, page_size=page, scale=scale, **extras)
        slow = ops.attention_exact(q, cache, torch.empty_like(q), pos, slot, table.to(DEV), heads, kv, hd, None, scale, **extras)
        assert relative_error(fast.float(), slow.float()) < 2e-2, sorted(extras)
        worst = (fast.float() - slow.float()).abs().view(T, heads, hd).amax(dim=(1, 2))
        assert float(worst.max()) < 0.06, (sorted(extras), int(worst.argmax()))


@pytest.mark.parametrize("dtype, mode", [("float32", "mixed"), ("bfloat16", "mixed"), ("float32", "portions")])
def test_replay_through_the_command_line(folders, tmp_path, dtype, mode):
    """bin/trace_run as a child process on a Fekorax folder: up to four live requests, portions beside single tokens, a pool that
    holds less than all requests together, so that pages and state slots are used again."""
    import json
    import random
    import subprocess
    from pathlib import Path
    import numpy as np
    import traces
    root = Path(__file__).resolve().parent.parent
    cfg = CONFIGS["A"]
    rng = random.Random(4)
    requests = {f"q{i}": [rng.randrange(cfg["vocab"]) for _ in range(n)] for i, n in enumerate([50, 1, 33, 77, 40, 9])}
    steps = traces.mixed(requests, seed=3) if mode == "mixed" else traces.portions(requests)
    out = tmp_path / "out"
    cmd = [str(root / "bin" / "trace_run"), "--model", str(folders["A"]), "--dtype", dtype, "--out", str(out), "--max-tokens", str(traces.peak_tokens(steps, 64)),
           "--page-size", "4"]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", (line, proc.stderr.read() if proc.poll() is not None else "")
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0, proc.stderr.read()
    finally:
        if proc.poll() is None:
            proc.kill()
    got = {}
    for step, rows in traces.wanted_positions(steps).items():
        data = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"])
        for key, row in zip(rows, data):
            got[key] = torch.from_numpy(row.copy())
    for rid, tokens in requests.items():
        mine = {p: row for (r, p), row in got.items() if r == rid}
        assert len(mine) > 0
        exact = plain_logits(folders, "A", tokens)
        if dtype == "float32":            # (the same bound as `check_against_plain`: four times what the plain model loses in 32-bit)
            single = plain_logits(folders, "A", tokens, dtype=torch.float32)
            noise = max(relative_error(single[p], exact[p]) for p in mine)
            assert max(relative_error(row, exact[p]) for p, row in mine.items()) < 4 * noise + 1e-5
        else:
            rounded = plain_logits(folders, "A", tokens, rounded=True)
            assert_within_bfloat16_noise(mine, lambda p: exact[p], lambda p: rounded[p], f"replay {mode} {rid}")


def test_generation_from_the_command_line_on_random_weights(tmp_path):
    """bin/gi_generate on the shipped example configuration, random weights, greedy: runs, and twice the same."""
    import subprocess
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    cmd = [str(root / "bin" / "gi_generate"), "--config", str(root / "configs" / "fekorax-small.json"), "--random-seed", "3", "--prompt-ids", "5 17 3 999 4",
           "--steps", "24", "--temperature", "0"]
    runs = [subprocess.run(cmd, capture_output=True, text=True, timeout=280) for _ in range(2)]
    assert all(r.returncode == 0 for r in runs), runs[0].stderr[-2000:]
    assert runs[0].stdout == runs[1].stdout and len(runs[0].stdout.split()) >= 20


def test_the_new_parts_serve_other_designs():
    """The parts are not Fekorax's own: a model put together by hand, one sandwich layer around the plain attention of a Llama layer
    and a SiLU-gated feed-forward, one pre-norm layer around a matrix memory and a GELU-gated feed-forward, through the same step
    function; against a plain computation from the two plain implementations' functions."""
    from geneinfer_amd.config import AttentionSpec, LayerSpec, MlstmSpec, ModelSpec, RmsNormSpec, RotarySpec, RunEntry, SwiGluSpec
    from geneinfer_amd.engine import Runner
    from geneinfer_amd.engine.model import DecoderModel
    from geneinfer_amd.parts import model_tensor_needs
    from geneinfer_amd.weights import random_tensors
    from plain_fekorax import capped
    from plain_llama import causal_attention, rms_norm, rope_inverse_frequencies, rope_rotate, swiglu
    d, vocab, eps = 64, 100, 1e-5
    norm = lambda name: RmsNormSpec(d, eps, name)
    spec = ModelSpec(architecture="by hand", vocab_size=vocab, hidden_size=d, max_positions=256, embedding="emb", final_norm=norm("fn"), lm_head="head", layers=(
        LayerSpec(mixer=AttentionSpec(d, 4, 2, 16, "a.q", "a.k", "a.v", "a.o", RotarySpec(16, 10000.0)), feed_forward=SwiGluSpec(d, 96, "f.g", "f.u", "f.d"),
                  mixer_norm=norm("n1"), feed_forward_norm=norm("n2"), block="sandwich", mixer_post_norm=norm("n1b"), feed_forward_post_norm=norm("n2b")),
        LayerSpec(mixer=MlstmSpec(d, 2, 8, 24, 7.0, eps, "m.q", "m.k", "m.v", "m.g", "m.o", "m.n", "m.i", "m.ib", "m.f", "m.fb"),
                  feed_forward=SwiGluSpec(d, 80, "g.g", "g.u", "g.d", activation="gelu_tanh"), mixer_norm=norm("p1"), feed_forward_norm=norm("p2"), block="prenorm")),
        run_order=(RunEntry(0), RunEntry(1)))
    host = random_tensors(model_tensor_needs(spec), seed=5, dtype="float32", std=0.2)
    model = DecoderModel(spec, {k: v.to(DEV) for k, v in host.items()}, torch.float32, DEV)
    runner = Runner(model, page_size=4, max_tokens=256, max_requests=2)
    tokens = _prompt(dict(vocab=vocab), 45, 2)
    got = {}
    for what, cuts in (("whole", [45]), ("cut", [3, 20, 2])):
        runner.open(what)
        got[what] = feed(runner, what, tokens, cuts)
        runner.close(what)
    assert torch.equal(got["whole"], got["cut"])

    w = {k: v.double() for k, v in host.items()}
    T, pos = len(tokens), torch.arange(len(tokens))
    x = w["emb"][torch.tensor(tokens)]
    h = rms_norm(x, w["n1"], eps)
    f = rope_inverse_frequencies(16, 10000.0)
    q, k = rope_rotate((h @ w["a.q"].T).view(T, 4, 16), pos, f), rope_rotate((h @ w["a.k"].T).view(T, 2, 16), pos, f)
    y = causal_attention(q, k, (h @ w["a.v"].T).view(T, 2, 16)).reshape(T, 64) @ w["a.o"].T
    x = x + rms_norm(y, w["n1b"], eps)
    x = x + rms_norm(swiglu(rms_norm(x, w["n2"], eps), w["f.g"], w["f.u"], w["f.d"]), w["n2b"], eps)
    h = rms_norm(x, w["p1"], eps)
    o = matrix_memory((h @ w["m.q"].T).view(T, 2, 8) * 8 ** -0.5, (h @ w["m.k"].T).view(T, 2, 8), (h @ w["m.v"].T).view(T, 2, 24),
                      capped(h @ w["m.i"].T + w["m.ib"], 7.0), torch.nn.functional.logsigmoid(capped(h @ w["m.f"].T + w["m.fb"], 7.0)))
    x = x + (unit_rms(o, eps).reshape(T, 48) * w["m.n"] * torch.sigmoid(h @ w["m.g"].T)) @ w["m.o"].T
    h = rms_norm(x, w["p2"], eps)
    x = x + (gelu_tanh(h @ w["g.g"].T) * (h @ w["g.u"].T)) @ w["g.d"].T
    want = rms_norm(x, w["fn"], eps) @ w["head"].T
    assert relative_error(got["whole"], want) < 5e-5
