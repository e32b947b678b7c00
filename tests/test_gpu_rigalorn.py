"""The Rigalorn design in the engine against the plain implementation (`plain_rigalorn.py`): each kernel alone, then whole models
of five small configurations under every way of cutting the work into steps, and generation through the entry point and the
scheduler.  In float32 the engine's logits must not depend on the cutting at all (equal bits); in bfloat16 they must lie as close
to the exact model as rounding alone explains."""
import math

import pytest
import torch

import plain_rigalorn as P
from model_folders import assert_within_bfloat16_noise, relative_error
from rigalorn_folders import CONFIGS, PAGE_SIZE, stored_weights, write_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _prompt(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("rigalorn")
    out = {}
    for name, cfg in CONFIGS.items():
        write_model(root / name, cfg, seed=17 + ord(name))
        out[name] = root / name
    return out


_plain_cache = {}


def plain_logits(folders, name, tokens, rounded=False, dtype=torch.float64):
    key = (name, tuple(tokens), rounded, dtype)
    if key not in _plain_cache:
        _plain_cache[key] = P.forward(CONFIGS[name], stored_weights(folders[name]), tokens, dtype, store=P.to_bfloat16_and_back if rounded else P.same)
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
    if dtype == "float32":            # within 4 times what the plain model itself loses in 32-bit
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
    for h, g, dk, dv, taps in ((1, 1, 1, 1, 1), (3, 1, 20, 72, 5), (6, 2, 48, 64, 4), (2, 2, 255, 129, 2)):
        assert ops.lib().gi_delta_state_floats(h, g, dk, dv, taps) == ops.delta_state_floats(h, g, dk, dv, taps)
        assert ops.lib().gi_delta_memory_floats(h, dk, dv) == ops.delta_memory_floats(h, dk, dv)
    assert ops.lib().gi_delta_max_key_dim() == ops.DELTA_MAX_KEY_DIM and ops.lib().gi_delta_max_taps() == ops.DELTA_MAX_TAPS


def test_activation_of_the_plain_feed_forward():
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    x = torch.cat([4 * torch.randn(7, 33, generator=g), torch.tensor([[0.0, -0.0, 1e-8, -1e-8, 30.0, -30.0, -90.0] + [0.5] * 26])])
    for p, q in ((0.3, -0.7), (-25.0, 24.0), (0.0, 0.0)):
        params = torch.tensor([p, q])
        want = P.xielu(x.double(), params[0].double(), params[1].double())
        out = torch.empty(8, 33, device=DEV)
        ops.xielu(x.to(DEV), out, params.to(DEV))
        assert relative_error(out, want) < 1e-6
        half = torch.empty(8, 33, device=DEV, dtype=torch.bfloat16)
        ops.xielu(x.to(DEV), half, params.to(DEV))
        assert torch.equal(half.cpu(), out.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("heads, kv, dk, dv, taps", [(4, 2, 16, 24, 4), (3, 3, 64, 64, 2), (2, 1, 130, 10, 5), (1, 1, 7, 201, 1), (5, 5, 3, 5, 3), (2, 2, 300, 6, 8), (1, 1, 20, 9, 13)])
def test_gated_delta_rule_kernels(heads, kv, dk, dv, taps):
    """Two requests of unequal length in one step; then the longer one again from a fresh slot in steps down to one and two rows:
    the memories and the convolutions' tails carry, and the bits do not change."""
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(dk + taps)
    n_conv = 2 * kv * dk + heads * dv
    lens, cols = [29, 90], n_conv + 2 * heads + 3
    conv_off, a_off, b_off = 3, 3 + n_conv, 3 + n_conv + heads
    proj = torch.randn(sum(lens), cols, generator=g)
    w_taps = 0.6 * torch.randn(n_conv, taps, generator=g)
    a_log, dt_bias = -1.0 + 0.8 * torch.randn(heads, generator=g), 0.5 * torch.randn(heads, generator=g)

    def plain(rows):
        x = rows.double()
        y = P.short_conv_silu(x[:, conv_off:conv_off + n_conv], w_taps.double())
        unit = lambda z: z / torch.sqrt((z * z).sum(-1, keepdim=True) + 1e-6)
        q, k = unit(y[:, :kv * dk].view(-1, kv, dk)) * dk ** -0.5, unit(y[:, kv * dk:2 * kv * dk].view(-1, kv, dk))
        v = y[:, 2 * kv * dk:].view(-1, heads, dv)
        decay = torch.exp(-torch.exp(a_log.double()) * P.softplus(x[:, a_off:a_off + heads] + dt_bias.double()))
        beta = torch.sigmoid(x[:, b_off:b_off + heads])
        return torch.cat([P.delta_rule(q[:, h // (heads // kv)], k[:, h // (heads // kv)], v[:, h], beta[:, h], decay[:, h]) for h in range(heads)], dim=-1)

    want = torch.cat([plain(proj[:lens[0]]), plain(proj[lens[0]:])])
    state = torch.zeros(5, ops.delta_state_floats(heads, kv, dk, dv, taps) + 3, device=DEV)
    dev = lambda t: t.to(DEV)

    def run(rows, seg_lens, slots, pos0):
        n = rows.shape[0]
        starts = [sum(seg_lens[:i]) for i in range(len(seg_lens))]
        row_slot = torch.tensor([s for s, m in zip(slots, seg_lens) for _ in range(m)], dtype=torch.int32, device=DEV)
        row_pos = torch.tensor([p + i for p, m in zip(pos0, seg_lens) for i in range(m)], dtype=torch.int32, device=DEV)
        seg_start, seg_len = torch.tensor(starts, dtype=torch.int32, device=DEV), torch.tensor(seg_lens, dtype=torch.int32, device=DEV)
        qkv, gates, out = torch.empty(n, n_conv, device=DEV), torch.empty(n, 2 * heads, device=DEV), torch.empty(n, heads * dv, device=DEV)
        rows = dev(rows)
        ops.delta_prepare(rows, conv_off, a_off, b_off, dev(w_taps), dev(a_log), dev(dt_bias), row_slot, row_pos, state, qkv, gates, heads, kv, dk, dv, dk ** -0.5)
        ops.delta_tail(rows, conv_off, taps, seg_start, seg_len, row_slot, state, heads, kv, dk, dv)
        ops.delta_scan(qkv, gates, seg_start, seg_len, row_slot, state, out, heads, kv, dk, dv)
        return out.cpu().double()

    got = run(proj, lens, [2, 0], [0, 0])
    assert relative_error(got, want) < 3e-5
    second = proj[lens[0]:]
    cuts, pieces, at = [2, 1, 1, 40, 1, 2, 3, 38, 2], [], 0
    for c in cuts:
        pieces.append(run(second[at:at + c], [c], [4], [at]))
        at += c
    assert at == lens[1] and torch.equal(torch.cat(pieces), got[lens[0]:])
    # two requests that both go on, side by side in one step, each from its own slot
    state[1], state[3] = state[2], state[4]
    more = torch.randn(11, cols, generator=g)
    both = run(torch.cat([more[:4], more[4:]]), [4, 7], [1, 3], [lens[0], lens[1]])
    alone = torch.cat([run(more[:4], [4], [2], [lens[0]]), run(more[4:], [7], [4], [lens[1]])])
    assert torch.equal(both, alone)


def test_head_norm_with_shared_weights_and_a_silu_gate():
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    n, heads, dv, eps = 9, 3, 37, 1e-3
    o, gate, w = torch.randn(n, heads * dv, generator=g), 2 * torch.randn(n, heads * dv, generator=g), 1 + 0.1 * torch.randn(dv, generator=g)
    od = o.double().view(n, heads, dv)
    want = (od / torch.sqrt((od * od).mean(-1, keepdim=True) + eps) * w.double()).reshape(n, -1) * (gate.double() * torch.sigmoid(gate.double()))
    out = torch.empty(n, heads * dv, device=DEV)
    ops.head_norm_gate(o.to(DEV), gate.to(DEV), w.to(DEV), eps, out, heads, dv, gate_activation="silu")
    assert relative_error(out, want) < 1e-6


def _paged(T, page, n_numbers, dtype, seed):
    """Pages for one request of T positions in slot 1, in a shuffled order, and its table."""
    n_pages = -(-T // page)
    order = torch.randperm(n_pages + 3, generator=torch.Generator().manual_seed(seed))[:n_pages]
    table = torch.full((3, n_pages + 2), -1, dtype=torch.int32)
    table[1, :n_pages] = order.to(torch.int32)
    cache = torch.zeros(n_pages + 3, page * n_numbers, dtype=dtype, device=DEV)
    return cache, table.to(DEV)


def _ctx(T, pos0=0, slot=1):
    from geneinfer_amd.parts import StepContext
    pos = torch.arange(pos0, pos0 + T, dtype=torch.int32, device=DEV)
    slots = torch.full((T,), slot, dtype=torch.int32, device=DEV)
    return StepContext(n_rows=T, dtype=torch.float32, device=torch.device(DEV), tokens=slots, row_pos=pos, row_slot=slots, seg_slot=[slot], seg_start=[0],
                       seg_len=[T], seg_pos0=[pos0])


@pytest.mark.parametrize("T, window, far", [(300, None, 3), (300, 36, 264), (300, 36, 263), (131, 17, 114), (131, 17, 113), (70, 1, 69), (70, 64, 6), (70, 64, 5)])
def test_attention_with_biases_blended_values_and_one_key_that_stands_out(T, window, far):
    """The last row's query points at the key of position `far`, which is scaled up so that, if seen, it takes nearly all the
    weight: just inside the window, just outside it, or hundreds of positions back.  Biases, a rotation of a part of the head with
    lengthened cosines, and values blended with another layer's are all on."""
    from geneinfer_amd.kernels import ops
    heads, kv, dk, dv, rot, page, scale = 4, 2, 24, 10, 8, 4, 0.3
    g = torch.Generator().manual_seed(T + far)
    q, k, v = torch.randn(T, heads * dk, generator=g), torch.randn(T, kv * dk, generator=g), torch.randn(T, kv * dv, generator=g)
    qb, kb, vb = torch.randn(heads * dk, generator=g), torch.randn(kv * dk, generator=g), torch.randn(kv * dv, generator=g)
    other, blend = torch.randn(T, kv * dv, generator=g), torch.tensor([0.35])
    freqs, mag = P.rotary_frequencies(rot, 30.0, dict(factor=4.0, original=16, fast=2.0, slow=0.5))
    # the unrotated channels of key `far` and of the last query line up, large
    k.view(T, kv, dk)[far, :, rot:] = 3.0
    q.view(T, heads, dk)[T - 1, :, rot:] = 3.0
    qd, kd = (q + qb).double().view(T, heads, dk), (k + kb).double().view(T, kv, dk)
    vd = (1 - 0.35) * (v + vb).double() + 0.35 * other.double()
    want = P.softmax_attention(P.rotate_half_split(qd, freqs, mag), P.rotate_half_split(kd, freqs, mag), vd.view(T, kv, dv), scale, window)
    seen = window is None or T - 1 - far < window
    weight = torch.softmax((torch.einsum("hd,shd->hs", P.rotate_half_split(qd, freqs, mag)[T - 1], P.rotate_half_split(kd, freqs, mag).repeat_interleave(2, 1)) * scale)
                           .masked_fill(~P.window_mask(T, window)[T - 1][None], float("-inf")), -1)[:, far]
    assert (weight > 0.9).all() if seen else (weight == 0).all()          # (the test's premise: the key matters exactly when it is seen)

    cache, table = _paged(T, page, kv * (dk + dv), torch.float32, seed=far)
    ctx = _ctx(T)
    cos, sin = torch.empty(T, rot // 2, device=DEV), torch.empty(T, rot // 2, device=DEV)
    ops.rope_cos_sin(ctx.row_pos, torch.tensor(freqs, dtype=torch.float64, device=DEV), cos, sin, mag)
    q_ready, keep = torch.empty(T, heads * dk, device=DEV), torch.empty(T, kv * dv, device=DEV)
    dev = lambda t: t.to(DEV)
    ops.norm_rope_store(dev(q), dev(k), dev(v), None, None, 1e-6, cos, sin, rot, ctx.row_pos, ctx.row_slot, table, q_ready, cache, page, heads, kv, dk, dv,
                        biases=(dev(qb), dev(kb), dev(vb)), blend=(dev(other), dev(blend)), keep=keep)
    assert relative_error(keep, (v + vb).double()) < 1e-6
    out = torch.empty(T, heads * dv, device=DEV)
    ops.attention_general(q_ready, cache, out, ctx, table, heads, kv, dk, page_size=page, value_dim=dv, window=window, scale=scale)
    assert relative_error(out.view(T, heads, dv), want) < 2e-5
    assert relative_error(out.view(T, heads, dv)[T - 1], want[T - 1]) < 2e-5


@pytest.mark.parametrize("T, window, far", [(200, None, 2), (200, 50, 150), (200, 50, 149), (45, 16, 29), (45, 16, 30)])
def test_attention_through_latents_against_keys_and_values_made_in_full(T, window, far):
    """The kernels around the latent cache and the attention over it, with the up projections folded into query and output by hand
    here, against the plain layer that makes every head's keys and values of every position."""
    from geneinfer_amd.kernels import ops
    H, d, r, dv, q_rank, rank, page, scale, eps = 3, 12, 6, 7, 20, 18, 4, 0.3, 1e-5
    g = torch.Generator().manual_seed(T + far)
    m = dict(heads=H, dim=d, rot_dim=r, vdim=dv, kv_rank=rank, q_rank=q_rank, scale=scale, rot=dict(dims=r, base=40.0), mask=None if window is None else dict(size=window))
    hidden = 16
    w = {"dq": torch.randn(q_rank, hidden, generator=g) * 0.3, "dq.norm": 1 + 0.1 * torch.randn(q_rank, generator=g), "uq": torch.randn(H * (d + r), q_rank, generator=g) * 0.3,
         "dkv": torch.randn(rank + r, hidden, generator=g) * 0.3, "dkv.norm": 1 + 0.1 * torch.randn(rank, generator=g), "uk": torch.randn(H * d, rank, generator=g) * 0.3,
         "uv": torch.randn(H * dv, rank, generator=g) * 0.3, "o": torch.eye(H * dv)}
    h = torch.randn(T, hidden, generator=g)
    h[far] *= 6.0                                                        # a position whose latent is long: its scores are large either way
    want = P.latent_attention(h.double(), {k: v.double() for k, v in w.items()}, m, eps)

    dev = lambda t: t.to(DEV)
    cache, table = _paged(T, page, 2 * rank + r, torch.float32, seed=far)
    ctx = _ctx(T)
    f, _ = P.rotary_frequencies(r, 40.0)
    cos, sin = torch.empty(T, r // 2, device=DEV), torch.empty(T, r // 2, device=DEV)
    ops.rope_cos_sin(ctx.row_pos, torch.tensor(f, dtype=torch.float64, device=DEV), cos, sin)
    down = dev(torch.cat([h @ w["dq"].T, h @ w["dkv"].T], dim=1).contiguous())
    cq = torch.empty(T, q_rank, device=DEV)
    ops.latent_prepare(down, q_rank, rank, r, dev(w["dq.norm"]), dev(w["dkv.norm"]), eps, cos, sin, ctx.row_pos, ctx.row_slot, table, cq, cache, page)
    q = (cq @ dev(w["uq"]).T).contiguous()
    plain_part, folded = torch.empty(T, H * d, device=DEV), torch.empty(T, H * (rank + r), device=DEV)
    ops.latent_queries(q, cos, sin, plain_part, folded, H, d, r, rank)
    uk = dev(w["uk"]).view(H, d, rank)
    folded.view(T, H, rank + r)[:, :, :rank] = torch.einsum("thd,hdr->thr", plain_part.view(T, H, d), uk)
    att = torch.empty(T, H * rank, device=DEV)
    ops.attention_general(folded, cache, att, ctx, table, H, 1, rank + r, page_size=page, value_dim=rank, window=window, scale=scale)
    got = torch.einsum("thr,hvr->thv", att.view(T, H, rank), dev(w["uv"]).view(H, dv, rank)).reshape(T, H * dv)
    assert relative_error(got, want) < 3e-5


@pytest.mark.parametrize("H, kd, vd, window, lens, pos0", [(20, 152, 136, 44, [1, 1, 1], [700, 43, 0]), (8, 80, 64, None, [130, 1], [0, 300]), (32, 288, 256, 100, [70], [50]),
                                                          (3, 24, 16, 17, [33, 2, 1], [15, 16, 17]), (16, 96, 64, 1, [20], [0]), (16, 576, 512, 48, [40, 1], [30, 200]),
                                                          (5, 296, 264, None, [3], [60]), (16, 576, 512, 48, [100, 1], [30, 200]), (20, 152, 136, 44, [130, 70, 1], [700, 0, 5]),
                                                          (40, 80, 64, None, [90], [10]), (8, 288, 256, 300, [129, 200], [77, 0]), (130, 32, 16, 20, [80], [3])])
def test_matrix_core_attention_over_latent_pages(H, kd, vd, window, lens, pos0):
    """Requests at other positions each, on shuffled pages: single rows whose context is shared out over several waves, and
    portions of prompts; heads that fill one and a half matrix instructions; keys that are no multiple of 32 channels.  One key
    just inside every row's window stands out."""
    from geneinfer_amd.kernels import ops
    from geneinfer_amd.parts import StepContext
    g = torch.Generator().manual_seed(H + kd)
    page, scale = 16, 0.2
    total = [p + n for p, n in zip(pos0, lens)]
    n_pages = sum(-(-t // page) for t in total)
    order = torch.randperm(n_pages + 2, generator=g).tolist()
    table = torch.full((len(lens) + 1, max(-(-t // page) for t in total) + 1), -1, dtype=torch.int32)
    cache = torch.zeros(n_pages + 2, page * (kd + vd), dtype=torch.bfloat16)
    keys = []
    for s, t in enumerate(total):
        k = torch.randn(t, kd, generator=g).to(torch.bfloat16)
        keys.append(k)
        for i in range(-(-t // page)):
            pg = order.pop()
            table[s, i] = pg
            block = k[i * page:(i + 1) * page]
            cache[pg, :block.shape[0] * kd] = block.reshape(-1)
            values = torch.zeros(vd, page, dtype=torch.bfloat16)
            values[:, :block.shape[0]] = block[:, :vd].T
            cache[pg, page * kd:] = values.reshape(-1)
    q = torch.randn(sum(lens), H * kd, generator=g)
    row = 0
    want = []
    for s, (p0, n) in enumerate(zip(pos0, lens)):
        kf = keys[s].double()
        for i in range(n):
            p = p0 + i
            lo = 0 if window is None else max(0, p - window + 1)
            q.view(-1, H, kd)[row + i, :, :8] = 4.0 * kf[lo, :8] / kf[lo, :8].norm()        # the oldest key the row sees stands out
        qb = q[row:row + n].to(torch.bfloat16).double().view(n, H, kd)
        scores = torch.einsum("thd,sd->hts", qb, kf) * scale
        i_, j_ = torch.arange(p0, p0 + n)[:, None], torch.arange(total[s])[None, :]
        seen = (j_ <= i_) & ((i_ - j_ < window) if window is not None else True)
        pr = torch.softmax(scores.masked_fill(~seen[None], float("-inf")), -1)
        want.append(torch.einsum("hts,sd->thd", pr, kf[:, :vd]).reshape(n, H * vd))
        row += n
    want = torch.cat(want)
    T = sum(lens)
    starts = [sum(lens[:i]) for i in range(len(lens))]
    pos = torch.tensor([p + i for p, n in zip(pos0, lens) for i in range(n)], dtype=torch.int32, device=DEV)
    slots = torch.tensor([s for s, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    ctx = StepContext(n_rows=T, dtype=torch.bfloat16, device=torch.device(DEV), tokens=slots, row_pos=pos, row_slot=slots, seg_slot=list(range(len(lens))),
                      seg_start=starts, seg_len=list(lens), seg_pos0=list(pos0))
    assert ops.latent_attention_bf16_supports(kd, vd, page)
    out = torch.empty(T, H * vd, dtype=torch.bfloat16, device=DEV)
    ops.latent_attention_bf16(q.to(DEV, torch.bfloat16), cache.to(DEV), out, ctx, table.to(DEV), H, kd, vd, page, window, scale)
    assert relative_error(out, want) < 1.5e-2                                   # (probabilities and outputs are kept in bfloat16)
    exact = torch.empty(T, H * vd, dtype=torch.bfloat16, device=DEV)
    ops.attention_general(q.to(DEV, torch.bfloat16), cache.to(DEV), exact, ctx, table.to(DEV), H, 1, kd, page_size=page, value_dim=vd, window=window, scale=scale)
    assert relative_error(exact, want) < 6e-3 and relative_error(out, exact.double()) < 1.5e-2


@pytest.mark.parametrize("rows, H, k, n", [(1, 8, 32, 128), (37, 3, 72, 40), (300, 32, 64, 256), (16, 2, 256, 64), (5, 1, 8, 7)])
def test_every_head_s_product_in_one_launch(rows, H, k, n):
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(rows + k)
    a, w = torch.randn(rows, H * k, generator=g).to(torch.bfloat16), torch.randn(H, n, k, generator=g).to(torch.bfloat16)
    want = torch.einsum("thk,hnk->thn", a.double().view(rows, H, k), w.double())
    for dtype, stride, tol in ((torch.float32, n, 1e-5), (torch.bfloat16, n + 24, 5e-3)):
        out = torch.zeros(rows, H * stride, dtype=dtype, device=DEV)
        assert ops.heads_product(a.to(DEV), w.to(DEV), out, H, stride)
        got = out.view(rows, H, stride)
        assert relative_error(got[:, :, :n], want) < tol and (got[:, :, n:] == 0).all()
    assert not ops.heads_product(a.to(DEV)[:, 1:], w.to(DEV), out, H, n)           # operands it does not take: the caller goes head by head


# =============================================================================================== whole models
def _portions(n, sizes=(7, 2, 5, 3, 2, 11, 1, 4, 2, 19)):
    out, i = [], 0
    while sum(out) + sizes[i % len(sizes)] <= n:
        out.append(sizes[i % len(sizes)])
        i += 1
    return out


CUTS = {"whole": lambda n: [n], "singly": lambda n: [], "most then singly": lambda n: [n - 9], "portions": _portions, "twos": lambda n: [2] * (n // 2)}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_float32_logits_match_the_plain_model_and_do_not_depend_on_the_cut(folders, name):
    tokens = _prompt(CONFIGS[name], 75, 5)
    runner = make_runner(folders, name, "float32")
    got = {}
    for what, cuts in CUTS.items():
        runner.open(what)
        got[what] = feed(runner, what, tokens, cuts(len(tokens)))
        runner.close(what)
    check_against_plain(folders, name, "float32", tokens, got["whole"], f"{name} whole")
    for what in CUTS:
        assert torch.equal(got[what], got["whole"]), f"{name}: the logits of '{what}' differ from those of the whole prompt"


@pytest.mark.parametrize("name", list(CONFIGS))
def test_bfloat16_logits_lie_within_rounding_noise(folders, name):
    tokens = _prompt(CONFIGS[name], 90, 6)
    runner = make_runner(folders, name, "bfloat16")
    for what in ("whole", "portions", "most then singly"):
        runner.open(what)
        got = feed(runner, what, tokens, CUTS[what](len(tokens)))
        runner.close(what)
        check_against_plain(folders, name, "bfloat16", tokens, got, f"{name} {what}")


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "float32"), ("D", "float32"), ("E", "float32"), ("A", "bfloat16"), ("C", "bfloat16")])
def test_mixed_batches_on_a_pool_that_is_used_again(folders, name, dtype):
    """Up to four live requests, portions of some beside single tokens of others, through a pool that holds less than all requests
    together and four state slots: pages and slots are freed and used again.  Every request's logits against itself alone."""
    import random
    import traces
    from geneinfer_amd.engine import StepEntry
    cfg = CONFIGS[name]
    rng = random.Random(8)
    requests = {f"q{i}": [rng.randrange(cfg["vocab"]) for _ in range(n)] for i, n in enumerate([50, 1, 33, 77, 40, 9, 2, 61])}
    steps = traces.mixed(requests, seed=5)
    runner = make_runner(folders, name, dtype, max_tokens=traces.peak_tokens(steps, 64), max_requests=4)
    got = {}
    where = traces.wanted_positions(steps)
    for s in steps:
        for e in s["entries"]:
            if not runner.is_open(e["id"]):
                runner.open(e["id"])
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            for key, row in zip(where[s["step"]], logits.cpu()):
                got[key] = row.clone()
        for rid in s["end"]:
            runner.close(rid)
    runner.cache.check_consistency()
    alone = make_runner(folders, name, dtype)
    for rid, tokens in requests.items():
        mine = {p: row for (r, p), row in got.items() if r == rid}
        assert len(mine) == len(tokens)
        if dtype == "float32":
            alone.open(rid)
            ref = feed(alone, rid, tokens, [len(tokens)])
            alone.close(rid)
            assert all(torch.equal(mine[p], ref[p]) for p in mine), f"{name} {rid}: a mixed batch changed the logits"
        else:
            exact, rounded = plain_logits(folders, name, tokens), plain_logits(folders, name, tokens, rounded=True)
            assert_within_bfloat16_noise(mine, lambda p: exact[p], lambda p: rounded[p], f"{name} mixed {rid}")


@pytest.mark.parametrize("name, dtype", [("C", "bfloat16"), ("C", "float32"), ("B", "float32")])
def test_long_portions_beside_single_rows(folders, name, dtype):
    """Steps that hold portions of a hundred rows and more of some requests (the kernels that take the rows of prompts tile by tile)
    beside single rows and short portions of others, every request at another position."""
    from geneinfer_amd.engine import StepEntry
    cfg = CONFIGS[name]
    tokens = {r: _prompt(cfg, n, 70 + n) for r, n in (("a", 330), ("b", 150), ("c", 171), ("d", 40))}
    schedule = [[("a", 100), ("c", 70)], [("a", 130), ("b", 1), ("c", 1)], [("b", 140), ("a", 1), ("c", 99), ("d", 3)], [("a", 99), ("b", 2), ("c", 1), ("d", 37)], [("b", 7)]]
    runner = make_runner(folders, name, dtype, max_tokens=1024, max_requests=4)
    at, got = {r: 0 for r in tokens}, {r: [] for r in tokens}
    for step in schedule:
        entries = []
        for r, n in step:
            if not runner.is_open(r):
                runner.open(r)
            entries.append(StepEntry(r, tokens[r][at[r]:at[r] + n], tuple(range(n))))
        logits = runner.step(entries).cpu()
        row = 0
        for r, n in step:
            got[r].append(logits[row:row + n])
            row += n
            at[r] += n
    assert all(at[r] == len(t) for r, t in tokens.items())
    alone = make_runner(folders, name, dtype)
    for r, t in tokens.items():
        mine = torch.cat(got[r])
        if dtype == "float32":
            alone.open(r)
            assert torch.equal(mine, feed(alone, r, t, [len(t)])), f"{name} {r}: a mixed step changed the logits"
            alone.close(r)
        check_against_plain(folders, name, dtype, t, mine, f"{name} {r} in mixed steps")


def test_long_decoding_carries_state_and_passes_windows(folders):
    """A short prompt and 300 tokens decoded one by one through the captured decode step: the memories carry, and every window
    passes over decoded tokens only."""
    tokens = _prompt(CONFIGS["A"], 312, 9)
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folders, "A", dtype)
        runner.open("r")
        got = feed(runner, "r", tokens, [12])
        assert runner.steps_replayed > 250
        check_against_plain(folders, "A", dtype, tokens, got, f"A decoding ({dtype})")


def test_first_layer_of_a_family_of_blended_values_may_come_anywhere(folders, tmp_path):
    """The same layers in another order: the family's first layer is now the model's last-but-one, and a layer that does not blend
    lies between."""
    import copy
    cfg = copy.deepcopy(CONFIGS["B"])
    cfg["layers"] = [cfg["layers"][i] for i in (4, 1, 3, 2, 0, 5)]
    cfg["layers"][2]["mixer"]["vdim"], cfg["layers"][2]["mixer"]["kv_heads"], cfg["layers"][2]["mixer"]["heads"] = 48, 3, 3
    write_model(tmp_path / "m", cfg, seed=4)
    from geneinfer_amd.engine import Runner, load_model
    tokens = _prompt(cfg, 40, 2)
    want = P.forward(cfg, stored_weights(tmp_path / "m"), tokens)
    runner = Runner(load_model(tmp_path / "m", "float32", DEV), page_size=8, max_tokens=256, max_requests=2)
    runner.open("r")
    got = feed(runner, "r", tokens, [13, 2])
    assert relative_error(got, want) < 5e-5


# =============================================================================================== entry points
@pytest.mark.parametrize("name", ["A", "D"])
def test_greedy_generation_through_the_entry_point_and_the_scheduler(folders, name):
    """Greedy tokens of several prompts, one by one through `LLM.generate` and together through the scheduler (more requests than
    it runs at once, prompts in portions), against the plain model's, as far as the plain model's two best logits are clearly apart."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig, EngineRequest
    from geneinfer_amd.sampling import SamplerConfig
    cfg, w = CONFIGS[name], stored_weights(folders[name])
    prompts = [_prompt(cfg, n, 30 + n) for n in (5, 23, 1, 40)]
    want, sure = [], []
    for p in prompts:
        tokens = P.greedy(cfg, w, p, 8)
        top2 = torch.topk(P.forward(cfg, w, p + tokens)[len(p) - 1:-1], 2, dim=-1).values
        clear = [bool(c) for c in (top2[:, 0] - top2[:, 1] > 1e-3)]
        want.append(tokens)
        sure.append(clear.index(False) if False in clear else len(clear))
    assert sum(sure) >= 24
    llm = gi.LLM(str(folders[name]), dtype="float32", page_size=PAGE_SIZE[name], max_tokens=512, max_running=2)
    assert type(llm.model.config).__name__ == "RigalornConfig"
    for p, t, n in zip(prompts, want, sure):
        assert llm.generate(p, steps=len(p) + 7, temperature=0.0).generated_tokens[:n] == t[:n]
    eng = llm.engine(EngineConfig(max_running=2, step_rows=16, prefill_chunk=6))
    ids = [eng.submit(EngineRequest(p, len(p) + 7, SamplerConfig(0.0))) for p in prompts]
    eng.run_until_idle()
    for i, t, n in zip(ids, want, sure):
        assert eng.result(i).generated_tokens[:n] == t[:n]


@pytest.mark.parametrize("dtype, mode", [("float32", "mixed"), ("bfloat16", "mixed"), ("float32", "portions")])
def test_replay_through_the_command_line(folders, tmp_path, dtype, mode):
    """bin/trace_run as a child process on a Rigalorn folder: up to four live requests, portions beside single tokens, a pool that
    holds less than all requests together, so that pages and state slots are used again."""
    import json
    import random
    import subprocess
    from pathlib import Path
    import numpy as np
    import traces
    root = Path(__file__).resolve().parent.parent
    cfg = CONFIGS["B"]
    rng = random.Random(4)
    requests = {f"q{i}": [rng.randrange(cfg["vocab"]) for _ in range(n)] for i, n in enumerate([50, 1, 33, 77, 40, 9])}
    steps = traces.mixed(requests, seed=3) if mode == "mixed" else traces.portions(requests)
    out = tmp_path / "out"
    cmd = [str(root / "bin" / "trace_run"), "--model", str(folders["B"]), "--dtype", dtype, "--out", str(out), "--max-tokens", str(traces.peak_tokens(steps, 64)),
           "--page-size", "8"]
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
        exact = plain_logits(folders, "B", tokens)
        if dtype == "float32":
            single = plain_logits(folders, "B", tokens, dtype=torch.float32)
            noise = max(relative_error(single[p], exact[p]) for p in mine)
            assert max(relative_error(row, exact[p]) for p, row in mine.items()) < 4 * noise + 1e-5
        else:
            rounded = plain_logits(folders, "B", tokens, rounded=True)
            assert_within_bfloat16_noise(mine, lambda p: exact[p], lambda p: rounded[p], f"replay {mode} {rid}")


def test_generation_from_the_command_line_on_random_weights():
    """bin/gi_generate on the shipped example configuration, random weights, greedy: runs, and twice the same."""
    import subprocess
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    cmd = [str(root / "bin" / "gi_generate"), "--config", str(root / "configs" / "rigalorn-small.json"), "--random-seed", "3", "--prompt-ids", "5 17 3 999 4",
           "--steps", "24", "--temperature", "0"]
    runs = [subprocess.run(cmd, capture_output=True, text=True, timeout=280) for _ in range(2)]
    assert all(r.returncode == 0 for r in runs), runs[0].stderr[-2000:]
    assert runs[0].stdout == runs[1].stdout and len(runs[0].stdout.split()) >= 20


def test_the_new_parts_serve_other_designs():
    """The parts are not Rigalorn's own: a model put together by hand, a pre-norm layer around the gated delta rule and a SiLU-gated
    feed-forward, and a parallel layer around a plain Llama attention and the feed-forward without a gate, through the same step
    function; against a plain computation from the plain implementations' functions."""
    from geneinfer_amd.config import (AttentionSpec, DenseMlpSpec, GatedDeltaSpec, LayerSpec, ModelSpec, RmsNormSpec, RotarySpec, RunEntry, SwiGluSpec)
    from geneinfer_amd.engine import Runner
    from geneinfer_amd.engine.model import DecoderModel
    from geneinfer_amd.parts import model_tensor_needs
    from geneinfer_amd.weights import random_tensors
    from plain_llama import causal_attention, rms_norm, rope_inverse_frequencies, rope_rotate, swiglu
    d, vocab, eps = 64, 100, 1e-5
    norm = lambda name: RmsNormSpec(d, eps, name)
    delta = GatedDeltaSpec(d, 2, 1, 8, 24, 3, eps, "m.q", "m.k", "m.v", "m.qc", "m.kc", "m.vc", "m.a", "m.al", "m.dt", "m.b", "m.g", "m.n", "m.o")
    spec = ModelSpec(architecture="by hand", vocab_size=vocab, hidden_size=d, max_positions=256, embedding="emb", final_norm=norm("fn"), lm_head="head", layers=(
        LayerSpec(mixer=delta, feed_forward=SwiGluSpec(d, 80, "g.g", "g.u", "g.d"), mixer_norm=norm("p1"), feed_forward_norm=norm("p2"), block="prenorm"),
        LayerSpec(mixer=AttentionSpec(d, 4, 2, 16, "a.q", "a.k", "a.v", "a.o", RotarySpec(16, 10000.0)), feed_forward=DenseMlpSpec(d, 96, "f.u", "f.d", "xielu", "f.act"),
                  mixer_norm=norm("n1"), feed_forward_norm=None, block="parallel")),
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
    h = rms_norm(x, w["p1"], eps)
    m = dict(heads=2, kv_heads=1, dim=8, vdim=24)
    names = {"q": "m.q", "k": "m.k", "v": "m.v", "q.conv": "m.qc", "k.conv": "m.kc", "v.conv": "m.vc", "a": "m.a", "A_log": "m.al", "dt_bias": "m.dt", "b": "m.b",
             "g": "m.g", "norm": "m.n", "o": "m.o"}
    x = x + P.delta(h, {k: w[v] for k, v in names.items()}, m, eps)
    x = x + swiglu(rms_norm(x, w["p2"], eps), w["g.g"], w["g.u"], w["g.d"])
    h = rms_norm(x, w["n1"], eps)
    f = rope_inverse_frequencies(16, 10000.0)
    q, k = rope_rotate((h @ w["a.q"].T).view(T, 4, 16), pos, f), rope_rotate((h @ w["a.k"].T).view(T, 2, 16), pos, f)
    y = causal_attention(q, k, (h @ w["a.v"].T).view(T, 2, 16)).reshape(T, 64) @ w["a.o"].T
    x = x + y + P.dense_mlp(h, w["f.u"], w["f.d"], w["f.act"])
    want = rms_norm(x, w["fn"], eps) @ w["head"].T
    assert relative_error(got["whole"], want) < 5e-5
