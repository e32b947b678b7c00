"""What pins the plain Fekorax implementation (each mechanism stated a second way), and the CPU side of the design's
integration: its configuration, its parts' needs, and the cache manager's pages under a mask cut into chunks."""
import math

import pytest
import torch

from fekorax_folders import CONFIGS, FEKORAX_A, FEKORAX_B, tensor_layout
from plain_fekorax import gelu_tanh, matrix_memory, scaled_frequencies, sink_attention, turn_first_channels, unit_rms, visible

D = torch.float64


def test_matrix_memory_equals_its_unrolled_sum():
    """S_t unrolled: the weight of token j at time t is exp(li_j + F_t - F_j - m_t) with F the running sum of the forget gates'
    logarithms, and m_t = max(F_t, max_j (li_j + F_t - F_j)) because m starts at 0 (not at minus infinity)."""
    g = torch.Generator().manual_seed(3)
    T, H, dk, dv = 19, 2, 5, 7
    q, k, v = (torch.randn(T, H, d, generator=g, dtype=D) for d in (dk, dk, dv))
    li = 3.0 * torch.randn(T, H, generator=g, dtype=D)
    lf = torch.nn.functional.logsigmoid(4.0 * torch.randn(T, H, generator=g, dtype=D))
    got = matrix_memory(q, k, v, li, lf)
    F = lf.cumsum(0)
    for h in range(H):
        for t in range(T):
            logw = li[:t + 1, h] + F[t, h] - F[:t + 1, h]
            m = torch.maximum(F[t, h], logw.max())
            w = torch.exp(logw - m) * (k[:t + 1, h] @ q[t, h])
            want = (w[:, None] * v[:t + 1, h]).sum(0) / (torch.maximum(w.sum().abs(), torch.exp(-m)) + 1e-6)
            assert torch.allclose(got[t, h], want, rtol=1e-10, atol=1e-12)
    # with every forget gate wide open and input gates far below zero, the start value of m decides: exp(-m) = 1 is the denominator
    tiny = matrix_memory(q, k, v, torch.full((T, H), -30.0, dtype=D), torch.zeros(T, H, dtype=D))
    assert tiny.abs().max() < 1e-9


def test_sink_is_a_key_without_a_value():
    g = torch.Generator().manual_seed(5)
    Tq, H, G, dk, dv = 6, 4, 2, 8, 3
    q, k, v = torch.randn(Tq, H, dk, generator=g, dtype=D), torch.randn(Tq, G, dk, generator=g, dtype=D), torch.randn(Tq, G, dv, generator=g, dtype=D)
    sinks = torch.tensor([0.5, -2.0, 3.0, 0.0], dtype=D)
    mask = visible(torch.arange(Tq), torch.arange(Tq))
    got = sink_attention(q, k, v, mask, 0.3, sinks)
    for h in range(H):
        kk, vv = k[:, h // 2], v[:, h // 2]
        score = (q[:, h] @ kk.T * 0.3).masked_fill(~mask, -math.inf)
        p = torch.softmax(torch.cat([score, sinks[h].expand(Tq, 1)], dim=1), dim=1)      # (the sink is not scaled)
        assert torch.allclose(got[:, h], p[:, :Tq] @ vv, rtol=1e-12, atol=1e-14)
    # a sink far above every score leaves next to nothing; one far below is as if it were not there
    assert sink_attention(q, k, v, mask, 0.3, torch.full((H,), 60.0, dtype=D)).abs().max() < 1e-20
    plain = sink_attention(q, k, v, mask, 0.3, torch.full((H,), -1e9, dtype=D))
    assert torch.allclose(plain[0], v[0].repeat_interleave(2, 0), atol=1e-14)           # the first token sees itself alone


def test_chunks_are_counted_from_the_start_of_the_sequence():
    p = torch.arange(10)
    m = visible(p, p, 4)
    assert m[3].tolist() == [True, True, True, True] + [False] * 6
    assert m[4].tolist() == [False] * 4 + [True] + [False] * 5           # a chunk's first token sees itself alone
    assert m[9].tolist() == [False] * 8 + [True, True]
    late = visible(torch.tensor([9]), p, 4)                               # a token fed alone, later: the same row
    assert late[0].tolist() == m[9].tolist()
    assert visible(p, p)[9].all()


def test_frequencies_by_hand():
    f = scaled_frequencies(8, 100.0, dict(factor=4.0, low=1.0, high=2.0, original=16))
    base = [100.0 ** (-2 * i / 8) for i in range(4)]
    # wavelengths 6.28, 19.9, 62.8, 198.7 against original/high = 8 and original/low = 16: the first stays, the others are divided
    assert f[0] == base[0] and all(abs(a - b / 4.0) < 1e-15 for a, b in zip(f[1:], base[1:]))
    mid = scaled_frequencies(2, 1.0, dict(factor=8.0, low=1.0, high=4.0, original=4 * math.pi))      # wavelength 2 pi: original/wavelength = 2
    assert abs(mid[0] - ((1 - 1 / 3) / 8.0 + 1 / 3)) < 1e-15
    assert scaled_frequencies(6, 10.0) == [10.0 ** (-2 * i / 6) for i in range(3)]


def test_rotation_turns_the_first_channels_only_and_scores_see_distance():
    g = torch.Generator().manual_seed(7)
    x, y = torch.randn(1, 1, 12, generator=g, dtype=D), torch.randn(1, 1, 12, generator=g, dtype=D)
    f = scaled_frequencies(8, 30.0)
    at = lambda t, p: turn_first_channels(t, torch.tensor([p]), 8, f)
    assert torch.equal(at(x, 5)[..., 8:], x[..., 8:]) and torch.equal(at(x, 0), x)
    assert abs(float(at(x, 11).norm() - x.norm())) < 1e-12
    assert abs(float((at(x, 9) * at(y, 4)).sum() - (at(x, 105) * at(y, 100)).sum())) < 1e-10
    # pair (0, 4) at position 1: (u cos a - v sin a, v cos a + u sin a)
    e = torch.zeros(1, 1, 12, dtype=D); e[..., 0] = 1.0
    r = at(e, 1)
    assert abs(float(r[0, 0, 0]) - math.cos(f[0])) < 1e-15 and abs(float(r[0, 0, 4]) - math.sin(f[0])) < 1e-15


def test_small_parts():
    x = torch.tensor([[3.0, 4.0]], dtype=D)
    assert torch.allclose(unit_rms(x, 0.0), x / math.sqrt(12.5))
    z = torch.tensor([-1.0, 0.0, 2.0], dtype=D)
    assert torch.allclose(gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"), atol=1e-15)


# ------------------------------------------------------------------------------------ the framework's side, on the CPU
def test_configuration_reads_back_and_translates():
    from geneinfer_amd.config import parse_config
    from geneinfer_amd.parts import model_tensor_needs
    for cfg in CONFIGS.values():
        c = parse_config(cfg)
        assert parse_config(c.to_dict()) == c
        spec = c.model_spec()
        assert [e.cache_of for e in spec.run_order] == [l["mixer"].get("kv_from") for l in cfg["layers"]]
        assert sorted((n.name, tuple(n.shape)) for n in {x.name: x for x in model_tensor_needs(spec)}.values()) == sorted(tensor_layout(cfg))
        assert spec.lm_head == spec.embedding and spec.after_embedding[0].factor == cfg["embedding"]["scale"]
    a, b = parse_config(FEKORAX_A).model_spec(), parse_config(FEKORAX_B).model_spec()
    assert a.layers[0].mixer.keep_chunk == 24 and a.layers[2].mixer.keep_chunk == 24            # owner and reader cut alike
    assert b.layers[1].mixer.keep_chunk is None and b.layers[2].mixer.keep_chunk is None        # the reader's chunks are other ones
    assert b.layers[1].mixer.position.kind == "rotary_half_split" and a.layers[0].mixer.position.kind == "rotary_partial"
    assert b.layers[3].mixer.position is None and b.layers[3].mixer.chunk is None and b.layers[0].feed_forward is None


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown type"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "no earlier attention layer"),
    (lambda c: c["layers"][2]["mixer"].update(dim=16), "differ"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=34), "rot.dims"),
    (lambda c: c["layers"][0].update(mlp=dict(kind="routed", ff=8)), "unknown kind"),
    (lambda c: c.pop("vocab"), "'vocab'"),
])
def test_configuration_refuses(change, message):
    import copy
    from geneinfer_amd.config import ConfigError, parse_config
    cfg = copy.deepcopy(FEKORAX_A)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        parse_config(cfg)


def test_pages_of_chunks_gone_by_are_given_back():
    from geneinfer_amd.cache import CacheManager, PagedKvNeed, StateNeed
    need = PagedKvNeed(2, 32, None, 16, 24)
    other = PagedKvNeed(1, 24, None, None, None)
    cm = CacheManager([need, StateNeed((10,)), need, other], [None, None, 0, None], page_size=4, n_pages=12, max_requests=2, max_positions=200,
                      allocate_storage=False)
    assert len(cm.groups) == 2
    cm.open("a")
    cm.reserve([("a", 30)])
    cm.advance("a", 30)                      # the next row, at 30, sees 24 .. 29: pages 0 .. 5 go, 6 and 7 stay
    g, keep_all = cm.groups
    assert g.held_pages(cm.slot("a")) == [int(p) for p in g.table_host[cm.slot("a"), 6:8]] and g.pool.free_count == 10
    assert keep_all.pool.free_count == 4     # the group without a mask keeps everything
    cm.reserve([("a", 17)])
    cm.advance("a", 17)                      # length 47: the chunk 24 .. 47 is whole and still seen by nobody after 47? the next row is 47 itself
    assert g.first_live[cm.slot("a")] == 6
    cm.reserve([("a", 1)])
    cm.advance("a", 1)                       # length 48: the next row opens a new chunk, everything before goes
    assert g.held_pages(cm.slot("a")) == [] and g.pool.free_count == 12
    cm.check_consistency()
    assert not cm.enable_prefix_sharing()
    cm.close("a")
    assert keep_all.pool.free_count == 12
