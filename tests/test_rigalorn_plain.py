"""What pins the plain Rigalorn implementation (`plain_rigalorn.py`) beside a reading of its equations, and what the
configuration class accepts and refuses.  All on the CPU."""
import copy
import math

import pytest
import torch

import plain_rigalorn as P
from rigalorn_folders import CONFIGS, random_weights, tensor_layout

D = torch.float64


def test_rotations_keep_lengths_and_depend_on_distance_only():
    g = torch.Generator().manual_seed(0)
    f, _ = P.rotary_frequencies(8, 50.0)
    q, k = torch.randn(12, 1, 14, generator=g, dtype=D), torch.randn(12, 1, 14, generator=g, dtype=D)
    for turn in (lambda x: P.rotate_half_split(x, f), lambda x: P.rotate_interleaved(x, f)):
        tq, tk = turn(q), turn(k)
        assert torch.allclose(tq.norm(dim=-1), q.norm(dim=-1)) and torch.equal(tq[..., 8:], q[..., 8:])
        # the same two vectors at positions (3, 1) and (9, 7): equal products
        a, b = q[0, 0], k[1, 0]
        at = lambda v, p: turn(torch.stack([v] * 12)[:, None, :])[p, 0]
        assert torch.allclose(at(a, 3) @ at(b, 1), at(a, 9) @ at(b, 7))
    # the two pairings differ by a permutation of the turned channels
    perm = torch.tensor([0, 4, 1, 5, 2, 6, 3, 7] + list(range(8, 14)))
    assert torch.allclose(P.rotate_half_split(q, f)[..., perm], P.rotate_interleaved(q[..., perm], f))


def test_stretched_frequencies_by_hand():
    """dims 8, base 16, original 16: pair i makes 16 / (2 pi 16^(i/4)) turns over the original context: 2.55, 1.27, 0.64, 0.32.
    With fast = 2 and slow = 0.5 the (fractional) pairs that make exactly those turns are 0.35 and 2.35: lo = 0, hi = 3, the ramp
    is i / 3."""
    f, mag = P.rotary_frequencies(8, 16.0, dict(factor=4.0, original=16, fast=2.0, slow=0.5))
    plain = [16.0 ** (-i / 4) for i in range(4)]
    for i in range(4):
        ramp = i / 3
        assert math.isclose(f[i], plain[i] / 4.0 * ramp + plain[i] * (1 - ramp), rel_tol=1e-12)
    assert f[0] == plain[0] and math.isclose(mag, 0.1 * math.log(4.0) + 1.0)
    assert P.rotary_frequencies(8, 16.0) == (plain, 1.0)


def test_the_engine_s_configuration_computes_the_same_frequencies():
    from geneinfer_amd.config.rigalorn import YarnScaling, yarn_frequencies
    for dims, base, s in ((8, 16.0, dict(factor=4.0, original=16, fast=2.0, slow=0.5)), (48, 20000.0, dict(factor=6.0, original=2048, fast=24.0, slow=2.0)),
                          (2, 7.0, dict(factor=2.0, original=8, fast=1.0, slow=1.0)), (16, 100.0, dict(factor=3.0, original=4096, fast=0.001, slow=0.0005))):
        scaling = YarnScaling(s["factor"], s["original"], s["fast"], s["slow"])
        f, mag = P.rotary_frequencies(dims, base, s)
        assert list(yarn_frequencies(dims, base, scaling)) == pytest.approx(f, rel=1e-14) and scaling.magnitude() == pytest.approx(mag)


def test_attention_against_the_library_routine():
    g = torch.Generator().manual_seed(1)
    T, H, G, d, dv = 21, 6, 2, 8, 5
    q, k, v = torch.randn(T, H, d, generator=g, dtype=D), torch.randn(T, G, d, generator=g, dtype=D), torch.randn(T, G, dv, generator=g, dtype=D)
    for window in (None, 1, 4, 21, 40):
        mask = P.window_mask(T, window)
        want = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(3, 1).transpose(0, 1), v.repeat_interleave(3, 1).transpose(0, 1),
                                                                attn_mask=mask, scale=0.3).transpose(0, 1)
        assert torch.allclose(P.softmax_attention(q, k, v, 0.3, window), want)
    assert P.window_mask(6, 2).tolist()[4] == [False, False, False, True, True, False]


def test_activation_is_smooth_at_zero_and_bounded_on_the_left():
    p, q = torch.tensor(0.3, dtype=D), torch.tensor(-0.4, dtype=D)
    z = torch.tensor([-1e-6, 0.0, 1e-6], dtype=D)
    y = P.xielu(z, p, q)
    assert y[1] == 0 and torch.allclose((y[2] - y[0]) / 2e-6, torch.tensor(0.5, dtype=D), atol=1e-5)
    an = 0.5 + math.log1p(math.exp(-0.4))
    assert math.isclose(float(P.xielu(torch.tensor(-40.0, dtype=D), p, q)), an * (-1 + 40) - 20, rel_tol=1e-12)
    assert math.isclose(float(P.xielu(torch.tensor(3.0, dtype=D), p, q)), math.log1p(math.exp(0.3)) * 9 + 1.5, rel_tol=1e-12)


def test_delta_rule_in_closed_form_for_two_tokens():
    """Token 0 writes beta0 k0 v0^T into an empty memory; token 1 reads g1 times that along k1, and corrects."""
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.randn(2, 5, generator=g, dtype=D), torch.randn(2, 5, generator=g, dtype=D), torch.randn(2, 3, generator=g, dtype=D)
    beta, decay = torch.tensor([0.7, 0.4], dtype=D), torch.tensor([0.9, 0.6], dtype=D)
    out = P.delta_rule(q, k, v, beta, decay)
    S0 = beta[0] * torch.outer(k[0], v[0])
    assert torch.allclose(out[0], S0.T @ q[0])
    S1 = decay[1] * S0
    S1 = S1 + torch.outer(k[1], beta[1] * (v[1] - S1.T @ k[1]))
    assert torch.allclose(out[1], S1.T @ q[1])
    # with beta = 1 and a unit key the memory returns the value just written
    ku = k[1] / k[1].norm()
    one = P.delta_rule(torch.stack([q[0], ku]), torch.stack([k[0], ku]), v, torch.tensor([0.7, 1.0], dtype=D), decay)
    assert torch.allclose(one[1], v[1])


def test_short_convolution_is_causal_and_ends_on_the_token_s_own_tap():
    x = torch.zeros(6, 2, dtype=D)
    x[2] = torch.tensor([1.0, 2.0])
    taps = torch.tensor([[0.1, 0.2, 0.3], [1.0, 0.0, -1.0]], dtype=D)
    got = P.short_conv_silu(x, taps)
    silu = lambda z: z * torch.sigmoid(z)
    want = torch.zeros(6, 2, dtype=D)
    want[2], want[3], want[4] = silu(torch.tensor([0.3, -2.0], dtype=D)), silu(torch.tensor([0.2, 0.0], dtype=D)), silu(torch.tensor([0.1, 2.0], dtype=D))
    assert torch.allclose(got, want)


def test_latents_folded_into_query_and_output_give_the_same_layer():
    """score = (W_uk^T q) . c + q_rot . k_rot and o = W_uv (sum p c): what an engine that caches only c and k_rot computes."""
    g = torch.Generator().manual_seed(3)
    H, d, r, dv, q_rank, rank, hidden, T, eps = 2, 6, 4, 5, 9, 7, 10, 17, 1e-5
    m = dict(heads=H, dim=d, rot_dim=r, vdim=dv, kv_rank=rank, scale=0.37, rot=dict(dims=r, base=25.0), mask=dict(size=6))
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=D) * 0.4
    w = {"dq": rnd(q_rank, hidden), "dq.norm": 1 + rnd(q_rank), "uq": rnd(H * (d + r), q_rank), "dkv": rnd(rank + r, hidden), "dkv.norm": 1 + rnd(rank),
         "uk": rnd(H * d, rank), "uv": rnd(H * dv, rank), "o": rnd(hidden, H * dv)}
    h = rnd(T, hidden)
    want = P.latent_attention(h, w, m, eps)
    f, _ = P.rotary_frequencies(r, 25.0)
    q = (P.rms_norm(h @ w["dq"].T, w["dq.norm"], eps) @ w["uq"].T).view(T, H, d + r)
    down = h @ w["dkv"].T
    c, k_rot = P.rms_norm(down[:, :rank], w["dkv.norm"], eps), P.rotate_interleaved(down[:, None, rank:], f)[:, 0]
    folded = torch.einsum("thd,hdr->thr", q[..., :d], w["uk"].view(H, d, rank))
    scores = (torch.einsum("thr,sr->hts", folded, c) + torch.einsum("thr,sr->hts", P.rotate_interleaved(q[..., d:], f), k_rot)) * 0.37
    p = torch.softmax(scores.masked_fill(~P.window_mask(T, 6)[None], float("-inf")), dim=-1)
    o = torch.einsum("thr,hvr->thv", torch.einsum("hts,sr->thr", p, c), w["uv"].view(H, dv, rank)).reshape(T, H * dv)
    assert torch.allclose(o @ w["o"].T, want)


def test_a_layer_adds_both_halves_of_one_norm_and_zeroed_outputs_leave_the_embedding():
    cfg = CONFIGS["A"]
    w = random_weights(cfg, 1)
    for name in w:
        if name.endswith((".mix.o", ".mlp.down")):
            w[name] = torch.zeros_like(w[name])
    tokens = [3, 9, 27, 81]
    x = w["embed"].double()[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    want = P.rms_norm(x, w["final.norm"].double(), cfg["norm"]["eps"]) @ w["head"].double().T
    assert torch.allclose(P.forward(cfg, w, tokens), want)


def test_blended_values_change_every_layer_of_the_family_but_the_first():
    cfg = CONFIGS["A"]
    w = random_weights(cfg, 2)
    tokens = list(range(5, 30))
    outs = []
    base = P.forward(cfg, w, tokens, layer_outputs=outs)
    w2 = dict(w)
    w2["l2.mix.vmix"] = torch.tensor(5.0)                     # the first layer's own weight is not read
    assert torch.equal(P.forward(cfg, w2, tokens), base)
    w3 = dict(w)
    w3["l4.mix.vmix"] = torch.tensor(0.0)                     # no blending: the layer's own values
    cfg_plain = copy.deepcopy(cfg)
    cfg_plain["layers"][4]["mixer"]["v_mix"] = False
    assert torch.allclose(P.forward(cfg, w3, tokens), P.forward(cfg_plain, w, tokens))
    assert not torch.allclose(P.forward(cfg, w3, tokens), base)


# ------------------------------------------------------------------------------------------------- the configuration
def test_configurations_read_back_equal_and_name_every_tensor():
    from geneinfer_amd.config import parse_config
    from geneinfer_amd.parts import model_tensor_needs
    import re
    for name, cfg in CONFIGS.items():
        config = parse_config(cfg)
        assert type(config).__name__ == "RigalornConfig" and type(config).from_dict(config.to_dict()) == config
        spec = config.model_spec()
        needs = {n.name: tuple(n.shape) for n in model_tensor_needs(spec)}
        have = dict(tensor_layout(cfg))
        unused = [n for n in have if n not in needs]
        assert all(any(re.fullmatch(p, n) for p in spec.ignorable_tensors) for n in unused) and len(unused) == (1 if name in "AB" else 0)
        assert all(have[n] == s for n, s in needs.items())
        assert all(l.block == "parallel" for l in spec.layers)


def test_configuration_refusals():
    from geneinfer_amd.config import ConfigError, parse_config
    def broken(change):
        cfg = copy.deepcopy(CONFIGS["A"])
        change(cfg)
        with pytest.raises(ConfigError):
            parse_config(cfg)
    broken(lambda c: c["layers"][0].update(type="mamba"))
    broken(lambda c: c["layers"][2]["mixer"].update(kv_heads=3))
    broken(lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7))
    broken(lambda c: c["layers"][2]["mixer"]["rot"].update(dims=64))
    broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=6))
    broken(lambda c: c["layers"][4]["mixer"].update(vdim=8))            # a family of blended values with value heads of two sizes
    broken(lambda c: c["layers"][0]["mlp"].update(kind="experts"))
    broken(lambda c: c["layers"][0]["mixer"].pop("conv"))
    broken(lambda c: c.pop("embedding"))
    broken(lambda c: c.update(layers=[]))


def test_cache_needs_by_layer_kind():
    from geneinfer_amd.cache import PagedKvNeed, StateNeed
    from geneinfer_amd.config import parse_config
    from geneinfer_amd.parts import block_class
    spec = parse_config(CONFIGS["A"]).model_spec()
    needs = [block_class(l.block).cache_need(l) for l in spec.layers]
    assert isinstance(needs[0], StateNeed) and needs[0].shape == (4 * 6 * 16 * 4 + 3 * (2 * 2 * 16 + 4 * 24),)
    assert needs[1] == PagedKvNeed(1, 40, 20, 32, None) and needs[1].elements_per_position() == 72
    assert needs[2] == PagedKvNeed(2, 32, 12, 16, None) and needs[4] == PagedKvNeed(2, 24, 9, 16, None)
    assert needs[1].first_visible(25) == 6 and needs[2].first_visible(11) == 0 and needs[2].first_visible(12) == 1
