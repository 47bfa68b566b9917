"""Host-side pieces of the Sizitar path that need no GPU: the config reader, the fused weight layout, the registry entry, and
identities and sensitivities of the oracle itself (causality, the reach of the convolutions, the delta rule as an error-correcting
write and its chunk-wise form, the sink, the routing weights, the loop)."""
import copy
import math

import pytest
import torch

from oracle import sizitar_ref as ZR
from tests import sizitar_util as Z

F32_BAR = 2e-4


def rel_err(got, want):
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).max())


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def small():
    return Z.config([Z.channel_delta(heads=4, kv_heads=2, dim=6, vdim=5, conv=4, decay_rank=3, gate_rank=7, mlp=Z.dense(14)),
                     Z.attention(heads=6, kv_heads=3, dim=8, vdim=10, conv=3, rot=4, base=500.0, scale=0.3, mlp=Z.moe()),
                     Z.delta(heads=3, kv_heads=1, dim=10, vdim=4, conv=2, mlp=None)], width=24, loop=(0, 2, 3), logit_scale=0.25)


def test_config_reader_takes_every_size_and_constant():
    from vox_serve_amd.model.sizitar import config_from_dict
    c = config_from_dict(Z.public(small()))
    assert (c.width, c.vocab, c.eps, c.norm_kind, c.norm_groups, c.norm_one_plus, c.logit_scale, c.loop) == (24, 40, 1e-5, "rms_groups", 1, True, 0.25, (0, 2, 3))
    a, b, d = c.layers
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.conv_taps, a.decay_channels, a.gate_act, a.layer_scale) == ("delta", 4, 2, 6, 5, 4, True, "sigmoid", True)
    assert (a.ff, a.ff_kind, a.ff_act, a.moe, a.block) == (14, "gated", "swish", None, "sequential")
    assert (b.kind, b.heads, b.kv_heads, b.dim, b.vdim, b.conv_taps, b.rot_dims, b.rot_base, b.scale, b.qk_norm_whole, b.sink) == \
        ("causal_attention", 6, 3, 8, 10, 3, 4, 500.0, 0.3, True, True)
    assert (b.moe.experts, b.moe.identity, b.moe.top, b.moe.ff, b.moe.shared_ff, b.moe.expert_form, b.moe.expert_act, b.moe.router_bias) == \
        (5, 0, 2, 12, 10, "up_down", "relu2", True)
    assert (b.moe.score, b.moe.renorm, b.moe.scale_input, b.moe.limit) == ("softmax", True, False, math.inf)
    assert (d.kind, d.decay_channels, d.lora, d.gate_rank, d.gate_act, d.ff, d.moe) == ("delta", False, 0, 0, "silu", 0, None)
    assert b.n_in == 48 + 24 + 30 and b.cache_values() == 3 * 18 and b.state_floats(24) == 2 * 102
    assert d.n_in == 10 + 10 + 12 + 3 + 3 + 12 and d.state_floats(24) == 3 * 10 * 4 + 1 * 32
    assert [i for i, _ in c.runs()] == [0, 1, 0, 1, 0, 1, 2]
    for key, val in (("architecture", "Other"),):
        bad = Z.public(small())
        bad[key] = val
        with pytest.raises(ValueError):
            config_from_dict(bad)
    bad = Z.public(small())
    bad["layers"][1]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        config_from_dict(bad)
    bad = Z.public(small())
    bad["layers"][0]["type"] = "other"
    with pytest.raises(ValueError):
        config_from_dict(bad)
    bad = Z.public(small())
    bad["layers"][0]["mixer"]["kv_heads"] = 3
    with pytest.raises(ValueError):
        config_from_dict(bad)
    bad = Z.public(small())
    bad["loop"]["stop"] = 4
    with pytest.raises(ValueError):
        config_from_dict(bad)
    plain = Z.public(small())
    del plain["loop"], plain["logit_scale"], plain["layers"][1]["mixer"]["rot"]
    c = config_from_dict(plain)
    assert c.loop is None and c.logit_scale == 1.0 and c.layers[1].rot_dims == 0
    once = Z.public(small())
    once["loop"]["times"] = 1
    assert config_from_dict(once).loop is None


def test_pack_weights_layout():
    from vox_serve_amd.model.sizitar import config_from_dict, pack_weights
    cfg = small()
    S = Z.random_checkpoint(cfg, seed=3)
    c = config_from_dict(Z.public(cfg))
    w = pack_weights(S, c)
    a, b, d = w["layers"]
    # the bottleneck widths come from the checkpoint's shapes
    assert (c.layers[0].lora, c.layers[0].gate_rank) == (3, 7) and c.layers[0].n_in == 12 + 12 + 20 + 4 + 3 + 7
    assert tuple(a["w_in"].shape) == (58, 24) and torch.equal(a["w_in"][12:24], S["l0.mix.k"]) and torch.equal(a["w_in"][44:48], S["l0.mix.b"])
    assert torch.equal(a["w_in"][48:51], S["l0.mix.a1"]) and torch.equal(a["w_in"][51:], S["l0.mix.g1"])
    assert a["w_decay2"] is S["l0.mix.a2"] and a["w_gate2"] is S["l0.mix.g2"] and a["head_norm"] is S["l0.mix.norm"]
    assert tuple(a["conv_w"].shape) == (44, 4) and torch.equal(a["conv_w"][24:], S["l0.mix.v.conv"].float())
    assert tuple(a["w_up"].shape) == (28, 24) and torch.equal(a["w_up"][14:], S["l0.mlp.up"]) and a["ls2"] is S["l0.ls2"]
    assert tuple(b["w_in"].shape) == (102, 24) and torch.equal(b["w_in"][48:72], S["l1.mix.k"]) and tuple(b["conv_w"].shape) == (102, 3)
    assert b["q_norm"] is S["l1.mix.q.norm"] and tuple(b["q_norm"].shape) == (48,)
    assert tuple(b["moe"]["w_gate_up"].shape) == (5, 12, 24) and torch.equal(b["moe"]["w_gate_up"][2], S["l1.mlp.e2.up"])
    assert tuple(b["moe"]["w_down"].shape) == (5, 24, 12) and b["moe"]["shared_gate_up"] is S["l1.mlp.shared.up"]
    assert torch.equal(b["moe"]["router_bias"], S["l1.mlp.router.b"])
    assert tuple(d["w_in"].shape) == (50, 24) and torch.equal(d["w_in"][35:38], S["l2.mix.a"]) and torch.equal(d["w_in"][38:], S["l2.mix.g"])
    assert "moe" not in d and "w_up" not in d and d["norm2"] is None and d["ls2"] is None
    short = dict(S)
    short["l0.mix.q.conv"] = S["l0.mix.q.conv"][:, :3].contiguous()
    with pytest.raises((ValueError, RuntimeError)):
        pack_weights(short, c)


def test_synthetic_weights_fit_the_reader():
    from vox_serve_amd.model.sizitar import config_from_dict, pack_weights, synth_weights
    c = config_from_dict(Z.public(small()))
    S = synth_weights(c)
    assert set(S) == set(Z.random_checkpoint(small()))
    assert len(pack_weights(S, c)["layers"]) == 3


def test_registry_names_the_design():
    from vox_serve_amd.model import MODEL_REGISTRY, get_model_class
    assert "sizitar" in MODEL_REGISTRY and get_model_class("Sizitar") is MODEL_REGISTRY["sizitar"]


def test_oracle_is_causal_and_deterministic():
    cfg = small()
    S = Z.random_checkpoint(cfg, seed=5)
    toks = tokens(30, 40, 6)
    full = ZR.forward(cfg, S, toks)
    assert torch.allclose(ZR.forward(cfg, S, toks[:17]), full[:17], atol=1e-12)
    other = list(toks)
    other[20] = (other[20] + 1) % 40
    assert torch.allclose(ZR.forward(cfg, S, other)[:20], full[:20], atol=1e-12)
    assert not torch.allclose(ZR.forward(cfg, S, other)[20:], full[20:], atol=1e-6)


def test_oracle_loop_is_the_unrolled_stack():
    """Layers 0..1 three times over the same weights = a six-layer stack that holds copies of them."""
    cfg = small()
    S = Z.random_checkpoint(cfg, seed=7)
    flat = copy.deepcopy(cfg)
    del flat["loop"]
    flat["layers"] = [copy.deepcopy(cfg["layers"][i]) for i in (0, 1, 0, 1, 0, 1, 2)]
    S2 = {k: v for k, v in S.items() if not k.startswith("l")}
    for new, old in enumerate((0, 1, 0, 1, 0, 1, 2)):
        S2.update({f"l{new}." + k[len(f"l{old}."):]: v for k, v in S.items() if k.startswith(f"l{old}.")})
    toks = tokens(20, 40, 8)
    trace = []
    assert torch.allclose(ZR.forward(cfg, S, toks, trace), ZR.forward(flat, S2, toks), atol=1e-12)
    assert len(trace) == 7


def test_short_convolution_reach_and_order():
    u = torch.arange(1.0, 7.0, dtype=torch.float64).view(6, 1)
    w = torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64)          # the last column is the current token's
    assert ZR.short_convolution(u, w).view(-1).tolist() == [1.0, 12.0, 123.0, 234.0, 345.0, 456.0]
    assert torch.equal(ZR.short_convolution(u, torch.tensor([[2.0]], dtype=torch.float64)), 2 * u)


def test_delta_rule_writes_what_is_missing():
    """Without decay and with beta = 1 a write makes the state return v for its key exactly (S^T k = v for a unit k); writing the same
    pair again changes nothing; the output reads the state after the write."""
    g = torch.Generator().manual_seed(11)
    T, d, e = 5, 6, 4
    k = ZR.unit_vectors(torch.randn(T, 1, d, generator=g, dtype=torch.float64))
    k[3] = k[1]
    v = torch.randn(T, 1, e, generator=g, dtype=torch.float64)
    v[3] = v[1]
    # (the unit-vector epsilon leaves |k|^2 = 1 - 1e-6: compare to that order)
    one = torch.ones(T, 1, dtype=torch.float64)
    o = ZR.delta_rule(k.clone(), k, v, one, torch.ones(T, 1, d, dtype=torch.float64))
    assert torch.allclose(o[0, 0], v[0, 0] * (k[0, 0] @ k[0, 0]), atol=1e-12)
    # token 3 repeats token 1's pair on a state that tokens 2 has disturbed along k_1 only by its own overlap: reading k_1 returns v_1
    assert torch.allclose(o[3, 0], v[1, 0], atol=1e-5)
    # a decay of zero forgets everything before the current token
    o0 = ZR.delta_rule(k.clone(), k, v, one, torch.zeros(T, 1, d, dtype=torch.float64))
    for t in range(T):
        assert torch.allclose(o0[t, 0], v[t, 0] * (k[t, 0] @ k[t, 0]), atol=1e-12)


def test_delta_rule_is_linear_in_the_state_chunk_by_chunk():
    """The chunk-wise form the engine uses for long portions: S_out = A S_in + B with A from the identity (zero values) and B from a zero
    state; the outputs of a chunk replayed from its carry equal the token-by-token ones."""
    g = torch.Generator().manual_seed(13)
    T, d, e, cut = 12, 5, 3, 7
    q = torch.randn(T, 1, d, generator=g, dtype=torch.float64)
    k = ZR.unit_vectors(torch.randn(T, 1, d, generator=g, dtype=torch.float64))
    v = torch.randn(T, 1, e, generator=g, dtype=torch.float64)
    beta = torch.rand(T, 1, generator=g, dtype=torch.float64)
    dec = torch.rand(T, 1, d, generator=g, dtype=torch.float64)

    def run(S, lo, hi, values=True):
        outs = []
        for t in range(lo, hi):
            S = dec[t, 0].unsqueeze(1) * S
            u = beta[t, 0] * ((v[t, 0] if values else torch.zeros(S.shape[1], dtype=torch.float64)) - S.T @ k[t, 0])
            S = S + torch.outer(k[t, 0], u)
            outs.append(S.T @ q[t, 0])
        return S, torch.stack(outs)
    whole = ZR.delta_rule(q, k, v, beta, dec)[:, 0]
    S1, o1 = run(torch.zeros(d, e, dtype=torch.float64), 0, cut)
    A, _ = run(torch.eye(d, dtype=torch.float64), cut, T, values=False)
    B, _ = run(torch.zeros(d, e, dtype=torch.float64), cut, T)
    S2, o2 = run(S1, cut, T)
    assert torch.allclose(A @ S1 + B, S2, atol=1e-12)
    assert torch.allclose(torch.cat([o1, o2]), whole, atol=1e-12)


def test_sink_softmax():
    s = torch.tensor([[0.0, math.log(3.0), -math.inf]], dtype=torch.float64)
    assert torch.allclose(ZR.sink_softmax(s), torch.tensor([[0.2, 0.6, 0.0]], dtype=torch.float64))
    big = torch.tensor([[800.0, 799.0]], dtype=torch.float64)
    assert torch.isfinite(ZR.sink_softmax(big)).all() and abs(float(ZR.sink_softmax(big).sum()) - 1.0) < 1e-12
    low = torch.tensor([[-800.0, -801.0]], dtype=torch.float64)
    assert float(ZR.sink_softmax(low).sum()) == 0.0


def test_rotation_depends_on_distance_only_and_leaves_the_rest():
    x = torch.randn(4, 2, 10, dtype=torch.float64, generator=torch.Generator().manual_seed(17))
    y = ZR.rotate_pairs(x, torch.arange(4), 6, 100.0)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.equal(y[0], x[0])
    a = ZR.rotate_pairs(x, torch.arange(4), 6, 100.0)
    b = ZR.rotate_pairs(x, torch.arange(4) + 9, 6, 100.0)
    assert torch.allclose(a[3, 0] @ a[1, 1], b[3, 0] @ b[1, 1], atol=1e-12)
    # the first pair turns by one radian a position
    e0 = torch.zeros(2, 1, 4, dtype=torch.float64)
    e0[:, :, 0] = 1.0
    r = ZR.rotate_pairs(e0, torch.arange(2), 4, 100.0)
    assert torch.allclose(r[1, 0, :2], torch.tensor([math.cos(1.0), math.sin(1.0)], dtype=torch.float64))


def test_attention_sensitivities():
    """Leaving out the sink, norming per head instead of over the whole projection, rotating before the norm's weight... each moves the
    oracle's logits by far more than the bar: the tests that compare the engine with the oracle would see them."""
    cfg = Z.config([Z.attention(heads=4, kv_heads=2, dim=8, vdim=8, conv=3, rot=4, scale=0.6)], width=16, vocab=32)
    S = Z.random_checkpoint(cfg, seed=41, qk_gain=2.0)
    toks = tokens(40, 32, 42)
    base = ZR.forward(cfg, S, toks)
    real = ZR.sink_softmax
    try:
        ZR.sink_softmax = lambda s: torch.softmax(s, -1)
        assert rel_err(ZR.forward(cfg, S, toks), base) > 50 * F32_BAR
    finally:
        ZR.sink_softmax = real
    real_rms = ZR.rms
    try:
        ZR.rms = lambda x, eps: real_rms(x.view(x.shape[0], -1, 8), eps).view(x.shape) if x.shape[-1] in (32, 16) and x.dim() == 2 else real_rms(x, eps)
        assert rel_err(ZR.forward(cfg, S, toks), base) > 50 * F32_BAR
    finally:
        ZR.rms = real_rms
    no_rot = copy.deepcopy(cfg)
    del no_rot["layers"][0]["mixer"]["rot"]
    assert rel_err(ZR.forward(no_rot, S, toks), base) > 50 * F32_BAR
    one_tap_less = dict(S)
    for n in ("q", "k", "v"):
        w = S[f"l0.mix.{n}.conv"].clone()
        w[:, 0] = 0
        one_tap_less[f"l0.mix.{n}.conv"] = w
    assert rel_err(ZR.forward(cfg, one_tap_less, toks), base) > 50 * F32_BAR


def test_delta_sensitivities():
    """The decay per channel against its mean over the head, half the write strength, the read before the write: each is far from the
    design by the oracle's own measure."""
    cfg = Z.config([Z.channel_delta(heads=2, kv_heads=1, dim=8, vdim=8, conv=3)], width=16, vocab=32)
    S = Z.random_checkpoint(cfg, seed=43, qk_gain=2.0)
    toks = tokens(40, 32, 44)
    base = ZR.forward(cfg, S, toks)
    real = ZR.delta_rule
    try:
        ZR.delta_rule = lambda q, k, v, beta, g: real(q, k, v, beta, g.mean(-1, keepdim=True).expand_as(g))
        assert rel_err(ZR.forward(cfg, S, toks), base) > 50 * F32_BAR
        ZR.delta_rule = lambda q, k, v, beta, g: real(q, k, v, beta * 0.5, g)
        assert rel_err(ZR.forward(cfg, S, toks), base) > 50 * F32_BAR

        def read_before_write(q, k, v, beta, g):
            # o_t from the decayed state without the current token's write: S^T q - u (k . q)
            T, H, d = q.shape
            out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
            for h in range(H):
                St = torch.zeros(d, v.shape[-1], dtype=q.dtype)
                for t in range(T):
                    St = g[t, h].unsqueeze(1) * St
                    out[t, h] = St.T @ q[t, h]
                    St = St + torch.outer(k[t, h], beta[t, h] * (v[t, h] - St.T @ k[t, h]))
            return out
        ZR.delta_rule = read_before_write
        assert rel_err(ZR.forward(cfg, S, toks), base) > 50 * F32_BAR
    finally:
        ZR.delta_rule = real


def test_oracle_routing_weights():
    g = torch.Generator().manual_seed(7)
    n = torch.randn(50, 8, generator=g, dtype=torch.float64)
    P = {"router": torch.randn(6, 8, generator=g, dtype=torch.float64), "router.b": torch.randn(6, generator=g, dtype=torch.float64)}
    chosen, w = ZR.route(P, n, 2)
    z = n @ P["router"].T + P["router.b"]
    assert torch.equal(chosen, z.topk(2, -1).indices)
    assert torch.allclose(w.sum(-1), torch.ones(50, dtype=torch.float64))
    # the softmax over the chosen logits = the softmax over all, renormalised over the chosen
    full = torch.softmax(z, -1).gather(1, chosen)
    assert torch.allclose(w, full / full.sum(-1, keepdim=True), atol=1e-12)
