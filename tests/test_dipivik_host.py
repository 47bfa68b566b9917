"""Host-side pieces of the Dipivik path that need no GPU: the config reader, the fused weight layout, the registry entry, and
identities and sensitivities of the oracle itself (causality, the window's edge, the closed form of retention, the bigram rows, the
routing weights)."""
import copy
import math

import pytest
import torch

from oracle import dipivik_ref as DR
from tests import dipivik_util as D

F32_BAR = 2e-4


def rel_err(got, want):
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).max())


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def small():
    return D.config([D.latent(mlp=D.moe()), D.retention(heads=3, dim=6, vdim=10, rot=4, decay=[0.5, 0.75, 0.875], mlp=D.dense(14)),
                     D.latent(heads=2, window=0, mlp=None)], width=24, softcap=5.0, bigram=(53, 7, 3))


def test_config_reader_takes_every_size_and_constant():
    from vox_serve_amd.model.dipivik import config_from_dict
    c = config_from_dict(small())
    assert (c.width, c.vocab, c.norm_kind, c.norm_groups, c.logit_softcap, c.bigram) == (24, 40, "rms_groups", 1, 5.0, (53, 7, 3))
    a, r, b = c.layers
    assert (a.kind, a.heads, a.dim, a.rot_dim, a.vdim, a.q_rank, a.kv_rank, a.window, a.rot_dims, a.rot_base) == \
        ("latent_attention", 3, 8, 4, 12, 10, 16, 7, 4, 100.0)
    assert a.block == r.block == b.block == "parallel_one_norm" and abs(a.scale - 1 / math.sqrt(12)) < 1e-12
    assert (a.moe.experts, a.moe.identity, a.moe.top, a.moe.ff, a.moe.shared_ff) == (5, 0, 2, 12, 10)
    assert (a.moe.score, a.moe.renorm, a.moe.scale_input, a.moe.up_offset, a.moe.act_alpha, a.moe.limit) == ("sigmoid", False, True, 0.0, 1.0, math.inf)
    assert (r.kind, r.heads, r.dim, r.vdim, r.rot_dims, r.rot_base, r.decay) == ("retention", 3, 6, 10, 4, 50.0, [0.5, 0.75, 0.875])
    assert (r.ff, r.ff_kind, r.ff_act, r.moe) == (14, "gated", "gelu_tanh", None)
    assert (b.window, b.ff, b.moe) == (0, 0, None)
    assert a.n_in == 10 + 16 + 4 + 3 and r.n_in == 2 * 18 + 2 * 30 and a.cache_values() == 20 and r.state_floats(24) == 3 * 6 * 10
    bad = small()
    bad["layers"][1]["mixer"]["decay"] = [0.5, 0.75]
    with pytest.raises(ValueError):
        config_from_dict(bad)
    bad = small()
    bad["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        config_from_dict(bad)
    bad = small()
    bad["architecture"] = "Other"
    with pytest.raises(ValueError):
        config_from_dict(bad)
    plain = small()
    del plain["embedding"], plain["logit_softcap"]
    c = config_from_dict(plain)
    assert c.bigram is None and c.logit_softcap == 0.0


def test_pack_weights_layout():
    from vox_serve_amd.model.dipivik import config_from_dict, pack_weights
    cfg = small()
    S = D.random_checkpoint(cfg, seed=3)
    c = config_from_dict(cfg)
    w = pack_weights(S, c)
    a, r, b = w["layers"]
    assert w["head"] is w["embedding"] and tuple(w["bigram"].shape) == (54, 24)
    assert tuple(a["w_in"].shape) == (33, 24) and torch.equal(a["w_in"][10:30], S["l0.mix.dkv"]) and torch.equal(a["w_in"][30:], S["l0.mix.g"])
    # head h of w_ukT is the transpose of its rows of uk: (plain query) @ w_ukT[h].T = the query against the latent
    assert tuple(a["w_ukT"].shape) == (3, 16, 8) and torch.equal(a["w_ukT"][1], S["l0.mix.uk"][8:16].T)
    q, lat = torch.randn(8, dtype=torch.float64), torch.randn(16, dtype=torch.float64)
    assert torch.allclose((a["w_ukT"][2].double() @ q) @ lat, q @ (S["l0.mix.uk"][16:24].double() @ lat))
    assert tuple(a["moe"]["w_gate_up"].shape) == (5, 24, 24) and torch.equal(a["moe"]["w_gate_up"][2, 12:], S["l0.mlp.e2.up"])
    assert tuple(a["moe"]["w_down"].shape) == (5, 24, 12) and tuple(a["moe"]["shared_gate_up"].shape) == (20, 24)
    assert tuple(r["w_in"].shape) == (96, 24) and torch.equal(r["w_in"][18:36], S["l1.mix.k"]) and torch.equal(r["w_in"][66:], S["l1.mix.g"])
    assert tuple(r["w_up"].shape) == (28, 24) and torch.equal(r["b_up"][14:], S["l1.mlp.up.b"].float()) and torch.equal(r["b_down"], S["l1.mlp.down.b"])
    assert "moe" not in b and "w_up" not in b


def test_synthetic_weights_fit_the_reader():
    from vox_serve_amd.model.dipivik import config_from_dict, pack_weights, synth_weights
    c = config_from_dict(small())
    S = synth_weights(c)
    assert set(S) == set(D.random_checkpoint(small()))
    assert len(pack_weights(S, c)["layers"]) == 3


def test_registry_names_the_design():
    from vox_serve_amd.model import MODEL_REGISTRY, get_model_class
    assert "dipivik" in MODEL_REGISTRY and get_model_class("Dipivik") is MODEL_REGISTRY["dipivik"]


def test_oracle_is_causal_and_deterministic():
    cfg = small()
    S = D.random_checkpoint(cfg, seed=5)
    toks = tokens(30, 40, 6)
    full = DR.forward(cfg, S, toks)
    assert torch.allclose(DR.forward(cfg, S, toks[:17]), full[:17], atol=1e-12)
    other = list(toks)
    other[20] = (other[20] + 1) % 40
    assert torch.allclose(DR.forward(cfg, S, other)[:20], full[:20], atol=1e-12)
    assert not torch.allclose(DR.forward(cfg, S, other)[20:], full[20:], atol=1e-6)
    assert float(full.abs().max()) < 5.0                      # the cap


def test_oracle_bigram_rows():
    S = {"embed": torch.zeros(40, 4, dtype=torch.float64), "bigram": torch.arange(54, dtype=torch.float64)[:, None].expand(54, 4).contiguous()}
    x = DR.embed_tokens(S, [3, 9, 9, 39], {"buckets": 53, "mul_prev": 7, "mul_cur": 3})
    assert x[:, 0].tolist() == [53.0, float((3 * 7 + 9 * 3) % 53), float((9 * 7 + 9 * 3) % 53), float((9 * 7 + 39 * 3) % 53)]


def test_first_token_row_sensitivity():
    """The first token takes the bigram table's extra row: with another row there the oracle's own logits move by far more than the
    bar; a portion that forgot its predecessor would embed its first token differently and all others alike."""
    cfg = small()
    S = D.random_checkpoint(cfg, seed=13)
    toks = tokens(12, 40, 20)
    base = DR.forward(cfg, S, toks)
    other = dict(S, bigram=torch.cat([S["bigram"][:-1], S["bigram"][:1]], 0))
    assert rel_err(DR.forward(cfg, other, toks)[:1], base[:1]) > 50 * F32_BAR
    Sd = {k: v.double() for k, v in S.items()}
    lost = DR.embed_tokens(Sd, toks[6:], cfg["embedding"]["bigram"])
    kept = DR.embed_tokens(Sd, toks, cfg["embedding"]["bigram"])[6:]
    assert (lost[0] - kept[0]).abs().max() > 0.1 and torch.equal(lost[1:], kept[1:])


def test_window_edge_sensitivity():
    """A window one token too long or too short moves the oracle's own logits by far more than the bar."""
    cfg = D.config([D.latent(heads=2, dim=16, rot_dim=4, vdim=16, q_rank=12, kv_rank=24, window=12, scale=1.0)], width=16, vocab=32)
    S = D.random_checkpoint(cfg, seed=31, qk_gain=3.0)
    toks = tokens(80, 32, 34)
    base = DR.forward(cfg, S, toks)
    for delta in (-1, 1):
        off = copy.deepcopy(cfg)
        off["layers"][0]["mixer"]["mask"]["size"] += delta
        assert rel_err(DR.forward(off, S, toks), base) > 50 * F32_BAR


def test_oracle_window_and_latent_expansion():
    """The attention equals a direct evaluation with explicit keys [uk c | k_rot] and a banded mask."""
    cfg = D.config([D.latent(heads=2, dim=6, rot_dim=4, vdim=5, q_rank=7, kv_rank=9, window=4)], width=12)
    S = D.random_checkpoint(cfg, seed=15)
    m, eps = cfg["layers"][0]["mixer"], 1e-5
    P = {k[len("l0.mix."):]: v.double() for k, v in S.items() if k.startswith("l0.mix.")}
    n = torch.randn(11, 12, dtype=torch.float64, generator=torch.Generator().manual_seed(16))
    got = DR.latent_attention(P, n, m, eps)
    q = (DR.rms_norm(n @ P["dq"].T, P["dq.norm"], eps) @ P["uq"].T).view(11, 2, 10)
    kv = n @ P["dkv"].T
    c = DR.rms_norm(kv[:, :9], P["dkv.norm"], eps)
    kr = DR.rotate_half(kv[:, 9:], 4, 100.0)
    out = torch.zeros(11, 2, 5, dtype=torch.float64)
    for h in range(2):
        qh = torch.cat([q[:, h, :6], DR.rotate_half(q[:, h, 6:], 4, 100.0)], -1)
        kh = torch.cat([c @ P["uk"][h * 6:(h + 1) * 6].T, kr], -1)
        sc = qh @ kh.T * m["scale"]
        i, j = torch.arange(11)[:, None], torch.arange(11)[None, :]
        sc = sc.masked_fill((j > i) | (i - j >= 4), -math.inf)
        out[:, h] = torch.softmax(sc, -1) @ (c @ P["uv"][h * 5:(h + 1) * 5].T)
    want = (out * torch.sigmoid(n @ P["g"].T)[:, :, None]).reshape(11, 10) @ P["o"].T
    assert torch.allclose(got, want, atol=1e-12)


def test_oracle_retention_closed_form():
    """o_t = sum_j decay^(t-j) (q_t . k_j) v_j with rotated q, k and k / sqrt(d)."""
    cfg = D.config([D.retention(heads=2, dim=6, vdim=4, rot=4, decay=[0.9, 0.5])], width=10)
    S = D.random_checkpoint(cfg, seed=17)
    m, eps = cfg["layers"][0]["mixer"], 1e-5
    P = {k[len("l0.mix."):]: v.double() for k, v in S.items() if k.startswith("l0.mix.")}
    n = torch.randn(9, 10, dtype=torch.float64, generator=torch.Generator().manual_seed(18))
    got = DR.retention(P, n, m, eps)
    q = DR.rotate_half((n @ P["q"].T).view(9, 2, 6), 4, 50.0)
    k = DR.rotate_half((n @ P["k"].T).view(9, 2, 6), 4, 50.0) / math.sqrt(6)
    v = (n @ P["v"].T).view(9, 2, 4)
    o = torch.zeros(9, 2, 4, dtype=torch.float64)
    for t in range(9):
        for j in range(t + 1):
            for h, a in enumerate(m["decay"]):
                o[t, h] += a ** (t - j) * (q[t, h] @ k[j, h]) * v[j, h]
    want = (DR.rms_norm(o, None, eps).reshape(9, 8) * DR.silu(n @ P["g"].T)) @ P["o"].T
    assert torch.allclose(got, want, atol=1e-12)


def test_retention_sensitivity():
    """A decay applied twice or a rotation left out move the oracle's logits by far more than the bar; turning q and k by the same
    extra angle changes nothing (only differences of positions count)."""
    cfg = D.config([D.retention(heads=2, dim=8, vdim=8, rot=8, decay=[0.9, 0.6])], width=16, vocab=32)
    S = D.random_checkpoint(cfg, seed=41, qk_gain=2.0)
    toks = tokens(40, 32, 42)
    base = DR.forward(cfg, S, toks)
    other = copy.deepcopy(cfg)
    other["layers"][0]["mixer"]["decay"] = [0.81, 0.36]
    assert rel_err(DR.forward(other, S, toks), base) > 50 * F32_BAR
    real = DR.rotate_half
    try:
        DR.rotate_half = lambda v, dims, base_, first_pos=0: real(v, dims, base_, first_pos + 1)
        assert rel_err(DR.forward(cfg, S, toks), base) < 1e-9
    finally:
        DR.rotate_half = real
    no_rot = copy.deepcopy(cfg)
    del no_rot["layers"][0]["mixer"]["rot"]
    assert rel_err(DR.forward(no_rot, S, toks), base) > 50 * F32_BAR


def test_oracle_routing_weights():
    g = torch.Generator().manual_seed(7)
    n = torch.randn(50, 8, generator=g, dtype=torch.float64)
    P = {"router": torch.randn(6, 8, generator=g, dtype=torch.float64)}
    chosen, w = DR.route(P, n, 2)
    s = torch.sigmoid(n @ P["router"].T)
    assert torch.equal(chosen, s.topk(2, -1).indices) and torch.allclose(w, torch.gather(s, 1, chosen))
    assert (w.sum(-1) - 1).abs().max() > 0.2                      # not renormalised


def test_bigram_multipliers_are_reduced_on_the_host():
    """(prev * a + cur * b) mod n = (prev * (a mod n) + cur * (b mod n)) mod n: what the engine is given always fits 32 bits."""
    from vox_serve_amd.engine_hybrid import reduced_bigram
    assert reduced_bigram((53, 7, 3)) == (53, 7, 3)
    n, a, b = reduced_bigram((5, 100003, 2 ** 40 + 1))
    assert (n, a, b) == (5, 100003 % 5, (2 ** 40 + 1) % 5)
    for prev, cur in ((0, 0), (39, 17), (123456, 654321)):
        assert (prev * 100003 + cur * (2 ** 40 + 1)) % 5 == (prev * a + cur * b) % 5
    assert reduced_bigram(None) == (0, 0, 0)
