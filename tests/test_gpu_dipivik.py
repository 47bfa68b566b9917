"""Dipivik on the hybrid engine (registry -> DipivikModel -> ModelWorker -> vox_hybrid_*) against the float64 restatement in
oracle/dipivik_ref.py, on small configurations with random checkpoints made here.

fp32 engine: logits within 2e-4 of the oracle (relative RMS over the vocabulary); bf16 engine: 4e-2.  A schedule may change
rounding only, so every schedule of the same tokens is held to the same bar against the same whole-sequence oracle.  Attention
cases sharpen the query / key expansions (a nearly one-hot softmax), so a key that is wrongly seen or lost moves the logits by far
more than the bar; the sensitivity tests check such claims on the oracle itself.
"""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import dipivik_ref as DR
from tests import dipivik_util as D
from tests import hybrid_util as U

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

F32_BAR, BF16_BAR = 2e-4, 4e-2


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def check(cfg, S, toks, cuts, dtype=torch.float32, bar=None, quantile=None, **kw):
    want = DR.forward(cfg, S, toks)
    d = U.Driver(cfg, S, dtype=dtype, **kw)
    try:
        got = d.run_cut("r", toks, cuts)
    finally:
        d.close()
    err = U.rel_err(got, want, quantile)
    assert err < (bar or (F32_BAR if dtype == torch.float32 else BF16_BAR)), err
    return got


MECHANISMS = {
    "latent_attention": [D.latent()],
    "latent_window_of_one": [D.latent(window=1)],
    "latent_no_window": [D.latent(window=0, heads=2)],
    "latent_one_head_wide_latent": [D.latent(heads=1, dim=6, rot_dim=2, vdim=5, q_rank=3, kv_rank=70, window=4)],
    "latent_seventeen_heads": [D.latent(heads=17, dim=4, rot_dim=2, vdim=3, kv_rank=8, window=9)],
    "latent_eighteen_heads_no_rotation": [D.latent(heads=18, dim=4, rot_dim=0, vdim=4, kv_rank=12, window=5)],
    "retention": [D.retention()],
    "retention_no_rotation_one_head": [D.retention(heads=1, dim=10, vdim=7, rot=0, decay=[0.97])],
    "retention_full_rotation": [D.retention(heads=3, dim=6, vdim=6, rot=6, decay=[0.5, 0.9, 0.999])],
    "retention_wide_heads": [D.retention(heads=2, dim=40, vdim=70, rot=16, decay=[0.99, 0.9])],
    "dense_ff": [D.retention(mlp=D.dense())],
    "moe": [D.retention(mlp=D.moe())],
    "moe_top1_no_shared": [D.latent(mlp=D.moe(experts=3, top=1, shared=None))],
    "moe_top3_of_4": [D.latent(mlp=D.moe(experts=4, top=3, ff=20, shared=6))],
    "moe_all_experts_chosen": [D.retention(mlp=D.moe(experts=2, top=2, ff=9, shared=None))],
}


@pytest.mark.parametrize("name", list(MECHANISMS))
def test_mechanism_alone_whole_prompt(name):
    cfg = D.config(MECHANISMS[name])
    S = D.random_checkpoint(cfg, seed=1, qk_gain=2.0)
    check(cfg, S, tokens(70, 40, 2), [70])


@pytest.mark.parametrize("name", list(MECHANISMS))
def test_mechanism_alone_token_by_token(name):
    cfg = D.config(MECHANISMS[name])
    S = D.random_checkpoint(cfg, seed=3, qk_gain=2.0)
    check(cfg, S, tokens(45, 40, 4), [])


@pytest.mark.parametrize("softcap,bigram", [(0.0, None), (2.5, (1, 1, 1)), (30.0, (997, 40, 41)), (1.0, (5, 100003, 99991))])
def test_embedding_and_head_options(softcap, bigram):
    """No bigram table and no cap; one bucket; more buckets than pairs; multipliers far beyond the bucket count."""
    cfg = D.config([D.latent(mlp=D.dense()), D.retention(mlp=D.moe())], softcap=softcap, bigram=bigram)
    S = D.random_checkpoint(cfg, seed=5)
    check(cfg, S, tokens(30, 40, 6), [22, 2])


def stack(sharp=True):
    g = 2.0 if sharp else 1.0
    layers = [D.retention(heads=3, dim=8, vdim=10, rot=8, decay=[0.9, 0.99, 0.99], mlp=D.moe(experts=6, top=2, ff=14, shared=9)),
              D.latent(heads=4, dim=6, rot_dim=6, vdim=5, q_rank=9, kv_rank=20, window=11, mlp=D.dense(18)),
              D.latent(heads=2, dim=12, rot_dim=2, vdim=16, q_rank=14, kv_rank=10, window=30, base=10000.0, mlp=D.moe(experts=3, top=1, ff=8, shared=None)),
              D.retention(heads=2, dim=12, vdim=6, rot=4, decay=[0.995, 0.75], mlp=None),
              D.latent(heads=5, dim=4, rot_dim=4, vdim=8, q_rank=6, kv_rank=12, window=3, mlp=D.moe(experts=4, top=3, ff=10, shared=12))]
    return D.config(layers, width=36, vocab=64, bigram=(61, 13, 29)), g


def stack_checkpoint(seed, sharp=True):
    cfg, g = stack(sharp)
    return cfg, D.random_checkpoint(cfg, seed=seed, qk_gain=g)


@pytest.mark.parametrize("order", [(0, 1, 2, 3, 4), (1, 2, 0, 3), (4, 3), (2, 1, 1, 0)])
def test_stack_in_other_orders(order):
    cfg, g = stack()
    cfg["layers"] = [copy.deepcopy(cfg["layers"][i]) for i in order]
    S = D.random_checkpoint(cfg, seed=7, qk_gain=g)
    check(cfg, S, tokens(90, 64, 8), [90])


@pytest.mark.parametrize("cuts", [[2, 2, 2, 2, 3, 5, 2, 30, 2, 17], [31, 2, 1, 1, 2, 40], [7] * 13, [64, 2, 2], [9, 12, 9, 30], [66, 3, 20]])
def test_portions(cuts):
    """Portions cut inside pages (8 tokens) and inside the windows (3, 11, 30), below and above the row counts at which the products and
    the routed feed-forward change form, and above the 64 rows from which the retention scan runs in chunks; the rest token by token."""
    cfg, S = stack_checkpoint(9)
    check(cfg, S, tokens(100, 64, 10), cuts)


def test_bf16_schedules():
    cfg, S = stack_checkpoint(11, sharp=False)
    toks = tokens(96, 64, 12)
    a = check(cfg, S, toks, [96], dtype=torch.bfloat16, quantile=0.95)
    b = check(cfg, S, toks, [5, 2, 40, 3], dtype=torch.bfloat16, quantile=0.95)
    # a routed choice that bf16 rounding flips changes a position by more than rounding in either schedule alike
    assert U.rel_err(a, b.double(), 0.9) < BF16_BAR


def test_first_tokens_and_single_token():
    cfg, S = stack_checkpoint(13)
    for n in (1, 2, 3):
        check(cfg, S, tokens(n, 64, 14 + n), [n])
    check(cfg, S, tokens(5, 64, 19), [1, 1, 3])


def run_plan(d, seqs, plan, skip=lambda k, step: False):
    got = {k: [] for k in seqs}
    done = {k: 0 for k in seqs}
    step = 0
    while any(done[k] < len(seqs[k]) for k in seqs):
        portions = []
        for k in seqs:
            if done[k] >= len(seqs[k]) or skip(k, step):
                continue
            n = plan[k].pop(0) if plan[k] else 1
            portions.append((k, seqs[k][done[k]:done[k] + n]))
            done[k] += len(portions[-1][1])
        if portions:
            for k, lg in d.feed(portions).items():
                got[k].append(lg)
        step += 1
    return {k: torch.cat(v, 0) for k, v in got.items()}


def test_mixed_batch_matches_each_alone():
    """Four unequal requests share steps (portions beside single tokens); every request's logits equal its oracle's."""
    cfg, S = stack_checkpoint(21)
    seqs = {"a": tokens(75, 64, 22), "b": tokens(33, 64, 23), "c": tokens(9, 64, 24), "d": tokens(50, 64, 25)}
    want = {k: DR.forward(cfg, S, v) for k, v in seqs.items()}
    plan = {"a": [20, 1, 1, 30, 2, 1, 1, 19], "b": [1, 1, 1, 10, 20], "c": [2, 2, 2, 2, 1], "d": [3, 40, 1, 1, 1, 1, 1, 1, 1]}
    d = U.Driver(cfg, S)
    try:
        # request c joins late, request b skips every third step
        got = run_plan(d, seqs, plan, skip=lambda k, step: (k == "c" and step < 2) or (k == "b" and step % 3 == 2))
        for k in seqs:
            assert U.rel_err(got[k], want[k]) < F32_BAR, k
    finally:
        d.close()


def test_long_step_shared_by_requests():
    """A step of more than 64 rows (the retention scan cuts every request's rows into chunks that run side by side, the routed
    feed-forward runs expert by expert) shared by a long portion, a short one, and single decoded tokens; then the long request goes on
    from the state the chunked form left."""
    cfg, S = stack_checkpoint(61)
    seqs = {"a": tokens(230, 64, 62), "b": tokens(40, 64, 63), "c": tokens(12, 64, 64)}
    want = {k: DR.forward(cfg, S, v) for k, v in seqs.items()}
    d = U.Driver(cfg, S, pages=64)
    try:
        got = {k: [] for k in seqs}
        steps = [[("c", 0, 10)], [("a", 0, 97), ("b", 0, 3), ("c", 10, 11)], [("a", 97, 98), ("b", 3, 40), ("c", 11, 12)], [("a", 98, 228)],
                 [("a", 228, 229)], [("a", 229, 230)]]
        for st in steps:
            out = d.feed([(k, seqs[k][lo:hi]) for k, lo, hi in st])
            for k, lg in out.items():
                got[k].append(lg)
        for k in seqs:
            assert U.rel_err(torch.cat(got[k], 0), want[k]) < F32_BAR, k
    finally:
        d.close()


def test_pages_and_slots_are_reused():
    """6 pages and 2 state slots serve six requests, two at a time: a stale latent, retention state or previous token of a slot's
    former owner must not leak into the next owner."""
    cfg, S = stack_checkpoint(27)
    d = U.Driver(cfg, S, pages=6, slots=2, page_size=8, max_batch=2)
    try:
        for rnd in range(3):
            x, y = tokens(24, 64, 28 + rnd), tokens(17, 64, 38 + rnd)
            gx = [d.feed([("x", x[:10])])["x"]]
            o = d.feed([("x", x[10:]), ("y", y[:16])])
            gx.append(o["x"])
            gy = [o["y"], d.feed([("y", y[16:])])["y"]]
            assert d.worker.empty_pages.qsize() == 0 and d.worker.empty_state_slots.qsize() == 0
            d.end("x"); d.end("y")
            assert d.worker.empty_pages.qsize() == 6 and d.worker.empty_state_slots.qsize() == 2
            assert U.rel_err(torch.cat(gx, 0), DR.forward(cfg, S, x)) < F32_BAR
            assert U.rel_err(torch.cat(gy, 0), DR.forward(cfg, S, y)) < F32_BAR
    finally:
        d.close()


# ---- windows, far keys, page borders ------------------------------------------------------------------------------------------------

def window_case(window, heads=2):
    """One latent-attention layer whose rotated query part is zero (scores hang on tokens, not on distances) with sharp plain parts."""
    cfg = D.config([D.latent(heads=heads, dim=16, rot_dim=4, vdim=16, q_rank=12, kv_rank=24, window=window, scale=1.0)], width=16, vocab=32,
                   bigram=None)
    S = D.random_checkpoint(cfg, seed=31, qk_gain=3.0)
    uq = S["l0.mix.uq"].view(heads, 20, 12).clone()
    uq[:, 16:] = 0
    S["l0.mix.uq"] = uq.view(heads * 20, 12)
    return cfg, S


def planted_pair(cfg, S):
    """(a, b): the token a whose query (head 0, plain part) prefers the key of token b over every other token's by the widest margin."""
    Sd = {k: v.double() for k, v in S.items()}
    m, eps = cfg["layers"][0]["mixer"], cfg["norm"]["eps"]
    n = DR.rms_norm(Sd["embed"], Sd["l0.norm1"], eps)
    q = (DR.rms_norm(n @ Sd["l0.mix.dq"].T, Sd["l0.mix.dq.norm"], eps) @ Sd["l0.mix.uq"].T).view(-1, m["heads"], m["dim"] + m["rot_dim"])[:, 0, :m["dim"]]
    c = DR.rms_norm((n @ Sd["l0.mix.dkv"].T)[:, :m["kv_rank"]], Sd["l0.mix.dkv.norm"], eps)
    k = (c @ Sd["l0.mix.uk"].T).view(-1, m["heads"], m["dim"])[:, 0]
    top2 = (q @ k.T).topk(2, dim=-1)
    a = int((top2.values[:, 0] - top2.values[:, 1]).argmax())
    return a, int(top2.indices[a, 0])


@pytest.mark.parametrize("window,page_size", [(40, 8), (64, 64), (65, 16), (130, 32)])
def test_planted_key_just_inside_and_just_outside_the_window(window, page_size):
    """A token whose key the queries at the end prefer to every other is planted once.  Just inside the window of the query at
    position p (p - window + 1) it decides the output, just outside (p - window) it must not be seen; checked in one prompt, with the
    query decoded alone, and with portions cut at the window's edge."""
    cfg, S = window_case(window)
    a, b = planted_pair(cfg, S)
    T = window + 90
    p = T - 1
    for where in (p - window + 1, p - window):
        toks = [t if t != b else (b + 1) % 32 for t in tokens(T, 32, 33)]
        toks[where] = b
        toks[-1] = a
        want = DR.forward(cfg, S, toks)
        hidden = list(toks)
        hidden[where] = (b + 1) % 32
        moved = U.rel_err(DR.forward(cfg, S, hidden)[-1:], want[-1:])
        assert (moved > 100 * F32_BAR) == (where == p - window + 1), (where, moved)      # inside: it matters; outside: invisible
        for cuts in ([T], [T - 1], [where, 1, 1], [where + 1, T - where - 2], [2, where - 1, window - 1]):
            d = U.Driver(cfg, S, page_size=page_size, pages=512 // page_size, max_rows=256)
            try:
                got = d.run_cut("r", toks, cuts)
            finally:
                d.close()
            assert U.rel_err(got, want) < F32_BAR, (where, cuts)


def test_far_keys_without_a_window():
    """No window: logits hang on single keys hundreds of tokens back (more than 256 keys: the few-row steps split them over blocks)."""
    cfg = D.config([D.latent(heads=2, dim=16, rot_dim=4, vdim=16, q_rank=12, kv_rank=24, window=0, scale=1.0)], width=16, vocab=32)
    S = D.random_checkpoint(cfg, seed=35, qk_gain=3.0)
    toks = tokens(300, 32, 36)
    check(cfg, S, toks, [300], max_rows=320)
    check(cfg, S, toks, [200], page_size=16, max_rows=320)
    check(cfg, S, toks, [3, 61, 2, 67, 2, 100], page_size=4, pages=128, max_rows=320)


@pytest.mark.parametrize("page_size", [4, 16, 64])
def test_keys_at_page_borders(page_size):
    cfg, S = window_case(page_size + 1)
    toks = tokens(2 * page_size + 3, 32, 37)
    # the prompt ends one before, at, and one after a page border; then decoding crosses the next border
    for first in (page_size - 1, page_size, page_size + 1):
        check(cfg, S, toks, [first], page_size=page_size, pages=16)


def test_retention_remembers_far_tokens():
    """A decay close to 1 keeps tokens hundreds of steps back in the state: an early token changed moves the last logits (oracle), and
    the engine follows the oracle through a prompt, a chunked prompt and long decoding."""
    cfg = D.config([D.retention(heads=2, dim=16, vdim=16, rot=8, decay=[0.9995, 0.999])], width=16, vocab=32)
    S = D.random_checkpoint(cfg, seed=39, qk_gain=2.0)
    toks = tokens(330, 32, 40)
    want = DR.forward(cfg, S, toks)
    early = list(toks)
    early[5] = (early[5] + 1) % 32
    assert U.rel_err(DR.forward(cfg, S, early)[-1:], want[-1:]) > 20 * F32_BAR
    check(cfg, S, toks, [330], max_rows=336)
    check(cfg, S, toks, [129, 70, 2, 65], max_rows=336)
    check(cfg, S, toks, [10], pages=48)                        # 320 tokens decoded one by one


def test_routing_is_not_degenerate():
    """Over the prompt every expert is chosen, the weights are the sigmoid scores themselves (they do not sum to one), and scaling the
    expert's output instead of its input would be seen."""
    cfg = D.config([D.retention(mlp=D.moe(experts=5, top=2, ff=12, shared=10))])
    S = D.random_checkpoint(cfg, seed=43)
    toks = tokens(120, 40, 44)
    Sd = {k: v.double() for k, v in S.items()}
    n = DR.rms_norm(DR.embed_tokens(Sd, toks, cfg["embedding"]["bigram"]), Sd["l0.norm1"], cfg["norm"]["eps"])
    P = {k[len("l0.mlp."):]: v for k, v in Sd.items() if k.startswith("l0.mlp.")}
    chosen, w = DR.route(P, n, 2)
    assert set(chosen.flatten().tolist()) == set(range(5))
    assert (w.sum(-1) - 1.0).abs().max() > 0.3 and float(w.min()) > 0.0 and float(w.max()) < 1.0
    out_scaled = torch.zeros_like(n)
    for t in range(n.shape[0]):
        for c, wt in zip(chosen[t].tolist(), w[t]):
            Pe = {k[len(f"e{c}."):]: v for k, v in P.items() if k.startswith(f"e{c}.")}
            out_scaled[t] += wt * DR.gated_unit(Pe, n[t:t + 1], DR.silu, False)[0]
    Ps = {k[len("shared."):]: v for k, v in P.items() if k.startswith("shared.")}
    full = DR.moe_ff(P, n, cfg["layers"][0]["mlp"])
    assert ((out_scaled + DR.gated_unit(Ps, n, DR.silu, False)) - full).abs().max() > 0.05
    check(cfg, S, toks, [50, 9, 2])


def test_long_decoding():
    cfg, S = stack_checkpoint(45)
    check(cfg, S, tokens(330, 64, 46), [10], pages=48)


def test_wide_sizes():
    """Sizes beyond one wave per head: 160 value columns and 96 key dims of a retention head, a latent of 200 values under 20 heads (two
    groups of ten), 130-wide experts, odd width and vocabulary."""
    layers = [D.retention(heads=2, dim=96, vdim=160, rot=40, decay=[0.99, 0.95], mlp=D.moe(experts=9, top=4, ff=100, shared=130)),
              D.latent(heads=20, dim=24, rot_dim=10, vdim=36, q_rank=50, kv_rank=200, window=33, mlp=D.dense(150))]
    cfg = D.config(layers, width=100, vocab=131, bigram=(211, 17, 5))
    S = D.random_checkpoint(cfg, seed=47)
    toks = tokens(80, 131, 48)
    check(cfg, S, toks, [37, 2, 30])
    check(cfg, S, toks, [80], dtype=torch.bfloat16, quantile=0.95)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matrix_core_sizes(dtype):
    """Sizes at which every product takes its matrix-core or 16-byte form (widths and inner sizes that are multiples of 32), with prompt
    portions of 130 / 9 / 2 / 33 rows and decoding: the row-tile, tile and per-expert gathered forms against the same oracle."""
    layers = [D.latent(heads=8, dim=32, rot_dim=32, vdim=64, q_rank=96, kv_rank=128, window=48, mlp=D.moe(experts=6, top=3, ff=96, shared=160)),
              D.retention(heads=4, dim=64, vdim=32, rot=32, decay=[0.9, 0.99, 0.999, 0.97], mlp=D.dense(256)),
              D.latent(heads=4, dim=64, rot_dim=32, vdim=32, q_rank=64, kv_rank=96, window=100, mlp=D.moe(experts=4, top=2, ff=128, shared=None)),
              D.retention(heads=6, dim=32, vdim=64, rot=32, decay=[0.98] * 6, mlp=D.moe(experts=5, top=1, ff=64, shared=96))]
    cfg = D.config(layers, width=384, vocab=500, bigram=(1009, 31, 7))
    S = D.random_checkpoint(cfg, seed=71)
    toks = tokens(190, 500, 72)
    q = None if dtype == torch.float32 else 0.95
    check(cfg, S, toks, [130, 9, 2, 33], dtype=dtype, quantile=q, page_size=64, pages=8, max_rows=192)
    check(cfg, S, toks, [190], dtype=dtype, quantile=q, page_size=64, pages=8, max_rows=192)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_odd_sizes(dtype):
    """Sizes that defeat every vector path: width 18, key dims 10 / 5 / 3, value dims 6 / 7, latents of 7, 5 and 3 values, rotated parts
    of 2 and 6 dims, a 37-entry vocabulary, expert widths 5 and 9."""
    layers = [D.latent(heads=3, dim=10, rot_dim=2, vdim=6, q_rank=7, kv_rank=5, window=6, mlp=D.moe(experts=3, top=2, ff=5, shared=7)),
              D.retention(heads=3, dim=5, vdim=7, rot=2, decay=[0.9, 0.8, 0.7], mlp=D.moe(experts=2, top=1, ff=9, shared=None)),
              D.latent(heads=2, dim=3, rot_dim=6, vdim=7, q_rank=5, kv_rank=3, window=13, mlp=D.dense(11)),
              D.retention(heads=1, dim=3, vdim=3, rot=0, decay=[0.93])]
    cfg = D.config(layers, width=18, vocab=37, bigram=(19, 3, 11))
    S = D.random_checkpoint(cfg, seed=51)
    toks = tokens(75, 37, 52)
    q = None if dtype == torch.float32 else 0.9
    check(cfg, S, toks, [75], dtype=dtype, quantile=q)
    check(cfg, S, toks, [9, 2, 33, 5], dtype=dtype, quantile=q)


@pytest.mark.parametrize("heads,kv_rank,rot_dim,window", [(5, 40, 8, 70), (20, 24, 0, 0), (16, 112, 16, 33), (3, 8, 8, 1), (2, 200, 136, 50),
                                                          (2, 272, 64, 90)])
def test_matrix_core_attention_against_the_few_row_form(heads, kv_rank, rot_dim, window):
    """bf16 engine, cached rows that are multiples of 16 bytes: steps of more than 32 rows take the matrix-core attention (row tiles of
    four, heads as the columns of every product; the last two cases have more than 320 key dims, the last more than 256 value columns:
    the kernel's larger register layouts).  Two requests whose lengths are no multiples of four share one long step; the same
    tokens in portions of at most 30 rows take the few-row form.  Both round the same operands, so they agree far more closely than
    either agrees with the float64 oracle (what is left are bf16 roundings that flip where the products are summed in another order); a sharp softmax makes a key that is wrongly masked show."""
    cfg = D.config([D.latent(heads=heads, dim=8, rot_dim=rot_dim, vdim=12, q_rank=16, kv_rank=kv_rank, window=window, scale=1.0, mlp=D.dense(16))],
                   width=32, vocab=48)
    S = D.random_checkpoint(cfg, seed=95, qk_gain=2.0)
    seqs = {"a": tokens(131, 48, 96), "b": tokens(46, 48, 97)}
    want = {k: DR.forward(cfg, S, v) for k, v in seqs.items()}
    d = U.Driver(cfg, S, dtype=torch.bfloat16, pages=64, max_rows=256)
    try:
        one = d.feed([("a", seqs["a"][:129]), ("b", seqs["b"][:45])])
        long_a = torch.cat([one["a"], d.feed([("a", seqs["a"][129:])])["a"]], 0)
        long_b = torch.cat([one["b"], d.feed([("b", seqs["b"][45:])])["b"]], 0)
        d.end("a"); d.end("b")
        few_a = d.run_cut("a", seqs["a"], [30, 30, 30, 30, 11])
        few_b = d.run_cut("b", seqs["b"], [30, 16])
    finally:
        d.close()
    assert U.rel_err(long_a, few_a.double()) < 6e-3 and U.rel_err(long_b, few_b.double()) < 6e-3
    assert U.rel_err(long_a, want["a"], 0.95) < BF16_BAR and U.rel_err(long_b, want["b"], 0.95) < BF16_BAR


# ---- through the framework's own entry points -----------------------------------------------------------------------------------------

def test_greedy_generation_through_the_scheduler():
    """Requests enter through the scheduler's transport, are prefilled in portions next to decoding requests and generate greedily
    (decode steps replay the captured graph, the previous token lives in the state slot); the ids equal the oracle's greedy
    continuation (fp32 engine)."""
    from vox_serve_amd.model import get_model_class
    from vox_serve_amd.model.dipivik import config_from_dict
    from vox_serve_amd.scheduler.base import Scheduler, encode_request
    from vox_serve_amd.worker.base import ModelWorker
    cfg, S = stack_checkpoint(53)
    n_new = 12
    model = get_model_class("dipivik")("dipivik-test", weights=S, config=config_from_dict(cfg), dtype=torch.float32, max_batch_size=4, page_size=8,
                                       max_num_pages=64, max_seq_len=512, max_prefill_tokens=64, state_slots=4, max_tokens=n_new)
    worker = ModelWorker(model=model, max_batch_size=4, max_num_pages=64, page_size=8, greedy=True, prefill_chunk_tokens=16)
    sched = Scheduler(worker, max_batch_size=4)
    prompts = {"p0": tokens(37, 64, 54), "p1": tokens(5, 64, 55), "p2": tokens(50, 64, 56)}
    try:
        for rid, p in prompts.items():
            sched.transport.requests.put(encode_request(rid, " ".join(map(str, p)), is_streaming=False))
        reqs = {}
        for _ in range(400):
            sched._step()
            for r in sched.active_requests:
                reqs[r.request_id] = r
            if not sched.active_requests and not sched.transport.pending():
                break
        assert set(reqs) == set(prompts)
        for rid, p in prompts.items():
            seq = list(p)
            for _ in range(n_new):
                seq.append(int(DR.forward(cfg, S, seq)[-1].argmax()))
            got = [int(t[0, 0]) for t in reqs[rid].lm_output_tokens]
            assert got == seq[len(p):], (rid, got, seq[len(p):])
        done = []
        while not sched.transport.results.empty():
            done.append(sched.transport.results.get())
        assert sum(b"|COMPLETION|" in m and json.loads(m.split(b"|", 2)[2])["status"] == "completed" for m in done) == 3
        assert worker.empty_pages.qsize() == 64 and worker.empty_state_slots.qsize() == 4
    finally:
        model.engine.close()


def test_top_k_sampling_and_async_scheduling():
    """Stochastic sampling goes through the library's sampler (every id is one of the oracle's five most likely continuations of the
    request's own prefix; the same seed repeats the ids), and the pipelined scheduler loop generates the greedy ids."""
    from vox_serve_amd.model import get_model_class
    from vox_serve_amd.model.dipivik import config_from_dict
    from vox_serve_amd.sampling import SamplingConfig
    from vox_serve_amd.scheduler.base import Scheduler, encode_request
    from vox_serve_amd.worker.base import ModelWorker
    cfg, S = stack_checkpoint(91, sharp=False)
    prompts = {"a": tokens(21, 64, 92), "b": tokens(9, 64, 93)}

    def generate(sampling, n_new, greedy, async_scheduling):
        model = get_model_class("dipivik")("dipivik-test", weights=S, config=config_from_dict(cfg), dtype=torch.float32, max_batch_size=2,
                                           page_size=8, max_num_pages=32, max_seq_len=256, max_prefill_tokens=64, state_slots=2,
                                           max_tokens=n_new, sampling=sampling)
        worker = ModelWorker(model=model, max_batch_size=2, max_num_pages=32, page_size=8, seed=7, greedy=greedy, prefill_chunk_tokens=16)
        sched = Scheduler(worker, max_batch_size=2, async_scheduling=async_scheduling)
        seen = {}
        orig = sched._prepare_requests

        def spy():
            orig()
            for r in sched.active_requests:
                seen[r.request_id] = r
        sched._prepare_requests = spy
        try:
            for rid, p in prompts.items():
                sched.transport.requests.put(encode_request(rid, " ".join(map(str, p)), is_streaming=False))
            sched.run_until_idle(max_steps=400)
            assert worker.empty_pages.qsize() == 32 and worker.empty_state_slots.qsize() == 2
            return {rid: [int(t[0, 0]) for t in seen[rid].lm_output_tokens][:n_new] for rid in prompts}
        finally:
            model.engine.close()
    first = generate(SamplingConfig(top_k=5, temperature=0.8, max_tokens=8), 8, False, False)
    for rid, p in prompts.items():
        assert len(first[rid]) == 8
        seq = list(p)
        for tok in first[rid]:
            top = DR.forward(cfg, S, seq)[-1].topk(5).indices.tolist()
            assert tok in top, (rid, tok, top)
            seq.append(tok)
    assert generate(SamplingConfig(top_k=5, temperature=0.8, max_tokens=8), 8, False, False) == first
    got = generate(None, 7, True, True)
    for rid, p in prompts.items():
        seq = list(p)
        for _ in range(7):
            seq.append(int(DR.forward(cfg, S, seq)[-1].argmax()))
        assert got[rid] == seq[len(p):], (rid, got[rid], seq[len(p):])


@pytest.mark.parametrize("dtype,bar", [("float32", 2e-4), ("bfloat16", 4e-2)])
def test_trace_replay_of_a_checkpoint_folder(tmp_path, dtype, bar):
    """bin/trace_run as a user runs it: config.json + model.safetensors in a folder (the registry picks the design by the config's
    architecture), a schedule of five requests in mixed steps over five pages and four slots, wanted places, requests that end and
    whose pages and slot the next one takes."""
    from safetensors.torch import save_file
    cfg, S = stack_checkpoint(81, sharp=False)
    cfg["vocab"] = 50
    S = D.random_checkpoint(cfg, seed=81)
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in S.items()}, str(model / "model.safetensors"))
    g = torch.Generator().manual_seed(82)
    seqs = {k: torch.randint(0, 50, (n,), generator=g).tolist() for k, n in (("a", 100), ("b", 70), ("c", 3), ("d", 90), ("e", 64))}
    want = {k: DR.forward(cfg, S, v) for k, v in seqs.items()}
    plan = [[("a", 60), ("c", 1)], [("a", 1), ("b", 30), ("c", 2)], [("a", 1), ("b", 40), ("d", 2)], [("a", 38), ("d", 1), ("e", 63)],
            [("d", 87), ("e", 1)]]
    at = {k: 0 for k in seqs}
    lines, asked = [], []
    for n, step in enumerate(plan):
        entries, end, rows = [], [], []
        for k, cnt in step:
            lo, hi = at[k], at[k] + cnt
            wanted = sorted({0, cnt - 1, cnt // 2})
            entries.append({"id": k, "tokens": seqs[k][lo:hi], "want": wanted})
            rows += [(k, lo + w) for w in wanted]
            at[k] = hi
            if hi == len(seqs[k]):
                end.append(k)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
        asked.append(rows)
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", str(5 * 64)], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done ")] == [f"done {n}" for n in range(len(plan))]
    worst = 0.0
    for n, rows in enumerate(asked):
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(len(rows), 50).copy())
        ref = torch.stack([want[k][i] for k, i in rows])
        worst = max(worst, U.rel_err(got, ref, None if dtype == "float32" else 0.95))
    assert worst < bar, worst
