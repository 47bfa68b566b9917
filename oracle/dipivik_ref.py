"""Slow float64 restatement of the Dipivik decoder, one function per mechanism, whole sequences only.

Test infrastructure: nothing under vox_serve_amd/ imports this, and this imports nothing from there.  The model is a dict
config (the checkpoint's config.json layout) and a dict of tensors under the checkpoint's names.
Notation: T tokens, n [T, width] the normed layer input, H heads, d unrotated and r rotated query / key dims, e value dims,
R the width of the key / value latent.

The design: x_0 = embed[token] + bigram[hash(previous token, token)]; every layer adds mixer(n) + ff(n) to x with ONE RMS norm
n = norm1(x) read by both; the mixer is either softmax attention over a sliding window whose keys and values are expanded from
a cached low-rank latent (plus one rotated key part shared by all heads), or retention (a matrix state with one fixed decay per
head); the feed-forward is a gated dense unit with biases or a sigmoid-routed mixture of experts whose routing weight scales
the expert's input; logits come from the embedding table itself and are soft-capped by a tanh.
"""
import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def embed_tokens(S, tokens, bigram):
    """Row `token` of the table, plus (bigram given) row (prev * mul_prev + token * mul_cur) mod buckets of the bigram table; the first
    token of a sequence has no predecessor and takes the table's extra last row."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = S["embed"][ids]
    if bigram:
        B = int(bigram["buckets"])
        rows = [B] + [(int(tokens[t - 1]) * int(bigram["mul_prev"]) + int(tokens[t]) * int(bigram["mul_cur"])) % B for t in range(1, len(tokens))]
        x = x + S["bigram"][torch.as_tensor(rows, dtype=torch.long)]
    return x


def rotate_half(v, dims, base, first_pos=0):
    """v [T, ..., D]: dims i and i + dims/2 (i < dims/2) of the last axis form a pair turned by the angle p * base^(-2i/dims) at
    position p; dims at or beyond `dims` pass unchanged."""
    if not dims:
        return v
    T, half = v.shape[0], dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    ang = (torch.arange(T, dtype=F64) + first_pos)[:, None] * f
    shape = [T] + [1] * (v.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], -1)


def latent_attention(P, n, m, eps, cache_round=None):
    """Queries through a normed latent of q_rank values; keys and values from a normed latent of kv_rank values (the only per-token
    memory besides one rotated key part of rot_dim values that every head shares).  A query at position i sees j with
    0 <= i - j < mask.size; softmax; each head's output times sigmoid of its own gate logit; output projection."""
    T, H, d, r, e, R = n.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    cq = rms_norm(n @ P["dq"].T, P["dq.norm"], eps)
    q = (cq @ P["uq"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate_half(q[..., d:], rot.get("dims", 0), rot.get("base", 10000.0))
    kv = n @ P["dkv"].T
    c = rms_norm(kv[:, :R], P["dkv.norm"], eps)
    k_rot = rotate_half(kv[:, R:], rot.get("dims", 0), rot.get("base", 10000.0))
    if cache_round is not None:
        c, k_rot = cache_round(c), cache_round(k_rot)
    k_plain = (c @ P["uk"].T).view(T, H, d)
    v = (c @ P["uv"].T).view(T, H, e)
    gate = torch.sigmoid(n @ P["g"].T)
    window = (m.get("mask") or {}).get("size") or T
    out = torch.zeros(T, H, e, dtype=F64)
    for t in range(T):
        lo = max(0, t - window + 1)
        for h in range(H):
            s = (k_plain[lo:t + 1, h] @ q_plain[t, h] + k_rot[lo:t + 1] @ q_rot[t, h]) * m["scale"]
            out[t, h] = torch.softmax(s, 0) @ v[lo:t + 1, h]
    return (out * gate[:, :, None]).reshape(T, H * e) @ P["o"].T


def retention(P, n, m, eps):
    """S_t = decay_h S_{t-1} + k_t v_t^T, o_t = S_t^T q_t per head, no softmax and no denominator; q and k are rotated, k is then
    divided by sqrt(d); each head's o is divided by its RMS; the concatenation is gated by silu(Wg n) and projected."""
    T, H, d, e = n.shape[0], m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    q = rotate_half((n @ P["q"].T).view(T, H, d), rot.get("dims", 0), rot.get("base", 10000.0))
    k = rotate_half((n @ P["k"].T).view(T, H, d), rot.get("dims", 0), rot.get("base", 10000.0)) * d ** -0.5
    v = (n @ P["v"].T).view(T, H, e)
    decay = torch.tensor([float(a) for a in m["decay"]], dtype=F64)
    S = torch.zeros(H, d, e, dtype=F64)
    out = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append((S * q[t][:, :, None]).sum(1))
    o = rms_norm(torch.stack(out), None, eps).reshape(T, H * e)
    return (o * silu(n @ P["g"].T)) @ P["o"].T


def gated_unit(P, n, act, biased):
    g, u = n @ P["gate"].T, n @ P["up"].T
    if biased:
        g, u = g + P["gate.b"], u + P["up.b"]
    y = (act(g) * u) @ P["down"].T
    return y + P["down.b"] if biased else y


def dense_ff(P, n):
    return gated_unit(P, n, gelu_tanh, True)


def route(P, n, top):
    """-> (chosen [T, top], weights [T, top]): the `top` largest sigmoid scores; the weights are those scores as they are."""
    s = torch.sigmoid(n @ P["router"].T)
    w, chosen = torch.topk(s, top, dim=-1)
    return chosen, w


def moe_ff(P, n, mlp):
    """sum over the chosen experts of expert(weight * n) -- the weight scales what the expert reads -- plus a shared expert on n."""
    chosen, w = route(P, n, int(mlp["router"]["top"]))
    out = torch.zeros_like(n)
    for t in range(n.shape[0]):
        for c, wt in zip(chosen[t].tolist(), w[t]):
            Pe = {k[len(f"e{c}."):]: v for k, v in P.items() if k.startswith(f"e{c}.")}
            out[t] += gated_unit(Pe, wt * n[t:t + 1], silu, False)[0]
    if mlp.get("shared"):
        Ps = {k[len("shared."):]: v for k, v in P.items() if k.startswith("shared.")}
        out = out + gated_unit(Ps, n, silu, False)
    return out


def forward(cfg, S, tokens, residuals=None, cache_round=None):
    """tokens: list of ids -> logits [T, vocab] (float64).  S: checkpoint tensors (any float dtype)."""
    S = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in S.items()}
    eps = cfg["norm"]["eps"]
    x = embed_tokens(S, tokens, (cfg.get("embedding") or {}).get("bigram"))
    for i, L in enumerate(cfg["layers"]):
        P = {k[len(f"l{i}.mix."):]: v for k, v in S.items() if k.startswith(f"l{i}.mix.")}
        n = rms_norm(x, S[f"l{i}.norm1"], eps)
        if L["type"] == "latent_attention":
            add = latent_attention(P, n, L["mixer"], eps, cache_round)
        elif L["type"] == "retention":
            add = retention(P, n, L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        mlp = L.get("mlp")
        if mlp is not None:
            F = {k[len(f"l{i}.mlp."):]: v for k, v in S.items() if k.startswith(f"l{i}.mlp.")}
            add = add + (dense_ff(F, n) if mlp["kind"] == "dense" else moe_ff(F, n, mlp))
        x = x + add
        if residuals is not None:
            residuals.append(x.clone())
    z = rms_norm(x, S["final.norm"], eps) @ S["embed"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
