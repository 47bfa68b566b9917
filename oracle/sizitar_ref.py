"""Float64 restatement of the Sizitar design, one function per mechanism, for the tests.  It shares no code with the engine: plain
loops over tokens and heads on the CPU, no cache, no state carried between calls (a whole sequence at a time).

Notation: n = a normed row, W_x = tensor `<prefix>x` ([out, in], applied as W n), T tokens, H heads, G key heads, d key dims, e value
dims.  Checkpoint layout: see vox_serve_amd/model/sizitar.py.
"""
import math

import torch

UNIT_EPS = 1e-6          # inside the root of the unit-vector norm of the delta rule's q and k


def silu(z):
    return z * torch.sigmoid(z)


def relu_squared(z):
    return torch.clamp(z, min=0.0) ** 2


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def zero_centred_norm(x, w, eps):
    """The residual stream's norm: weights are stored around zero."""
    return rms(x, eps) * (1.0 + w)


def short_convolution(u, w):
    """u [T, C], w [C, taps]: y[t] = sum_j w[:, j] * u[t - (taps - 1) + j], inputs before the sequence are zero."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def unit_vectors(x):
    """Every vector along the last axis divided by sqrt(sum of squares + 1e-6)."""
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + UNIT_EPS)


def delta_rule(q, k, v, beta, g):
    """q, k [T, H, d]; v [T, H, e]; beta [T, H]; g [T, H, d] (a decay per key channel; a per-head decay is the same value d times).
    S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q (read after the write).  -> o [T, H, e]"""
    T, H, d = q.shape
    e = v.shape[-1]
    out = torch.zeros(T, H, e, dtype=q.dtype)
    for h in range(H):
        S = torch.zeros(d, e, dtype=q.dtype)
        for t in range(T):
            S = g[t, h].unsqueeze(1) * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + torch.outer(k[t, h], u)
            out[t, h] = S.T @ q[t, h]
    return out


def delta_mixer(P, n, m, eps, channel):
    """P: the mixer's tensors by their short names.  channel: one decay per head and key channel through a bottleneck and a sigmoid gate
    through a bottleneck; else one decay per head and a silu gate."""
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = n.shape[0]
    q = silu(short_convolution(n @ P["q"].T, P["q.conv"])).view(T, G, d)
    k = silu(short_convolution(n @ P["k"].T, P["k.conv"])).view(T, G, d)
    v = silu(short_convolution(n @ P["v"].T, P["v.conv"])).view(T, H, e)
    q = unit_vectors(q) / math.sqrt(d)
    k = unit_vectors(k)
    share = H // G
    q = torch.stack([q[:, h // share] for h in range(H)], 1)
    k = torch.stack([k[:, h // share] for h in range(H)], 1)
    beta = torch.sigmoid(n @ P["b"].T)
    rate = torch.exp(P["A_log"])                                       # [H]
    if channel:
        step = softplus((n @ P["a1"].T) @ P["a2"].T + P["dt_bias"]).view(T, H, d)
        g = torch.exp(-rate.view(1, H, 1) * step)
        gate = torch.sigmoid((n @ P["g1"].T) @ P["g2"].T).view(T, H, e)
    else:
        step = softplus(n @ P["a"].T + P["dt_bias"])                   # [T, H]
        g = torch.exp(-rate * step).unsqueeze(-1).expand(T, H, d)
        gate = silu(n @ P["g"].T).view(T, H, e)
    o = delta_rule(q, k, v, beta, g)
    o = rms(o, eps) * P["norm"] * gate
    return o.reshape(T, H * e) @ P["o"].T


def rotate_pairs(x, positions, dims, base):
    """x [T, heads, d]: dims 2i and 2i+1 (i < dims/2) form a pair turned by the angle position * base^(-2i/dims)."""
    if not dims:
        return x
    y = x.clone()
    for i in range(dims // 2):
        ang = positions.to(x.dtype) * (base ** (-2.0 * i / dims))
        c, s = torch.cos(ang).unsqueeze(1), torch.sin(ang).unsqueeze(1)
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        y[..., 2 * i] = a * c - b * s
        y[..., 2 * i + 1] = b * c + a * s
    return y


def sink_softmax(scores):
    """exp(s_j) / (1 + sum_j exp(s_j)) over the last axis (-inf entries are masked keys)."""
    m = torch.clamp(scores.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(scores - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def attention_mixer(P, n, m, eps):
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = n.shape[0]
    q = short_convolution(n @ P["q"].T, P["q.conv"])
    k = short_convolution(n @ P["k"].T, P["k.conv"])
    v = short_convolution(n @ P["v"].T, P["v.conv"]).view(T, G, e)
    q = (rms(q, eps) * P["q.norm"]).view(T, H, d)                      # one norm over the whole projection, before the split
    k = (rms(k, eps) * P["k.norm"]).view(T, G, d)
    rot = m.get("rot") or {}
    pos = torch.arange(T)
    q = rotate_pairs(q, pos, int(rot.get("dims", 0)), float(rot.get("base", 10000.0)))
    k = rotate_pairs(k, pos, int(rot.get("dims", 0)), float(rot.get("base", 10000.0)))
    share = H // G
    out = torch.zeros(T, H, e, dtype=n.dtype)
    causal = torch.ones(T, T, dtype=torch.bool).tril()
    for h in range(H):
        s = (q[:, h] @ k[:, h // share].T) * m["scale"]
        s = s.masked_fill(~causal, float("-inf"))
        out[:, h] = sink_softmax(s) @ v[:, h // share]
    return out.reshape(T, H * e) @ P["o"].T


def dense_ff(P, n):
    return (silu(n @ P["gate"].T) * (n @ P["up"].T)) @ P["down"].T


def up_down_unit(P, n):
    return relu_squared(n @ P["up"].T) @ P["down"].T


def sub(P, prefix):
    return {k[len(prefix):]: v for k, v in P.items() if k.startswith(prefix)}


def route(P, n, top):
    """-> (chosen experts [T, top], weights [T, top]): the largest biased logits, softmax over the chosen logits only."""
    z = n @ P["router"].T + P["router.b"]
    best = z.topk(top, dim=-1)
    return best.indices, torch.softmax(best.values, -1)


def moe_ff(P, n, mlp):
    chosen, w = route(P, n, mlp["router"]["top"])
    out = torch.zeros_like(n)
    for t in range(n.shape[0]):
        for c, wt in zip(chosen[t].tolist(), w[t]):
            out[t] += wt * up_down_unit(sub(P, f"e{c}."), n[t:t + 1])[0]
    if mlp.get("shared"):
        out = out + up_down_unit(sub(P, "shared."), n)
    return out


def layer_order(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, t = lp["start"], lp["stop"], lp["times"]
    return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


def forward(cfg, S, tokens, trace=None):
    """-> logits [T, vocab] (float64) of one whole sequence.  trace: a list that receives the residual stream after every layer run."""
    S = {k: v.double() for k, v in S.items()}
    eps = cfg["norm"]["eps"]
    x = S["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i in layer_order(cfg):
        L = cfg["layers"][i]
        n = zero_centred_norm(x, S[f"l{i}.norm1"], eps)
        P = sub(S, f"l{i}.mix.")
        if L["type"] == "attention":
            y = attention_mixer(P, n, L["mixer"], eps)
        elif L["type"] in ("delta", "channel_delta"):
            y = delta_mixer(P, n, L["mixer"], eps, L["type"] == "channel_delta")
        else:
            raise ValueError(L["type"])
        x = x + S[f"l{i}.ls1"] * y
        mlp = L.get("mlp")
        if mlp:
            n = zero_centred_norm(x, S[f"l{i}.norm2"], eps)
            P = sub(S, f"l{i}.mlp.")
            x = x + S[f"l{i}.ls2"] * (dense_ff(P, n) if mlp["kind"] == "dense" else moe_ff(P, n, mlp))
        if trace is not None:
            trace.append(x.clone())
    ls = cfg.get("logit_scale")
    return (zero_centred_norm(x, S["final.norm"], eps) @ S["head"].T) * (1.0 if ls is None else ls)
