"""Small Dipivik configurations and random checkpoints for the tests (the checkpoint's config.json layout and tensor names)."""
import math

import torch


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=12, shared=10):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def latent(heads=3, dim=8, rot_dim=4, vdim=12, q_rank=10, kv_rank=16, window=7, base=100.0, scale=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "rot": {"base": base, "dims": rot_dim}, "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim)}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def retention(heads=2, dim=8, vdim=12, rot=4, base=50.0, decay=None, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay) if decay else [1.0 - 2.0 ** -(3 + h) for h in range(heads)]}
    if rot:
        m["rot"] = {"base": base, "dims": rot}
    return {"type": "retention", "mixer": m, "mlp": mlp}


def config(layers, width=24, vocab=40, eps=1e-5, softcap=8.0, bigram=(53, 7, 3)):
    c = {"architecture": "Dipivik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if softcap:
        c["logit_softcap"] = softcap
    if bigram:
        c["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    return c


def random_checkpoint(cfg, seed=0, gain=1.0, qk_gain=1.0):
    """bf16 tensors under the checkpoint's names.  gain sharpens every projection; qk_gain the query and key projections only (scores
    that stand out)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * (s * gain / math.sqrt(shape[-1]))).to(torch.bfloat16)

    def vec(n, mean=0.0, std=0.2):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)
    S = {"embed": (torch.randn(cfg["vocab"], W, generator=g) * 0.7).to(torch.bfloat16), "final.norm": vec(W, 1.0)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        S["bigram"] = (torch.randn(bg["buckets"] + 1, W, generator=g) * 0.7).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        m, p, q = L["mixer"], f"l{i}.mix.", f"l{i}.mlp."
        S[f"l{i}.norm1"] = vec(W, 1.0)
        H, d, e = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "latent_attention":
            r, R, Q = m["rot_dim"], m["kv_rank"], m["q_rank"]
            S.update({p + "dq": mat(Q, W), p + "dq.norm": vec(Q, 1.0, 0.3), p + "uq": mat(H * (d + r), Q, s=qk_gain),
                      p + "dkv": mat(R + r, W, s=1.5), p + "dkv.norm": vec(R, 1.0, 0.3), p + "uk": mat(H * d, R, s=qk_gain),
                      p + "uv": mat(H * e, R), p + "g": mat(H, W, s=2.0), p + "o": mat(W, H * e)})
        else:
            S.update({p + "q": mat(H * d, W, s=qk_gain), p + "k": mat(H * d, W, s=qk_gain), p + "v": mat(H * e, W), p + "g": mat(H * e, W, s=2.0),
                      p + "o": mat(W, H * e)})
        mlp = L.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            f = mlp["ff"]
            S.update({q + "gate": mat(f, W, s=2.0), q + "gate.b": vec(f, 0.0, 0.5), q + "up": mat(f, W, s=2.0), q + "up.b": vec(f, 0.0, 0.5),
                      q + "down": mat(W, f), q + "down.b": vec(W, 0.0, 0.5)})
        else:
            f = mlp["expert"]["ff"]
            for j in range(mlp["router"]["experts"]):
                S.update({f"{q}e{j}.gate": mat(f, W, s=2.0), f"{q}e{j}.up": mat(f, W, s=2.0), f"{q}e{j}.down": mat(W, f)})
            S[q + "router"] = mat(mlp["router"]["experts"], W, s=3.0)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                S.update({q + "shared.gate": mat(sf, W, s=2.0), q + "shared.up": mat(sf, W, s=2.0), q + "shared.down": mat(W, sf)})
    return S
