"""Small Sizitar configurations and random checkpoints for the tests (the checkpoint's config.json layout and tensor names)."""
import math

import torch


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=12, shared=10):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def delta(heads=2, kv_heads=1, dim=8, vdim=12, conv=3, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def channel_delta(heads=2, kv_heads=2, dim=8, vdim=12, conv=4, decay_rank=5, gate_rank=6, mlp=None):
    """decay_rank / gate_rank are no config keys: they are the shapes of a1 / g1 in the checkpoint (random_checkpoint reads them here)."""
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp, "_ranks": (decay_rank, gate_rank)}


def attention(heads=4, kv_heads=2, dim=8, vdim=6, conv=2, rot=4, base=100.0, scale=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if rot:
        m["rot"] = {"base": base, "dims": rot}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def config(layers, width=24, vocab=40, eps=1e-5, loop=None, logit_scale=0.7):
    c = {"architecture": "Sizitar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if logit_scale is not None:
        c["logit_scale"] = logit_scale
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def public(cfg):
    """The config as a checkpoint folder holds it (without the helpers' private keys)."""
    c = dict(cfg)
    c["layers"] = [{k: v for k, v in L.items() if not k.startswith("_")} for L in cfg["layers"]]
    return c


def random_checkpoint(cfg, seed=0, gain=1.0, qk_gain=1.0):
    """bf16 tensors under the checkpoint's names.  gain sharpens every projection; qk_gain the query and key projections only."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * (s * gain / math.sqrt(shape[-1]))).to(torch.bfloat16)

    def vec(n, mean=0.0, std=0.2):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)
    S = {"embed": (torch.randn(cfg["vocab"], W, generator=g) * 0.7).to(torch.bfloat16), "head": mat(cfg["vocab"], W), "final.norm": vec(W, 0.0, 0.3)}
    for i, L in enumerate(cfg["layers"]):
        m, p, q = L["mixer"], f"l{i}.mix.", f"l{i}.mlp."
        H, G, d, e, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        S[f"l{i}.norm1"], S[f"l{i}.ls1"] = vec(W, 0.0, 0.3), vec(W, 0.8, 0.3)
        if L["type"] == "attention":
            S.update({p + "q": mat(H * d, W, s=qk_gain), p + "k": mat(G * d, W, s=qk_gain), p + "v": mat(G * e, W), p + "q.norm": vec(H * d, 1.0, 0.3),
                      p + "k.norm": vec(G * d, 1.0, 0.3), p + "q.conv": mat(H * d, taps, s=1.5), p + "k.conv": mat(G * d, taps, s=1.5),
                      p + "v.conv": mat(G * e, taps, s=1.5), p + "o": mat(W, H * e)})
        else:
            S.update({p + "q": mat(G * d, W, s=qk_gain), p + "k": mat(G * d, W, s=qk_gain), p + "v": mat(H * e, W, s=2.0), p + "b": mat(H, W, s=2.0),
                      p + "q.conv": mat(G * d, taps, s=1.5), p + "k.conv": mat(G * d, taps, s=1.5), p + "v.conv": mat(H * e, taps, s=1.5),
                      p + "A_log": vec(H, -2.0, 1.0), p + "norm": vec(e, 1.0, 0.3), p + "o": mat(W, H * e)})
            if L["type"] == "channel_delta":
                ra, rg = L.get("_ranks", (5, 6))
                S.update({p + "a1": mat(ra, W), p + "a2": mat(H * d, ra, s=2.0), p + "dt_bias": vec(H * d, -1.0, 1.5), p + "g1": mat(rg, W),
                          p + "g2": mat(H * e, rg, s=2.0)})
            else:
                S.update({p + "a": mat(H, W, s=2.0), p + "dt_bias": vec(H, -1.0, 1.5), p + "g": mat(H * e, W, s=2.0)})
        mlp = L.get("mlp")
        if mlp is None:
            continue
        S[f"l{i}.norm2"], S[f"l{i}.ls2"] = vec(W, 0.0, 0.3), vec(W, 0.8, 0.3)
        if mlp["kind"] == "dense":
            f = mlp["ff"]
            S.update({q + "gate": mat(f, W, s=2.0), q + "up": mat(f, W, s=2.0), q + "down": mat(W, f)})
        else:
            f = mlp["expert"]["ff"]
            for j in range(mlp["router"]["experts"]):
                S.update({f"{q}e{j}.up": mat(f, W, s=2.0), f"{q}e{j}.down": mat(W, f)})
            S[q + "router"], S[q + "router.b"] = mat(mlp["router"]["experts"], W, s=3.0), vec(mlp["router"]["experts"], 0.0, 1.0)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                S.update({q + "shared.up": mat(sf, W, s=2.0), q + "shared.down": mat(W, sf)})
    return S
