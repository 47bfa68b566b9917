"""Dipivik: a decoder-only language model on the hybrid engine (`engine_hybrid.HybridEngine`).

A checkpoint is a folder with `config.json` and `model.safetensors`.  config.json:
  architecture "Dipivik"; vocab, width; norm.eps; logit_softcap; embedding.bigram = {buckets, mul_prev, mul_cur};
  layers[i] = {type: "latent_attention" | "retention", mixer: {...},
               mlp: null | {kind: "dense", ff} | {kind: "moe", router: {experts, top}, expert: {ff}, shared: {ff}}}.
Tensors (bf16, linear weights [out, in]): embed, bigram [buckets + 1, width], final.norm, and per layer l<i>.norm1, l<i>.mix.*,
l<i>.mlp.*.  There is no separate output matrix: logits = embed . norm(x), then cap * tanh(. / cap).

x0 = embed[token] + bigram[(previous token * mul_prev + token * mul_cur) mod buckets] (row `buckets` for a sequence's first token).
Every layer is parallel behind ONE RMS norm: n = norm1 x; x += mixer(n) + ff(n).  The mixers:
  latent_attention  query latent dq n (RMS norm, weight) expanded by uq to heads of [dim plain | rot_dim rotated]; dkv n = key / value
                    latent (kv_rank, RMS norm, weight: all the cache keeps) | one rotated key part of rot_dim shared by the heads; plain
                    keys uk latent and values uv latent per head; rotate-half rotary; window of mask.size tokens; softmax; a sigmoid gate
                    per head; output projection.
  retention         q, k (heads x dim, rotated on rot.dims, k then / sqrt(dim)), v, gate (heads x vdim); S <- decay_h S + k v^T, o = S^T q;
                    unit RMS per head, times silu(gate), output projection.
The feed-forward is a gated unit with biases down(gelu_tanh(gate n) * up n), or a mixture of experts: sigmoid router scores, the `top`
largest chosen, each chosen expert reads score * n (silu gated unit without biases), a shared expert reads n.
The plugin fuses each mixer's projections into the engine's row order at load time.
"""
from typing import Dict

import torch

from ..engine_hybrid import HybridCfg, MixerCfg, MoECfg
from .hybrid_lm import HybridLM

ARCHITECTURE = "Dipivik"
NO_LIMIT = float("inf")         # the experts' gated units are not clamped


def _ff_from_dict(i: int, mlp) -> dict:
    """-> the MixerCfg fields of the layer's feed-forward."""
    if mlp is None:
        return {}
    kind = mlp.get("kind")
    if kind == "dense":
        return dict(ff=int(mlp["ff"]), ff_kind="gated", ff_act="gelu_tanh")
    if kind != "moe":
        raise ValueError(f"layer {i}: feed-forward kind {kind!r} is not part of this design")
    r, sh = mlp["router"], mlp.get("shared")
    return dict(moe=MoECfg(experts=int(r["experts"]), identity=0, top=int(r["top"]), ff=int(mlp["expert"]["ff"]), limit=NO_LIMIT,
                           shared_ff=int(sh["ff"]) if sh else 0, shared_limit=NO_LIMIT, act_alpha=1.0, score="sigmoid", renorm=False,
                           scale_input=True, up_offset=0.0))


def config_from_dict(d: dict) -> HybridCfg:
    if d.get("architecture") != ARCHITECTURE:
        raise ValueError(f"not a {ARCHITECTURE} config: architecture = {d.get('architecture')!r}")
    layers = []
    for i, l in enumerate(d["layers"]):
        t, m = l["type"], l["mixer"]
        rot = m.get("rot") or {}
        common = dict(rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), block="parallel_one_norm",
                      **_ff_from_dict(i, l.get("mlp")))
        if t == "latent_attention":
            if common["rot_dims"] > int(m["rot_dim"]):
                raise ValueError(f"layer {i}: {common['rot_dims']} rotated dims in a part of {m['rot_dim']}")
            layers.append(MixerCfg("latent_attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]), q_rank=int(m["q_rank"]),
                                   kv_rank=int(m["kv_rank"]), rot_dim=int(m["rot_dim"]), window=int((m.get("mask") or {}).get("size", 0)),
                                   scale=float(m["scale"]), **common))
        elif t == "retention":
            decay = [float(a) for a in m["decay"]]
            if len(decay) != int(m["heads"]):
                raise ValueError(f"layer {i}: {len(decay)} decays for {m['heads']} heads")
            layers.append(MixerCfg("retention", int(m["heads"]), int(m["dim"]), int(m["vdim"]), decay=decay, **common))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {t!r}")
    bg = (d.get("embedding") or {}).get("bigram")
    return HybridCfg(int(d["width"]), int(d["vocab"]), float(d["norm"]["eps"]), layers, None, norm_kind="rms_groups", norm_groups=1,
                     logit_softcap=float(d.get("logit_softcap") or 0.0),
                     bigram=(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None)


def _cat_bias(S, names):
    return torch.cat([S[n].float() for n in names])


def pack_weights(S: Dict[str, torch.Tensor], cfg: HybridCfg) -> Dict:
    """Checkpoint tensors -> the engine's fused layout."""
    layers = []
    for i, m in enumerate(cfg.layers):
        p, q = f"l{i}.mix.", f"l{i}.mlp."
        lw = dict(norm1=S[f"l{i}.norm1"], w_out=S[p + "o"])
        if m.kind == "latent_attention":
            H, d, R = m.heads, m.dim, m.kv_rank
            assert tuple(S[p + "dkv"].shape)[0] == R + m.rot_dim and tuple(S[p + "uq"].shape) == (H * (d + m.rot_dim), m.q_rank), (i, "latent shapes")
            lw.update(w_in=torch.cat([S[p + "dq"], S[p + "dkv"], S[p + "g"]], 0).contiguous(), w_uq=S[p + "uq"],
                      # per head the transpose of its rows of uk: [H][R][d], so that (plain query) x (this) is the query against the latent
                      w_ukT=S[p + "uk"].view(H, d, R).transpose(1, 2).contiguous(), w_uv=S[p + "uv"],
                      q_lat_norm=S[p + "dq.norm"], kv_lat_norm=S[p + "dkv.norm"])
        else:
            lw.update(w_in=torch.cat([S[p + n] for n in ("q", "k", "v", "g")], 0).contiguous())
        if m.moe is not None:
            e = m.moe
            mw = dict(router=S[q + "router"], correction=None)
            if e.experts:
                mw["w_gate_up"] = torch.stack([torch.cat([S[f"{q}e{j}.gate"], S[f"{q}e{j}.up"]], 0) for j in range(e.experts)]).contiguous()
                mw["w_down"] = torch.stack([S[f"{q}e{j}.down"] for j in range(e.experts)]).contiguous()
            if e.shared_ff:
                mw["shared_gate_up"] = torch.cat([S[q + "shared.gate"], S[q + "shared.up"]], 0).contiguous()
                mw["shared_down"] = S[q + "shared.down"]
            lw["moe"] = mw
        elif m.ff:
            lw.update(w_up=torch.cat([S[q + "gate"], S[q + "up"]], 0).contiguous(), b_up=_cat_bias(S, (q + "gate.b", q + "up.b")),
                      w_down=S[q + "down"], b_down=S[q + "down.b"])
        layers.append(lw)
    emb = S["embed"]
    return dict(embedding=emb, head=emb, final_norm=S["final.norm"], loop_in=None, bigram=S.get("bigram"), layers=layers)


def synth_weights(cfg: HybridCfg, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random checkpoint tensors (bf16, the checkpoint's names) for a config: benchmarks."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.width

    def lin(*shape):
        return (torch.randn(*shape, generator=g) / shape[-1] ** 0.5).to(torch.bfloat16)

    def vec(n, mean=0.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)
    S = {"embed": (torch.randn(cfg.vocab, W, generator=g) * 0.5).to(torch.bfloat16), "final.norm": vec(W, 1.0)}
    if cfg.bigram:
        S["bigram"] = (torch.randn(cfg.bigram[0] + 1, W, generator=g) * 0.5).to(torch.bfloat16)
    for i, m in enumerate(cfg.layers):
        p, q = f"l{i}.mix.", f"l{i}.mlp."
        S[f"l{i}.norm1"] = vec(W, 1.0)
        H, d, e = m.heads, m.dim, m.vdim
        if m.kind == "latent_attention":
            S.update({p + "dq": lin(m.q_rank, W), p + "dq.norm": vec(m.q_rank, 1.0), p + "uq": lin(H * (d + m.rot_dim), m.q_rank),
                      p + "dkv": lin(m.kv_rank + m.rot_dim, W), p + "dkv.norm": vec(m.kv_rank, 1.0), p + "uk": lin(H * d, m.kv_rank),
                      p + "uv": lin(H * e, m.kv_rank), p + "g": lin(H, W), p + "o": lin(W, H * e)})
        else:
            S.update({p + "q": lin(H * d, W), p + "k": lin(H * d, W), p + "v": lin(H * e, W), p + "g": lin(H * e, W), p + "o": lin(W, H * e)})
        if m.moe is not None:
            x = m.moe
            for j in range(x.experts):
                S.update({f"{q}e{j}.gate": lin(x.ff, W), f"{q}e{j}.up": lin(x.ff, W), f"{q}e{j}.down": lin(W, x.ff)})
            S[q + "router"] = lin(x.experts, W)
            if x.shared_ff:
                S.update({q + "shared.gate": lin(x.shared_ff, W), q + "shared.up": lin(x.shared_ff, W), q + "shared.down": lin(W, x.shared_ff)})
        elif m.ff:
            S.update({q + "gate": lin(m.ff, W), q + "gate.b": vec(m.ff), q + "up": lin(m.ff, W), q + "up.b": vec(m.ff), q + "down": lin(W, m.ff),
                      q + "down.b": vec(W)})
    return S


class DipivikModel(HybridLM):
    """The text-only plugin of `hybrid_lm.HybridLM` with this design's config reader and weight packer."""

    default_name = "dipivik"
    config_from_dict = staticmethod(config_from_dict)
    pack_weights = staticmethod(pack_weights)
