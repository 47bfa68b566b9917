"""Sizitar: a decoder-only language model on the hybrid engine (`engine_hybrid.HybridEngine`).

A checkpoint is a folder with `config.json` and `model.safetensors`.  config.json:
  architecture "Sizitar"; vocab, width; norm.eps; logit_scale; loop = {start, stop, times} (layers start .. stop-1 run `times` times in
  a row over the same weights, every pass with its own cache and state);
  layers[i] = {type: "delta" | "channel_delta" | "attention", mixer: {...},
               mlp: null | {kind: "dense", ff} | {kind: "moe", router: {experts, top}, expert: {ff}, shared: {ff}}}.
Tensors (bf16, linear weights [out, in]): embed, head, final.norm, and per layer l<i>.norm1, l<i>.norm2, l<i>.ls1, l<i>.ls2,
l<i>.mix.*, l<i>.mlp.*.

Every layer is sequential and pre-normed with a layer scale: x += ls1 * mixer(norm1 x); x += ls2 * ff(norm2 x).  A norm divides by the
root mean square and multiplies by 1 + w (weights stored around zero).  Logits = head . norm(x) * logit_scale.  The mixers:
  delta          q, k (kv_heads x dim), v (heads x vdim): causal convolution over `conv` taps per channel, silu; q and k unit vectors per
                 head, q / sqrt(dim); beta = sigmoid(b h); decay g = exp(-exp(A_log) softplus(a h + dt_bias)) per head;
                 S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q; unit RMS per head, a weight shared by heads, times
                 silu(g h); output projection.
  channel_delta  the same rule with one decay per head and key channel from a bottleneck a2 (a1 h), and a sigmoid gate from a
                 bottleneck g2 (g1 h).
  attention      grouped-query causal softmax attention whose q, k, v pass a causal convolution (no activation) right behind their
                 projections; q and k RMS-normed over their whole projection with weights; the first rot.dims dims of every head rotated
                 (interleaved pairs, frequencies rot.base^(-2i/dims)); scores times `scale`; one added to the softmax denominator.
The dense feed-forward is down(silu(gate h) * up h).  The routed one adds a bias to the router logits, takes the `top` largest, weighs
them by the softmax over the chosen logits; experts and the always-on shared expert are down(relu(up h)^2).
The plugin fuses each mixer's projections into the engine's row order at load time.
"""
from typing import Dict

import torch

from ..engine_hybrid import HybridCfg, MixerCfg, MoECfg
from .hybrid_lm import HybridLM

ARCHITECTURE = "Sizitar"
NO_LIMIT = float("inf")         # the experts' units are not clamped


def _ff_from_dict(i: int, mlp) -> dict:
    """-> the MixerCfg fields of the layer's feed-forward."""
    if mlp is None:
        return {}
    kind = mlp.get("kind")
    if kind == "dense":
        return dict(ff=int(mlp["ff"]), ff_kind="gated", ff_act="swish")
    if kind != "moe":
        raise ValueError(f"layer {i}: feed-forward kind {kind!r} is not part of this design")
    r, sh = mlp["router"], mlp.get("shared")
    return dict(moe=MoECfg(experts=int(r["experts"]), identity=0, top=int(r["top"]), ff=int(mlp["expert"]["ff"]), limit=NO_LIMIT,
                           shared_ff=int(sh["ff"]) if sh else 0, shared_limit=NO_LIMIT, act_alpha=1.0, score="softmax", renorm=True,
                           scale_input=False, up_offset=0.0, expert_form="up_down", expert_act="relu2", router_bias=True))


def config_from_dict(d: dict) -> HybridCfg:
    if d.get("architecture") != ARCHITECTURE:
        raise ValueError(f"not a {ARCHITECTURE} config: architecture = {d.get('architecture')!r}")
    layers = []
    for i, l in enumerate(d["layers"]):
        t, m = l["type"], l["mixer"]
        common = dict(kv_heads=int(m["kv_heads"]), conv_taps=int(m["conv"]), layer_scale=True, **_ff_from_dict(i, l.get("mlp")))
        if int(m["heads"]) % int(m["kv_heads"]):
            raise ValueError(f"layer {i}: {m['kv_heads']} key heads do not divide {m['heads']} heads")
        if t == "attention":
            rot = m.get("rot") or {}
            layers.append(MixerCfg("causal_attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]), scale=float(m["scale"]),
                                   rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), qk_norm_whole=True, sink=True,
                                   **common))
        elif t == "delta":
            layers.append(MixerCfg("delta", int(m["heads"]), int(m["dim"]), int(m["vdim"]), gate_act="silu", **common))
        elif t == "channel_delta":
            # the bottleneck widths are shapes of the checkpoint: pack_weights fills them in
            layers.append(MixerCfg("delta", int(m["heads"]), int(m["dim"]), int(m["vdim"]), decay_channels=True, lora=-1, gate_rank=-1,
                                   gate_act="sigmoid", **common))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {t!r}")
    lp = d.get("loop")
    loop = None
    if lp and int(lp.get("times", 1)) != 1:
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not (0 <= loop[0] < loop[1] <= len(layers)) or loop[2] < 1:
            raise ValueError(f"loop {loop} over {len(layers)} layers")
    ls = d.get("logit_scale")
    return HybridCfg(int(d["width"]), int(d["vocab"]), float(d["norm"]["eps"]), layers, loop, norm_kind="rms_groups", norm_groups=1,
                     logit_scale=1.0 if ls is None else float(ls), norm_one_plus=True)


def pack_weights(S: Dict[str, torch.Tensor], cfg: HybridCfg) -> Dict:
    """Checkpoint tensors -> the engine's fused layout.  Sizes a config does not give (the bottlenecks) come from the shapes."""
    layers = []
    for i, m in enumerate(cfg.layers):
        p, q = f"l{i}.mix.", f"l{i}.mlp."
        lw = dict(norm1=S[f"l{i}.norm1"], norm2=S.get(f"l{i}.norm2"), ls1=S[f"l{i}.ls1"], ls2=S.get(f"l{i}.ls2"), w_out=S[p + "o"],
                  conv_w=torch.cat([S[p + n + ".conv"].float() for n in ("q", "k", "v")], 0).contiguous())
        if tuple(lw["conv_w"].shape)[1] != m.conv_taps:
            raise ValueError(f"layer {i}: convolution of {tuple(lw['conv_w'].shape)[1]} taps, config says {m.conv_taps}")
        if m.kind == "causal_attention":
            lw.update(w_in=torch.cat([S[p + "q"], S[p + "k"], S[p + "v"]], 0).contiguous(), q_norm=S[p + "q.norm"], k_norm=S[p + "k.norm"])
        elif m.decay_channels:
            m.lora, m.gate_rank = int(S[p + "a1"].shape[0]), int(S[p + "g1"].shape[0])
            lw.update(w_in=torch.cat([S[p + n] for n in ("q", "k", "v", "b", "a1", "g1")], 0).contiguous(), w_decay2=S[p + "a2"],
                      w_gate2=S[p + "g2"], a_log=S[p + "A_log"], dt_bias=S[p + "dt_bias"], head_norm=S[p + "norm"])
        else:
            lw.update(w_in=torch.cat([S[p + n] for n in ("q", "k", "v", "b", "a", "g")], 0).contiguous(), a_log=S[p + "A_log"],
                      dt_bias=S[p + "dt_bias"], head_norm=S[p + "norm"])
        if m.moe is not None:
            e = m.moe
            mw = dict(router=S[q + "router"], router_bias=S[q + "router.b"], correction=None)
            if e.experts:
                mw["w_gate_up"] = torch.stack([S[f"{q}e{j}.up"] for j in range(e.experts)]).contiguous()
                mw["w_down"] = torch.stack([S[f"{q}e{j}.down"] for j in range(e.experts)]).contiguous()
            if e.shared_ff:
                mw["shared_gate_up"], mw["shared_down"] = S[q + "shared.up"], S[q + "shared.down"]
            lw["moe"] = mw
        elif m.ff:
            lw.update(w_up=torch.cat([S[q + "gate"], S[q + "up"]], 0).contiguous(), w_down=S[q + "down"])
        layers.append(lw)
    return dict(embedding=S["embed"], head=S["head"], final_norm=S["final.norm"], loop_in=None, layers=layers)


def synth_weights(cfg: HybridCfg, seed: int = 0, decay_rank: int = 16, gate_rank: int = 16) -> Dict[str, torch.Tensor]:
    """Random checkpoint tensors (bf16, the checkpoint's names) for a config: benchmarks and tests."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.width

    def lin(*shape):
        return (torch.randn(*shape, generator=g) / shape[-1] ** 0.5).to(torch.bfloat16)

    def vec(n, mean=0.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)
    S = {"embed": (torch.randn(cfg.vocab, W, generator=g) * 0.5).to(torch.bfloat16), "head": lin(cfg.vocab, W), "final.norm": vec(W)}
    for i, m in enumerate(cfg.layers):
        p, q = f"l{i}.mix.", f"l{i}.mlp."
        H, G, d, e = m.heads, m.kv_heads, m.dim, m.vdim
        S.update({f"l{i}.norm1": vec(W), f"l{i}.ls1": vec(W, 0.5, 0.1)})
        if m.kind == "causal_attention":
            S.update({p + "q": lin(H * d, W), p + "k": lin(G * d, W), p + "v": lin(G * e, W), p + "q.norm": vec(H * d, 1.0), p + "k.norm": vec(G * d, 1.0),
                      p + "q.conv": lin(H * d, m.conv_taps), p + "k.conv": lin(G * d, m.conv_taps), p + "v.conv": lin(G * e, m.conv_taps)})
        else:
            S.update({p + "q": lin(G * d, W), p + "k": lin(G * d, W), p + "v": lin(H * e, W), p + "b": lin(H, W), p + "norm": vec(e, 1.0),
                      p + "q.conv": lin(G * d, m.conv_taps), p + "k.conv": lin(G * d, m.conv_taps), p + "v.conv": lin(H * e, m.conv_taps),
                      p + "A_log": vec(H, -1.0, 0.5)})
            if m.decay_channels:
                ra, rg = (m.lora if m.lora > 0 else decay_rank), (m.gate_rank if m.gate_rank > 0 else gate_rank)
                S.update({p + "a1": lin(ra, W), p + "a2": lin(H * d, ra), p + "dt_bias": vec(H * d, 0.0, 1.0), p + "g1": lin(rg, W), p + "g2": lin(H * e, rg)})
            else:
                S.update({p + "a": lin(H, W), p + "dt_bias": vec(H, 0.0, 1.0), p + "g": lin(H * e, W)})
        S[p + "o"] = lin(W, H * e)
        if m.moe is not None or m.ff:
            S.update({f"l{i}.norm2": vec(W), f"l{i}.ls2": vec(W, 0.5, 0.1)})
        if m.moe is not None:
            x = m.moe
            for j in range(x.experts):
                S.update({f"{q}e{j}.up": lin(x.ff, W), f"{q}e{j}.down": lin(W, x.ff)})
            S[q + "router"], S[q + "router.b"] = lin(x.experts, W), vec(x.experts, 0.0, 0.5)
            if x.shared_ff:
                S.update({q + "shared.up": lin(x.shared_ff, W), q + "shared.down": lin(W, x.shared_ff)})
        elif m.ff:
            S.update({q + "gate": lin(m.ff, W), q + "up": lin(m.ff, W), q + "down": lin(W, m.ff)})
    return S


class SizitarModel(HybridLM):
    """The text-only plugin of `hybrid_lm.HybridLM` with this design's config reader and weight packer."""

    default_name = "sizitar"
    config_from_dict = staticmethod(config_from_dict)
    pack_weights = staticmethod(pack_weights)
