"""Prefill and decode throughput of the Dipivik design (random weights) at layer sizes of a real model, beside the framework's
closest existing model, Fusanex (parallel blocks with routed feed-forwards on the same engine), at the same width and number of
layers.  bf16, one GPU; both are driven directly (plan upload + one native step).

    python tools/bench_dipivik.py [--sizes 1024,2048] [--prompt 512,2048] [--batch 1,8] [--steps 30] [--warmup 5]

Dipivik layers per block of four: retention (heads = width/128, 128 key and value dims, 64 rotated) with a gated dense feed-forward
of 3 x width | latent attention (heads = width/128 of 128 plain + 64 rotated dims, values of 128, query latent width/2, cached
latent width/4 + 64 rotated key dims, window 1024) with a routed feed-forward of 8 experts, 2 per token, expert width = width, and
a shared expert of width `width` | latent attention with the dense feed-forward | retention with the routed one.  Vocabulary 32 000,
bigram table of 65 521 buckets, tied head.  Prints one JSON object.
"""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from tools.bench_fusanex import fusanex_cfg
from tools.bench_fusanex import step_bytes as fusanex_step_bytes
from tools.bench_sirodra import bench_hybrid_cfg


def dipivik_cfg(width, blocks, vocab, experts=8, top=2, window=1024):
    from vox_serve_amd.engine_hybrid import HybridCfg, MixerCfg, MoECfg
    h = width // 128

    def moe():
        return dict(moe=MoECfg(experts=experts, identity=0, top=top, ff=width, limit=float("inf"), shared_ff=width, shared_limit=float("inf"),
                               act_alpha=1.0, score="sigmoid", renorm=False, scale_input=True, up_offset=0.0))

    def dense():
        return dict(ff=3 * width, ff_kind="gated", ff_act="gelu_tanh")

    def ret(ff):
        return MixerCfg("retention", h, 128, 128, rot_dims=64, rot_base=1e6, decay=[1.0 - 2.0 ** -(5 + i % 8) for i in range(h)],
                        block="parallel_one_norm", **ff)

    def lat(ff):
        return MixerCfg("latent_attention", h, 128, 128, q_rank=width // 2, kv_rank=width // 4, rot_dim=64, rot_dims=64, rot_base=5e4, window=window,
                        scale=192 ** -0.5, block="parallel_one_norm", **ff)
    layers = []
    for _ in range(blocks):
        layers += [ret(dense()), lat(moe()), lat(dense()), ret(moe())]
    return HybridCfg(width, vocab, 1e-5, layers, None, norm_kind="rms_groups", norm_groups=1, logit_softcap=30.0, bigram=(65521, 127, 17))


def step_bytes(cfg):
    """bf16 weight bytes a one-row decode step streams: all mixers, the chosen experts, the shared expert, router (fp32), head."""
    W = cfg.width
    n = cfg.vocab * W
    for m in cfg.layers:
        n += m.n_in * W + W * m.heads * m.vdim
        if m.kind == "latent_attention":
            n += m.heads * ((m.dim + m.rot_dim) * m.q_rank + m.kv_rank * m.dim + m.vdim * m.kv_rank)
        e = m.moe
        n += 3 * m.ff * W if e is None else 3 * e.top * e.ff * W + 3 * e.shared_ff * W + 2 * e.experts * W
    return 2 * n


def run(sizes=(1024, 2048), prompts=(512, 2048), batches=(1, 8), blocks=3, vocab=32000, ctx=1024, steps=30, warmup=5, device="cuda:0", only=None):
    from vox_serve_amd.model import dipivik, fusanex
    res = {"workload": "Dipivik layer pattern (retention + gated dense FF | latent attention + routed FF | latent attention + dense | retention + "
                       "routed) x %d blocks vs the Fusanex pattern of the same depth, bf16, random weights, decode context %d" % (blocks, ctx),
           "sizes": {}}
    for W in sizes:
        ent = {}
        if only in (None, "dipivik"):
            cfg = dipivik_cfg(W, blocks, vocab)
            packed = dipivik.pack_weights(dipivik.synth_weights(cfg), cfg)
            ent["dipivik"] = bench_hybrid_cfg(cfg, packed, step_bytes(cfg), prompts, batches, ctx, steps, warmup, device)
        if only in (None, "fusanex"):
            cfg = fusanex_cfg(W, (4 * blocks) // 3, vocab)
            packed = fusanex.pack_weights(fusanex.synth_weights(cfg, lora=64), cfg)
            ent["fusanex"] = bench_hybrid_cfg(cfg, packed, fusanex_step_bytes(cfg, 64), prompts, batches, ctx, steps, warmup, device)
        res["sizes"][str(W)] = ent
    return res


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", default="1024,2048")
    ap.add_argument("--prompt", default="512,2048")
    ap.add_argument("--batch", default="1,8")
    ap.add_argument("--blocks", type=int, default=3)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", default=None, choices=[None, "dipivik", "fusanex"])
    a = ap.parse_args()
    ints = lambda s: tuple(int(x) for x in s.split(","))
    print(json.dumps(run(ints(a.sizes), ints(a.prompt), ints(a.batch), a.blocks, steps=a.steps, warmup=a.warmup, only=a.only)))
