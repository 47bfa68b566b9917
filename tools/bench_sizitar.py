"""Prefill and decode throughput of the Sizitar design (random weights) at layer sizes of a real model, beside the framework's
closest existing model, Fusanex (causal attention beside a matrix state with a decay per key channel, short convolutions, routed
feed-forwards on the same engine), at the same width and number of layers.  bf16, one GPU; both are driven directly (plan upload +
one native step).

    python tools/bench_sizitar.py [--sizes 1024,2048] [--prompt 512,2048] [--batch 1,8] [--steps 30] [--warmup 5]

Sizitar layers per block of three: channel-wise gated delta rule (heads = width/128 on half as many key heads, 128 key and value
dims, 4 taps, bottlenecks of 64) with a gated dense feed-forward of 3 x width | sink attention behind a 3-tap convolution (heads =
width/128 on a quarter as many key heads, 128 dims, 64 rotated) with a routed feed-forward of 8 relu-squared experts, 2 per token,
expert width = width, and a shared expert of width `width` | gated delta rule with one decay per head and the routed feed-forward.
The first two blocks run twice (a loop over shared weights).  Vocabulary 32 000.  Prints one JSON object.
"""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from tools.bench_fusanex import fusanex_cfg
from tools.bench_fusanex import step_bytes as fusanex_step_bytes
from tools.bench_sirodra import bench_hybrid_cfg

RANK = 64


def sizitar_cfg(width, blocks, vocab, experts=8, top=2, loop_blocks=2):
    from vox_serve_amd.engine_hybrid import HybridCfg, MixerCfg, MoECfg
    h = width // 128

    def moe():
        return dict(moe=MoECfg(experts=experts, identity=0, top=top, ff=width, limit=float("inf"), shared_ff=width, shared_limit=float("inf"),
                               act_alpha=1.0, score="softmax", renorm=True, scale_input=False, up_offset=0.0, expert_form="up_down",
                               expert_act="relu2", router_bias=True))

    def dense():
        return dict(ff=3 * width, ff_kind="gated", ff_act="swish")
    layers = []
    for _ in range(blocks):
        layers += [MixerCfg("delta", h, 128, 128, kv_heads=max(1, h // 2), conv_taps=4, decay_channels=True, lora=RANK, gate_rank=RANK,
                            gate_act="sigmoid", layer_scale=True, **dense()),
                   MixerCfg("causal_attention", h, 128, 128, kv_heads=max(1, h // 4), conv_taps=3, scale=128 ** -0.5, rot_dims=64, rot_base=1e4,
                            qk_norm_whole=True, sink=True, layer_scale=True, **moe()),
                   MixerCfg("delta", h, 128, 128, kv_heads=max(1, h // 2), conv_taps=4, gate_act="silu", layer_scale=True, **moe())]
    # the loop's second pass stands for a block of its own: (blocks - loop_blocks) blocks of weights run as `blocks` blocks
    n_own = blocks - loop_blocks
    return HybridCfg(width, vocab, 1e-5, layers[:3 * n_own], (0, 3 * loop_blocks, 2) if loop_blocks else None, norm_kind="rms_groups",
                     norm_groups=1, logit_scale=0.25, norm_one_plus=True)


def step_bytes(cfg):
    """bf16 weight bytes a one-row decode step streams: every run's mixer, its chosen experts and shared expert, router (fp32), head."""
    W = cfg.width
    n = cfg.vocab * W
    for i, _ in cfg.runs():
        m = cfg.layers[i]
        n += m.n_in * W + W * m.heads * m.vdim
        if m.kind == "delta":
            n += (m.heads * m.dim * m.lora if m.lora else 0) + (m.heads * m.vdim * m.gate_rank if m.gate_rank else 0)
        e = m.moe
        n += 3 * m.ff * W if e is None else 2 * e.top * e.ff * W + 2 * e.shared_ff * W + 2 * e.experts * W
    return 2 * n


def run(sizes=(1024, 2048), prompts=(512, 2048), batches=(1, 8), blocks=4, vocab=32000, ctx=1024, steps=30, warmup=5, device="cuda:0", only=None):
    from vox_serve_amd.model import fusanex, sizitar
    res = {"workload": "Sizitar layer pattern (channel-wise delta rule + gated dense FF | sink attention behind a convolution + routed FF | "
                       "delta rule + routed FF) x %d blocks, the first two through a loop, vs the Fusanex pattern of the same depth, bf16, "
                       "random weights, decode context %d" % (blocks, ctx), "sizes": {}}
    for W in sizes:
        ent = {}
        if only in (None, "sizitar"):
            cfg = sizitar_cfg(W, blocks, vocab)
            packed = sizitar.pack_weights(sizitar.synth_weights(cfg), cfg)
            ent["sizitar"] = bench_hybrid_cfg(cfg, packed, step_bytes(cfg), prompts, batches, ctx, steps, warmup, device)
        if only in (None, "fusanex"):
            cfg = fusanex_cfg(W, blocks, vocab)
            packed = fusanex.pack_weights(fusanex.synth_weights(cfg, lora=64), cfg)
            ent["fusanex"] = bench_hybrid_cfg(cfg, packed, fusanex_step_bytes(cfg, 64), prompts, batches, ctx, steps, warmup, device)
        res["sizes"][str(W)] = ent
    return res


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", default="1024,2048")
    ap.add_argument("--prompt", default="512,2048")
    ap.add_argument("--batch", default="1,8")
    ap.add_argument("--blocks", type=int, default=4)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", default=None, choices=[None, "sizitar", "fusanex"])
    a = ap.parse_args()
    ints = lambda s: tuple(int(x) for x in s.split(","))
    print(json.dumps(run(ints(a.sizes), ints(a.prompt), ints(a.batch), a.blocks, steps=a.steps, warmup=a.warmup, only=a.only)))
