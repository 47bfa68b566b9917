"""Host side of `vox_hybrid_*`: the engine for decoders that mix tokens with linear recurrences (HGRN2, mLSTM, a real-gated
diagonal unit behind a short convolution, a matrix state with token shift and per-channel decay, retention with a fixed decay
per head, the gated delta rule behind short convolutions) and with attention over a paged cache (a sliding window with pooled
history, plain causal attention with normed q / k / v -- optionally behind a short convolution, rotated, with a softmax sink --, or
windowed attention whose keys and values are expanded from a cached low-rank latent), optionally two mixers side by
side, sequential or parallel layers with an optional layer scale, a dense or a routed feed-forward, and a range of layers looped over
shared weights.

It reuses the plan / stream / hipGraph machinery of the other LM engines (`Qwen3Engine`): one pinned int32 plan block per
step, decode steps captured per batch size.  Beyond the K / V pages that the worker hands out, every request holds one
recurrent-state slot (`state` in the plan); the engine owns the slot arrays, the worker owns the free list.

A step is ragged: `prefill(n_rows, n_req, ...)` takes prompt portions of any length next to single decoded tokens, `frame(batch,
...)` is the one-row-per-request special case whose inputs feed back on the device.
"""
import ctypes
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from . import _native as N
from .engine import Qwen3Engine

MIXER_HGRN2, MIXER_POOLED_WINDOW_ATTN, MIXER_MLSTM, MIXER_RGLRU, MIXER_CAUSAL_ATTN, MIXER_SHIFT_DECAY = 0, 1, 2, 3, 4, 5
MIXER_LATENT_ATTN, MIXER_RETENTION, MIXER_DELTA = 6, 7, 8
MIXER_KINDS = {"hgrn2": MIXER_HGRN2, "attention": MIXER_POOLED_WINDOW_ATTN, "mlstm": MIXER_MLSTM, "rglru": MIXER_RGLRU,
               "causal_attention": MIXER_CAUSAL_ATTN, "shift_decay": MIXER_SHIFT_DECAY, "latent_attention": MIXER_LATENT_ATTN,
               "retention": MIXER_RETENTION, "delta": MIXER_DELTA}
ATTENTION_KINDS = ("attention", "causal_attention", "latent_attention")
NORM_KINDS = {"layer": 0, "rms_groups": 1}
BLOCK_FORMS = {"sequential": 0, "parallel": 1, "parallel_one_norm": 2}
FF_KINDS = {"up_down": 0, "gated": 1}
ACT_KINDS = {"gelu_tanh": 0, "swish": 1, "relu2": 2}
ROUTER_SCORES = {"softmax": 0, "sigmoid": 1}
EXPERT_FORMS = {"gated": 0, "up_down": 1}
GATE_KINDS = {"none": 0, "sigmoid": 1, "silu": 2}


@dataclass
class MoECfg:
    """Routed feed-forward: `experts` clamped gated units + `identity` pass-through outputs, `top` per token, optional shared expert."""
    experts: int
    identity: int
    top: int
    ff: int
    limit: float
    shared_ff: int = 0
    shared_limit: float = 0.0
    act_alpha: float = 1.702
    score: str = "softmax"          # "softmax" over all router outputs | "sigmoid" of each
    renorm: bool = True             # weights divided by the sum of the chosen scores
    scale_input: bool = False       # the weight multiplies what the expert reads, not what it returns
    up_offset: float = 1.0          # y = g * sigmoid(act_alpha g) * (u + up_offset)
    expert_form: str = "gated"      # "gated" clamped gated units | "up_down" down(act(up h)): experts and the shared one
    expert_act: str = "swish"       # activation of the up_down form ("relu2" | "swish" with slope act_alpha)
    router_bias: bool = False       # a bias [experts + identity] is added to the router logits


@dataclass
class MixerCfg:
    kind: str                       # a key of MIXER_KINDS
    heads: int                      # rglru: blocks of the gate matrices
    dim: int                        # rglru: channels per block
    vdim: int                       # rglru, shift_decay: = dim
    kv_heads: int = 0               # attention
    window: int = 0                 # attention: tokens a position sees, itself included
    pool: int = 0                   # attention: tokens per pooled block
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_factor: float = 1.0         # linear position scaling: every rotary frequency is divided by it
    scale: float = 1.0              # attention score scale
    gate_cap: float = 0.0           # mLSTM: soft cap of the gate pre-activations
    ff: int = 0                     # dense feed-forward width (0: none)
    q_temp_coef: float = 0.0        # causal attention: q *= 1 + coef * ln(floor((p + 1) / every) + 1)
    q_temp_every: int = 1
    v_unit_rms: bool = False        # causal attention: values divided by their RMS per head before they are cached
    conv_taps: int = 0              # rglru: taps of the causal convolution
    rec_scale: float = 8.0          # rglru: a = exp(-rec_scale * r * softplus(lam))
    lora: int = 0                   # shift_decay: width of the decay bottleneck
    out_scale: float = 1.0          # the mixer's output is multiplied by this before it joins the residual sum
    block: str = "sequential"       # "sequential": x += mixer(norm1 x); x += ff(norm2 x) | "parallel": x += mixer(norm1 x) + ff(norm2 x)
                                    # | "parallel_one_norm": x += mixer(n) + ff(n), n = norm1 x
    ff_kind: str = "up_down"        # dense feed-forward: "up_down" down(gelu(up h)) | "gated" down(act(gate h + b) * (up h + b)) + b
    ff_act: str = "gelu_tanh"       # activation of the gated form ("gelu_tanh" | "swish")
    q_rank: int = 0                 # latent attention: width of the query latent
    kv_rank: int = 0                # latent attention: width of the cached key / value latent
    rot_dim: int = 0                # latent attention: rotated query / key dims per head (the key part is shared by all heads)
    decay: Optional[List[float]] = None     # retention: one decay per head
    layer_scale: bool = False       # the mixer's and the feed-forward's outputs are multiplied by a vector each (ls1, ls2)
    qk_norm_whole: bool = False     # causal attention behind a convolution: q / k RMS-normed over the whole projection
    sink: bool = False              # causal attention: one is added to the softmax denominator
    decay_channels: bool = False    # delta: one decay per head and key channel (else per head)
    gate_rank: int = 0              # delta: width of the gate bottleneck (0: one projection); `lora` is the decay bottleneck's
    gate_act: str = "silu"          # delta: activation of the output gate ("none" | "sigmoid" | "silu")
    side: Optional["MixerCfg"] = None   # a second mixer on the same normed input, added to the same sum
    moe: Optional[MoECfg] = None    # routed feed-forward (instead of the dense one)

    @property
    def n_in(self) -> int:
        """Rows of the fused input projection."""
        h, d, v = self.heads, self.dim, self.vdim
        if self.kind == "hgrn2":
            return 2 * h * d + h * v
        if self.kind == "attention":
            return h * d + self.kv_heads * (d + v) + h
        if self.kind == "rglru":
            return 2 * h * d
        if self.kind == "causal_attention":
            return h * d + self.kv_heads * (d + v)
        if self.kind == "delta":
            nd = h * d if self.decay_channels else h
            return 2 * self.kv_heads * d + h * v + h + (self.lora or nd) + (self.gate_rank or h * v)
        if self.kind == "shift_decay":
            return 4 * h * d + self.lora
        if self.kind == "latent_attention":
            return self.q_rank + self.kv_rank + self.rot_dim + h
        if self.kind == "retention":
            return 2 * h * d + 2 * h * v
        return 2 * h * d + 2 * h * v + 2 * h

    def cache_values(self) -> int:
        """Values one token leaves in the paged cache of an attention mixer."""
        if self.kind == "latent_attention":
            return self.kv_rank + self.rot_dim
        return self.kv_heads * (self.dim + self.vdim) if self.kind in ATTENTION_KINDS else 0

    def state_floats(self, width: int) -> int:
        """fp32 values of one recurrent-state slot (0 for attention)."""
        h, d, v = self.heads, self.dim, self.vdim
        if self.kind == "delta":
            return h * d * v + (self.conv_taps - 1) * (2 * self.kv_heads * d + h * v)
        if self.kind == "causal_attention":
            return max(self.conv_taps - 1, 0) * self.n_in         # the convolution's history (0: no state slot)
        return {"hgrn2": h * d * v, "mlstm": h * (d * v + d + 1), "rglru": max(self.conv_taps, 1) * h * d,
                "shift_decay": h * d * d + width, "retention": h * d * v}.get(self.kind, 0)


@dataclass
class HybridCfg:
    width: int
    vocab: int
    eps: float
    layers: List[MixerCfg] = field(default_factory=list)
    loop: Optional[tuple] = None    # (start, stop, times): layers start..stop-1 run `times` times in a row
    norm_kind: str = "layer"        # "layer": weight-only layer norm | "rms_groups": RMS norm over norm_groups equal slices
    norm_groups: int = 1
    embed_scale: float = 1.0
    logit_softcap: float = 0.0      # > 0: logits <- cap * tanh(logits / cap)
    bigram: Optional[tuple] = None  # (buckets, mul_prev, mul_cur): x0 += bigram[(prev * mul_prev + id * mul_cur) mod buckets]
    logit_scale: float = 1.0        # logits <- logits * logit_scale
    norm_one_plus: bool = False     # norm weights are stored around zero: the engine multiplies by 1 + w

    def runs(self):
        """[(layer index, loop_in)] in execution order; loop_in marks the first layer of every pass of the looped range."""
        n = len(self.layers)
        if not self.loop:
            return [(i, False) for i in range(n)]
        a, b, t = self.loop
        out = [(i, False) for i in range(a)]
        for _ in range(t):
            out += [(i, i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]


class HybridMoEC(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("experts", "identity", "top", "ff", "shared_ff")] + \
               [(n, ctypes.c_float) for n in ("limit", "shared_limit", "act_alpha")] + \
               [(n, ctypes.c_void_p) for n in ("router", "correction", "w_gate_up", "w_down", "shared_gate_up", "shared_down")] + \
               [(n, ctypes.c_int32) for n in ("score_kind", "renorm", "scale_input")] + [("up_offset", ctypes.c_float)] + \
               [("expert_form", ctypes.c_int32), ("expert_act", ctypes.c_int32), ("router_bias", ctypes.c_void_p)]


class HybridLayerC(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("kind", "heads", "kv_heads", "dim", "vdim", "window", "pool", "rot_dims")] + \
               [("scale", ctypes.c_float), ("gate_cap", ctypes.c_float), ("ff", ctypes.c_int32)] + \
               [(n, ctypes.c_void_p) for n in ("norm1", "norm2", "w_in", "b_in", "w_out", "lower", "head_norm", "inv_freq",
                                               "w_up", "w_down")] + \
               [("block", ctypes.c_int32), ("sibling", ctypes.c_int32), ("out_scale", ctypes.c_float),
                ("q_norm", ctypes.c_void_p), ("k_norm", ctypes.c_void_p), ("q_temp_coef", ctypes.c_float),
                ("q_temp_every", ctypes.c_int32), ("v_unit_rms", ctypes.c_int32),
                ("conv_taps", ctypes.c_int32), ("rec_scale", ctypes.c_float), ("conv_w", ctypes.c_void_p), ("conv_b", ctypes.c_void_p),
                ("w_gates", ctypes.c_void_p), ("b_gates", ctypes.c_void_p), ("lam", ctypes.c_void_p),
                ("lora", ctypes.c_int32), ("shift_mu", ctypes.c_void_p), ("w_decay2", ctypes.c_void_p), ("decay0", ctypes.c_void_p),
                ("bonus", ctypes.c_void_p), ("moe", ctypes.POINTER(HybridMoEC)),
                ("ff_kind", ctypes.c_int32), ("ff_act", ctypes.c_int32), ("b_up", ctypes.c_void_p), ("b_down", ctypes.c_void_p),
                ("q_rank", ctypes.c_int32), ("kv_rank", ctypes.c_int32), ("rot_dim", ctypes.c_int32),
                ("w_uq", ctypes.c_void_p), ("w_ukT", ctypes.c_void_p), ("w_uv", ctypes.c_void_p),
                ("q_lat_norm", ctypes.c_void_p), ("kv_lat_norm", ctypes.c_void_p), ("decay", ctypes.c_void_p),
                ("ls1", ctypes.c_void_p), ("ls2", ctypes.c_void_p), ("qk_norm_whole", ctypes.c_int32), ("sink", ctypes.c_int32),
                ("decay_channels", ctypes.c_int32), ("gate_rank", ctypes.c_int32), ("gate_act", ctypes.c_int32),
                ("w_gate2", ctypes.c_void_p), ("a_log", ctypes.c_void_p), ("dt_bias", ctypes.c_void_p)]


class HybridRunC(ctypes.Structure):
    _fields_ = [("layer", ctypes.c_int32), ("loop_in", ctypes.c_int32), ("cache", ctypes.c_void_p), ("pool", ctypes.c_void_p),
                ("state", ctypes.c_void_p), ("side_cache", ctypes.c_void_p), ("side_pool", ctypes.c_void_p),
                ("side_state", ctypes.c_void_p)]


class HybridConfigC(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("width", "vocab", "n_layers", "n_runs", "dtype", "page_size", "max_rows",
                                              "max_batch", "max_out", "max_pages", "max_seq_len")] + [("eps", ctypes.c_float)] + \
               [("norm_kind", ctypes.c_int32), ("norm_groups", ctypes.c_int32), ("embed_scale", ctypes.c_float),
                ("logit_softcap", ctypes.c_float), ("bigram_buckets", ctypes.c_int32), ("bigram_mul_prev", ctypes.c_int32),
                ("bigram_mul_cur", ctypes.c_int32), ("logit_scale", ctypes.c_float)]


class HybridWeightsC(ctypes.Structure):
    _fields_ = [("layers", ctypes.POINTER(HybridLayerC)), ("runs", ctypes.POINTER(HybridRunC))] + \
               [(n, ctypes.c_void_p) for n in ("embedding", "loop_in", "head", "final_norm", "bigram", "prev_token")]


class HybridIO(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in ("pos", "row_req", "page", "slot", "req_rows", "req_state", "page_table")] + \
               [("pt_stride", ctypes.c_int32)] + \
               [(n, ctypes.c_void_p) for n in ("out_rows", "logits", "trace", "input_ids", "out_ids", "rng_offset")]


def rotary_frequencies(rot_dims: int, base: float, factor: float) -> torch.Tensor:
    """f_i = base^(-2i/rot_dims) / factor, i < rot_dims/2, in fp32 arithmetic."""
    i = torch.arange(rot_dims // 2, dtype=torch.float32)
    return torch.pow(torch.tensor(base, dtype=torch.float32), -(2.0 * i) / rot_dims) / factor


ROTARY_KINDS = ("attention", "latent_attention", "retention", "causal_attention")


def reduced_bigram(bigram) -> tuple:
    """(buckets, mul_prev, mul_cur) with the multipliers taken modulo the bucket count (the hash is unchanged, every product of a
    token id and a multiplier stays far inside 64 bits); (0, 0, 0) for none."""
    if not bigram:
        return (0, 0, 0)
    n, a, b = (int(v) for v in bigram)
    if n < 1 or n >= 1 << 31:
        raise ValueError(f"bigram buckets {n}")
    return (n, a % n, b % n)


class HybridEngine(Qwen3Engine):
    """`weights`: {"embedding", "head", "final_norm", "loop_in" (or None), "layers": [per layer dict with norm1, norm2, w_in,
    b_in, w_out, lower, head_norm, w_up, w_down, b_up, b_down; per mixer kind also q_norm, k_norm | conv_w, conv_b, w_gates, b_gates,
    lam | shift_mu, w_decay2, decay0, bonus | w_uq, w_ukT, w_uv, q_lat_norm, kv_lat_norm | conv_w, w_decay2, w_gate2, a_log, dt_bias
    (delta rule); ls1, ls2 (layer scale); "moe": {router, router_bias, correction, w_gate_up (up rows only in the up / down form),
    w_down, shared_gate_up, shared_down}; "side": the same mixer keys for a sibling mixer], "bigram" (or None)} — matrices in any
    float dtype (stored as the engine's dtype), vectors and the router stored as fp32.  dtype: torch.bfloat16 or torch.float32."""

    needs_state_slots = True

    def __init__(self, cfg: HybridCfg, weights: Dict, dtype=torch.bfloat16, max_batch=8, page_size=128, max_pages=256,
                 max_seq_len=4096, max_prefill_rows=1024, max_out=None, state_slots=None, device="cuda"):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"HybridEngine: dtype {dtype} (bfloat16 or float32)")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.max_batch, self.page_size, self.max_pages, self.max_seq_len = max_batch, page_size, max_pages, max_seq_len
        self.max_rows = max(max_prefill_rows, max_batch)
        self.max_out = max(max_out or max_batch, max_batch)
        self.state_slots = state_slots or max_batch
        self.L, self.ctx = N.lib(), N.ctx()
        L, vp, ci = self.L, ctypes.c_void_p, ctypes.c_int
        L.vox_hybrid_create.restype, L.vox_hybrid_create.argtypes = ci, [vp, ctypes.POINTER(HybridConfigC), ctypes.POINTER(HybridWeightsC), ctypes.POINTER(vp)]
        L.vox_hybrid_destroy.restype, L.vox_hybrid_destroy.argtypes = None, [vp]
        L.vox_hybrid_step.restype, L.vox_hybrid_step.argtypes = ci, [vp, vp, ctypes.POINTER(HybridIO), vp, ci, ci, ci, ci, ctypes.POINTER(N.SamplingCfg), ctypes.c_uint64, ci]
        dev = self.device
        self._keep = []

        def mat(t):
            if t is None:
                return None
            self._keep.append(t.to(dev, dtype).contiguous())
            return self._keep[-1].data_ptr()

        def vec(t):
            if t is None:
                return None
            self._keep.append(t.to(dev, torch.float32).contiguous())
            return self._keep[-1].data_ptr()

        def norm_w(t):
            """A norm weight of the residual stream: stored around zero when the config says so (1 + w, formed in fp32)."""
            return vec(t.float() + 1.0) if (t is not None and cfg.norm_one_plus) else vec(t)

        W = cfg.width
        sides = [(i, m.side) for i, m in enumerate(cfg.layers) if m.side is not None]
        larr = (HybridLayerC * (len(cfg.layers) + len(sides)))()
        self._moes = []

        def fill(c, m, lw, i):
            assert tuple(lw["w_in"].shape) == (m.n_in, W), (i, m.kind, tuple(lw["w_in"].shape), m.n_in)
            assert tuple(lw["w_out"].shape) == (W, m.heads * m.vdim), (i, m.kind, tuple(lw["w_out"].shape))
            c.kind, c.heads, c.kv_heads, c.dim, c.vdim = MIXER_KINDS[m.kind], m.heads, m.kv_heads, m.dim, m.vdim
            c.window, c.pool, c.rot_dims, c.scale, c.gate_cap, c.ff = m.window, m.pool, m.rot_dims, m.scale, m.gate_cap, m.ff
            c.norm1, c.norm2 = norm_w(lw["norm1"]), norm_w(lw.get("norm2"))
            c.ls1, c.ls2 = vec(lw.get("ls1")), vec(lw.get("ls2"))
            c.qk_norm_whole, c.sink = int(m.qk_norm_whole), int(m.sink)
            c.decay_channels, c.gate_rank, c.gate_act = int(m.decay_channels), m.gate_rank, GATE_KINDS[m.gate_act]
            c.w_gate2, c.a_log, c.dt_bias = mat(lw.get("w_gate2")), vec(lw.get("a_log")), vec(lw.get("dt_bias"))
            c.w_in, c.b_in, c.w_out = mat(lw["w_in"]), vec(lw.get("b_in")), mat(lw["w_out"])
            c.lower, c.head_norm = vec(lw.get("lower")), vec(lw.get("head_norm"))
            c.inv_freq = vec(rotary_frequencies(m.rot_dims, m.rot_base, m.rot_factor)) if m.kind in ROTARY_KINDS and m.rot_dims else None
            c.w_up, c.w_down = mat(lw.get("w_up")), mat(lw.get("w_down"))
            c.block, c.sibling, c.out_scale = BLOCK_FORMS[m.block], -1, m.out_scale
            c.q_norm, c.k_norm = vec(lw.get("q_norm")), vec(lw.get("k_norm"))
            c.q_temp_coef, c.q_temp_every, c.v_unit_rms = m.q_temp_coef, m.q_temp_every, int(m.v_unit_rms)
            c.conv_taps, c.rec_scale = m.conv_taps, m.rec_scale
            c.conv_w, c.conv_b, c.w_gates, c.b_gates, c.lam = vec(lw.get("conv_w")), vec(lw.get("conv_b")), mat(lw.get("w_gates")), \
                vec(lw.get("b_gates")), vec(lw.get("lam"))
            c.lora, c.shift_mu, c.w_decay2 = m.lora, vec(lw.get("shift_mu")), mat(lw.get("w_decay2"))
            c.decay0, c.bonus = vec(lw.get("decay0")), vec(lw.get("bonus"))
            c.ff_kind, c.ff_act, c.b_up, c.b_down = FF_KINDS[m.ff_kind], ACT_KINDS[m.ff_act], vec(lw.get("b_up")), vec(lw.get("b_down"))
            c.q_rank, c.kv_rank, c.rot_dim = m.q_rank, m.kv_rank, m.rot_dim
            c.w_uq, c.w_ukT, c.w_uv = mat(lw.get("w_uq")), mat(lw.get("w_ukT")), mat(lw.get("w_uv"))
            c.q_lat_norm, c.kv_lat_norm = vec(lw.get("q_lat_norm")), vec(lw.get("kv_lat_norm"))
            if m.kind == "retention":
                if m.decay is None or len(m.decay) != m.heads:
                    raise ValueError(f"layer {i}: retention needs one decay per head")
                c.decay = vec(torch.tensor([float(a) for a in m.decay], dtype=torch.float32))
            if m.moe is not None:
                e, ew = m.moe, lw["moe"]
                mc = HybridMoEC(e.experts, e.identity, e.top, e.ff, e.shared_ff, e.limit, e.shared_limit, e.act_alpha,
                                vec(ew["router"]), vec(ew.get("correction")), mat(ew.get("w_gate_up")), mat(ew.get("w_down")),
                                mat(ew.get("shared_gate_up")), mat(ew.get("shared_down")), ROUTER_SCORES[e.score], int(e.renorm),
                                int(e.scale_input), e.up_offset, EXPERT_FORMS[e.expert_form], ACT_KINDS[e.expert_act],
                                vec(ew.get("router_bias")) if e.router_bias else None)
                self._moes.append(mc)
                c.moe = ctypes.pointer(mc)

        for i, (m, lw) in enumerate(zip(cfg.layers, weights["layers"])):
            fill(larr[i], m, lw, i)
        for j, (i, sm) in enumerate(sides):
            # the sibling's record: its own mixer tensors; norms, block form and feed-forward are the primary layer's business
            fill(larr[len(cfg.layers) + j], sm, dict(weights["layers"][i]["side"], norm1=weights["layers"][i]["norm1"]), i)
            larr[i].sibling = len(cfg.layers) + j
        runs = cfg.runs()
        rarr = (HybridRunC * len(runs))()
        self.caches, self.pools, self.states = [], [], []

        def storage(m):
            """(cache, pool, state) of one mixer of one run."""
            if m.kind in ATTENTION_KINDS:
                kv = torch.zeros(max_pages * page_size * m.cache_values(), dtype=dtype, device=dev)
                self.caches.append(kv)
                if m.kind == "attention":
                    pool = torch.zeros(max_pages, (page_size - 1) // m.pool + 1, m.kv_heads, m.dim + m.vdim, dtype=torch.float32, device=dev)
                    self.pools.append(pool)
                    return kv.data_ptr(), pool.data_ptr(), None
                if m.state_floats(W):
                    # what the attention keeps per request besides its pages (the history of a convolution in front of it)
                    st = torch.zeros(self.state_slots, m.state_floats(W), dtype=torch.float32, device=dev)
                    self.states.append(st)
                    return kv.data_ptr(), None, st.data_ptr()
                return kv.data_ptr(), None, None
            st = torch.zeros(self.state_slots, m.state_floats(W), dtype=torch.float32, device=dev)
            self.states.append(st)
            return None, None, st.data_ptr()

        for j, (li, loop_in) in enumerate(runs):
            m = cfg.layers[li]
            # a loop without an input matrix just runs the range again: nothing happens between the passes
            rarr[j].layer, rarr[j].loop_in = li, int(loop_in and weights.get("loop_in") is not None)
            rarr[j].cache, rarr[j].pool, rarr[j].state = storage(m)
            if m.side is not None:
                rarr[j].side_cache, rarr[j].side_pool, rarr[j].side_state = storage(m.side)
        self.n_runs = len(runs)
        bg = reduced_bigram(cfg.bigram)
        cc = HybridConfigC(W, cfg.vocab, len(larr), len(runs), 0 if dtype == torch.bfloat16 else 1, page_size, self.max_rows,
                           max_batch, self.max_out, max_pages, max_seq_len, cfg.eps, NORM_KINDS[cfg.norm_kind], cfg.norm_groups,
                           cfg.embed_scale, cfg.logit_softcap, int(bg[0]), int(bg[1]), int(bg[2]), float(cfg.logit_scale))
        # the last token every state slot's sequence has seen (what a bigram embedding needs of the step before)
        self.prev_token = torch.zeros(self.state_slots, dtype=torch.int32, device=dev)
        if cfg.bigram and tuple(weights["bigram"].shape) != (int(bg[0]) + 1, W):
            raise ValueError(f"bigram table {tuple(weights['bigram'].shape)}: expected {(int(bg[0]) + 1, W)}")
        emb = mat(weights["embedding"])
        head = emb if weights["head"] is weights["embedding"] else mat(weights["head"])      # a tied head shares the table
        cw = HybridWeightsC(ctypes.cast(larr, ctypes.POINTER(HybridLayerC)), ctypes.cast(rarr, ctypes.POINTER(HybridRunC)),
                            emb, mat(weights.get("loop_in")), head, norm_w(weights["final_norm"]),
                            mat(weights.get("bigram")) if cfg.bigram else None, self.prev_token.data_ptr())
        self._larr, self._rarr = larr, rarr
        h = ctypes.c_void_p()
        N.check(L.vox_hybrid_create(self.ctx, ctypes.byref(cc), ctypes.byref(cw), ctypes.byref(h)))
        self.h = h
        i32 = dict(dtype=torch.int32, device=dev)
        R = self.max_rows
        self.input_ids = torch.zeros(max_batch, 1, **i32)
        self.row_ids = torch.zeros(R, 1, **i32)
        self.row_masks = torch.zeros(R, dtype=torch.uint8, device=dev)           # (unused: kept for the worker's staging code)
        self.pt_stride = (max_seq_len + page_size - 1) // page_size + 1
        self._plan_layout, off = {}, 0
        for name, n in (("pos", R), ("kvlen", R), ("page", R), ("slot", R), ("q_req", R), ("last_rows", self.max_out),
                        ("indptr", max_batch + 1), ("indices", max_pages), ("ptab", max_batch * self.pt_stride),
                        ("req_rows", max_batch + 1), ("state", max_batch)):
            self._plan_layout[name] = (off, n)
            off += n
        self.plan_dev = torch.zeros(off, **i32)
        self._init_plan_host(off)
        self.out_ids = torch.zeros(max_batch, **i32)
        self.out_logits = torch.zeros(self.max_out, cfg.vocab, dtype=torch.float32, device=dev)
        self.rng_offset = torch.zeros(1, dtype=torch.int64, device=dev)
        self.trace = None
        self.rep_cache = None
        self._graphs, self.keep_hidden = {}, False

    def enable_trace(self):
        """Keep the residual stream after every layer run of the next steps: trace[run, row, :]."""
        if self.trace is None:
            self.trace = torch.zeros(self.n_runs, self.max_rows, self.cfg.width, dtype=torch.float32, device=self.device)
            self._drop_graphs()
        return self.trace

    def _io(self):
        return HybridIO(self._pd("pos").data_ptr(), self._pd("q_req").data_ptr(), self._pd("page").data_ptr(),
                        self._pd("slot").data_ptr(), self._pd("req_rows").data_ptr(), self._pd("state").data_ptr(),
                        self._pd("ptab").data_ptr(), self.pt_stride, self._pd("last_rows").data_ptr(), self.out_logits.data_ptr(),
                        self.trace.data_ptr() if self.trace is not None else None, self.input_ids.data_ptr(),
                        self.out_ids.data_ptr(), self.rng_offset.data_ptr())

    def _mutable_state(self):
        # a decode step advances the recurrent states and appends K / V: the warm-up run before a capture must leave no trace
        return [self.input_ids, self.rng_offset, self.prev_token] + self.states

    def _native_frame(self, io, st, batch, bucket, sampling, seed, feedback):
        N.check(self.L.vox_hybrid_step(self.h, st, ctypes.byref(io), self.input_ids.data_ptr(), batch, batch, batch, int(bucket),
                                       ctypes.byref(sampling), seed, int(feedback)))

    def _native_destroy(self):
        self.L.vox_hybrid_destroy(self.h)

    def step(self, n_rows, n_req, n_out=None, sampling=None, seed=0, feedback=True, sample=True, max_kvlen=0):
        """One ragged step, eagerly: rows staged in row_ids + plan arrays.  n_out rows (plan `last_rows`) get logits in
        out_logits[:n_out]; with `sample`, requests 0..n_req-1 are sampled from output rows 0..n_req-1."""
        n_out = n_req if n_out is None else n_out
        io = self._io()
        sc = ctypes.byref(sampling or self.sampling_cfg()) if sample else None
        self._log_launch("prefill", (n_rows, n_req, n_out), n_req)
        N.check(self.L.vox_hybrid_step(self.h, N.stream(), ctypes.byref(io), self.row_ids.data_ptr(), n_rows, n_req, n_out, int(max_kvlen), sc,
                                       seed, int(feedback and sample)))

    def _prefill_on_stream(self, n_rows, n_req, max_kvlen, sampling, seed, feedback):
        if n_req == 0:
            raise N.VoxError("HybridEngine: a step without requests")
        io = self._io()
        N.check(self.L.vox_hybrid_step(self.h, N.stream(), ctypes.byref(io), self.row_ids.data_ptr(), n_rows, n_req, n_req, int(max_kvlen),
                                       ctypes.byref(sampling), seed, int(feedback)))

    @staticmethod
    def sampling_cfg(greedy=True, top_k=0, top_p=1.0, min_p=0.0, temperature=1.0, repetition_penalty=1.0):
        return N.SamplingCfg(int(greedy), int(top_k or 0), float(1.0 if top_p is None else top_p), float(min_p or 0.0),
                             float(temperature), 1.0)
