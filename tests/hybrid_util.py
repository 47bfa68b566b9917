"""Helpers of the hybrid-engine tests (Sirodra, Fusanex, Dipivik, Sizitar): small configurations, random checkpoints, and a driver that feeds token
portions through ModelWorker the way a serving step does."""
import math

import torch


def hgrn2(heads=2, dim=8, vdim=16, ff=0):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def mlstm(heads=2, dim=8, vdim=16, cap=10.0, ff=0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def attention(heads=4, kv_heads=2, dim=16, vdim=16, window=6, pool=4, rot=8, base=100.0, factor=1.0, scale=None, ff=0):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window, "pool": pool},
                      "rot": {"dims": rot, "base": base, "scaling": {"factor": factor}},
                      "scale": scale if scale is not None else 1.0 / math.sqrt(dim)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=32, vocab=50, loop=None, eps=1e-5):
    c = {"architecture": "Sirodra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def random_checkpoint(cfg, seed=0, gain=1.0):
    """bf16 tensors under the checkpoint's names; gain > 1 sharpens every projection (scores that stand out)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * (s * gain / math.sqrt(i))).to(torch.bfloat16)

    def vec(n, mean=0.0, std=0.2):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)
    S = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(torch.bfloat16), "head": mat(cfg["vocab"], W), "final.norm": vec(W, 1.0)}
    if cfg.get("loop"):
        S["loop.in"] = mat(W, 2 * W, 1.4)
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], f"l{i}."
        H, d, e = m["heads"], m["dim"], m["vdim"]
        S[p + "norm1"] = vec(W, 1.0)
        if L["type"] == "hgrn2":
            S.update({p + "mix.q": mat(H * d, W), p + "mix.f": mat(H * d, W, 2.0), p + "mix.f.b": vec(H * d, 1.0, 1.5),
                      p + "mix.lower": (torch.rand(H * d, generator=g) * 0.95).to(torch.bfloat16), p + "mix.v": mat(H * e, W),
                      p + "mix.norm": vec(e, 1.0), p + "mix.o": mat(W, H * e)})
        elif L["type"] == "mlstm":
            S.update({p + "mix.q": mat(H * d, W), p + "mix.k": mat(H * d, W), p + "mix.v": mat(H * e, W), p + "mix.g": mat(H * e, W),
                      p + "mix.o": mat(W, H * e), p + "mix.norm": vec(H * e, 1.0), p + "mix.i": mat(H, W, 3.0), p + "mix.i.b": vec(H, 0.0, 2.0),
                      p + "mix.f": mat(H, W, 3.0), p + "mix.f.b": vec(H, 2.0, 2.0)})
        else:
            G = m["kv_heads"]
            S.update({p + "mix.q": mat(H * d, W), p + "mix.q.b": vec(H * d), p + "mix.k": mat(G * d, W), p + "mix.k.b": vec(G * d),
                      p + "mix.v": mat(G * e, W), p + "mix.v.b": vec(G * e), p + "mix.g": mat(H, W), p + "mix.o": mat(W, H * e)})
        if L["mlp"]:
            S.update({p + "norm2": vec(W, 1.0), p + "mlp.up": mat(L["mlp"]["ff"], W), p + "mlp.down": mat(W, L["mlp"]["ff"])})
    return S


class Driver:
    """A model + ModelWorker on the GPU; `feed` runs one step of token portions and returns the logits of every fed token."""

    def __init__(self, cfg, S, dtype=torch.float32, page_size=8, pages=64, slots=4, max_rows=256, max_batch=4):
        from vox_serve_amd.model import get_model_class
        from vox_serve_amd.worker.base import ModelWorker
        # the registry entry of the config's architecture builds the model, as for a checkpoint folder
        from vox_serve_amd.model import dipivik, fusanex, sirodra, sizitar
        mod = {"Sirodra": sirodra, "Fusanex": fusanex, "Dipivik": dipivik, "Sizitar": sizitar}[cfg["architecture"]]
        self.model = get_model_class(cfg["architecture"])(cfg["architecture"].lower() + "-test", weights=S, config=mod.config_from_dict(cfg),
                                                          dtype=dtype, max_batch_size=max_batch, page_size=page_size, max_num_pages=pages,
                                                          max_seq_len=pages * page_size, max_prefill_tokens=max_rows,
                                                          max_logit_rows=max_rows + max_batch, state_slots=slots)
        self.worker = ModelWorker(model=self.model, max_batch_size=max_batch, max_num_pages=pages, page_size=page_size, greedy=True)
        self.live = {}

    def feed(self, portions):
        """portions: [(request id, [token ids])] -> {id: logits [n, vocab] (cpu float32)} for the tokens fed in this step."""
        from vox_serve_amd.requests import Request
        reqs, rows, n = [], [], 0
        for rid, toks in portions:
            t = torch.tensor(toks, dtype=torch.long).view(-1, 1)
            r = self.live.get(rid)
            if r is None:
                r = self.live[rid] = Request(request_id=rid, prompt_open=True)
                r.input_tokens, r._preprocessed = t, True
            else:
                r.input_tokens = torch.cat([r.input_tokens, t], 0)
            r.step_budget = len(toks)
            reqs.append(r)
            rows += list(range(n, n + len(toks)))
            n += len(toks)
        li = self.worker.prepare_lm_inputs(reqs, [])
        li["logit_rows"] = rows
        self.worker.run_lm_prefill(reqs, li)
        lg = self.model.engine.out_logits[len(reqs): len(reqs) + n].to("cpu", torch.float32)
        out, o = {}, 0
        for rid, toks in portions:
            out[rid] = lg[o:o + len(toks)].clone()
            o += len(toks)
        return out

    def end(self, rid):
        self.worker.free_kv_cache(self.live.pop(rid))

    def run_cut(self, rid, tokens, cuts):
        """One request alone, its tokens cut into portions of the given sizes (the rest one by one) -> logits [T, vocab]."""
        outs, o = [], 0
        for c in list(cuts) + [1] * len(tokens):
            if o >= len(tokens):
                break
            outs.append(self.feed([(rid, tokens[o:o + c])])[rid])
            o += c
        self.end(rid)
        return torch.cat(outs, 0)

    def close(self):
        self.model.engine.close()


def rel_err(got, want, quantile=None):
    """Per position: RMS over the vocabulary of the mean-free difference, relative to the RMS of the mean-free reference.
    The worst position, or (bf16 runs through ill-conditioned gates) the given quantile over positions."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()
    return (e.max() if quantile is None else e.quantile(quantile)).item()
