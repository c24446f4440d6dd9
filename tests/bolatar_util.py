"""Helpers for the Bolatar tests: random checkpoints written to disk (so the
engine loads them through its own config reader and weight loader), engines
over them, and schedule replays compared with the slow oracle."""
import copy
import json
import os

import torch
from safetensors.torch import save_file

import bolatar_oracle as oracle

# Small layouts that avoid equal or trivial sizes: kv_heads != 1 and
# != heads, dim != vdim, heads*dim != width, odd vocab, several conv widths.
DELTA = {"type": "delta",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "conv": 3},
         "mlp": None}
DELTA_WIDE = {"type": "delta",
              "mixer": {"heads": 3, "kv_heads": 3, "dim": 40, "vdim": 72,
                        "conv": 5},
              "mlp": {"kind": "dense", "ff": 100, "limit": 1.5}}
PARALLEL = {"type": "parallel",
            "mixer": {"left": {"heads": 6, "kv_heads": 3, "dim": 24,
                               "vdim": 40, "scale": 0.25,
                               "q_temp": {"coef": 0.9, "every": 16}},
                      "right": {"heads": 3, "dim": 40}},
            "mlp": {"kind": "dense", "ff": 144, "limit": 3.0}}
MLSTM = {"type": "mlstm",
         "mixer": {"heads": 2, "dim": 16, "vdim": 48, "gate_cap": 10.0},
         "mlp": {"kind": "dense", "ff": 120, "limit": 2.5}}


def make_config(layers, width=96, vocab=157, max_positions=640):
    return {"architecture": "Bolatar", "embedding": {"scale": 2.5},
            "layers": copy.deepcopy(layers), "logit_softcap": 25.0,
            "max_positions": max_positions, "norm": {"eps": 1e-5},
            "vocab": vocab, "width": width}


def random_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, std=None):
        return torch.randn(o, i, generator=g) * (std or i ** -0.5)

    def uni(shape, lo, hi):
        shape = (shape,) if isinstance(shape, int) else shape
        return lo + (hi - lo) * torch.rand(tuple(shape), generator=g)

    t = {"embed": mat(cfg["vocab"], W, 0.3),
         "pos": mat(cfg["max_positions"], W, 0.3),
         "final.norm": uni((), 0.8, 1.3), "head": mat(cfg["vocab"], W, 1.0)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = uni((), 0.8, 1.3)
        x = p + "mix."
        if L["type"] == "delta":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, rows in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
                t[x + n] = mat(rows, W)
                t[x + n + ".conv"] = uni((rows, m["conv"]), -0.7, 1.0)
            t[x + "g"] = mat(H * dv, W)
            t[x + "b"] = mat(H, W)
            t[x + "a"] = mat(H, W)
            t[x + "A_log"] = uni(H, -3.0, -0.5)
            t[x + "dt_bias"] = uni(H, -2.0, 0.0)
            t[x + "norm"] = uni(dv, 0.6, 1.4)
            t[x + "o"] = mat(W, H * dv)
        elif L["type"] == "mlstm":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            t[x + "q"], t[x + "k"] = mat(H * dk, W), mat(H * dk, W)
            t[x + "v"], t[x + "g"] = mat(H * dv, W), mat(H * dv, W)
            t[x + "i"], t[x + "f"] = mat(H, W), mat(H, W)
            t[x + "i.b"], t[x + "f.b"] = uni(H, -1, 1), uni(H, 0.5, 5.0)
            t[x + "norm"] = uni(H * dv, 0.6, 1.4)
            t[x + "o"] = mat(W, H * dv)
        else:
            l, r = m["left"], m["right"]
            H, G, dk, dv = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
            t[x + "left.q"], t[x + "left.k"] = mat(H * dk, W), mat(G * dk, W)
            t[x + "left.v"], t[x + "left.o"] = mat(G * dv, W), mat(W, H * dv)
            t[x + "left.r1"], t[x + "left.r2"] = uni(H, 0, 2), uni(H, 0.1, 0.3)
            HD, rank = r["heads"] * r["dim"], 12
            for s in "rkvgw":
                t[x + "right.mu." + s] = uni(W, 0, 0.8)
            for s in "rkvg":
                t[x + "right." + s] = mat(HD, W)
            t[x + "right.w1"], t[x + "right.w2"] = mat(rank, W), mat(HD, rank, 0.2)
            t[x + "right.w0"] = uni(HD, -5.0, -0.3)
            t[x + "right.u"] = uni((r["heads"], r["dim"]), -0.4, 1.5)
            t[x + "right.norm"] = uni(HD, 0.6, 1.4)
            t[x + "right.o"] = mat(W, HD)
            t[x + "left.out"], t[x + "right.out"] = uni(W, 0.6, 1.3), uni(W, 0.6, 1.3)
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            t[p + "norm2"] = uni((), 0.8, 1.3)
            t[p + "mlp.gate"], t[p + "mlp.up"] = mat(F, W), mat(F, W)
            t[p + "mlp.down"] = mat(W, F)
    # checkpoints hold bf16 values; keep them exactly representable
    return {k: v.to(torch.bfloat16) for k, v in t.items()}


def write_checkpoint(path, cfg, weights):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
    return str(path)


def make_engine(path, device="cpu", dtype="float32", pages=24, slots=4,
                page_size=16, graphs=False, **kw):
    from dynamo_amd.engine import EngineConfig, LLMEngine
    from dynamo_amd.models.registry import resolve_model_config
    model = resolve_model_config(path)
    cfg = EngineConfig(model=model, device=device, dtype=dtype,
                       page_size=page_size, max_num_seqs=slots,
                       max_model_len=model.max_position, kv_pool_pages=pages,
                       enable_hip_graphs=graphs, **kw)
    return LLMEngine(cfg)


def replay(engine, rid, tokens, sizes, end=True):
    """Feed one request in portions of the given sizes (the last size
    repeats); returns logits of every position [T, vocab]."""
    out, pos, k = [], 0, 0
    while pos < len(tokens):
        n = min(sizes[min(k, len(sizes) - 1)], len(tokens) - pos)
        last = pos + n == len(tokens)
        lg = engine.replay_step([(rid, tokens[pos:pos + n], list(range(n)))],
                                [rid] if (last and end) else [])
        out.append(lg.cpu())
        pos += n
        k += 1
    return torch.cat(out, 0)


def rel_err(got, want):
    """RMS difference over the vocabulary (mean removed) relative to the
    RMS spread of the expected logits, worst position."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).max())


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


TOL = {"float32": 2e-4, "bfloat16": 6e-2}
