"""Helpers for the Fironex tests: layer layouts, random checkpoints written
to disk (so the engine loads them through its own config reader and weight
loader) and engines over them. Replay and error helpers are shared with the
other layer-list model's tests."""
import copy
import json
import os

import torch
from safetensors.torch import save_file

from bolatar_util import make_engine, rel_err, replay, TOL  # noqa: F401

# Layouts that avoid equal or trivial sizes: kv_heads != heads and != 1,
# dim != vdim != kv_rank, partial rotation, three gate blocks, odd vocab.
ROT_SCALED = {"base": 10000.0, "dims": 12,
              "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0,
                          "original": 64}}
ATTN = {"type": "attention",
        "mixer": {"heads": 6, "kv_heads": 3, "dim": 24, "vdim": 40,
                  "scale": 0.21, "diff": 0.3, "mask": {"size": 19},
                  "rot": ROT_SCALED},
        "mlp": {"kind": "dense", "ff": 100}}
ATTN_FULL = {"type": "attention",     # no window, whole head rotated, no mlp
             "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 24,
                       "scale": 0.3, "diff": 0.7,
                       "rot": {"base": 500.0, "dims": 16}},
             "mlp": None}
LATENT = {"type": "latent_attention",
          "mixer": {"heads": 3, "dim": 24, "rot_dim": 8, "vdim": 20,
                    "kv_rank": 40, "scale": 0.17,
                    "rot": {"base": 5000.0, "dims": 8}},
          "mlp": {"kind": "dense", "ff": 144}}


def latent_from(src, heads=2, dim=16, vdim=28, scale=0.22, mlp=True):
    """A latent layer that reads layer `src`'s cache (same latent sizes and
    rotation as LATENT, its own heads and head sizes)."""
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": 8, "vdim": vdim,
                      "kv_rank": 40, "scale": scale, "kv_from": src,
                      "rot": {"base": 5000.0, "dims": 8}},
            "mlp": {"kind": "dense", "ff": 120} if mlp else None}


RGLRU = {"type": "rglru", "mixer": {"width": 72, "blocks": 3, "conv": 3},
         "mlp": None}
RGLRU_WIDE = {"type": "rglru", "mixer": {"width": 130, "blocks": 1, "conv": 5},
              "mlp": {"kind": "dense", "ff": 90}}


def make_config(layers, width=96, vocab=157, mult=0.8, eps=1e-5):
    return {"architecture": "Fironex", "layers": copy.deepcopy(layers),
            "norm": {"eps": eps}, "residual_mult": mult, "vocab": vocab,
            "width": width}


def random_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, std=None):
        return torch.randn(o, i, generator=g) * (std or i ** -0.5)

    def uni(shape, lo, hi):
        shape = (shape,) if isinstance(shape, int) else shape
        return lo + (hi - lo) * torch.rand(tuple(shape), generator=g)

    t = {"embed": mat(cfg["vocab"], W, 0.6), "final.norm": uni(W, 0.7, 1.3)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"], t[p + "norm1b"] = uni(W, 0.7, 1.3), uni(W, 0.7, 1.3)
        x = p + "mix."
        if L["type"] == "rglru":
            C, nb, taps = m["width"], m["blocks"], m["conv"]
            bw = C // nb
            t[x + "y"], t[x + "y.b"] = mat(C, W), uni(C, -0.3, 0.3)
            t[x + "x"], t[x + "x.b"] = mat(C, W), uni(C, -0.3, 0.3)
            t[x + "conv"], t[x + "conv.b"] = uni((C, taps), -0.6, 0.9), uni(C, -0.2, 0.2)
            t[x + "ra"] = torch.randn(nb, bw, bw, generator=g) * bw ** -0.5
            t[x + "ri"] = torch.randn(nb, bw, bw, generator=g) * bw ** -0.5
            t[x + "ra.b"], t[x + "ri.b"] = uni((nb, bw), -1, 1), uni((nb, bw), -1, 1)
            t[x + "lam"] = uni(C, -5.0, -0.5)
            t[x + "o"] = mat(W, C)
        elif L["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[x + "q"], t[x + "k"] = mat(2 * H * dk, W), mat(2 * G * dk, W)
            t[x + "v"], t[x + "g"] = mat(G * dv, W), mat(H * dv, W)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                t[x + n] = uni(dk, -0.3, 0.3)
            t[x + "o"] = mat(W, H * dv)
        else:
            H, dk, rd, dv, R = (m["heads"], m["dim"], m["rot_dim"], m["vdim"],
                                m["kv_rank"])
            t[x + "q"] = mat(H * (dk + rd), W)
            if m.get("kv_from") is None:
                t[x + "dkv"] = mat(R + rd, W)
                t[x + "dkv.norm"] = uni(R, 0.6, 1.4)
            t[x + "uk"], t[x + "uv"] = mat(H * dk, R), mat(H * dv, R)
            t[x + "g"] = mat(H, W)
            t[x + "o"] = mat(W, H * dv)
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            t[p + "norm2"], t[p + "norm2b"] = uni(W, 0.7, 1.3), uni(W, 0.7, 1.3)
            t[p + "mlp.up"], t[p + "mlp.down"] = mat(F, W), mat(W, F)
            t[p + "mlp.act"] = uni(2, -1.0, 1.5)
    # checkpoints hold bf16 values; keep them exactly representable
    return {k: v.to(torch.bfloat16) for k, v in t.items()}


def write_checkpoint(path, cfg, weights):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
    return str(path)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(2000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
