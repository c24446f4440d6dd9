"""Bolatar: a decoder-only LM whose layers are listed in its config, each
with one of three mixers - a gated delta rule ('delta'), softmax attention
with a distance bias beside RWKV-style time mixing ('parallel'), or an
mLSTM matrix memory ('mlstm') - and an optional clamped-GLU feed-forward.

The residual stream is fp32; every norm on it has a single scalar gain.
Token embeddings are scaled and a learned position vector is added. Logits
are soft-capped. Recurrent state lives in the engine's slot-addressed state
pool, attention keys/values in its paged cache (per-layer head sizes).

config.json keys read here: architecture, vocab, width, max_positions,
embedding.scale, norm.eps, logit_softcap, layers[].{type, mixer, mlp}.
Checkpoint tensor names: embed, pos, l<i>.norm1, l<i>.norm2, l<i>.mix.*,
l<i>.mlp.{gate,up,down}, final.norm, head.
"""
from __future__ import annotations

import json
import os
from typing import List, Optional

import torch
import torch.nn.functional as F

from dynamo_amd.engine.config import ModelConfig
from dynamo_amd.ops import seq as sops
from .layers import AttnMetadata, TPContext
from .mixers import (BiasedAttention, ClampedGLU, GatedDeltaMixer, MixContext,
                     MLSTMMixer, ParallelMixer, RWKVTimeMix, _Init, _put)


def config_from_json(hf: dict, name: str = "bolatar") -> ModelConfig:
    return ModelConfig(
        name=name, arch="bolatar", hidden_size=hf["width"],
        vocab_size=hf["vocab"], max_position=hf["max_positions"],
        num_layers=len(hf["layers"]), rms_eps=float(hf["norm"]["eps"]),
        learned_pos_emb=True, layer_specs=hf["layers"],
        embed_scale=float(hf["embedding"]["scale"]),
        logit_softcap=float(hf.get("logit_softcap") or 0.0),
        # the uniform-attention fields do not apply; keep them inert
        intermediate_size=0, num_q_heads=1, num_kv_heads=1, head_dim=1)


def build_mixer(kind: str, m: dict, width: int, eps: float, init: _Init):
    if kind == "delta":
        return GatedDeltaMixer(width, m["heads"], m["kv_heads"], m["dim"],
                               m["vdim"], m["conv"], eps, init)
    if kind == "mlstm":
        return MLSTMMixer(width, m["heads"], m["dim"], m["vdim"],
                          m["gate_cap"], eps, init)
    if kind == "parallel":
        l, r = m["left"], m["right"]
        qt = l.get("q_temp") or {}
        left = BiasedAttention(width, l["heads"], l["kv_heads"], l["dim"],
                               l["vdim"], l["scale"], eps, init,
                               temp_coef=float(qt.get("coef", 0.0)),
                               temp_every=int(qt.get("every", 1)))
        right = RWKVTimeMix(width, r["heads"], r["dim"], eps, init)
        return ParallelMixer(width, left, right, eps, init)
    raise ValueError(f"unknown Bolatar layer type {kind!r}")


class BolatarLayer(torch.nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, init: _Init):
        super().__init__()
        self.eps = eps
        self.norm1 = init.vec(1, 0.8, 1.2)
        self.mixer = build_mixer(spec["type"], spec["mixer"], width, eps, init)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            self.norm2 = init.vec(1, 0.8, 1.2)
            self.mlp = ClampedGLU(width, mlp["ff"], mlp["limit"], init)


class BolatarForCausalLM(torch.nn.Module):
    needs_seq_batch = True       # the runner builds SeqBatch descriptors

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16,
                 tp: Optional[TPContext] = None, seed: int = 0):
        super().__init__()
        self.cfg = cfg
        self.tp = tp or TPContext()
        if self.tp.size != 1:
            raise ValueError("Bolatar runs with tensor-parallel size 1")
        self.dtype = dtype
        gen = torch.Generator(device="cpu")
        gen.manual_seed(seed)
        init = _Init(device, dtype, gen)
        W = cfg.hidden_size
        self.embed = init.mat(cfg.vocab_size, W, std=0.3)
        self.pos = init.mat(cfg.max_position, W, std=0.3)
        self.layers = torch.nn.ModuleList(
            [BolatarLayer(s, W, cfg.rms_eps, init) for s in cfg.layer_specs])
        self.final_norm = init.vec(1, 0.8, 1.2)
        self.lm_head = init.mat(cfg.vocab_size, W, std=1.0)

    # -- what the engine must hold ------------------------------------
    def kv_layer_shapes(self):
        """Per layer: (kv_heads, key_dim, value_dim) or None."""
        return [l.mixer.kv_shape() for l in self.layers]

    def state_layer_shapes(self):
        """Per layer: list of per-slot fp32 state shapes."""
        return [l.mixer.state_shapes() for l in self.layers]

    # -- weights --------------------------------------------------------
    def load_checkpoint(self, path: str) -> int:
        from .loader import _iter_safetensors
        tensors = dict(_iter_safetensors(path))
        used = set()

        def get(name):
            used.add(name)
            return tensors[name]
        _put(self.embed, get("embed"))
        _put(self.pos, get("pos"))
        _put(self.final_norm, get("final.norm").reshape(1))
        _put(self.lm_head, get("head"))
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            _put(layer.norm1, get(p + "norm1").reshape(1))
            layer.mixer.load(lambda n, p=p: get(p + "mix." + n))
            if layer.mlp is not None:
                _put(layer.norm2, get(p + "norm2").reshape(1))
                layer.mlp.load(lambda n, p=p: get(p + "mlp." + n))
        extra = set(tensors) - used
        if extra:
            raise ValueError(f"checkpoint tensors not consumed: {sorted(extra)}")
        return len(used)

    # -- forward ----------------------------------------------------------
    def forward(self, input_ids, kv_pool, meta: AttnMetadata,
                tap: Optional[list] = None):
        sb = meta.seq_batch
        states = meta.state_pool
        x = sops.embed_scale_pos(input_ids, meta.positions, self.embed,
                                 self.pos, self.cfg.embed_scale)
        if meta.inputs_embeds is not None:
            x = x.index_copy(0, meta.embeds_rows, meta.inputs_embeds.float())
        delta = None
        for i, layer in enumerate(self.layers):
            h = sops.add_scalar_rmsnorm(x, delta, layer.norm1, layer.eps,
                                        self.dtype)
            has_kv = layer.mixer.kv_shape() is not None
            ctx = MixContext(sb, meta.positions, meta.slot_mapping,
                             states.layer(i),
                             kv_pool.kcache(i) if has_kv else None,
                             kv_pool.vcache(i) if has_kv else None)
            delta = layer.mixer.forward(h, ctx)
            if layer.mlp is not None:
                h = sops.add_scalar_rmsnorm(x, delta, layer.norm2, layer.eps,
                                            self.dtype)
                delta = layer.mlp.forward(h)
            if tap is not None:     # residual after the layer (diagnostics)
                tap.append(x + delta.float())
        return sops.add_scalar_rmsnorm(x, delta, self.final_norm,
                                       self.cfg.rms_eps, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = F.linear(hidden, self.lm_head).float()
        if self.cfg.logit_softcap:
            logits = sops.softcap_(logits.contiguous(), self.cfg.logit_softcap)
        return logits
