"""Fironex: a decoder-only LM whose config lists its layers, each with one
of three mixers - a real-gated linear recurrent unit ('rglru'), differential
attention under a sliding window ('attention'), or attention over a shared
compressed latent ('latent_attention', optionally reading the cache of an
earlier latent layer) - and an optional xIELU feed-forward.

The residual stream is fp32. Every sublayer is normed on both sides with a
weight-only layer norm: x <- x + m * LN_b(sublayer(LN_a(x))), m being the
config's residual multiplier. Logits use the embedding table. Recurrent
state lives in the engine's slot-addressed state pool, keys/values and
latents in its paged cache (per-layer row sizes).

config.json keys read here: architecture, vocab, width, norm.eps,
residual_mult, layers[].{type, mixer, mlp}.
Checkpoint tensor names: embed, l<i>.norm1, l<i>.norm1b, l<i>.norm2,
l<i>.norm2b, l<i>.mix.*, l<i>.mlp.{up,down,act}, final.norm.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from dynamo_amd.engine.config import ModelConfig
from dynamo_amd.ops import seq as sops
from .layers import AttnMetadata, TPContext
from .mixers import (DifferentialAttention, LatentAttention, MixContext,
                     RGLRUMixer, XIELUMLP, _Init, _put)


def config_from_json(hf: dict, name: str = "fironex") -> ModelConfig:
    return ModelConfig(
        name=name, arch="fironex", hidden_size=hf["width"],
        vocab_size=hf["vocab"], num_layers=len(hf["layers"]),
        rms_eps=float(hf["norm"]["eps"]), layer_specs=hf["layers"],
        residual_mult=float(hf.get("residual_mult", 1.0)),
        tie_embeddings=True, norm="layernorm",
        # the uniform-attention fields do not apply; keep them inert
        intermediate_size=0, num_q_heads=1, num_kv_heads=1, head_dim=1)


def build_mixer(kind: str, m: dict, width: int, eps: float, init: _Init):
    if kind == "rglru":
        return RGLRUMixer(width, m["width"], m["blocks"], m["conv"], init)
    if kind == "attention":
        return DifferentialAttention(
            width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"],
            m["diff"], m["rot"], (m.get("mask") or {}).get("size"), eps, init)
    if kind == "latent_attention":
        return LatentAttention(
            width, m["heads"], m["dim"], m["rot_dim"], m["vdim"],
            m["kv_rank"], m["scale"], m["rot"], eps, init,
            shared_cache=m.get("kv_from") is not None)
    raise ValueError(f"unknown Fironex layer type {kind!r}")


class FironexLayer(torch.nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, init: _Init):
        super().__init__()
        self.norm1 = init.vec(width, 0.8, 1.2)
        self.norm1b = init.vec(width, 0.8, 1.2)
        self.mixer = build_mixer(spec["type"], spec["mixer"], width, eps, init)
        self.kv_from = (spec["mixer"].get("kv_from")
                        if spec["type"] == "latent_attention" else None)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            self.norm2 = init.vec(width, 0.8, 1.2)
            self.norm2b = init.vec(width, 0.8, 1.2)
            self.mlp = XIELUMLP(width, mlp["ff"], init)


class FironexForCausalLM(torch.nn.Module):
    needs_seq_batch = True       # the runner builds SeqBatch descriptors

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16,
                 tp: Optional[TPContext] = None, seed: int = 0):
        super().__init__()
        self.cfg = cfg
        self.tp = tp or TPContext()
        if self.tp.size != 1:
            raise ValueError("Fironex runs with tensor-parallel size 1")
        self.dtype = dtype
        self.eps = cfg.rms_eps
        self.mult = cfg.residual_mult
        gen = torch.Generator(device="cpu")
        gen.manual_seed(seed)
        init = _Init(device, dtype, gen)
        W = cfg.hidden_size
        self.embed = init.mat(cfg.vocab_size, W, std=0.5)
        self.layers = torch.nn.ModuleList(
            [FironexLayer(s, W, cfg.rms_eps, init) for s in cfg.layer_specs])
        self.final_norm = init.vec(W, 0.8, 1.2)
        for i, layer in enumerate(self.layers):
            j = layer.kv_from
            if j is None:
                continue
            src = self.layers[j].mixer if 0 <= j < i else None
            me = layer.mixer
            if (not isinstance(src, LatentAttention) or src.shared_cache
                    or (src.rank, src.rd) != (me.rank, me.rd)
                    or not torch.equal(src.freqs, me.freqs)):
                raise ValueError(
                    f"layer {i}: kv_from must name an earlier latent layer "
                    "with a cache of its own and the same latent sizes and "
                    "rotation")

    # -- what the engine must hold ------------------------------------
    def kv_layer_shapes(self):
        """Per layer: (kv_heads, key_row, value_row) or None."""
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
        _put(self.final_norm, get("final.norm"))
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            _put(layer.norm1, get(p + "norm1"))
            _put(layer.norm1b, get(p + "norm1b"))
            layer.mixer.load(lambda n, p=p: get(p + "mix." + n))
            if layer.mlp is not None:
                _put(layer.norm2, get(p + "norm2"))
                _put(layer.norm2b, get(p + "norm2b"))
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
        x = sops.embed_scale_pos(input_ids, meta.positions, self.embed, None,
                                 1.0)
        if meta.inputs_embeds is not None:
            x = x.index_copy(0, meta.embeds_rows, meta.inputs_embeds.float())
        # a sublayer's output waits here until the next norm call, which
        # post-norms it, adds it to the residual and norms the sum in one pass
        delta, post = None, None

        def norm(w):
            return sops.residual_layernorm(x, delta, post, self.mult, w,
                                           self.eps, self.dtype)
        for i, layer in enumerate(self.layers):
            h = norm(layer.norm1)
            src = i if layer.kv_from is None else layer.kv_from
            has_kv = self.layers[src].mixer.kv_shape() is not None
            own_v = layer.mixer.kv_shape() is not None and \
                layer.mixer.kv_shape()[2] > 0
            ctx = MixContext(sb, meta.positions, meta.slot_mapping,
                             states.layer(i),
                             kv_pool.kcache(src) if has_kv else None,
                             kv_pool.vcache(src) if own_v else None)
            delta, post = layer.mixer.forward(h, ctx), layer.norm1b
            if layer.mlp is not None:
                h = norm(layer.norm2)
                delta, post = layer.mlp.forward(h), layer.norm2b
            if tap is not None:     # residual after the layer (diagnostics)
                norm(None)
                delta, post = None, None
                tap.append(x.clone())
        return norm(self.final_norm)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.embed).float()
