"""Kefesun: a decoder-only LM whose config lists its layers, each with one
of two mixers - attention with unnormalised sigmoid weights under a sliding
window that keeps the first tokens ('attention'), or a minimal gated
recurrent unit ('mingru') - and an optional mixture-of-experts feed-forward.

The residual stream is fp32. A sublayer reads the stream itself, passed
through a short causal per-channel convolution over time that is added to
its input (h = x + conv(x)); only the sublayer's output is normed, with a
weight-only layer norm: x <- x + LN(sublayer(h)). The token embedding is
scaled; logits use the unscaled embedding table after a final layer norm.

The engine holds, per layer and sequence slot, the last taps - 1 rows of x
that each of the two convolutions has seen, the recurrent state of a mingru
layer, and the paged keys/values of an attention layer.

config.json keys read here: architecture, vocab, width, norm.eps,
embedding.scale, canon.taps, layers[].{type, mixer, mlp}.
Checkpoint tensor names: embed, l<i>.canon1, l<i>.canon2, l<i>.norm1,
l<i>.norm2, l<i>.mix.*, l<i>.mlp.*, final.norm.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from dynamo_amd.engine.config import ModelConfig
from dynamo_amd.ops import seq as sops
from .layers import AttnMetadata, TPContext
from .mixers import (MinGRUMixer, MixContext, RoutedExperts, SigmoidAttention,
                     _Init, _put)


def config_from_json(hf: dict, name: str = "kefesun") -> ModelConfig:
    return ModelConfig(
        name=name, arch="kefesun", hidden_size=hf["width"],
        vocab_size=hf["vocab"], num_layers=len(hf["layers"]),
        rms_eps=float(hf["norm"]["eps"]), layer_specs=hf["layers"],
        embed_scale=float((hf.get("embedding") or {}).get("scale", 1.0)),
        conv_taps=int((hf.get("canon") or {}).get("taps", 0)),
        tie_embeddings=True, norm="layernorm",
        # the uniform-attention fields do not apply; keep them inert
        intermediate_size=0, num_q_heads=1, num_kv_heads=1, head_dim=1)


def build_mixer(kind: str, m: dict, width: int, eps: float, init: _Init):
    if kind == "attention":
        mask = m.get("mask") or {}
        return SigmoidAttention(
            width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"],
            m.get("rot"), mask.get("size"), mask.get("keep_first", 0), eps,
            init)
    if kind == "mingru":
        return MinGRUMixer(width, m["width"], init)
    raise ValueError(f"unknown Kefesun layer type {kind!r}")


def build_mlp(mlp: dict, width: int, init: _Init):
    if mlp.get("kind", "moe") != "moe":
        raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
    r = mlp["router"]
    grp = r.get("groups") or {}
    shared = mlp.get("shared") or {}
    return RoutedExperts(
        width, r["experts"], mlp["expert"]["ff"], r["top"],
        float(r.get("scale", 1.0)), int(r.get("identity", 0)),
        int(grp.get("count", 1)), int(grp.get("keep", 1)),
        shared.get("ff"), init)


class KefesunLayer(torch.nn.Module):
    def __init__(self, spec: dict, width: int, taps: int, eps: float,
                 init: _Init):
        super().__init__()
        self.canon1 = init.vec((width, taps), -0.3, 0.3) if taps else None
        self.mixer = build_mixer(spec["type"], spec["mixer"], width, eps, init)
        self.norm1 = init.vec(width, 0.8, 1.2)
        self.mlp = None
        if spec.get("mlp"):
            self.canon2 = init.vec((width, taps), -0.3, 0.3) if taps else None
            self.mlp = build_mlp(spec["mlp"], width, init)
            self.norm2 = init.vec(width, 0.8, 1.2)


class KefesunForCausalLM(torch.nn.Module):
    needs_seq_batch = True       # the runner builds SeqBatch descriptors

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16,
                 tp: Optional[TPContext] = None, seed: int = 0):
        super().__init__()
        self.cfg = cfg
        self.tp = tp or TPContext()
        if self.tp.size != 1:
            raise ValueError("Kefesun runs with tensor-parallel size 1")
        self.dtype = dtype
        self.eps = cfg.rms_eps
        self.taps = cfg.conv_taps
        gen = torch.Generator(device="cpu")
        gen.manual_seed(seed)
        init = _Init(device, dtype, gen)
        W = cfg.hidden_size
        self.embed = init.mat(cfg.vocab_size, W, std=W ** -0.5)
        self.layers = torch.nn.ModuleList(
            [KefesunLayer(s, W, self.taps, cfg.rms_eps, init)
             for s in cfg.layer_specs])
        self.final_norm = init.vec(W, 0.8, 1.2)

    # -- what the engine must hold ------------------------------------
    def kv_layer_shapes(self):
        """Per layer: (kv_heads, key_row, value_row) or None."""
        return [l.mixer.kv_shape() for l in self.layers]

    def state_layer_shapes(self):
        """Per layer: the convolution tails of its sublayers (rows of the
        residual stream), then the mixer's own state."""
        W, K = self.cfg.hidden_size, max(self.taps - 1, 0)
        return [[(K, W)] * (self._nconv(l)) + l.mixer.state_shapes()
                for l in self.layers]

    def _nconv(self, layer) -> int:
        if not self.taps:
            return 0
        return 2 if layer.mlp is not None else 1

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
            if self.taps:
                _put(layer.canon1, get(p + "canon1"))
            _put(layer.norm1, get(p + "norm1"))
            layer.mixer.load(lambda n, p=p: get(p + "mix." + n))
            if layer.mlp is not None:
                if self.taps:
                    _put(layer.canon2, get(p + "canon2"))
                _put(layer.norm2, get(p + "norm2"))
                layer.mlp.load(lambda n, p=p: get(p + "mlp." + n))
        extra = set(tensors) - used
        # a layer without feed-forward has no use for a second norm or
        # convolution, should a checkpoint carry them
        extra -= {f"l{i}.{n}" for i, layer in enumerate(self.layers)
                  if layer.mlp is None for n in ("norm2", "canon2")}
        if extra:
            raise ValueError(f"checkpoint tensors not consumed: {sorted(extra)}")
        return len(used)

    # -- forward ----------------------------------------------------------
    def forward(self, input_ids, kv_pool, meta: AttnMetadata,
                tap: Optional[list] = None):
        sb = meta.seq_batch
        states = meta.state_pool
        x = sops.embed_scale_pos(input_ids, meta.positions, self.embed, None,
                                 self.cfg.embed_scale)
        if meta.inputs_embeds is not None:
            x = x.index_copy(0, meta.embeds_rows, meta.inputs_embeds.float())

        def join(delta, w):     # x += LN(delta) * w
            sops.residual_layernorm(x, delta, w, 1.0, None, self.eps,
                                    self.dtype)

        def read(last, conv_w, tail):
            """The waiting sublayer output joins the stream; returns what
            the next sublayer reads: x + conv(x)."""
            delta, post = last if last is not None else (None, None)
            if conv_w is None:
                if delta is not None:
                    join(delta, post)
                return x.to(self.dtype)
            return sops.join_conv(x, delta, post, self.eps, conv_w, tail, sb,
                                  self.dtype)
        last = None     # (sublayer output, its norm weight) not yet joined
        for i, layer in enumerate(self.layers):
            st = states.layer(i)
            nconv = self._nconv(layer)
            h = read(last, layer.canon1, st[0] if nconv else None)
            shape = layer.mixer.kv_shape()
            ctx = MixContext(sb, meta.positions, meta.slot_mapping, st[nconv:],
                             kv_pool.kcache(i) if shape else None,
                             kv_pool.vcache(i) if shape else None)
            last = (layer.mixer.forward(h, ctx), layer.norm1)
            if layer.mlp is not None:
                h = read(last, layer.canon2, st[1] if nconv else None)
                last = (layer.mlp.forward(h), layer.norm2)
            if tap is not None:     # residual after the layer (diagnostics)
                join(*last)
                last = None
                tap.append(x.clone())
        delta, post = last if last is not None else (None, None)
        return sops.residual_layernorm(x, delta, post, 1.0, self.final_norm,
                                       self.eps, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.embed).float()
