"""Muzulorn: a decoder-only LM whose config lists its layers, each with one
of three mixers - grouped-query attention with a soft cap and a learned bias
by bucketed distance ('attention', optionally reading the keys and values of
an earlier layer), attention over a compressed latent under a sliding window
with a softmax sink ('latent_attention'), or a state-space mixer ('mamba2') -
and an optional feed-forward: dense GELU, or routed gated experts with a
gated shared expert.

The residual is fp32 and may be several parallel streams joined by learned
hyper-connections: a sublayer reads a weighted sum of the streams, RMS-normed
with a weight stored as an offset from one, and its output, times the
config's residual multiplier, is written to every stream with a weight of
its own while a small matrix mixes the old streams. The token embedding gets
a second row added from a table indexed by a hash of the previous and the
current token, so the previous token is part of a sequence's state.

The engine holds, per sequence slot, the previous token, a state-space
layer's matrix state and convolution tail, and in its paged cache the normed
keys and values of an attention layer or the latent rows of a latent layer.

config.json keys read here: architecture, vocab, width, norm.eps,
residual_mult, streams, embedding.bigram.{buckets, mul_prev, mul_cur},
layers[].{type, mixer, mlp}.
Checkpoint tensor names: embed, bigram, l<i>.norm1, l<i>.norm2,
l<i>.hc<q>.{in, out, mix}, l<i>.mix.*, l<i>.mlp.*, final.norm, head.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from dynamo_amd.engine.config import ModelConfig
from dynamo_amd.ops import seq as sops
from .layers import AttnMetadata, TPContext
from .mixers import (CappedAttention, GeluMLP, LatentAttention, MixContext,
                     RoutedExperts, SSDMixer, _Init, _put)


def config_from_json(hf: dict, name: str = "muzulorn") -> ModelConfig:
    bigram = (hf.get("embedding") or {}).get("bigram")
    return ModelConfig(
        name=name, arch="muzulorn", hidden_size=hf["width"],
        vocab_size=hf["vocab"], num_layers=len(hf["layers"]),
        rms_eps=float(hf["norm"]["eps"]), layer_specs=hf["layers"],
        residual_mult=float(hf.get("residual_mult", 1.0)),
        residual_streams=int(hf.get("streams", 0)),
        pair_hash=dict(bigram) if bigram else None,
        tie_embeddings=False, norm="rmsnorm",
        # the uniform-attention fields do not apply; keep them inert
        intermediate_size=0, num_q_heads=1, num_kv_heads=1, head_dim=1)


def build_mixer(kind: str, m: dict, width: int, eps: float, init: _Init):
    shared = m.get("kv_from") is not None
    if kind == "attention":
        temp = m.get("q_temp") or {}
        return CappedAttention(
            width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"],
            eps, init, temp_coef=temp.get("coef", 0.0),
            temp_every=temp.get("every", 1), softcap=m.get("softcap", 0.0),
            # a checkpoint's table brings its own row count
            buckets=m.get("buckets", 32) if "bias_max" in m else 0,
            bias_max=m.get("bias_max", 0), shared_cache=shared)
    if kind == "latent_attention":
        return LatentAttention(
            width, m["heads"], m["dim"], m["rot_dim"], m["vdim"],
            m["kv_rank"], m["scale"], m["rot"], eps, init,
            shared_cache=shared, interleaved=True, q_rank=m.get("q_rank"),
            window=(m.get("mask") or {}).get("size"), sink=True,
            gate="element")
    if kind == "mamba2":
        return SSDMixer(width, m["heads"], m["vdim"], m["state"], m["groups"],
                        m["norm_groups"], m["conv"], eps, init)
    raise ValueError(f"unknown Muzulorn layer type {kind!r}")


def build_mlp(mlp: dict, width: int, init: _Init):
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return GeluMLP(width, mlp["ff"], init)
    if kind == "moe":
        r = mlp["router"]
        shared = mlp.get("shared") or {}
        return RoutedExperts(
            width, r["experts"], mlp["expert"]["ff"], r["top"], 1.0, 0, 1, 1,
            shared.get("ff"), init, glu=True, route="topk_logits",
            shared_gate=bool(shared))
    raise ValueError(f"unknown feed-forward kind {kind!r}")


class HyperConnection(torch.nn.Module):
    """Weights of one sublayer on S residual streams: read weights [S],
    write weights [S] and the stream mixing matrix [from, to]. The identity
    setting (S = 1) is the plain residual sum."""

    def __init__(self, streams: int, init: _Init):
        super().__init__()
        S = max(streams, 1)
        dev = init.device
        if streams:
            self.read = init.vec(S, 0.3, 0.9)
            self.write = init.vec(S, 0.5, 1.2)
            self.mix = (torch.eye(S, device=dev)
                        + init.vec((S, S), -0.15, 0.15))
        else:
            self.read = torch.ones(1, device=dev)
            self.write = torch.ones(1, device=dev)
            self.mix = torch.ones(1, 1, device=dev)

    def load(self, get):
        _put(self.read, get("in"))
        _put(self.write, get("out"))
        _put(self.mix, get("mix"))


class MuzulornLayer(torch.nn.Module):
    def __init__(self, spec: dict, width: int, streams: int, eps: float,
                 init: _Init):
        super().__init__()
        self.norm1 = init.vec(width, -0.2, 0.2)
        self.hc1 = HyperConnection(streams, init)
        self.mixer = build_mixer(spec["type"], spec["mixer"], width, eps, init)
        self.kv_from = spec["mixer"].get("kv_from")
        self.mlp = None
        if spec.get("mlp"):
            self.norm2 = init.vec(width, -0.2, 0.2)
            self.hc2 = HyperConnection(streams, init)
            self.mlp = build_mlp(spec["mlp"], width, init)


class MuzulornForCausalLM(torch.nn.Module):
    needs_seq_batch = True       # the runner builds SeqBatch descriptors

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16,
                 tp: Optional[TPContext] = None, seed: int = 0):
        super().__init__()
        self.cfg = cfg
        self.tp = tp or TPContext()
        if self.tp.size != 1:
            raise ValueError("Muzulorn runs with tensor-parallel size 1")
        self.dtype = dtype
        self.eps = cfg.rms_eps
        self.mult = cfg.residual_mult
        self.streams = int(cfg.residual_streams)
        self.S = max(self.streams, 1)
        gen = torch.Generator(device="cpu")
        gen.manual_seed(seed)
        init = _Init(device, dtype, gen)
        W = cfg.hidden_size
        if cfg.vocab_size >= 1 << 24:
            raise ValueError("the previous token is held as an fp32 number")
        self.embed = init.mat(cfg.vocab_size, W, std=0.5)
        self.pair = cfg.pair_hash
        self.pair_table = None
        if self.pair:
            self.pair_table = init.mat(int(self.pair["buckets"]) + 1, W,
                                       std=0.3)
        self.layers = torch.nn.ModuleList(
            [MuzulornLayer(s, W, self.streams, cfg.rms_eps, init)
             for s in cfg.layer_specs])
        self.final_norm = init.vec(W, -0.2, 0.2)
        self.head = init.mat(cfg.vocab_size, W)
        self.ones = torch.ones(self.S, device=device)
        for i, layer in enumerate(self.layers):
            j = layer.kv_from
            if j is None:
                continue
            src = self.layers[j].mixer if 0 <= j < i else None
            me = layer.mixer
            ok = (type(src) is type(me) and src.kv_shape() is not None)
            if ok and isinstance(me, CappedAttention):
                ok = (src.G, src.dk, src.dv) == (me.G, me.dk, me.dv)
            elif ok:
                ok = ((src.rank, src.rd) == (me.rank, me.rd)
                      and torch.equal(src.freqs, me.freqs))
            if not ok:
                raise ValueError(
                    f"layer {i}: kv_from must name an earlier layer of the "
                    "same kind with a cache of its own and the same key and "
                    "value sizes")

    # -- what the engine must hold ------------------------------------
    def kv_layer_shapes(self):
        """Per layer: (kv_heads, key_row, value_row) or None."""
        return [l.mixer.kv_shape() for l in self.layers]

    def state_layer_shapes(self):
        """Per layer: list of per-slot fp32 state shapes; one more entry at
        the end holds the embedding's previous token."""
        return [l.mixer.state_shapes() for l in self.layers] + \
            [[(1,)] if self.pair else []]

    # -- weights --------------------------------------------------------
    def load_checkpoint(self, path: str) -> int:
        from .loader import _iter_safetensors
        tensors = dict(_iter_safetensors(path))
        used = set()

        def get(name):
            used.add(name)
            return tensors[name]
        _put(self.embed, get("embed"))
        if self.pair:
            _put(self.pair_table, get("bigram"))
        _put(self.final_norm, get("final.norm"))
        _put(self.head, get("head"))
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            _put(layer.norm1, get(p + "norm1"))
            if self.streams:
                layer.hc1.load(lambda n, p=p: get(p + "hc1." + n))
            layer.mixer.load(lambda n, p=p: get(p + "mix." + n))
            if layer.mlp is not None:
                _put(layer.norm2, get(p + "norm2"))
                if self.streams:
                    layer.hc2.load(lambda n, p=p: get(p + "hc2." + n))
                layer.mlp.load(lambda n, p=p: get(p + "mlp." + n))
        extra = set(tensors) - used
        # a layer without feed-forward has no use for a second norm or
        # connection, should a checkpoint carry them
        extra -= {f"l{i}.{n}" for i, layer in enumerate(self.layers)
                  if layer.mlp is None
                  for n in ("norm2", "hc2.in", "hc2.out", "hc2.mix")}
        if extra:
            raise ValueError(f"checkpoint tensors not consumed: {sorted(extra)}")
        return len(used)

    # -- forward ----------------------------------------------------------
    def forward(self, input_ids, kv_pool, meta: AttnMetadata,
                tap: Optional[list] = None):
        sb = meta.seq_batch
        states = meta.state_pool
        if self.pair:
            x = sops.embed_pair_hash(
                input_ids, self.embed, self.pair_table,
                int(self.pair["mul_prev"]), int(self.pair["mul_cur"]),
                states.layer(len(self.layers))[0], sb)
        else:
            x = sops.embed_scale_pos(input_ids, meta.positions, self.embed,
                                     None, 1.0)
        if meta.inputs_embeds is not None:
            x = x.index_copy(0, meta.embeds_rows, meta.inputs_embeds.float())
        T, W = x.shape
        xs = x.unsqueeze(1).expand(T, self.S, W).contiguous()
        # a sublayer's output waits here until the next read, which writes
        # it to the streams and forms the next sublayer's input in one pass
        delta, hc = None, None

        def step(nxt, w):
            return sops.stream_step(
                xs, delta, hc.mix if hc else None, hc.write if hc else None,
                self.mult, nxt, w, self.eps, self.dtype)
        for i, layer in enumerate(self.layers):
            h = step(layer.hc1.read, layer.norm1)
            src = i if layer.kv_from is None else layer.kv_from
            shape = self.layers[src].mixer.kv_shape()
            ctx = MixContext(sb, meta.positions, meta.slot_mapping,
                             states.layer(i),
                             kv_pool.kcache(src) if shape else None,
                             kv_pool.vcache(src) if shape and shape[2] else None)
            delta, hc = layer.mixer.forward(h, ctx), layer.hc1
            if layer.mlp is not None:
                h = step(layer.hc2.read, layer.norm2)
                delta, hc = layer.mlp.forward(h), layer.hc2
            if tap is not None:     # sum of the streams after the layer
                tap.append(step(self.ones, None).clone())
                delta, hc = None, None
        return step(self.ones, self.final_norm)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.head).float()
