"""Token mixers beyond rotary softmax attention: recurrent mixers with a
slot-addressed fp32 state (matrix memories, a gated linear unit), and
softmax attention over the paged cache with a distance bias / query
temperature / value norm, with differential heads under a sliding window,
or over a shared compressed latent; attention with unnormalised sigmoid
weights under a window that keeps the first tokens; a minimal gated
recurrent unit; and a routed mixture of small feed-forward experts.

Every mixer takes the normed hidden rows h [T, W] of the engine's flat
batch and a `MixContext` (sequence spans, state tensors of its layer, cache
views) and returns [T, W] in the activation dtype. Constants of a mechanism
are constructor parameters; sizes come from the weights' shapes.

Big projections are one fused GEMM where the inputs allow it (hipBLASLt via
F.linear); what follows them runs in the HIP kernels of ops.seq. Small
per-channel parameters are kept in fp32.

Each class declares what the engine must hold for it:
  state_shapes()  per-slot shapes of its recurrent state tensors (fp32)
  kv_shape()      (kv_heads, key_dim, value_dim) of its paged cache, or None
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional, Tuple

import torch
import torch.nn.functional as F

from dynamo_amd.ops import seq as sops


@dataclass
class MixContext:
    sb: "sops.SeqBatch"
    positions: torch.Tensor                 # [T] int32
    slot_mapping: torch.Tensor              # [T] int64 cache slots
    states: List[torch.Tensor]              # this layer's state tensors
    kcache: Optional[torch.Tensor] = None   # [P, G, ps, dk]
    vcache: Optional[torch.Tensor] = None   # [P, G, ps, dv]


class _Init:
    """Seeded random weights (benchmarks and tests run on random models)."""

    def __init__(self, device, dtype, gen):
        self.device, self.dtype, self.gen = device, dtype, gen

    def mat(self, out, inp, std=None):
        std = inp ** -0.5 if std is None else std
        w = torch.randn(out, inp, generator=self.gen, dtype=torch.float32) * std
        return w.to(self.dtype).to(self.device)

    def vec(self, shape, lo, hi):
        if isinstance(shape, int):
            shape = (shape,)
        w = torch.rand(*shape, generator=self.gen, dtype=torch.float32)
        return (lo + (hi - lo) * w).to(self.device)


Getter = Callable[[str], torch.Tensor]


def _put(dst: torch.Tensor, src: torch.Tensor):
    if tuple(dst.shape) != tuple(src.shape):
        raise ValueError(f"shape mismatch {tuple(dst.shape)} vs "
                         f"{tuple(src.shape)}")
    with torch.no_grad():
        dst.copy_(src.to(dst.dtype))


class GatedDeltaMixer(torch.nn.Module):
    """Gated delta rule with short causal convolutions on q, k, v.

    S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, with unit
    q/k per head, q scaled by dk^-1/2, g = exp(-exp(A_log) softplus(a + dt)).
    Output: per-head RMS norm (weight shared by heads) * silu(gate) -> W_o.
    """

    def __init__(self, width, heads, kv_heads, dim, vdim, conv, eps, init):
        super().__init__()
        self.W, self.H, self.G, self.dk, self.dv = width, heads, kv_heads, dim, vdim
        self.taps, self.eps = conv, eps
        self.Cq = kv_heads * dim
        self.Cv = heads * vdim
        self.Cc = 2 * self.Cq + self.Cv
        # fused rows: q | k | v | gate | beta | a
        self.off_g = self.Cc
        self.off_b = self.Cc + self.Cv
        self.off_a = self.off_b + heads
        self.w_in = init.mat(self.off_a + heads, width)
        self.conv_w = init.vec((self.Cc, conv), -0.6, 0.9)
        self.A_log = init.vec(heads, -4.0, -1.5)
        self.dt_bias = init.vec(heads, -3.2, -2.8)
        self.norm_w = init.vec(vdim, 0.7, 1.4)
        self.w_o = init.mat(width, self.Cv)

    def state_shapes(self):
        return [(self.H, self.dk, self.dv), (self.taps - 1, self.Cc)]

    def kv_shape(self):
        return None

    def load(self, get: Getter):
        rows = [get("q"), get("k"), get("v"), get("g"), get("b"), get("a")]
        _put(self.w_in, torch.cat(rows, 0))
        _put(self.conv_w, torch.cat([get("q.conv"), get("k.conv"),
                                     get("v.conv")], 0))
        _put(self.A_log, get("A_log"))
        _put(self.dt_bias, get("dt_bias"))
        _put(self.norm_w, get("norm"))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        proj = F.linear(h, self.w_in)
        S, conv_state = ctx.states
        qkv = sops.causal_conv_silu(proj, self.Cc, self.conv_w, conv_state,
                                    ctx.sb)
        o = sops.gated_delta_rule(qkv, proj, self.off_b, self.off_a,
                                  self.A_log, self.dt_bias, S, ctx.sb, self.H,
                                  self.G, self.dv, self.dk ** -0.5)
        y = sops.head_norm_gate(o, self.norm_w, 0, proj[:, self.off_g:],
                                sops.GATE_SILU, self.eps, h.dtype)
        return F.linear(y, self.w_o)


class BiasedAttention(torch.nn.Module):
    """Grouped-query softmax attention without rotation over the paged
    cache. Options: query temperature 1 + coef ln(floor((p+1)/every) + 1),
    RMS-normed values (cached normed), and a per-head distance penalty
    r1 ln(1 + r2 (i - j)) subtracted from the scaled scores."""

    def __init__(self, width, heads, kv_heads, dim, vdim, scale, eps, init,
                 temp_coef=0.0, temp_every=1, value_norm=True,
                 distance_bias=True):
        super().__init__()
        self.W, self.H, self.G, self.dk, self.dv = width, heads, kv_heads, dim, vdim
        self.scale, self.eps = scale, eps
        self.temp_coef, self.temp_every = temp_coef, temp_every
        self.value_norm = value_norm
        self.off_k = heads * dim
        self.off_v = self.off_k + kv_heads * dim
        self.w_in = init.mat(self.off_v + kv_heads * vdim, width)
        self.r1 = init.vec(heads, 0.0, 2.0) if distance_bias else None
        self.r2 = init.vec(heads, 0.1, 0.3) if distance_bias else None
        self.w_o = init.mat(width, heads * vdim)

    def state_shapes(self):
        return []

    def kv_shape(self):
        return (self.G, self.dk, self.dv)

    def load(self, get: Getter):
        _put(self.w_in, torch.cat([get("q"), get("k"), get("v")], 0))
        if self.r1 is not None:
            _put(self.r1, get("r1"))
            _put(self.r2, get("r2"))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        proj = F.linear(h, self.w_in)
        sops.kv_append_norm(ctx.kcache, ctx.vcache, proj, self.off_k,
                            self.off_v, ctx.slot_mapping, self.value_norm,
                            self.eps)
        y = sops.biased_attention(proj, 0, self.H, ctx.kcache, ctx.vcache,
                                  ctx.positions, ctx.sb, self.r1, self.r2,
                                  self.scale, self.temp_coef, self.temp_every)
        return F.linear(y, self.w_o)


class RWKVTimeMix(torch.nn.Module):
    """RWKV-style time mixing: token-shift interpolations feed r, k, v, gate
    and a low-rank data-dependent decay w = exp(-exp(W2 tanh(W1 x) + w0));
    o = (S + diag(u) k v^T)^T r; S <- diag(w) S + k v^T.
    Output: per-head RMS norm * weight * silu(gate) -> W_o."""

    SHIFTS = ("r", "k", "v", "g", "w")

    def __init__(self, width, heads, dim, eps, init, decay_rank=None):
        super().__init__()
        self.W, self.H, self.d, self.eps = width, heads, dim, eps
        HD = heads * dim
        rank = decay_rank or max(8, width // 16)
        self.mu = init.vec((5, width), 0.0, 0.8)
        # r, k, v, gate share a batched GEMM: [4, W, HD] (x @ w)
        self.w_rkvg = torch.stack(
            [init.mat(HD, width).t().contiguous() for _ in range(4)])
        self.w1 = init.mat(rank, width)
        self.w2 = init.mat(HD, rank, std=0.2)
        self.w0 = init.vec(HD, -6.0, -1.0)
        self.u = init.vec((heads, dim), -0.4, 1.4)
        self.norm_w = init.vec(HD, 0.6, 1.4)
        self.w_o = init.mat(width, HD)

    def state_shapes(self):
        return [(self.H, self.d, self.d), (self.W,)]

    def kv_shape(self):
        return None

    def load(self, get: Getter):
        _put(self.mu, torch.stack([get("mu." + s) for s in self.SHIFTS]))
        _put(self.w_rkvg, torch.stack([get(s).t() for s in "rkvg"]))
        if get("w1").shape != self.w1.shape:      # rank comes from the file
            self.w1 = torch.empty_like(get("w1"), dtype=self.w1.dtype,
                                       device=self.w1.device)
            self.w2 = torch.empty_like(get("w2"), dtype=self.w2.dtype,
                                       device=self.w2.device)
        _put(self.w1, get("w1"))
        _put(self.w2, get("w2"))
        _put(self.w0, get("w0"))
        _put(self.u, get("u"))
        _put(self.norm_w, get("norm"))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        S, prev = ctx.states
        mix = sops.token_shift_mix(h, self.mu, prev, ctx.sb)     # [5, T, W]
        rkvg = torch.bmm(mix[:4], self.w_rkvg)                   # [4, T, HD]
        wraw = F.linear(torch.tanh(F.linear(mix[4], self.w1)), self.w2)
        o = sops.rwkv_time_mix(rkvg[0], rkvg[1], rkvg[2], wraw, self.w0,
                               self.u, S, ctx.sb, self.H)
        y = sops.head_norm_gate(o, self.norm_w, self.d, rkvg[3],
                                sops.GATE_SILU, self.eps, h.dtype)
        return F.linear(y, self.w_o)


class MLSTMMixer(torch.nn.Module):
    """mLSTM matrix memory with exponential gating, soft-capped gate
    pre-activations and a running stabiliser that starts at 0.
    Output: per-head RMS norm * weight * sigmoid(gate) -> W_o."""

    def __init__(self, width, heads, dim, vdim, gate_cap, eps, init):
        super().__init__()
        self.W, self.H, self.dk, self.dv = width, heads, dim, vdim
        self.cap, self.eps = gate_cap, eps
        HK, HV = heads * dim, heads * vdim
        # fused rows: q | k | v | gate | i | f
        self.off_k, self.off_v, self.off_g = HK, 2 * HK, 2 * HK + HV
        self.off_i = self.off_g + HV
        self.off_f = self.off_i + heads
        self.w_in = init.mat(self.off_f + heads, width)
        self.i_bias = init.vec(heads, -1.0, 1.0)
        self.f_bias = init.vec(heads, 1.0, 6.0)
        self.norm_w = init.vec(HV, 0.6, 1.4)
        self.w_o = init.mat(width, HV)

    def state_shapes(self):
        return [(self.H, self.dk, self.dv), (self.H, self.dk), (self.H,)]

    def kv_shape(self):
        return None

    def load(self, get: Getter):
        _put(self.w_in, torch.cat([get("q"), get("k"), get("v"), get("g"),
                                   get("i"), get("f")], 0))
        _put(self.i_bias, get("i.b"))
        _put(self.f_bias, get("f.b"))
        _put(self.norm_w, get("norm"))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        proj = F.linear(h, self.w_in)
        S, n, m = ctx.states
        o = sops.mlstm_memory(
            proj, (0, self.off_k, self.off_v, self.off_i, self.off_f),
            self.i_bias, self.f_bias, S, n, m, ctx.sb, self.H, self.dv,
            self.dk ** -0.5, self.cap)
        y = sops.head_norm_gate(o, self.norm_w, self.dv, proj[:, self.off_g:],
                                sops.GATE_SIGMOID, self.eps, h.dtype)
        return F.linear(y, self.w_o)


class ParallelMixer(torch.nn.Module):
    """Two mixers on the same input; the result is the mean of their
    outputs, each RMS-normed over the width with its own weight."""

    def __init__(self, width, left, right, eps, init):
        super().__init__()
        self.left, self.right, self.eps = left, right, eps
        self.left_out = init.vec(width, 0.6, 1.3)
        self.right_out = init.vec(width, 0.6, 1.3)

    def state_shapes(self):
        return self.left.state_shapes() + self.right.state_shapes()

    def kv_shape(self):
        return self.left.kv_shape() or self.right.kv_shape()

    def load(self, get: Getter):
        self.left.load(lambda n: get("left." + n))
        self.right.load(lambda n: get("right." + n))
        _put(self.left_out, get("left.out"))
        _put(self.right_out, get("right.out"))

    def forward(self, h, ctx: MixContext):
        nl = len(self.left.state_shapes())
        cl = MixContext(ctx.sb, ctx.positions, ctx.slot_mapping,
                        ctx.states[:nl], ctx.kcache, ctx.vcache)
        cr = MixContext(ctx.sb, ctx.positions, ctx.slot_mapping,
                        ctx.states[nl:], ctx.kcache, ctx.vcache)
        a = self.left.forward(h, cl)
        b = self.right.forward(h, cr)
        return sops.dual_rmsnorm_mean(a, b, self.left_out, self.right_out,
                                      self.eps)


class ClampedGLU(torch.nn.Module):
    """Dense feed-forward: g = min(W_gate h, L); u = clamp(W_up h, -L, L);
    W_down (g sigmoid(alpha g) (u + 1))."""

    def __init__(self, width, ff, limit, init, alpha=1.702):
        super().__init__()
        self.limit, self.alpha = limit, alpha
        self.w_gate_up = init.mat(2 * ff, width)
        self.w_down = init.mat(width, ff)

    def load(self, get: Getter):
        _put(self.w_gate_up, torch.cat([get("gate"), get("up")], 0))
        _put(self.w_down, get("down"))

    def forward(self, h):
        act = sops.clamped_glu(F.linear(h, self.w_gate_up), self.limit,
                               self.alpha)
        return F.linear(act, self.w_down)


def rotary_frequencies(rot: dict) -> torch.Tensor:
    """fp32 [2, dims/2]: angular frequencies base^(-2i/dims) of a rotary
    spec {"base", "dims", "scaling"?} as float pairs (row 0 + row 1). The
    optional scaling {factor, low, high, original} slows long wavelengths
    (above original/low) by `factor`, keeps short ones (below
    original/high) and blends linearly in between. Evaluated in float64;
    the kernels form position * frequency in fp32 with the pair's low part
    and the product's rounding error as a correction."""
    import math
    n = int(rot["dims"])
    f = [float(rot["base"]) ** (-2.0 * i / n) for i in range(n // 2)]
    sc = rot.get("scaling")
    if sc:
        lo_wl = sc["original"] / sc["high"]
        hi_wl = sc["original"] / sc["low"]
        for i, fi in enumerate(f):
            wl = 2 * math.pi / fi
            if wl > hi_wl:
                f[i] = fi / sc["factor"]
            elif wl >= lo_wl:
                s = (sc["original"] / wl - sc["low"]) / (sc["high"] - sc["low"])
                f[i] = (1 - s) * fi / sc["factor"] + s * fi
    f64 = torch.tensor(f, dtype=torch.float64)
    hi = f64.to(torch.float32)
    lo = (f64 - hi.double()).to(torch.float32)
    return torch.stack([hi, lo])


class RGLRUMixer(torch.nn.Module):
    """Recurrent block around a real-gated linear recurrent unit: a gate
    branch gelu_tanh(W_y h + b_y) beside u = conv(W_x h + b_x) (short causal
    per-channel convolution with bias, no activation). Per channel, with
    block-diagonal gate matrices over `blocks` equal parts of u:
      r = sigmoid(A_r u + b_r), i = sigmoid(A_i u + b_i),
      a = exp(-decay r softplus(lam)), S <- a S + sqrt(1 - a^2) i u.
    Output W_o (S * gate branch). Gates and the recurrence run in fp32."""

    def __init__(self, width, channels, blocks, conv, init, decay=8.0):
        super().__init__()
        if channels % blocks:
            raise ValueError("recurrence width must divide into its blocks")
        self.W, self.C, self.nb, self.taps = width, channels, blocks, conv
        self.bw = channels // blocks
        self.decay = decay
        f32 = dict(dtype=torch.float32, device=init.device)
        # fused rows: x (convolved) | y (gate branch)
        self.w_in = init.mat(2 * channels, width)
        self.b_in = init.vec(2 * channels, -0.2, 0.2).to(init.dtype)
        self.conv_w = init.vec((channels, conv), -0.5, 0.8)
        self.conv_b = init.vec(channels, -0.2, 0.2)
        # gate matrices as x @ w per block: [nb, bw(in), 2 bw (r | i)]
        self.w_gates = (torch.randn(blocks, self.bw, 2 * self.bw,
                                    generator=init.gen) * self.bw ** -0.5
                        ).to(**f32)
        self.b_r = init.vec(channels, -0.5, 0.5)
        self.b_i = init.vec(channels, -0.5, 0.5)
        self.lam = init.vec(channels, -4.0, -1.0)
        self.w_o = init.mat(width, channels)

    def state_shapes(self):
        return [(self.C,), (self.taps - 1, self.C)]

    def kv_shape(self):
        return None

    def load(self, get: Getter):
        _put(self.w_in, torch.cat([get("x"), get("y")], 0))
        _put(self.b_in, torch.cat([get("x.b"), get("y.b")], 0))
        _put(self.conv_w, get("conv"))
        _put(self.conv_b, get("conv.b"))
        # checkpoint matrices are [block, out, in]
        _put(self.w_gates, torch.cat([get("ra").transpose(1, 2),
                                      get("ri").transpose(1, 2)], 2))
        _put(self.b_r, get("ra.b").reshape(-1))
        _put(self.b_i, get("ri.b").reshape(-1))
        _put(self.lam, get("lam"))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        T = h.shape[0]
        proj = F.linear(h, self.w_in, self.b_in)
        S, conv_state = ctx.states
        u = sops.causal_conv(proj, self.C, self.conv_w, self.conv_b, False,
                             conv_state, ctx.sb)
        gates = torch.bmm(u.view(T, self.nb, self.bw).transpose(0, 1),
                          self.w_gates)
        y = sops.rglru_scan(u, gates, self.b_r, self.b_i, self.lam,
                            proj[:, self.C:], S, ctx.sb, self.decay, h.dtype)
        return F.linear(y, self.w_o)


class DifferentialAttention(torch.nn.Module):
    """Grouped-query attention whose heads each run two softmax maps over
    the same values and subtract them: o = a1 - lam a2, then a weightless
    RMS norm per head times (1 - diff) and an element-wise sigmoid output
    gate. lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff for the whole layer.
    Queries/keys of both maps are rotated (interleaved pairs, first
    rot.dims entries); an optional sliding window bounds the visible keys.
    The paged cache row of a kv head holds both maps' keys back to back."""

    def __init__(self, width, heads, kv_heads, dim, vdim, scale, diff, rot,
                 window, eps, init):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("query heads must be a multiple of kv heads")
        self.W, self.H, self.G, self.dk, self.dv = width, heads, kv_heads, dim, vdim
        self.scale, self.diff, self.eps = scale, diff, eps
        self.window = int(window or 0)
        self.off_k = heads * 2 * dim
        self.off_v = self.off_k + kv_heads * 2 * dim
        self.off_g = self.off_v + kv_heads * vdim
        # fused rows: q | k | v | gate
        self.w_in = init.mat(self.off_g + heads * vdim, width)
        self.freqs = rotary_frequencies(rot).to(init.device)
        if 2 * self.freqs.shape[1] > dim:
            raise ValueError("rotary dims exceed the head size")
        self.lq1, self.lk1 = init.vec(dim, -0.3, 0.3), init.vec(dim, -0.3, 0.3)
        self.lq2, self.lk2 = init.vec(dim, -0.3, 0.3), init.vec(dim, -0.3, 0.3)
        self.w_o = init.mat(width, heads * vdim)
        self.refresh()

    def refresh(self):
        """The layer's lambda from its four vectors (fp32)."""
        self.lam = (torch.exp((self.lq1 * self.lk1).sum())
                    - torch.exp((self.lq2 * self.lk2).sum())
                    + self.diff).reshape(1).float()

    def state_shapes(self):
        return []

    def kv_shape(self):
        return (self.G, 2 * self.dk, self.dv)

    def load(self, get: Getter):
        _put(self.w_in, torch.cat([get("q"), get("k"), get("v"), get("g")], 0))
        for n in ("lq1", "lk1", "lq2", "lk2"):
            _put(getattr(self, n), get(n))
        _put(self.w_o, get("o"))
        self.refresh()

    def forward(self, h, ctx: MixContext):
        proj = F.linear(h, self.w_in)
        # q and k of both maps are 2H + 2G vectors of dk, back to back
        sops.rope_rows(proj, 0, self.dk, proj, 0, self.dk, ctx.positions,
                       self.freqs, 2 * (self.H + self.G), self.dk, True)
        sops.kv_append_norm(ctx.kcache, ctx.vcache, proj, self.off_k,
                            self.off_v, ctx.slot_mapping, False, self.eps)
        a = sops.paged_attention_rows(proj, 0, self.H, 2, ctx.kcache,
                                      ctx.vcache, self.dv, ctx.positions,
                                      ctx.sb, self.scale, self.window)
        y = sops.diff_norm_gate(a, self.lam, 1.0 - self.diff,
                                proj[:, self.off_g:], self.eps, h.dtype)
        return F.linear(y, self.w_o)


class LatentAttention(torch.nn.Module):
    """Causal attention over a compressed cache: per token only an
    RMS-normed latent c [rank] and one rotated key part [rot_dim] shared by
    all heads are stored. Head keys W_uk c and values W_uv c are never
    materialised: W_uk is folded into the query and W_uv applied to the
    attention-weighted latent, so the kernel runs as multi-query attention
    whose values are the first `rank` entries of the cached rows. With
    shared_cache the layer has no down-projection of its own and reads
    another latent layer's cache.

    Options: rotation pairs (i, i + dims/2) or interleaved (2i, 2i + 1)
    over the rot_dim part; queries projected directly or through an
    RMS-normed latent of q_rank entries (W_uq norm(W_dq h)); a sliding
    window; a per-head sink in the softmax denominator; the output gate
    sigmoid(W_g h) one value per head ("head", applied before W_uv, with
    which it commutes) or one per output channel ("element", applied to the
    concatenated heads)."""

    def __init__(self, width, heads, dim, rot_dim, vdim, rank, scale, rot, eps,
                 init, shared_cache=False, interleaved=False, q_rank=None,
                 window=None, sink=False, gate="head"):
        super().__init__()
        if gate not in ("head", "element"):
            raise ValueError(f"unknown output gate {gate!r}")
        self.W, self.H, self.dk, self.rd, self.dv = width, heads, dim, rot_dim, vdim
        self.rank, self.scale, self.eps = rank, scale, eps
        self.shared_cache = shared_cache
        self.interleaved, self.gate = interleaved, gate
        self.q_rank = int(q_rank or 0)
        self.window = int(window or 0)
        self.freqs = rotary_frequencies(rot).to(init.device)
        if 2 * self.freqs.shape[1] > rot_dim:
            raise ValueError("rotary dims exceed the rotated part")
        nq = heads * (dim + rot_dim)
        self.off_z = self.q_rank or nq
        self.off_g = self.off_z + (0 if shared_cache else rank + rot_dim)
        ng = heads if gate == "head" else heads * vdim
        # fused rows: q (or its latent) | [latent down-projection] | gate
        self.w_in = init.mat(self.off_g + ng, width)
        self.dq_norm = self.w_uq = None
        if self.q_rank:
            self.dq_norm = init.vec(self.q_rank, 0.7, 1.3)
            self.w_uq = init.mat(nq, self.q_rank)
        self.dkv_norm = None if shared_cache else init.vec(rank, 0.7, 1.3)
        self.w_uk = torch.stack([init.mat(dim, rank) for _ in range(heads)])
        self.w_uv_t = torch.stack([init.mat(vdim, rank).t().contiguous()
                                   for _ in range(heads)])
        self.sink = init.vec(heads, -1.0, 1.0) if sink else None
        self.w_o = init.mat(width, heads * vdim)

    def state_shapes(self):
        return []

    def kv_shape(self):
        return None if self.shared_cache else (1, self.rank + self.rd, 0)

    def load(self, get: Getter):
        rows = [get("dq") if self.q_rank else get("q")]
        rows += [] if self.shared_cache else [get("dkv")]
        _put(self.w_in, torch.cat(rows + [get("g")], 0))
        if self.q_rank:
            _put(self.dq_norm, get("dq.norm"))
            _put(self.w_uq, get("uq"))
        if not self.shared_cache:
            _put(self.dkv_norm, get("dkv.norm"))
        _put(self.w_uk, get("uk").view(self.H, self.dk, self.rank))
        _put(self.w_uv_t, get("uv").view(self.H, self.dv,
                                         self.rank).transpose(1, 2))
        if self.sink is not None:
            _put(self.sink, get("sink"))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        T, H, R, rd = h.shape[0], self.H, self.rank, self.rd
        proj = F.linear(h, self.w_in)
        if not self.shared_cache:
            sops.latent_append(ctx.kcache, proj, self.off_z, self.dkv_norm,
                               ctx.slot_mapping, ctx.positions, self.freqs,
                               self.interleaved, self.eps)
        if self.q_rank:
            cq = sops.rms_norm_cols(proj, 0, self.q_rank, self.dq_norm,
                                    self.eps, h.dtype)
            qsrc = F.linear(cq, self.w_uq)
        else:
            qsrc = proj
        qh = qsrc[:, :H * (self.dk + rd)].view(T, H, self.dk + rd)
        q = torch.empty(T, H * (R + rd), dtype=h.dtype, device=h.device)
        q.view(T, H, R + rd)[:, :, :R].copy_(
            torch.bmm(qh[:, :, :self.dk].transpose(0, 1),
                      self.w_uk).transpose(0, 1))
        sops.rope_rows(q, R, R + rd, qsrc, self.dk, self.dk + rd,
                       ctx.positions, self.freqs, H, rd, self.interleaved)
        lat = sops.paged_attention_rows(q, 0, H, 1, ctx.kcache, None, R,
                                        ctx.positions, ctx.sb, self.scale,
                                        self.window, sink=self.sink)
        if self.gate == "head":
            g = sops.head_sigmoid_scale(lat.view(T, H, R),
                                        proj[:, self.off_g:], h.dtype)
            o = torch.bmm(g, self.w_uv_t)                   # [H, T, dv]
            y = o.transpose(0, 1).reshape(T, H * self.dv)
        else:
            o = torch.bmm(sops.heads_major(lat.view(T, H, R), h.dtype),
                          self.w_uv_t)
            y = sops.heads_gate(o, proj[:, self.off_g:], h.dtype)
        return F.linear(y, self.w_o)


class XIELUMLP(torch.nn.Module):
    """Dense feed-forward W_down xIELU(W_up h) with the activation's two raw
    parameters (softplus-ed inside the kernel)."""

    def __init__(self, width, ff, init):
        super().__init__()
        self.w_up = init.mat(ff, width)
        self.w_down = init.mat(width, ff)
        self.act = init.vec(2, -1.0, 1.0)

    def load(self, get: Getter):
        _put(self.w_up, get("up"))
        _put(self.w_down, get("down"))
        _put(self.act, get("act"))

    def forward(self, h):
        return F.linear(sops.xielu(F.linear(h, self.w_up), self.act),
                        self.w_down)


class SigmoidAttention(torch.nn.Module):
    """Grouped-query attention whose weight of a visible key is
    sigmoid(scale q.k + b_h), not normalised over the keys. q, k, v carry
    biases; q and k are RMS-normed per head (one weight of the head size for
    all heads), then rotated over their first rot.dims entries (pairs
    (i, i + dims/2), or interleaved). Row i sees key j <= i when
    i - j < window or j < keep_first; window None = every earlier key."""

    def __init__(self, width, heads, kv_heads, dim, vdim, scale, rot, window,
                 keep_first, eps, init, interleaved=False, sigmoid=True):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("query heads must be a multiple of kv heads")
        self.W, self.H, self.G, self.dk, self.dv = width, heads, kv_heads, dim, vdim
        self.scale, self.eps = scale, eps
        self.window, self.keep_first = int(window or 0), int(keep_first or 0)
        self.interleaved, self.sigmoid = interleaved, sigmoid
        self.off_k = heads * dim
        self.off_v = self.off_k + kv_heads * dim
        # fused rows: q | k | v, each with its bias
        self.w_in = init.mat(self.off_v + kv_heads * vdim, width)
        self.b_in = init.vec(self.off_v + kv_heads * vdim, -0.2, 0.2).to(
            init.dtype)
        self.q_norm = init.vec(dim, 0.7, 1.3)
        self.k_norm = init.vec(dim, 0.7, 1.3)
        self.freqs = None
        if rot:
            self.freqs = rotary_frequencies(rot).to(init.device)
            if 2 * self.freqs.shape[1] > dim:
                raise ValueError("rotary dims exceed the head size")
        self.head_bias = init.vec(heads, -3.0, -1.0)
        self.w_o = init.mat(width, heads * vdim)

    def state_shapes(self):
        return []

    def kv_shape(self):
        return (self.G, self.dk, self.dv)

    def load(self, get: Getter):
        _put(self.w_in, torch.cat([get("q"), get("k"), get("v")], 0))
        _put(self.b_in, torch.cat([get("q.b"), get("k.b"), get("v.b")], 0))
        _put(self.q_norm, get("q.norm"))
        _put(self.k_norm, get("k.norm"))
        _put(self.head_bias, get("pb"))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        proj = F.linear(h, self.w_in, self.b_in)
        sops.headnorm_rope_append(
            proj, self.H, self.G, self.dk, self.dv, self.off_k, self.off_v,
            self.q_norm, self.k_norm, self.freqs, self.interleaved, self.eps,
            ctx.positions, ctx.kcache, ctx.vcache, ctx.slot_mapping)
        y = sops.paged_attention_rows(
            proj, 0, self.H, 1, ctx.kcache, ctx.vcache, self.dv,
            ctx.positions, ctx.sb, self.scale, self.window, self.keep_first,
            self.head_bias, self.sigmoid, out_dtype=h.dtype)
        return F.linear(y.view(h.shape[0], self.H * self.dv), self.w_o)


class MinGRUMixer(torch.nn.Module):
    """Minimal gated recurrent unit: gate z = sigmoid(W_z h + b_z) and
    candidate c(W_x h + b_x) read the current token only (c(u) = u + 1/2 for
    u >= 0, sigmoid(u) below); S <- (1 - z) S + z c per channel in fp32;
    output W_o (S * silu(W_g h))."""

    def __init__(self, width, channels, init):
        super().__init__()
        self.W, self.C = width, channels
        # fused rows: z | x | g (the output gate has no bias)
        self.w_in = init.mat(3 * channels, width)
        self.b_in = torch.cat([init.vec(2 * channels, -0.5, 0.5),
                               torch.zeros(channels, device=init.device)]
                              ).to(init.dtype)
        self.w_o = init.mat(width, channels)

    def state_shapes(self):
        return [(self.C,)]

    def kv_shape(self):
        return None

    def load(self, get: Getter):
        _put(self.w_in, torch.cat([get("z"), get("x"), get("g")], 0))
        b = torch.cat([get("z.b"), get("x.b")], 0)
        _put(self.b_in, torch.cat([b, torch.zeros(self.C, dtype=b.dtype)], 0))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        proj = F.linear(h, self.w_in, self.b_in)
        y = sops.mingru_scan(proj, self.C, ctx.states[0], ctx.sb, h.dtype)
        return F.linear(y, self.w_o)


class RoutedExperts(torch.nn.Module):
    """Mixture of feed-forward experts without biases, W_down relu(W_up h)^2
    or, with `glu`, W_down (silu(W_gate h) * W_up h). The router is fp32.

    route = "corrected_softmax": all router outputs are scored with a
    softmax; the `top` outputs with the largest corrected scores are chosen,
    among the `keep` best of `groups` equal groups of neighbouring outputs;
    the chosen ones weigh in with their uncorrected score times `scale`.
    route = "topk_logits": the `top` largest logits (router product plus a
    bias) are chosen and weigh in with the softmax over the chosen logits.

    The last `identity` router outputs are identity experts (output =
    input). A shared expert of the same form, when present, runs for every
    token; with `shared_gate` it is multiplied by sigmoid(w_sg . h), one
    value per token (w_sg is kept as one more row of the router matrix).

    Chosen (token, expert) pairs get a row of a gathered batch - expert e
    owns rows base[e] + rank - so that each expert is one GEMM over its
    rows: per expert when the counts are read on the host (prompts), or one
    batched GEMM over fixed-capacity blocks without any host read (few
    rows: decoding, graph capture)."""

    PADDED_MAX_ROWS = 64

    def __init__(self, width, experts, ff, top, scale, identity, groups, keep,
                 shared_ff, init, glu=False, route="corrected_softmax",
                 shared_gate=False):
        super().__init__()
        n = experts + identity
        if route not in ("corrected_softmax", "topk_logits"):
            raise ValueError(f"unknown router {route!r}")
        if n % groups or not 1 <= keep <= groups:
            raise ValueError("router outputs must divide into their groups")
        if top > keep * (n // groups):
            raise ValueError("more experts per token than the kept groups hold")
        if shared_gate and (route != "topk_logits" or not shared_ff):
            raise ValueError("a gated shared expert needs the logit router "
                             "and a shared expert")
        self.W, self.E, self.n, self.ff = width, experts, n, ff
        self.top, self.scale = top, scale
        self.groups, self.keep = groups, keep
        self.glu, self.route, self.shared_gate = glu, route, shared_gate
        self.act = sops.silu_glu if glu else sops.relu_squared
        up = 2 * ff if glu else ff
        f32 = dict(dtype=torch.float32, device=init.device)
        self.router = (torch.randn(n + (1 if shared_gate else 0), width,
                                   generator=init.gen)
                       * width ** -0.5).to(**f32)
        # per-output constant: correction of the choice, or logit bias
        self.correction = init.vec(n, -0.05, 0.05)
        self.w_up = torch.stack([init.mat(up, width) for _ in range(experts)])
        self.w_down = torch.stack([init.mat(width, ff) for _ in range(experts)])
        self.shared_up = self.shared_down = None
        if shared_ff:
            self.shared_up = init.mat(2 * shared_ff if glu else shared_ff,
                                      width)
            self.shared_down = init.mat(width, shared_ff)
        self._pad_base = {}

    def _up_rows(self, get, prefix):
        if self.glu:      # fused rows: gate | up
            return torch.cat([get(prefix + "gate"), get(prefix + "up")], 0)
        return get(prefix + "up")

    def load(self, get: Getter):
        if self.route == "topk_logits":
            rows = [get("router")] + ([get("shared.sg").reshape(1, -1)]
                                      if self.shared_gate else [])
            _put(self.router, torch.cat(rows, 0))
            _put(self.correction, get("router.b"))
        else:
            _put(self.router, get("router"))
            _put(self.correction, get("correction"))
        _put(self.w_up, torch.stack([self._up_rows(get, f"e{e}.")
                                     for e in range(self.E)]))
        _put(self.w_down,
             torch.stack([get(f"e{e}.down") for e in range(self.E)]))
        if self.shared_up is not None:
            _put(self.shared_up, self._up_rows(get, "shared."))
            _put(self.shared_down, get("shared.down"))

    def _padded_base(self, cap, device):
        key = (cap, str(device))
        if key not in self._pad_base:
            self._pad_base[key] = (torch.arange(self.n, dtype=torch.int32)
                                   * cap).to(device)
        return self._pad_base[key]

    def forward(self, h):
        T, E = h.shape[0], self.E
        sgate = None
        if self.route == "topk_logits":
            logits = F.linear(h.float(), self.router)
            idx, wgt = sops.moe_route_topk(logits, self.n, self.correction,
                                           self.top)
            if self.shared_gate:
                sgate = logits[:, self.n]
        else:
            idx, wgt = sops.moe_route_rows(h, self.router, self.correction,
                                           self.groups, self.keep, self.top,
                                           self.scale)
        rank, counts = sops.moe_dispatch(idx, self.n)
        if T <= self.PADDED_MAX_ROWS:
            # every expert gets a block of T rows: static shapes, no host read
            base = self._padded_base(T, h.device)
            xg = sops.moe_gather(h, idx, rank, base, E, E * T)
            a = self.act(torch.bmm(xg.view(E, T, self.W),
                                   self.w_up.transpose(1, 2)))
            y = torch.bmm(a, self.w_down.transpose(1, 2)).view(E * T, self.W)
        else:
            cnt = counts[:E].tolist()
            base = torch.zeros(E + 1, dtype=torch.int32, device=h.device)
            base[1:] = torch.cumsum(counts[:E], 0).to(torch.int32)
            rows = sum(cnt)
            xg = sops.moe_gather(h, idx, rank, base, E, rows)
            y = torch.empty(rows, self.W, dtype=h.dtype, device=h.device)
            r0 = 0
            for e, n in enumerate(cnt):
                if n:
                    a = self.act(F.linear(xg[r0:r0 + n], self.w_up[e]))
                    y[r0:r0 + n] = F.linear(a, self.w_down[e])
                r0 += n
        shared = None
        if self.shared_up is not None:
            shared = F.linear(self.act(F.linear(h, self.shared_up)),
                              self.shared_down)
        return sops.moe_combine(y, h, idx, wgt, rank, base, E, shared,
                                h.dtype, sgate)


def distance_bias_table(rel: torch.Tensor, max_dist: int) -> torch.Tensor:
    """fp32 [H, D + 1] from a bucketed table rel [B, H]: column n is the
    bias of key distance n (the last serves every distance >= D; a head's
    distances lie side by side, as a tile of scores reads them). Buckets:
    n itself below B // 2; from there logarithmic steps that reach the last
    bucket at distance D = max_dist:
    min(B - 1, B//2 + floor(ln(n / (B//2)) / ln(D / (B//2)) * (B - B//2)))."""
    import math
    B = rel.shape[0]
    half = B // 2
    rows = []
    for n in range(int(max_dist) + 1):
        if n < half:
            rows.append(n)
        else:
            rows.append(min(B - 1, half + int(math.floor(
                math.log(n / half) / math.log(max_dist / half) * (B - half)))))
    return rel.float()[torch.tensor(rows, dtype=torch.long,
                                    device=rel.device)].t().contiguous()


class CappedAttention(torch.nn.Module):
    """Grouped-query softmax attention without rotation, with biases on
    q, k, v and the output projection. q and k are RMS-normed over their
    whole projection (all heads at once, one weight per entry) before being
    split into heads; keys are cached normed. Options: a query temperature
    1 + coef ln(floor((p + 1) / every) + 1), a soft cap c tanh(s / c) on the
    scaled scores, and a learned bias by bucketed key distance (a table
    [buckets, heads], see distance_bias_table) added after the cap. With
    shared_cache the layer has no key/value projections and reads another
    layer's cached keys and values with its own queries."""

    def __init__(self, width, heads, kv_heads, dim, vdim, scale, eps, init,
                 temp_coef=0.0, temp_every=1, softcap=0.0, buckets=0,
                 bias_max=0, shared_cache=False):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("query heads must be a multiple of kv heads")
        self.W, self.H, self.G, self.dk, self.dv = width, heads, kv_heads, dim, vdim
        self.scale, self.eps = scale, eps
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.softcap, self.bias_max = float(softcap or 0.0), int(bias_max)
        self.shared_cache = shared_cache
        self.nq = heads * dim
        self.nk = 0 if shared_cache else kv_heads * dim
        self.nv = 0 if shared_cache else kv_heads * vdim
        self.off_k, self.off_v = self.nq, self.nq + self.nk
        # fused rows: q | k | v, each with its bias
        self.w_in = init.mat(self.off_v + self.nv, width)
        self.b_in = init.vec(self.off_v + self.nv, -0.2, 0.2).to(init.dtype)
        self.q_norm = init.vec(self.nq, 0.7, 1.3)
        self.k_norm = None if shared_cache else init.vec(self.nk, 0.7, 1.3)
        # random weights: no more buckets than the largest distance allows
        # (a checkpoint's table brings its own row count)
        while buckets > 2 and not self.bias_max > buckets // 2:
            buckets -= 1
        self.rel = init.vec((buckets, heads), -1.0, 1.0) if buckets else None
        self.w_o = init.mat(width, heads * vdim)
        self.b_o = init.vec(width, -0.2, 0.2).to(init.dtype)
        self.refresh()

    def refresh(self):
        """The bias by distance from the bucket table."""
        self.dist_bias = None
        if self.rel is not None:
            if not self.bias_max > self.rel.shape[0] // 2 >= 1:
                raise ValueError("the distance bias needs at least two "
                                 "buckets and a largest distance beyond the "
                                 "exact ones")
            self.dist_bias = distance_bias_table(self.rel, self.bias_max)

    def state_shapes(self):
        return []

    def kv_shape(self):
        return None if self.shared_cache else (self.G, self.dk, self.dv)

    def load(self, get: Getter):
        names = ["q"] + ([] if self.shared_cache else ["k", "v"])
        _put(self.w_in, torch.cat([get(n) for n in names], 0))
        _put(self.b_in, torch.cat([get(n + ".b") for n in names], 0))
        _put(self.q_norm, get("q.norm"))
        if not self.shared_cache:
            _put(self.k_norm, get("k.norm"))
        if self.rel is not None:
            rel = get("rel")
            if rel.shape != self.rel.shape:     # buckets come from the file
                self.rel = torch.empty(rel.shape, dtype=self.rel.dtype,
                                       device=self.rel.device)
            _put(self.rel, rel)
        _put(self.w_o, get("o"))
        _put(self.b_o, get("o.b"))
        self.refresh()

    def forward(self, h, ctx: MixContext):
        proj = F.linear(h, self.w_in, self.b_in)
        own = not self.shared_cache
        sops.rownorm_append(proj, self.nq, self.off_k, self.nk, self.off_v,
                            self.nv, self.q_norm, self.k_norm, self.eps,
                            ctx.kcache if own else None,
                            ctx.vcache if own else None, ctx.slot_mapping)
        y = sops.paged_attention_rows(
            proj, 0, self.H, 1, ctx.kcache, ctx.vcache, self.dv,
            ctx.positions, ctx.sb, self.scale, out_dtype=h.dtype,
            temp_coef=self.temp_coef, temp_every=self.temp_every,
            softcap=self.softcap, dist_bias=self.dist_bias)
        return F.linear(y.view(h.shape[0], self.H * self.dv), self.w_o,
                        self.b_o)


class SSDMixer(torch.nn.Module):
    """State-space mixer in the scalar-decay (state-space duality) form.
    W_in h = z | x | B | C | dt with inner = heads * vdim channels for z
    and x, groups * state for B and C, one dt per head. x, B, C pass a
    short causal per-channel convolution with bias and SiLU. Per head
    (sharing B, C with its group): dt = softplus(dt + dt_bias),
    S <- exp(-exp(A_log) dt) S + dt B x^T (S is state x vdim),
    y = S^T C + D x. Output: y * silu(z), RMS-normed in norm_groups equal
    parts of the row, times a weight, then W_o. The decay, step size and
    state are fp32."""

    def __init__(self, width, heads, vdim, state, groups, norm_groups, conv,
                 eps, init):
        super().__init__()
        inner = heads * vdim
        if heads % groups or inner % norm_groups:
            raise ValueError("heads must divide into groups, channels into "
                             "norm groups")
        self.W, self.H, self.P, self.N, self.G = width, heads, vdim, state, groups
        self.inner, self.ng, self.taps, self.eps = inner, norm_groups, conv, eps
        self.Cc = inner + 2 * groups * state
        self.off_dt = inner + self.Cc
        self.w_in = init.mat(self.off_dt + heads, width)
        self.conv_w = init.vec((self.Cc, conv), -0.5, 0.8)
        self.conv_b = init.vec(self.Cc, -0.2, 0.2)
        self.dt_bias = init.vec(heads, -3.0, 0.0)
        self.A_log = init.vec(heads, -1.0, 1.5)
        self.D = init.vec(heads, 0.5, 1.5)
        self.norm_w = init.vec(inner, 0.7, 1.3)
        self.w_o = init.mat(width, inner)

    def state_shapes(self):
        return [(self.H, self.N, self.P), (self.taps - 1, self.Cc)]

    def kv_shape(self):
        return None

    def load(self, get: Getter):
        _put(self.w_in, get("in"))
        _put(self.conv_w, get("conv"))
        _put(self.conv_b, get("conv.b"))
        _put(self.dt_bias, get("dt_bias"))
        _put(self.A_log, get("A_log"))
        _put(self.D, get("D"))
        _put(self.norm_w, get("norm"))
        _put(self.w_o, get("o"))

    def forward(self, h, ctx: MixContext):
        proj = F.linear(h, self.w_in)
        S, conv_state = ctx.states
        xbc = sops.causal_conv(proj[:, self.inner:], self.Cc, self.conv_w,
                               self.conv_b, True, conv_state, ctx.sb)
        y = sops.ssd_scan(xbc, proj[:, self.off_dt:], self.dt_bias, self.A_log,
                          self.D, S, ctx.sb, self.H, self.P, self.N, self.G)
        y = sops.gated_group_norm(y, proj, self.norm_w, self.ng, self.eps,
                                  h.dtype)
        return F.linear(y, self.w_o)


class GeluMLP(torch.nn.Module):
    """Dense feed-forward W_down gelu(W_up h) with the exact (erf) GELU."""

    def __init__(self, width, ff, init):
        super().__init__()
        self.w_up = init.mat(ff, width)
        self.w_down = init.mat(width, ff)

    def load(self, get: Getter):
        _put(self.w_up, get("up"))
        _put(self.w_down, get("down"))

    def forward(self, h):
        return F.linear(sops.gelu_erf(F.linear(h, self.w_up)), self.w_down)
