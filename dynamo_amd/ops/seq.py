"""Sequence-mixer ops: recurrent matrix-state mixers (gated delta rule,
RWKV-style time mixing, mLSTM), softmax attention with a distance bias over
the paged cache, and their row-wise companions.

GPU tensors go to the HIP kernels of dynamo_amd._hip_seq (required there -
a missing extension raises); CPU tensors go to the plain torch versions in
seq_ref. Both take the same arguments.

The batch is the engine's flat run of token rows; `SeqBatch` says which rows
belong to which sequence, where each sequence's portion starts in position
space, and which state slot it owns. A decoded token is a portion of one.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch

from . import seq_ref

_mod = None


def hip_seq():
    global _mod
    if _mod is None:
        try:
            from dynamo_amd import _hip_seq as m
        except Exception as e:  # pragma: no cover
            raise RuntimeError(
                "dynamo_amd._hip_seq native extension is not available on a "
                "GPU device path. Build it with `DYNAMO_AMD_EXTS=_hip_seq "
                "python setup.py build_ext --inplace`. Original error: "
                f"{e}") from e
        _mod = m
    return _mod


@dataclass
class SeqBatch:
    tok_seq: torch.Tensor      # [T] int32: sequence index of each row
    seq_start: torch.Tensor    # [B] int32: first row
    seq_len: torch.Tensor      # [B] int32: rows this step (0 = padding)
    seq_slot: torch.Tensor     # [B] int32: recurrent-state slot
    seq_pos0: torch.Tensor     # [B] int32: position of the first row
    page_table: Optional[torch.Tensor] = None   # [B, maxp] int32
    # rows [0, num_decode) are single decoded tokens; the prompt portions
    # after them are also listed as tiles of at most 64 rows of one
    # sequence: (first row [NT], rows [NT]) int32, for the matrix-core
    # attention kernel. None = no tiling (every row takes the row kernel).
    num_decode: int = 0
    tiles: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
    # host copy [(start, len, slot, pos0)] for the CPU path
    host: Optional[List[Tuple[int, int, int, int]]] = None

    def spans(self):
        if self.host is not None:
            return self.host
        return list(zip(self.seq_start.tolist(), self.seq_len.tolist(),
                        self.seq_slot.tolist(), self.seq_pos0.tolist()))


def _args(sb: SeqBatch):
    return sb.seq_start, sb.seq_len, sb.seq_slot, sb.seq_pos0


# -- row-wise ----------------------------------------------------------------
def embed_scale_pos(ids, positions, embed, pos_table, scale: float):
    """fp32 [T, W]: embed[id] * scale (+ pos_table[position])."""
    if embed.is_cuda:
        out = torch.empty(ids.shape[0], embed.shape[1], dtype=torch.float32,
                          device=embed.device)
        hip_seq().embed_scale_pos(out, ids, positions, embed, pos_table,
                                  float(scale))
        return out
    return seq_ref.embed_scale_pos(ids, positions, embed, pos_table, scale)


def add_scalar_rmsnorm(res, delta, g, eps: float, out_dtype):
    """res (fp32, in place) += delta; returns res / rms(res) * g[0]."""
    if res.is_cuda:
        out = torch.empty(res.shape, dtype=out_dtype, device=res.device)
        hip_seq().add_scalar_rmsnorm(out, res, delta, g, float(eps))
        return out
    return seq_ref.add_scalar_rmsnorm(res, delta, g, eps, out_dtype)


def causal_conv_silu(x, C: int, w, conv_state, sb: SeqBatch):
    """silu of a short causal convolution over the first C columns of x;
    the slot's saved inputs continue earlier portions and are updated."""
    if x.is_cuda:
        out = torch.empty(x.shape[0], C, dtype=torch.float32, device=x.device)
        hip_seq().causal_conv_silu(out, x, w, conv_state, sb.tok_seq,
                                   *_args(sb))
        return out
    return seq_ref.causal_conv_silu(x, C, w, conv_state, sb)


def token_shift_mix(h, mu, prev_state, sb: SeqBatch):
    """[S, T, W]: h + (h_prev - h) * mu_s for each of the S rows of mu."""
    if h.is_cuda:
        out = torch.empty(mu.shape[0], *h.shape, dtype=h.dtype,
                          device=h.device)
        hip_seq().token_shift_mix(out, h, mu, prev_state, sb.tok_seq,
                                  *_args(sb))
        return out
    return seq_ref.token_shift_mix(h, mu, prev_state, sb)


GATE_NONE, GATE_SILU, GATE_SIGMOID = 0, 1, 2


def head_norm_gate(o, w, w_stride: int, gate, gate_act: int, eps: float,
                   out_dtype):
    """o [T, H, dv] fp32 -> [T, H*dv]: per-head RMS norm, weight
    w[h * w_stride + :], times act(gate[:, h*dv + :])."""
    if o.is_cuda:
        out = torch.empty(o.shape[0], o.shape[1] * o.shape[2], dtype=out_dtype,
                          device=o.device)
        hip_seq().head_norm_gate(out, o, w, w_stride, gate, gate_act,
                                 float(eps))
        return out
    return seq_ref.head_norm_gate(o, w, w_stride, gate, gate_act, eps,
                                  out_dtype)


def clamped_glu(gate_up, limit: float, alpha: float):
    """[T, 2F] (gate | up) -> min(g, L) * sigmoid(alpha g) * (clamp(u) + 1)."""
    if gate_up.is_cuda:
        out = torch.empty(gate_up.shape[0], gate_up.shape[1] // 2,
                          dtype=gate_up.dtype, device=gate_up.device)
        hip_seq().clamped_glu(out, gate_up, float(limit), float(alpha))
        return out
    return seq_ref.clamped_glu(gate_up, limit, alpha)


def dual_rmsnorm_mean(a, b, wa, wb, eps: float):
    if a.is_cuda:
        out = torch.empty_like(a)
        hip_seq().dual_rmsnorm_mean(out, a, b, wa, wb, float(eps))
        return out
    return seq_ref.dual_rmsnorm_mean(a, b, wa, wb, eps)


def softcap_(x, cap: float):
    if x.is_cuda:
        hip_seq().softcap_(x, float(cap))
        return x
    return seq_ref.softcap_(x, cap)


# -- recurrences ---------------------------------------------------------------
def gated_delta_rule(qkv, proj, off_b: int, off_a: int, A_log, dt_bias, state,
                     sb: SeqBatch, H: int, G: int, dv: int, qscale: float,
                     unit_eps: float = 1e-6):
    """qkv fp32 [T, 2*G*dk + H*dv]; gates read raw from proj. -> [T, H, dv]."""
    if qkv.is_cuda:
        out = torch.empty(qkv.shape[0], H, dv, dtype=torch.float32,
                          device=qkv.device)
        hip_seq().gated_delta_rule(out, qkv, proj, off_b, off_a, A_log,
                                   dt_bias, state, *_args(sb), G,
                                   float(qscale), float(unit_eps))
        return out
    return seq_ref.gated_delta_rule(qkv, proj, off_b, off_a, A_log, dt_bias,
                                    state, sb, H, G, dv, qscale, unit_eps)


def rwkv_time_mix(r, k, v, wraw, w0, u, state, sb: SeqBatch, H: int):
    if r.is_cuda:
        d = r.shape[1] // H
        out = torch.empty(r.shape[0], H, d, dtype=torch.float32,
                          device=r.device)
        hip_seq().rwkv_time_mix(out, r, k, v, wraw, w0, u, state, *_args(sb))
        return out
    return seq_ref.rwkv_time_mix(r, k, v, wraw, w0, u, state, sb, H)


def mlstm_memory(proj, offs, i_bias, f_bias, state_S, state_n, state_m,
                 sb: SeqBatch, H: int, dv: int, qscale: float, cap: float,
                 den_eps: float = 1e-6):
    """offs = (q, k, v, i, f) column offsets into proj. -> [T, H, dv] fp32."""
    if proj.is_cuda:
        out = torch.empty(proj.shape[0], H, dv, dtype=torch.float32,
                          device=proj.device)
        hip_seq().mlstm_memory(out, proj, *offs, i_bias, f_bias, state_S,
                               state_n, state_m, *_args(sb), float(qscale),
                               float(cap), float(den_eps))
        return out
    return seq_ref.mlstm_memory(proj, offs, i_bias, f_bias, state_S, state_n,
                                state_m, sb, H, dv, qscale, cap, den_eps)


# -- attention -----------------------------------------------------------------
def kv_append_norm(kcache, vcache, proj, off_k: int, off_v: int, slot_mapping,
                   vnorm: bool, eps: float):
    if proj.is_cuda:
        hip_seq().kv_append_norm(kcache, vcache, proj, off_k, off_v,
                                 slot_mapping, bool(vnorm), float(eps))
    else:
        seq_ref.kv_append_norm(kcache, vcache, proj, off_k, off_v,
                               slot_mapping, vnorm, eps)


def biased_attention(proj, off_q: int, H: int, kcache, vcache, positions,
                     sb: SeqBatch, r1, r2, scale: float, temp_coef: float,
                     temp_every: int):
    """-> [T, H*dv] in proj's dtype."""
    dv = vcache.shape[3]
    if proj.is_cuda:
        T = proj.shape[0]
        out = torch.empty(T, H, dv, dtype=proj.dtype, device=proj.device)
        m = hip_seq()
        # prompt portions in bf16 go to the MFMA kernel when the head sizes
        # fit it; decoded tokens, fp32 and other sizes take the row kernel
        tiled = (sb.tiles is not None and proj.dtype == torch.bfloat16
                 and m.biased_attention_mfma_supported(kcache.shape[3], dv)
                 and kcache.data_ptr() % 16 == 0
                 and vcache.data_ptr() % 16 == 0)
        nrow = sb.num_decode if tiled else T
        if nrow:
            m.biased_attention(out[:nrow], proj[:nrow], off_q, kcache, vcache,
                               sb.page_table, sb.tok_seq[:nrow],
                               positions[:nrow], sb.seq_len, r1, r2,
                               float(scale), float(temp_coef),
                               int(temp_every))
        if tiled and sb.tiles[0].numel():
            m.biased_attention_mfma(out, proj, off_q, kcache, vcache,
                                    sb.page_table, sb.tiles[0], sb.tiles[1],
                                    64, sb.tok_seq, positions, r1, r2,
                                    float(scale), float(temp_coef),
                                    int(temp_every))
        return out.view(T, H * dv)
    return seq_ref.biased_attention(proj, off_q, H, kcache, vcache, positions,
                                    sb, r1, r2, scale, temp_coef, temp_every)


# -- layer-norm sandwiched layers ----------------------------------------------
def residual_layernorm(res, delta, post_w, mult: float, w, eps: float,
                       out_dtype):
    """res (fp32, in place) += mult * LN(delta) * post_w when delta is given
    (plain += delta without post_w); returns LN(res) * w in out_dtype, or
    None when w is None. LN is the weight-only layer norm."""
    if res.is_cuda:
        out = (torch.empty(res.shape, dtype=out_dtype, device=res.device)
               if w is not None else None)
        hip_seq().residual_layernorm(out, res, delta, post_w, float(mult), w,
                                     float(eps))
        return out
    return seq_ref.residual_layernorm(res, delta, post_w, mult, w, eps,
                                      out_dtype)


def xielu(x, pq):
    """xIELU with raw parameters pq = (p, q): softplus(p) z^2 + z/2 for
    z > 0, (1/2 + softplus(q)) (e^z - 1 - z) + z/2 otherwise."""
    if x.is_cuda:
        out = torch.empty_like(x)
        hip_seq().xielu(out, x, pq)
        return out
    return seq_ref.xielu(x, pq)


def rope_rows(dst, dst_col: int, dst_vec: int, src, src_col: int,
              src_vec: int, positions, freqs, nvec: int, length: int,
              interleaved: bool):
    """For each token row, `nvec` vectors of `length` entries (vector v at
    column col + v * vec) go from src to dst with their first dims entries
    rotated by position * f, f = freqs[0] + freqs[1] (fp32 [2, dims/2], see
    models.mixers.rotary_frequencies); dst may be src."""
    if src.is_cuda:
        hip_seq().rope_rows(dst, dst_col, dst_vec, src, src_col, src_vec,
                            positions, freqs, nvec, length, bool(interleaved))
    else:
        seq_ref.rope_rows(dst, dst_col, dst_vec, src, src_col, src_vec,
                          positions, freqs, nvec, length, interleaved)


def latent_append(cache, z, z_col: int, norm_w, slot_mapping, positions,
                  freqs, interleaved: bool, eps: float):
    """cache [P, 1, ps, rank + rd] <- [rmsnorm(z[:rank]) * norm_w |
    rotated z[rank:rank + rd]] at each token's slot."""
    if z.is_cuda:
        hip_seq().latent_append(cache, z, z_col, norm_w, slot_mapping,
                                positions, freqs, bool(interleaved),
                                float(eps))
    else:
        seq_ref.latent_append(cache, z, z_col, norm_w, slot_mapping,
                              positions, freqs, interleaved, eps)


def paged_attention_rows(q, off_q: int, H: int, kmaps: int, kcache, vcache,
                         dv: int, positions, sb: SeqBatch, scale: float,
                         window: int = 0, keep_first: int = 0, head_bias=None,
                         sigmoid: bool = False, out_dtype=torch.float32,
                         temp_coef: float = 0.0, temp_every: int = 1,
                         softcap: float = 0.0, dist_bias=None, sink=None):
    """Causal attention of every row over its sequence's pages.
    -> [T, H, kmaps, dv] (fp32 unless out_dtype says otherwise). Queries lie
    in q at off_q as [H][kmaps][dk]; kcache [P, G, ps, kmaps * dk]; values
    from vcache [P, G, ps, dv] or, without one, from the first dv entries of
    the key rows. window > 0: row i sees keys j with 0 <= i - j < window,
    and also the keys j < keep_first whatever their distance. head_bias
    (fp32 [H]) is added to the scaled scores. The weights are a softmax over
    the visible keys, or with `sigmoid` the plain sigmoid of each score
    (not normalised over the keys). Further options of the softmax form: a
    query temperature 1 + temp_coef ln(floor((i + 1) / temp_every) + 1) on
    the scaled scores, a soft cap c tanh(score / c) after it, a bias by
    distance dist_bias[h, min(i - j, D)] (fp32 [H, D + 1]) added after the
    cap, and a per-head sink (fp32 [H]): exp(sink_h) joins the softmax
    denominator without a key or value."""
    if q.is_cuda:
        T = q.shape[0]
        out = torch.empty(T, H, kmaps, dv, dtype=out_dtype, device=q.device)
        m = hip_seq()
        # bf16 rows whose sizes fit go to the matrix cores: prompt portions
        # as 64-row tiles, decoded tokens (rows [0, num_decode)) with their
        # heads as tile rows when at least 8 heads share a kv head. fp32,
        # other sizes and the remaining rows take the row kernel.
        krow, G = kcache.shape[3], kcache.shape[1]
        f32out = out_dtype == torch.float32
        extras = softcap > 0 or dist_bias is not None
        fits = (q.dtype == torch.bfloat16
                and m.paged_attention_mfma_supported(krow // kmaps, dv, f32out,
                                                     extras)
                and krow % 8 == 0 and kcache.data_ptr() % 16 == 0
                and (vcache is None or vcache.data_ptr() % 16 == 0))
        tiled = fits and sb.tiles is not None
        ndec = min(sb.num_decode, T)
        done = 0
        opts = (int(window), int(keep_first), head_bias, bool(sigmoid),
                float(softcap), dist_bias, sink)
        temp = (float(temp_coef), int(temp_every))
        if (fits and ndec and H // G >= 8 and f32out
                and m.paged_attention_mfma_supported(krow // kmaps, dv, True,
                                                     extras)):
            # about one workgroup per compute unit: more key splits only
            # add staging and merge work (measured with and without a window)
            nsplit = max(1, min(16, 256 // (ndec * G * kmaps)))
            part = torch.empty(ndec, H, kmaps, nsplit, dv + 2,
                               dtype=torch.float32, device=q.device)
            m.paged_attention_mfma_decode(
                out[:ndec], part, q[:ndec], off_q, kcache, vcache,
                sb.page_table, sb.tok_seq[:ndec], positions[:ndec],
                sb.seq_len, float(scale), *temp, int(kmaps), *opts)
            done = ndec
        end = ndec if tiled else T
        if end > done:
            m.paged_attention_rows(
                out[done:end], q[done:end], off_q, kcache, vcache,
                sb.page_table, sb.tok_seq[done:end], positions[done:end],
                sb.seq_len, None, None, float(scale), *temp, int(kmaps),
                *opts)
        if tiled and sb.tiles[0].numel():
            m.paged_attention_mfma(
                out, q, off_q, kcache, vcache, sb.page_table, sb.tiles[0],
                sb.tiles[1], 64, sb.tok_seq, positions, None, None,
                float(scale), *temp, int(kmaps), *opts)
        return out
    return seq_ref.paged_attention_rows(
        q, off_q, H, kmaps, kcache, vcache, dv, positions, sb, scale, window,
        keep_first, head_bias, sigmoid, temp_coef, temp_every, softcap,
        dist_bias, sink).to(out_dtype)


def diff_norm_gate(a, lam, post: float, gate, eps: float, out_dtype):
    """a fp32 [T, H, 2, dv] -> [T, H*dv]: (a1 - lam a2) / rms * post *
    sigmoid(gate)."""
    if a.is_cuda:
        T, H, _two, dv = a.shape
        out = torch.empty(T, H * dv, dtype=out_dtype, device=a.device)
        hip_seq().diff_norm_gate(out, a, lam, float(post), gate, float(eps))
        return out
    return seq_ref.diff_norm_gate(a, lam, post, gate, eps, out_dtype)


def head_sigmoid_scale(x, gate, out_dtype):
    """x fp32 [T, H, R], gate [T, >=H] -> [H, T, R] = x * sigmoid(gate)."""
    if x.is_cuda:
        T, H, R = x.shape
        out = torch.empty(H, T, R, dtype=out_dtype, device=x.device)
        hip_seq().head_sigmoid_scale(out, x, gate)
        return out
    return seq_ref.head_sigmoid_scale(x, gate, out_dtype)


def causal_conv(x, C: int, w, bias, silu: bool, conv_state, sb: SeqBatch):
    """Short causal convolution over the first C columns of x with optional
    bias and SiLU; fp32 out. The slot's saved inputs continue earlier
    portions and are updated."""
    if x.is_cuda:
        out = torch.empty(x.shape[0], C, dtype=torch.float32, device=x.device)
        hip_seq().causal_conv(out, x, w, bias, bool(silu), conv_state,
                              sb.tok_seq, *_args(sb))
        return out
    return seq_ref.causal_conv(x, C, w, bias, silu, conv_state, sb)


def rglru_scan(u, gates, br, bi, lam, y, state, sb: SeqBatch, decay: float,
               out_dtype):
    """Real-gated linear recurrence over fp32 u [T, C] with gate
    pre-activations gates [nb, T, 2*bw]; returns S * gelu_tanh(y[:, :C])."""
    if u.is_cuda:
        out = torch.empty(u.shape, dtype=out_dtype, device=u.device)
        # long portions are scanned in parallel chunks; the kernel needs an
        # upper bound of the longest portion (known on the host, or all rows)
        longest = (max((n for _s, n, _l, _p in sb.host), default=1)
                   if sb.host is not None else u.shape[0])
        hip_seq().rglru_scan(out, u, gates, br, bi, lam, y, state, *_args(sb),
                             float(decay), max(1, int(longest)))
        return out
    return seq_ref.rglru_scan(u, gates, br, bi, lam, y, state, sb, decay,
                              out_dtype)


# -- input convolution of a sublayer, normed rotated heads into the cache,
# -- minimal gated recurrence, routed experts ---------------------------------
def residual_conv(res, w, conv_state, sb: SeqBatch, out_dtype):
    """res + conv(res): a short causal per-channel convolution over the fp32
    rows res [T, W] (w fp32 [W, taps], the last tap weighs the current
    token, no bias), added to its own input. The slot's saved rows
    [slots, taps - 1, W] continue earlier portions and are updated."""
    if res.is_cuda:
        out = torch.empty(res.shape, dtype=out_dtype, device=res.device)
        hip_seq().residual_conv(out, res, w, conv_state, sb.tok_seq,
                                *_args(sb))
        return out
    return seq_ref.residual_conv(res, w, conv_state, sb, out_dtype)


def join_conv(res, delta, post_w, eps: float, w, conv_state, sb: SeqBatch,
              out_dtype):
    """The step between two sublayers of a conv-fed layer: the waiting
    sublayer output joins the stream, res += LN(delta) * post_w (weight-only
    layer norm; skipped without delta), and the next sublayer's input
    res + conv(res) is returned (see residual_conv). When every row is a
    decoded token both happen in one kernel."""
    if res.is_cuda and sb.num_decode >= res.shape[0] and w.shape[1] <= 4:
        out = torch.empty(res.shape, dtype=out_dtype, device=res.device)
        if hip_seq().join_conv_single(out, res, delta, post_w, float(eps), w,
                                      conv_state, sb.tok_seq, sb.seq_len,
                                      sb.seq_slot, sb.seq_pos0):
            return out
    if delta is not None:
        residual_layernorm(res, delta, post_w, 1.0, None, eps, out_dtype)
    return residual_conv(res, w, conv_state, sb, out_dtype)


def headnorm_rope_append(proj, H: int, G: int, dk: int, dv: int, off_k: int,
                         off_v: int, qw, kw, freqs, interleaved: bool,
                         eps: float, positions, kcache, vcache, slot_mapping):
    """Per token row of proj (q at column 0 as [H][dk], k at off_k as
    [G][dk], v at off_v as [G][dv]): every query and key vector is divided
    by its root mean square, multiplied by qw / kw (fp32 [dk], shared by the
    heads) and has its first rot dims rotated by position * f (freqs as in
    rope_rows; None = no rotation). Queries are rewritten in place; keys and
    the raw values go to the token's cache slot."""
    if proj.is_cuda:
        hip_seq().headnorm_rope_append(
            proj, H, G, dk, dv, off_k, off_v, qw, kw, freqs,
            bool(interleaved), float(eps), positions, kcache, vcache,
            slot_mapping)
    else:
        seq_ref.headnorm_rope_append(
            proj, H, G, dk, dv, off_k, off_v, qw, kw, freqs, interleaved,
            eps, positions, kcache, vcache, slot_mapping)


def _longest(sb: SeqBatch, T: int) -> int:
    """Upper bound of the longest portion of the step (known on the host,
    or all rows)."""
    if sb.host is not None:
        return max(1, max((n for _s, n, _l, _p in sb.host), default=1))
    return max(1, T)


def mingru_scan(proj, C: int, state, sb: SeqBatch, out_dtype):
    """Minimal gated recurrent unit over proj [T, 3C] = z | u | g
    pre-activations: S <- (1 - sigmoid(z)) S + sigmoid(z) c(u) with
    c(u) = u + 1/2 for u >= 0 and sigmoid(u) below; returns S * silu(g).
    state fp32 [slots, C]."""
    if proj.is_cuda:
        out = torch.empty(proj.shape[0], C, dtype=out_dtype,
                          device=proj.device)
        hip_seq().mingru_scan(out, proj, state, *_args(sb),
                              _longest(sb, proj.shape[0]))
        return out
    return seq_ref.mingru_scan(proj, C, state, sb, out_dtype)


def relu_squared(x):
    if x.is_cuda:
        out = torch.empty_like(x)
        hip_seq().relu_squared(out, x)
        return out
    return seq_ref.relu_squared(x)


def moe_route(logits, correction, groups: int, keep: int, top: int,
              scale: float):
    """Router of a mixture of experts. logits fp32 [T, n]; scores are their
    softmax; the choice adds `correction` [n] and is limited to the `keep`
    best of `groups` equal groups of neighbouring outputs (a group's score
    is its largest choice score). -> (chosen outputs int32 [T, top], their
    uncorrected scores * scale fp32 [T, top])."""
    if logits.is_cuda:
        T = logits.shape[0]
        idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
        wgt = torch.empty(T, top, dtype=torch.float32, device=logits.device)
        hip_seq().moe_route(idx, wgt, logits, None, correction, int(groups),
                            int(keep), float(scale))
        return idx, wgt
    return seq_ref.moe_route(logits, correction, groups, keep, top, scale)


def moe_route_rows(h, router, correction, groups: int, keep: int, top: int,
                   scale: float):
    """moe_route of the fp32 logits h @ router^T (h [T, W] in the activation
    type, router fp32 [n, W]). Few rows with few router outputs form their
    logits inside the routing kernel."""
    T, n = h.shape[0], router.shape[0]
    if h.is_cuda and T <= 256 and n <= 64:
        idx = torch.empty(T, top, dtype=torch.int32, device=h.device)
        wgt = torch.empty(T, top, dtype=torch.float32, device=h.device)
        hip_seq().moe_route(idx, wgt, h, router, correction, int(groups),
                            int(keep), float(scale))
        return idx, wgt
    logits = torch.nn.functional.linear(h.float(), router)
    return moe_route(logits, correction, groups, keep, top, scale)


def moe_dispatch(idx, n_out: int):
    """-> (rank int32 [T, k]: how many earlier entries of idx chose the same
    output, counts int32 [n_out])."""
    if idx.is_cuda:
        rank = torch.empty_like(idx)
        counts = torch.empty(n_out, dtype=torch.int32, device=idx.device)
        hip_seq().moe_dispatch(rank, counts, idx)
        return rank, counts
    return seq_ref.moe_dispatch(idx, n_out)


def moe_gather(h, idx, rank, base, E: int, rows: int):
    """xg [rows, W]: row base[e] + rank[t, j] holds h[t] for every choice
    e = idx[t, j] < E (outputs >= E are identity experts and take no row)."""
    if h.is_cuda:
        # rows nobody owns stay as they are: nothing reads what the experts
        # make of them
        xg = torch.empty(rows, h.shape[1], dtype=h.dtype, device=h.device)
        hip_seq().moe_gather(xg, h, idx, rank, base, int(E))
        return xg
    return seq_ref.moe_gather(h, idx, rank, base, E, rows)


def moe_combine(y, h, idx, wgt, rank, base, E: int, shared, out_dtype,
                shared_gate=None):
    """out[t] = sum_j wgt[t, j] * (y[base[e] + rank[t, j]] if e < E else
    h[t]) (+ shared[t], times sigmoid(shared_gate[t]) when a raw gate value
    per token is given), summed in fp32 in the order of j."""
    if h.is_cuda:
        out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
        hip_seq().moe_combine(out, y, h, idx, wgt, rank, base, int(E), shared,
                              shared_gate)
        return out
    return seq_ref.moe_combine(y, h, idx, wgt, rank, base, E, shared,
                               out_dtype, shared_gate)


# -- hashed pair embedding, stream mixing, whole-projection norms, state-space
# -- scan, grouped gated norm, top-k router over logits -----------------------
def embed_pair_hash(ids, embed, table, mul_prev: int, mul_cur: int,
                    prev_state, sb: SeqBatch):
    """fp32 [T, W]: embed[id] + table[(prev * mul_prev + id * mul_cur) mod n]
    with n = rows of table - 1; a sequence's first token takes row n. The
    previous token of a portion's first row comes from prev_state
    (fp32 [slots, 1], the token id as a number), which is left holding the
    portion's last token."""
    if embed.is_cuda:
        out = torch.empty(ids.shape[0], embed.shape[1], dtype=torch.float32,
                          device=embed.device)
        hip_seq().embed_pair_hash(out, ids, embed, table, int(mul_prev),
                                  int(mul_cur), prev_state, sb.tok_seq,
                                  *_args(sb))
        return out
    return seq_ref.embed_pair_hash(ids, embed, table, mul_prev, mul_cur,
                                   prev_state, sb)


def stream_step(xs, delta, mix, out_w, mult: float, in_w, norm_w, eps: float,
                out_dtype):
    """One step on S parallel residual streams xs (fp32 [T, S, W], in
    place). With delta (a sublayer's output): every stream t becomes
    sum_s mix[s, t] xs[s] + mult * out_w[t] * delta, all from the old
    streams. Then, with in_w: the read u = sum_s in_w[s] xs[s] is returned
    RMS-normed times (1 + norm_w) in out_dtype, or - without norm_w - as it
    is in fp32. mix fp32 [S, S], out_w / in_w fp32 [S]."""
    if xs.is_cuda:
        T, S, W = xs.shape
        out = None
        if in_w is not None:
            out = torch.empty(T, W, device=xs.device,
                              dtype=out_dtype if norm_w is not None
                              else torch.float32)
        hip_seq().stream_step(out, xs, delta, mix, out_w, float(mult), in_w,
                              norm_w, float(eps))
        return out
    return seq_ref.stream_step(xs, delta, mix, out_w, mult, in_w, norm_w, eps,
                               out_dtype)


def rms_norm_cols(x, col: int, n: int, w, eps: float, out_dtype):
    """[T, n]: columns [col, col + n) of x divided by their root mean
    square, times w (fp32 [n])."""
    if x.is_cuda:
        out = torch.empty(x.shape[0], n, dtype=out_dtype, device=x.device)
        hip_seq().rms_norm_cols(out, x, int(col), w, float(eps))
        return out
    return seq_ref.rms_norm_cols(x, col, n, w, eps, out_dtype)


def rownorm_append(proj, nq: int, off_k: int, nk: int, off_v: int, nv: int,
                   qw, kw, eps: float, kcache, vcache, slot_mapping):
    """Per token row of proj: the whole query run [0, nq) is divided by its
    root mean square and multiplied by qw (fp32 [nq]) in place; with caches,
    the whole key run [off_k, off_k + nk) likewise with kw, written with the
    raw values [off_v, off_v + nv) to the token's cache slot (kcache
    [P, G, ps, nk / G], vcache [P, G, ps, nv / G])."""
    if proj.is_cuda:
        hip_seq().rownorm_append(proj, int(nq), int(off_k), int(nk),
                                 int(off_v), int(nv), qw, kw, float(eps),
                                 kcache, vcache, slot_mapping)
    else:
        seq_ref.rownorm_append(proj, nq, off_k, nk, off_v, nv, qw, kw, eps,
                               kcache, vcache, slot_mapping)


def heads_major(x, out_dtype):
    """x [T, H, R] -> [H, T, R] in out_dtype (the layout a per-head batched
    product reads)."""
    if x.is_cuda:
        T, H, R = x.shape
        out = torch.empty(H, T, R, dtype=out_dtype, device=x.device)
        hip_seq().heads_major(out, x)
        return out
    return seq_ref.heads_major(x, out_dtype)


def heads_gate(o, gate, out_dtype):
    """o [H, T, dv] (head-major), gate [T, >= H*dv] -> [T, H*dv] =
    o * sigmoid(gate), element by element."""
    if o.is_cuda:
        H, T, dv = o.shape
        out = torch.empty(T, H * dv, dtype=out_dtype, device=o.device)
        hip_seq().heads_gate(out, o, gate)
        return out
    return seq_ref.heads_gate(o, gate, out_dtype)


def ssd_scan(xbc, dt_raw, dt_bias, A_log, D, state, sb: SeqBatch, H: int,
             P: int, N: int, G: int):
    """State-space recurrence over fp32 xbc [T, H*P + 2*G*N] = x | B | C:
    per head h (group h // (H / G)), dt = softplus(dt_raw + dt_bias),
    S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x.
    state fp32 [slots, H, N, P]; dt_raw [T, H] (any row stride).
    -> fp32 [T, H*P]."""
    if xbc.is_cuda:
        out = torch.empty(xbc.shape[0], H * P, dtype=torch.float32,
                          device=xbc.device)
        hip_seq().ssd_scan(out, xbc, dt_raw, dt_bias, A_log, D, state,
                           *_args(sb), int(G))
        return out
    return seq_ref.ssd_scan(xbc, dt_raw, dt_bias, A_log, D, state, sb, H, P,
                            N, G)


def gated_group_norm(y, z, w, groups: int, eps: float, out_dtype):
    """fp32 y [T, C] times silu(z[:, :C]), RMS-normed in `groups` equal
    parts of the row, times w (fp32 [C])."""
    if y.is_cuda:
        out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
        hip_seq().gated_group_norm(out, y, z, w, int(groups), float(eps))
        return out
    return seq_ref.gated_group_norm(y, z, w, groups, eps, out_dtype)


def gelu_erf(x):
    if x.is_cuda:
        out = torch.empty_like(x)
        hip_seq().gelu_erf(out, x)
        return out
    return seq_ref.gelu_erf(x)


def silu_glu(gate_up):
    """[..., 2F] (gate | up) -> silu(gate) * up."""
    if gate_up.is_cuda:
        Fd = gate_up.shape[-1] // 2
        out = torch.empty(*gate_up.shape[:-1], Fd, dtype=gate_up.dtype,
                          device=gate_up.device)
        hip_seq().silu_glu(out.view(-1, Fd), gate_up.view(-1, 2 * Fd))
        return out
    return seq_ref.silu_glu(gate_up)


def moe_route_topk(logits, n: int, bias, top: int):
    """Router that keeps the `top` largest of the first n columns of the
    fp32 logits (+ bias fp32 [n]); the weights are the softmax over the
    chosen ones only. -> (int32 [T, top], fp32 [T, top])."""
    if logits.is_cuda:
        T = logits.shape[0]
        idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
        wgt = torch.empty(T, top, dtype=torch.float32, device=logits.device)
        hip_seq().moe_route_topk(idx, wgt, logits, int(n), bias)
        return idx, wgt
    return seq_ref.moe_route_topk(logits, n, bias, top)
