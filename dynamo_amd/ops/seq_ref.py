"""Plain torch versions of the sequence-mixer ops (the CPU path).

Same arguments and state layout as the HIP kernels: fp32 state tensors
indexed by slot, a portion that starts at position 0 ignores what its slot
holds. Token loops are explicit; this path is for CPU engines and tests.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def embed_scale_pos(ids, positions, embed, pos_table, scale):
    x = embed[ids.long()].float() * scale
    if pos_table is not None:
        x = x + pos_table[positions.long()].float()
    return x


def add_scalar_rmsnorm(res, delta, g, eps, out_dtype):
    if delta is not None:
        res.add_(delta.float())
    inv = torch.rsqrt(res.pow(2).mean(-1, keepdim=True) + eps)
    return (res * inv * g.float().reshape(())).to(out_dtype)


def causal_conv_silu(x, C, w, conv_state, sb):
    taps = w.shape[1]
    K = taps - 1
    xin = x[:, :C].float()
    out = torch.empty(x.shape[0], C, dtype=torch.float32)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        hist = (conv_state[slot].clone() if pos0 > 0
                else torch.zeros(K, C, dtype=torch.float32))
        if 0 < pos0 < K:
            hist[:K - pos0] = 0
        full = torch.cat([hist, xin[start:start + n]], 0)      # [K + n, C]
        acc = torch.zeros(n, C, dtype=torch.float32)
        for j in range(taps):
            acc += full[j:j + n] * w[:, j]
        out[start:start + n] = F.silu(acc)
        if K:
            conv_state[slot] = full[-K:]
    return out


def token_shift_mix(h, mu, prev_state, sb):
    hf = h.float()
    prev = torch.zeros_like(hf)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        if pos0 > 0:
            prev[start] = prev_state[slot]
        prev[start + 1:start + n] = hf[start:start + n - 1]
        prev_state[slot] = hf[start + n - 1]
    return (hf.unsqueeze(0) + (prev - hf).unsqueeze(0) *
            mu.float().unsqueeze(1)).to(h.dtype)


def head_norm_gate(o, w, w_stride, gate, gate_act, eps, out_dtype):
    T, H, dv = o.shape
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
    wh = torch.stack([w[h * w_stride:h * w_stride + dv] for h in range(H)])
    y = y * wh
    if gate_act:
        g = gate[:, :H * dv].float().view(T, H, dv)
        y = y * (F.silu(g) if gate_act == 1 else torch.sigmoid(g))
    return y.reshape(T, H * dv).to(out_dtype)


def clamped_glu(gate_up, limit, alpha):
    Fd = gate_up.shape[1] // 2
    g = gate_up[:, :Fd].float().clamp(max=limit)
    u = gate_up[:, Fd:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1)).to(gate_up.dtype)


def dual_rmsnorm_mean(a, b, wa, wb, eps):
    def n(x, w):
        x = x.float()
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w
    return (0.5 * (n(a, wa) + n(b, wb))).to(a.dtype)


def softcap_(x, cap):
    return x.copy_(cap * torch.tanh(x / cap))


def gated_delta_rule(qkv, proj, off_b, off_a, A_log, dt_bias, state, sb, H, G,
                     dv, qscale, unit_eps):
    T = qkv.shape[0]
    dk = state.shape[2]
    Cq = G * dk
    q = qkv[:, :Cq].view(T, G, dk)
    k = qkv[:, Cq:2 * Cq].view(T, G, dk)
    v = qkv[:, 2 * Cq:].view(T, H, dv)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + unit_eps) * qscale
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + unit_eps)
    beta = torch.sigmoid(proj[:, off_b:off_b + H].float())
    g = torch.exp(-torch.exp(A_log) *
                  F.softplus(proj[:, off_a:off_a + H].float() + dt_bias))
    rep = H // G
    out = torch.empty(T, H, dv, dtype=torch.float32)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        S = state[slot].clone() if pos0 > 0 else torch.zeros_like(state[slot])
        for t in range(start, start + n):
            kt = k[t].repeat_interleave(rep, 0)            # [H, dk]
            qt = q[t].repeat_interleave(rep, 0)
            S = S * g[t].view(H, 1, 1)
            u = beta[t].view(H, 1) * (v[t] - torch.einsum("hkv,hk->hv", S, kt))
            S = S + kt.unsqueeze(2) * u.unsqueeze(1)
            out[t] = torch.einsum("hkv,hk->hv", S, qt)
        state[slot] = S
    return out


def rwkv_time_mix(r, k, v, wraw, w0, u, state, sb, H):
    T = r.shape[0]
    d = r.shape[1] // H
    r, k, v = (x.float().view(T, H, d) for x in (r, k, v))
    w = torch.exp(-torch.exp(wraw.float() + w0)).view(T, H, d)
    uu = u.view(H, d)
    out = torch.empty(T, H, d, dtype=torch.float32)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        S = state[slot].clone() if pos0 > 0 else torch.zeros_like(state[slot])
        for t in range(start, start + n):
            kv = k[t].unsqueeze(2) * v[t].unsqueeze(1)       # [H, d, d]
            out[t] = torch.einsum("hkv,hk->hv", S + uu.unsqueeze(2) * kv, r[t])
            S = w[t].unsqueeze(2) * S + kv
        state[slot] = S
    return out


def mlstm_memory(proj, offs, i_bias, f_bias, state_S, state_n, state_m, sb, H,
                 dv, qscale, cap, den_eps):
    T = proj.shape[0]
    dk = state_S.shape[2]
    oq, ok, ov, oi, of = offs
    p = proj.float()
    q = p[:, oq:oq + H * dk].view(T, H, dk) * qscale
    k = p[:, ok:ok + H * dk].view(T, H, dk)
    v = p[:, ov:ov + H * dv].view(T, H, dv)
    ig = cap * torch.tanh((p[:, oi:oi + H] + i_bias) / cap)
    fg = F.logsigmoid(cap * torch.tanh((p[:, of:of + H] + f_bias) / cap))
    out = torch.empty(T, H, dv, dtype=torch.float32)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        if pos0 > 0:
            S, nn, m = (state_S[slot].clone(), state_n[slot].clone(),
                        state_m[slot].clone())
        else:
            S, nn, m = (torch.zeros_like(state_S[slot]),
                        torch.zeros_like(state_n[slot]),
                        torch.zeros_like(state_m[slot]))
        for t in range(start, start + n):
            mn = torch.maximum(fg[t] + m, ig[t])
            a, b = torch.exp(fg[t] + m - mn), torch.exp(ig[t] - mn)
            m = mn
            S = a.view(H, 1, 1) * S + b.view(H, 1, 1) * (
                k[t].unsqueeze(2) * v[t].unsqueeze(1))
            nn = a.view(H, 1) * nn + b.view(H, 1) * k[t]
            num = torch.einsum("hkv,hk->hv", S, q[t])
            nq = (nn * q[t]).sum(-1)
            den = torch.maximum(nq.abs(), torch.exp(-m)) + den_eps
            out[t] = num / den.view(H, 1)
        state_S[slot], state_n[slot], state_m[slot] = S, nn, m
    return out


def kv_append_norm(kcache, vcache, proj, off_k, off_v, slot_mapping, vnorm,
                   eps):
    P, G, ps, dk = kcache.shape
    dv = vcache.shape[3]
    T = proj.shape[0]
    k = proj[:, off_k:off_k + G * dk].view(T, G, dk)
    v = proj[:, off_v:off_v + G * dv].float().view(T, G, dv)
    if vnorm:
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    v = v.to(vcache.dtype)
    for t, slot in enumerate(slot_mapping.tolist()):
        if slot < 0:
            continue
        kcache[slot // ps, :, slot % ps] = k[t]
        vcache[slot // ps, :, slot % ps] = v[t]


def biased_attention(proj, off_q, H, kcache, vcache, positions, sb, r1, r2,
                     scale, temp_coef, temp_every):
    P, G, ps, dk = kcache.shape
    dv = vcache.shape[3]
    T = proj.shape[0]
    q = proj[:, off_q:off_q + H * dk].float().view(T, H, dk)
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    pos = positions.tolist()
    rep = H // G
    for si, (start, n, slot, pos0) in enumerate(sb.spans()):
        if n == 0:
            continue
        pages = sb.page_table[si].long()
        ctx = pos0 + n
        npg = (ctx + ps - 1) // ps
        # [G, ctx, d] gathered from the pages
        kk = kcache[pages[:npg]].float().permute(1, 0, 2, 3).reshape(
            G, npg * ps, dk)[:, :ctx]
        vv = vcache[pages[:npg]].float().permute(1, 0, 2, 3).reshape(
            G, npg * ps, dv)[:, :ctx]
        kk = kk.repeat_interleave(rep, 0)
        vv = vv.repeat_interleave(rep, 0)
        for t in range(start, start + n):
            i = pos[t]
            temp = 1.0
            if temp_coef != 0.0:
                temp += temp_coef * math.log((i + 1) // temp_every + 1)
            s = torch.einsum("hd,hjd->hj", q[t] * (temp * scale),
                             kk[:, :i + 1])
            if r1 is not None:
                dist = (i - torch.arange(i + 1)).float()
                s = s - r1.view(H, 1) * torch.log1p(r2.view(H, 1) * dist)
            out[t] = torch.einsum("hj,hjd->hd", torch.softmax(s, -1),
                                  vv[:, :i + 1])
    return out.to(proj.dtype).view(T, H * dv)


# -- layer-norm sandwiched layers, rotary, differential / latent attention -----
def _ln(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = (x - mu).pow(2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def residual_layernorm(res, delta, post_w, mult, w, eps, out_dtype):
    if delta is not None:
        d = delta.float()
        res.add_(mult * _ln(d, post_w, eps) if post_w is not None else d)
    if w is None:
        return None
    return _ln(res, w, eps).to(out_dtype)


def xielu(x, pq):
    z = x.float()
    ap, aq = F.softplus(pq[0]), 0.5 + F.softplus(pq[1])
    y = torch.where(z > 0, ap * z * z + 0.5 * z,
                    aq * (torch.expm1(z.clamp(max=0)) - z) + 0.5 * z)
    return y.to(x.dtype)


def _rotate(x, positions, freqs, interleaved):
    """x fp32 [T, n, len]; freqs [2, dims/2] (hi, lo float pairs); the
    first dims entries are rotated."""
    dims = 2 * freqs.shape[1]
    ang = positions.double()[:, None] * (freqs[0].double()
                                         + freqs[1].double())[None, :]
    c = torch.cos(ang).float()[:, None, :]
    s = torch.sin(ang).float()[:, None, :]
    y = x.clone()
    if interleaved:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        y[..., 0:dims:2] = a * c - b * s
        y[..., 1:dims:2] = b * c + a * s
    else:
        h = dims // 2
        a, b = x[..., :h], x[..., h:dims]
        y[..., :h] = a * c - b * s
        y[..., h:dims] = b * c + a * s
    return y


def rope_rows(dst, dst_col, dst_vec, src, src_col, src_vec, positions, freqs,
              nvec, length, interleaved):
    T = src.shape[0]
    if T == 0 or nvec == 0:
        return
    x = torch.stack([src[:, src_col + v * src_vec:src_col + v * src_vec + length]
                     for v in range(nvec)], 1).float()
    y = _rotate(x, positions, freqs, interleaved).to(dst.dtype)
    for v in range(nvec):
        dst[:, dst_col + v * dst_vec:dst_col + v * dst_vec + length] = y[:, v]


def latent_append(cache, z, z_col, norm_w, slot_mapping, positions, freqs,
                  interleaved, eps):
    P, _one, ps, row = cache.shape
    rank = norm_w.numel()
    zz = z[:, z_col:z_col + row].float()
    c = zz[:, :rank]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w
    kr = _rotate(zz[:, None, rank:], positions, freqs, interleaved)[:, 0]
    rows = torch.cat([c, kr], -1).to(cache.dtype)
    for t, slot in enumerate(slot_mapping.tolist()):
        if slot >= 0:
            cache[slot // ps, 0, slot % ps] = rows[t]


def paged_attention_rows(q, off_q, H, kmaps, kcache, vcache, dv, positions, sb,
                         scale, window, keep_first=0, head_bias=None,
                         sigmoid=False, temp_coef=0.0, temp_every=1,
                         softcap=0.0, dist_bias=None, sink=None):
    """fp32 [T, H, kmaps, dv]; see ops.seq.paged_attention_rows."""
    P, G, ps, krow = kcache.shape
    dk = krow // kmaps
    T = q.shape[0]
    qq = q[:, off_q:off_q + H * kmaps * dk].float().view(T, H, kmaps, dk)
    out = torch.zeros(T, H, kmaps, dv, dtype=torch.float32)
    pos = positions.tolist()
    rep = H // G
    for si, (start, n, slot, pos0) in enumerate(sb.spans()):
        if n == 0:
            continue
        pages = sb.page_table[si].long()
        ctx = pos0 + n
        npg = (ctx + ps - 1) // ps
        kk = kcache[pages[:npg]].float().permute(1, 0, 2, 3).reshape(
            G, npg * ps, kmaps, dk)[:, :ctx]
        if vcache is not None:
            vv = vcache[pages[:npg]].float().permute(1, 0, 2, 3).reshape(
                G, npg * ps, dv)[:, :ctx]
        else:
            vv = kk.reshape(G, ctx, krow)[:, :, :dv]
        kk = kk.repeat_interleave(rep, 0)
        vv = vv.repeat_interleave(rep, 0)
        for t in range(start, start + n):
            i = pos[t]
            j = torch.arange(i + 1)
            seen = ((i - j < window) | (j < keep_first)) if window else j >= 0
            temp = 1.0
            if temp_coef != 0.0:
                temp += temp_coef * math.log((i + 1) // temp_every + 1)
            s = torch.einsum("hmd,hjmd->hmj", qq[t] * (temp * scale),
                             kk[:, :i + 1])
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            if dist_bias is not None:
                dist = (i - j).clamp(max=dist_bias.shape[1] - 1)
                s = s + dist_bias[:, dist].view(H, 1, i + 1)
            if head_bias is not None:
                s = s + head_bias.view(H, 1, 1)
            if sigmoid:
                wgt = torch.sigmoid(s) * seen
            elif sink is not None:
                s = s.masked_fill(~seen, float("-inf"))
                full = torch.cat([s, sink.view(H, 1, 1).expand(H, kmaps, 1)], -1)
                wgt = torch.softmax(full, -1)[..., :-1]
            else:
                wgt = torch.softmax(s.masked_fill(~seen, float("-inf")), -1)
            out[t] = torch.einsum("hmj,hjd->hmd", wgt, vv[:, :i + 1])
    return out


def diff_norm_gate(a, lam, post, gate, eps, out_dtype):
    T, H, _two, dv = a.shape
    o = a[:, :, 0] - lam.reshape(()) * a[:, :, 1]
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * post
    if gate is not None:
        o = o * torch.sigmoid(gate[:, :H * dv].float().view(T, H, dv))
    return o.reshape(T, H * dv).to(out_dtype)


def head_sigmoid_scale(x, gate, out_dtype):
    T, H, R = x.shape
    g = torch.sigmoid(gate[:, :H].float())
    return (x * g[:, :, None]).transpose(0, 1).contiguous().to(out_dtype)


def causal_conv(x, C, w, bias, silu, conv_state, sb):
    taps = w.shape[1]
    K = taps - 1
    xin = x[:, :C].float()
    out = torch.empty(x.shape[0], C, dtype=torch.float32)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        hist = (conv_state[slot].clone() if pos0 > 0
                else torch.zeros(K, C, dtype=torch.float32))
        if 0 < pos0 < K:
            hist[:K - pos0] = 0
        full = torch.cat([hist, xin[start:start + n]], 0)
        acc = torch.zeros(n, C, dtype=torch.float32)
        if bias is not None:
            acc += bias
        for j in range(taps):
            acc += full[j:j + n] * w[:, j]
        out[start:start + n] = F.silu(acc) if silu else acc
        if K:
            conv_state[slot] = full[-K:]
    return out


def rglru_scan(u, gates, br, bi, lam, y, state, sb, decay, out_dtype):
    T, C = u.shape
    nb, _t, two_bw = gates.shape
    bw = two_bw // 2
    gr = gates[:, :, :bw].permute(1, 0, 2).reshape(T, C)
    gi = gates[:, :, bw:].permute(1, 0, 2).reshape(T, C)
    r = torch.sigmoid(gr + br)
    ig = torch.sigmoid(gi + bi)
    la = -decay * F.softplus(lam) * r
    a = torch.exp(la)
    b = torch.sqrt(-torch.expm1(2 * la)) * (ig * u)
    yy = F.gelu(y[:, :C].float(), approximate="tanh")
    out = torch.empty(T, C, dtype=torch.float32)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        S = state[slot].clone() if pos0 > 0 else torch.zeros(C)
        for t in range(start, start + n):
            S = a[t] * S + b[t]
            out[t] = S * yy[t]
        state[slot] = S
    return out.to(out_dtype)


# -- sigmoid attention, minimal gated recurrence, routed experts ---------------
def residual_conv(res, w, conv_state, sb, out_dtype):
    """res + causal_conv(res) over the fp32 rows; see ops.seq.residual_conv."""
    y = causal_conv(res, res.shape[1], w, None, False, conv_state, sb)
    return (res + y).to(out_dtype)


def headnorm_rope_append(proj, H, G, dk, dv, off_k, off_v, qw, kw, freqs,
                         interleaved, eps, positions, kcache, vcache,
                         slot_mapping):
    T = proj.shape[0]
    P, _g, ps, _d = kcache.shape

    def normed(col, n, w):
        x = proj[:, col:col + n * dk].float().view(T, n, dk)
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w
        if freqs is not None:
            x = _rotate(x, positions, freqs, interleaved)
        return x
    q = normed(0, H, qw)
    k = normed(off_k, G, kw).to(kcache.dtype)
    proj[:, :H * dk] = q.reshape(T, H * dk).to(proj.dtype)
    v = proj[:, off_v:off_v + G * dv].view(T, G, dv)
    for t, slot in enumerate(slot_mapping.tolist()):
        if slot < 0:
            continue
        kcache[slot // ps, :, slot % ps] = k[t]
        vcache[slot // ps, :, slot % ps] = v[t]


def mingru_scan(proj, C, state, sb, out_dtype):
    """proj [T, 3C] = gate | candidate | output gate pre-activations."""
    p = proj.float()
    z = torch.sigmoid(p[:, :C])
    keep = torch.sigmoid(-p[:, :C])
    u = p[:, C:2 * C]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = F.silu(p[:, 2 * C:3 * C])
    out = torch.empty(p.shape[0], C, dtype=torch.float32)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        S = state[slot].clone() if pos0 > 0 else torch.zeros(C)
        for t in range(start, start + n):
            S = keep[t] * S + z[t] * cand[t]
            out[t] = S * g[t]
        state[slot] = S
    return out.to(out_dtype)


def relu_squared(x):
    y = x.float().clamp(min=0)
    return (y * y).to(x.dtype)


def moe_route(logits, correction, groups, keep, top, scale):
    T, n = logits.shape
    s = torch.softmax(logits.float(), -1)
    choice = s + correction
    if groups > 1:
        size = n // groups
        gs = choice.view(T, groups, size).max(-1).values
        best = gs.topk(keep, -1).indices
        ok = torch.zeros(T, groups, dtype=torch.bool)
        ok.scatter_(1, best, True)
        ok = ok[:, :, None].expand(T, groups, size).reshape(T, n)
        choice = choice.masked_fill(~ok, float("-inf"))
    idx = choice.topk(top, -1).indices
    return idx.to(torch.int32), s.gather(1, idx) * scale


def moe_dispatch(idx, n_out):
    """rank [T, k]: how many earlier rows chose the same output;
    counts [n_out]."""
    T, k = idx.shape
    flat = idx.reshape(-1).long()
    onehot = F.one_hot(flat, n_out)
    before = onehot.cumsum(0) - onehot
    rank = before.gather(1, flat[:, None]).reshape(T, k)
    return rank.to(torch.int32), onehot.sum(0).to(torch.int32)


def moe_gather(h, idx, rank, base, E, rows):
    xg = torch.zeros(rows, h.shape[1], dtype=h.dtype)
    T, k = idx.shape
    for t in range(T):
        for j in range(k):
            e = int(idx[t, j])
            if e < E:
                xg[int(base[e]) + int(rank[t, j])] = h[t]
    return xg


def moe_combine(y, h, idx, wgt, rank, base, E, shared, out_dtype,
                shared_gate=None):
    T, k = idx.shape
    out = torch.zeros(T, h.shape[1], dtype=torch.float32)
    hf = h.float()
    for t in range(T):
        for j in range(k):
            e = int(idx[t, j])
            src = (y[int(base[e]) + int(rank[t, j])].float() if e < E
                   else hf[t])
            out[t] += wgt[t, j] * src
    if shared is not None:
        sh = shared.float()
        if shared_gate is not None:     # one raw gate value per token
            sh = sh * torch.sigmoid(shared_gate.float()).view(T, 1)
        out += sh
    return out.to(out_dtype)


# -- hashed pair embedding, stream mixing, whole-projection norms, state-space
# -- scan, grouped gated norm, top-k router over logits -----------------------
def embed_pair_hash(ids, embed, table, mul_prev, mul_cur, prev_state, sb):
    """fp32 [T, W]: embed[id] + table[(prev * mul_prev + id * mul_cur) mod n],
    n = rows of table - 1; a sequence's first token takes row n. The last
    token of each portion is left in prev_state[slot] for the next one."""
    x = embed[ids.long()].float()
    n = table.shape[0] - 1
    tok = ids.long()
    rows = torch.empty_like(tok)
    for start, cnt, slot, pos0 in sb.spans():
        if cnt == 0:
            continue
        prev = torch.empty(cnt, dtype=torch.long)
        prev[1:] = tok[start:start + cnt - 1]
        prev[0] = int(prev_state[slot, 0]) if pos0 > 0 else 0
        r = (prev * mul_prev + tok[start:start + cnt] * mul_cur) % n
        if pos0 == 0:
            r[0] = n
        rows[start:start + cnt] = r
        prev_state[slot, 0] = float(tok[start + cnt - 1])
    return x + table[rows].float()


def stream_step(xs, delta, mix, out_w, mult, in_w, norm_w, eps, out_dtype):
    """xs fp32 [T, S, W], in place: with delta, stream t becomes
    sum_s mix[s, t] xs[s] + mult * out_w[t] * delta. Then, with in_w, returns
    the read u = sum_s in_w[s] xs[s] RMS-normed times (1 + norm_w) in
    out_dtype (u itself in fp32 without norm_w)."""
    if delta is not None:
        new = torch.einsum("st,nsw->ntw", mix.float(), xs) \
            + mult * out_w.float()[None, :, None] * delta.float()[:, None, :]
        xs.copy_(new)
    if in_w is None:
        return None
    u = torch.einsum("s,nsw->nw", in_w.float(), xs)
    if norm_w is None:
        return u
    u = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)
    return (u * (1.0 + norm_w.float())).to(out_dtype)


def rms_norm_cols(x, col, n, w, eps, out_dtype):
    v = x[:, col:col + n].float()
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    return (v * w.float()).to(out_dtype)


def rownorm_append(proj, nq, off_k, nk, off_v, nv, qw, kw, eps, kcache,
                   vcache, slot_mapping):
    T = proj.shape[0]
    q = rms_norm_cols(proj, 0, nq, qw, eps, proj.dtype)
    proj[:, :nq] = q
    if kcache is None:
        return
    P, G, ps, dk = kcache.shape
    dv = vcache.shape[3]
    k = rms_norm_cols(proj, off_k, nk, kw, eps, kcache.dtype).view(T, G, dk)
    v = proj[:, off_v:off_v + nv].view(T, G, dv)
    for t, slot in enumerate(slot_mapping.tolist()):
        if slot < 0:
            continue
        kcache[slot // ps, :, slot % ps] = k[t]
        vcache[slot // ps, :, slot % ps] = v[t]


def heads_gate(o, gate, out_dtype):
    """o [H, T, dv], gate [T, >= H*dv] -> [T, H*dv] = o * sigmoid(gate)."""
    H, T, dv = o.shape
    y = o.float().transpose(0, 1).reshape(T, H * dv)
    return (y * torch.sigmoid(gate[:, :H * dv].float())).to(out_dtype)


def heads_major(x, out_dtype):
    """x [T, H, R] -> [H, T, R] in out_dtype."""
    return x.transpose(0, 1).contiguous().to(out_dtype)


def ssd_scan(xbc, dt_raw, dt_bias, A_log, D, state, sb, H, P, N, G):
    """State-space recurrence per head over fp32 xbc [T, H*P + 2*G*N] =
    x | B | C (after convolution and activation):
    dt = softplus(dt_raw + dt_bias); S <- exp(-exp(A_log) dt) S + dt B x^T;
    y = S^T C + D x. state fp32 [slots, H, N, P]. -> fp32 [T, H*P]."""
    T = xbc.shape[0]
    inner = H * P
    x = xbc[:, :inner].view(T, H, P)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:inner + 2 * G * N].view(T, G, N)
    rep = H // G
    dt = F.softplus(dt_raw[:, :H].float() + dt_bias, threshold=20.0)  # [T, H]
    decay = torch.exp(-torch.exp(A_log) * dt)
    out = torch.empty(T, H, P, dtype=torch.float32)
    for start, n, slot, pos0 in sb.spans():
        if n == 0:
            continue
        S = state[slot].clone() if pos0 > 0 else torch.zeros_like(state[slot])
        for t in range(start, start + n):
            Bt = Bm[t].repeat_interleave(rep, 0)                   # [H, N]
            Ct = Cm[t].repeat_interleave(rep, 0)
            S = decay[t].view(H, 1, 1) * S + \
                (dt[t].view(H, 1) * Bt).unsqueeze(2) * x[t].unsqueeze(1)
            out[t] = torch.einsum("hnp,hn->hp", S, Ct) + D.view(H, 1) * x[t]
        state[slot] = S
    return out.view(T, inner)


def gated_group_norm(y, z, w, groups, eps, out_dtype):
    """(y * silu(z)) RMS-normed in `groups` equal parts, times w."""
    T, C = y.shape
    v = y.float() * F.silu(z[:, :C].float())
    v = v.view(T, groups, C // groups)
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    return (v.reshape(T, C) * w.float()).to(out_dtype)


def gelu_erf(x):
    return F.gelu(x.float()).to(x.dtype)


def silu_glu(gate_up):
    Fd = gate_up.shape[-1] // 2
    g, u = gate_up[..., :Fd].float(), gate_up[..., Fd:].float()
    return (F.silu(g) * u).to(gate_up.dtype)


def moe_route_topk(logits, n, bias, top):
    """The `top` largest of the first n columns of logits (+ bias); weights
    are the softmax over the chosen ones only."""
    z = logits[:, :n].float()
    if bias is not None:
        z = z + bias
    val, idx = z.topk(top, -1)
    return idx.to(torch.int32), torch.softmax(val, -1)
