"""Slow float64 oracle for the Muzulorn design, one function per mechanism.

Written from the design's equations only; shares no code with the engine.
Every function takes whole sequences (no cache, no state, no batches), so
anything the engine gets wrong through pages, slots, portions or batching
shows as a difference.

Layer i of a model reads tensors `l<i>.*`; `W` is a dict name -> tensor.
"""
import math

import torch

F64 = torch.float64


def d(t):
    return t.to(F64)


# -- small pieces --------------------------------------------------------------
def rms(x, eps):
    return torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plus_one(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return x / rms(x, eps) * (1.0 + d(w))


def norm_plain(x, w, eps):
    return x / rms(x, eps) * d(w)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def lin(h, W, name, bias=False):
    y = h @ d(W[name]).t()
    return y + d(W[name + ".b"]) if bias else y


# -- embedding ---------------------------------------------------------------
def embed_bigram(cfg, W, toks):
    """Token row plus a hashed row for the (previous, current) pair; the
    first token of a sequence takes the table's last row."""
    x = d(W["embed"])[toks]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        n = bg["buckets"]
        rows = [n] + [(toks[t - 1] * bg["mul_prev"] + toks[t] * bg["mul_cur"]) % n
                      for t in range(1, len(toks))]
        x = x + d(W["bigram"])[rows]
    return x


# -- attention with a bucketed distance bias ------------------------------------
def distance_bucket(n, B, D):
    """Exact below B // 2, logarithmic up to D above, last bucket beyond."""
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + int(math.floor(
        math.log(n / half) / math.log(D / half) * (B - half))))


def biased_attention(m, W, p, h, eps, kv=None):
    """h [T, width] -> [T, width]. kv: (k, v) of another layer to use in
    place of own keys and values. Returns (out, (k, v))."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = norm_plain(lin(h, W, p + "q", True), W[p + "q.norm"], eps)
    if kv is None:
        k = norm_plain(lin(h, W, p + "k", True), W[p + "k.norm"], eps)
        v = lin(h, W, p + "v", True)
        kv = (k, v)
    k, v = kv
    pos = torch.arange(T, dtype=F64)
    qt = m.get("q_temp")
    if qt:
        temp = 1.0 + qt["coef"] * torch.log(
            torch.floor((pos + 1) / qt["every"]) + 1.0)
        q = q * temp[:, None]
    q = q.view(T, H, dk)
    k = k.view(T, G, dk)
    v = v.view(T, G, dv)
    rel = d(W[p + "rel"]) if "bias_max" in m else None
    cap = m.get("softcap")
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        for i in range(T):
            s = (k[:i + 1, g] @ q[i, hh]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            if rel is not None:
                B = rel.shape[0]
                s = s + torch.stack([rel[distance_bucket(i - j, B, m["bias_max"]), hh]
                                     for j in range(i + 1)])
            a = torch.softmax(s, 0)
            out[i, hh] = a @ v[:i + 1, g]
    return lin(out.reshape(T, H * dv), W, p + "o", True), kv


# -- rotation ---------------------------------------------------------------
def rotate_pairs(x, rot):
    """x [T, n]: entries (2i, 2i+1) of the first rot.dims turn by
    position * base^(-2i/dims)."""
    T = x.shape[0]
    n = rot["dims"]
    y = x.clone()
    for t in range(T):
        for i in range(n // 2):
            a = t * rot["base"] ** (-2.0 * i / n)
            u, w = x[t, 2 * i], x[t, 2 * i + 1]
            y[t, 2 * i] = u * math.cos(a) - w * math.sin(a)
            y[t, 2 * i + 1] = w * math.cos(a) + u * math.sin(a)
    return y


# -- latent attention ---------------------------------------------------------
def latent_attention(m, W, p, h, eps, kv=None):
    """Queries through a normed low-rank latent; keys and values expanded
    from a cached normed latent plus one rotated key part shared by all
    heads; sliding window; softmax with a per-head sink in the denominator;
    element-wise sigmoid gate on the concatenated heads."""
    T = h.shape[0]
    H, dk, rd, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = norm_plain(lin(h, W, p + "dq"), W[p + "dq.norm"], eps)
    q = lin(cq, W, p + "uq").view(T, H, dk + rd)
    if kv is None:
        z = lin(h, W, p + "dkv")
        c = norm_plain(z[:, :R], W[p + "dkv.norm"], eps)
        kr = rotate_pairs(z[:, R:], m["rot"])
        kv = (c, kr)
    c, kr = kv
    kn = lin(c, W, p + "uk").view(T, H, dk)
    v = lin(c, W, p + "uv").view(T, H, dv)
    window = (m.get("mask") or {}).get("size")
    sink = d(W[p + "sink"]) if p + "sink" in W else None
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        qr = rotate_pairs(q[:, hh, dk:], m["rot"])
        for i in range(T):
            lo = max(0, i - window + 1) if window else 0
            s = (kn[lo:i + 1, hh] @ q[i, hh, :dk]
                 + kr[lo:i + 1] @ qr[i]) * m["scale"]
            mx = s.max() if sink is None else torch.maximum(s.max(), sink[hh])
            e = torch.exp(s - mx)
            den = e.sum() + (torch.exp(sink[hh] - mx) if sink is not None else 0.0)
            out[i, hh] = (e / den) @ v[lo:i + 1, hh]
    y = out.reshape(T, H * dv) * sigmoid(lin(h, W, p + "g"))
    return lin(y, W, p + "o"), kv


# -- state-space mixer ---------------------------------------------------------
def causal_conv(x, w, b):
    """x [T, C], w [C, taps]: the last column weighs the current token;
    zeros before the sequence."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], 0)
    y = d(b).repeat(T, 1)
    for t in range(T):
        for j in range(taps):
            y[t] = y[t] + d(w)[:, j] * pad[t + j]
    return y


def mamba2(m, W, p, h, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = lin(h, W, p + "in")
    z = proj[:, :inner]
    xbc = silu(causal_conv(proj[:, inner:2 * inner + 2 * G * N],
                           W[p + "conv"], W[p + "conv.b"]))
    dt = softplus(proj[:, 2 * inner + 2 * G * N:] + d(W[p + "dt_bias"]))
    x = xbc[:, :inner].view(T, H, P)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    A = torch.exp(d(W[p + "A_log"]))
    Dd = d(W[p + "D"])
    y = torch.zeros(T, H, P, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = torch.exp(-A[hh] * dt[t, hh]) * S \
                + dt[t, hh] * torch.outer(Bm[t, g], x[t, hh])
            y[t, hh] = S.t() @ Cm[t, g] + Dd[hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = y.view(T, ng, inner // ng)
    y = (y / rms(y, eps)).reshape(T, inner) * d(W[p + "norm"])
    return lin(y, W, p + "o")


# -- feed-forward -------------------------------------------------------------
def dense_ff(W, p, h):
    return lin(gelu_erf(lin(h, W, p + "up")), W, p + "down")


def glu_expert(W, p, h):
    return lin(silu(lin(h, W, p + "gate")) * lin(h, W, p + "up"), W, p + "down")


def moe_ff(mlp, W, p, h):
    T = h.shape[0]
    top = mlp["router"]["top"]
    logits = lin(h, W, p + "router", True)
    out = torch.zeros_like(h)
    for t in range(T):
        best = torch.topk(logits[t], top).indices.tolist()
        wts = torch.softmax(logits[t, best], 0)
        for e, a in zip(best, wts):
            out[t] += a * glu_expert(W, f"{p}e{e}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        gate = sigmoid(lin(h, W, p + "shared.sg"))          # [T, 1]
        out = out + gate * glu_expert(W, p + "shared.", h)
    return out


def feed_forward(mlp, W, p, h):
    if mlp["kind"] == "dense":
        return dense_ff(W, p, h)
    return moe_ff(mlp, W, p, h)


# -- the model -------------------------------------------------------------
def forward(cfg, W, toks, taps=None):
    """Logits [T, vocab] of one sequence; `taps` collects the residual
    stream (the sum of the streams) after every layer."""
    eps = cfg["norm"]["eps"]
    mult = cfg.get("residual_mult", 1.0)
    ns = cfg.get("streams", 0)
    x0 = embed_bigram(cfg, W, toks)
    xs = [x0.clone() for _ in range(max(ns, 1))]
    caches = {}

    def sublayer(q, p, f):
        """One pre-normed sublayer on the stream(s)."""
        nonlocal xs
        w = W[f"{p}norm{q}"]
        if not ns:
            xs = [xs[0] + mult * f(norm_plus_one(xs[0], w, eps))]
            return
        a, o, mix = (d(W[f"{p}hc{q}.{n}"]) for n in ("in", "out", "mix"))
        u = sum(a[s] * xs[s] for s in range(ns))
        y = f(norm_plus_one(u, w, eps))
        xs = [sum(mix[s, t] * xs[s] for s in range(ns)) + mult * o[t] * y
              for t in range(ns)]

    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]

        def mixer(h):
            src = m.get("kv_from")
            kv = caches[src] if src is not None else None
            if L["type"] == "attention":
                y, caches[i] = biased_attention(m, W, p + "mix.", h, eps, kv)
            elif L["type"] == "latent_attention":
                y, caches[i] = latent_attention(m, W, p + "mix.", h, eps, kv)
            elif L["type"] == "mamba2":
                y = mamba2(m, W, p + "mix.", h, eps)
            else:
                raise ValueError(L["type"])
            return y
        sublayer(1, p, mixer)
        if L.get("mlp"):
            sublayer(2, p, lambda h: feed_forward(L["mlp"], W, p + "mlp.", h))
        if taps is not None:
            taps.append(sum(xs))
    x = norm_plus_one(sum(xs), W["final.norm"], eps)
    return x @ d(W["head"]).t()
