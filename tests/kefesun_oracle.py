"""Slow float64 oracle for the Kefesun design, one function per mechanism.

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
def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * d(w)


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * d(w)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def time_conv(h, w):
    """h [T, C], w [C, taps]: y_t = sum_j w[:, j] h_(t - taps + 1 + j), with
    zeros before the first token. The last column weighs the current token."""
    T, C = h.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), h], 0)
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            y[t] += d(w)[:, j] * pad[t + j]
    return y


def rotate_half(x, rot):
    """x [T, n_vec, size]: entries i and i + dims/2 of the first rot.dims
    form a pair turned by angle position * base^(-2i/dims)."""
    T = x.shape[0]
    n = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / n) for i in range(n // 2)],
                     dtype=F64)
    ang = torch.arange(T, dtype=F64)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    y = x.clone()
    a, b = x[..., :n // 2], x[..., n // 2:n]
    y[..., :n // 2] = a * c - b * s
    y[..., n // 2:n] = b * c + a * s
    return y


def visible(T, window, keep_first):
    """[T, T] bool: row i sees column j when j <= i and the key is either
    inside the window (i - j < window) or one of the first keep_first."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


# -- mixers --------------------------------------------------------------------
def sigmoid_attention_mixer(h, W, p, m, eps):
    """Grouped-query attention whose weights are sigmoid(score + head bias),
    not normalised over the keys."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ d(W[p + "q"]).t() + d(W[p + "q.b"])).view(T, H, dk)
    k = (h @ d(W[p + "k"]).t() + d(W[p + "k.b"])).view(T, G, dk)
    v = (h @ d(W[p + "v"]).t() + d(W[p + "v.b"])).view(T, G, dv)
    q = rms_norm(q, W[p + "q.norm"], eps)
    k = rms_norm(k, W[p + "k.norm"], eps)
    if m.get("rot"):
        q, k = rotate_half(q, m["rot"]), rotate_half(k, m["rot"])
    mask = m.get("mask") or {}
    ok = visible(T, mask.get("size"), mask.get("keep_first", 0))
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].t()) * m["scale"] + d(W[p + "pb"])[hh]
        wgt = torch.where(ok, sigmoid(s), torch.zeros((), dtype=F64))
        heads.append(wgt @ v[:, g])
    return torch.cat(heads, -1) @ d(W[p + "o"]).t()


def mingru_mixer(h, W, p, m):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t with gate and candidate read from
    the current token only; c = u + 1/2 for u >= 0, sigmoid(u) below."""
    T = h.shape[0]
    z = sigmoid(h @ d(W[p + "z"]).t() + d(W[p + "z.b"]))
    u = h @ d(W[p + "x"]).t() + d(W[p + "x.b"])
    cand = torch.where(u >= 0, u + 0.5, sigmoid(u))
    g = h @ d(W[p + "g"]).t()
    S = torch.zeros(m["width"], dtype=F64)
    out = torch.zeros(T, m["width"], dtype=F64)
    for t in range(T):
        S = (1 - z[t]) * S + z[t] * cand[t]
        out[t] = S * (g[t] * sigmoid(g[t]))
    return out @ d(W[p + "o"]).t()


def relu_squared_expert(h, up, down):
    a = torch.clamp(h @ d(up).t(), min=0)
    return (a * a) @ d(down).t()


def route(h, W, p, r):
    """Chosen experts [T, top] and their weights. Softmax over all router
    outputs; the choice adds a correction and is limited to the best groups
    of neighbouring outputs; the weights are the uncorrected scores."""
    s = torch.softmax(h @ d(W[p + "router"]).t(), -1)
    choice = s + d(W[p + "correction"])
    T, n = s.shape
    grp = r.get("groups") or {"count": 1, "keep": 1}
    size = n // grp["count"]
    gscore = choice.view(T, grp["count"], size).max(-1).values
    best = gscore.topk(grp["keep"], -1).indices
    allowed = torch.zeros(T, grp["count"], dtype=torch.bool)
    allowed.scatter_(1, best, True)
    allowed = allowed[:, :, None].expand(T, grp["count"], size).reshape(T, n)
    choice = choice.masked_fill(~allowed, -math.inf)
    idx = choice.topk(r["top"], -1).indices
    return idx, s.gather(1, idx) * r["scale"]


def moe_feed_forward(h, W, p, mlp):
    r = mlp["router"]
    E = r["experts"]
    idx, wgt = route(h, W, p, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wgt[t]):
            if e >= E:                       # identity expert
                out[t] += w * h[t]
            else:
                out[t] += w * relu_squared_expert(
                    h[t:t + 1], W[f"{p}e{e}.up"], W[f"{p}e{e}.down"])[0]
    if mlp.get("shared"):
        out = out + relu_squared_expert(h, W[p + "shared.up"],
                                        W[p + "shared.down"])
    return out


# -- the model -----------------------------------------------------------------
def forward(cfg, W, tokens, taps=None):
    """Logits [T, vocab] (float64) of one whole sequence. `taps`, a list,
    receives the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = d(W["embed"])[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = x + time_conv(x, W[p + "canon1"])
        if L["type"] == "attention":
            y = sigmoid_attention_mixer(h, W, p + "mix.", m, eps)
        elif L["type"] == "mingru":
            y = mingru_mixer(h, W, p + "mix.", m)
        else:
            raise ValueError(L["type"])
        x = x + layer_norm(y, W[p + "norm1"], eps)
        if L.get("mlp"):
            h = x + time_conv(x, W[p + "canon2"])
            x = x + layer_norm(moe_feed_forward(h, W, p + "mlp.", L["mlp"]),
                               W[p + "norm2"], eps)
        if taps is not None:
            taps.append(x.clone())
    x = layer_norm(x, W["final.norm"], eps)
    return x @ d(W["embed"]).t()
