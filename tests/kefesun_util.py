"""Helpers for the Kefesun tests: layer layouts, random checkpoints written
to disk (so the engine loads them through its own config reader and weight
loader) and engines over them. Replay and error helpers are shared with the
other layer-list models' tests."""
import copy
import json
import os

import torch
from safetensors.torch import save_file

from bolatar_util import make_engine, rel_err, replay, TOL  # noqa: F401

# Layouts that avoid equal or trivial sizes: three query heads per kv head,
# dim != vdim, partial rotation, a window that crosses 16-token pages, more
# kept first keys than one, groups of three router outputs of which two
# survive, one identity expert, shared and routed experts of other sizes.
MOE = {"kind": "moe", "expert": {"ff": 40},
       "router": {"experts": 5, "identity": 1, "top": 3, "scale": 1.7,
                  "groups": {"count": 3, "keep": 2}},
       "shared": {"ff": 56}}
MOE_PLAIN = {"kind": "moe", "expert": {"ff": 24},     # no groups, no identity,
             "router": {"experts": 4, "identity": 0,  # no shared expert
                        "top": 2, "scale": 1.0,
                        "groups": {"count": 1, "keep": 1}},
             "shared": None}
MOE_IDENT = {"kind": "moe", "expert": {"ff": 32},     # mostly identity experts
             "router": {"experts": 2, "identity": 4, "top": 1, "scale": 0.6,
                        "groups": {"count": 2, "keep": 1}},
             "shared": {"ff": 16}}
ATTN = {"type": "attention",
        "mixer": {"heads": 6, "kv_heads": 2, "dim": 24, "vdim": 40,
                  "scale": 0.21, "mask": {"size": 19, "keep_first": 3},
                  "rot": {"base": 10000.0, "dims": 12}},
        "mlp": MOE}
ATTN_FULL = {"type": "attention",   # no window, whole head rotated, no mlp
             "mixer": {"heads": 2, "kv_heads": 2, "dim": 16, "vdim": 8,
                       "scale": 0.3, "rot": {"base": 500.0, "dims": 16}},
             "mlp": None}
GRU = {"type": "mingru", "mixer": {"width": 72}, "mlp": MOE_PLAIN}
GRU_BARE = {"type": "mingru", "mixer": {"width": 130}, "mlp": None}


def with_mlp(layer, mlp):
    out = copy.deepcopy(layer)
    out["mlp"] = copy.deepcopy(mlp)
    return out


def make_config(layers, width=96, vocab=157, taps=3, eps=1e-5, scale=4.5):
    return {"architecture": "Kefesun", "canon": {"taps": taps},
            "embedding": {"scale": scale}, "layers": copy.deepcopy(layers),
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, taps = cfg["width"], cfg["canon"]["taps"]

    def mat(o, i, std=None):
        return torch.randn(o, i, generator=g) * (std or i ** -0.5)

    def uni(shape, lo, hi):
        shape = (shape,) if isinstance(shape, int) else shape
        return lo + (hi - lo) * torch.rand(tuple(shape), generator=g)

    t = {"embed": mat(cfg["vocab"], W, 0.25), "final.norm": uni(W, 0.7, 1.3)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = uni(W, 0.7, 1.3)
        t[p + "canon1"] = uni((W, taps), -0.4, 0.4)
        x = p + "mix."
        if L["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[x + "q"], t[x + "q.b"] = mat(H * dk, W), uni(H * dk, -0.3, 0.3)
            t[x + "k"], t[x + "k.b"] = mat(G * dk, W), uni(G * dk, -0.3, 0.3)
            t[x + "v"], t[x + "v.b"] = mat(G * dv, W), uni(G * dv, -0.3, 0.3)
            t[x + "q.norm"], t[x + "k.norm"] = uni(dk, 0.6, 1.6), uni(dk, 0.6, 1.6)
            t[x + "pb"] = uni(H, -3.0, -0.5)
            t[x + "o"] = mat(W, H * dv)
        else:
            C = m["width"]
            t[x + "z"], t[x + "z.b"] = mat(C, W), uni(C, -1.0, 1.0)
            t[x + "x"], t[x + "x.b"] = mat(C, W), uni(C, -0.5, 0.5)
            t[x + "g"], t[x + "o"] = mat(C, W), mat(W, C)
        mlp = L.get("mlp")
        if mlp:
            r, F = mlp["router"], mlp["expert"]["ff"]
            n = r["experts"] + r.get("identity", 0)
            y = p + "mlp."
            t[p + "norm2"] = uni(W, 0.7, 1.3)
            t[p + "canon2"] = uni((W, taps), -0.4, 0.4)
            for e in range(r["experts"]):
                t[f"{y}e{e}.up"], t[f"{y}e{e}.down"] = mat(F, W), mat(W, F)
            t[y + "router"] = mat(n, W, 2.0 * W ** -0.5)
            # corrections of the size of the scores, of both signs: a choice
            # score below zero must still beat an excluded group's
            t[y + "correction"] = uni(n, -0.4, 0.2)
            if mlp.get("shared"):
                S = mlp["shared"]["ff"]
                t[y + "shared.up"], t[y + "shared.down"] = mat(S, W), mat(W, S)
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
    g = torch.Generator().manual_seed(3000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def calm_routers(W):
    """For comparisons in bf16: sharpen every router and shrink its
    corrections, so that the experts at the edge of being chosen carry
    next to no weight and a choice flipped by rounding does not show."""
    for k in W:
        if k.endswith(".router"):
            W[k] = (W[k].float() * 6).to(W[k].dtype)
        elif k.endswith(".correction"):
            W[k] = (W[k].float() * 0.05).to(W[k].dtype)


def rel_err_rows(got, want):
    """rel_err of every position (RMS difference over the vocabulary, mean
    removed, relative to the RMS spread of the expected logits)."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()


def close_bf16(got, want, tol=0.1):
    """bf16 against the float64 oracle on small random models: nine
    positions in ten within `tol`, and the median well below. A router
    whose two best candidates are a rounding error apart may pick the other
    one in bf16, which moves single positions by much more; the float32
    comparisons are the sharp ones."""
    e = rel_err_rows(got, want)
    return bool(e.median() < 0.6 * tol and (e < tol).float().mean() >= 0.9)
