"""Helpers for the Muzulorn tests: layer layouts, random checkpoints written
to disk (so the engine loads them through its own config reader and weight
loader) and engines over them. Replay and error helpers are shared with the
other layer-list models' tests."""
import copy
import json
import os

import torch
from safetensors.torch import save_file

from bolatar_util import make_engine, rel_err, replay, TOL  # noqa: F401
from kefesun_util import close_bf16, rel_err_rows  # noqa: F401

# Layouts that avoid equal or trivial sizes: two query heads per kv head,
# dim != vdim, three streams, a window that crosses 16-token pages, a bias
# table whose largest distance lies inside the test prompts, three state
# groups under six heads, norm groups that are not heads.
DENSE = {"kind": "dense", "ff": 100}
MOE = {"kind": "moe", "expert": {"ff": 24},
       "router": {"experts": 5, "top": 3}, "shared": {"ff": 40}}
MOE_BARE = {"kind": "moe", "expert": {"ff": 16},     # one expert per token,
            "router": {"experts": 3, "top": 1},      # no shared expert
            "shared": None}
ATTN = {"type": "attention",
        "mixer": {"heads": 6, "kv_heads": 3, "dim": 20, "vdim": 12,
                  "scale": 0.3, "softcap": 6.0, "bias_max": 37,
                  "q_temp": {"coef": 0.7, "every": 16}},
        "mlp": MOE}
ATTN_PLAIN = {"type": "attention",   # no temperature, cap or distance bias
              "mixer": {"heads": 2, "kv_heads": 2, "dim": 16, "vdim": 24,
                        "scale": 0.25},
              "mlp": None}
LATENT = {"type": "latent_attention",
          "mixer": {"heads": 3, "dim": 24, "rot_dim": 8, "vdim": 20,
                    "kv_rank": 40, "q_rank": 28, "scale": 0.2,
                    "mask": {"size": 19},
                    "rot": {"base": 10000.0, "dims": 8}},
          "mlp": DENSE}
LATENT_FULL = {"type": "latent_attention",   # no window, part of the rotated
               "mixer": {"heads": 2, "dim": 8, "rot_dim": 12, "vdim": 8,
                         "kv_rank": 16, "q_rank": 12, "scale": 0.3,
                         "rot": {"base": 500.0, "dims": 8}},   # part turned
               "mlp": MOE_BARE}
SSM = {"type": "mamba2",
       "mixer": {"heads": 6, "vdim": 10, "state": 12, "groups": 3,
                 "norm_groups": 2, "conv": 3},
       "mlp": MOE}
SSM_BARE = {"type": "mamba2",
            "mixer": {"heads": 2, "vdim": 36, "state": 20, "groups": 1,
                      "norm_groups": 1, "conv": 5},
            "mlp": None}


def with_mlp(layer, mlp):
    out = copy.deepcopy(layer)
    out["mlp"] = copy.deepcopy(mlp)
    return out


def shared_from(layer, src):
    out = copy.deepcopy(layer)
    out["mixer"]["kv_from"] = src
    return out


def make_config(layers, width=72, vocab=131, streams=3, eps=1e-5, mult=0.6,
                bigram=(61, 29, 7)):
    cfg = {"architecture": "Muzulorn", "layers": copy.deepcopy(layers),
           "norm": {"eps": eps}, "residual_mult": mult, "vocab": vocab,
           "width": width}
    if streams:
        cfg["streams"] = streams
    if bigram:
        cfg["embedding"] = {"bigram": {"buckets": bigram[0],
                                       "mul_prev": bigram[1],
                                       "mul_cur": bigram[2]}}
    return cfg


def random_weights(cfg, seed=0, rel_rows=10):
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams", 0)

    def mat(o, i, std=None):
        return torch.randn(o, i, generator=g) * (std or i ** -0.5)

    def uni(shape, lo, hi):
        shape = (shape,) if isinstance(shape, int) else shape
        return lo + (hi - lo) * torch.rand(tuple(shape), generator=g)

    t = {"embed": mat(cfg["vocab"], W, 0.6), "final.norm": uni(W, -0.3, 0.3),
         "head": mat(cfg["vocab"], W)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        t["bigram"] = mat(bg["buckets"] + 1, W, 0.6)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        x = p + "mix."
        for q in (1, 2) if L.get("mlp") else (1,):
            t[f"{p}norm{q}"] = uni(W, -0.3, 0.3)
            if S:
                t[f"{p}hc{q}.in"] = uni(S, 0.2, 0.9)
                t[f"{p}hc{q}.out"] = uni(S, 0.4, 1.3)
                t[f"{p}hc{q}.mix"] = torch.eye(S) * 0.8 + uni((S, S), -0.3, 0.3)
        own = m.get("kv_from") is None
        if L["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            names = [("q", H * dk)] + ([("k", G * dk), ("v", G * dv)] if own else [])
            for n, rows in names:
                t[x + n], t[x + n + ".b"] = mat(rows, W), uni(rows, -0.3, 0.3)
            t[x + "q.norm"] = uni(H * dk, 0.6, 1.8)
            if own:
                t[x + "k.norm"] = uni(G * dk, 0.6, 1.8)
            if "bias_max" in m:
                t[x + "rel"] = uni((rel_rows, H), -1.5, 1.5)
            t[x + "o"], t[x + "o.b"] = mat(W, H * dv), uni(W, -0.2, 0.2)
        elif L["type"] == "latent_attention":
            H, dk, rd, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            R, Q = m["kv_rank"], m["q_rank"]
            t[x + "dq"], t[x + "dq.norm"] = mat(Q, W), uni(Q, 0.6, 1.6)
            t[x + "uq"] = mat(H * (dk + rd), Q)
            if own:
                t[x + "dkv"], t[x + "dkv.norm"] = mat(R + rd, W), uni(R, 0.6, 1.6)
            t[x + "uk"], t[x + "uv"] = mat(H * dk, R), mat(H * dv, R)
            t[x + "sink"] = uni(H, -1.0, 2.0)
            t[x + "g"], t[x + "o"] = mat(H * dv, W), mat(W, H * dv)
        else:
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            C = H * P + 2 * G * N
            t[x + "in"] = mat(2 * H * P + 2 * G * N + H, W)
            t[x + "conv"] = uni((C, m["conv"]), -0.6, 0.9)
            t[x + "conv.b"] = uni(C, -0.3, 0.3)
            t[x + "dt_bias"] = uni(H, -2.5, 0.5)
            t[x + "A_log"] = uni(H, -2.0, 1.0)
            t[x + "D"] = uni(H, 0.3, 1.5)
            t[x + "norm"] = uni(H * P, 0.6, 1.5)
            t[x + "o"] = mat(W, H * P)
        mlp = L.get("mlp")
        y = p + "mlp."
        if mlp and mlp["kind"] == "dense":
            t[y + "up"], t[y + "down"] = mat(mlp["ff"], W), mat(W, mlp["ff"])
        elif mlp:
            F, n = mlp["expert"]["ff"], mlp["router"]["experts"]
            for e in range(n):
                t[f"{y}e{e}.gate"], t[f"{y}e{e}.up"] = mat(F, W), mat(F, W)
                t[f"{y}e{e}.down"] = mat(W, F)
            t[y + "router"] = mat(n, W, 2.0 * W ** -0.5)
            t[y + "router.b"] = uni(n, -0.5, 0.5)
            if mlp.get("shared"):
                Fs = mlp["shared"]["ff"]
                t[y + "shared.gate"], t[y + "shared.up"] = mat(Fs, W), mat(Fs, W)
                t[y + "shared.down"] = mat(W, Fs)
                t[y + "shared.sg"] = mat(1, W)
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
    g = torch.Generator().manual_seed(5000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def calm_routers(W):
    """For comparisons in bf16: sharpen every router, so that the experts at
    the edge of being chosen carry next to no weight and a choice flipped by
    rounding does not show."""
    for k in W:
        if k.endswith(".router"):
            W[k] = (W[k].float() * 6).to(W[k].dtype)
