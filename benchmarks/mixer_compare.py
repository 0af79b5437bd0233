"""Prefill and decode throughput of a layer-list design (Bolatar, Fironex,
Kefesun or Muzulorn) beside the dense-attention Llama layout - or, for a design with
routed experts, the Mixtral layout - at equal width, depth, feed-forward
size and vocabulary, random weights, one GPU, through the engine's own
add_request/step loop (chunked prefill, then hipGraph decode).

    python bench.py --mixer-compare [--mixer-sizes small,medium]
                    [--mixer-model bolatar|fironex|kefesun|muzulorn]
                    [--mixer-baseline llama|mixtral|kefesun]

Prints one JSON line: per size and model, prefill tokens/s (B prompts of
ISL tokens until every request has its first token) and decode tokens/s
(the following steps, all requests decoding).
"""
from __future__ import annotations

import json
import time

import torch

SIZES = {
    # width, layers, ff, prompts, isl, decode batch, decode steps
    "small": dict(width=1024, layers=4, ff=4096, prompts=4, isl=1024,
                  conc=32, steps=64),
    "medium": dict(width=2048, layers=8, ff=8192, prompts=4, isl=2048,
                   conc=32, steps=64),
    "wide": dict(width=4096, layers=4, ff=14336, prompts=2, isl=2048,
                 conc=64, steps=48),
}
VOCAB = 32000


def bolatar_config(width, layers, ff):
    from dynamo_amd.engine.config import ModelConfig
    hd = 128
    H = width // hd
    mlp = {"kind": "dense", "ff": ff, "limit": 7.0}
    delta = {"type": "delta", "mlp": mlp,
             "mixer": {"heads": H, "kv_heads": max(1, H // 2), "dim": hd,
                       "vdim": hd, "conv": 4}}
    par = {"type": "parallel", "mlp": mlp,
           "mixer": {"left": {"heads": H, "kv_heads": max(1, H // 4),
                              "dim": hd, "vdim": hd, "scale": hd ** -0.5,
                              "q_temp": {"coef": 0.1, "every": 1024}},
                     "right": {"heads": width // 64, "dim": 64}}}
    mlstm = {"type": "mlstm", "mlp": mlp,
             "mixer": {"heads": max(1, H // 2), "dim": hd, "vdim": 2 * hd,
                       "gate_cap": 15.0}}
    pattern = [delta, par, mlstm, delta]
    specs = [pattern[i % 4] for i in range(layers)]
    return ModelConfig(name=f"bolatar-w{width}", arch="bolatar",
                       hidden_size=width, vocab_size=VOCAB, max_position=8192,
                       num_layers=layers, rms_eps=1e-6, learned_pos_emb=True,
                       layer_specs=specs, embed_scale=1.0, logit_softcap=30.0,
                       intermediate_size=0, num_q_heads=1, num_kv_heads=1,
                       head_dim=1)


def fironex_config(width, layers, ff):
    """Layer pattern: differential attention under a 1024-token window,
    latent attention, a second latent layer on the first one's cache, and
    a gated linear recurrent unit; head sizes of current models."""
    from dynamo_amd.engine.config import ModelConfig
    H = width // 128
    mlp = {"kind": "dense", "ff": ff}
    rot = {"base": 500000.0, "dims": 64,
           "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0,
                       "original": 8192}}
    specs = []
    for i in range(layers):
        k = i % 4
        if k == 0:
            specs.append({"type": "attention", "mlp": mlp, "mixer": {
                "heads": H, "kv_heads": max(1, H // 4), "dim": 64,
                "vdim": 128, "scale": 0.125, "diff": 0.5,
                "mask": {"size": 1024}, "rot": rot}})
        elif k in (1, 2):
            m = {"heads": H, "dim": 128, "rot_dim": 64, "vdim": 128,
                 "kv_rank": 512, "scale": 192 ** -0.5,
                 "rot": {"base": 10000.0, "dims": 64}}
            if k == 2:
                m["kv_from"] = i - 1
            specs.append({"type": "latent_attention", "mlp": mlp, "mixer": m})
        else:
            specs.append({"type": "rglru", "mlp": mlp, "mixer": {
                "width": width, "blocks": H, "conv": 4}})
    return ModelConfig(name=f"fironex-w{width}", arch="fironex",
                       hidden_size=width, vocab_size=VOCAB, max_position=8192,
                       num_layers=layers, rms_eps=1e-6, residual_mult=0.7,
                       tie_embeddings=True, norm="layernorm",
                       layer_specs=specs, intermediate_size=0, num_q_heads=1,
                       num_kv_heads=1, head_dim=1)


def kefesun_config(width, layers, ff):
    """Layer pattern: three sigmoid-attention layers (128-wide heads, four
    query heads per kv head, a 1024-token window that keeps the first four
    tokens) to one minimal gated recurrent unit of the model's width; every
    layer with eight routed experts and four identity experts in three
    groups of which two stay in the running, two per token, and a shared
    expert. A token's active feed-forward
    weights equal those of a dense gated feed-forward of size ff."""
    from dynamo_amd.engine.config import ModelConfig
    H = width // 128
    mlp = {"kind": "moe", "expert": {"ff": ff // 2},
           "router": {"experts": 8, "identity": 4, "top": 2, "scale": 1.0,
                      "groups": {"count": 3, "keep": 2}},
           "shared": {"ff": ff // 2}}
    attn = {"type": "attention", "mlp": mlp, "mixer": {
        "heads": H, "kv_heads": max(1, H // 4), "dim": 128, "vdim": 128,
        "scale": 128 ** -0.5, "mask": {"size": 1024, "keep_first": 4},
        "rot": {"base": 10000.0, "dims": 64}}}
    gru = {"type": "mingru", "mlp": mlp, "mixer": {"width": width}}
    specs = [gru if i % 4 == 2 else attn for i in range(layers)]
    return ModelConfig(name=f"kefesun-w{width}", arch="kefesun",
                       hidden_size=width, vocab_size=VOCAB, max_position=8192,
                       num_layers=layers, rms_eps=1e-6, embed_scale=1.0,
                       conv_taps=4, tie_embeddings=True, norm="layernorm",
                       layer_specs=specs, intermediate_size=0, num_q_heads=1,
                       num_kv_heads=1, head_dim=1)


def muzulorn_config(width, layers, ff):
    """Layer pattern: capped attention with a distance table (128-wide
    heads, four query heads per kv head), latent attention under a
    1024-token window (rank 512 + 64 rotated, queries through a latent of
    three quarters of the width), a state-space layer (64-wide heads over
    twice the width, state 128, eight groups), and a second attention layer
    on the first one's keys and values; two residual streams; every layer
    with eight gated experts of size ff / 2, two per token, and a gated
    shared expert - the expert form and sizes of the Mixtral layout."""
    from dynamo_amd.engine.config import ModelConfig
    H = width // 128
    mlp = {"kind": "moe", "expert": {"ff": ff // 2},
           "router": {"experts": 8, "top": 2}, "shared": {"ff": ff // 2}}
    attn = {"heads": H, "kv_heads": max(1, H // 4), "dim": 128, "vdim": 128,
            "scale": 128 ** -0.5, "softcap": 30.0, "bias_max": 4096,
            "buckets": 32, "q_temp": {"coef": 0.1, "every": 1024}}
    lat = {"heads": H, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512,
           "q_rank": 3 * width // 4, "scale": 192 ** -0.5,
           "mask": {"size": 1024}, "rot": {"base": 10000.0, "dims": 64}}
    sh = 2 * width // 64
    ssm = {"heads": sh, "vdim": 64, "state": 128, "groups": min(8, sh),
           "norm_groups": min(8, sh), "conv": 4}
    specs = []
    for i in range(layers):
        k = i % 4
        if k == 0:
            specs.append({"type": "attention", "mlp": mlp, "mixer": attn})
        elif k == 1:
            specs.append({"type": "latent_attention", "mlp": mlp, "mixer": lat})
        elif k == 2:
            specs.append({"type": "mamba2", "mlp": mlp, "mixer": ssm})
        else:
            specs.append({"type": "attention", "mlp": mlp,
                          "mixer": dict(attn, kv_from=i - 3)})
    return ModelConfig(name=f"muzulorn-w{width}", arch="muzulorn",
                       hidden_size=width, vocab_size=VOCAB, max_position=8192,
                       num_layers=layers, rms_eps=1e-6, residual_mult=0.5,
                       residual_streams=2,
                       pair_hash={"buckets": 65521, "mul_prev": 31,
                                  "mul_cur": 17},
                       tie_embeddings=False, norm="rmsnorm",
                       layer_specs=specs, intermediate_size=0, num_q_heads=1,
                       num_kv_heads=1, head_dim=1)


def mixtral_config(width, layers, ff):
    """Eight gated experts of size ff / 2, two per token: a token's active
    feed-forward weights equal a dense gated feed-forward of size ff."""
    from dynamo_amd.engine.config import ModelConfig
    H = width // 128
    return ModelConfig(name=f"mixtral-w{width}", arch="mixtral",
                       hidden_size=width, intermediate_size=ff // 2,
                       num_layers=layers, num_q_heads=H,
                       num_kv_heads=max(1, H // 4), head_dim=128,
                       vocab_size=VOCAB, max_position=8192, rope_theta=1e4,
                       num_experts=8, num_experts_per_tok=2)


def llama_config(width, layers, ff):
    from dynamo_amd.engine.config import ModelConfig
    H = width // 128
    return ModelConfig(name=f"llama-w{width}", arch="llama", hidden_size=width,
                       intermediate_size=ff, num_layers=layers, num_q_heads=H,
                       num_kv_heads=max(1, H // 4), head_dim=128,
                       vocab_size=VOCAB, max_position=8192, rope_theta=1e4)


def measure(mc, s, device):
    from dynamo_amd.engine import EngineConfig, LLMEngine, SamplingParams
    n = max(s["prompts"], s["conc"])
    cfg = EngineConfig(model=mc, device=device, dtype="bfloat16",
                       page_size=64, max_num_seqs=n,
                       max_batched_tokens=s["prompts"] * s["isl"],
                       max_model_len=s["isl"] + s["steps"] + 128,
                       kv_pool_pages=n * ((s["isl"] + s["steps"]) // 64 + 3),
                       enable_prefix_caching=False, kv_events=False)
    eng = LLMEngine(cfg, seed=0)
    g = torch.Generator().manual_seed(0)

    def prompts(k, tag):
        for i in range(k):
            toks = torch.randint(0, mc.vocab_size, (s["isl"],), generator=g)
            eng.add_request(f"{tag}{i}", toks.tolist(),
                            SamplingParams(max_tokens=s["steps"] + 8,
                                           ignore_eos=True))

    def drain_until(pred):
        while eng.has_work() and not pred():
            eng.step()
        torch.cuda.synchronize()

    def first_tokens():
        return all(r.output_tokens for r in eng.requests.values())

    # warm-up: one prompt through prefill and a few decode steps
    prompts(1, "w")
    drain_until(first_tokens)
    for _ in range(3):
        eng.step()
    for rid in list(eng.requests):
        eng.abort(rid)
    torch.cuda.synchronize()

    prompts(s["prompts"], "p")
    t0 = time.perf_counter()
    drain_until(first_tokens)
    prefill_s = time.perf_counter() - t0
    # fill up to the decode batch (untimed), then time pure decode steps
    prompts(s["conc"] - s["prompts"], "d")
    drain_until(first_tokens)
    for _ in range(4):           # graph capture for this batch size
        eng.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    done = 0
    for _ in range(s["steps"] - 8):
        done += len(eng.step())
    torch.cuda.synchronize()
    decode_s = time.perf_counter() - t0
    out = {"prefill_tok_s": round(s["prompts"] * s["isl"] / prefill_s, 1),
           "decode_tok_s": round(done / decode_s, 1),
           "decode_ms_per_step": round(1000 * decode_s / (s["steps"] - 8), 3)}
    del eng
    torch.cuda.empty_cache()
    return out


def run(sizes, device="cuda:0", model="bolatar", with_llama=True,
        baseline=None):
    res = {}
    make = {"bolatar": bolatar_config, "fironex": fironex_config,
            "kefesun": kefesun_config, "muzulorn": muzulorn_config}[model]
    baseline = baseline or ("mixtral" if model in ("kefesun", "muzulorn")
                            else "llama")
    base = {"llama": llama_config, "mixtral": mixtral_config,
            "kefesun": kefesun_config}[baseline]
    for name in sizes:
        s = SIZES[name]
        args = (s["width"], s["layers"], s["ff"])
        res[name] = {
            "shape": {k: s[k] for k in ("width", "layers", "ff", "prompts",
                                        "isl", "conc")},
            model: measure(make(*args), s, device)}
        if with_llama:
            res[name][baseline] = measure(base(*args), s, device)
        print(f"# {name}: {json.dumps(res[name])}", flush=True)
    print(json.dumps({"metric": "mixer_compare", "dtype": "bf16",
                      "data": "synthetic", "sizes": res}), flush=True)
    return res
