"""Muzulorn through the engine against the slow oracle
(tests/muzulorn_oracle): each mechanism alone, whole prompts against
portions and single-token decoding, mixed batches, reuse of cache pages and
state slots, keys far back, at page borders, at the window's edges and at
the last distance bucket, the first tokens, long decoding, other sizes and
stream counts, and greedy generation through add_request/step. Runs on CPU;
the same cases run on the HIP kernels under the gpu marker."""
import copy
import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(__file__))
import muzulorn_oracle as oracle  # noqa: E402
import muzulorn_util as U  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
# layer 4 reads layer 0's keys and values, layer 6 the latent rows of layer 1
FULL = [U.ATTN, U.LATENT, U.SSM, U.ATTN_PLAIN, U.shared_from(U.ATTN, 0),
        U.LATENT_FULL, U.shared_from(U.with_mlp(U.LATENT, U.MOE_BARE), 1),
        U.SSM_BARE]


@pytest.fixture(scope="module")
def full_ckpt(tmp_path_factory):
    cfg = U.make_config(FULL)
    W = U.random_weights(cfg, 1)
    return U.write_checkpoint(tmp_path_factory.mktemp("full"), cfg, W), cfg, W


# in bf16 a router whose best two logits lie a rounding error apart may pick
# the other expert; with one expert per token that moves a position by more
# than any kernel fault would, so the bf16 comparison leaves that layout out
CALM = [L if (L.get("mlp") or {}).get("router", {}).get("top") != 1
        else U.with_mlp(L, U.DENSE) for L in FULL]


@pytest.fixture(scope="module")
def calm_ckpt(tmp_path_factory):
    cfg = U.make_config(CALM)
    W = U.random_weights(cfg, 1)
    U.calm_routers(W)
    return U.write_checkpoint(tmp_path_factory.mktemp("calm"), cfg, W), cfg, W


def _case(tmp_path, layers, seed=0, edit=None, rel_rows=10, **kw):
    cfg = U.make_config(layers, **kw)
    W = U.random_weights(cfg, seed, rel_rows)
    if edit:
        edit(W)
    return U.write_checkpoint(tmp_path, cfg, W), cfg, W


def _check(eng, cfg, W, toks, plans, tol=U.TOL["float32"], want=None):
    want = oracle.forward(cfg, W, toks) if want is None else want
    for k, sizes in enumerate(plans):
        got = U.replay(eng, f"r{k}", toks, sizes)
        assert U.rel_err(got, want) < tol, sizes
    return want


# -- each mechanism alone ------------------------------------------------------
LAYERS_ALONE = {
    "attention": [U.with_mlp(U.ATTN, None)], "attention_plain": [U.ATTN_PLAIN],
    "attention_shared": [U.with_mlp(U.ATTN, None),
                         U.shared_from(U.with_mlp(U.ATTN, None), 0)],
    "latent": [U.with_mlp(U.LATENT, None)],
    "latent_full": [U.with_mlp(U.LATENT_FULL, None)],
    "ssm": [U.with_mlp(U.SSM, None)], "ssm_bare": [U.SSM_BARE],
    "dense": [U.with_mlp(U.SSM_BARE, U.DENSE)],
    "moe": [U.with_mlp(U.SSM_BARE, U.MOE)],
    "moe_bare": [U.with_mlp(U.SSM_BARE, U.MOE_BARE)]}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(LAYERS_ALONE))
def test_single_mechanism(tmp_path, device, name):
    path, cfg, W = _case(tmp_path, LAYERS_ALONE[name], seed=3)
    toks = U.tokens_for(cfg, 45, 0)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[45], [1]])


def test_residual_stream_after_every_layer(full_ckpt):
    """The model's layer taps (sum of the streams) against the oracle's."""
    from dynamo_amd.engine.scheduler import ScheduledSeq, SchedulerOutput
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 30, 1)
    want = []
    oracle.forward(cfg, W, toks, want)
    eng = U.make_engine(path, "cpu")
    eng.replay_step([("t", [], [])])
    req = eng.requests["t"]
    req.prompt_tokens.extend(toks)
    req.kv.ensure_capacity(len(toks))
    sched = SchedulerOutput()
    sched.prefills.append(ScheduledSeq(req, len(toks), False))
    ids, meta = eng.runner.prepare(sched)
    got = []
    with torch.inference_mode():
        eng.runner.model.forward(ids, eng.runner.kv_pool, meta, tap=got)
    assert len(got) == len(want) == len(FULL)
    for a, b in zip(got, want):
        assert float((a.double() - b).abs().max()) < 2e-4 * float(b.abs().max())


# -- ops against the oracle's pieces -------------------------------------------
def _span(spans, dev="cpu", page_table=None, num_decode=0):
    """SeqBatch of [(rows, slot, first position)] laid out back to back."""
    from dynamo_amd.ops import seq as sops
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
    start, host, tok = 0, [], []
    for k, (n, slot, pos0) in enumerate(spans):
        host.append((start, n, slot, pos0))
        tok += [k] * n
        start += n
    cols = list(zip(*host))
    return sops.SeqBatch(i32(tok), i32(cols[0]), i32(cols[1]), i32(cols[2]),
                         i32(cols[3]), page_table=page_table,
                         num_decode=num_decode, host=host)


@pytest.mark.parametrize("B,D", [(10, 37), (16, 120), (7, 9), (2, 2), (32, 128)])
def test_distance_table_against_buckets(B, D):
    from dynamo_amd.models.mixers import distance_bias_table
    rel = torch.arange(B * 3, dtype=torch.float32).view(B, 3)
    tab = distance_bias_table(rel, D)
    assert tab.shape == (3, D + 1)
    for n in range(D + 1):
        assert torch.equal(tab[:, n], rel[oracle.distance_bucket(n, B, D)]), n
    # beyond the table every distance is the last bucket
    assert oracle.distance_bucket(10 * D + 3, B, D) == B - 1
    assert torch.equal(tab[:, D], rel[B - 1])


@pytest.mark.parametrize("device", DEVICES)
def test_pair_hash_embedding_carries_the_previous_token(device):
    """Portions of two sequences in used slots: the first row of a later
    portion hashes with the token the slot kept, a sequence's first token
    takes the last table row whatever the slot holds."""
    from dynamo_amd.ops import seq as sops
    g = torch.Generator().manual_seed(0)
    V, W, n = 50, 24, 13
    embed = torch.randn(V, W, generator=g).to(device)
    table = torch.randn(n + 1, W, generator=g).to(device)
    state = torch.full((3, 1), 7.0, device=device)
    a = torch.randint(0, V, (9,), generator=g).tolist()
    b = torch.randint(0, V, (4,), generator=g).tolist()

    def want(toks):
        rows = [n] + [(toks[i - 1] * 31 + toks[i] * 5) % n
                      for i in range(1, len(toks))]
        return embed.cpu()[toks] + table.cpu()[rows]
    ids = lambda x: torch.tensor(x, dtype=torch.int32, device=device)  # noqa: E731
    o1 = sops.embed_pair_hash(ids(a[:4] + b[:1]), embed, table, 31, 5, state,
                              _span([(4, 2, 0), (1, 0, 0)], device))
    o2 = sops.embed_pair_hash(ids(b[1:2] + a[4:]), embed, table, 31, 5, state,
                              _span([(1, 0, 1), (5, 2, 4)], device))
    o3 = sops.embed_pair_hash(ids(b[2:]), embed, table, 31, 5, state,
                              _span([(2, 0, 2)], device))
    ga = torch.cat([o1[:4], o2[1:]]).cpu()
    gb = torch.cat([o1[4:], o2[:1], o3]).cpu()
    assert torch.allclose(ga, want(a), atol=1e-6)
    assert torch.allclose(gb, want(b), atol=1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S", [1, 2, 3, 4, 5])
def test_stream_step(device, S):
    from dynamo_amd.ops import seq as sops
    g = torch.Generator().manual_seed(S)
    T, W = 5, 37
    xs = torch.randn(T, S, W, generator=g)
    delta = torch.randn(T, W, generator=g)
    mix, ow, iw = (torch.randn(S, S, generator=g), torch.randn(S, generator=g),
                   torch.randn(S, generator=g))
    nw = torch.randn(W, generator=g) * 0.2
    new = torch.einsum("st,nsw->ntw", mix.double(), xs.double()) + \
        0.7 * ow.double()[None, :, None] * delta.double()[:, None, :]
    u = torch.einsum("s,nsw->nw", iw.double(), new)
    want = oracle.norm_plus_one(u, nw, 1e-5)
    x = xs.clone().to(device)
    got = sops.stream_step(x, delta.to(device), mix.to(device), ow.to(device),
                           0.7, iw.to(device), nw.to(device), 1e-5,
                           torch.float32)
    assert torch.allclose(x.cpu().double(), new, atol=1e-5)
    assert torch.allclose(got.cpu().double(), want, atol=1e-5)
    # read without a write, without a norm: the weighted sum itself
    got = sops.stream_step(x, None, None, None, 0.7, iw.to(device), None, 1e-5,
                           torch.float32)
    assert torch.allclose(got.cpu().double(), u, atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n,top", [(5, 3), (8, 2), (3, 1), (70, 4), (4, 4)])
def test_router_keeps_largest_logits(device, n, top):
    from dynamo_amd.ops import seq as sops
    g = torch.Generator().manual_seed(n)
    logits = torch.randn(9, n + 1, generator=g)      # one more column: unused
    bias = torch.randn(n, generator=g)
    idx, wgt = sops.moe_route_topk(logits.to(device), n, bias.to(device), top)
    z = logits[:, :n].double() + bias.double()
    for t in range(9):
        best = torch.topk(z[t], top).indices
        assert idx[t].cpu().tolist() == best.tolist()
        assert torch.allclose(wgt[t].cpu().double(),
                              torch.softmax(z[t, best], 0), atol=1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,P,N,G", [(6, 10, 12, 3), (2, 36, 20, 1),
                                     (4, 64, 128, 4), (3, 7, 5, 3)])
def test_state_space_scan_carries_state(device, H, P, N, G):
    """Two sequences in portions (one of them in a used slot) against the
    whole recurrence in float64."""
    from dynamo_amd.ops import seq as sops
    g = torch.Generator().manual_seed(H * P)
    lens = (11, 6)
    C = H * P + 2 * G * N
    par = dict(dt_bias=torch.randn(H, generator=g) - 1,
               A_log=torch.randn(H, generator=g) - 0.5,
               D=torch.randn(H, generator=g))
    data = [(torch.randn(n, C, generator=g), torch.randn(n, H + 2, generator=g))
            for n in lens]

    def whole(xbc, dt_raw):
        T = xbc.shape[0]
        x = xbc[:, :H * P].double().view(T, H, P)
        Bm = xbc[:, H * P:H * P + G * N].double().view(T, G, N)
        Cm = xbc[:, H * P + G * N:].double().view(T, G, N)
        dt = oracle.softplus(dt_raw[:, :H].double() + par["dt_bias"].double())
        y = torch.zeros(T, H, P, dtype=torch.float64)
        for h in range(H):
            S = torch.zeros(N, P, dtype=torch.float64)
            for t in range(T):
                S = torch.exp(-torch.exp(par["A_log"][h].double()) * dt[t, h]) * S \
                    + dt[t, h] * torch.outer(Bm[t, h // (H // G)], x[t, h])
                y[t, h] = S.t() @ Cm[t, h // (H // G)] + par["D"][h].double() * x[t, h]
        return y.view(T, H * P)
    state = torch.randn(3, H, N, P, generator=g).to(device)   # dirty slots
    p = {k: v.to(device) for k, v in par.items()}
    cuts = [((0, 4), (0, 1)), ((4, 5), (1, 6)), ((5, 11), None)]
    got = [[], []]
    for ca, cb in cuts:
        parts, spans = [], []
        for k, c in ((0, ca), (1, cb)):
            if c is not None:
                parts.append((k, c))
                spans.append((c[1] - c[0], 2 - k, c[0]))
        xbc = torch.cat([data[k][0][c[0]:c[1]] for k, c in parts]).to(device)
        dtr = torch.cat([data[k][1][c[0]:c[1]] for k, c in parts]).to(device)
        out = sops.ssd_scan(xbc, dtr, p["dt_bias"], p["A_log"], p["D"], state,
                            _span(spans, device), H, P, N, G).cpu()
        r = 0
        for k, c in parts:
            got[k].append(out[r:r + c[1] - c[0]])
            r += c[1] - c[0]
    for k in (0, 1):
        want = whole(*data[k])
        assert torch.allclose(torch.cat(got[k]).double(), want,
                              atol=2e-4 * float(want.abs().max()))


# -- portions, decoding, batches -----------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 2, 17, 5, 1], [31, 33, 2, 1],
                                   [16, 16, 16, 1]])
def test_portions_match_whole(full_ckpt, device, sizes):
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 70, 2)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [sizes])


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode(full_ckpt, device):
    """130 single-token steps: the window passes over decoded tokens, the
    query temperature steps up, distances pass the last bucket, pages fill
    and the state-space memory and its convolution tail are carried."""
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 135, 3)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[5, 1]])


def _run_plan(eng, toks, plan):
    lens = {k: len(v) for k, v in toks.items()}
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            entries.append((rid, toks[rid][at[rid]:at[rid] + n], list(range(n))))
            at[rid] += n
            if at[rid] == lens[rid]:
                end.append(rid)
        lg = eng.replay_step(entries, end).cpu()
        row = 0
        for rid, n in step:
            got[rid].append(lg[row:row + n])
            row += n
    assert at == lens
    return {k: torch.cat(v) for k, v in got.items()}


PLAN = [  # (request, tokens this step)
    [("a", 2), ("b", 5), ("d", 1)],
    [("a", 30), ("b", 1)],
    [("a", 1), ("b", 1), ("c", 17)],
    [("b", 2), ("c", 3), ("a", 1)],
    [("a", 36), ("c", 1)],
    [("c", 16), ("e", 2)],
    [("e", 31), ("f", 23)],
    [("e", 1)], [("e", 16)],
]
LENS = {"a": 70, "b": 9, "c": 37, "d": 1, "e": 50, "f": 23}


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_with_reuse(full_ckpt, device):
    """Unequal requests share steps (portions beside single tokens); the
    pool is so small that finished requests' pages and slots are taken
    again at once, at other places than before."""
    path, cfg, W = full_ckpt
    toks = {k: U.tokens_for(cfg, n, 10 + i) for i, (k, n) in enumerate(LENS.items())}
    want = {k: oracle.forward(cfg, W, t) for k, t in toks.items()}
    eng = U.make_engine(path, device, pages=11, slots=3, page_size=16)
    got = _run_plan(eng, toks, PLAN)
    for rid in LENS:
        assert U.rel_err(got[rid], want[rid]) < U.TOL["float32"], rid
    assert eng.alloc.num_free == 11 and eng.state_slots.num_free == 3


@pytest.mark.gpu
def test_mixed_batches_bf16(calm_ckpt):
    """The kernels the engine serves with (bf16 activations, matrix-core
    attention for prompt portions) on the same plan."""
    path, cfg, W = calm_ckpt
    toks = {k: U.tokens_for(cfg, n, 10 + i) for i, (k, n) in enumerate(LENS.items())}
    want = {k: oracle.forward(cfg, W, t) for k, t in toks.items()}
    eng = U.make_engine(path, "cuda:0", dtype="bfloat16", pages=11, slots=3,
                        page_size=16)
    got = _run_plan(eng, toks, PLAN)
    for rid in ("a", "c", "e", "f"):
        assert U.close_bf16(got[rid], want[rid]), rid
    # and each request alone, whole: the batch and the cut change nothing
    # beyond the rounding of differently shaped matrix products
    for rid in ("a", "c", "e"):
        alone = U.replay(eng, rid + "-alone", toks[rid], [len(toks[rid])])
        assert float(U.rel_err_rows(got[rid], alone).max()) < 0.03, rid


# -- edges made visible ----------------------------------------------------------
def _sharpen(names, factor):
    def edit(W):
        for k in W:
            if any(k.endswith(n) for n in names):
                W[k] = (W[k].float() * factor).to(W[k].dtype)
    return edit


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("size", [1, 2, 16, 17, 33, 200])
def test_window_sizes(tmp_path, device, size):
    """Sharp latent attention (keys and the rotated part scaled up) under
    windows of one token, one page, one more than a page and longer than
    the prompt; a key just outside the window must weigh nothing, the one
    just inside in full, in prompts and in decoding."""
    layer = copy.deepcopy(U.with_mlp(U.LATENT, None))
    layer["mixer"]["mask"]["size"] = size
    layer["mixer"]["scale"] = 0.9
    path, cfg, W = _case(tmp_path, [layer], seed=size,
                         edit=_sharpen(["mix.uk", "mix.uq"], 2.0))
    toks = U.tokens_for(cfg, 60, 4)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[60], [35, 1], [7, 2, 1]])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sink", [-30.0, 0.0, 6.0])
def test_sink_weighs_in_the_denominator(tmp_path, device, sink):
    """A sink far below the scores changes nothing, a large one takes most
    of the weight: left out, or counted with a value, it shows."""
    def edit(W):
        W["l0.mix.sink"] = torch.full_like(W["l0.mix.sink"], sink)
    path, cfg, W = _case(tmp_path, [U.with_mlp(U.LATENT, None)], seed=5,
                         edit=edit)
    toks = U.tokens_for(cfg, 40, 5)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[40], [20, 1]])


@pytest.mark.parametrize("device", DEVICES)
def test_far_keys_and_last_bucket(tmp_path, device):
    """The last distance bucket carries a large bonus for some heads and a
    large penalty for others, so rows far into a 150-token prompt put their
    weight on keys 37 and more tokens back: a bucket that is one off, or a
    table that ends early, shows. Pages of 16 tokens; decoded rows too."""
    def edit(W):
        rel = W["l0.mix.rel"].float()
        rel[-1] = torch.tensor([9.0, -9.0, 7.0, 0.0, -7.0, 5.0])
        rel[-2] = torch.tensor([-6.0, 6.0, 0.0, 5.0, 3.0, -5.0])
        W["l0.mix.rel"] = rel.to(torch.bfloat16)
    path, cfg, W = _case(tmp_path, [U.with_mlp(U.ATTN, None)], seed=6,
                         edit=edit)
    toks = U.tokens_for(cfg, 150, 6)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[150], [120, 1], [33, 31, 2]])


@pytest.mark.parametrize("device", DEVICES)
def test_soft_cap_binds(tmp_path, device):
    """Large query and key norm weights push the raw scores far past the
    cap; without the cap the softmax would be one-hot."""
    path, cfg, W = _case(tmp_path, [U.with_mlp(U.ATTN, None)], seed=7,
                         edit=_sharpen(["q.norm", "k.norm"], 3.0))
    toks = U.tokens_for(cfg, 50, 7)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[50], [30, 1]])


@pytest.mark.parametrize("device", DEVICES)
def test_slow_decay_keeps_old_tokens(tmp_path, device):
    """A state-space layer that forgets almost nothing (tiny A) and one
    that forgets at once: the state must come from the slot, from the first
    token on, across portions."""
    def edit(W):
        W["l0.mix.A_log"] = torch.tensor([-9.0, -9.0, -6.0, 3.0, 2.0, -9.0]
                                         ).to(torch.bfloat16)
    path, cfg, W = _case(tmp_path, [U.with_mlp(U.SSM, None)], seed=8, edit=edit)
    toks = U.tokens_for(cfg, 90, 8)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[90], [50, 1], [3, 2, 40, 1]])


# -- other sizes ---------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("streams", [0, 1, 2, 4])
def test_stream_counts(tmp_path, device, streams):
    """No hyper-connections at all (plain residual), one stream with
    weights, and more."""
    path, cfg, W = _case(tmp_path, [U.ATTN, U.SSM_BARE, U.LATENT], seed=9,
                         streams=streams, mult=1.0 if streams == 0 else 0.4)
    toks = U.tokens_for(cfg, 40, 9)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[40], [11, 2, 1]])


@pytest.mark.parametrize("device", DEVICES)
def test_odd_sizes(tmp_path, device):
    """Sizes that are no multiples of 8 or 16, one kv head, heads = groups,
    two taps, a single bucket pair, no pair-hash table."""
    layers = [
        {"type": "attention",
         "mixer": {"heads": 5, "kv_heads": 1, "dim": 6, "vdim": 10,
                   "scale": 0.4, "softcap": 50.0, "bias_max": 3},
         "mlp": {"kind": "dense", "ff": 30}},
        {"type": "mamba2",
         "mixer": {"heads": 3, "vdim": 7, "state": 5, "groups": 3,
                   "norm_groups": 3, "conv": 2},
         "mlp": {"kind": "moe", "expert": {"ff": 10},
                 "router": {"experts": 2, "top": 2}, "shared": {"ff": 6}}},
        {"type": "latent_attention",
         "mixer": {"heads": 1, "dim": 5, "rot_dim": 6, "vdim": 9,
                   "kv_rank": 11, "q_rank": 7, "scale": 0.5,
                   "mask": {"size": 3}, "rot": {"base": 100.0, "dims": 6}},
         "mlp": None}]
    path, cfg, W = _case(tmp_path, layers, seed=10, rel_rows=4, width=38,
                         vocab=53, streams=2, bigram=None)
    toks = U.tokens_for(cfg, 37, 10)
    eng = U.make_engine(path, device)
    want = _check(eng, cfg, W, toks, [[37], [9, 2, 1]])
    if device != "cpu":
        # the same sizes in bf16: none fits the matrix-core or the 16-byte
        # paths, so the scalar forms of the row kernels run
        eng = U.make_engine(path, device, dtype="bfloat16")
        for k, sizes in enumerate([[37], [9, 2, 1]]):
            got = U.replay(eng, f"b{k}", toks, sizes)
            assert U.close_bf16(got, want, tol=0.15), sizes


@pytest.mark.parametrize("device", DEVICES)
def test_large_heads(tmp_path, device):
    """Head sizes of served models (128-wide heads, a 256 + 32 latent row,
    eight latent heads on one cached row, a 64 x 128 state)."""
    layers = [
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 128, "vdim": 128,
                   "scale": 0.09, "softcap": 30.0, "bias_max": 64,
                   "q_temp": {"coef": 0.3, "every": 32}},
         "mlp": None},
        {"type": "latent_attention",
         "mixer": {"heads": 8, "dim": 32, "rot_dim": 32, "vdim": 32,
                   "kv_rank": 256, "q_rank": 96, "scale": 0.12,
                   "mask": {"size": 70},
                   "rot": {"base": 10000.0, "dims": 32}},
         "mlp": None},
        {"type": "mamba2",
         "mixer": {"heads": 4, "vdim": 64, "state": 128, "groups": 2,
                   "norm_groups": 4, "conv": 4},
         "mlp": None}]
    path, cfg, W = _case(tmp_path, layers, seed=11, rel_rows=32, width=128,
                         vocab=97, streams=2)
    toks = U.tokens_for(cfg, 100, 11)
    eng = U.make_engine(path, device, pages=10, page_size=64)
    _check(eng, cfg, W, toks, [[100], [70, 1]])


@pytest.mark.gpu
def test_large_heads_bf16_on_the_matrix_cores(tmp_path):
    """The same sizes in bf16: prompt tiles and the decoded rows of the
    eight latent heads run on the matrix cores with soft cap, distance
    table, window and sink."""
    test = [
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 128, "vdim": 128,
                   "scale": 0.09, "softcap": 30.0, "bias_max": 64,
                   "q_temp": {"coef": 0.3, "every": 32}},
         "mlp": None},
        {"type": "latent_attention",
         "mixer": {"heads": 8, "dim": 32, "rot_dim": 32, "vdim": 32,
                   "kv_rank": 256, "q_rank": 96, "scale": 0.12,
                   "mask": {"size": 70},
                   "rot": {"base": 10000.0, "dims": 32}},
         "mlp": None}]
    path, cfg, W = _case(tmp_path, test, seed=12, rel_rows=32, width=128,
                         vocab=97, streams=2)
    toks = U.tokens_for(cfg, 150, 12)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, "cuda:0", dtype="bfloat16", pages=10,
                        page_size=64)
    for k, sizes in enumerate([[150], [100, 1], [64, 3, 40, 1]]):
        got = U.replay(eng, f"r{k}", toks, sizes)
        assert U.close_bf16(got, want), sizes


OTHER = [   # another order: state-space first, shared layers of both kinds
    {"type": "mamba2",
     "mixer": {"heads": 5, "vdim": 32, "state": 24, "groups": 1,
               "norm_groups": 5, "conv": 2},
     "mlp": {"kind": "dense", "ff": 200}},
    {"type": "latent_attention",
     "mixer": {"heads": 8, "dim": 48, "rot_dim": 16, "vdim": 40,
               "kv_rank": 96, "q_rank": 64, "scale": 0.13,
               "mask": {"size": 65}, "rot": {"base": 50000.0, "dims": 16}},
     "mlp": {"kind": "moe", "expert": {"ff": 48},
             "router": {"experts": 6, "top": 3}, "shared": {"ff": 24}}},
    {"type": "attention",
     "mixer": {"heads": 5, "kv_heads": 5, "dim": 32, "vdim": 48,
               "scale": 0.18, "softcap": 12.0, "bias_max": 100,
               "q_temp": {"coef": 1.1, "every": 64}},
     "mlp": None},
    {"type": "latent_attention",
     "mixer": {"heads": 8, "dim": 48, "rot_dim": 16, "vdim": 40,
               "kv_rank": 96, "q_rank": 64, "scale": 0.13, "kv_from": 1,
               "mask": {"size": 130}, "rot": {"base": 50000.0, "dims": 16}},
     "mlp": {"kind": "dense", "ff": 120}},
    {"type": "attention",
     "mixer": {"heads": 5, "kv_heads": 5, "dim": 32, "vdim": 48,
               "scale": 0.18, "bias_max": 100, "kv_from": 2},
     "mlp": {"kind": "moe", "expert": {"ff": 48},
             "router": {"experts": 6, "top": 3}, "shared": {"ff": 24}}}]


@pytest.mark.parametrize("device", DEVICES)
def test_other_layout_on_64_token_pages(tmp_path, device):
    """Another layer order and other sizes on the page size the replay
    command uses: windows of one page + 1 and two pages + 2 (the shared
    latent layer has a window of its own on the other layer's rows), a
    shared attention layer without cap and temperature on capped keys, 24
    bias buckets, three streams; a 200-token prompt whole, cut at and
    around page borders, and decoded; in bf16 on the GPU as well."""
    def edit(W):
        for k in W:
            if k.endswith(".router"):
                W[k] = (W[k].float() * 6).to(W[k].dtype)
    path, cfg, W = _case(tmp_path, OTHER, seed=21, rel_rows=24, width=160,
                         vocab=211, streams=3, mult=0.7,
                         bigram=(257, 1009, 13), edit=edit)
    toks = U.tokens_for(cfg, 200, 21)
    eng = U.make_engine(path, device, pages=8, page_size=64, slots=2)
    plans = [[200], [63, 2, 63, 1], [64, 64, 3, 1]]
    want = _check(eng, cfg, W, toks, plans)
    if device != "cpu":
        eng = U.make_engine(path, device, dtype="bfloat16", pages=8,
                            page_size=64, slots=2)
        for k, sizes in enumerate(plans):
            got = U.replay(eng, f"b{k}", toks, sizes)
            assert U.close_bf16(got, want), sizes


def test_bad_configs_are_refused(tmp_path):
    from dynamo_amd.models.registry import build_model, resolve_model_config
    bad = copy.deepcopy(U.ATTN)
    bad["mixer"]["kv_heads"] = 4          # 6 query heads over 4 kv heads
    path, _cfg, _W = _case(tmp_path / "a", [U.ATTN])
    cfg = resolve_model_config(path)
    import dataclasses
    with pytest.raises(ValueError):
        build_model(dataclasses.replace(cfg, layer_specs=[bad]), "cpu",
                    torch.float32)
    # kv_from must name an earlier layer of the same kind and sizes
    for spec in ([U.ATTN, U.shared_from(U.ATTN_PLAIN, 0)],
                 [U.shared_from(U.ATTN, 1), U.ATTN],
                 [U.ATTN, U.shared_from(U.LATENT, 0)]):
        with pytest.raises(ValueError):
            build_model(dataclasses.replace(cfg, layer_specs=spec), "cpu",
                        torch.float32)
    with pytest.raises(ValueError):
        build_model(dataclasses.replace(
            cfg, layer_specs=[{"type": "rwkv", "mixer": {}, "mlp": None}]),
            "cpu", torch.float32)


def test_unused_checkpoint_tensor_is_an_error(tmp_path):
    cfg = U.make_config([U.SSM_BARE])
    W = U.random_weights(cfg, 0)
    W["l0.mix.extra"] = torch.zeros(3, dtype=torch.bfloat16)
    path = U.write_checkpoint(tmp_path, cfg, W)
    with pytest.raises(ValueError, match="not consumed"):
        U.make_engine(path, "cpu")


# -- through the scheduler ----------------------------------------------------------
def _greedy_oracle(cfg, W, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(oracle.forward(cfg, W, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(full_ckpt, device):
    """add_request / step with the engine's scheduler, chunked prefill and
    sampling: three requests of unequal length in two sequence slots."""
    from dynamo_amd.engine import SamplingParams
    path, cfg, W = full_ckpt
    prompts = {f"g{i}": U.tokens_for(cfg, n, 30 + i)
               for i, n in enumerate((21, 5, 40))}
    eng = U.make_engine(path, device, slots=2, pages=12, page_size=16,
                        max_batched_tokens=16)
    for rid, p in prompts.items():
        eng.add_request(rid, p, SamplingParams(max_tokens=6, temperature=0.0,
                                               ignore_eos=True))
    out = {rid: [] for rid in prompts}
    for _ in range(200):
        if not eng.has_work():
            break
        for so in eng.step():
            out[so.req_id].append(so.new_token)
    assert not eng.has_work()
    for rid, p in prompts.items():
        assert out[rid] == _greedy_oracle(cfg, W, p, 6), rid


@pytest.mark.gpu
def test_graph_decode_matches_eager(full_ckpt):
    """Decoding under hipGraph capture (padded batch buckets, persistent
    descriptors, the previous token kept on the device) against the oracle."""
    from dynamo_amd.engine import SamplingParams
    path, cfg, W = full_ckpt
    prompts = {f"g{i}": U.tokens_for(cfg, n, 40 + i)
               for i, n in enumerate((30, 7, 19))}
    want = {rid: _greedy_oracle(cfg, W, p, 8) for rid, p in prompts.items()}
    eng = U.make_engine(path, "cuda:0", slots=4, pages=16, page_size=16,
                        graphs=True)
    for rid, p in prompts.items():
        eng.add_request(rid, p, SamplingParams(max_tokens=8, temperature=0.0,
                                               ignore_eos=True))
    out = {rid: [] for rid in prompts}
    for _ in range(200):
        if not eng.has_work():
            break
        for so in eng.step():
            out[so.req_id].append(so.new_token)
    assert out == want


def test_preset_and_state_declaration():
    """The random-weight preset builds, declares its caches and state, and
    generates through the scheduler."""
    from dynamo_amd.engine import EngineConfig, LLMEngine, SamplingParams
    from dynamo_amd.engine.config import PRESETS
    from dynamo_amd.models.registry import native_extensions
    cfg = PRESETS["tiny-muzulorn"]
    assert native_extensions(cfg, "cuda:0") == ["_core", "_hip_seq"]
    eng = LLMEngine(EngineConfig(model=cfg, device="cpu", dtype="float32",
                                 page_size=16, max_num_seqs=2,
                                 max_model_len=128, kv_pool_pages=12,
                                 enable_hip_graphs=False), seed=0)
    model = eng.runner.model
    assert model.kv_layer_shapes() == [(2, 20, 12), (1, 32, 0), None, None]
    assert model.state_layer_shapes() == [[], [], [(4, 12, 10), (2, 88)], [],
                                          [(1,)]]
    eng.add_request("a", list(range(3, 40)),
                    SamplingParams(max_tokens=4, temperature=0.0,
                                   ignore_eos=True))
    out = []
    for _ in range(50):
        if not eng.has_work():
            break
        out += [so.new_token for so in eng.step()]
    assert len(out) == 4 and eng.state_slots.num_free == 2


def test_trace_run_command(full_ckpt, tmp_path):
    """The command-line replay: two requests sharing steps, portions beside
    single tokens, logits written only where they are wanted."""
    import subprocess
    import numpy as np
    path, cfg, W = full_ckpt
    a, b = U.tokens_for(cfg, 20, 40), U.tokens_for(cfg, 9, 41)
    E = lambda i, t, w: {"id": i, "tokens": t, "want": w}  # noqa: E731
    steps = [{"step": 0, "entries": [E("a", a[:13], [0, 12]), E("b", b[:2], [])],
              "end": []},
             {"step": 1, "entries": [E("a", a[13:14], []), E("b", b[2:3], [])],
              "end": []},
             {"step": 2, "entries": [E("b", b[3:], [5]), E("a", a[14:], [5])],
              "end": ["a", "b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", path,
                        "--dtype", "float32", "--out", str(tmp_path / "o"),
                        "--max-tokens", "128", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [x for x in r.stdout.splitlines() if x.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    wa, wb = oracle.forward(cfg, W, a), oracle.forward(cfg, W, b)
    first = np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, -1)
    last = np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(2, -1)
    assert not (tmp_path / "o" / "1.f32").exists()
    got = torch.from_numpy(np.concatenate([first, last]))
    want = torch.stack([wa[0], wa[12], wb[8], wa[19]])
    assert U.rel_err(got, want) < U.TOL["float32"]
