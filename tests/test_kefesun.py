"""Kefesun through the engine against the slow oracle (tests/kefesun_oracle):
each mechanism alone, whole prompts against portions and single-token
decoding, mixed batches, reuse of cache pages and state slots, keys far
back, at page borders, at the edges of the sliding window and of the kept
first tokens, the first tokens, long decoding, odd sizes, the router's
groups, and greedy generation through add_request/step. Runs on CPU; the
same cases run on the HIP kernels under the gpu marker."""
import copy
import json
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(__file__))
import kefesun_oracle as oracle  # noqa: E402
import kefesun_util as U  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
FULL = [U.ATTN, U.GRU, U.ATTN_FULL, U.with_mlp(U.GRU_BARE, U.MOE_IDENT),
        U.with_mlp(U.ATTN, U.MOE_PLAIN)]


@pytest.fixture(scope="module")
def full_ckpt(tmp_path_factory):
    cfg = U.make_config(FULL)
    W = U.random_weights(cfg, 1)
    return U.write_checkpoint(tmp_path_factory.mktemp("full"), cfg, W), cfg, W


@pytest.fixture(scope="module")
def calm_ckpt(tmp_path_factory):
    cfg = U.make_config(FULL)
    W = U.random_weights(cfg, 1)
    U.calm_routers(W)
    return U.write_checkpoint(tmp_path_factory.mktemp("calm"), cfg, W), cfg, W


def _case(tmp_path, layers, seed=0, edit=None, **kw):
    cfg = U.make_config(layers, **kw)
    W = U.random_weights(cfg, seed)
    if edit:
        edit(W)
    return U.write_checkpoint(tmp_path, cfg, W), cfg, W


def _check(eng, cfg, W, toks, plans, tol=U.TOL["float32"], want=None,
           bf16=False):
    want = oracle.forward(cfg, W, toks) if want is None else want
    for k, sizes in enumerate(plans):
        got = U.replay(eng, f"r{k}", toks, sizes)
        if bf16:
            assert U.close_bf16(got, want), sizes
        else:
            assert U.rel_err(got, want) < tol, sizes
    return want


# -- each mechanism alone ------------------------------------------------------
LAYERS_ALONE = {
    "attention": [U.with_mlp(U.ATTN, None)], "attention_full": [U.ATTN_FULL],
    "mingru": [U.GRU_BARE],
    "moe_groups": [U.with_mlp(U.GRU_BARE, U.MOE)],
    "moe_plain": [U.with_mlp(U.GRU_BARE, U.MOE_PLAIN)],
    "moe_identity": [U.with_mlp(U.GRU_BARE, U.MOE_IDENT)]}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(LAYERS_ALONE))
def test_single_mechanism(tmp_path, device, name):
    path, cfg, W = _case(tmp_path, LAYERS_ALONE[name], seed=3)
    toks = U.tokens_for(cfg, 45, 0)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[45], [1]])


def test_residual_stream_after_every_layer(full_ckpt):
    """The model's layer taps against the oracle's, layer by layer."""
    from dynamo_amd.engine.scheduler import ScheduledSeq, SchedulerOutput
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 30, 1)
    want = []
    oracle.forward(cfg, W, toks, want)
    eng = U.make_engine(path, "cpu")
    # one prefill step by hand so that the tap list can be passed
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


def _span(n, slot, pos0, dev="cpu", page_table=None, num_decode=0):
    from dynamo_amd.ops import seq as sops
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
    return sops.SeqBatch(torch.zeros(n, dtype=torch.int32, device=dev),
                         i32([0]), i32([n]), i32([slot]), i32([pos0]),
                         page_table=page_table, num_decode=num_decode,
                         host=[(0, n, slot, pos0)])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_ops_carry_state_across_portions(device, taps):
    """Op level: the input convolution and the gated scan continued over
    portions from a dirty slot equal one pass; a portion longer than one
    scan chunk is cut inside the kernel."""
    from dynamo_amd.ops import seq as sops
    torch.manual_seed(0)
    T, W, C = 150, 20, 12
    x = torch.randn(T, W, device=device)
    cw = torch.randn(W, taps, device=device)
    proj = torch.randn(T, 3 * C, device=device)

    def run(cuts):
        S = torch.full((3, C), 5.0, device=device)             # dirty slots
        cs = torch.full((3, taps - 1, W), -3.0, device=device)
        hs, ys, pos = [], [], 0
        for n in cuts:
            sb = _span(n, 1, pos, device)
            hs.append(sops.residual_conv(x[pos:pos + n].contiguous(), cw, cs,
                                         sb, torch.float32))
            ys.append(sops.mingru_scan(proj[pos:pos + n].contiguous(), C, S,
                                       sb, torch.float32))
            pos += n
        return torch.cat(hs).cpu(), torch.cat(ys).cpu()
    h0, y0 = run([T])
    want_h = x.double().cpu() + oracle.time_conv(x.double().cpu(), cw.cpu())
    assert torch.allclose(h0.double(), want_h, atol=1e-5)
    for cuts in ([2, 1, 70, 77], [1] * 9 + [141]):
        h1, y1 = run(cuts)
        assert torch.allclose(h0, h1, atol=1e-5)
        assert torch.allclose(y0, y1, atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps,W", [(1, 20), (2, 33), (4, 20), (5, 20),
                                    (3, 700), (4, 4100)])
def test_join_and_convolution_of_decoded_rows(device, taps, W):
    """Rows that are all decoded tokens take the fused step (the waiting
    output is normed and added, the convolution reads and advances the
    slot's rows): three sequences at different positions, one of them at
    its second token, against the whole-sequence computation."""
    from dynamo_amd.ops import seq as sops
    g = torch.Generator().manual_seed(taps * W)
    lens = [9, 2, 5]
    xs = [torch.randn(n, W, generator=g) for n in lens]      # streams
    ds = [torch.randn(n, W, generator=g) for n in lens]      # waiting outputs
    cw = torch.randn(W, taps, generator=g)
    pw = torch.rand(W, generator=g) + 0.5
    want = []
    for x, d in zip(xs, ds):
        y = x.double() + oracle.layer_norm(d.double(), pw, 1e-5)
        want.append(y + oracle.time_conv(y, cw))
    cs = torch.full((4, taps - 1, W), 7.0, device=device)    # dirty slots
    slots = [2, 0, 3]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    # all but the last token of each sequence as a prompt portion
    for k, n in enumerate(lens):
        sb = _span(n - 1, slots[k], 0, device)
        sops.join_conv(xs[k][:n - 1].clone().to(device),
                       ds[k][:n - 1].to(device), pw.to(device), 1e-5,
                       cw.to(device), cs, sb, torch.float32)
    # the last tokens together, as decoded rows
    res = torch.stack([x[-1] for x in xs]).to(device)
    delta = torch.stack([d[-1] for d in ds]).to(device)
    sb = sops.SeqBatch(i32([0, 1, 2]), i32([0, 1, 2]), i32([1, 1, 1]),
                       i32(slots), i32([n - 1 for n in lens]), num_decode=3,
                       host=[(k, 1, slots[k], lens[k] - 1) for k in range(3)])
    got = sops.join_conv(res, delta, pw.to(device), 1e-5, cw.to(device), cs,
                         sb, torch.float32).cpu()
    for k in range(3):
        assert torch.allclose(got[k].double(), want[k][-1], atol=1e-4)
        y = xs[k].double() + oracle.layer_norm(ds[k].double(), pw, 1e-5)
        if taps > 1:      # the slot now ends with this token's stream row
            assert torch.allclose(cs[slots[k], -1].cpu().double(), y[-1],
                                  atol=1e-5)


# -- the router -----------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n,groups,keep,top", [(6, 3, 2, 3), (8, 1, 1, 2),
                                               (12, 4, 1, 3), (70, 5, 2, 9),
                                               (3, 3, 3, 1)])
def test_router_against_oracle(device, n, groups, keep, top):
    """Corrections are as large as the scores and mostly negative, so that
    choice scores below zero occur in kept groups: an excluded group must
    count as minus infinity, not as zero; the weights must be the
    uncorrected scores."""
    from dynamo_amd.ops import seq as sops
    g = torch.Generator().manual_seed(n)
    T, Wd = 40, 16
    h = torch.randn(T, Wd, generator=g, dtype=torch.float64)
    Wt = {"p.router": torch.randn(n, Wd, generator=g) * 0.8,
          "p.correction": torch.rand(n, generator=g) * 0.5 - 0.45}
    r = {"experts": n, "top": top, "scale": 1.7,
         "groups": {"count": groups, "keep": keep}}
    want_idx, want_w = oracle.route(h, Wt, "p.", r)
    logits = (h @ Wt["p.router"].double().t()).float().to(device)
    idx, wgt = sops.moe_route(logits, Wt["p.correction"].to(device), groups,
                              keep, top, 1.7)
    assert torch.equal(idx.cpu().long().sort(-1).values,
                       want_idx.sort(-1).values)
    order = idx.cpu().long().argsort(-1)
    worder = want_idx.argsort(-1)
    assert torch.allclose(wgt.cpu().double().gather(1, order),
                          want_w.gather(1, worder), atol=1e-6)
    # the same from the router's input rows (few rows: logits formed in
    # the routing kernel), fp32 and bf16 rows
    for dt in (torch.float32, torch.bfloat16):
        hh = h.to(dt)
        want_idx2, want_w2 = oracle.route(hh.double(), Wt, "p.", r)
        idx2, wgt2 = sops.moe_route_rows(
            hh.to(device), Wt["p.router"].to(device),
            Wt["p.correction"].to(device), groups, keep, top, 1.7)
        same = (idx2.cpu().long().sort(-1).values
                == want_idx2.sort(-1).values).all(-1)
        assert float(same.float().mean()) > 0.9      # near-ties may flip
        o2, w2 = idx2.cpu().long().argsort(-1), want_idx2.argsort(-1)
        assert torch.allclose(wgt2.cpu().double().gather(1, o2)[same],
                              want_w2.gather(1, w2)[same], atol=1e-5)
    if groups > 1 and keep < groups:
        s = torch.softmax(h @ Wt["p.router"].double().t(), -1)
        choice = s + Wt["p.correction"].double()
        assert bool((choice.gather(1, want_idx) < 0).any())


@pytest.mark.parametrize("device", DEVICES)
def test_dispatch_gather_combine(device):
    """Rows of the gathered batch: every (token, expert) pair lands once, in
    token order inside its expert; identity choices take no row and add the
    input itself."""
    from dynamo_amd.ops import seq as sops
    g = torch.Generator().manual_seed(5)
    T, k, E, n, Wd = 300, 3, 4, 6, 24
    idx = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(T)]
                      ).to(torch.int32).to(device)
    h = torch.randn(T, Wd, generator=g).to(device)
    wgt = torch.rand(T, k, generator=g).to(device)
    shared = torch.randn(T, Wd, generator=g).to(device)
    rank, counts = sops.moe_dispatch(idx, n)
    flat = idx.cpu().reshape(-1).tolist()
    assert counts.cpu().tolist() == [flat.count(e) for e in range(n)]
    seen = [0] * n
    for i, e in enumerate(flat):
        assert int(rank.reshape(-1)[i]) == seen[e]
        seen[e] += 1
    base = torch.zeros(E + 1, dtype=torch.int32)
    base[1:] = torch.cumsum(counts.cpu()[:E], 0)
    rows = int(base[E])
    xg = sops.moe_gather(h, idx, rank, base.to(device), E, rows)
    y = xg * 2.0      # stand-in for the experts
    out = sops.moe_combine(y, h, idx, wgt, rank, base.to(device), E, shared,
                           torch.float32).cpu()
    mult = torch.where(idx.cpu() < E, 2.0, 1.0)
    want = h.cpu() * (wgt.cpu() * mult).sum(1, keepdim=True) + shared.cpu()
    assert torch.allclose(out, want, atol=1e-5)


# -- portions, decoding, first tokens -----------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 2, 17, 5, 1], [31, 33, 2, 1],
                                   [64, 1], [70, 2]], ids=str)
def test_portions_match_whole(full_ckpt, device, sizes):
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 83, 2)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device)
    got = U.replay(eng, "r", toks, sizes)
    assert U.rel_err(got, want) < U.TOL["float32"]
    # the first tokens of a sequence, alone
    assert U.rel_err(got[:3], want[:3]) < U.TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode(full_ckpt, device):
    """145 single-token steps: the window passes over decoded tokens and
    leaves the kept first ones behind, pages fill, and the recurrent state
    and both convolution tails are carried step by step."""
    path, cfg, W = full_ckpt
    toks = U.tokens_for(cfg, 150, 3)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[5, 1]])


# -- batches, reuse of pages and slots ----------------------------------------
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
    path, cfg, W = calm_ckpt
    toks = {k: U.tokens_for(cfg, n, 10 + i) for i, (k, n) in enumerate(LENS.items())}
    want = {k: oracle.forward(cfg, W, t) for k, t in toks.items()}
    eng = U.make_engine(path, "cuda:0", dtype="bfloat16", pages=11, slots=3,
                        page_size=16)
    got = _run_plan(eng, toks, PLAN)
    alone = {k: U.replay(eng, k + "'", t, [4096]) for k, t in toks.items()}
    for rid in LENS:
        assert U.close_bf16(got[rid], want[rid]), rid
    # what else is in the batch, and which pages and slots a request got,
    # changes nothing beyond rounding
    both = torch.cat([U.rel_err_rows(got[k], alone[k]) for k in LENS])
    assert float(both.median()) < 0.02 and float((both < 0.05).float().mean()) > 0.9


# -- window edges, kept first keys, far keys, page borders ---------------------
def _edge_case(T, i, j, dk=8, dv=6, strong=60.0, seed=0):
    """One kv head, T tokens: key j points along query i with a large norm.
    With a strongly negative head bias every other key weighs ~0 and key j,
    if visible, ~1: the output of row i is v[j] or ~0."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(T, 1, dk, generator=g)
    k = torch.randn(T, 1, dk, generator=g) * 0.3
    v = torch.randn(T, 1, dv, generator=g)
    k[j, 0] = strong * q[i, 0] / q[i, 0].norm() / q[i, 0].norm()
    return q, k, v


def _sigmoid_attention_oracle(q, k, v, scale, bias, window, keep):
    T = q.shape[0]
    s = (q.double() @ k.double().t()) * scale + bias
    ok = oracle.visible(T, window, keep)
    return torch.where(ok, oracle.sigmoid(s), torch.zeros((), dtype=torch.float64)
                       ) @ v.double()


def _op_attention(device, q, k, v, ps, rows, decode, window, keep, bias,
                  scale=1.0, dtype=torch.float32, tiled=False):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] over scattered pages; the
    rows `rows` (consecutive positions) as one prompt portion or one decoded
    token. -> [len(rows), H, dv]."""
    from dynamo_amd.ops import seq as sops
    T, H, dk = q.shape
    G, dv = k.shape[1], v.shape[2]
    npg = -(-T // ps)
    perm = torch.randperm(npg + 3, generator=torch.Generator().manual_seed(T)
                          )[:npg]
    kc = torch.zeros(npg + 3, G, ps, dk)
    vc = torch.zeros(npg + 3, G, ps, dv)
    for t in range(T):
        kc[perm[t // ps], :, t % ps] = k[t]
        vc[perm[t // ps], :, t % ps] = v[t]
    n = len(rows)
    dev = torch.device(device)
    sb = _span(n, 0, rows[0], dev, perm.to(torch.int32).view(1, -1).to(dev),
               1 if decode else 0)
    if dev.type == "cuda":
        sb.host = None
    if tiled:
        sb.tiles = (torch.arange(0, n, 64, dtype=torch.int32, device=dev),
                    torch.tensor([min(64, n - a) for a in range(0, n, 64)],
                                 dtype=torch.int32, device=dev))
    pos = torch.tensor(rows, dtype=torch.int32, device=dev)
    qq = q[rows].reshape(n, -1).contiguous().to(dtype).to(dev)
    hb = torch.full((H,), float(bias)) if not torch.is_tensor(bias) else bias
    got = sops.paged_attention_rows(
        qq, 0, H, 1, kc.to(dtype).to(dev), vc.to(dtype).to(dev), dv, pos, sb,
        scale, window, keep, hb.float().to(dev), True)
    return got.float().cpu()[:, :, 0]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window,keep,ps", [(5, 2, 4), (16, 16, 16),
                                            (64, 1, 16), (70, 5, 64),
                                            (1, 3, 4), (40, 70, 16)])
@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoded"])
def test_window_and_kept_edges_at_op_level(device, window, keep, ps, decode):
    """A dominating key placed just outside and just inside the window of
    the last row, and just inside and just outside the kept first keys: an
    edge that is one token off moves the whole output. Rows run as one
    prompt portion, or the last row as a decoded token over a cache filled
    before."""
    i = 2 * window + keep + 37
    T = i + 1
    cases = [(i - window, False), (i - window + 1, True)]
    if keep - 1 < i - window:
        cases.append((keep - 1, True))
    if keep < i - window:
        cases.append((keep, False))
    for j, inside in cases:
        q, k, v = _edge_case(T, i, j, seed=window + j)
        rows = [i] if decode else list(range(T))
        got = _op_attention(device, q, k, v, ps, rows, decode, window, keep,
                            -25.0)
        want = _sigmoid_attention_oracle(q[:, 0], k[:, 0], v[:, 0], 1.0, -25.0,
                                         window, keep)
        assert torch.allclose(got[-1, 0].double(), want[i], atol=2e-4), j
        hit = torch.allclose(got[-1, 0], v[j, 0], atol=1e-3)
        assert hit == inside, (j, inside)
        if not inside:
            assert float(got[-1, 0].abs().max()) < 1e-3


@pytest.mark.parametrize("device", DEVICES)
def test_sharp_attention_far_keys_and_page_edges(tmp_path, device):
    """Unwindowed attention whose queries and keys are scaled up and whose
    head bias is pushed down, so that a few keys - often hundreds of tokens
    back - carry the output. A key read from a wrong page slot shows; so
    does a second request over the same, now used, pages."""
    def edit(W):
        W["l0.mix.q.norm"].mul_(4.0)
        W["l0.mix.k.norm"].mul_(4.0)
        W["l0.mix.pb"].fill_(-12.0)
    layer = copy.deepcopy(U.ATTN_FULL)
    layer["mixer"].update(heads=4, kv_heads=2)
    path, cfg, W = _case(tmp_path, [layer], seed=7, edit=edit)
    toks = U.tokens_for(cfg, 300, 4)
    eng = U.make_engine(path, device, pages=20, page_size=16)
    _check(eng, cfg, W, toks, [[15, 1, 1, 1, 32, 200, 1]])
    _check(eng, cfg, W, toks[::-1], [[17, 2]])
    # the construction is only a test if far keys do carry weight
    m = cfg["layers"][0]["mixer"]
    x = oracle.d(W["embed"])[torch.tensor(toks)] * cfg["embedding"]["scale"]
    h = x + oracle.time_conv(x, W["l0.canon1"])
    p = "l0.mix."
    q = oracle.rotate_half(oracle.rms_norm(
        (h @ oracle.d(W[p + "q"]).t() + oracle.d(W[p + "q.b"])).view(300, 4, -1),
        W[p + "q.norm"], 1e-5), m["rot"])
    k = oracle.rotate_half(oracle.rms_norm(
        (h @ oracle.d(W[p + "k"]).t() + oracle.d(W[p + "k.b"])).view(300, 2, -1),
        W[p + "k.norm"], 1e-5), m["rot"])
    wgt = oracle.sigmoid((q[299, 0] @ k[:, 0].t()) * m["scale"] - 12.0)
    assert float(wgt[:200].sum()) > 0.2 * float(wgt.sum())


@pytest.mark.parametrize("device", DEVICES)
def test_sharp_window_attention_through_engine(tmp_path, device):
    """Sharp attention under a small window with kept first keys over a
    long prompt and long decoding: the strongest visible key often lies at
    the window's far edge, at a page border, or among the kept ones."""
    def edit(W):
        W["l0.mix.q.norm"].mul_(3.0)
        W["l0.mix.k.norm"].mul_(3.0)
        W["l0.mix.pb"].fill_(-6.0)
    layer = copy.deepcopy(U.ATTN)
    layer["mixer"]["mask"] = {"size": 17, "keep_first": 5}   # crosses pages
    path, cfg, W = _case(tmp_path, [layer], seed=9, edit=edit)
    toks = U.tokens_for(cfg, 140, 5)
    eng = U.make_engine(path, device, pages=20, page_size=16)
    _check(eng, cfg, W, toks, [[140], [40, 1], [16, 17, 1, 15, 2, 1]])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("size,keep", [(1, 0), (2, 1), (16, 16), (200, 2),
                                       (5, 40), (64, 7)])
def test_window_sizes(tmp_path, device, size, keep):
    """A window of one token (each sees only itself), no kept keys, as many
    kept keys as the window, more kept keys than the window, a window that
    equals the page size, and one longer than the prompt."""
    layer = copy.deepcopy(U.ATTN)
    layer["mixer"]["mask"] = {"size": size, "keep_first": keep}
    path, cfg, W = _case(tmp_path, [layer], seed=11)
    toks = U.tokens_for(cfg, 90, 6)
    eng = U.make_engine(path, device, page_size=16)
    _check(eng, cfg, W, toks, [[90], [7, 9, 1], [70, 2, 1]])


@pytest.mark.parametrize("device", DEVICES)
def test_far_positions_rotate_exactly(tmp_path, device):
    """Positions in the thousands: angles must be formed in fp32 from the
    position, not accumulated; the kept first keys are then over a thousand
    tokens away. Only the last tokens are compared."""
    layer = copy.deepcopy(U.ATTN)
    layer["mixer"]["mask"] = {"size": 100, "keep_first": 4}
    path, cfg, W = _case(tmp_path, [layer, U.ATTN_FULL], seed=13, width=64)
    toks = U.tokens_for(cfg, 1500, 7)
    want = oracle.forward(cfg, W, toks)
    eng = U.make_engine(path, device, pages=30, page_size=64)
    got = U.replay(eng, "r", toks, [1490, 1])
    assert U.rel_err(got[-12:], want[-12:]) < U.TOL["float32"]


# -- recurrence -------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 6])
def test_convolution_widths(tmp_path, device, taps):
    path, cfg, W = _case(tmp_path, [U.GRU, U.ATTN], seed=15, taps=taps)
    toks = U.tokens_for(cfg, 24, 8)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[24], [1], [2, 3, 1, 1, 9, 2]])


@pytest.mark.parametrize("device", DEVICES)
def test_slow_gate_keeps_old_tokens(tmp_path, device):
    """A strongly negative gate bias makes z tiny: the state then remembers
    tokens hundreds back, and 1 - z must not be rounded to 1 where z
    matters. A state lost between steps shows."""
    def edit(W):
        W["l0.mix.z.b"].fill_(-7.0)
    path, cfg, W = _case(tmp_path, [U.GRU_BARE], seed=17, edit=edit)
    toks = U.tokens_for(cfg, 260, 9)
    eng = U.make_engine(path, device)
    _check(eng, cfg, W, toks, [[260], [200, 1], [3, 64, 1, 1, 100, 2]])


# -- sizes ----------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_odd_sizes(tmp_path, device):
    """Sizes that fit no vector width (the scalar paths of the kernels),
    three query heads per kv head, one head, no rotation, one expert per
    token, a vocabulary and widths that are odd."""
    at = copy.deepcopy(U.ATTN)
    at["mixer"].update(heads=3, kv_heads=1, dim=10, vdim=7,
                       rot={"base": 100.0, "dims": 6},
                       mask={"size": 9, "keep_first": 2})
    at["mlp"]["expert"]["ff"] = 13
    at["mlp"]["router"].update(experts=7, identity=2, top=1,
                               groups={"count": 3, "keep": 1})
    at["mlp"]["shared"]["ff"] = 5
    a1 = copy.deepcopy(U.ATTN_FULL)
    a1["mixer"].update(heads=1, kv_heads=1, dim=9, vdim=11)
    del a1["mixer"]["rot"]
    gr = copy.deepcopy(U.GRU)
    gr["mixer"]["width"] = 35
    path, cfg, W = _case(tmp_path, [gr, at, a1], seed=19, width=66, vocab=91,
                         eps=1e-3, taps=2, scale=1.0, edit=U.calm_routers)
    toks = U.tokens_for(cfg, 40, 10)
    eng = U.make_engine(path, device, page_size=8, pages=12)
    want = _check(eng, cfg, W, toks, [[40], [3, 1, 1, 19, 2]])
    if device != "cpu":
        e16 = U.make_engine(path, device, dtype="bfloat16", page_size=8,
                            pages=12)
        _check(e16, cfg, W, toks, [[40], [3, 1, 1, 19, 2]], want=want,
               bf16=True)


@pytest.mark.parametrize("device", DEVICES)
def test_large_heads(tmp_path, device):
    """Head sizes of real models: 128-wide heads with 64-wide values, eight
    and sixteen query heads per kv head (the vector and matrix-core paths
    of the kernels), many experts in many groups."""
    at = copy.deepcopy(U.ATTN)
    at["mixer"].update(heads=8, kv_heads=1, dim=128, vdim=64, scale=0.09,
                       rot={"base": 10000.0, "dims": 64},
                       mask={"size": 33, "keep_first": 4})
    at["mlp"]["router"].update(experts=30, identity=2, top=6,
                               groups={"count": 8, "keep": 3})
    a2 = copy.deepcopy(U.ATTN_FULL)
    a2["mixer"].update(heads=16, kv_heads=1, dim=64, vdim=128,
                       rot={"base": 10000.0, "dims": 32})
    path, cfg, W = _case(tmp_path, [at, a2], seed=21, width=128,
                         edit=U.calm_routers)
    toks = U.tokens_for(cfg, 90, 11)
    eng = U.make_engine(path, device, page_size=16, pages=12)
    want = _check(eng, cfg, W, toks, [[90], [70, 1]])
    if device != "cpu":
        e16 = U.make_engine(path, device, dtype="bfloat16", page_size=16,
                            pages=12)
        _check(e16, cfg, W, toks, [[90], [70, 1], [33, 2, 1]], want=want,
               bf16=True)


def test_bad_configs_are_refused(tmp_path):
    from dynamo_amd.models.registry import build_model, resolve_model_config
    groups = U.make_config([U.ATTN])
    groups["layers"][0]["mlp"]["router"]["groups"] = {"count": 4, "keep": 1}
    top = U.make_config([U.ATTN])
    top["layers"][0]["mlp"]["router"]["top"] = 5      # two groups hold four
    kind = U.make_config([U.ATTN])
    kind["layers"][0]["type"] = "conv"
    for k, cfg in enumerate((groups, top, kind)):
        d = tmp_path / str(k)
        os.makedirs(d)
        with open(d / "config.json", "w") as f:
            json.dump(cfg, f)
        with pytest.raises(ValueError):
            build_model(resolve_model_config(str(d)), "cpu", torch.float32)


def test_unused_checkpoint_tensor_is_an_error(tmp_path):
    cfg = U.make_config([U.GRU_BARE])
    W = U.random_weights(cfg, 0)
    W["l0.mix.extra"] = torch.zeros(3, dtype=torch.bfloat16)
    path = U.write_checkpoint(tmp_path, cfg, W)
    with pytest.raises(ValueError):
        U.make_engine(path, "cpu")


# -- bf16 prompt portions on the matrix cores ---------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk,dv,window,keep", [
    (4, 2, 64, 128, 100, 3),
    (6, 3, 24, 40, 19, 70),         # sizes padded inside the kernel
    (2, 1, 128, 56, 0, 0),          # every earlier key visible
    (2, 2, 16, 8, 1, 2),            # a window of one token
    (16, 1, 64, 64, 50, 1),
])
def test_mfma_sigmoid_attention_matches_oracle(H, G, dk, dv, window, keep):
    """bf16 prompt rows from position 0 and a portion continued from
    position 150 (its tiles start inside a page, beyond the window and
    beyond the kept keys) through the matrix-core kernel."""
    g = torch.Generator().manual_seed(H * dk)
    T = 230
    q = torch.randn(T, H, dk, generator=g).bfloat16().float()
    k = torch.randn(T, G, dk, generator=g).bfloat16().float()
    v = torch.randn(T, G, dv, generator=g).bfloat16().float()
    bias = -torch.rand(H, generator=g) * 3
    for rows in (list(range(T)), list(range(150, T))):
        got = _op_attention("cuda:0", q, k, v, 16, rows, False, window, keep,
                            bias, scale=dk ** -0.5, dtype=torch.bfloat16,
                            tiled=True)
        for hh in range(H):
            want = _sigmoid_attention_oracle(
                q[:, hh], k[:, hh // (H // G)], v[:, hh // (H // G)],
                dk ** -0.5, float(bias[hh]), window or None, keep)[rows]
            err = (got[:, hh].double() - want).abs().max() / want.abs().max()
            assert float(err) < 1e-2, (hh, rows[0])
    # the last row as a decoded token: head groups of eight and more run on
    # the matrix cores with their keys split over workgroups, the others on
    # the row kernel
    got = _op_attention("cuda:0", q, k, v, 16, [T - 1], True, window, keep,
                        bias, scale=dk ** -0.5, dtype=torch.bfloat16)
    for hh in range(H):
        want = _sigmoid_attention_oracle(
            q[:, hh], k[:, hh // (H // G)], v[:, hh // (H // G)], dk ** -0.5,
            float(bias[hh]), window or None, keep)[T - 1]
        err = (got[0, hh].double() - want).abs().max() / want.abs().max()
        assert float(err) < 1e-2, hh


# -- the engine's own entry point ---------------------------------------------
def _greedy_oracle(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(oracle.forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


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
    descriptors) against the oracle."""
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
    generates through the scheduler; identity and grouped routers, a layer
    without feed-forward and one without window are all in it."""
    from dynamo_amd.engine import EngineConfig, LLMEngine, SamplingParams
    from dynamo_amd.engine.config import PRESETS
    from dynamo_amd.models.registry import native_extensions
    cfg = PRESETS["tiny-kefesun"]
    assert native_extensions(cfg, "cuda:0") == ["_core", "_hip_seq"]
    eng = LLMEngine(EngineConfig(model=cfg, device="cpu", dtype="float32",
                                 page_size=16, max_num_seqs=2,
                                 max_model_len=128, kv_pool_pages=12,
                                 enable_hip_graphs=False), seed=0)
    model = eng.runner.model
    K, W = cfg.conv_taps - 1, cfg.hidden_size
    assert model.kv_layer_shapes() == [(2, 24, 16), None, (1, 16, 24)]
    assert model.state_layer_shapes() == [[(K, W), (K, W)], [(K, W), (72,)],
                                          [(K, W), (K, W)]]
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
