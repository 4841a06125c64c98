"""The Netovik design in the engine against the plain implementation: each mechanism alone at
the level of its op, then whole models through the step function (whole prompts, decoding
token by token, portions down to two tokens, mixed batches on a pool whose pages and slots are
used again), and greedy generation through the engine's own entry point and scheduler."""
import types

import pytest
import torch

import plain_netovik as plain
import replay_lib as rl
from helpers import note_error, oracle_logits, random_tokens, read_config, rel_err, tol
from netovik_models import CLOSE_CALL, NETOVIK_LENGTHS, NETOVIK_PAGE, comparable_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
NAMES = ["nvA", "nvB", "nvC", "nvD"]


def _ops():
    from tffinfer_amd.kernels import ops
    return ops


def _err(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def _i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def _batch(lengths, starts, slots=None):
    """The device tables of a step in which request r brings lengths[r] tokens after starts[r]."""
    cu, pos, req = [0], [], []
    for r, (n, s) in enumerate(zip(lengths, starts)):
        cu.append(cu[-1] + n)
        pos += list(range(s, s + n))
        req += [r] * n
    return types.SimpleNamespace(token_req=_i32(req), positions=_i32(pos), cu_tokens=_i32(cu), num_reqs=len(lengths),
                                 max_new_tokens=max(lengths), host_cu_tokens=cu,
                                 state_slots=_i32(slots if slots is not None else list(range(len(lengths)))))


# ---------------------------------------------------------------- mechanisms, one by one ---

@pytest.mark.parametrize("H,groups", [(60, 1), (60, 3), (256, 2), (1000, 5), (4096, 2), (5000, 1)])
@pytest.mark.parametrize("planes", [1, 3])
def test_norm_on_a_sublayers_output(H, groups, planes):
    ops = _ops()
    g = torch.Generator().manual_seed(H + planes)
    n, eps = 5, 1e-3
    x = torch.randn(n, H, generator=g) * 2
    w = 1 + 0.2 * torch.randn(H, generator=g)
    delta = torch.randn(planes, n, H, generator=g) * 3
    normed = plain.group_norm(delta.double().sum(0), w.double(), groups, eps)
    resid = x.clone().to(DEV)
    d = (delta[0] if planes == 1 else delta).contiguous().to(DEV)
    out = ops.group_rmsnorm_add(resid, d, w.to(DEV), groups, eps, torch.bfloat16)
    assert _err(resid, x.double() + normed) < 2e-6
    assert torch.equal(out.cpu(), resid.cpu().to(torch.bfloat16))      # the copy is the stream, rounded once
    resid = x.clone().to(DEV)
    assert ops.group_rmsnorm_add(resid, d, w.to(DEV), groups, eps, None) is None
    assert _err(resid, x.double() + normed) < 2e-6
    if planes == 1:     # the norm of chosen rows of the stream itself (the model's last norm)
        rows = _i32([4, 0, 2])
        y = ops.group_rmsnorm_add(None, d, w.to(DEV), groups, eps, torch.float32, rows=rows)
        assert _err(y, normed[[4, 0, 2]]) < 2e-6


@pytest.mark.parametrize("T,W", [(1, 48), (7, 321), (33, 1024)])
def test_sum_over_depth(T, W):
    ops = _ops()
    g = torch.Generator().manual_seed(T)
    depths = 5
    hist = torch.zeros(depths, T, W, device=DEV)
    ref_hist = []
    x = torch.randn(T, W, generator=g)
    for n in range(1, depths + 1):
        coef = torch.randn(n, generator=g)
        ref_hist.append(x.double())
        want = sum(coef[j].double() * ref_hist[j] for j in range(n))
        xd = x.to(DEV)
        out = ops.depth_average(hist, n, coef.to(DEV), xd, torch.bfloat16)
        assert _err(xd, want) < 2e-6 and torch.equal(out.cpu(), xd.cpu().to(torch.bfloat16))
        assert torch.equal(hist[n - 1].cpu(), x)
        x = xd.cpu() + torch.randn(T, W, generator=g)      # what a next layer would make of it


def test_mixes_with_the_token_before():
    """Three requests in one step: one at its start (zeros before it), one whose portion goes on from the
    state, one of a single token; the row before a portion's first token comes from the request's slot."""
    ops = _ops()
    g = torch.Generator().manual_seed(3)
    W, lengths, starts, slots = 40, [5, 1, 3], [0, 7, 2], [2, 0, 3]
    x = torch.randn(sum(lengths), W, generator=g)
    mu = torch.rand(5, W, generator=g)
    state = torch.randn(5, 16 + W, generator=g)
    state[2, 16:] = 0
    out = ops.token_shift_mix(x.to(DEV), state.to(DEV), 16, mu.to(DEV), _batch(lengths, starts, slots), torch.float32).cpu()
    at = 0
    for n, s, slot in zip(lengths, starts, slots):
        rows = x[at:at + n].double()
        before = plain.shifted(rows, state[slot, 16:].double())
        for m in range(5):
            assert _err(out[m, at:at + n], rows + (before - rows) * mu[m].double()) < 1e-6
        at += n


@pytest.mark.parametrize("H,D", [(3, 8), (2, 16), (2, 24), (1, 40), (2, 48), (2, 64), (1, 100), (2, 128)])
def test_recurrence_whole_and_in_portions(H, D):
    """The recurrence over 70 tokens at once, and the same tokens in portions of 1 to 30 beside another
    request, with the state carried in a slot: the same numbers, bit for bit; decays from almost 0 to almost 1."""
    ops = _ops()
    g = torch.Generator().manual_seed(D)
    T, W = 70, 16
    r, k, v = (torch.randn(T, H * D, generator=g) for _ in range(3))
    z = 3 * torch.randn(T, H * D, generator=g)
    w0 = torch.rand(H * D, generator=g) * 3.5 - 3
    u = torch.randn(H * D, generator=g)
    x = torch.randn(T, W, generator=g)
    w = torch.exp(-torch.exp(z.double() + w0.double()))
    ref, S_ref = plain.wkv_recurrence(r.double().view(T, H, D), k.double().view(T, H, D), v.double().view(T, H, D),
                                      w.view(T, H, D), u.double().view(H, D))
    row = H * D * D + W
    state = torch.zeros(4, row, device=DEV)
    dev = [t.to(DEV) for t in (r, k, v, z)]
    whole = ops.wkv_recurrence(*dev, w0.to(DEV), u.to(DEV), state, _batch([T], [0], [1]), H, D, x=x.to(DEV), prev_off=H * D * D)
    assert _err(whole, ref.reshape(T, H * D)) < 2e-5
    assert _err(state[1, :H * D * D].view(H, D, D), S_ref) < 2e-5
    assert torch.equal(state[1, H * D * D:].cpu(), x[-1])
    assert float(state[0].abs().max()) == 0 and float(state[2].abs().max()) == 0
    # in portions, in slot 3, beside a second request in slot 0 whose tokens are the same ones shifted
    state.zero_()
    got, at = [], 0
    for n in (1, 2, 30, 1, 7, 29):
        other = min(at + 1, T - n)
        idx = list(range(at, at + n)) + [other]
        step = [t[idx].contiguous() for t in dev]
        o = ops.wkv_recurrence(*step, w0.to(DEV), u.to(DEV), state, _batch([n, 1], [at, 0], [3, 0]), H, D,
                               x=x[idx].to(DEV), prev_off=H * D * D)
        got.append(o[:n])
        at += n
    # (heads of 64 and 128 run long portions in a form of their own, whose sums go in another order)
    if D in (64, 128):
        assert _err(torch.cat(got, 0), whole) < 2e-6
    else:
        assert torch.equal(torch.cat(got, 0), whole)


@pytest.mark.parametrize("H,D", [(3, 8), (2, 40), (1, 128)])
def test_norm_over_each_head_and_gate(H, D):
    ops = _ops()
    g = torch.Generator().manual_seed(H)
    T, eps = 9, 1e-4
    o, gz = 5 * torch.randn(T, H * D, generator=g), 2 * torch.randn(T, H * D, generator=g)
    w = 1 + 0.3 * torch.randn(H * D, generator=g)
    ref = plain.unit_rms(o.double().view(T, H, D), eps).reshape(T, H * D) * w.double() * plain.silu(gz.double())
    assert _err(ops.head_norm_gate(o.to(DEV), gz.to(DEV), w.to(DEV), eps, H, D, torch.float32), ref) < 2e-6


def test_distance_buckets_of_the_package():
    from tffinfer_amd.parts.mixed_attention import distance_buckets
    for B, Dmax in ((32, 120), (6, 25), (16, 64), (8, 33), (12, 40)):
        got = distance_buckets(B, Dmax).tolist()
        assert got == [plain.distance_bucket(n, B, Dmax) for n in range(Dmax + 1)]
        assert got[-1] == B - 1 and plain.distance_bucket(10 * Dmax, B, Dmax) == B - 1


class _Cache:
    """Keys and values of one request (or several) in pages that lie in a shuffled order."""

    def __init__(self, G, D, page, lengths, dtype, seed=0):
        self.page = page
        blocks = [-(-n // page) for n in lengths]
        total = sum(blocks) + 3
        perm = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
        self.tables, at = [], 0
        for b in blocks:
            self.tables.append(perm[at:at + b])
            at += b
        self.k = torch.zeros(total, G, page, D, dtype=dtype, device=DEV)
        self.v = torch.zeros(total, G, D, page, dtype=dtype, device=DEV)
        width = max(blocks)
        self.bt = _i32([t + [0] * (width - len(t)) for t in self.tables])

    def view(self, reqs, starts, lengths):
        slots = []
        for r, s, n in zip(reqs, starts, lengths):
            slots += [self.tables[r][j // self.page] * self.page + j % self.page for j in range(s, s + n)]
        bt = self.bt[torch.tensor(reqs, device=DEV)].contiguous()
        return types.SimpleNamespace(k_cache=self.k, v_cache=self.v, block_tables=bt, slot_mapping=_i32(slots),
                                     page_size=self.page)


def _attention_case(H, G, D, T, seed, loud=None):
    """Random unit queries and keys; ``loud`` = (query, key, head): that pair's score stands out."""
    g = torch.Generator().manual_seed(seed)
    qk = torch.randn(T, (H + G) * D, generator=g)
    qb, kb = 0.3 * torch.randn(H * D, generator=g), 0.3 * torch.randn(G * D, generator=g)
    if loud is not None:
        i, j, h = loud
        kv = h // (H // G)
        direction = torch.randn(D, generator=g)
        qk[i, h * D:(h + 1) * D] = 6 * direction - qb[h * D:(h + 1) * D]
        qk[j, (H + kv) * D:(H + kv + 1) * D] = 6 * direction - kb[kv * D:(kv + 1) * D]
    return qk, qb, kb


def _plain_attention(qk, qb, kb, H, G, D, eps, **kw):
    T = qk.shape[0]
    q = (qk[:, :H * D].double() + qb.double()).view(T, H, D)
    k = (qk[:, H * D:].double() + kb.double()).view(T, G, D)
    kw = {n: (v.double() if isinstance(v, torch.Tensor) else v) for n, v in kw.items()}
    return plain.attend(plain.unit_rms(q, eps), plain.unit_rms(k, eps), k, **kw).reshape(T, H * D)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,page", [(4, 2, 16, 16), (3, 3, 8, 8), (12, 4, 8, 32), (1, 1, 40, 8), (6, 1, 64, 16), (5, 5, 12, 16),
                                        (5, 5, 32, 16), (32, 8, 128, 32), (9, 3, 64, 8), (16, 16, 32, 16), (12, 4, 64, 16), (20, 2, 32, 32)])
def test_attention_with_every_term(H, G, D, page, dtype):
    """Bias, cap, exchange between heads, window with kept first tokens and the 1 in the denominator, on a
    prompt in one step and on the same tokens as a prompt's portion followed by single tokens; then each
    term left out in turn.  (In bfloat16, heads of 32, 64 and 128 run portions of 64 tokens and more on the
    matrix cores, sixteen queries a block.)"""
    ops = _ops()
    g = torch.Generator().manual_seed(H * D)
    T, eps, window, keep, B, Dmax = 150, 1e-5, 37, 5, 10, 50
    qk, qb, kb = _attention_case(H, G, D, T, H + D)
    rel = torch.randn(B, H, generator=g)
    talk = torch.eye(H) + 0.5 * torch.randn(H, H, generator=g)
    from tffinfer_amd.parts.mixed_attention import distance_buckets
    table = rel[distance_buckets(B, Dmax)].contiguous().to(DEV)
    limit = 2e-5 if dtype == torch.float32 else 3e-2
    scale = min(0.7, 6.0 / D)       # (unit queries and keys: their products reach D)
    variants = [dict(cap=4.0, rel=rel, talk=talk, window=window, keep=keep, sink=True),
                dict(cap=0.0, rel=None, talk=None, window=None, keep=0, sink=False),
                dict(cap=4.0, rel=rel, talk=None, window=window, keep=0, sink=True),
                dict(cap=0.0, rel=None, talk=talk, window=window, keep=keep, sink=False)]
    for kw in variants:
        ref = _plain_attention(qk, qb, kb, H, G, D, eps, scale=scale, bias_max=Dmax, **kw)
        args = dict(scale=scale, softcap=kw["cap"], bias=table if kw["rel"] is not None else None,
                    mix=kw["talk"].to(DEV) if kw["talk"] is not None else None, window=kw["window"] or 0,
                    keep_first=kw["keep"], sink=kw["sink"])
        for cuts in ([T], [100] + [1] * 50, [3, 2, 61, 64, 20]):
            cache = _Cache(G, D, page, [T], dtype, seed=len(cuts))
            outs, at = [], 0
            for n in cuts:
                kv = cache.view([0], [at], [n])
                q = ops.qk_bias_norm_store(qk[at:at + n].contiguous().to(DEV), qb.to(DEV), kb.to(DEV), eps, H, G, D, kv)
                outs.append(ops.mixed_attention(q, H, G, D, kv, _batch([n], [at]), **args))
                at += n
            err = _err(torch.cat(outs, 0), ref)
            assert err < limit, f"{[k for k, v in kw.items() if v is not None and v is not False and v != 0]} cut {cuts[:3]}: {err:.3e}"


@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("edge", ["inside", "outside", "kept", "not_kept"])
def test_a_loud_key_at_the_windows_and_the_kept_tokens_edges(edge, decode):
    """One key whose score with the last query stands far out: just inside the window the output is that
    key's value, just outside it is not; the last of the kept first tokens is seen from anywhere, the one
    after it is not.  Among 300 keys, across page borders, in a prompt and in decoding."""
    ops = _ops()
    H, G, D, T, page, eps, window, keep = 2, 1, 16, 300, 16, 1e-6, 130, 6
    j = {"inside": T - window, "outside": T - window - 1, "kept": keep - 1, "not_kept": keep}[edge]
    qk, qb, kb = _attention_case(H, G, D, T, 5, loud=(T - 1, j, 1))
    cache = _Cache(G, D, page, [T], torch.float32)
    outs, at = [], 0
    for n in ([T - 1, 1] if decode else [T]):
        kv = cache.view([0], [at], [n])
        q = ops.qk_bias_norm_store(qk[at:at + n].contiguous().to(DEV), qb.to(DEV), kb.to(DEV), eps, H, G, D, kv)
        outs.append(ops.mixed_attention(q, H, G, D, kv, _batch([n], [at]), scale=3.0, window=window, keep_first=keep,
                                        sink=True))
        at += n
    out = torch.cat(outs, 0)[-1].view(H, D)[1].cpu()
    value = (qk[j, H * D:] + kb).float()
    near = torch.allclose(out, value, atol=2e-2)
    assert near == (edge in ("inside", "kept")), edge
    ref = _plain_attention(qk, qb, kb, H, G, D, eps, scale=3.0, cap=0.0, rel=None, bias_max=0, talk=None, window=window, keep=keep)
    assert _err(torch.cat(outs, 0), ref) < 2e-5


def test_the_sink_takes_weight():
    """Keys that all score far below zero: the 1 in the denominator takes nearly all the weight and the
    output nearly vanishes; without it the output is an average of values."""
    ops = _ops()
    H, G, D, T, eps = 2, 2, 8, 20, 1e-6
    qk, qb, kb = _attention_case(H, G, D, T, 9)
    cache = _Cache(G, D, 8, [T], torch.float32)
    kv = cache.view([0], [0], [T])
    q = ops.qk_bias_norm_store(qk.to(DEV), qb.to(DEV), kb.to(DEV), eps, H, G, D, kv)
    low = torch.full((4, H), -12.0, device=DEV)
    with_sink = ops.mixed_attention(q, H, G, D, kv, _batch([T], [0]), scale=0.1, bias=low, sink=True)
    without = ops.mixed_attention(q, H, G, D, kv, _batch([T], [0]), scale=0.1, bias=low, sink=False)
    assert float(with_sink.abs().max()) < 1e-3 < float(without.abs().max())


def test_batches_of_unequal_requests_share_the_attention():
    """Three requests in one step (a prompt's portion, a single token, a whole short prompt) give what each
    gives alone, bit for bit."""
    ops = _ops()
    H, G, D, page, eps = 4, 2, 16, 16, 1e-6
    lengths = [90, 41, 7]
    cases = [_attention_case(H, G, D, n, 20 + n) for n in lengths]
    qb, kb = cases[0][1], cases[0][2]
    args = dict(scale=0.5, softcap=6.0, window=33, keep_first=2, sink=True, splits=1)
    alone, cache = [], _Cache(G, D, page, lengths, torch.float32, seed=4)
    for r, (n, c) in enumerate(zip(lengths, cases)):
        kv = cache.view([r], [0], [n])
        q = ops.qk_bias_norm_store(c[0].to(DEV), qb.to(DEV), kb.to(DEV), eps, H, G, D, kv)
        alone.append(ops.mixed_attention(q, H, G, D, kv, _batch([n], [0]), **args))
    cache2 = _Cache(G, D, page, lengths, torch.float32, seed=5)
    firsts = [60, 40, 0]
    for r in (0, 1):        # what came before this step
        kv = cache2.view([r], [0], [firsts[r]])
        ops.qk_bias_norm_store(cases[r][0][:firsts[r]].contiguous().to(DEV), qb.to(DEV), kb.to(DEV), eps, H, G, D, kv)
    news = [n - f for n, f in zip(lengths, firsts)]
    kv = cache2.view([0, 1, 2], firsts, news)
    rows = torch.cat([c[0][f:] for c, f in zip(cases, firsts)], 0).contiguous().to(DEV)
    q = ops.qk_bias_norm_store(rows, qb.to(DEV), kb.to(DEV), eps, H, G, D, kv)
    got = ops.mixed_attention(q, H, G, D, kv, _batch(news, firsts), **args)
    want = torch.cat([a[f:] for a, f in zip(alone, firsts)], 0)
    assert torch.equal(got, want)
    # the keys of each token dealt to several blocks and merged: the same to rounding
    for splits in (None, 2, 5):
        assert _err(ops.mixed_attention(q, H, G, D, kv, _batch(news, firsts), **dict(args, splits=splits)), want) < 2e-6


@pytest.mark.parametrize("E,top", [(8, 3), (2, 2), (5, 1), (70, 4)])
def test_softmax_router_and_plain_gated_experts(E, top):
    ops = _ops()
    g = torch.Generator().manual_seed(E)
    T, W, ff = 40, 48, 24
    x = torch.randn(T, W, generator=g)
    P = {"router": torch.randn(E, W, generator=g).double()}
    for e in range(E):
        P[f"e{e}.gate"], P[f"e{e}.up"] = (0.3 * torch.randn(ff, W, generator=g).double() for _ in range(2))
        P[f"e{e}.down"] = 0.3 * torch.randn(W, ff, generator=g).double()
    ref = plain.moe_ff({"router": {"top": top}}, P, x.double())
    s = plain.router_scores(P, x.double())
    logits = (x.double() @ P["router"].T).float().to(DEV)
    idx, wts = ops.route_topk(None, None, None, top, logits=logits, softmax=True)
    want_idx = torch.argsort(s, dim=-1, descending=True, stable=True)[:, :top]
    assert torch.equal(idx.cpu().long(), want_idx)
    assert _err(wts, torch.gather(s, 1, want_idx)) < 1e-5
    stack = lambda n: torch.stack([P[f"e{e}.{n}"] for e in range(E)], 0).float().to(DEV)     # noqa: E731
    out = ops.routed_experts(x.to(DEV), stack("gate"), stack("up"), stack("down"), idx, wts, float("inf"), 1.0, up_offset=0.0)
    assert _err(ops.as_tensor(out), ref) < 2e-5
    b16 = lambda t: t.to(torch.bfloat16)        # noqa: E731
    for by_tiles in (False, True):
        out = ops.routed_experts(b16(x).to(DEV), b16(stack("gate")), b16(stack("up")), b16(stack("down")), idx, wts,
                                 float("inf"), 1.0, by_tiles=by_tiles, up_offset=0.0)
        assert _err(ops.as_tensor(out), ref) < 3e-2


# ---------------------------------------------------------------------- whole models ---

def requests_for(name, model_dir):
    V = read_config(model_dir)["vocab"]
    return {f"{name}{i}": random_tokens(n, V, 2000 + 11 * i + n) for i, n in enumerate(NETOVIK_LENGTHS[name])}


def check(model_dir, reqs, steps, results, dtype, name):
    """A request's rows before its first close call: in bfloat16 among the experts' scores, in both types a first
    token whose recurrence output all but cancels."""
    before = {rid: comparable_tokens(model_dir, tuple(toks), dtype) for rid, toks in reqs.items()}
    total = sum(len(t) for t in reqs.values())
    assert sum(before.values()) >= total // (5 if dtype == "bfloat16" else 2), "too little of these requests can be compared"
    return rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype, compare_before=before)


def make_runner(model_dir, dtype, page_size, num_pages, max_seqs=4, use_graphs=False):
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    model = load_model(model_dir, DTYPES[dtype], DEV)
    return ModelRunner(model, page_size=page_size, num_pages=num_pages, max_seqs=max_seqs, max_model_len=512,
                       use_graphs=use_graphs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_residual_stream_after_every_layer(netovik_dirs, name, dtype):
    """Layer by layer, so that a fault names its layer."""
    from tffinfer_amd.engine.batch import StepEntry, build_step_batch
    from tffinfer_amd.engine.runner import StepContext
    d = netovik_dirs[name]
    V = read_config(d)["vocab"]
    # (the first of a few sequences of which bfloat16 can be compared for twenty tokens and more)
    toks = next(t for t in (random_tokens(45, V, 77 + s) for s in range(40)) if comparable_tokens(d, tuple(t)) >= 20)
    want = []
    plain.forward(*plain.load(d), toks, want)
    upto = len(toks) if dtype == "float32" else comparable_tokens(d, tuple(toks))
    runner = make_runner(d, dtype, NETOVIK_PAGE[name], 16)
    model = runner.model
    runner.add_request("a")
    e = [StepEntry("a", toks, [])]
    runner.reserve(e)
    batch = build_step_batch(e, runner.cache, runner.device, runner._pinned)
    ctx = StepContext(runner.ops, runner.act_dtype, batch, runner.max_model_len, runner._calls, runner.cache)
    resid, pending = model.embedding.forward(ctx, batch.token_ids), None
    assert len(model.schedule) == len(want)
    for it, call in enumerate(model.schedule):
        pending = model.blocks[call.layer].forward(ctx.for_call(it), resid, pending)
        assert pending is None
        err = _err(resid[:upto], want[it][:upto])
        assert err < (4e-5 if dtype == "float32" else 4e-2), f"layer call {it} (layer {call.layer}): {err:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("mode", ["whole", "tail", "chunks", "mixed"])
def test_replay_modes(netovik_dirs, name, dtype, mode):
    model_dir = netovik_dirs[name]
    reqs = requests_for(name, model_dir)
    steps = {"whole": rl.trace_whole, "tail": rl.trace_tail, "chunks": rl.trace_chunks,
             "mixed": rl.trace_mixed}[mode](reqs)
    ps = NETOVIK_PAGE[name]
    # the pool holds what is live at the worst moment and no more, so pages and slots are used again
    num_pages = rl.max_live_tokens(steps, unit=ps) // ps
    runner = make_runner(model_dir, dtype, ps, num_pages)
    results = rl.run_steps_in_process(runner, steps)
    worst = check(model_dir, reqs, steps, results, dtype, name)
    print(f"{name} {dtype} {mode}: worst rel. error {worst:.3e} over {len(steps)} steps, {num_pages} pages")
    assert all(g.pool.num_used == 0 for g in runner.cache.groups)


def test_a_windows_pages_go_back_but_the_kept_tokens_stay(netovik_dirs):
    """While a request grows far past its windows, every group with a window holds the pages of the window
    and of its kept first tokens and no more."""
    from tffinfer_amd.engine.batch import StepEntry
    d = netovik_dirs["nvB"]
    ps = NETOVIK_PAGE["nvB"]
    toks = random_tokens(130, read_config(d)["vocab"], 2130)
    runner = make_runner(d, "float32", ps, 20)
    runner.add_request("a")
    ref = oracle_logits(d, toks)
    at = 0
    for n in [50] + [1] * 80:
        lg = runner.step([StepEntry("a", toks[at:at + n], [n - 1])])
        at += n
        assert rel_err(lg[0], ref[at - 1]) <= tol("float32", "nvB")
    for g in runner.cache.groups:
        if g.spec.window:
            held = [b for b, p in enumerate(g.tables["a"]) if p >= 0]
            kept = -(-g.spec.keep_first // ps)
            assert held[:kept] == list(range(kept)) and len(held) <= kept + -(-(g.spec.window - 1) // ps) + 1
            assert held[kept] > kept        # (pages in between went back)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["nvB", "nvC"])
def test_long_decoding_through_captured_graphs(netovik_dirs, name, dtype):
    """Three requests decode some 150 tokens each, far past every window, as replays of captured
    HIP graphs beside eager prompt steps; state slots and pages of windows are used again."""
    model_dir = netovik_dirs[name]
    V = read_config(model_dir)["vocab"]
    reqs = {f"g{i}": random_tokens(n, V, 300 + n) for i, n in enumerate((160, 171, 190))}
    steps = rl.trace_mixed(reqs, max_live=3, prompt_frac=0.1, want_all=True)
    ps = NETOVIK_PAGE[name]
    runner = make_runner(model_dir, dtype, ps, rl.max_live_tokens(steps, unit=ps) // ps, use_graphs=True)
    results = rl.run_steps_in_process(runner, steps)
    check(model_dir, reqs, steps, results, dtype, name)
    assert runner._graphs, "no decode step ran as a graph"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(netovik_dirs, tmp_path, dtype):
    """The program itself, as a user calls it, on a model of this architecture, with its four state slots."""
    model_dir = netovik_dirs["nvA"]
    reqs = requests_for("nvA", model_dir)
    steps = rl.trace_mixed(reqs, want_all=False)
    out = rl.run_steps_subprocess(model_dir, dtype, steps, str(tmp_path / "out"), rl.max_live_tokens(steps, 64))
    check(model_dir, reqs, steps, out, dtype, "nvA")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["nvA", "nvB"])
def test_greedy_generation_through_the_engine(netovik_dirs, name, dtype):
    """The engine's own entry point: scheduler, portions beside decoding requests, graphs, sampler.
    Every kept row of logits matches the plain logits of the engine's own sequence, and every
    token is the first maximum of its row."""
    from tffinfer_amd import EngineOptions, LLMEngine
    d = netovik_dirs[name]
    V = read_config(d)["vocab"]
    prompts = [random_tokens(n, V, 80 + n) for n in (1, 9, 40, 70)]
    eng = LLMEngine.from_model_dir(d, EngineOptions(dtype=dtype, page_size=16, kv_tokens=512, max_num_seqs=3,
                                                    max_num_batched_tokens=48, prefill_chunk=24, max_model_len=256))
    eng.keep_logits = True
    res = eng.generate(prompts, max_new_tokens=40, ignore_eos=True)
    for r in res:
        assert len(r.output) == 40 and r.finish_reason == "length"
        ref = oracle_logits(d, r.prompt + r.output)
        margins = []
        plain.forward(*plain.load(d), r.prompt + r.output, margins=margins)
        close = torch.stack(margins).min(0).values < CLOSE_CALL if margins else torch.zeros(len(ref), dtype=torch.bool)
        for i, (row, tok) in enumerate(zip(r.logits, r.output)):
            assert tok == int(torch.argmax(row))
            if dtype == "bfloat16" and bool(close[:len(r.prompt) + i].any()):
                break       # (the sequence the engine chose made a close call: what follows may differ by more than rounding)
            err = rel_err(row, ref[len(r.prompt) + i - 1])
            note_error(dtype, d, err)
            assert err <= tol(dtype, d), f"output {i}: {err:.3e}"
    if dtype == "float32":
        cfg, W = plain.load(d)
        assert res[1].output[:8] == plain.greedy(cfg, W, prompts[1], 8)


def test_a_preempted_request_starts_its_state_again(netovik_dirs):
    """A pool so small that requests are preempted and computed again gives the tokens of a large pool:
    the state of a request that comes back starts at zero."""
    from tffinfer_amd import EngineOptions, LLMEngine
    d = netovik_dirs["nvC"]        # (its second layer keeps every key, so a small pool runs out)
    V = read_config(d)["vocab"]
    prompts = [random_tokens(n, V, 400 + n) for n in (30, 33, 28)]
    outs, preempted = [], []
    for pages in (64, 9):
        eng = LLMEngine.from_model_dir(d, EngineOptions(dtype="float32", page_size=16, num_pages=pages, max_num_seqs=3,
                                                        max_model_len=128))
        res = eng.generate(prompts, max_new_tokens=30, ignore_eos=True)
        outs.append([r.output for r in res])
        preempted.append(sum(r.num_preemptions for r in res))
    assert outs[0] == outs[1]
    assert preempted[0] == 0 and preempted[1] > 0


def test_the_command_line_with_a_configuration_file_of_this_architecture(tmp_path):
    """--config FILE --random-weights through bin/tffinfer: the weights are those of the folder that
    --save-model writes, the dumped rows are the logits that chose each token; a pool so small that
    requests are preempted and computed again gives the same tokens."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from netovik_models import NV_C
    prog = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "tffinfer")
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(NV_C))
    folder, dump = str(tmp_path / "nvC"), str(tmp_path / "logits.f32")
    common = [sys.executable, prog, "--config", str(cfg), "--random-weights", "--seed", "5", "--fp32", "--n-ctx", "256",
              "--n-predict", "12", "--ignore-eos", "--json", "--random-prompts", "3:30", "--page-size", "8",
              "--max-batches", "3"]
    p = subprocess.run(common + ["--save-model", folder, "--dump-logits", dump, "--kv-tokens", "512"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    recs = [json.loads(ln) for ln in p.stdout.strip().splitlines()]
    meta = json.load(open(dump + ".json"))
    V = NV_C["vocab"]
    rows = np.fromfile(dump, dtype="<f4").reshape(meta["shape"])
    assert meta["shape"] == [36, V]
    for i, r in enumerate(recs):
        ref = oracle_logits(folder, r["prompt"] + r["output"])
        first = meta["requests"][i]["first_row"]
        for j, tok in enumerate(r["output"]):
            row = torch.from_numpy(rows[first + j].copy())
            assert rel_err(row, ref[len(r["prompt"]) - 1 + j]) <= tol("float32", "nvC")
            assert tok == int(torch.argmax(row))
    tight = subprocess.run(common + ["--num-pages", "11"], capture_output=True, text=True, timeout=300)
    assert tight.returncode == 0, tight.stderr[-3000:]
    assert "preemption" in tight.stderr
    assert [json.loads(ln)["output"] for ln in tight.stdout.strip().splitlines()] == [r["output"] for r in recs]


@pytest.mark.parametrize("mode", ["chunks", "mixed"])
def test_prompt_attention_on_the_matrix_cores_beside_single_tokens(netovik_dirs, mode, monkeypatch):
    """Steps in which a prompt's portion of 16 tokens and more stands beside other requests' single tokens and
    short portions, all run by the kernel for prompts (its threshold on a step's tokens lowered for the test)."""
    ops = _ops()
    monkeypatch.setattr(ops, "MIXED_ATTENTION_Q16_TOKENS", 16)
    model_dir = netovik_dirs["nvC"]
    reqs = requests_for("nvC", model_dir)
    steps = {"chunks": rl.trace_chunks, "mixed": rl.trace_mixed}[mode](reqs)
    assert any(max(len(e["tokens"]) for e in s["entries"]) >= 16 and len(s["entries"]) > (1 if mode == "mixed" else 0) for s in steps)
    ps = NETOVIK_PAGE["nvC"]
    runner = make_runner(model_dir, "bfloat16", ps, rl.max_live_tokens(steps, unit=ps) // ps)
    results = rl.run_steps_in_process(runner, steps)
    check(model_dir, reqs, steps, results, "bfloat16", "nvC")
