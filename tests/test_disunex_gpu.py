"""The Disunex design in the engine against the plain implementation: each mechanism alone at
the level of its op, then whole models through the step function (whole prompts, decoding
token by token, portions down to two tokens, mixed batches on a pool whose pages and slots are
used again), and greedy generation through the engine's own entry point and scheduler."""
import math

import pytest
import torch

import plain_disunex as plain
import replay_lib as rl
from disunex_models import DISUNEX_LENGTHS, DISUNEX_PAGE, MIN_MARGIN, clear_tokens
from helpers import note_error, oracle_logits, random_tokens, read_config, rel_err, tol

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
NAMES = ["dxP", "dxQ", "dxR", "dxS", "dxT"]


def _ops():
    from tffinfer_amd.kernels import ops
    return ops


def _err(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


# ---------------------------------------------------------------- mechanisms, one by one ---

@pytest.mark.parametrize("H", [60, 256, 1000, 4096, 5000])
@pytest.mark.parametrize("alpha", [1.0, 2.5])
@pytest.mark.parametrize("planes", [0, 1, 3])
def test_norm_after_the_sum(H, alpha, planes):
    ops = _ops()
    g = torch.Generator().manual_seed(H + planes)
    n, eps = 5, 1e-3
    x = torch.randn(n, H, generator=g) * 2
    w = 0.2 * torch.randn(H, generator=g)
    delta = torch.randn(max(planes, 1), n, H, generator=g)
    ref = plain.norm_around_zero(alpha * x.double() + (delta.double().sum(0) if planes else 0.0), w.double(), eps)
    resid = x.clone().to(DEV)
    d = None if planes == 0 else (delta[0] if planes == 1 else delta).contiguous().to(DEV)
    out = ops.scale_add_rmsnorm(resid, d, (1.0 + w).to(DEV), eps, alpha, torch.bfloat16)
    assert _err(resid, ref) < 2e-6
    assert torch.equal(out.cpu(), resid.cpu().to(torch.bfloat16))      # the copy is the stream, rounded once
    resid = x.clone().to(DEV)
    assert ops.scale_add_rmsnorm(resid, d, (1.0 + w).to(DEV), eps, alpha, None) is None
    assert _err(resid, ref) < 2e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gelu(dtype):
    ops = _ops()
    z = torch.linspace(-6, 6, 1001).to(dtype)
    ref = plain.gelu_erf(z.double())
    assert _err(ops.gelu(z.to(DEV)), ref) < (1e-6 if dtype == torch.float32 else 5e-3)
    tanh_ref = 0.5 * z.double() * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z.double() + 0.044715 * z.double() ** 3)))
    assert _err(ops.gelu(z.to(DEV), tanh_form=True), tanh_ref) < (1e-6 if dtype == torch.float32 else 5e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,width", [(7, 3, 40), (5, 1, 64), (12, 2, 256), (70, 8, 100)])
def test_router_choice_goes_by_the_corrected_scores_and_weights_by_the_plain_ones(dtype, E, top, width):
    ops = _ops()
    g = torch.Generator().manual_seed(E * top)
    T = 33
    h = torch.randn(T, width, generator=g).to(dtype)
    router = (torch.randn(E, width, generator=g) * 0.3).to(torch.bfloat16).float()
    corr = torch.randn(E, generator=g)          # of the scores' own size: it changes who is chosen
    ref_idx, ref_w = plain.route(h.double(), router.double(), corr.double(), top)
    plain_idx, _ = plain.route(h.double(), router.double(), None, top)
    assert not torch.equal(ref_idx, plain_idx)
    idx, w = ops.route_topk(h.to(DEV), router.to(DEV), corr.to(DEV), top)
    assert torch.equal(idx.cpu().long(), ref_idx)
    assert _err(w, ref_w) < 1e-5
    assert torch.allclose(w.sum(-1).cpu(), torch.ones(T), atol=1e-5)
    idx0, _ = ops.route_topk(h.to(DEV), router.to(DEV), None, top)
    assert torch.equal(idx0.cpu().long(), plain_idx)
    # the logits from the engine's own product: a bfloat16 router times bfloat16 rows is exact in float32
    w_dev = router.to(dtype).to(DEV)
    z = ops.linear(h.to(DEV), ops.pack_weight(w_dev) if dtype == torch.bfloat16 else w_dev, out_dtype=torch.float32)
    idx1, w1 = ops.route_topk(None, None, corr.to(DEV), top, logits=z)
    assert torch.equal(idx1.cpu().long(), ref_idx) and _err(w1, ref_w) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [19, 150, 700])          # (700: tiles of 128 pairs where the experts are few)
@pytest.mark.parametrize("E,top,width,ff,limit", [(5, 2, 64, 40, 0.7), (3, 1, 100, 24, 1.5), (6, 3, 72, 17, 0.5),
                                                  (40, 4, 264, 136, 0.8)])
def test_experts(dtype, E, top, width, ff, limit, T):
    ops = _ops()
    g = torch.Generator().manual_seed(E + ff)
    h = torch.randn(T, width, generator=g).to(dtype)
    wg = (torch.randn(E, ff, width, generator=g) * 0.2).to(dtype)       # large enough that both clamps bite
    wu = (torch.randn(E, ff, width, generator=g) * 0.2).to(dtype)
    wd = (torch.randn(E, width, ff, generator=g) * 0.2).to(dtype)
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wts = torch.rand(T, top, generator=g)
    ref = torch.zeros(T, width, dtype=torch.float64)
    clamped = 0
    for t in range(T):
        for k in range(top):
            e = int(idx[t, k])
            ref[t] += wts[t, k].double() * plain.expert(h[t].double(), wg[e].double(), wu[e].double(), wd[e].double(), limit)
            clamped += int(((h[t].double() @ wu[e].double().T).abs() > limit).sum())
    assert clamped > 0
    args = (h.to(DEV), wg.to(DEV), wu.to(DEV), wd.to(DEV), idx.to(DEV), wts.to(DEV), limit, 1.702)
    out = ops.as_tensor(ops.routed_experts(*args))      # (150 tokens in bfloat16: dealt to the experts in tiles)
    assert _err(out, ref) < (2e-6 if dtype == torch.float32 else 1.5e-2)
    if dtype == torch.bfloat16:
        # a pair's row does not depend on how the pairs were dealt: the two paths agree to rounding,
        # and a token alone gives what it gives among the others
        few = ops.as_tensor(ops.routed_experts(*args, by_tiles=False))
        tiles = ops.as_tensor(ops.routed_experts(*args, by_tiles=True)) if ff % 8 == 0 and width % 8 == 0 else few
        assert _err(tiles, few) < 1e-2
        one = [a[7:8].contiguous() if isinstance(a, torch.Tensor) and a.shape[0] == T else a for a in args]
        alone = ops.as_tensor(ops.routed_experts(*one, by_tiles=ff % 8 == 0 and width % 8 == 0))
        assert torch.equal(alone[0], tiles[7])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rank,rot,dims,ps,Dp", [(40, 8, 8, 16, 48), (24, 16, 16, 8, 48), (150, 10, 6, 16, 192),
                                                 (20, 6, 6, 32, 32), (11, 0, 0, 8, 16)])
def test_latent_vector_and_rotated_key_go_to_their_slots(dtype, rank, rot, dims, ps, Dp):
    ops = _ops()
    from tffinfer_amd.parts.position import RotaryEmbedding
    g = torch.Generator().manual_seed(rank)
    T, pages, base, eps = 21, 7, 500.0, 1e-3
    x = torch.randn(T, 5 + rank + rot, generator=g).to(dtype)          # the part lies inside a wider row
    w = 1 + 0.2 * torch.randn(rank, generator=g)
    positions = torch.randint(0, 90, (T,), generator=g).to(torch.int32)
    slots = torch.randperm(pages * ps, generator=g)[:T].to(torch.int32)
    slots[3] = -1                                                       # a token that writes no key
    table = RotaryEmbedding(rot, base, "interleaved", dims).table(100, DEV) if dims else None
    kc = torch.zeros(pages, 1, ps, Dp, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, 1, Dp, ps, dtype=dtype, device=DEV)
    ops.latent_kv_store(x.to(DEV)[:, 5:], rank, rot, w.to(DEV), eps, table, positions.to(DEV), slots.to(DEV), kc, vc)
    c = plain.norm_plain(x[:, 5:5 + rank].double(), w.double(), eps)
    kr = x[:, 5 + rank:].double()
    if dims:
        kr = plain.rotate_pairs(kr, positions.tolist(), base, dims)
    t_ = 2e-6 if dtype == torch.float32 else 5e-3
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        row = kc[s // ps, 0, s % ps].cpu()
        assert _err(row[:rank], c[t]) < t_ and _err(vc[s // ps, 0, :rank, s % ps], c[t]) < t_
        if rot:
            assert _err(row[rank:rank + rot], kr[t]) < t_
        assert float(row[rank + rot:].abs().max() if Dp > rank + rot else 0) == 0
    written = sorted(int(s) for s in slots if s >= 0)
    assert int((kc.reshape(-1, Dp).abs().sum(-1) > 0).sum()) == len(written)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 8, 29, 300])
@pytest.mark.parametrize("H,K,N,tail,dims,pad", [(4, 16, 40, 8, 8, 48), (3, 300, 7, 0, 0, 7), (20, 8, 150, 10, 6, 192),
                                                 (2, 5, 11, 2, 2, 16), (3, 72, 100, 24, 24, 128), (2, 136, 70, 0, 0, 70)])
def test_products_per_head_with_gate_and_rotated_tail(dtype, T, H, K, N, tail, dims, pad):
    ops = _ops()
    from tffinfer_amd.parts.position import RotaryEmbedding
    g = torch.Generator().manual_seed(H * K + T)
    base = 300.0
    lead = 8 if K % 8 == 0 else 3        # (aligned rows run on the matrix cores in bfloat16, others on the general kernel)
    x = torch.randn(T, lead + H * (K + tail) + (-(lead + H * (K + tail))) % 8, generator=g).to(dtype)
    wt = (torch.randn(H, N, K, generator=g) * 0.3).to(dtype)
    positions = torch.randint(0, 50, (T,), generator=g).to(torch.int32)
    table = RotaryEmbedding(tail, base, "interleaved", dims).table(64, DEV) if dims else None
    out = ops.head_linear(x.to(DEV)[:, lead:], K + tail, wt.to(DEV), out_head=pad, tail=tail, cos_sin=table,
                          positions=positions.to(DEV)).view(T, H, pad)
    xh = x[:, lead:lead + H * (K + tail)].double().view(T, H, K + tail)
    ref = torch.einsum("thk,hnk->thn", xh[..., :K], wt.double())
    t_ = 3e-6 if dtype == torch.float32 else 8e-3
    assert _err(out[..., :N], ref) < t_
    if tail:
        rt = plain.rotate_pairs(xh[..., K:], positions.tolist(), base, dims) if dims else xh[..., K:]
        assert _err(out[..., N:N + tail], rt) < t_
    if pad > N + tail:
        assert float(out[..., N + tail:].abs().max()) == 0
    gate = torch.randn(T, H * N + 4, generator=g).to(dtype)
    gated = ops.head_linear(x.to(DEV)[:, lead:], K + tail, wt.to(DEV), gate=gate.to(DEV)[:, :H * N]).view(T, H, N)
    assert _err(gated, ref * torch.sigmoid(gate[:, :H * N].double().view(T, H, N))) < t_


def _sink_ref(q, keys, vals, positions, window, scale, sinks):
    """q [T, nq, d] against one key head: keys [S, d], vals [S, dv]."""
    T, nq, _ = q.shape
    out = torch.zeros(T, nq, vals.shape[1], dtype=torch.float64)
    S = keys.shape[0]
    for t in range(T):
        p = int(positions[t])
        vis = torch.tensor([[(0 <= p - j) and (not window or p - j < window) for j in range(S)]])
        for h in range(nq):
            s = (keys.double() @ q[t, h].double())[None] * scale
            out[t, h] = plain.softmax_with_sink(s, vis, None if sinks is None else sinks[h].double())[0] @ vals.double()
    return out


@pytest.mark.parametrize("nq,d,ps,window", [(8, 96, 16, 96), (4, 48, 16, 12), (20, 192, 16, 33), (3, 48, 8, 0),
                                            (1, 32, 32, 5), (5, 112, 8, 37)])
def test_attention_with_a_sink_on_every_kernel(nq, d, ps, window):
    """Prompt portions (blocks and single waves), single tokens beside them (runs of keys and
    their merge), the general kernel: the sink's term stands in every denominator once."""
    from test_kernels_gpu import _fake_step
    ops = _ops()
    entries = [(0, 37), (50, 13), (300, 1), (0, 1), (63, 2), (7, 70), (140, 1)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, 1, d, torch.bfloat16, seed=nq + d)
    T = batch.num_tokens
    g = torch.Generator().manual_seed(4)
    q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
    sinks = 2.0 + torch.randn(nq, generator=g)            # heavy: a third or more of every denominator
    scale = 1 / math.sqrt(d)
    ref = torch.zeros(T, nq, d, dtype=torch.float64)
    ref0 = torch.zeros(T, nq, d, dtype=torch.float64)
    for r in range(len(entries)):
        sel = (token_req == r).nonzero().flatten()
        ref[sel] = _sink_ref(q[sel], ks[r][:, 0], vs[r][:, 0], positions[sel], window, scale, sinks)
        ref0[sel] = _sink_ref(q[sel], ks[r][:, 0], vs[r][:, 0], positions[sel], window, scale, None)
    assert _err(ref0, ref) > 0.1          # leaving the sink out shows
    qd = q.reshape(T, nq * d).to(DEV)
    out = ops.attention_mfma(qd, nq, 1, d, kv, batch, window, scale, sinks=sinks.to(DEV))
    assert _err(out.reshape(T, nq, d), ref) < 1.2e-2
    gen = ops.attention_generic(qd, nq, 1, d, kv.k_cache, kv.v_cache, kv.block_tables, batch.token_req,
                                batch.positions, window, scale, sinks=sinks.to(DEV))
    assert _err(gen.reshape(T, nq, d), ref) < 1.2e-2
    for splits in (1, 3):                 # a decode-only step: keys split alike, merged by the reduce kernel
        dec = [(P + n - 1, 1) for P, n in entries]
        b2, kv2, ks2, vs2, pos2, tr2 = _fake_step(dec, ps, 1, d, torch.bfloat16, seed=nq)
        q2 = torch.randn(len(dec), nq, d, generator=g).to(torch.bfloat16)
        ref2 = torch.stack([_sink_ref(q2[r:r + 1], ks2[r][:, 0], vs2[r][:, 0], pos2[r:r + 1], window, scale, sinks)[0]
                            for r in range(len(dec))])
        out2 = ops.attention_mfma(q2.reshape(len(dec), nq * d).to(DEV), nq, 1, d, kv2, b2, window, scale,
                                  splits=splits, sinks=sinks.to(DEV))
        assert _err(out2.reshape(len(dec), nq, d), ref2) < 1.2e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("edge", ["inside", "outside"])
@pytest.mark.parametrize("decode", [False, True])
def test_a_key_at_the_windows_edge_is_seen_or_not(dtype, edge, decode):
    """One key is made to dominate its query's scores.  Just inside the window the output is that
    key's value; just outside, the output does not know it."""
    from test_kernels_gpu import _fake_step
    ops = _ops()
    nq, d, ps, window, ctx = 4, 48, 16, 29, 200
    entries = [(ctx - 1, 1)] if decode else [(ctx - 40, 40)]
    batch, kv, ks, vs, positions, token_req = _fake_step(entries, ps, 1, d, dtype, seed=7)
    T = batch.num_tokens
    q = torch.randn(T, nq, d).to(dtype)
    p = ctx - 1                                   # the last query's position
    j = p - window + 1 if edge == "inside" else p - window
    bt = kv.block_tables[0].cpu()
    loud = (40 * q[-1, 0].float() / q[-1, 0].float().norm()).to(dtype)
    kv.k_cache[bt[j // ps], 0, j % ps] = loud.to(DEV)
    out = ops.paged_attention(q.reshape(T, nq * d).to(DEV), nq, 1, d, kv, batch, window, 1.0,
                              sinks=torch.zeros(nq, device=DEV)).reshape(T, nq, d).cpu().float()
    near = torch.allclose(out[-1, 0], vs[0][j, 0].float(), atol=3e-2)
    assert near == (edge == "inside")


# ---------------------------------------------------------------------- whole models ---

def requests_for(name, model_dir):
    V = read_config(model_dir)["vocab"]
    # (sequences in which no choice of experts is a close call that rounding could turn)
    return {f"{name}{i}": list(clear_tokens(model_dir, n, V, 2000 + 11 * i + n)) for i, n in enumerate(DISUNEX_LENGTHS[name])}


def make_runner(model_dir, dtype, page_size, num_pages, max_seqs=4, use_graphs=False):
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    model = load_model(model_dir, DTYPES[dtype], DEV)
    return ModelRunner(model, page_size=page_size, num_pages=num_pages, max_seqs=max_seqs, max_model_len=512,
                       use_graphs=use_graphs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_residual_stream_after_every_layer(disunex_dirs, name, dtype):
    """Layer by layer, so that a fault names its layer: the stream after every call of the run order."""
    from tffinfer_amd.engine.batch import StepEntry, build_step_batch
    from tffinfer_amd.engine.runner import StepContext
    d = disunex_dirs[name]
    toks = list(clear_tokens(d, 45, read_config(d)["vocab"], 77))
    want = []
    plain.forward(*plain.load(d), toks, want)
    runner = make_runner(d, dtype, DISUNEX_PAGE[name], 16)
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
        err = _err(resid, want[it])
        assert err < (1e-5 if dtype == "float32" else 4e-2), f"layer call {it} (layer {call.layer}): {err:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("mode", ["whole", "tail", "chunks", "mixed"])
def test_replay_modes(disunex_dirs, name, dtype, mode):
    model_dir = disunex_dirs[name]
    reqs = requests_for(name, model_dir)
    steps = {"whole": rl.trace_whole, "tail": rl.trace_tail, "chunks": rl.trace_chunks,
             "mixed": rl.trace_mixed}[mode](reqs)
    ps = DISUNEX_PAGE[name]
    # the pool holds what is live at the worst moment and no more, so pages and slots are used again
    num_pages = rl.max_live_tokens(steps, unit=ps) // ps
    runner = make_runner(model_dir, dtype, ps, num_pages)
    results = rl.run_steps_in_process(runner, steps)
    worst = rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype)
    print(f"{name} {dtype} {mode}: worst rel. error {worst:.3e} over {len(steps)} steps, {num_pages} pages")
    assert all(g.pool.num_used == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["dxQ", "dxR"])
def test_long_decoding_through_captured_graphs(disunex_dirs, name, dtype):
    """Three requests decode 150 tokens each, far past every window, as replays of captured
    HIP graphs beside eager prompt steps; pages that a window has passed are given back on the way."""
    model_dir = disunex_dirs[name]
    V = read_config(model_dir)["vocab"]
    reqs = {f"g{i}": list(clear_tokens(model_dir, n, V, 300 + n)) for i, n in enumerate((160, 171, 190))}
    steps = rl.trace_mixed(reqs, max_live=3, prompt_frac=0.1, want_all=True)
    ps = DISUNEX_PAGE[name]
    runner = make_runner(model_dir, dtype, ps, rl.max_live_tokens(steps, unit=ps) // ps, use_graphs=True)
    results = rl.run_steps_in_process(runner, steps)
    rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype)
    assert runner._graphs, "no decode step ran as a graph"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(disunex_dirs, tmp_path, dtype):
    """The program itself, as a user calls it, on a model of this architecture."""
    model_dir = disunex_dirs["dxQ"]
    reqs = requests_for("dxQ", model_dir)
    steps = rl.trace_mixed(reqs, want_all=False)
    out = rl.run_steps_subprocess(model_dir, dtype, steps, str(tmp_path / "out"), rl.max_live_tokens(steps, 64))
    rl.check_against_oracle(model_dir, reqs, steps, out, tol(dtype, "dxQ"), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["dxQ", "dxS"])
def test_greedy_generation_through_the_engine(disunex_dirs, name, dtype):
    """The engine's own entry point: scheduler, portions beside decoding requests, graphs, sampler.
    Every kept row of logits matches the plain logits of the engine's own sequence, and every
    token is the first maximum of its row."""
    from tffinfer_amd import EngineOptions, LLMEngine
    d = disunex_dirs[name]
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
        close = torch.stack(margins).min(0).values < MIN_MARGIN if margins else torch.zeros(len(ref), dtype=torch.bool)
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


def test_the_command_line_with_a_configuration_file_of_this_architecture(tmp_path):
    """--config FILE --random-weights through bin/tffinfer: the weights are those of the folder that
    --save-model writes, the dumped rows are the logits that chose each token; a pool so small that
    requests are preempted and computed again gives the same tokens."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from disunex_models import DX_Q
    prog = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "tffinfer")
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(DX_Q))
    folder, dump = str(tmp_path / "dxQ"), str(tmp_path / "logits.f32")
    common = [sys.executable, prog, "--config", str(cfg), "--random-weights", "--seed", "5", "--fp32", "--n-ctx", "256",
              "--n-predict", "12", "--ignore-eos", "--json", "--random-prompts", "3:30", "--page-size", "8",
              "--max-batches", "3"]
    p = subprocess.run(common + ["--save-model", folder, "--dump-logits", dump, "--kv-tokens", "512"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    recs = [json.loads(ln) for ln in p.stdout.strip().splitlines()]
    meta = json.load(open(dump + ".json"))
    V = DX_Q["vocab"]
    rows = np.fromfile(dump, dtype="<f4").reshape(meta["shape"])
    assert meta["shape"] == [36, V]
    for i, r in enumerate(recs):
        ref = oracle_logits(folder, r["prompt"] + r["output"])
        first = meta["requests"][i]["first_row"]
        for j, tok in enumerate(r["output"]):
            row = torch.from_numpy(rows[first + j].copy())
            assert rel_err(row, ref[len(r["prompt"]) - 1 + j]) <= tol("float32", "dxQ")
            assert tok == int(torch.argmax(row))
    tight = subprocess.run(common + ["--num-pages", "11"], capture_output=True, text=True, timeout=300)
    assert tight.returncode == 0, tight.stderr[-3000:]
    assert "preemption" in tight.stderr
    assert [json.loads(ln)["output"] for ln in tight.stdout.strip().splitlines()] == [r["output"] for r in recs]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_forty_requests_decode_together(disunex_dirs, dtype):
    """Forty requests decode side by side as replays of a captured graph: in bfloat16 such a step deals
    its (token, expert) pairs to the experts in tiles, inside the graph, padding rows and all."""
    from tffinfer_amd import EngineOptions, LLMEngine
    d = disunex_dirs["dxQ"]
    V = read_config(d)["vocab"]
    prompts = [random_tokens(3 + i % 5, V, 500 + i) for i in range(40)]
    eng = LLMEngine.from_model_dir(d, EngineOptions(dtype=dtype, page_size=16, kv_tokens=40 * 32, max_num_seqs=40,
                                                    max_model_len=64))
    eng.keep_logits = True
    res = eng.generate(prompts, max_new_tokens=8, ignore_eos=True)
    assert eng.runner._graphs and max(eng.runner._graphs) >= 40
    checked = 0
    for r in res:
        assert len(r.output) == 8
        ref = oracle_logits(d, r.prompt + r.output)
        margins = []
        plain.forward(*plain.load(d), r.prompt + r.output, margins=margins)
        close = torch.stack(margins).min(0).values < MIN_MARGIN
        for i, (row, tok) in enumerate(zip(r.logits, r.output)):
            assert tok == int(torch.argmax(row))
            if dtype == "bfloat16" and bool(close[:len(r.prompt) + i].any()):
                break
            assert rel_err(row, ref[len(r.prompt) + i - 1]) <= tol(dtype, d), f"request {r.prompt}: output {i}"
            checked += 1
    assert checked > 200
