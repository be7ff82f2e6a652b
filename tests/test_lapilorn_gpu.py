"""Lapilorn on the GPU against the plain statement in ``oracle/lapilorn.py``: every mechanism alone, then whole
models through the engine -- whole prompts, token-by-token decoding, portions down to two tokens, mixed batches,
pages and state slots that are reused, greedy generation through ``LLM.generate``, the replay entry point.

The models are small and random (``tests/lapilorn_util.py``); where random numbers would hide a fault (one far key
among hundreds, a key on a page border or at a window's edge) the inputs are built so that it shows.
"""
import math
import random
from types import SimpleNamespace

import pytest
import torch

import lapilorn_util as lu
from oracle import lapilorn as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


def ragged(seqs, width=None):
    """seqs: [(ctx_len, new tokens, state slot, block table)] -> the step's ragged layout on the device."""
    q_start, token_seq = [0], []
    for i, (_, n, _, _) in enumerate(seqs):
        q_start.append(q_start[-1] + n)
        token_seq += [i] * n
    width = width or max(len(s[3]) for s in seqs) or 1
    tables = [list(s[3]) + [0] * (width - len(s[3])) for s in seqs]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)          # noqa: E731
    return SimpleNamespace(
        q_start=i32(q_start), ctx_len=i32([s[0] for s in seqs]), token_seq=i32(token_seq),
        state_slot=i32([s[2] for s in seqs]), block_tables=i32(tables).reshape(len(seqs), width), num_seqs=len(seqs),
        max_query_len=max(s[1] for s in seqs), max_pages_used=width,
        max_page_id=max([max(s[3]) for s in seqs if s[3]] or [0]), max_state_slot=max(s[2] for s in seqs))


def ops():
    from splitwise_amd import _C
    return _C.mixer_ops


def tol_of(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [48, 200, 1030])
def test_stream_add_norm(dtype, width):
    g = torch.Generator().manual_seed(width)
    rows = 7
    x = torch.randn(rows, width, generator=g) * 3
    a = torch.randn(rows, 2 * width, generator=g).to(dtype)[:, 5:5 + width]       # a view with a row stride
    b = torch.randn(rows, width, generator=g).to(dtype)
    c = torch.randn(rows, width, generator=g)
    w = torch.randn(width, generator=g) * 0.3
    for use in [(False, False, False), (True, False, False), (True, True, False), (True, True, True), (True, False, True)]:
        res = x.clone().to(DEV)
        out = torch.empty(rows, width, dtype=dtype, device=DEV)
        args = [t.to(DEV) if u else None for t, u in zip((a, b, c), use)]
        ops().stream_add_norm(res, w.to(DEV), 1.0, 1e-5, out, *args)
        want_res = x.double() + sum(t.double() for t, u in zip((a, b, c), use) if u)
        torch.testing.assert_close(res.cpu().double(), want_res, atol=1e-5, rtol=1e-6)
        torch.testing.assert_close(out.cpu().double(), oracle.offset_norm(want_res, w.double(), 1e-5), **tol_of(dtype))
    # the sum alone, no norm
    res = x.clone().to(DEV)
    ops().stream_add_norm(res, None, 1.0, 1e-5, None, None, b.to(DEV), None)
    torch.testing.assert_close(res.cpu().double(), x.double() + b.double(), atol=1e-5, rtol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff,limit", [(40, 0.8), (320, 1.25), (2100, 7.0), (33, math.inf)])
def test_feed_forward_activations(dtype, ff, limit):
    g = torch.Generator().manual_seed(ff)
    x = (torch.randn(5, 2 * ff + 3, generator=g) * 2).to(dtype)[:, 3:]
    out = torch.empty(5, ff, dtype=dtype, device=DEV)
    ops().clamped_glu(out, x.to(DEV), 1.702, limit, 1.0)
    gate = x[:, :ff].double().clamp(max=limit)
    up = x[:, ff:].double().clamp(-limit, limit)
    torch.testing.assert_close(out.cpu().double(), gate * torch.sigmoid(1.702 * gate) * (up + 1.0), **tol_of(dtype))
    y = x[:, :ff]
    out = torch.empty(5, ff, dtype=dtype, device=DEV)
    ops().relu2(out, y.to(DEV))
    torch.testing.assert_close(out.cpu().double(), torch.relu(y.double()).pow(2), **tol_of(dtype))


_SCALING = {"factor": 3.0, "low": 2.0, "high": 5.0, "original": 40}


@pytest.mark.parametrize("H,G,d,dv,rot,scaling", [(4, 2, 16, 32, 8, _SCALING), (3, 3, 8, 8, 8, None), (6, 2, 20, 24, 4, _SCALING),
                                                  (2, 1, 96, 64, 24, {"factor": 2.5, "low": 0.5, "high": 3.0, "original": 64}),
                                                  (2, 2, 10, 6, 0, None)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_and_cache_write(H, G, d, dv, rot, scaling, dtype):
    from splitwise_amd.model_executor.layers.basic import scaled_rotary_frequencies
    g = torch.Generator().manual_seed(H * 100 + d)
    rows, page = 9, 16
    positions = torch.tensor([0, 1, 2, 15, 16, 17, 300, 2047, 70000])
    proj = torch.randn(rows, H * d + G * d + G * dv + 7, generator=g).to(dtype)
    q, k, v = proj[:, :H * d], proj[:, H * d:H * d + G * d], proj[:, H * d + G * d:H * d + G * d + G * dv]
    cfg = {"base": 50.0, "dims": rot, "scaling": scaling}
    freqs = oracle.rotary_frequencies(cfg) if rot else []
    inv = scaled_rotary_frequencies(rot, 50.0, scaling) if rot else None
    if rot:
        torch.testing.assert_close(inv.double(), torch.tensor(freqs, dtype=F64), atol=0, rtol=1e-7)
        # the three regimes of the slowdown are all present where the test wants them
        if scaling is _SCALING and rot >= 8:
            plain = [50.0 ** (-2.0 * i / rot) for i in range(rot // 2)]
            ratios = [f / p for f, p in zip(freqs, plain)]
            assert ratios[0] == 1.0 and abs(ratios[-1] - 1 / 3.0) < 1e-12 and any(1 / 3.0 + 1e-6 < r < 1 - 1e-6 for r in ratios)
    slots = torch.tensor([40, 3, 17, 64, 65, 0, 99, 31, 32])
    kc = torch.zeros(8, page, G * d, dtype=dtype, device=DEV)
    vc = torch.zeros(8, page, G * dv, dtype=dtype, device=DEV)
    q_out = torch.empty(rows, H * d, dtype=torch.float32, device=DEV)
    dev = proj.to(DEV)
    ops().rope_cache(q_out, dev[:, :H * d], dev[:, H * d:H * d + G * d], dev[:, H * d + G * d:H * d + G * d + G * dv],
                     positions.to(DEV), None if inv is None else inv.to(DEV), H, G, d, dv, kc, vc, slots.to(DEV))
    for t in range(rows):
        want_q = oracle.rotate(q[t].double().view(H, d), int(positions[t]), freqs).reshape(-1)
        want_k = oracle.rotate(k[t].double().view(G, d), int(positions[t]), freqs).reshape(-1)
        torch.testing.assert_close(q_out[t].cpu().double(), want_q, atol=2e-5, rtol=2e-5)
        torch.testing.assert_close(kc.view(-1, G * d)[slots[t]].cpu().double(), want_k, **tol_of(dtype))
        torch.testing.assert_close(vc.view(-1, G * dv)[slots[t]].cpu(), v[t])
    # a layer that reads another layer's keys rotates its queries only
    q2 = torch.empty_like(q_out)
    ops().rope_cache(q2, dev[:, :H * d], None, None, positions.to(DEV), None if inv is None else inv.to(DEV), H, G, d, dv,
                     None, None, None)
    torch.testing.assert_close(q2, q_out, atol=0, rtol=0)


def _attention_case(H, G, d, dv, n, spikes, seed, big=6.0):
    """Random q, k, v with, for every (query position, key position, head) in ``spikes``, that query and key made
    long along a direction of their own, so that the pair's score towers over the query's other scores."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n, H, d, generator=g) * 0.5
    k = torch.randn(n, G, d, generator=g) * 0.5
    v = torch.randn(n, G, dv, generator=g)
    for num, (i, j, a) in enumerate(spikes):
        e = torch.zeros(d)
        e[num % d] = 1.0
        q[i, a] = big * e + 0.05 * q[i, a]
        k[j, a // (H // G)] = big * e + 0.05 * k[j, a // (H // G)]
    return q, k, v


def _paged(k, v, G, d, dv, page, dtype, seed):
    """Keys / values in pages handed out in a shuffled order; unused pages hold NaN."""
    n = k.shape[0]
    pages = -(-n // page)
    order = list(range(pages + 3))
    random.Random(seed).shuffle(order)
    table = order[:pages]
    kc = torch.full((pages + 3, page, G * d), float("nan"), dtype=dtype)
    vc = torch.full((pages + 3, page, G * dv), float("nan"), dtype=dtype)
    for t in range(n):
        kc[table[t // page], t % page] = k[t].reshape(-1).to(dtype)
        vc[table[t // page], t % page] = v[t].reshape(-1).to(dtype)
    return kc.to(DEV), vc.to(DEV), table


@pytest.mark.parametrize("H,G,d,dv,page", [(4, 2, 16, 32, 16), (6, 6, 8, 8, 16), (3, 1, 24, 72, 8), (8, 2, 20, 40, 16),
                                           (2, 1, 128, 128, 64), (5, 1, 12, 130, 16), (4, 4, 64, 16, 32)])
@pytest.mark.parametrize("mode", ["prompt", "decode", "pairs", "portions"])
@pytest.mark.parametrize("cache_dtype,cap,window", [(torch.float32, 5.0, 0), (torch.bfloat16, 5.0, 0), (torch.float32, 0.0, 0),
                                                    (torch.float32, 5.0, 37)])
def test_capped_attention_edges(H, G, d, dv, page, mode, cache_dtype, cap, window):
    n = 300
    last = n - 1
    # a far key among hundreds, keys on both sides of a page border and of a 32-key tile, the query's own key, the
    # first key; with a window: the last key inside it and the first one outside (which must not be seen)
    spikes = [(last, 2, 0), (last - 1, page - 1, H - 1), (last - 2, page, 0), (last - 3, 31, H - 1), (last - 4, 32, 0),
              (last - 5, last - 5, H - 1), (100, 0, 0), (129, 127, H - 1), (128, 128, 0), (40, 39, H - 1)]
    if window:
        spikes += [(last - 6, last - 6 - window + 1, 0), (last - 7, last - 7 - window, H - 1), (200, 200 - window, 0)]
    q, k, v = _attention_case(H, G, d, dv, n, spikes, seed=H * 1000 + d)
    kc, vc, table = _paged(k, v, G, d, dv, page, cache_dtype, seed=d)
    kq, vq = kc.cpu().double(), vc.cpu().double()                     # what the cache holds after rounding
    kk = torch.stack([kq[table[t // page], t % page].view(G, d) for t in range(n)])
    vv = torch.stack([vq[table[t // page], t % page].view(G, dv) for t in range(n)])
    scale = 0.9
    want = oracle.causal_attention(q.double(), kk, vv, scale, cap or None, window).reshape(n, H * dv)
    gate = torch.randn(n, H * dv + 5, generator=torch.Generator().manual_seed(1)).to(cache_dtype)[:, 5:]
    if mode == "prompt":
        seqs, rows = [(0, n, 0, table)], list(range(n))
    elif mode == "decode":
        rows = list(range(n - 45, n)) + [0, 1, 33]
        seqs = [(t, 1, 0, table) for t in rows]
    elif mode == "pairs":                                             # steps of two tokens, and one of a single token
        firsts = list(range(n - 46, n, 2)) + [0, 32, 127]
        seqs = [(t, 2, 0, table) for t in firsts] + [(n - 47, 1, 0, table)]
        rows = [t + i for t in firsts for i in range(2)] + [n - 47]
    else:
        cuts, at = [], 0
        for size in [3, 2, 27, 1, 31, 2, 64, 2, 33, 5, 32, 98]:
            cuts.append((at, size, 0, table))
            at += size
        assert at == n
        random.Random(3).shuffle(cuts)                                # portions of "different sequences" in any order
        seqs, rows = cuts, [c[0] + i for c in cuts for i in range(c[1])]
    batch = ragged(seqs)
    qd = q[rows].reshape(len(rows), H * d).contiguous().to(DEV)
    for use_gate in (False, True):
        out = torch.empty(len(rows), H * dv, dtype=cache_dtype, device=DEV)
        gd = gate[rows].to(DEV) if use_gate else None
        ops().capped_attention(out, qd, kc, vc, gd, batch, H, G, d, dv, scale, cap, window)
        ref = want[rows] * (torch.sigmoid(gate[rows].double()) if use_gate else 1.0)
        tol = dict(atol=3e-5, rtol=3e-5) if cache_dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(out.cpu().double(), ref, **tol)


def _run_lightning(proj, sizes, decay, state, steps, H, d, dv):
    """steps: [[(sequence, first token, tokens, slot)]]; proj[s]: the sequence's projections [n, q | k | v]."""
    nk, nv = sizes
    outs = {s: torch.zeros(p.shape[0], nv, dtype=torch.float32) for s, p in proj.items()}
    for step in steps:
        x = torch.cat([proj[s][lo:lo + n] for s, lo, n, _ in step]).to(DEV)
        batch = ragged([(lo, n, slot, []) for _, lo, n, slot in step], width=1)
        o = torch.empty(x.shape[0], nv, dtype=torch.float32, device=DEV)
        ops().lightning(o, x[:, :nk], x[:, nk:2 * nk], x[:, 2 * nk:2 * nk + nv], decay, state, batch, H, d, dv)
        at = 0
        for s, lo, n, _ in step:
            outs[s][lo:lo + n] = o[at:at + n].cpu()
            at += n
    return outs


@pytest.mark.parametrize("H,d,dv,decay", [(3, 24, 16, (0.5, 0.9, 0.99)), (1, 8, 8, (0.999,)), (2, 64, 48, (0.61, 0.97)),
                                          (2, 100, 48, (0.2, 1.0)), (4, 40, 130, (0.9, 0.8, 0.999, 0.05)), (1, 256, 64, (0.95,))])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lightning_recurrence(H, d, dv, decay, dtype):
    """Two sequences interleaved over three state slots that held other sequences before: whole chunks, chunk
    borders (31, 32, 33 tokens), portions of one and two tokens, a first portion of one token, a run long enough
    to be cut into segments that run side by side (from a carried state, beside a single token of the other
    sequence), and 70 tokens decoded one by one; against the recurrence run token by token in double precision."""
    g = torch.Generator().manual_seed(H * 100 + d)
    nk, nv = H * d, H * dv
    lens = {"a": 640, "b": 139}
    proj = {s: (torch.randn(n, 2 * nk + nv + 3, generator=g) * 1.2).to(dtype) for s, n in lens.items()}
    state = torch.full((3, H, d, dv), float("nan"), dtype=torch.float32, device=DEV)     # slots are never cleared
    dec = torch.tensor(decay, dtype=torch.float32, device=DEV)
    steps = [[("a", 0, 1, 2)], [("a", 1, 31, 2), ("b", 0, 33, 0)], [("b", 33, 2, 0), ("a", 32, 32, 2)],
             [("a", 64, 33, 2)], [("a", 97, 2, 2), ("b", 35, 64, 0)], [("a", 99, 471, 2), ("b", 99, 1, 0)]]
    steps += [[("a", 570 + i, 1, 2)] + ([("b", 100 + i, 1, 0)] if i < 39 else []) for i in range(70)]
    outs = _run_lightning(proj, (nk, nv), dec, state, steps, H, d, dv)
    silu = torch.nn.functional.silu
    final = {}
    for s, n in lens.items():
        p = proj[s].double()
        want, final[s] = oracle.decayed_outer_products(silu(p[:, :nk]).view(n, H, d), silu(p[:, nk:2 * nk]).view(n, H, d),
                                                       silu(p[:, 2 * nk:2 * nk + nv]).view(n, H, dv), list(decay))
        scale = want.abs().max()
        assert (outs[s].double() - want.reshape(n, nv)).abs().max() < 2e-5 * scale, s
    assert (state[2].cpu().double() - final["a"]).abs().max() < 2e-5 * final["a"].abs().max()
    assert (state[0].cpu().double() - final["b"]).abs().max() < 2e-5 * final["b"].abs().max()
    # a new sequence in a used slot starts from nothing, and one long run equals the portions
    whole = _run_lightning(proj, (nk, nv), dec, state, [[("b", 0, lens["b"], 2), ("a", 0, lens["a"], 1)]], H, d, dv)
    for s in lens:
        assert (whole[s] - outs[s]).abs().max() < 2e-5 * outs[s].abs().max()
    assert (state[1].cpu().double() - final["a"]).abs().max() < 2e-5 * final["a"].abs().max()


@pytest.mark.parametrize("E,top,groups,keep", [(8, 2, 4, 3), (6, 2, 3, 2), (5, 1, 1, 1), (12, 4, 4, 2), (4, 2, 4, 3), (16, 6, 2, 1),
                                               (9, 9, 3, 3), (64, 8, 8, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_group_router(E, top, groups, keep, dtype):
    """Selection biases large enough to change the choice and to make choice scores negative; the weights come
    from the scores without them."""
    g = torch.Generator().manual_seed(E * 10 + top)
    rows, width = 50, 36
    h = torch.randn(rows, width + 4, generator=g).to(dtype)[:, 4:]
    router = torch.randn(E, width, generator=g) * 0.5
    correction = torch.randn(E, generator=g) * 0.6 - 0.5
    spec = {"experts": E, "top": top, "scale": 1.7, "groups": {"count": groups, "keep": keep}}
    for corr in (correction, None):
        logits = torch.matmul(h.to(DEV).float(), router.to(DEV).t())
        chosen, weights = ops().group_router(logits, None if corr is None else corr.to(DEV), top, groups, keep, 1.7)
        w = {"router": router.double()}
        if corr is not None:
            w["correction"] = corr.double()
        changed = 0
        for t in range(rows):
            want_e, want_w = oracle.route(h[t].double(), w, spec)
            got = dict(zip(chosen[t].tolist(), weights[t].tolist()))
            assert sorted(got) == sorted(want_e), (t, got, want_e)
            for e, x in zip(want_e, want_w):
                assert abs(got[e] - float(x)) < 1e-5
            plain_e, _ = oracle.route(h[t].double(), {"router": router.double()}, {"experts": E, "top": top})
            changed += sorted(plain_e) != sorted(want_e)
        if corr is not None and top < E:
            assert changed > 0                                       # the test would not notice a missing bias or limit


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,ff,shared,groups,keep,width", [(6, 2, 24, 40, 3, 2, 48), (3, 1, 70, None, 1, 1, 24), (8, 3, 16, 8, 2, 1, 20),
                                                             (5, 5, 33, 65, 1, 1, 40)])
def test_group_routed_experts(E, top, ff, shared, groups, keep, width, dtype):
    from splitwise_amd.model_executor.layers.moe import GroupRoutedExperts
    g = torch.Generator().manual_seed(E + ff)
    layer = GroupRoutedExperts(width, E, top, ff, shared, groups, keep, 1.4, dtype).to(DEV)
    rows = 90                                                         # more than a tile of rows for some expert
    mlp = lu.moe(E, top, ff, shared, groups if groups > 1 else None, keep, 1.4)
    cfg = lu.config([lu.lightning()], [mlp], width=width)
    sd = lu.random_weights(cfg, 5)
    w = {k[len("l0.mlp."):]: v for k, v in sd.items() if k.startswith("l0.mlp.")}
    layer.load_named({k: (v if k in ("router", "correction") else v.to(dtype)).to(DEV) for k, v in w.items()})
    h = torch.randn(rows, width, generator=g).to(dtype)
    shared_out, routed = layer(h.to(DEV))
    got = routed.cpu().double() + (shared_out.cpu().double() if shared_out is not None else 0.0)
    want = oracle.moe_ff(h.double(), {k: v.double() for k, v in w.items()}, mlp)
    # bf16: the hidden layer is rounded once and squared; errors are judged against the outputs' size
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert (got - want).abs().max() < tol * want.abs().max()


# --------------------------------------------------------------- whole models through the engine
def _cfg_a():
    sc = {"factor": 3.0, "low": 2.0, "high": 5.0, "original": 40}
    layers = [lu.attention(4, 2, 16, 32, rot_dims=8, scaling=sc), lu.lightning(3, 24, 16, (0.5, 0.9, 0.99)),
              lu.attention(4, 2, 16, 32, rot_dims=8, scaling=sc, kv_from=0), lu.lightning(2, 40, 8, (0.97, 0.3)),
              lu.attention(4, 2, 16, 32, rot_dims=8, scaling=sc, kv_from=0)]
    mlps = [lu.dense(40, 0.8), lu.moe(6, 2, 24, 40, 3, 2), lu.dense(24, 2.5), lu.moe(5, 1, 16, None, None), None]
    return lu.config(layers, mlps, vocab=97, width=48)


def _cfg_b():
    layers = [lu.lightning(1, 8, 8, (0.999,)), lu.attention(3, 3, 8, 8, scale=0.5, softcap=3.0, rot_dims=8),
              lu.attention(6, 2, 20, 24, scale=0.2, softcap=30.0, rot_dims=4, base=1000.0), lu.lightning(2, 36, 20, (0.8, 0.9)),
              lu.attention(3, 3, 8, 8, scale=0.5, softcap=3.0, rot_dims=8, kv_from=1)]
    mlps = [lu.moe(4, 3, 16, None, 4, 3, scale=1.0), None, lu.moe(8, 3, 12, 8, 2, 1), lu.dense(30, 1.5), lu.dense(8, 0.3)]
    return lu.config(layers, mlps, vocab=53, width=20, eps=1e-6)


_CASES = {"a": (_cfg_a, 11), "b": (_cfg_b, 12)}
FP32_TOL = 2e-4


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (make, seed) in _CASES.items():
        cfg = make()
        sd = lu.random_weights(cfg, seed)
        path = lu.write_model(str(tmp_path_factory.mktemp("lapilorn_" + name)), cfg, sd)
        g = torch.Generator().manual_seed(seed)
        reqs = {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
                for i, n in enumerate([70, 41, 18, 1, 33, 52, 150])}
        want = {rid: oracle.logits(cfg, sd, toks, dtype=F64) for rid, toks in reqs.items()}
        out[name] = SimpleNamespace(cfg=cfg, sd=sd, path=path, reqs=reqs, want=want)
    return out


@pytest.fixture(scope="module")
def engines(models):
    cache = {}

    def get(name, dtype, **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in cache:
            cache[key] = lu.make_engine(models[name].path, dtype, **kw)
        return cache[key]
    return get


@pytest.mark.parametrize("name", ["a", "b"])
def test_residual_stream_after_every_layer(models, engines, name):
    m = models[name]
    engine = engines(name, "float32")
    model = engine.model_executor.driver_worker.model_runner.model
    toks = m.reqs["r4"]
    want = []
    oracle.logits(m.cfg, m.sd, toks, residuals=want, dtype=F64)
    model.keep_residuals = []
    try:
        lu.Replayer(engine, {"r4": toks}).run_alone("r4", [len(toks)])
        got = [r.cpu().double() for r in model.keep_residuals]
    finally:
        model.keep_residuals = None
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a - b).abs().max() < 1e-4 * b.abs().max(), f"layer {i} ({m.cfg['layers'][i]['type']})"


@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompts_match_the_plain_statement(models, engines, name):
    m = models[name]
    for rid, toks in m.reqs.items():
        got = lu.Replayer(engines(name, "float32"), {rid: toks}).run_alone(rid, [len(toks)])
        assert lu.row_error(got, m.want[rid]) < FP32_TOL, rid


@pytest.mark.parametrize("name", ["a", "b"])
def test_decoding_token_by_token(models, engines, name):
    """Most of a prompt at once and then 45 (and 100) tokens one by one, and a sequence fed one token at a time
    from its very first."""
    m = models[name]
    for rid, first in (("r0", 25), ("r6", 50)):
        toks = m.reqs[rid]
        got = lu.Replayer(engines(name, "float32"), {rid: toks}).run_alone(rid, [first] + [1] * (len(toks) - first))
        assert lu.row_error(got, m.want[rid]) < FP32_TOL
    toks = m.reqs["r2"]
    got = lu.Replayer(engines(name, "float32"), {"r2": toks}).run_alone("r2", [1] * len(toks))
    assert lu.row_error(got, m.want["r2"]) < FP32_TOL


@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("portions", [[2] * 35, [3, 2, 16, 1, 2, 7, 17, 2, 2, 18], [15, 1, 16, 17, 2, 19], [33, 31, 2, 4]])
def test_portions_of_prompts(models, engines, name, portions):
    m = models[name]
    toks = m.reqs["r0"]
    assert sum(portions) == len(toks)
    got = lu.Replayer(engines(name, "float32"), {"r0": toks}).run_alone("r0", portions)
    assert lu.row_error(got, m.want["r0"]) < FP32_TOL


@pytest.mark.parametrize("name,dtype,tol", [("a", "float32", FP32_TOL), ("b", "float32", FP32_TOL), ("a", "bfloat16", 0.08)])
def test_mixed_batches_reuse_pages_and_slots(models, engines, name, dtype, tol):
    """Six unequal requests over three state slots and a pool of 9 pages: portions beside single tokens, requests
    that sit out steps, pages and slots handed on as requests end.  Every request must come out as it does alone."""
    m = models[name]
    reqs = {r: t for r, t in m.reqs.items() if r != "r6"}
    engine = engines(name, dtype, max_tokens=144, max_requests=3)
    rp = lu.Replayer(engine, reqs)
    free_before = engine.scheduler.block_manager.get_num_free_gpu_blocks()
    steps = [{"r0": 3, "r2": 16}, {"r0": 16, "r2": 1, "r3": 1}, {"r0": 2, "r1": 29, "r2": 1}, {"r0": 17, "r1": 2},
             {"r0": 30, "r1": 1}, {"r1": 9, "r0": 1}, {"r0": 1, "r4": 20}]
    for step in steps:
        rp.step(step)
    rnd = random.Random(7)
    pending = ["r5"]
    while any(rp.at[r] < len(reqs[r]) for r in reqs):
        live = [r for r in rp.live if rp.at[r] < len(reqs[r])]
        while pending and len(live) < 3:
            nxt = pending[0]
            need = -(-len(reqs[nxt]) // 16)
            held = sum(-(-len(reqs[r]) // 16) for r in live)
            if held + need > 9:
                break
            live.append(pending.pop(0))
        step = {}
        for r in live:
            left = len(reqs[r]) - rp.at[r]
            step[r] = min(left, rnd.choice([1, 1, 2, 3, 16, 21]))
        if rnd.random() < 0.3 and len(step) > 1:
            step.pop(rnd.choice(sorted(step)))                  # somebody sits this step out
        rp.step(step)
    for rid in reqs:
        assert lu.row_error(rp.result(rid), m.want[rid]) < tol, rid
    assert engine.scheduler.block_manager.get_num_free_gpu_blocks() == free_before
    assert engine.scheduler.state_slots.num_free() == 3


def test_bfloat16_is_close_and_does_not_depend_on_the_cut(models, engines):
    m = models["a"]
    toks = m.reqs["r0"]
    whole = lu.Replayer(engines("a", "bfloat16"), {"r0": toks}).run_alone("r0", [len(toks)])
    cut = lu.Replayer(engines("a", "bfloat16"), {"r0": toks}).run_alone("r0", [2, 3, 16, 1, 1, 30, 17])
    assert lu.row_error(whole, m.want["r0"]) < 0.08
    assert lu.row_error(cut, m.want["r0"]) < 0.08
    assert lu.row_error(cut, whole) < 0.05


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation_through_the_entry_point(models, name):
    """``LLM.generate`` with the scheduler's own policy: a token budget of 16 cuts the prompts into portions that
    run beside other requests' decoded tokens.  Every generated token must be (within rounding) the arg-max of
    the plain statement's logits for the text before it."""
    from splitwise_amd import LLM, SamplingParams
    m = models[name]
    llm = LLM(model=m.path, dtype="float32", block_size=16, max_model_len=128, max_num_seqs=3,
              max_num_batched_tokens=16, num_gpu_blocks_override=20, swap_space=0, enforce_eager=True)
    prompts = [m.reqs["r1"], m.reqs["r2"], m.reqs["r3"], m.reqs["r4"][:20]]
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(temperature=0.0, max_tokens=12,
                                                                                 ignore_eos=True))
    assert len(outs) == len(prompts)
    for prompt, out in zip(prompts, outs):
        new = out.outputs[0].token_ids
        assert len(new) == 12
        full = oracle.logits(m.cfg, m.sd, list(prompt) + list(new), dtype=F64)
        for k, tok in enumerate(new):
            row = full[len(prompt) + k - 1]
            assert row[tok] >= row.max() - 1e-3 * (row.max() - row.min()), (k, tok, int(row.argmax()))
    sched = llm.llm_engine.scheduler
    assert sched.state_slots.num_free() == 3 and not sched.running and not sched.waiting


def test_trace_run_replays_a_schedule(models, tmp_path):
    """``bin/trace_run`` as a user starts it: steps on standard input, ``done <step>`` after each, logits files in
    the order of the entries; requests that sit out a step, end, and hand their pages and slot on."""
    import json
    import os
    import subprocess
    import numpy as np
    m = models["b"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b, c = m.reqs["r1"], m.reqs["r2"], m.reqs["r4"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:7], "want": [0, 6]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [15]}, {"id": "a", "tokens": a[7:8], "want": [0]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[8:], "want": [len(a) - 9]}, {"id": "c", "tokens": c, "want": [0, len(c) - 1]}],
         "end": ["a", "c"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b, "want": [len(b) - 1]}], "end": ["b"]},        # the name comes back
    ]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", m.path, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "128", "--max-requests", "2"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    vocab = m.cfg["vocab"]
    want = {0: [m.want["r1"][0], m.want["r1"][6]], 1: [m.want["r2"][17], m.want["r1"][7]],
            2: [m.want["r1"][len(a) - 1], m.want["r4"][0], m.want["r4"][len(c) - 1]], 3: [m.want["r2"][len(b) - 1]]}
    for step, rows in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, vocab))
        assert got.shape[0] == len(rows)
        assert lu.row_error(got, torch.stack(rows)) < FP32_TOL, step
