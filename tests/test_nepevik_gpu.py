"""Nepevik on the GPU against the plain statement in ``oracle/nepevik.py``: every mechanism alone, then whole
models through the engine -- whole prompts, token-by-token decoding, portions down to two tokens, mixed
batches, pages and state slots that are reused, greedy generation through ``LLM.generate``.

The models are small and random (``tests/nepevik_util.py``); where random numbers would hide a fault (a key at a
window's edge among many) the inputs are built so that it shows.
"""
import random
from types import SimpleNamespace

import pytest
import torch

import nepevik_util as nu
from oracle import nepevik as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


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


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [48, 200, 1030])
def test_scalar_norms(dtype, width):
    from splitwise_amd import _C
    torch.manual_seed(width)
    rows = 7
    x = torch.randn(rows, width, device=DEV)
    y = (torch.randn(rows, width, device=DEV) * 3).to(dtype)
    gain = torch.tensor([0.7], device=DEV)
    want = oracle.scalar_norm(y.double(), gain.double(), 1e-5) + x.double()
    res, cast = x.clone(), torch.empty(rows, width, dtype=dtype, device=DEV)
    _C.mixer_ops.scalar_norm_add(res, y, gain, 1e-5, cast)
    torch.testing.assert_close(res.double(), want, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(cast, res.to(dtype))
    out = torch.empty(rows, width, dtype=dtype, device=DEV)
    _C.mixer_ops.scalar_norm(out, res, gain, 1e-5)
    torch.testing.assert_close(out.double(), oracle.scalar_norm(res.double(), gain.double(), 1e-5).to(dtype).double(),
                               atol=1e-2 if dtype == torch.bfloat16 else 1e-5, rtol=1e-2 if dtype == torch.bfloat16 else 1e-5)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_short_conv_in_portions(taps):
    """Two sequences in different slots, cut into portions shorter and longer than the taps, interleaved."""
    from splitwise_amd import _C
    torch.manual_seed(taps)
    channels, lens = 70, {0: 23, 1: 9}
    x = {s: torch.randn(n, channels, device=DEV) for s, n in lens.items()}
    w = torch.randn(channels, taps, device=DEV)
    want = {s: oracle.causal_conv_silu(x[s].double().cpu(), w.double().cpu()) for s in lens}
    state = torch.full((5, max(taps - 1, 0), channels), 7.0, device=DEV)      # stale values of an earlier owner
    slot = {0: 3, 1: 1}
    done = {0: 0, 1: 0}
    got = {s: [] for s in lens}
    plan = [{0: 1}, {0: 2, 1: 1}, {1: 2}, {0: 9, 1: 1}, {0: 1, 1: 5}, {0: 10}]
    for step in plan:
        seqs, xs = [], []
        for s, n in step.items():
            seqs.append((done[s], n, slot[s], []))
            xs.append(x[s][done[s]:done[s] + n])
        xin = torch.cat(xs)
        out = torch.empty(xin.shape, dtype=torch.float32, device=DEV)
        _C.mixer_ops.short_conv(out, xin, w, state, ragged(seqs))
        row = 0
        for s, n in step.items():
            got[s].append(out[row:row + n])
            row += n
            done[s] += n
    for s in lens:
        torch.testing.assert_close(torch.cat(got[s]).double().cpu(), want[s], atol=1e-5, rtol=1e-5)


def _attention_case(H, G, d, dv, window, keep, n, spikes, seed):
    """Inputs for which the mask decides the result: for every (query i, key j) in ``spikes`` the score of j under
    i towers over all others, and key j's value is a large marker."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n, H, d, generator=g) * 0.3
    k = torch.randn(n, G, d, generator=g) * 0.3
    v = torch.randn(n, G, dv, generator=g)
    for i, j in spikes:
        direction = torch.randn(d, generator=g)
        direction /= direction.norm()
        k[j] += 6.0 * direction
        q[i] += 6.0 * direction
        v[j] += 25.0
    return q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)


def _attention_oracle(q, k, v, H, G, d, dv, window, keep, scale, talk, qn, kn, eps):
    width = q.shape[1] + k.shape[1] + v.shape[1]
    h = torch.cat([q, k, v], 1).double()
    eye = torch.eye(width, dtype=torch.float64)
    nq, nk = q.shape[1], k.shape[1]
    w = {"q": eye[:nq], "k": eye[nq:nq + nk], "v": eye[nq + nk:], "q.norm": qn.double(), "k.norm": kn.double(),
         "talk": talk.double(), "o": torch.eye(H * dv, dtype=torch.float64)}
    cfg = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": scale, "mask": {"size": window, "keep_first": keep}}
    return oracle.attention_mixer(h, w, cfg, eps)[0]


@pytest.mark.parametrize("H,G,d,dv,window,keep", [(4, 2, 16, 32, 8, 3), (6, 6, 8, 8, 5, 0), (3, 1, 24, 72, 17, 1),
                                                  (8, 4, 32, 130, 40, 6), (2, 1, 30, 20, 9, 2), (16, 16, 8, 16, 12, 1)])
@pytest.mark.parametrize("mode", ["prompt", "decode", "portions", "decode_split"])
@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
def test_window_attention_edges(H, G, d, dv, window, keep, mode, cache_dtype):
    """Keys just inside and just outside the window, the last kept first token and the one after it, a key far
    back, keys on both sides of a page border -- as a whole prompt, decoded one by one, and in portions; pages
    are scattered over the pool."""
    from splitwise_amd import _C
    page, n = 16, 3 * window + 21
    spikes = []
    for i in (n - 1, n - 2, window + keep + 5, 2 * page, 2 * page + 1):
        if i >= n:
            continue
        spikes += [(i, i - window + 1), (i, i - window)]              # last visible, first hidden
        if keep:
            spikes += [(i, keep - 1)]
        spikes += [(i, keep)] if i - keep >= window else []
    spikes = [(i, j) for i, j in spikes if 0 <= j <= i]
    q, k, v = _attention_case(H, G, d, dv, window, keep, n, spikes, seed=H * 100 + window)
    g = torch.Generator().manual_seed(1)
    talk = torch.eye(H) + 0.5 * torch.randn(H, H, generator=g)
    qn, kn = torch.rand(H * d, generator=g) + 0.5, torch.rand(G * d, generator=g) + 0.5
    scale, eps = 0.9, 1e-5
    want = _attention_oracle(q, k, v, H, G, d, dv, window, keep, scale, talk, qn, kn, eps)

    pages = -(-n // page)
    pool = 3 * pages + 2
    table = random.Random(5).sample(range(pool), pages)
    kc = torch.full((pool, page, G * d), 50.0, device=DEV, dtype=cache_dtype)          # whatever an earlier owner left
    vc = torch.full((pool, page, G * dv), 50.0, device=DEV, dtype=cache_dtype)
    proj = torch.cat([q, k, v], 1).to(DEV).to(cache_dtype)
    if cache_dtype == torch.bfloat16:                  # the statement sees the inputs as the kernels do
        q, k, v = (t.to(torch.bfloat16).float() for t in (q, k, v))
        want = _attention_oracle(q, k, v, H, G, d, dv, window, keep, scale, talk, qn, kn, eps)
    nq, nk = H * d, G * d
    portions = {"prompt": [n], "decode": [n - 12] + [1] * 12, "portions": [2, 3, window, 1, 2, page + 1],
                "decode_split": [n - 12] + [1] * 12}[mode]
    splits = {"decode_split": 3, "portions": 2}.get(mode)              # runs of keys joined by a second launch
    portions = portions + ([n - sum(portions)] if sum(portions) < n else [])
    outs, done = [], 0
    for m in portions:
        rows = proj[done:done + m]
        slots = torch.tensor([table[p // page] * page + p % page for p in range(done, done + m)], device=DEV)
        q32 = torch.empty(m, nq, dtype=torch.float32, device=DEV)
        _C.mixer_ops.qk_norm_cache(q32, rows[:, :nq], rows[:, nq:nq + nk], rows[:, nq + nk:], qn.to(DEV), kn.to(DEV), eps,
                                   kc, vc, slots)
        out = torch.empty(m, H * dv, dtype=cache_dtype, device=DEV)
        _C.mixer_ops.window_attention(out, q32, kc, vc, talk.to(DEV), ragged([(done, m, 0, table)]), H, G, d, dv, scale,
                                      window, keep, splits=splits)
        outs.append(out)
        done += m
    got = torch.cat(outs).double().cpu()
    if cache_dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=2e-4, rtol=2e-4)
    else:
        # the cache holds the normed keys rounded to bf16, which moves scores of this size by a tenth or so and with
        # them the split between two towering keys; a key on the wrong side of an edge would move the result by
        # about the size of its marker (25, times the head mix: a good part of the largest output)
        size = float(want.abs().max())
        assert float((got - want).abs().max()) < 0.03 * size
        assert float((got - want).abs().mean()) < 0.004 * size


def _mixer_portions(mixer, h, state_shapes, plan, lens, slot):
    state = [torch.full((4, *shape), 3.0, device=DEV) for shape in state_shapes]      # stale contents
    md = SimpleNamespace(ragged=None)
    done = {s: 0 for s in lens}
    got = {s: [] for s in lens}
    for step in plan:
        seqs, xs = [], []
        for s, n in step.items():
            seqs.append((done[s], n, slot[s], []))
            xs.append(h[s][done[s]:done[s] + n])
        md.ragged = ragged(seqs)
        out = mixer(torch.cat(xs), state, md)
        row = 0
        for s, n in step.items():
            got[s].append(out[row:row + n])
            row += n
            done[s] += n
    return {s: torch.cat(got[s]).double().cpu() for s in lens}


_PLAN = [{0: 2}, {0: 3, 1: 1}, {1: 2}, {0: 1, 1: 1}, {0: 17, 1: 4}, {0: 1}, {0: 1, 1: 2}, {0: 6}]
_LENS = {0: 31, 1: 10}


@pytest.mark.parametrize("H,G,d,dv,taps", [(4, 2, 16, 32, 4), (2, 2, 8, 16, 2), (3, 1, 40, 20, 3), (2, 1, 72, 130, 4),
                                           (2, 1, 30, 24, 3), (1, 1, 160, 16, 2)])
def test_channel_delta_mixer(H, G, d, dv, taps):
    from splitwise_amd.model_executor.layers.recurrent import ChannelDeltaMixer
    width, eps = 40, 1e-5
    cfg = nu.config([nu.channel_delta(H, G, d, dv, taps)], [None], width=width)
    sd = nu.random_weights(cfg, seed=H * 10 + d)
    w = {k[len("l0.mix."):]: v for k, v in sd.items() if k.startswith("l0.mix.")}
    with torch.device(DEV):
        mixer = ChannelDeltaMixer(width, H, G, d, dv, taps, w["a1"].shape[0], w["g1"].shape[0], eps, torch.float32)
    mixer.load_named({k: v.float().to(DEV) for k, v in w.items()})
    torch.manual_seed(0)
    h = {s: torch.randn(n, width, device=DEV) for s, n in _LENS.items()}
    got = _mixer_portions(mixer, h, mixer.state_shapes(), _PLAN, _LENS, {0: 2, 1: 0})
    for s in _LENS:
        want = oracle.channel_delta_mixer(h[s].double().cpu(), {k: v.double() for k, v in w.items()},
                                          cfg["layers"][0]["mixer"], eps)
        torch.testing.assert_close(got[s], want, atol=3e-4, rtol=3e-4)


@pytest.mark.parametrize("H,d", [(3, 24), (1, 12), (2, 64), (2, 100), (2, 10), (1, 160)])
def test_general_delta_mixer(H, d):
    from splitwise_amd.model_executor.layers.recurrent import GeneralDeltaMixer
    width, eps = 40, 1e-5
    cfg = nu.config([nu.general_delta(H, d)], [None], width=width)
    sd = nu.random_weights(cfg, seed=H * 10 + d)
    w = {k[len("l0.mix."):]: v for k, v in sd.items() if k.startswith("l0.mix.")}
    with torch.device(DEV):
        mixer = GeneralDeltaMixer(width, H, d, w["w1"].shape[0], eps, torch.float32)
    mixer.load_named({k: v.float().to(DEV) for k, v in w.items()})
    torch.manual_seed(0)
    h = {s: torch.randn(n, width, device=DEV) for s, n in _LENS.items()}
    got = _mixer_portions(mixer, h, mixer.state_shapes(), _PLAN, _LENS, {0: 1, 1: 3})
    for s in _LENS:
        want = oracle.general_delta_mixer(h[s].double().cpu(), {k: v.double() for k, v in w.items()},
                                          cfg["layers"][0]["mixer"], eps)
        torch.testing.assert_close(got[s], want, atol=3e-4, rtol=3e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,top,ff,shared", [(5, 2, 24, 40), (3, 1, 70, None), (4, 3, 16, 8), (9, 1, 33, 65),
                                                   (2, 1, 136, None)])
def test_table_routed_experts(experts, top, ff, shared, dtype):
    from splitwise_amd.model_executor.layers.moe import TableRoutedExperts
    width, vocab = 40, 61
    cfg = nu.config([nu.general_delta(1, 8)], [nu.moe(experts, top, ff, shared)], vocab=vocab, width=width)
    sd = nu.random_weights(cfg, seed=experts)
    w = {k[len("l0.mlp."):]: v for k, v in sd.items() if k.startswith("l0.mlp.")}
    with torch.device(DEV):
        mlp = TableRoutedExperts(width, vocab, experts, top, ff, shared, dtype)
    mlp.load_named({k: (v.to(dtype) if v.dtype.is_floating_point else v).to(DEV) for k, v in w.items()})
    g = torch.Generator().manual_seed(3)
    tokens = torch.randint(0, vocab, (177,), generator=g)
    tokens[:90] = tokens[0]                              # one expert gets more than a tile of rows
    h = torch.randn(177, width, generator=g).to(dtype)
    want = oracle.table_moe(h.double(), tokens.tolist(), {k: (v.double() if v.dtype.is_floating_point else v)
                                                          for k, v in w.items()}, cfg["layers"][0]["mlp"])
    got = mlp(h.to(DEV), tokens.to(DEV)).double().cpu()
    tol = 2e-4 if dtype == torch.float32 else 6e-2       # bf16: the hidden activations are rounded once
    torch.testing.assert_close(got, want, atol=tol, rtol=tol)


# --------------------------------------------------------------- whole models through the engine
def _cfg_a():
    layers = [nu.attention(4, 2, 16, 32, window=8, keep_first=3), nu.channel_delta(4, 2, 16, 32, conv=4),
              nu.general_delta(3, 24), nu.attention(4, 2, 16, 32, window=11, keep_first=1, kv_from=0),
              nu.channel_delta(2, 2, 8, 16, conv=2)]
    mlps = [nu.moe(5, 2, 24, 40), None, nu.moe(3, 1, 16, None), nu.moe(5, 2, 24, 40), None]
    return nu.config(layers, mlps, vocab=97, width=48)


def _cfg_b():
    layers = [nu.general_delta(1, 12), nu.attention(2, 2, 8, 8, window=5, keep_first=0), nu.attention(3, 1, 8, 24, 20, 2)]
    mlps = [nu.moe(4, 3, 16, None), nu.moe(2, 1, 8, 8), None]
    return nu.config(layers, mlps, vocab=53, width=24, eps=1e-6)


_CASES = {"a": (_cfg_a, 11), "b": (_cfg_b, 12)}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (make, seed) in _CASES.items():
        cfg = make()
        sd = nu.random_weights(cfg, seed)
        path = nu.write_model(str(tmp_path_factory.mktemp("nepevik_" + name)), cfg, sd)
        g = torch.Generator().manual_seed(seed)
        reqs = {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
                for i, n in enumerate([70, 41, 18, 1, 33, 52])}
        want = {rid: oracle.logits(sd, cfg, toks, torch.float64) for rid, toks in reqs.items()}
        out[name] = SimpleNamespace(cfg=cfg, sd=sd, path=path, reqs=reqs, want=want)
    return out


@pytest.fixture(scope="module")
def engines(models):
    cache = {}

    def get(name, dtype, **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in cache:
            cache[key] = nu.make_engine(models[name].path, dtype, **kw)
        return cache[key]
    return get


FP32_TOL = 2e-4


@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompts_match_the_plain_statement(models, engines, name):
    m = models[name]
    for rid, toks in m.reqs.items():
        got = nu.Replayer(engines(name, "float32"), {rid: toks}).run_alone(rid, [len(toks)])
        assert nu.row_error(got, m.want[rid]) < FP32_TOL, rid


@pytest.mark.parametrize("name", ["a", "b"])
def test_decoding_token_by_token(models, engines, name):
    """Most of a prompt at once, then 45 tokens one by one: every window passes over decoded tokens; and a
    sequence fed one token at a time from its very first."""
    m = models[name]
    toks = m.reqs["r0"]
    got = nu.Replayer(engines(name, "float32"), {"r0": toks}).run_alone("r0", [25] + [1] * 45)
    assert nu.row_error(got, m.want["r0"]) < FP32_TOL
    toks = m.reqs["r2"]
    got = nu.Replayer(engines(name, "float32"), {"r2": toks}).run_alone("r2", [1] * len(toks))
    assert nu.row_error(got, m.want["r2"]) < FP32_TOL


@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("portions", [[2] * 35, [3, 2, 16, 1, 2, 7, 17, 2, 2, 18], [15, 1, 16, 17, 2, 19]])
def test_portions_of_prompts(models, engines, name, portions):
    m = models[name]
    toks = m.reqs["r0"]
    assert sum(portions) == len(toks)
    got = nu.Replayer(engines(name, "float32"), {"r0": toks}).run_alone("r0", portions)
    assert nu.row_error(got, m.want["r0"]) < FP32_TOL


@pytest.mark.parametrize("name,dtype,tol", [("a", "float32", FP32_TOL), ("b", "float32", FP32_TOL), ("a", "bfloat16", 0.08)])
def test_mixed_batches_reuse_pages_and_slots(models, engines, name, dtype, tol):
    """Six unequal requests over three state slots and a pool of 9 pages: portions beside single tokens, requests
    that sit out steps, pages and slots handed on as requests end.  Every request must come out as it does alone."""
    m = models[name]
    engine = engines(name, dtype, max_tokens=144, max_requests=3)
    rp = nu.Replayer(engine, m.reqs)
    free_before = engine.scheduler.block_manager.get_num_free_gpu_blocks()
    steps = [{"r0": 3, "r2": 16}, {"r0": 16, "r2": 1, "r3": 1}, {"r0": 2, "r1": 29, "r2": 1}, {"r0": 17, "r1": 2},
             {"r0": 30, "r1": 1}, {"r1": 9, "r0": 1}, {"r0": 1, "r4": 20}]
    for step in steps:
        rp.step(step)
    # the rest goes in rounds of uneven portions; the last request joins when its pages fit
    rnd = random.Random(7)
    pending = ["r5"]
    while any(rp.at[r] < len(m.reqs[r]) for r in m.reqs):
        live = [r for r in rp.live if rp.at[r] < len(m.reqs[r])]
        while pending and len(live) < 3:
            nxt = pending[0]
            need = -(-len(m.reqs[nxt]) // 16)
            held = sum(-(-len(m.reqs[r]) // 16) for r in live)
            if held + need > 9:
                break
            live.append(pending.pop(0))
        step = {}
        for r in live:
            left = len(m.reqs[r]) - rp.at[r]
            step[r] = min(left, rnd.choice([1, 1, 2, 3, 16, 21]))
        if rnd.random() < 0.3 and len(step) > 1:
            step.pop(rnd.choice(sorted(step)))                  # somebody sits this step out
        rp.step(step)
    for rid in m.reqs:
        assert nu.row_error(rp.result(rid), m.want[rid]) < tol, rid
    assert engine.scheduler.block_manager.get_num_free_gpu_blocks() == free_before
    assert engine.scheduler.state_slots.num_free() == 3


def test_bfloat16_is_close_and_does_not_depend_on_the_cut(models, engines):
    m = models["a"]
    toks = m.reqs["r0"]
    whole = nu.Replayer(engines("a", "bfloat16"), {"r0": toks}).run_alone("r0", [len(toks)])
    cut = nu.Replayer(engines("a", "bfloat16"), {"r0": toks}).run_alone("r0", [2, 3, 16, 1, 1, 30, 17])
    assert nu.row_error(whole, m.want["r0"]) < 0.08
    assert nu.row_error(cut, m.want["r0"]) < 0.08
    assert nu.row_error(cut, whole) < 0.05


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
        full = oracle.logits(m.sd, m.cfg, list(prompt) + list(new), torch.float64)
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
        assert nu.row_error(got, torch.stack(rows)) < FP32_TOL, step
