"""The Risizen decoder on the GPU against the plain implementation (tests/plain_risizen.py): every new kernel alone,
then whole models of several shapes through the step function, the cache manager and the engine."""
import numpy as np
import pytest
import torch

import plain_risizen as R
from risizen_helpers import CONFIGS, model_folder, oracle, oracle_logits, tokens_for

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a), dtype=dtype).to(DEV).contiguous()


def close(got, want, dtype="float32", what=""):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if dtype == "float32":
        tol = 3e-5 * max(1.0, float(np.abs(want).max()))
        assert float(np.abs(got - want).max()) <= tol, (what, float(np.abs(got - want).max()), tol)
    else:
        # bfloat16 activations: a few parts in a thousand a stored value, over a handful of layers
        rms = float(np.sqrt(np.mean((got - want) ** 2))) / max(1e-9, float(np.sqrt(np.mean(want ** 2))))
        assert rms <= 0.04, (what, rms)


def make_step(segments, page_tokens, tables, slots):
    """segments: [(pos0, rows)]; a step description on the device through the Python packer."""
    from allpaca_amd.engine.batch import Entry, pack_step
    entries = [Entry(i, [0] * n) for i, (_, n) in enumerate(segments)]
    return pack_step(entries, [p for p, _ in segments], slots, [tables], torch.device(DEV), [0])


# =========================================================================================== kernels alone
@pytest.mark.parametrize("taps, H, G, dk, dv", [(4, 3, 1, 24, 16), (2, 2, 2, 8, 40), (1, 2, 1, 16, 16), (0, 2, 1, 16, 24), (3, 2, 0, 72, 0),
                                                 # rows wide enough for the larger blocks of the 16-byte kernel
                                                 (4, 32, 8, 128, 128), (3, 16, 4, 128, 64), (2, 40, 8, 128, 128)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_conv_heads_against_the_plain_convolution_and_norm(taps, H, G, dk, dv, dtype):
    """Three requests in one step: one starting (zeros ahead of it), two going on from states that an earlier step
    left, with 5, 1 and 2 rows (fewer rows than taps: old rows of the state shift down)."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(taps * 7 + H)
    P_, eps = 4, 1e-5
    width = H * dk + G * (dk + dv)
    segs = [(0, 5), (6, 1), (3, 2)]
    slots = [2, 0, 1]
    T = sum(n for _, n in segs)
    tables = [[1, 2], [3, 4], [5, 6]]
    step = make_step(segs, P_, tables, slots)
    tdt = DTYPES[dtype]
    proj = torch.as_tensor(rng.normal(size=(T, width)), dtype=torch.float32).to(tdt)
    bias = rng.normal(size=width).astype(np.float32)
    conv = rng.normal(size=(width, taps)).astype(np.float32) if taps >= 1 else None     # 0: no convolution at all
    taps = max(taps, 1)
    state0 = rng.normal(size=(4, max(taps - 1, 1), width)).astype(np.float32)
    state0[2] = 0.0                                             # the slot of the request that starts
    state = dev(state0[:, :taps - 1]) if taps > 1 else None
    q_out = torch.empty((T, H * dk), dtype=tdt, device=DEV)
    cache = torch.zeros((8, max(G, 1), P_ * (dk + dv)), dtype=tdt, device=DEV) if G else None
    ops.conv_heads(proj.to(DEV), 0, H * dk, (H + G) * dk, H, G, dk, dv, dev(bias), dev(conv) if conv is not None else None,
                   state, step, step.state_slots, True, eps, q_out, step.block_tables[0] if G else None, cache, P_)
    torch.cuda.synchronize()
    u_all = proj.float().numpy().astype(np.float64) + bias
    r0 = 0
    for (pos0, n), slot, table in zip(segs, slots, tables):
        u = u_all[r0:r0 + n]
        before = state0[slot, :taps - 1].astype(np.float64)
        y = R.short_conv(u, conv.astype(np.float64), before) if conv is not None else u
        close(q_out[r0:r0 + n].float().cpu(), R.unit_rms(y[:, :H * dk].reshape(n, H, dk), eps).reshape(n, -1), dtype, "q")
        if taps > 1:
            want_state = np.concatenate([before, u])[-(taps - 1):]
            close(state[slot].cpu(), want_state, "float32", "state")
        for i in range(n):
            pos = pos0 + i
            page = cache[table[pos // P_]].float().cpu().numpy() if G else None
            for g in range(G):
                k = R.unit_rms(y[i, H * dk + g * dk: H * dk + (g + 1) * dk], eps)
                v = y[i, (H + G) * dk + g * dv: (H + G) * dk + (g + 1) * dv]
                close(page[g, (pos % P_) * dk:(pos % P_ + 1) * dk], k, dtype, "k")
                close(page[g, P_ * dk + (pos % P_)::P_][:dv], v, dtype, "v")
        r0 += n


def fill_pages(k, v, P_, table, cache_dtype):
    """Pages [pages, G, P (dk + dv)] holding keys k [T, G, dk] and values v [T, G, dv] at the pages of `table`."""
    T, G, dk = k.shape
    dv = v.shape[2]
    cache = np.full((max(table) + 2, G, P_ * (dk + dv)), 1e30, dtype=np.float32)     # what no row may read is huge
    for t in range(T):
        pg, sl = table[t // P_], t % P_
        cache[pg, :, sl * dk:(sl + 1) * dk] = k[t]
        for g in range(G):
            cache[pg, g, P_ * dk + sl: P_ * (dk + dv): P_] = v[t, g]
    return torch.as_tensor(cache).to(cache_dtype).to(DEV)


@pytest.mark.parametrize("mask, size", [("chunk", 7), ("chunk", 64), ("chunk", 100), ("window", 9), ("causal", 0)])
@pytest.mark.parametrize("sink", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_masked_attention_against_the_plain_one(mask, size, sink, dtype):
    """A prompt portion that starts in the middle of a chunk and of a page beside two decode rows of other requests;
    pages in a scattered order; keys of 24 and values of 40 elements; 6 heads over 2."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(size + sink)
    H, G, dk, dv, P_, scale = 6, 2, 24, 40, 8, 0.4
    lens = [150, 71, 9]                                  # tokens of each request once the step is done
    rows = [83, 1, 1]                                    # rows each brings
    tdt = DTYPES[dtype]
    tables, ks, vs = [], [], []
    free = list(rng.permutation(np.arange(1, 40)))
    for L in lens:
        tables.append([int(free.pop()) for _ in range(-(-L // P_))])
        ks.append(R.unit_rms(rng.normal(size=(L, G, dk)), 1e-6))
        vs.append(rng.normal(size=(L, G, dv)))
    cache = np.full((41, G, P_ * (dk + dv)), 1e30, dtype=np.float32)
    for t_, k, v in zip(tables, ks, vs):
        c = fill_pages(k, v, P_, t_, torch.float32).cpu().numpy()
        for pg in t_:
            cache[pg] = c[pg]
    cache = torch.as_tensor(cache).to(tdt).to(DEV)
    segs = [(L - n, n) for L, n in zip(lens, rows)]
    step = make_step(segs, P_, tables, [0, 1, 2])
    T = sum(rows)
    qs = [R.unit_rms(rng.normal(size=(n, H, dk)), 1e-6) * 1.5 for n in rows]
    q = torch.as_tensor(np.concatenate(qs).reshape(T, H * dk), dtype=torch.float32).to(tdt).to(DEV)
    out = torch.empty((T, H * dv), dtype=tdt, device=DEV)
    if dtype == "bfloat16":       # these sizes are ones the matrix-core kernels take: they must not pass them on
        from allpaca_amd.kernels import tuned
        assert tuned.masked_attention_bf16(q, out, H, G, dk, dv, cache, P_, step.block_tables[0], step, mask, size,
                                           sink, scale)
    else:
        ops.masked_attention(q, out, H, G, dk, dv, cache, P_, step.block_tables[0], step, mask, size, sink, scale)
    want = []
    for k, v, qq in zip(ks, vs, qs):
        if dtype == "bfloat16":
            k, v, qq = (torch.as_tensor(a).to(tdt).double().numpy() for a in (k, v, qq))
        want.append(R.sink_attention(qq, k, v, scale, size if mask == "chunk" else None, sink=sink,
                                     window=size if mask == "window" else None))
    close(out.float().cpu(), np.concatenate(want), dtype, f"{mask} {size}")


@pytest.mark.parametrize("mask, size, pos, key, seen", [
    ("chunk", 80, 79, 0, True), ("chunk", 80, 80, 79, False), ("chunk", 80, 80, 80, True), ("chunk", 80, 159, 80, True),
    ("chunk", 80, 160, 159, False), ("chunk", 500, 499, 3, True), ("window", 33, 400, 368, True),
    ("window", 33, 400, 367, False), ("causal", 0, 900, 0, True), ("causal", 0, 900, 15, True),
    ("causal", 0, 900, 16, True)])
@pytest.mark.parametrize("rows", [1, 70])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_key_stands_out(mask, size, pos, key, seen, rows, dtype):
    """The last row's query points at one key with a large score: if the mask lets the row see it, the output is that
    key's value (a far key among hundreds, at a page's border, just inside a chunk or window); if not, it is not."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(pos + key)
    H, G, dk, dv, P_ = 2, 1, 16, 8, 16
    L = pos + 1
    k = R.unit_rms(rng.normal(size=(L, G, dk)), 1e-6)
    v = rng.normal(size=(L, G, dv))
    v[key] = 100.0 + np.arange(dv)
    table = [int(p) for p in rng.permutation(np.arange(1, -(-L // P_) + 1))]
    tdt = DTYPES[dtype]
    cache = fill_pages(k, v, P_, table, tdt)
    n = min(rows, L)
    step = make_step([(L - n, n)], P_, [table], [0])
    qn = rng.normal(size=(n, H, dk))
    qn[-1, :] = k[key, 0] * 4.0                                 # score 4 * dk * scale = 32 against |others| of about 2
    q = dev(qn.reshape(n, H * dk), tdt)
    out = torch.empty((n, H * dv), dtype=tdt, device=DEV)
    ops.masked_attention(q, out, H, G, dk, dv, cache, P_, step.block_tables[0], step, mask, size, True, 0.5)
    last = out[-1].float().cpu().numpy().reshape(H, dv)
    hit = np.allclose(last, 100.0 + np.arange(dv), atol=0.5 if dtype == "float32" else 1.5)     # (hundreds of other keys keep a sliver)
    assert hit == seen, (last[0, :3], seen)


@pytest.mark.parametrize("S, D", [(1, 40), (2, 192), (3, 1000), (4, 64), (2, 50), (3, 4100), (8, 8192), (12, 64), (16, 30)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_streams_read_write_and_both(S, D, dtype):
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(S * D)
    T, eps = 7, 1e-5
    x0 = rng.normal(size=(T, S, D)).astype(np.float32)
    y = rng.normal(size=(T, D)).astype(np.float32)
    w_in, w_out = rng.normal(size=S).astype(np.float32), rng.normal(size=S).astype(np.float32)
    mix, w_in2 = rng.normal(size=(S, S)).astype(np.float32), rng.normal(size=S).astype(np.float32)
    nw = (1 + 0.1 * rng.normal(size=D)).astype(np.float32)
    tdt = DTYPES[dtype]
    xs = np.moveaxis(x0.astype(np.float64), 1, 0)
    # read
    h = torch.empty((T, D), dtype=tdt, device=DEV)
    x = dev(x0.reshape(T, S * D))
    ops.streams_step(x, S, in_w=dev(w_in), norm_w=dev(nw), eps=eps, h=h)
    close(h.float().cpu(), R.rms_norm(R.hyper_read(xs, w_in), nw, eps), dtype, "read")
    assert torch.equal(x.cpu(), torch.as_tensor(x0.reshape(T, S * D)))
    # read of chosen rows, summing the streams
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    h3 = torch.empty((3, D), dtype=tdt, device=DEV)
    ops.streams_step(x, S, in_w=dev(np.ones(S)), norm_w=dev(nw), eps=eps, h=h3, rows=rows)
    close(h3.float().cpu(), R.rms_norm(xs.sum(0), nw, eps)[[5, 0, 5]], dtype, "rows")
    # write, then write and read at once
    new = R.hyper_write(xs, y.astype(np.float64), mix, w_out)
    ops.streams_step(x, S, y=dev(y), mix=dev(mix), out_w=dev(w_out))
    close(x.cpu().view(T, S, D), np.moveaxis(new, 0, 1), "float32", "write")
    x = dev(x0.reshape(T, S * D))
    ops.streams_step(x, S, y=dev(y), mix=dev(mix), out_w=dev(w_out), in_w=dev(w_in2), norm_w=dev(nw), eps=eps, h=h)
    close(x.cpu().view(T, S, D), np.moveaxis(new, 0, 1), "float32", "write+read x")
    close(h.float().cpu(), R.rms_norm(R.hyper_read(new, w_in2), nw, eps), dtype, "write+read h")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_clamped_glu_and_embedding_into_streams(dtype):
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(3)
    tdt = DTYPES[dtype]
    T, D, F, limit = 5, 24, (50 if dtype == "float32" else 56), 0.8      # (56: the kernel of 16-byte loads)
    h = torch.as_tensor(rng.normal(size=(T, D)), dtype=torch.float32).to(tdt)
    wg = torch.as_tensor(rng.normal(size=(F, D)), dtype=torch.float32).to(tdt)
    wu = torch.as_tensor(rng.normal(size=(F, D)), dtype=torch.float32).to(tdt)
    out = torch.empty((T, F), dtype=tdt, device=DEV)
    ops.clamped_glu(h.to(DEV), torch.cat([wg, wu]).to(DEV), out, 1.702, limit)
    want = R.clamped_glu(h.double().numpy(), wg.double().numpy(), wu.double().numpy(), np.eye(F), limit)
    close(out.float().cpu(), want, dtype, "glu")
    if dtype == "bfloat16":       # the activation alone on gate and up rows kept in 16 bits
        gu = torch.cat([h.float() @ wg.float().T, h.float() @ wu.float().T], dim=1).to(tdt)
        ops.clamped_glu_mul(gu.to(DEV), out, 1.702, limit)
        g, u = gu.double().numpy()[:, :F], gu.double().numpy()[:, F:]
        g, u = np.minimum(g, limit), np.clip(u, -limit, limit)
        close(out.float().cpu(), g / (1 + np.exp(-1.702 * g)) * (u + 1), dtype, "activation")
    assert float(want.max()) > 0.7 * 1.8 * 0.8 and float(np.abs(h.double().numpy() @ wg.double().numpy().T).max()) > limit
    # embedding rows, normalised, into every stream
    V, S = 19, 3
    table = torch.as_tensor(rng.normal(size=(V, D)), dtype=torch.float32).to(tdt)
    nw = (1 + 0.1 * rng.normal(size=D)).astype(np.float32)
    toks = torch.tensor([3, 18, 0, 3], dtype=torch.int32, device=DEV)
    x = torch.empty((4, S * D), dtype=torch.float32, device=DEV)
    ops.embed_streams(table.to(DEV), toks, dev(nw), 1e-6, x, S)
    e = R.rms_norm(table.double().numpy()[[3, 18, 0, 3]], nw, 1e-6)
    for a in range(S):
        close(x.cpu().view(4, S, D)[:, a], e, "float32", "embed")


# =========================================================================================== whole models
def make_runner(name, dtype, page_tokens=4, num_pages=64, max_requests=3, poison=False, use_graphs=False):
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    _, model = load_model(model_folder(name), DTYPES[dtype], DEV, max_positions=512, beyond_configured_positions=False)
    return ModelRunner(model, page_tokens, num_pages, max_requests=max_requests, poison_free_pages=poison,
                       use_graphs=use_graphs)


def run_cut(runner, toks, cuts, seq="s"):
    """All logits of `toks` fed in portions of the sizes `cuts` (the last size repeats)."""
    from allpaca_amd.engine.batch import Entry
    runner.admit(seq)
    out, at, i = [], 0, 0
    while at < len(toks):
        n = min(cuts[min(i, len(cuts) - 1)], len(toks) - at)
        out.append(runner.step([Entry(seq, toks[at:at + n], list(range(n)))]).cpu().numpy())
        at += n
        i += 1
    runner.release(seq)
    return np.concatenate(out)


@pytest.mark.parametrize("name", ["RA", "RB", "RC", "RD"])
@pytest.mark.parametrize("dtype, page_tokens", [("float32", 4), ("bfloat16", 4), ("bfloat16", 16)])
def test_whole_prompts_decoding_and_portions(name, dtype, page_tokens):
    """(Pages of 16 positions: the bfloat16 run's attention on the matrix-core kernels; of 4: on the plain one.)"""
    toks = tokens_for(name, 61, 1)
    want = oracle_logits(model_folder(name), toks)
    runner = make_runner(name, dtype, page_tokens=page_tokens)
    close(run_cut(runner, toks, [61]), want, dtype, "whole")
    close(run_cut(runner, toks, [1]), want, dtype, "token by token")
    close(run_cut(runner, toks, [29, 1]), want, dtype, "prompt, then decoding")
    for cuts in ([2], [3, 2, 7, 1, 5], [6, 13, 2, 2, 30], [17, 1, 1, 2, 19, 3]):
        close(run_cut(runner, toks, cuts), want, dtype, f"portions {cuts}")
    runner.cache.check()


@pytest.mark.parametrize("name", ["RA", "RC"])
def test_first_tokens_and_page_sizes(name):
    for P_ in (1, 3, 16):
        runner = make_runner(name, "float32", page_tokens=P_, num_pages=80)
        for n in (1, 2, 3, 5):
            toks = tokens_for(name, n, 40 + n)
            close(run_cut(runner, toks, [n]), oracle_logits(model_folder(name), toks), "float32", f"{n} tokens")
            close(run_cut(runner, toks, [1]), oracle_logits(model_folder(name), toks), "float32", f"{n} tokens, singly")


@pytest.mark.parametrize("name, dtype, page_tokens", [("RA", "float32", 4), ("RC", "float32", 4), ("RC", "bfloat16", 4),
                                                     ("RC", "bfloat16", 8), ("RB", "float32", 4)])
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, page_tokens):
    """Five requests of unequal lengths through three slots and a pool that cannot hold them all at once: portions of
    some beside single tokens of others, free pages filled with a huge number."""
    from allpaca_amd.engine.batch import Entry
    rng = np.random.default_rng(9)
    lens = [37, 5, 58, 21, 44]
    reqs = {f"r{i}": tokens_for(name, n, 70 + i) for i, n in enumerate(lens)}
    P_ = page_tokens
    runner = make_runner(name, dtype, page_tokens=P_, num_pages=34 * 4 // P_, max_requests=3, poison=True)
    waiting, live, at, got = list(reqs), [], {}, {k: [] for k in reqs}
    while waiting or live:
        while waiting and len(live) < 3 and runner.cache.free_pages(0) >= -(-len(reqs[waiting[0]]) // P_) + 2:
            s = waiting.pop(0)
            runner.admit(s)
            live.append(s)
            at[s] = 0
        entries = []
        for s in live:
            if rng.random() < 0.2 and len(live) > 1:
                continue                                   # left out of this step
            left = len(reqs[s]) - at[s]
            n = min(left, int(rng.choice([1, 1, 2, 3, 9, 16])))
            if runner.cache.pages_needed(s, n)[0] > runner.cache.free_pages(0) - 2 * len(entries):
                n = 1
            entries.append(Entry(s, reqs[s][at[s]:at[s] + n], list(range(n))))
        if not entries:
            continue
        logits = runner.step(entries).cpu().numpy()
        r = 0
        for e in entries:
            n = len(e.tokens)
            got[e.seq].append(logits[r:r + n])
            r += n
            at[e.seq] += n
            if at[e.seq] == len(reqs[e.seq]):
                runner.release(e.seq)
                live.remove(e.seq)
    assert runner.cache.paged_groups[0].pool.allocations > 34 * 4 // P_          # pages came back and went out again
    for s, toks in reqs.items():
        close(np.concatenate(got[s]), oracle_logits(model_folder(name), toks), dtype, s)
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_chunk_edges(dtype):
    """A short prompt, then 150 tokens one by one: the chunks of 48 and 80 positions of RC pass three times and once."""
    toks = tokens_for("RC", 170, 2)
    close(run_cut(make_runner("RC", dtype, page_tokens=16, num_pages=16), toks, [20, 1]),
          oracle_logits(model_folder("RC"), toks), dtype, "long decoding")


def test_greedy_generation_through_the_engine():
    """Requests of unequal lengths through the engine's scheduler, sampler and decode graphs, in float32: the tokens
    are the plain implementation's."""
    from allpaca_amd.engine import Engine
    from allpaca_amd.sampling import GenerationParams
    for name in ("RA", "RC"):
        folder = model_folder(name)
        cfg, w = oracle(folder)
        prompts = [tokens_for(name, n, 90 + n) for n in (1, 9, 30, 4, 17)]
        for graphs in (True, False):
            engine = Engine(folder, dtype="float32", max_tokens=256, page_tokens=4, max_active_requests=3,
                            chunk_tokens=8, max_batch_tokens=16, use_graphs=graphs)
            outs = engine.generate(prompts, GenerationParams(max_tokens=12, temperature=0.0))
            for p, o in zip(prompts, outs):
                assert o.token_ids == R.greedy(cfg, w, p, 12), (name, graphs, len(p))


def test_command_line_generates_with_the_design():
    """The command line on a model folder of the design (float32, greedy: the plain implementation's tokens) and on
    the design's preset with random weights."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = model_folder("RA")
    cfg, w = oracle(folder)
    prompts = [tokens_for("RA", 7, 5), tokens_for("RA", 19, 6)]
    spec = ";".join(",".join(str(t) for t in p) for p in prompts)
    cmd = [sys.executable, os.path.join(root, "bin", "allpaca-amd"), "generate", "--model", folder, "--dtype", "fp32",
           "--prompt-tokens", spec, "--max-tokens", "6", "--temperature", "0", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    outs = [json.loads(ln) for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert [o["token_ids"] for o in outs] == [R.greedy(cfg, w, p, 6) for p in prompts]
    cmd = [sys.executable, os.path.join(root, "bin", "allpaca-amd"), "generate", "--synthetic", "risizen-tiny",
           "--prompt-tokens", "1,2,3;4,5", "--max-tokens", "5", "--temperature", "0", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    outs = [json.loads(ln) for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert len(outs) == 2 and all(len(o["token_ids"]) == 5 for o in outs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_tool_with_two_slots_and_a_small_pool(tmp_path, dtype):
    """The replay program on a model folder of the design: three requests through two state slots and a pool that holds
    two of them, portions beside single tokens, a request left out of a step; its files against the plain logits."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    name = "RC"
    folder = model_folder(name)
    a, b, c = tokens_for(name, 70, 31), tokens_for(name, 9, 32), tokens_for(name, 50, 33)
    steps = [
        dict(step=0, entries=[dict(id="a", tokens=a[:33], want=list(range(33))), dict(id="b", tokens=b[:1], want=[0])], end=[]),
        dict(step=1, entries=[dict(id="b", tokens=b[1:3], want=[0, 1])], end=[]),
        dict(step=2, entries=[dict(id="a", tokens=a[33:69], want=list(range(36))), dict(id="b", tokens=b[3:], want=list(range(6)))],
             end=["b"]),
        dict(step=3, entries=[dict(id="a", tokens=a[69:], want=[0]), dict(id="c", tokens=c[:2], want=[0, 1])], end=["a"]),
        dict(step=4, entries=[dict(id="c", tokens=c[2:], want=list(range(48)))], end=["c"]),
    ]
    out = str(tmp_path / "replay")
    cmd = [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out,
           "--max-tokens", "192", "--max-live", "2", "--poison-free-pages"]
    r = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stderr[-3000:]
    assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == [f"done {i}" for i in range(5)]
    V = CONFIGS[name][0]["vocab"]
    got = {k: [] for k in "abc"}
    for s in steps:
        rows = np.fromfile(os.path.join(out, f"{s['step']}.f32"), dtype="<f4").reshape(-1, V)
        at = 0
        for e in s["entries"]:
            got[e["id"]].append(rows[at:at + len(e["want"])])
            at += len(e["want"])
        assert at == rows.shape[0]
    for k, toks in zip("abc", (a, b, c)):
        close(np.concatenate(got[k]), oracle_logits(folder, toks), dtype, f"replay {k}")
