"""The Gulidra decoder on the GPU against the plain implementation (tests/plain_gulidra.py): every new kernel alone,
then whole models of several shapes through the step function, the cache manager and the engine."""
import numpy as np
import pytest
import torch

import plain_gulidra as P
from gulidra_helpers import CONFIGS, model_folder, oracle, oracle_logits, tokens_for

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a), dtype=dtype).to(DEV).contiguous()


def bf(a):
    """The values bfloat16 holds of `a`, as float64."""
    return torch.as_tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).double().numpy()


def close(got, want, dtype="float32", what="", rel=0.04):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if dtype == "float32":
        tol = 3e-5 * max(1.0, float(np.abs(want).max()))
        assert float(np.abs(got - want).max()) <= tol, (what, float(np.abs(got - want).max()), tol)
    else:
        rms = float(np.sqrt(np.mean((got - want) ** 2))) / max(1e-9, float(np.sqrt(np.mean(want ** 2))))
        assert rms <= rel, (what, rms)


def make_step(segments, tables, slots):
    """segments: [(pos0, rows)]; a step description on the device through the Python packer."""
    from allpaca_amd.engine.batch import Entry, pack_step
    entries = [Entry(i, [0] * n) for i, (_, n) in enumerate(segments)]
    return pack_step(entries, [p for p, _ in segments], slots, [tables], torch.device(DEV), [0])


# =========================================================================================== kernels alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_with_scale_and_position_vectors(dtype):
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(1)
    V, D, N = 23, 40, 50
    table, pos = bf(rng.normal(size=(V, D))), bf(rng.normal(size=(N, D)))
    step = make_step([(7, 3), (0, 1), (48, 2)], [[0], [0], [0]], [0, 1, 2])
    toks = torch.tensor([5, 22, 0, 5, 9, 1], dtype=torch.int32, device=DEV)
    x = torch.empty((6, D), dtype=torch.float32, device=DEV)
    ops.embed_positions(dev(table, DTYPES[dtype]), toks, dev(pos, DTYPES[dtype]), step.positions, 3.5, x)
    want = np.concatenate([P.embed(table, pos, [5, 22, 0], 7, 3.5), P.embed(table, pos, [5], 0, 3.5),
                           P.embed(table, pos, [9, 1], 48, 3.5)])
    close(x.cpu(), want, "float32", "embedding")


@pytest.mark.parametrize("D", [40, 256, 1030])
def test_normed_residual_sum(D):
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(D)
    x0, y, w = rng.normal(size=(5, D)), 3 * rng.normal(size=(5, D)), 1 + 0.2 * rng.normal(size=D)
    for narrow in (False, True):
        x = dev(x0)
        copy = torch.empty((5, D), dtype=torch.bfloat16, device=DEV) if narrow else None
        ops.rmsnorm_add(dev(y), dev(w), 1e-5, 0.6, x, copy)
        want = np.float32(x0) + 0.6 * P.rms_norm(np.float32(y).astype(np.float64), np.float32(w), 1e-5)
        close(x.cpu(), want, "float32", "sum")
        if narrow:
            assert torch.equal(copy.cpu(), x.cpu().to(torch.bfloat16))


def _linear_attention_case(rng, H, dk, dv, segs, sharp_at=None):
    T = sum(n for _, n in segs)
    q, k, v = (bf(rng.normal(size=(T, H * d))) for d in (dk, dk, dv))
    if sharp_at is not None:           # one early key and one late query far larger than the rest
        k[sharp_at] *= 8.0             # (powers of two: the values stay ones that bfloat16 holds)
        q[-1] *= 4.0
    return q, k, v


@pytest.mark.parametrize("H, dk, dv, decay", [(2, 20, 12, (0.7, 0.97)), (3, 6, 28, (0.5, 0.9, 0.999)),
                                              (2, 64, 64, (0.8, 0.995)), (2, 128, 32, (0.9, 1.0)),
                                              (1, 48, 136, (0.99,))])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_linear_attention_with_decay_and_states_from_earlier_steps(H, dk, dv, decay, dtype):
    """Three requests in one step: one starting, two going on from states that earlier steps left, with 150, 1 and 67
    rows (a chunk of the matrix-core kernel is 64 rows: whole chunks, a last chunk of 22 rows and one of 3), then a
    second step of 1, 2 and 70 more rows from the states the first left."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(H * 100 + dk)
    tdt = DTYPES[dtype]
    slots = [2, 0, 1]
    state0 = rng.normal(size=(4, H, dk, dv)).astype(np.float32)
    state0[2] = 0.0
    state = dev(state0)
    want_state = state0.astype(np.float64)
    width = H * (2 * dk + dv)
    for segs in ([(0, 150), (9, 1), (30, 67)], [(150, 1), (10, 2), (97, 70)]):
        T = sum(n for _, n in segs)
        q, k, v = _linear_attention_case(rng, H, dk, dv, segs, sharp_at=1)
        proj = dev(np.concatenate([q, k, v], axis=1), tdt)
        step = make_step(segs, [[0]] * 3, slots)
        out = torch.empty((T, H * dv), dtype=torch.float32, device=DEV)
        ops.linear_attention(proj, 0, H * dk, 2 * H * dk, H, dk, dv, True, dev(np.float32(decay)), state, step,
                             step.state_slots, out)
        r = 0
        for (_, n), s in zip(segs, slots):
            sl = slice(r, r + n)
            o, want_state[s] = P.decayed_linear_attention(
                bf(P.silu(q[sl])).reshape(n, H, dk) if dtype == "bfloat16" else P.silu(q[sl]).reshape(n, H, dk),
                bf(P.silu(k[sl])).reshape(n, H, dk) if dtype == "bfloat16" else P.silu(k[sl]).reshape(n, H, dk),
                bf(P.silu(v[sl])).reshape(n, H, dv) if dtype == "bfloat16" else P.silu(v[sl]).reshape(n, H, dv),
                np.float32(decay).astype(np.float64), want_state[s])
            # (the kernels keep 16 bits of every float32 operand: far closer than bfloat16 activations would be)
            close(out[sl].cpu(), o.reshape(n, H * dv), dtype, f"rows of slot {s}", rel=2e-3)
            r += n
        for s in slots:
            close(state[s].cpu(), want_state[s], dtype, f"state of slot {s}", rel=2e-3)
    assert np.array_equal(state[3].cpu().numpy(), state0[3])        # a slot no request of the steps holds


def test_gated_norm_over_heads_and_map_combination():
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(5)
    T, H, dv = 5, 3, 20
    o, w, gate = rng.normal(size=(T, H * dv)), 1 + 0.2 * rng.normal(size=H * dv), bf(2 * rng.normal(size=(T, H * dv)))
    for dtype in ("float32", "bfloat16"):
        out = torch.empty((T, H * dv), dtype=DTYPES[dtype], device=DEV)
        ops.gated_rmsnorm(dev(o), dev(w), 1e-5, dev(gate, DTYPES[dtype]), out)
        want = P.rms_norm(np.float32(o).astype(np.float64), np.float32(w), 1e-5) * P.sigmoid(gate)
        close(out.float().cpu(), want, dtype, "gated norm", rel=4e-3)
    a = rng.normal(size=(T, H, 2, dv))
    a[:, :, 1] = a[:, :, 0] + 0.05 * rng.normal(size=(T, H, dv))       # two maps that nearly cancel
    g = bf(2 * rng.normal(size=(T, H)))
    lam, diff = 0.93, 0.3
    for dtype in ("float32", "bfloat16"):
        out = torch.empty((T, H * dv), dtype=DTYPES[dtype], device=DEV)
        ops.diff_combine(dev(a.reshape(T, -1)), lam, 1 - diff, 1e-6, dev(g, DTYPES[dtype]), out, H, dv)
        a32 = np.float32(a).astype(np.float64)
        want = P.unit_rms(a32[:, :, 0] - np.float64(np.float32(lam)) * a32[:, :, 1], 1e-6) * (1 - diff) * P.sigmoid(g)[:, :, None]
        close(out.float().cpu(), want.reshape(T, -1), dtype, "combination", rel=4e-3)


@pytest.mark.parametrize("H, G, dq, dv, P_", [(4, 2, 12, 20, 4), (2, 2, 10, 6, 3), (4, 2, 32, 64, 16), (8, 2, 16, 32, 8),
                                              (2, 1, 64, 128, 16)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_two_maps_a_head_over_pages_with_one_key_that_stands_out(H, G, dq, dv, P_, dtype):
    """Attention with two maps a head (keys of 2 dq side by side in the pages, the same values) on scattered pages:
    a portion of 70 rows that starts at position 200 beside two decoded rows at positions 300 and 64.  Map 1 of the
    last row of the portion and of the first decoded row asks, with a large query, for one key each: far back
    (position 1), at a page's border, and the last one it may see; map 2 stays flat.  Asking for the position after the
    row's own must change nothing."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(H + dq)
    tdt = DTYPES[dtype]
    dk = 2 * dq
    lens = [270, 301, 65]
    segs = [(200, 70), (300, 1), (64, 1)]
    n_pages = sum(-(-L // P_) for L in lens) + 3
    perm = (rng.permutation(n_pages - 1) + 1).tolist()
    tables = []
    for L in lens:
        n = -(-L // P_)
        tables.append(perm[:n])
        perm = perm[n:]
    keys = [bf(rng.normal(size=(L, G, 2, dq))) * 0.5 for L in lens]
    vals = [bf(rng.normal(size=(L, G, dv))) for L in lens]
    targets = (1, (200 // P_) * P_ - 1, (200 // P_) * P_, 269, 270)
    for t_ in targets[:4]:             # the keys that will be asked for, four times as long as the others
        keys[0][t_, 0, 0] *= 4.0
        keys[1][t_, 0, 0] *= 4.0
    pages = np.full((n_pages + 1, G, P_ * (dk + dv)), np.nan, dtype=np.float32)     # what no request wrote is NaN
    for tb, k_, v_ in zip(tables, keys, vals):
        for pos in range(k_.shape[0]):
            page, slot = tb[pos // P_], pos % P_
            pages[page, :, slot * dk:(slot + 1) * dk] = k_[pos].reshape(G, dk)
            pages[page, :, P_ * dk + slot::P_] = v_[pos]
    cache = dev(pages, tdt)
    step = make_step(segs, tables, [0, 1, 2])
    T = 72
    for target in targets:
        q = bf(rng.normal(size=(T, H, 2, dq))) * 0.5
        if target < 270:
            q[69, 0, 0] = bf(keys[0][target, 0, 0] / np.linalg.norm(keys[0][target, 0, 0]) * 8.0)
            q[70, 0, 0] = bf(keys[1][target, 0, 0] / np.linalg.norm(keys[1][target, 0, 0]) * 8.0)
        out = torch.empty((T, H * 2 * dv), dtype=torch.float32, device=DEV)
        ops.masked_attention(dev(q.reshape(T, -1), tdt), out, 2 * H, G, dk, dv, cache, P_, step.block_tables[0], step,
                             "causal", 0, False, 0.8, key_parts=2)
        got = out.cpu().numpy().reshape(T, H, 2, dv)
        r = 0
        for (p0, n), k_, v_ in zip(segs, keys, vals):
            for h in range(H):
                g = h // (H // G)
                for m in range(2):
                    want = P.softmax_attention(q[r:r + n, h, m], k_[:p0 + n, g, m], v_[:p0 + n, g], 0.8)
                    close(got[r:r + n, h, m], want, dtype, f"target {target} head {h} map {m}", rel=0.02)
            r += n
        if target < 270:
            # the planted key carries the row, almost alone
            w = P.softmax_attention(q[69:70, 0, 0], keys[0][:270, 0, 0], np.eye(270), 0.8)[0]
            assert w[target] > 0.5, (target, w[target])
            w = P.softmax_attention(q[70:71, 0, 0], keys[1][:301, 0, 0], np.eye(301), 0.8)[0]
            assert w[target] > 0.5, (target, w[target])


@pytest.mark.parametrize("N, K", [(7, 3), (18, 2), (4, 4), (70, 5), (2, 1)])
def test_router_choice_with_correction(N, K):
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(N)
    T = 33
    z = np.float32(2 * rng.normal(size=(T, N)))
    corr = np.float32(0.3 * rng.normal(size=N))
    ids = torch.empty((T, K), dtype=torch.int32, device=DEV)
    w = torch.empty((T, K), dtype=torch.float32, device=DEV)
    ops.route_topk(dev(z), dev(corr), K, ids, w)
    e = np.exp(z.astype(np.float64) - z.max(axis=1, keepdims=True))
    s = e / e.sum(axis=1, keepdims=True)
    want_ids = np.argsort(-(np.float32(s) + corr), axis=1, kind="stable")[:, :K]
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    close(w.cpu(), np.take_along_axis(s, want_ids, axis=1), "float32", "weights")
    # the correction changes who is chosen, never the weight
    ops.route_topk(dev(z), None, K, ids, w)
    plain_ids = np.argsort(-np.float32(s), axis=1, kind="stable")[:, :K]
    assert np.array_equal(ids.cpu().numpy(), plain_ids) and (N == K or not np.array_equal(plain_ids, want_ids))


@pytest.mark.parametrize("D, F, E, I, K, T", [(36, 20, 5, 2, 3, 19), (128, 64, 8, 1, 2, 150), (64, 32, 3, 0, 3, 40),
                                             (32, 16, 1, 1, 2, 7), (256, 96, 4, 3, 2, 700),
                                             (32, 4096, 4, 0, 4, 5)])      # a row's activations larger than LDS
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_routed_experts_with_identities(D, F, E, I, K, T, dtype):
    """Few rows (tiles of 16 of the matrix-core kernels, most of them nearly empty) and many (tiles of 64), experts that
    nobody chooses, identity experts, every expert chosen."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(D + T)
    tdt = DTYPES[dtype]
    h = bf(rng.normal(size=(T, D)))
    gate, up = bf(rng.normal(size=(E, F, D)) / D ** 0.5), bf(rng.normal(size=(E, F, D)) / D ** 0.5)
    down = bf(rng.normal(size=(E, D, F)) / F ** 0.5)
    pool = [e for e in range(E + I) if not (e == 1 and E + I - 1 >= K and E > 2)]      # expert 1: nobody's choice
    ids = np.stack([rng.permutation(pool)[:K] for _ in range(T)]).astype(np.int32)
    w = np.float32(rng.random(size=(T, K)))
    gu, dn = ops.prepare_experts(dev(np.concatenate([gate, up], axis=1), tdt), dev(down, tdt), tdt)
    y = torch.empty((T, D), dtype=torch.float32, device=DEV)
    ops.routed_experts(dev(h, tdt), gu, dn, E, F, dev(ids, torch.int32), dev(w), K, y)
    want = np.zeros((T, D))
    for t in range(T):
        for e, wt in zip(ids[t], w[t]):
            if e < E:
                a = P.silu(h[t] @ gate[e].T) * (h[t] @ up[e].T)
                want[t] += wt * ((bf(a) if dtype == "bfloat16" else a) @ down[e].T)
            else:
                want[t] += wt * h[t]
    close(y.cpu(), want, dtype, "experts", rel=4e-3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_over_pieces_of_a_head_with_weights(dtype):
    """The convolution kernel's norm over each half of a head of two maps, with weights shared by heads and maps."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(3)
    tdt = DTYPES[dtype]
    for H, G, dq, dv, taps in ((3, 1, 12, 20, 3), (4, 2, 16, 32, 4), (2, 2, 8, 8, 1)):
        dk, P_ = 2 * dq, 8
        width = H * dk + G * (dk + dv)
        segs, slots = [(0, 5), (9, 1), (3, 12)], [2, 0, 1]
        T = 18
        tables = [[1, 2], [3, 4], [5, 6]]
        step = make_step(segs, tables, slots)
        proj = bf(rng.normal(size=(T, width)))
        conv = np.float32(rng.normal(size=(width, taps)))
        qw, kw = np.float32(1 + 0.3 * rng.normal(size=dq)), np.float32(1 + 0.3 * rng.normal(size=dq))
        st0 = np.float32(rng.normal(size=(4, max(taps - 1, 1), width)))
        st0[2] = 0
        state = dev(st0) if taps > 1 else None
        cache = torch.zeros((8, G, P_ * (dk + dv)), dtype=tdt, device=DEV)
        q = torch.empty((T, H * dk), dtype=tdt, device=DEV)
        ops.conv_heads(dev(proj, tdt), 0, H * dk, (H + G) * dk, H, G, dk, dv, None, dev(conv), state, step,
                       step.state_slots if taps > 1 else None, True, 1e-5, q, step.block_tables[0], cache, P_,
                       norm_dim=dq, q_norm_w=dev(qw), k_norm_w=dev(kw))
        r = 0
        for (p0, n), s, tb in zip(segs, slots, tables):
            y = P.short_conv(proj[r:r + n], conv, st0[s][:taps - 1] if taps > 1 else None)
            wq = P.rms_norm(y[:, :H * dk].reshape(n, H, 2, dq), qw, 1e-5).reshape(n, -1)
            close(q[r:r + n].float().cpu(), wq, dtype, "q", rel=6e-3)
            wk = P.rms_norm(y[:, H * dk:(H + G) * dk].reshape(n, G, 2, dq), kw, 1e-5).reshape(n, G, dk)
            for i in range(n):
                pos = p0 + i
                page = cache[tb[pos // P_]].float().cpu().numpy()
                for g in range(G):
                    close(page[g, (pos % P_) * dk:(pos % P_ + 1) * dk], wk[i, g], dtype, "k", rel=6e-3)
            r += n


# =========================================================================================== whole models
def make_runner(name, dtype, page_tokens=4, num_pages=96, max_requests=3, poison=False, use_graphs=False):
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    _, model = load_model(model_folder(name), DTYPES[dtype], DEV)
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


def test_layers_one_by_one_in_32_bit():
    """The residual after every layer against the plain implementation's, for a prompt and for its last token alone."""
    for name in CONFIGS:
        toks = tokens_for(name, 37, 3)
        want = []
        oracle(model_folder(name)).forward(toks, layers_out=want)
        runner = make_runner(name, "float32")
        got = []
        runner.model.layer_tap = lambda i, x: got.append(x.detach().cpu().numpy().copy())
        run_cut(runner, toks, [36, 1])
        n = len(want)
        for i in range(n):
            close(np.concatenate([got[i], got[n + i]]), want[i], "float32", f"{name} layer {i}")


@pytest.mark.parametrize("name", ["GA", "GB", "GC", "GD", "GE"])
@pytest.mark.parametrize("dtype, page_tokens", [("float32", 4), ("bfloat16", 4), ("bfloat16", 16)])
def test_whole_prompts_decoding_and_portions(name, dtype, page_tokens):
    """(Pages of 16 positions: the bfloat16 run's attention on the matrix-core kernels; of 4: on the plain one.)"""
    toks = tokens_for(name, 101, 1)
    want = oracle_logits(model_folder(name), toks)
    runner = make_runner(name, dtype, page_tokens=page_tokens)
    close(run_cut(runner, toks, [101]), want, dtype, "whole")
    close(run_cut(runner, toks, [1]), want, dtype, "token by token")
    close(run_cut(runner, toks, [70, 1]), want, dtype, "prompt, then decoding")
    for cuts in ([2], [3, 2, 7, 1, 5], [6, 13, 2, 2, 66], [65, 1, 1, 2, 19, 3]):
        close(run_cut(runner, toks, cuts), want, dtype, f"portions {cuts}")
    runner.cache.check()


def test_cuttings_agree_to_the_bit_in_32_bit():
    toks = tokens_for("GA", 50, 8)
    runner = make_runner("GA", "float32")
    whole = run_cut(runner, toks, [50])
    for cuts in ([1], [2], [7, 3, 1]):
        assert np.array_equal(whole, run_cut(runner, toks, cuts)), cuts


@pytest.mark.parametrize("name", ["GA", "GB"])
def test_first_tokens_and_page_sizes(name):
    for P_ in (1, 3, 16):
        runner = make_runner(name, "float32", page_tokens=P_, num_pages=80)
        for n in (1, 2, 3, 5):
            toks = tokens_for(name, n, 40 + n)
            close(run_cut(runner, toks, [n]), oracle_logits(model_folder(name), toks), "float32", f"{n} tokens")
            close(run_cut(runner, toks, [1]), oracle_logits(model_folder(name), toks), "float32", f"{n} tokens, singly")


@pytest.mark.parametrize("name, dtype, page_tokens", [("GA", "float32", 4), ("GB", "float32", 4), ("GB", "bfloat16", 16),
                                                     ("GB", "bfloat16", 8), ("GC", "float32", 4), ("GE", "bfloat16", 16)])
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, page_tokens):
    """Five requests of unequal lengths through three slots and a pool that cannot hold them all at once: portions of
    some beside single tokens of others, free pages filled with a huge number.  A slot that comes back carries the
    last request's recurrent state and convolution rows until it is cleared for the next one."""
    from allpaca_amd.engine.batch import Entry
    rng = np.random.default_rng(9)
    lens = [37, 5, 90, 21, 70]
    reqs = {f"r{i}": tokens_for(name, n, 70 + i) for i, n in enumerate(lens)}
    P_ = page_tokens
    total = 50 * 4 // P_
    runner = make_runner(name, dtype, page_tokens=P_, num_pages=total, max_requests=3, poison=True)
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
            n = min(left, int(rng.choice([1, 1, 2, 3, 9, 16, 40])))
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
    assert runner.cache.paged_groups[0].pool.allocations > total          # pages came back and went out again
    for s, toks in reqs.items():
        close(np.concatenate(got[s]), oracle_logits(model_folder(name), toks), dtype, s)
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    """A short prompt, then 280 tokens one by one: the decode attention's passes of 256 keys and many pages go by, and
    the recurrent state is carried through 280 steps."""
    toks = tokens_for("GB", 300, 2)
    close(run_cut(make_runner("GB", dtype, page_tokens=16, num_pages=24), toks, [20, 1]),
          oracle_logits(model_folder("GB"), toks), dtype, "long decoding")


def test_a_position_beyond_the_position_table_is_refused():
    runner = make_runner("GC", "float32", num_pages=64)
    from allpaca_amd.engine.batch import Entry
    runner.admit("s")
    with pytest.raises(Exception, match="position"):
        runner.step([Entry("s", [1] * 129, [128])])


def test_greedy_generation_through_the_engine():
    """Requests of unequal lengths through the engine's scheduler, sampler and decode graphs, in float32: the tokens
    are the plain implementation's."""
    from allpaca_amd.engine import Engine
    from allpaca_amd.sampling import GenerationParams
    for name in ("GA", "GB"):
        folder = model_folder(name)
        prompts = [tokens_for(name, n, 90 + n) for n in (1, 9, 30, 4, 17)]
        for graphs in (True, False):
            engine = Engine(folder, dtype="float32", max_tokens=256, page_tokens=4, max_active_requests=3,
                            chunk_tokens=8, max_batch_tokens=16, use_graphs=graphs)
            outs = engine.generate(prompts, GenerationParams(max_tokens=12, temperature=0.0))
            for p, o in zip(prompts, outs):
                assert o.token_ids == P.greedy(oracle(folder), p, 12), (name, graphs, len(p))


def test_graphs_replay_decode_steps_in_bfloat16():
    """Decode steps recorded as graphs and replayed give the tokens of the same engine without graphs."""
    from allpaca_amd.engine import Engine
    from allpaca_amd.sampling import GenerationParams
    folder = model_folder("GB", "bfloat16")
    prompts = [tokens_for("GB", n, 50 + n) for n in (3, 40, 11)]
    outs = []
    for graphs in (True, False):
        engine = Engine(folder, dtype="bfloat16", max_tokens=512, page_tokens=16, max_active_requests=3,
                        use_graphs=graphs)
        outs.append([o.token_ids for o in engine.generate(prompts, GenerationParams(max_tokens=20, temperature=0.0))])
    assert outs[0] == outs[1]


def test_command_line_and_replay_program(tmp_path):
    """The command line on a model folder of the design (float32, greedy: the plain implementation's tokens), and the
    replay program: three requests through two state slots and a pool that holds two of them."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = model_folder("GA")
    prompts = [tokens_for("GA", 7, 5), tokens_for("GA", 19, 6)]
    spec = ";".join(",".join(str(t) for t in p) for p in prompts)
    cmd = [sys.executable, os.path.join(root, "bin", "allpaca-amd"), "generate", "--model", folder, "--dtype", "fp32",
           "--prompt-tokens", spec, "--max-tokens", "6", "--temperature", "0", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    outs = [json.loads(ln) for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert [o["token_ids"] for o in outs] == [P.greedy(oracle(folder), p, 6) for p in prompts]
    # the design's preset with random weights, sampled with temperature, top-k and top-p in bfloat16
    cmd = [sys.executable, os.path.join(root, "bin", "allpaca-amd"), "generate", "--synthetic", "gulidra-tiny",
           "--prompt-tokens", "1,2,3;4,5", "--max-tokens", "5", "--temperature", "0.8", "--top-k", "20", "--top-p",
           "0.9", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    outs = [json.loads(ln) for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert len(outs) == 2 and all(len(o["token_ids"]) == 5 for o in outs)

    name = "GB"
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
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / f"replay_{dtype}")
        cmd = [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out,
               "--max-tokens", "192", "--max-live", "2", "--poison-free-pages"]
        r = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
                           timeout=280)
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
