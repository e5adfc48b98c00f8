"""Zinesun (models/zinesun.py) against the plain float64 implementation in tests/zinesun_oracle.py:
every mechanism alone, then whole models through the engine: prefill vs token-by-token decoding,
prompt portions of many sizes, mixed batches of unequal requests, pages and state slots that are
freed and used again, window and page edges, the first tokens, long decoding, greedy generation
through the scheduler. Each case runs on the CPU reference ops (f32) and, marked gpu, on the HIP
kernels in f32 and bf16. Configurations and weights are made here; nothing is read from disk but
what a test wrote itself."""
import json
import math

import pytest
import torch
from safetensors.torch import save_file

from butterfly_amd import ops
from butterfly_amd.ckpt import load_into, model_config
from butterfly_amd.config import EngineConfig
from butterfly_amd.engine.engine import LLMEngine
from butterfly_amd.engine.sampler import SamplingParams
from butterfly_amd.models import build_model

from . import zinesun_oracle as O

gpu = pytest.mark.gpu
TARGETS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
           pytest.param(("cuda", torch.float32), id="gpu-f32", marks=gpu),
           pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=gpu)]
F64 = torch.float64


@pytest.fixture(params=TARGETS)
def target(request):
    dev, dt = request.param
    if dev == "cuda":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        ops.require_library()
    return torch.device(dev), dt


def rel_err(got, want):
    """Per-row error as a logit comparison sees it: mean removed, RMS over the last dim, relative
    to the RMS of the expected row."""
    got, want = got.detach().cpu().to(F64), want.to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / (w.pow(2).mean(-1).sqrt() + 1e-9)


def assert_rows(got, want, dt, what=""):
    e = rel_err(got, want).flatten()
    if dt == torch.float32:
        assert e.max() < 3e-4, f"{what}: worst row {int(e.argmax())} err {e.max():.3g}"
    else:
        # bf16 rounding in models this narrow is a few percent per row, and a near-tie in a router
        # can move single rows far; the f32 runs carry the exact comparison, this one checks that
        # the bf16 kernels compute the same thing: the bulk must agree
        assert e.median() < 0.05 and e.quantile(0.9) < 0.15, \
            f"{what}: median {e.median():.3g}, 90th percentile {e.quantile(0.9):.3g}"


def bf(t):
    """bf16-representable f64 values (every tensor a bf16 run sees exactly)."""
    return t.to(torch.bfloat16).to(F64)


def close(got, want, dt, f32_tol=2e-5, bf16_tol=2e-2):
    want = want.to(F64)
    err = (got.detach().cpu().to(F64) - want).abs().max()
    return err < (f32_tol if dt == torch.float32 else bf16_tol) * (1 + want.abs().max())


def i32(v, dev):
    return torch.tensor(v, dtype=torch.int32, device=dev)


# ---------------------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------------------
def test_scaled_embedding(target):
    dev, dt = target
    g = torch.Generator().manual_seed(1)
    table = bf(torch.randn(37, 24, generator=g, dtype=F64))
    ids = [5, 0, 36, 5, 17]
    got = ops.embed_scaled(i32(ids, dev), table.to(dev, dt), 3.25)
    assert got.dtype == torch.float32 and close(got, O.scaled_embedding(table, ids, 3.25), torch.float32)


@pytest.mark.parametrize("taps", [1, 2, 3, 5, 9])
def test_input_convolution_over_steps_and_slots(target, taps):
    """Three sequences fed in portions (one token, two tokens, longer than the kernel, shorter
    than it), interleaved in packed steps, through two history slots of which one is handed from a
    finished sequence to a new one. Every step's rows equal the convolution of the whole sequence."""
    dev, dt = target
    g = torch.Generator().manual_seed(taps)
    C = 70
    w = bf(0.5 * torch.randn(C, taps, generator=g, dtype=F64))
    seqs = {n: torch.randn(L, C, generator=g, dtype=F64).float().to(F64) for n, L in (("a", 19), ("b", 9), ("c", 6))}
    want = {n: O.causal_conv_residual(x, w) for n, x in seqs.items()}
    state = torch.full((2, max(taps - 1, 0), C), 7.0, dtype=torch.float32, device=dev)     # stale values
    slot = {"a": 0, "b": 1, "c": 1}
    steps = [[("a", 1), ("b", 2)], [("b", 1), ("a", 2)], [("a", 7), ("b", 6)], [("a", 1)], [("c", 1), ("a", 2)],
             [("a", 6), ("c", 5)]]
    at = {n: 0 for n in seqs}
    for step in steps:
        rows, cu, pos, sl = [], [0], [], []
        for n, c in step:
            rows.append(seqs[n][at[n]:at[n] + c])
            pos += list(range(at[n], at[n] + c))
            cu.append(cu[-1] + c)
            sl.append(slot[n])
        x = torch.cat(rows).to(dev, torch.float32)
        args = (state if taps > 1 else None, i32(sl, dev) if taps > 1 else None, i32(cu, dev), i32(pos, dev))
        h = ops.conv_mix(x, w.to(dev, torch.float32), *args, dt)
        if taps > 1:
            ops.conv_state_update_(x, state, i32(sl, dev), i32(cu, dev), i32(pos, dev))
        assert h.dtype == dt
        r = 0
        for n, c in step:
            assert close(h[r:r + c], want[n][at[n]:at[n] + c], dt, bf16_tol=1e-2), (taps, n, at[n], c)
            at[n] += c
            r += c
    assert all(at[n] == len(seqs[n]) for n in seqs)


@pytest.mark.parametrize("taps,C", [(4, 64), (3, 50), (8, 24)])
def test_input_convolution_long_steps(target, taps, C):
    """Steps of more than a thousand rows (several rows per workgroup slide over sequence starts,
    one-row sequences and an empty one), continued from a first step's history."""
    dev, dt = target
    g = torch.Generator().manual_seed(taps + C)
    w = bf(0.5 * torch.randn(C, taps, generator=g, dtype=F64))
    lens = {"a": 1500, "b": 3, "c": 1, "d": 900}
    seqs = {n: torch.randn(L, C, generator=g, dtype=F64).float().to(F64) for n, L in lens.items()}
    want = {n: O.causal_conv_residual(x, w) for n, x in seqs.items()}
    state = torch.full((4, taps - 1, C), -3.0, dtype=torch.float32, device=dev)
    slot = {"a": 2, "b": 0, "c": 3, "d": 1}
    at = {n: 0 for n in seqs}
    for step in ([("a", 2), ("d", 1)], [("b", 3), ("a", 1098), ("c", 1), ("d", 0), ("d", 899)], [("a", 400)]):
        rows, cu, pos, sl = [], [0], [], []
        for n, c in step:
            rows.append(seqs[n][at[n]:at[n] + c])
            pos += list(range(at[n], at[n] + c))
            cu.append(cu[-1] + c)
            sl.append(slot[n])
        x = torch.cat(rows).to(dev, torch.float32)
        h = ops.conv_mix(x, w.to(dev, torch.float32), state, i32(sl, dev), i32(cu, dev), i32(pos, dev), dt)
        ops.conv_state_update_(x, state, i32(sl, dev), i32(cu, dev), i32(pos, dev))
        r = 0
        for n, c in step:
            assert c == 0 or close(h[r:r + c], want[n][at[n]:at[n] + c], dt, bf16_tol=1e-2), (n, at[n], c)
            at[n] += c
            r += c


def test_convolution_leaves_padding_sequences_alone(target):
    """A fixed-shape decode step pads with sequences that have no slot: their rows pass through and
    no history is written."""
    dev, dt = target
    x = torch.arange(12, dtype=torch.float32).view(3, 4).to(dev)
    w = torch.ones(4, 3, dtype=torch.float32, device=dev)
    state = torch.full((1, 2, 4), 5.0, dtype=torch.float32, device=dev)
    sl, cu, pos = i32([0, -1, -1], dev), i32([0, 1, 2, 3], dev), i32([4, 0, 0], dev)
    h = ops.conv_mix(x, w, state, sl, cu, pos, torch.float32)
    ops.conv_state_update_(x, state, sl, cu, pos)
    assert torch.equal(h[0].cpu(), x[0].cpu() * 2 + 10) and torch.equal(h[1:].cpu(), 2 * x[1:].cpu())
    assert torch.equal(state[0, 1].cpu(), x[0].cpu()) and torch.equal(state[0, 0].cpu(), torch.full((4,), 5.0))


@pytest.mark.parametrize("T,C", [(1, 8), (7, 50), (33, 256)])
def test_post_norm_residual_and_depth_average(target, T, C):
    dev, dt = target
    g = torch.Generator().manual_seed(T + C)
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=F64)        # noqa: E731
    x, y = rnd(T, C).float().to(F64) * 5, bf(rnd(T, C) * 3 + 1)
    nw, nb, ls = bf(1 + 0.3 * rnd(C)), bf(0.3 * rnd(C)), bf(0.5 + 0.2 * rnd(C))
    eps = 1e-4
    f32 = lambda t: t.to(dev, torch.float32)        # noqa: E731
    want = x + ls * O.layer_norm(y, nw, nb, eps)
    out = torch.empty(T, C, dtype=torch.float32, device=dev)
    cast = ops.post_norm_add(f32(x), y.to(dev, dt), f32(nw), f32(nb), eps, f32(ls), out=out, cast_dtype=dt)
    assert close(out, want, torch.float32) and cast.dtype == dt and close(cast, want, dt, bf16_tol=1e-2)
    xin = f32(x)
    assert ops.post_norm_add(xin, y.to(dev, dt), f32(nw), f32(nb), eps, f32(ls), out=xin) is None      # in place
    assert close(xin, want, torch.float32)
    # the fused update + average over four earlier results, then the average alone (no sublayer)
    stack = torch.zeros(6, T, C, dtype=torch.float32, device=dev)
    prev = [rnd(T, C).float().to(F64) for _ in range(4)]
    for j, t in enumerate(prev):
        stack[j] = f32(t)
    avg = bf(rnd(5))
    xx = f32(x)
    ops.post_norm_add_avg(xx, y.to(dev, dt), f32(nw), f32(nb), eps, f32(ls), stack, 4, f32(avg))
    assert close(stack[4], want, torch.float32)
    assert close(xx, O.depth_average(prev + [want], avg), torch.float32)
    avg2 = bf(rnd(6))
    x2 = rnd(T, C).float().to(F64)
    xx = f32(x2)
    ops.post_norm_add_avg(xx, None, None, None, eps, None, stack, 5, f32(avg2))
    assert close(stack[5], x2, torch.float32) and close(xx, O.depth_average(prev + [want, x2], avg2), torch.float32)


@pytest.mark.parametrize("M,N,K", [(5, 7, 13), (70, 130, 50), (3, 256, 128), (600, 384, 192), (260, 256, 64), (16, 128, 64)])
def test_xielu_projection(target, M, N, K):
    dev, dt = target
    g = torch.Generator().manual_seed(M + N)
    x, w = bf(torch.randn(M, K, generator=g, dtype=F64)), bf(torch.randn(N, K, generator=g, dtype=F64) / math.sqrt(K) * 2)
    p, q = 0.4, -0.7
    want = O.xielu(x @ w.T, p, q)
    got = ops.linear_act(x.to(dev, dt), w.to(dev, dt), act="xielu", act_params=(O.softplus(p), 0.5 + O.softplus(q)))
    assert got.dtype == dt and close(got, want, dt, f32_tol=1e-4, bf16_tol=3e-2)


@pytest.mark.parametrize("T,H,K,N", [(1, 3, 12, 24), (9, 5, 20, 7), (130, 2, 64, 96), (600, 4, 32, 64)])
def test_per_head_projection_on_views(target, T, H, K, N):
    dev, dt = target
    g = torch.Generator().manual_seed(T + H)
    wide = bf(torch.randn(T, H, K + 5, generator=g, dtype=F64))
    w = bf(torch.randn(H, N, K, generator=g, dtype=F64) / math.sqrt(K))
    xin = wide.to(dev, dt)
    out = torch.full((T, H, N + 3), 9.0, dtype=dt, device=dev)
    ops.linear_heads(xin[:, :, :K], w.to(dev, dt), out[:, :, :N])
    want = torch.einsum("thk,hnk->thn", wide[:, :, :K], w)
    assert close(out[:, :, :N], want, dt, f32_tol=1e-4) and bool((out[:, :, N:] == 9.0).all())


def test_rotated_copy_of_head_slices(target):
    dev, dt = target
    g = torch.Generator().manual_seed(4)
    T, H, D, n, nd = 6, 3, 10, 8, 13
    src = bf(torch.randn(T, H, D + n, generator=g, dtype=F64))
    pos = [0, 1, 2, 77, 1000, 31]
    base, dims = 50.0, 6                      # three rotated pairs, one pair passes unchanged
    inv = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float32)
    dst = torch.full((T, H, 4 + nd), 3.0, dtype=dt, device=dev)
    s = src.to(dev, dt)
    ops.rope_heads_copy(s[:, :, D:], dst[:, :, 4:], i32(pos, dev), inv.to(dev))
    want = torch.stack([O.rotate_pairs(src[t, :, D:], pos[t], base, dims) for t in range(T)])
    assert close(dst[:, :, 4:4 + n], want, dt, bf16_tol=1e-2)
    assert bool((dst[:, :, 4 + n:] == 0).all()) and bool((dst[:, :, :4] == 3.0).all())


def paged(seq_rows, width_k, width_v, bs, dev, dt, order):
    """Lay per-sequence key rows [L, >= width] and value rows out in shuffled pages."""
    nblk = sum((len(k) + bs - 1) // bs for k, _ in seq_rows) + 1
    kc = torch.zeros(nblk, 1, bs, width_k, dtype=dt, device=dev)
    vc = torch.zeros(nblk, 1, width_v, bs, dtype=dt, device=dev)
    free = list(order(nblk))
    tables = []
    for k, v in seq_rows:
        tab = []
        for b0 in range(0, len(k), bs):
            blk = free.pop()
            tab.append(blk)
            n = min(bs, len(k) - b0)
            kc[blk, 0, :n, :k.shape[1]] = k[b0:b0 + n].to(dev, dt)
            vc[blk, 0, :v.shape[1], :n] = v[b0:b0 + n].T.to(dev, dt)
        tables.append(tab)
    mb = max(len(t) for t in tables)
    return kc, vc, i32([t + [0] * (mb - len(t)) for t in tables], dev)


@pytest.mark.parametrize("H,D,Dv,window", [(3, 20, 12, 9), (5, 96, 64, 33), (16, 128, 96, 40), (2, 32, 32, 1),
                                          (4, 64, 64, 500), (16, 96, 64, 33), (32, 64, 32, 9), (16, 256, 192, 100),
                                          (24, 192, 128, 64), (16, 256, 256, 77)])
def test_shared_head_attention_edges(target, H, D, Dv, window):
    """Folded multi-query attention over one shared cached head, no sink, with an output gate. A
    long prompt chunk, a short chunk and decoded rows in one packed step. For chosen rows one key
    is made to stand out: the key just inside the window, just outside it, at a page border, and
    far back; a window off by one token or a lost page moves the output by the whole value."""
    dev, dt = target
    bs = 32
    g = torch.Generator().manual_seed(H * D + window)
    rnd = lambda *s: bf(torch.randn(*s, generator=g, dtype=F64))        # noqa: E731
    lens = [150, 70, 97, 33]                     # cached tokens per sequence after this step
    rows = [(0, 150), (60, 70), (96, 97), (32, 33)]      # (first new position, end): whole, portion, two decoded rows
    seqs = [(0.3 * rnd(L, D), rnd(L, Dv)) for L in lens]
    q, pos, cu = [], [], [0]
    for s, (a, b) in enumerate(rows):
        qs = 0.3 * rnd(b - a, H, D)
        for i in range(a, b):           # aim row i, head i % H, at one key
            for j in {i - window + 1, i - window, (i // bs) * bs, (i // bs) * bs - 1, max(0, i - 140)}:
                if 0 <= j <= i and (i + j) % 3 == 0:
                    u = rnd(D)
                    u = u / u.norm()
                    seqs[s][0][j] = bf(4.0 * u)
                    qs[i - a, i % H] = bf(6.0 * u)
        q.append(qs)
        pos += list(range(a, b))
        cu.append(cu[-1] + (b - a))
    q = torch.cat(q)
    T = q.shape[0]
    gate = torch.rand(T, H, generator=g, dtype=F64).float().to(F64)
    scale = 0.9
    kc, vc, tables = paged(seqs, ops.attn_window_pad(D, dt), ops.attn_window_pad(Dv, dt), bs, dev, dt,
                           lambda n: torch.randperm(n, generator=g).tolist())
    qd = torch.zeros(T, H, kc.shape[3], dtype=dt, device=dev)
    qd[:, :, :D] = q.to(dev, dt)
    got = ops.attn_window_paged(qd, kc, vc, tables, i32(cu, dev), i32(pos, dev), scale, window, 0, None,
                                fold_heads=True, out_scale=gate.to(dev, torch.float32))[:, :, :Dv]
    want = torch.zeros(T, H, Dv, dtype=F64)
    for s, (a, b) in enumerate(rows):
        k, v = seqs[s]
        for h in range(H):
            full = torch.zeros(b, D, dtype=F64)
            full[a:b] = q[cu[s]:cu[s + 1], h]
            want[cu[s]:cu[s + 1], h] = O.windowed_softmax_attention(full, k, v, scale, window)[a:b]
    want = want * gate[:, :, None]
    assert close(got, want, dt, f32_tol=1e-4, bf16_tol=4e-2)
    # unfolded (a workgroup per head) gives the same
    got2 = ops.attn_window_paged(qd, kc, vc, tables, i32(cu, dev), i32(pos, dev), scale, window, 0, None,
                                 fold_heads=False, out_scale=gate.to(dev, torch.float32))[:, :, :Dv]
    assert close(got2, want, dt, f32_tol=1e-4, bf16_tol=4e-2)


@pytest.mark.parametrize("H,D,Dv,window", [(16, 96, 64, 2000), (5, 256, 192, 700), (8, 40, 24, 640)])
def test_shared_head_attention_decoding_long_contexts(target, H, D, Dv, window):
    """Decoded rows only, over hundreds of cached tokens: the shape whose pages the matrix-core
    form splits over several workgroups and merges. One key far back and the key at the window's
    edge stand out for some heads."""
    dev, dt = target
    bs = 32
    g = torch.Generator().manual_seed(H + window)
    rnd = lambda *s: bf(torch.randn(*s, generator=g, dtype=F64))        # noqa: E731
    lens = [1000, 641, 33, 900]
    seqs = [(0.3 * rnd(L, D), rnd(L, Dv)) for L in lens]
    q = 0.3 * rnd(len(lens), H, D)
    for s, L in enumerate(lens):
        i = L - 1
        for h, j in ((0, max(0, i - window + 1)), (1, i - window), (2, 5), (3, i)):
            if h < H and 0 <= j <= i:
                u = rnd(D)
                u = u / u.norm()
                seqs[s][0][j] = bf(4.0 * u)
                q[s, h] = bf(6.0 * u)
    pos = [L - 1 for L in lens]
    cu = list(range(len(lens) + 1))
    gate = torch.rand(len(lens), H, generator=g, dtype=F64).float().to(F64)
    kc, vc, tables = paged(seqs, ops.attn_window_pad(D, dt), ops.attn_window_pad(Dv, dt), bs, dev, dt,
                           lambda n: torch.randperm(n, generator=g).tolist())
    qd = torch.zeros(len(lens), H, kc.shape[3], dtype=dt, device=dev)
    qd[:, :, :D] = q.to(dev, dt)
    want = torch.zeros(len(lens), H, Dv, dtype=F64)
    for s, L in enumerate(lens):
        k, v = seqs[s]
        for h in range(H):
            full = torch.zeros(L, D, dtype=F64)
            full[L - 1] = q[s, h]
            want[s, h] = O.windowed_softmax_attention(full, k, v, 0.7, window)[L - 1]
    want = want * gate[:, :, None]
    for fold in (True, False):
        got = ops.attn_window_paged(qd, kc, vc, tables, i32(cu, dev), i32(pos, dev), 0.7, window, 0, None,
                                    fold_heads=fold, out_scale=gate.to(dev, torch.float32))[:, :, :Dv]
        assert close(got, want, dt, f32_tol=1e-4, bf16_tol=4e-2), fold


def test_latent_preparation_and_cache_append(target):
    dev, dt = target
    g = torch.Generator().manual_seed(9)
    T, Q, R, rd, H, bs, eps = 11, 10, 24, 6, 3, 32, 1e-3
    z = bf(torch.randn(T, Q + R + rd + H + 4, generator=g, dtype=F64) * 2)
    qn, kn = bf(1 + 0.3 * torch.randn(Q, generator=g, dtype=F64)), bf(1 + 0.3 * torch.randn(R, generator=g, dtype=F64))
    pos = list(range(60, 60 + T))
    slots = [3 * bs + 28 + i if i < 4 else 1 * bs + (i - 4) for i in range(T)]       # crosses into another page
    slots[7] = -1                                                                      # a row without a cache slot
    base = 1000.0
    inv = torch.tensor([base ** (-2.0 * i / rd) for i in range(rd // 2)], dtype=torch.float32)
    dk, dv = ops.attn_window_pad(R + rd, dt), ops.attn_window_pad(R, dt)
    kc = torch.zeros(5, 1, bs, dk, dtype=dt, device=dev)
    vc = torch.zeros(5, 1, dv, bs, dtype=dt, device=dev)
    cq, gate = ops.latent_prep(z.to(dev, dt), Q, R, rd, H, qn.to(dev, torch.float32), kn.to(dev, torch.float32), eps,
                               i32(pos, dev), inv.to(dev), i32(slots, dev), kc, vc, dt)
    assert close(cq, O.rms_norm(z[:, :Q], qn, eps), dt, bf16_tol=1e-2)
    assert close(gate, torch.sigmoid(z[:, Q + R + rd:Q + R + rd + H]), torch.float32)
    c = O.rms_norm(z[:, Q:Q + R], kn, eps)
    written = 0
    for t in range(T):
        if slots[t] < 0:
            continue
        b, o = divmod(slots[t], bs)
        kr = O.rotate_pairs(z[t, Q + R:Q + R + rd], pos[t], base, rd)
        assert close(kc[b, 0, o, :R + rd], torch.cat([c[t], kr]), dt, bf16_tol=1e-2)
        assert close(vc[b, 0, :R, o], c[t], dt, bf16_tol=1e-2)
        written += 1
    assert int((kc.float().abs().sum(-1) > 0).sum()) == written        # nothing else was touched


@pytest.mark.parametrize("E,top", [(5, 2), (3, 1), (4, 4), (70, 6)])
def test_router_and_weighted_experts(target, E, top):
    dev, dt = target
    g = torch.Generator().manual_seed(E + top)
    T, C, F = 23, 40, 12
    x = bf(torch.randn(T, C, generator=g, dtype=F64))
    P = {"router": bf(torch.randn(E, C, generator=g, dtype=F64) / 3), "router.b": bf(torch.randn(E, generator=g, dtype=F64))}
    for e in range(E):
        P[f"e{e}.gate"], P[f"e{e}.up"] = (bf(torch.randn(F, C, generator=g, dtype=F64) / 6) for _ in range(2))
        P[f"e{e}.down"] = bf(torch.randn(C, F, generator=g, dtype=F64) / 3)
    ids, w = ops.moe_route_scores(x.to(dev, dt), P["router"].to(dev, dt), top, scoring="softmax", renorm=True,
                                  bias=P["router.b"].to(dev, torch.float32))
    want_ids, want_w = O.route(x, P["router"], P["router.b"], top)
    assert torch.equal(ids.cpu().long().sort(-1).values, want_ids.sort(-1).values)
    order = ids.cpu().long().argsort(-1), want_ids.argsort(-1)
    assert close(w.cpu().gather(1, order[0]), want_w.gather(1, order[1]), torch.float32, f32_tol=1e-5)
    gu = torch.stack([torch.cat([P[f"e{e}.gate"], P[f"e{e}.up"]]) for e in range(E)]).to(dev, dt)
    dn = torch.stack([P[f"e{e}.down"] for e in range(E)]).to(dev, dt)
    got = ops.moe_glu_ffn(x.to(dev, dt), ids, w, gu, dn, float("inf"), 1.0, up_offset=0.0, scale_input=False)
    assert close(got, O.moe_ffn(x, P, E, top), dt, f32_tol=1e-4, bf16_tol=3e-2)


# ---------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------
def cfg_a():
    """Layers that differ from one another in every size; sizes no MFMA tile divides; a short
    window, a routed layer with two of five experts, a dense one, a layer without feed-forward."""
    return O.config([
        O.latent_layer(3, 12, 4, 20, 24, 10, 10000.0, 0.3, 7, O.moe(5, 2, 12)),
        O.latent_layer(2, 8, 6, 10, 14, 18, 100.0, 0.2, 5, O.dense(56)),
        O.latent_layer(4, 6, 2, 6, 9, 7, 1e6, 0.4, 40, None),
    ], width=40, vocab=70, eps=1e-5, taps=3, embed_scale=6.0)


def cfg_b():
    """What another model may make equal or 1 made unequal here, and the other way round: one head,
    one expert chosen of three, every expert chosen of two, a two-tap and unscaled model, a window
    longer than the sequences and a window of one token, query rank above the key/value rank."""
    return O.config([
        O.latent_layer(1, 16, 8, 24, 12, 30, 500.0, 0.25, 4096, O.moe(3, 1, 20)),
        O.latent_layer(5, 4, 8, 4, 20, 6, 500.0, 0.5, 1, O.moe(2, 2, 16)),
        O.latent_layer(2, 8, 4, 12, 16, 16, 50.0, 0.3, 31, O.dense(32)),
    ], width=48, vocab=50, eps=1e-6, taps=2, embed_scale=1.0)


def cfg_c():
    """Sizes the matrix-core kernels tile (bf16): cached rows 64 + 32 and 128 + 64, windows that
    end inside a page and span several, four taps, eight experts."""
    return O.config([
        O.latent_layer(4, 32, 32, 48, 64, 48, 5e5, 0.12, 44, O.dense(256)),
        O.latent_layer(8, 16, 64, 32, 128, 64, 1e4, 0.1, 70, O.moe(8, 2, 96)),
        O.latent_layer(4, 32, 32, 48, 64, 48, 5e5, 0.12, 33, O.moe(8, 3, 96)),
    ], width=128, vocab=256, eps=1e-5, taps=4, embed_scale=11.3)


def cfg_d():
    """A single-tap convolution (no history, no state slots) and one layer."""
    return O.config([O.latent_layer(2, 8, 8, 8, 16, 12, 1e4, 0.3, 20, O.dense(40))],
                    width=32, vocab=40, eps=1e-5, taps=1, embed_scale=2.0)


_ORACLE = {}


def oracle_logits(name, cfg, W, tokens):
    key = (name, tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = O.forward(cfg, W, tokens)
    return _ORACLE[key]


def make_engine(tmp_path, cfg, W, dev, dt, max_batch=4, cache_tokens=512, graphs=False, **kw):
    d = tmp_path / "model"
    d.mkdir(exist_ok=True)
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(d / "model.safetensors"))
    mc = model_config(str(d))
    assert mc.arch == "zinesun"
    m = build_model(mc, device=dev, dtype=dt)
    load_into(m, str(d))
    ecfg = EngineConfig(max_batch=max_batch, max_seq_len=cache_tokens, max_prefill_tokens=kw.pop("budget", cache_tokens),
                        kv_cache_tokens=cache_tokens, use_graphs=graphs, dtype="fp32" if dt == torch.float32 else "bf16",
                        async_decode=kw.pop("async_decode", False), graph_batch_sizes=[1, 2, 4], **kw)
    return LLMEngine(mc, engine_cfg=ecfg, model=m, device=dev)


def tokens_of(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def replay(eng, reqs, schedule):
    """Run `schedule` (steps of [(name, count)]) asking for every row; -> {name: logits [len, V]}."""
    at = {n: 0 for n in reqs}
    rid = {n: i for i, n in enumerate(reqs)}
    out = {n: [] for n in reqs}
    for step in schedule:
        entries, end = [], []
        for n, c in step:
            entries.append((rid[n], reqs[n][at[n]:at[n] + c], list(range(c))))
            at[n] += c
            if at[n] == len(reqs[n]):
                end.append(rid[n])
        lg = eng.replay_step(entries, end).cpu()
        r = 0
        for n, c in step:
            out[n].append(lg[r:r + c])
            r += c
    assert all(at[n] == len(reqs[n]) for n in reqs)
    return {n: torch.cat(v) for n, v in out.items()}


def test_weights_round_trip_and_layer_outputs(tmp_path):
    """Loading a folder and reading the tensors back gives the file's tensors (also the fused and
    transposed ones), and every layer hands on what the oracle's layer does."""
    cfg = cfg_a()
    W = O.random_weights(cfg, seed=5)
    eng = make_engine(tmp_path, cfg, W, torch.device("cpu"), torch.float32)
    back = {lp.name: lp.get() for lp in eng.model.logical_params()}
    assert set(back) == set(W)
    for k, v in W.items():
        assert torch.equal(back[k].reshape(v.shape).float(), v.float()), k
    toks = tokens_of(cfg, 20, 1)
    seen, want = [], []
    eng.model.layer_probe = lambda i, x: seen.append(x.clone())
    eng.replay_step([(0, toks, [0])], [0])
    O.forward(cfg, W, toks, want)
    assert len(seen) == len(want) == 3
    for a, b in zip(seen, want):
        assert close(a, b, torch.float32, f32_tol=1e-4)


@pytest.mark.parametrize("name,mk", [("a", cfg_a), ("b", cfg_b), ("c", cfg_c), ("d", cfg_d)])
def test_prompt_decode_and_portions(target, tmp_path, name, mk):
    """One request: whole prompt; prompt then token-by-token decoding (long, the window passes
    over decoded tokens); portions of many sizes down to two tokens, ending on single tokens; the
    first tokens one by one. Same logits as the oracle every way."""
    dev, dt = target
    cfg = mk()
    W = O.random_weights(cfg, seed=11)
    toks = tokens_of(cfg, 150, 3)
    want = oracle_logits(name, cfg, W, toks)
    eng = make_engine(tmp_path, cfg, W, dev, dt, cache_tokens=160)    # 5 pages: nothing to spare
    got = replay(eng, {"r": toks}, [[("r", 150)]])["r"]
    assert_rows(got, want, dt, "whole prompt")
    got = replay(eng, {"r": toks}, [[("r", 50)]] + [[("r", 1)]] * 100)["r"]          # pages / slot reused
    assert_rows(got, want, dt, "prompt + 100 decoded tokens")
    cuts = [2, 3, 5, 31, 23, 2, 32, 33, 7, 2] + [1] * 10
    assert sum(cuts) == 150
    got = replay(eng, {"r": toks}, [[("r", c)] for c in cuts])["r"]
    assert_rows(got, want, dt, "portions")
    got = replay(eng, {"r": toks[:4]}, [[("r", 1)]] * 4)["r"]                         # first tokens, one by one
    assert_rows(got, want[:4], dt, "first tokens")


@pytest.mark.parametrize("name,mk", [("a", cfg_a), ("b", cfg_b), ("c", cfg_c)])
def test_mixed_batches_reuse_pages_and_slots(target, tmp_path, name, mk):
    """Six requests of unequal length through three state slots and a cache that holds about
    half of them: portions beside decoded tokens of other requests, requests that pause,
    pages and slots handed from finished requests to new ones. Each equals the request alone."""
    dev, dt = target
    cfg = mk()
    W = O.random_weights(cfg, seed=12)
    lens = {"p": 70, "q": 33, "r": 1, "s": 96, "t": 64, "u": 40}
    reqs = {n: tokens_of(cfg, L, 20 + i) for i, (n, L) in enumerate(lens.items())}
    eng = make_engine(tmp_path, cfg, W, dev, dt, max_batch=3, cache_tokens=224)
    sched = [[("p", 40), ("q", 2)], [("p", 1), ("q", 30), ("r", 1)], [("q", 1), ("p", 20)],
             [("p", 1), ("s", 33)], [("s", 31), ("p", 1)], [("p", 1), ("s", 1)]] + \
            [[("p", 1), ("s", 1), ("t", 3)]] * 6 + [[("s", 24), ("t", 46)], [("u", 2)], [("u", 37), ("s", 1)],
                                                    [("u", 1)]]
    got = replay(eng, reqs, sched)
    for n in reqs:
        assert_rows(got[n], oracle_logits(name, cfg, W, reqs[n]), dt, f"request {n}")
    m = eng.kv.manager
    assert m.num_free == m.num_blocks and m.num_free_state_slots == 3


@pytest.mark.parametrize("graphs", [False, pytest.param(True, marks=gpu)])
def test_greedy_generation_through_the_scheduler(target, tmp_path, graphs):
    """LLMEngine.generate: the scheduler's own admission, chunked prompts (a small token budget),
    mixed steps, decode (hipGraph replays on the GPU) and the sampler; tokens equal the oracle's
    greedy continuation."""
    dev, dt = target
    if graphs and dev.type != "cuda":
        pytest.skip("graphs need a GPU")
    cfg = cfg_a()
    W = O.random_weights(cfg, seed=13)
    prompts = [tokens_of(cfg, n, 40 + n) for n in (37, 5, 64, 18, 2)]
    eng = make_engine(tmp_path, cfg, W, dev, dt, max_batch=3, cache_tokens=512, graphs=graphs, budget=24,
                      async_decode=graphs)
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        if dt == torch.float32:
            assert o == O.greedy(cfg, W, p, 12)
        else:       # bf16: every generated token is (nearly) the oracle's best continuation of its prefix
            lg = O.forward(cfg, W, p + o)
            for i, t in enumerate(o):
                row = lg[len(p) + i - 1]
                assert row[t] >= row.max() - 0.15 * (row.max() - row.mean())
    m = eng.kv.manager
    assert m.num_free == m.num_blocks and m.num_free_state_slots == 3


def test_random_init_and_registry():
    """The family is built from a configuration alone (random weights, as the benchmarks do)."""
    from butterfly_amd.config import ModelConfig

    mc = ModelConfig.from_zinesun(cfg_b())
    assert mc.arch == "zinesun" and mc.conv_taps == 2 and mc.embed_scale == 1.0 and mc.tie_embeddings
    m = build_model(mc, device="cpu", dtype=torch.float32)
    m.init_random(3)
    assert m.has_state and m.state_bytes_per_slot() == 4 * 1 * 48 * 3
    eng = LLMEngine(mc, engine_cfg=EngineConfig(max_batch=2, max_seq_len=64, kv_cache_tokens=128, use_graphs=False,
                                                dtype="fp32", async_decode=False), model=m, device=torch.device("cpu"))
    out = eng.generate([[1, 2, 3], [4]], SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in out] == [3, 3]


def test_llm_entry_point_from_a_model_folder(tmp_path):
    """butterfly_amd.LLM on a folder: family chosen by config.json, a data-parallel-only plan from
    the partitioner, the default (overlapped) engine settings, greedy tokens equal the oracle's."""
    from butterfly_amd.api import LLM

    cfg = cfg_b()
    W = O.random_weights(cfg, seed=21)
    d = tmp_path / "model"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(d / "model.safetensors"))
    llm = LLM(str(d), engine_config=EngineConfig(max_batch=3, max_seq_len=96, kv_cache_tokens=256, dtype="fp32"))
    assert llm.cfg.arch == "zinesun" and (llm.plan.mesh.tp, llm.plan.mesh.pp) == (1, 1)
    prompts = [tokens_of(cfg, n, 60 + n) for n in (9, 33, 2)]
    outs = llm.generate(prompts, SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.token_ids == O.greedy(cfg, W, p, 5)
    llm.close()
