"""The Sabezen decoder on the GPU against the plain implementation: the new kernels alone, each
mechanism as a model of one layer, the whole model under four ways of cutting the same requests into
steps (whole, bulk then single tokens, portions down to two tokens, mixed batches on a small page pool
with four state slots, pages and slots used again), in 32-bit and in bfloat16, on configurations with
even and with odd sizes and on one without any attention; keys far away and at the edges of a chunk;
long decoding through graph replays; greedy generation through the entry point and its scheduler; the
trace runner and the command line as subprocesses."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_sabezen as ps
import sabezen_util as su
import trace_util as tu
from conftest import ROOT

pytestmark = pytest.mark.gpu

TOL = {"float32": 3e-5, "bfloat16": 8e-2}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
LENGTHS = {"A": [5, 17, 64, 1, 100, 33, 129, 49, 2], "B": [40, 3, 100, 65, 2, 31], "C": [90, 3, 41, 1, 130],
           "D": [700, 47, 313, 1, 161]}


def dev(a, dtype=None):
    t = torch.as_tensor(np.asarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda().contiguous()


def i32(a):
    return torch.as_tensor(np.asarray(a, dtype=np.int32)).cuda()


# ------------------------------------------------------------------ kernels alone

def test_layernorm_and_scaled_embedding():
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 90, generator=g) * 3 + 1.5
    w = 1 + torch.randn(90, generator=g) * 0.3
    for dt in (torch.float32, torch.bfloat16):
        out = torch.zeros(7, 90, dtype=dt, device="cuda")
        ops.layernorm(out, x.cuda(), w.to(dt).cuda(), 1e-5)
        want = ps.layer_norm(x.double(), w.to(dt).double(), 1e-5)
        assert su.rel(out.double().cpu(), want) < (2e-6 if dt == torch.float32 else 6e-3)
    rows = i32([5, 0, 5])
    out = torch.zeros(3, 90, device="cuda")
    ops.layernorm(out, x.cuda(), w.cuda(), 1e-5, rows)
    assert su.rel(out.cpu(), ps.layer_norm(x.double(), w.double(), 1e-5)[[5, 0, 5]]) < 2e-6
    table = torch.randn(20, 24, generator=g)
    for dt in (torch.float32, torch.bfloat16):
        emb = torch.zeros(4, 24, device="cuda")
        ops.embed(emb, table.to(dt).cuda(), i32([3, 19, 0, 3]), scale=7.5)
        assert torch.equal(emb.cpu(), table.to(dt).float()[[3, 19, 0, 3]] * 7.5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_xielu(dtype):
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    z = torch.linspace(-6, 6, 333).reshape(3, 111).to(dt)
    p, q = torch.tensor(0.7, dtype=torch.float64), torch.tensor(-0.4, dtype=torch.float64)
    a, b = float(torch.nn.functional.softplus(p)), 0.5 + float(torch.nn.functional.softplus(q))
    out = torch.zeros(3, 111, dtype=dt, device="cuda")
    ops.bias_act(out, z.cuda(), None, "xielu", (a, b))
    want = ps.xielu(z.double(), p, q)
    assert su.rel(out.double().cpu(), want) < (1e-6 if dtype == "float32" else 5e-3)


def _paged(positions_of_segments, page_size=16, seed=0):
    """positions [n], token_segment [n], tables [segments, blocks] with pages in a shuffled order."""
    rng = np.random.default_rng(seed)
    most = max(p[-1] for p in positions_of_segments) + 1
    blocks = -(-most // page_size)
    pages = rng.permutation(len(positions_of_segments) * blocks + 2)
    tables = pages[:len(positions_of_segments) * blocks].reshape(len(positions_of_segments), blocks)
    pos = np.concatenate(positions_of_segments)
    seg = np.concatenate([np.full(len(p), s) for s, p in enumerate(positions_of_segments)])
    return i32(pos), i32(seg), i32(tables), len(pages)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("chunk,H,G,D,half", [(24, 4, 2, 16, 4), (70, 3, 3, 20, 10), (0, 2, 1, 8, 0)])
def test_mixed_attention_kernels_with_a_key_that_stands_out(dtype, chunk, H, G, D, half):
    """One key far back in the query's chunk, one just outside it and the chunk's first and last keys are
    made to stand out (their key and the queries behind them scaled up): a kernel that loses a far key,
    reads one key too many at the chunk's edge or one too few shows.  The cache is written in portions
    (one of them two tokens) and the last tokens one by one."""
    from hfee_amd.kernels import ops
    from hfee_amd.parts.rotary import rope_frequencies
    dt, T, page = DT[dtype], 150, 16
    g = torch.Generator().manual_seed(chunk + H)
    size = chunk or T
    q = torch.randn(T, H, D, generator=g)
    k = torch.randn(T, G, D, generator=g)
    last = T - 1
    first = last // size * size
    marked = [first, max(first - 1, 0), first + 1, last, 2]
    for j in marked:
        k[j] *= 3.0
    q[last] = k[marked[0]].repeat_interleave(H // G, dim=0) * 1.5 + q[last] * 0.1      # looks at its chunk's first key
    if first > 0:
        q[last - 1] = k[first - 1].repeat_interleave(H // G, dim=0) * 1.5                  # looks just outside: must not see it
    q, k = q.to(dt), k.to(dt)
    talk = torch.eye(H) + torch.randn(H, H, generator=g) * 0.3
    m = {"heads": H, "kv_heads": G, "dim": D, "scale": 0.3, "mask": {"size": size}, "rot": {"dims": 2 * half, "base": 100.0}}
    # the plain mixer with identity projections: its input is [q | k]
    hidden = (H + G) * D
    w = {"m.q": torch.eye(hidden)[:H * D], "m.k": torch.eye(hidden)[H * D:], "m.talk": talk, "m.o": torch.eye(H * D)}
    want = ps.chunked_talking_attention(torch.cat([q.reshape(T, -1), k.reshape(T, -1)], dim=1).double(),
                                        {n: t.double() for n, t in w.items()}, "m.", m, 1e-6)
    inv = rope_frequencies(2 * half, 100.0) if half else np.zeros(0)
    ang = np.arange(T)[:, None] * inv[None, :]
    cos, sin = (dev(np.cos(ang), torch.float32), dev(np.sin(ang), torch.float32)) if half else (None, None)
    got = torch.zeros(T, H * D, dtype=dt, device="cuda")
    cuts = [0, 37, 39, 100, 140] + list(range(141, T + 1))
    pos_all, seg_all, tables, pages = _paged([np.arange(T)], page, seed=1)
    cache = torch.full((pages, G, page * 2 * D), float("nan"), dtype=dt, device="cuda")
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        qs, ks = q[lo:hi].reshape(hi - lo, -1).cuda().contiguous(), k[lo:hi].reshape(hi - lo, -1).cuda().contiguous()
        pos, seg = pos_all[lo:hi].contiguous(), seg_all[lo:hi].contiguous()
        ops.attention_mix_prepare(qs, ks, pos, seg, tables, cos, sin, cache, H, G, D, page, hi - 1, norm=True, eps=1e-6)
        out = torch.zeros(hi - lo, H * D, dtype=dt, device="cuda")
        ops.attention_mix(out, qs, cache, pos, seg, tables, H, G, D, page, 0.3, mix=talk.cuda(), chunk=chunk, sink="zero")
        got[lo:hi] = out
    tol = 3e-5 if dtype == "float32" else 3e-2
    assert su.rel(got.double().cpu(), want) < tol
    for t in (last, last - 1, first, min(first + 1, last)):
        assert su.rel(got[t].double().cpu(), want[t]) < tol, f"token {t}"


@pytest.mark.parametrize("chunk,H,G,D,half", [(24, 4, 2, 32, 8), (70, 8, 2, 64, 16), (0, 4, 4, 32, 0), (16, 8, 8, 32, 16)])
def test_mixed_attention_on_the_matrix_cores(chunk, H, G, D, half):
    """The matrix-core kernel against the plain mixer in float64 and against the plain kernel, with keys
    that stand out at the chunk's first and last place and just outside it; the sequence comes in
    portions whose items end at every chunk's edge, then token by token, beside a second sequence."""
    from hfee_amd.kernels import ops
    from hfee_amd.parts.rotary import rope_frequencies
    T, page = 150, 16
    g = torch.Generator().manual_seed(chunk + H)
    size = chunk or T
    q = torch.randn(2, T, H, D, generator=g)
    k = torch.randn(2, T, G, D, generator=g)
    last = T - 1
    first = last // size * size
    for j in (first, max(first - 1, 0), min(first + 1, last), last, 2):
        k[:, j] *= 3.0
    q[0, last] = k[0, first].repeat_interleave(H // G, dim=0) * 1.5 + q[0, last] * 0.1
    if first > 0:
        q[0, last - 1] = k[0, first - 1].repeat_interleave(H // G, dim=0) * 1.5
    q, k = q.bfloat16(), k.bfloat16()
    talk = torch.eye(H) + torch.randn(H, H, generator=g) * 0.3
    m = {"heads": H, "kv_heads": G, "dim": D, "scale": 0.3, "mask": {"size": size}, "rot": {"dims": 2 * half, "base": 100.0}}
    hidden = (H + G) * D
    w = {"m.q": torch.eye(hidden)[:H * D].double(), "m.k": torch.eye(hidden)[H * D:].double(), "m.talk": talk.double(),
         "m.o": torch.eye(H * D).double()}
    want = [ps.chunked_talking_attention(torch.cat([q[s].reshape(T, -1), k[s].reshape(T, -1)], dim=1).double(), w, "m.", m, 1e-6)
            for s in range(2)]
    inv = rope_frequencies(2 * half, 100.0) if half else np.zeros(0)
    ang = np.arange(T)[:, None] * inv[None, :]
    cos, sin = (dev(np.cos(ang), torch.float32), dev(np.sin(ang), torch.float32)) if half else (None, None)
    _, _, tables, pages = _paged([np.arange(T), np.arange(T)], page, seed=2)
    cache = torch.zeros((pages, G, page * 2 * D), dtype=torch.bfloat16, device="cuda")
    got = torch.zeros(2, T, H * D, dtype=torch.bfloat16, device="cuda")
    plain = torch.zeros(2, T, H * D, dtype=torch.bfloat16, device="cuda")
    fed = [0, 0]
    steps = [(37, 5), (2, 60), (61, 0), (40, 45), (0, 30)] + [(1, 1)] * 10
    for sizes in steps:
        segs = [(s, n) for s, n in enumerate(sizes) if n]
        pos = np.concatenate([np.arange(fed[s], fed[s] + n) for s, n in segs])
        seg = np.concatenate([np.full(n, s) for s, n in segs])        # (the block table's row is the sequence)
        qs = torch.cat([q[s, fed[s]:fed[s] + n].reshape(n, -1) for s, n in segs]).cuda().contiguous()
        ks = torch.cat([k[s, fed[s]:fed[s] + n].reshape(n, -1) for s, n in segs]).cuda().contiguous()
        ops.attention_mix_prepare(qs, ks, i32(pos), i32(seg), tables, cos, sin, cache, H, G, D, page, int(pos.max()),
                                  norm=True, eps=1e-6)
        items, row = [], 0
        for s, n in segs:
            off = 0
            while off < n:
                p = fed[s] + off
                room = min(16, n - off, (chunk - p % chunk) if chunk else 16)
                items.append((row + off, room, p, s))
                off += room
            row += n
        out = torch.zeros(len(pos), H * D, dtype=torch.bfloat16, device="cuda")
        splits = 1 + len(pos) % 4                      # (the key tiles of an item over one to four workgroups)
        partial = torch.full((ops.attention_mix_partial_words(len(items), H, D, splits),), float("nan"), device="cuda")
        ops.attention_mix_bf16(out, qs, cache, i32(np.asarray(items).reshape(-1, 4)), tables, H, G, D, page, 0.3,
                               mix_t=talk.t().contiguous().cuda(), chunk=chunk, sink="zero", splits=splits,
                               partial=partial if splits > 1 else None)
        ref = torch.zeros_like(out)
        ops.attention_mix(ref, qs, cache, i32(pos), i32(seg), tables, H, G, D, page, 0.3, mix=talk.cuda(), chunk=chunk, sink="zero")
        row = 0
        for s, n in segs:
            got[s, fed[s]:fed[s] + n] = out[row:row + n]
            plain[s, fed[s]:fed[s] + n] = ref[row:row + n]
            row += n
            fed[s] += n
    assert fed == [T, T]
    for s in range(2):
        assert su.rel(plain[s].double().cpu(), want[s]) < 3e-2
        assert su.rel(got[s].double().cpu(), want[s]) < 3e-2
        assert su.rel(got[s].double().cpu(), plain[s].double().cpu()) < 2e-2
        for t in (last, last - 1, first, min(first + 1, last), 0, 1, 15, 16, 17):
            assert su.rel(got[s, t].double().cpu(), want[s][t]) < 3e-2, f"sequence {s} token {t}"


@pytest.mark.parametrize("rule", ["delta", "decay_add"])
@pytest.mark.parametrize("H,G,D,V", [(4, 2, 8, 16), (3, 3, 20, 12), (2, 1, 33, 70)])
def test_linear_scan_in_portions(rule, H, G, D, V):
    """The recurrence by its definition, token by token in float64, against the kernel fed the same
    sequence in portions of unequal size for two requests side by side in other slots."""
    from hfee_amd.kernels import ops
    if rule == "decay_add":
        G = H
    g = torch.Generator().manual_seed(D)
    T = [45, 23]
    data = []
    for t in T:
        q, k = torch.randn(t, G, D, generator=g) * 0.4, torch.randn(t, G, D, generator=g) * 0.4
        v = torch.randn(t, H, V, generator=g)
        a = torch.rand(t, H, D, generator=g) * 0.3 + 0.7
        b = torch.rand(t, H, generator=g)
        data.append((q, k, v, a, b))
    want, final = [], []
    for q, k, v, a, b in data:
        o = torch.zeros(q.shape[0], H, V, dtype=torch.float64)
        final.append([])
        for h in range(H):
            S = torch.zeros(D, V, dtype=torch.float64)
            for t in range(q.shape[0]):
                qt, kt = q[t, h // (H // G)].double(), k[t, h // (H // G)].double()
                S = a[t, h].double()[:, None] * S
                u = b[t, h].double() * (v[t, h].double() - S.T @ kt) if rule == "delta" else v[t, h].double()
                S = S + kt[:, None] * u[None, :]
                o[t, h] = S.T @ qt
            final[-1].append(S)
        want.append(o.reshape(q.shape[0], -1))
    state = torch.zeros(5, H, *ops.scan_state_shape(D, V), device="cuda")
    state[1].fill_(float("nan"))                    # a slot that nobody uses
    slots = [3, 0]
    fed = [0, 0]
    got = [torch.zeros(t, H * V) for t in T]
    for sizes in ([7, 2], [1, 1], [20, 0], [2, 13], [15, 7]):
        segs = [(s, n) for s, n in enumerate(sizes) if n]
        parts = [tuple(x[fed[s]:fed[s] + n] for x in data[s]) for s, n in segs]
        cat = [torch.cat([p[i].reshape(p[i].shape[0], -1) for p in parts]).cuda().contiguous() for i in range(5)]
        rows = np.cumsum([0] + [n for _, n in segs])[:-1]
        out = torch.zeros(sum(n for _, n in segs), H * V, device="cuda")
        ops.linear_scan(out, state, cat[0], cat[1], cat[2], cat[3], cat[4] if rule == "delta" else None, i32(rows),
                        i32([n for _, n in segs]), i32([slots[s] for s, _ in segs]), H, G, D, V, rule)
        for (s, n), r in zip(segs, rows):
            got[s][fed[s]:fed[s] + n] = out[r:r + n].cpu()
            fed[s] += n
    assert fed == T
    for s in range(2):
        assert su.rel(got[s], want[s]) < 2e-5
        assert su.rel(ops.scan_state_matrix(state[slots[s]], D, V).cpu(), torch.stack(final[s])) < 2e-5
    assert bool(torch.isnan(state[1]).all()) and float(state[2].abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("K", [1, 2, 4, 5])
def test_short_convolution_carries_its_inputs(dtype, K):
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(K)
    C, T = 37, 30
    x = torch.randn(T, C, generator=g).to(dt)
    taps = torch.randn(C, K, generator=g)
    want = ps.short_conv_silu(x.double(), taps.double())
    state = torch.zeros(3, K - 1, C, dtype=dt, device="cuda")
    got = torch.zeros(T, C)
    at = 0
    for n in (1, 1, 2, 9, 1, 3, 13):       # (portions shorter than the taps keep a part of the old state)
        xs = x[at:at + n].cuda().contiguous()
        y = torch.zeros(n, C, device="cuda")
        ops.short_conv_silu(y, xs, state, taps.cuda(), i32([0] * n), i32([0]), i32([2]))
        ops.short_conv_keep(state, xs, i32([0]), i32([n]), i32([2]))
        got[at:at + n] = y.cpu()
        at += n
    assert at == T and su.rel(got, want) < 2e-6
    assert float(state[:2].abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_experts_by_table(dtype):
    from hfee_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(4)
    n, width, F, E, top, vocab = 9, 40, 22, 5, 3, 30
    h = torch.randn(n, width, generator=g).to(dt)
    wg, wu = (torch.randn(E, F, width, generator=g) * 0.2).to(dt), (torch.randn(E, F, width, generator=g) * 0.2).to(dt)
    wd = (torch.randn(E, width, F, generator=g) * 0.2).to(dt)
    table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(vocab)]).to(torch.int32)
    ids = torch.randint(0, vocab, (n,), generator=g)
    w = {"m.table": table}
    for e in range(E):
        w.update({f"m.e{e}.gate": wg[e].double(), f"m.e{e}.up": wu[e].double(), f"m.e{e}.down": wd[e].double()})
    want = ps.table_moe(h.double(), ids, w, "m.", {"router": {"top": top}})
    x = torch.ones(n, width, device="cuda")
    act = torch.zeros(n * top, F, dtype=dt, device="cuda")
    ops.moe_up(act, h.cuda(), wg.cuda(), wu.cuda(), top, table=table.cuda(), token_ids=i32(ids))
    ops.moe_down(x, act, wd.cuda(), top, weight=1.0 / top, table=table.cuda(), token_ids=i32(ids))
    assert su.rel(x.double().cpu() - 1.0, want) < (1e-5 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("n,top,E,F,width", [(300, 2, 5, 96, 64), (70, 1, 3, 32, 96), (9, 3, 4, 64, 32), (129, 4, 40, 320, 128)])
def test_experts_grouped_on_the_matrix_cores(n, top, E, F, width):
    """Pairs grouped by expert against the token-by-token kernels and the plain sum: experts with no
    token, with one, with more than a tile of 64; every token's own result whatever shares its tile."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(n)
    vocab = 50
    h = torch.randn(n, width, generator=g).bfloat16()
    wg, wu = (torch.randn(E, F, width, generator=g) * 0.2).bfloat16(), (torch.randn(E, F, width, generator=g) * 0.2).bfloat16()
    wd = (torch.randn(E, width, F, generator=g) * 0.2).bfloat16()
    table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(vocab)]).to(torch.int32)
    if E > 4:
        table[table == 1] = 0 if top == 1 else table[table == 1]        # (an expert that nobody uses, where rows stay distinct)
    ids = torch.randint(0, vocab, (n,), generator=g)
    x0 = torch.randn(n, width, generator=g)
    one = x0.clone().cuda()
    act = torch.zeros(n * top, F, dtype=torch.bfloat16, device="cuda")
    ops.moe_up(act, h.cuda(), wg.cuda(), wu.cuda(), top, table=table.cuda(), token_ids=i32(ids))
    ops.moe_down(one, act, wd.cuda(), top, weight=1.0 / top, table=table.cuda(), token_ids=i32(ids))
    grouped = x0.clone().cuda()
    order = torch.zeros(n * top, dtype=torch.int32, device="cuda")
    tiles = torch.zeros(3 * ops.moe_group_tiles(n, top, E) + 1, dtype=torch.int32, device="cuda")
    act2 = torch.zeros(n * top, F, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(n * top, width, device="cuda") if top > 1 else None
    ops.moe_grouped(grouped, h.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), top, order, tiles, act2, y, weight=1.0 / top,
                    table=table.cuda(), token_ids=i32(ids))
    assert sorted(order.cpu().tolist()) == list(range(n * top))
    assert su.rel((grouped - x0.cuda()).cpu(), (one - x0.cuda()).cpu()) < 1e-2
    # the same tokens in another company: a token's numbers stay what they were, bit for bit
    keep = torch.arange(0, n, 3)
    again = x0[keep].clone().cuda()
    ops.moe_grouped(again, h[keep].cuda().contiguous(), wg.cuda(), wu.cuda(), wd.cuda(), top, order, tiles, act2, y,
                    weight=1.0 / top, table=table.cuda(), token_ids=i32(ids[keep]))
    assert torch.equal(again.cpu(), grouped.cpu()[keep])


# ------------------------------------------------------------------ the whole model

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("sabezen")
    out = {(name, dtype): su.make_folder(base / f"{name}_{dtype}", cj, seed=7 + ord(name[0]), dtype=dtype)
           for name, cj in list(su.CONFIGS.items()) + list(su.SINGLE.items()) for dtype in ("float32", "bfloat16")}
    return out


def plain_logits(folder, tokens):
    cj, w = su.load_plain(folder)
    return ps.forward(cj, w, tokens, dtype=torch.float64).numpy()


@pytest.fixture(scope="module")
def plain_rows(folders):
    cache = {}

    def get(name, dtype, lengths=None):
        key = (name, dtype, tuple(lengths or LENGTHS[name]))
        if key not in cache:
            cj = (su.CONFIGS.get(name) or su.SINGLE[name])
            reqs = tu.make_requests(cj["vocab"], list(key[2]), seed=ord(name[0]))
            rows = {}
            for rid, toks in reqs.items():
                logits = plain_logits(folders[(name, dtype)], toks)
                rows.update({(rid, i): logits[i] for i in range(len(toks))})
            cache[key] = (reqs, rows)
        return cache[key]
    return get


def compare(got, want, tol, what):
    assert set(got) == set(want), f"{what}: positions differ"
    worst, where, errors = 0.0, None, []
    for key in want:
        e = su.rel(got[key], want[key])
        errors.append(e)
        if not e <= worst:
            worst, where = e, key
    assert worst < tol, f"{what}: worst relative error {worst:.3e} at {where}"
    assert np.median(errors) < tol / 2, f"{what}: median relative error {np.median(errors):.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(su.SINGLE))
def test_each_mechanism_as_a_model_of_one_layer(folders, plain_rows, name, dtype):
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows(name, dtype, [37, 2, 11])
    for what, steps in (("whole", tu.whole(reqs)), ("bulk then single tokens", tu.bulk_then_tail(reqs, 9)),
                        ("portions", tu.portions(reqs, sizes=(2, 5, 3, 2, 7)))):
        rep = Replayer(folders[(name, dtype)], dtype, 64, max_requests=2)
        compare(tu.run(rep, steps), want, TOL[dtype], f"{name} {dtype} {what}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_every_way_of_cutting_gives_the_plain_logits(folders, plain_rows, name, dtype):
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows(name, dtype)
    longest = max(len(t) for t in reqs.values())
    one = (longest + 63) // 64 * 64
    for what, steps, room in (("whole", tu.whole(reqs), one), ("bulk then single tokens", tu.bulk_then_tail(reqs, 40), one),
                              ("portions", tu.portions(reqs), one), ("mixed", *tu.mixed(reqs, seed=len(name)))):
        rep = Replayer(folders[(name, dtype)], dtype, room, max_requests=4)
        got = tu.run(rep, steps)
        compare(got, want, TOL[dtype], f"{name} {dtype} {what}")
        rep.engine.cache.check()
        assert not rep.engine.cache.requests


def test_cuts_agree_closely_in_32_bit(folders, plain_rows):
    """Whole prompts against portions and single tokens: rounding apart, the same logits."""
    from hfee_amd.trace_replay import Replayer
    reqs, _ = plain_rows("A", "float32")
    runs = []
    for steps in (tu.whole(reqs), tu.portions(reqs, sizes=(2, 3, 16, 1, 15, 17, 2)), tu.bulk_then_tail(reqs, 20)):
        runs.append(tu.run(Replayer(folders[("A", "float32")], "float32", 192, max_requests=4), steps))
    for other in runs[1:]:
        for key in runs[0]:
            assert su.rel(other[key], runs[0][key]) < 3e-6


@pytest.mark.parametrize("name", ["A", "C"])
def test_a_slot_that_is_used_again_starts_from_nothing(folders, plain_rows, name):
    """One state slot and a pool of one request's pages: every request inherits the slot and the pages of
    the one before, whose state and convolution inputs must be gone."""
    from hfee_amd.trace_replay import Replayer
    reqs, want = plain_rows(name, "float32")
    longest = max(len(t) for t in reqs.values())
    rep = Replayer(folders[(name, "float32")], "float32", (longest + 63) // 64 * 64, max_requests=1)
    got = tu.run(rep, tu.portions(reqs, sizes=(9, 2, 30)))
    compare(got, want, TOL["float32"], f"{name}: one slot for all")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """300 single tokens after a short prompt: decode steps replayed from captured graphs, across page
    borders and across several chunks, the states carried through every replay."""
    from hfee_amd.trace_replay import Replayer
    rng = np.random.default_rng(9)
    toks = rng.integers(0, 500, size=330).tolist()
    rep = Replayer(folders[("D", dtype)], dtype, 384, max_requests=4)
    steps = [{"entries": [("a", toks[:30], [29])], "end": []}]
    steps += [{"entries": [("a", toks[i:i + 1], [0])], "end": ["a"] if i == 329 else []} for i in range(30, 330)]
    got = tu.run(rep, steps)
    assert rep.engine.graph_replays > 250
    want = plain_logits(folders[("D", dtype)], toks)
    compare(got, {("a", i): want[i] for i in range(29, 330)}, TOL[dtype], f"long decoding {dtype}")


def test_grouped_experts_inside_replayed_decode_steps(tmp_path):
    """Three requests decode side by side on a model of two experts, both for every token: more pairs than
    experts, so the grouped kernels (their ordering on the device included) run inside the recorded graphs."""
    from hfee_amd.trace_replay import Replayer
    cj = su.config(70, 64, 1e-6, 2.0, [su.moe(su.gla(2, 16, 16, 6.0, 8), 32, 2, 2), su.moe(su.attention(4, 2, 32, 16, 24, 0.2), 64, 3, 2)])
    folder = su.make_folder(tmp_path / "few", cj, seed=5, dtype="bfloat16")
    reqs = tu.make_requests(70, [50, 47, 44], seed=1)
    steps = [{"entries": [(rid, toks[:4], [3]) for rid, toks in reqs.items()], "end": []}]
    for i in range(4, 44):
        steps.append({"entries": [(rid, toks[i:i + 1], [0]) for rid, toks in reqs.items()], "end": []})
    steps.append({"entries": [(rid, toks[44:], [len(toks) - 45]) for rid, toks in reqs.items() if len(toks) > 44],
                  "end": list(reqs)})
    rep = Replayer(folder, "bfloat16", 256, max_requests=4)
    got = tu.run(rep, steps)
    assert rep.engine.graph_replays > 30
    want = {}
    for rid, toks in reqs.items():
        logits = plain_logits(folder, toks)
        want.update({(rid, i): logits[i] for i in range(3, 44)})
        if len(toks) > 44:
            want[(rid, len(toks) - 1)] = logits[len(toks) - 1]
    compare(got, want, TOL["bfloat16"], "grouped experts in graphs")


def test_a_far_token_shows_through_the_states(folders):
    """Two sequences that differ in their first token only: hundreds of tokens later the recurrent layers
    still carry the difference (no attention layer could: the chunks are long past), and the engine's
    logits follow the plain ones in both."""
    from hfee_amd.trace_replay import Replayer
    rng = np.random.default_rng(2)
    a = rng.integers(0, 60, size=260).tolist()
    b = [(a[0] + 7) % 60] + a[1:]
    rep = Replayer(folders[("C", "float32")], "float32", 640, max_requests=2)
    got = tu.run(rep, [{"entries": [("a", a[:200], []), ("b", b[:200], [])], "end": []},
                       {"entries": [("a", a[200:], [59]), ("b", b[200:], [59])], "end": ["a", "b"]}])
    wa, wb = plain_logits(folders[("C", "float32")], a)[259], plain_logits(folders[("C", "float32")], b)[259]
    assert su.rel(got[("a", 259)], wa) < TOL["float32"] and su.rel(got[("b", 259)], wb) < TOL["float32"]


def greedy(folder, prompt, count):
    seq = list(prompt)
    for _ in range(count):
        seq.append(int(np.argmax(plain_logits(folder, seq)[-1])))
    return seq[len(prompt):]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    from hfee_amd import LLM, SamplingParams
    folder = folders[("A", dtype)]
    llm = LLM(folder, dtype=dtype, num_ctx=128, num_parallel=3, max_batch_tokens=24)
    g = np.random.default_rng(5)
    prompts = [g.integers(0, 131, size=n).tolist() for n in (5, 40, 1, 17, 33)]
    outs = llm.generate(prompts, SamplingParams.greedy(num_predict=8))
    for p, o in zip(prompts, outs):
        want = greedy(folder, p, 8)
        if dtype == "float32":
            assert o.token_ids == want
        else:
            logits = plain_logits(folder, p + want)
            margins = []
            for i in range(8):
                row = np.sort(logits[len(p) - 1 + i])
                margins.append(float((row[-1] - row[-2]) / np.abs(row).max()))
            tu.agree_until_a_near_tie(o.token_ids, want, margins, f"greedy {dtype}")


def test_trace_runner_as_a_subprocess(folders, tmp_path):
    folder = folders[("B", "float32")]
    toks = list(range(1, 40))
    lines = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:21], "want": [0, 20]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[21:22], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[22:], "want": [16]}, {"id": "y", "tokens": toks[:2], "want": [1]}],
              "end": ["x", "y"]}]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(l) for l in lines) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = plain_logits(folder, toks)
    a = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    c = np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)
    assert not (out / "1.f32").exists()
    assert su.rel(a[0], want[0]) < 3e-5 and su.rel(a[1], want[20]) < 3e-5
    assert su.rel(c[0], want[38]) < 3e-5 and su.rel(c[1], want[1]) < 3e-5


def test_the_command_line_runs_the_design(folders):
    """`hfee run <folder> --tokens ...`: the greedy continuation's ids."""
    folder = folders[("B", "float32")]
    prompt = tu.make_requests(97, [11], seed=8)["r0"]
    want = greedy(folder, prompt, 7)
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "hfee"), "run", folder, "--tokens",
                        ",".join(map(str, prompt)), "--dtype", "float32", "--temperature", "0", "--repeat-penalty", "1",
                        "--num-predict", "7", "--num-ctx", "128", "--verbose"],
                       capture_output=True, text=True, timeout=300, stdin=subprocess.DEVNULL)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [int(t) for t in p.stdout.strip().splitlines()[0].split()] == want


def test_seeded_sampling_does_not_depend_on_the_batch(folders):
    from hfee_amd import LLM, SamplingParams
    folder = folders[("A", "float32")]
    g = np.random.default_rng(3)
    prompts = [g.integers(0, 131, size=n).tolist() for n in (9, 30, 2)]
    params = [SamplingParams(temperature=0.9, top_k=20, top_p=0.95, seed=100 + i, num_predict=10) for i in range(3)]
    together = LLM(folder, dtype="float32", num_ctx=128, num_parallel=3).generate(prompts, params)
    for i in range(3):
        alone = LLM(folder, dtype="float32", num_ctx=128, num_parallel=1).generate([prompts[i]], [params[i]])[0]
        assert alone.token_ids == together[i].token_ids
