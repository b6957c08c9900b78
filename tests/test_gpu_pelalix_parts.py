"""Every mechanism of the Pelalix design alone: the framework's kernels against the plain functions of
`plain_pelalix.py`, on sizes and inputs made here."""
import math

import pytest
import torch

import plain_pelalix as pp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64
TYPES = [(torch.float32, 2e-6), (torch.bfloat16, 6e-3)]


def rnd(shape, seed, std=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def close(got, want, tol, what):
    scale = max(float(want.abs().max()), 1e-6)
    err = float((got.detach().cpu().to(F64) - want).abs().max()) / scale
    assert err <= tol, f"{what}: error {err:.3e} of the largest value, tolerance {tol:.1e}"


def step_arrays(new, cached):
    """The device arrays of a step in which request s brings new[s] tokens after cached[s]."""
    seq, pos, q_start = [], [], [0]
    for s, (n, c) in enumerate(zip(new, cached)):
        seq += [s] * n
        pos += list(range(c, c + n))
        q_start.append(q_start[-1] + n)
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    return i32(seq), i32(pos), i32(q_start)


# ---- Dynamic Tanh with the add, the gain and the picked rows -----------------------------------------------------
@pytest.mark.parametrize("dtype,tol", TYPES)
@pytest.mark.parametrize("width", [40, 256, 1000])
def test_dynamic_tanh_adds_with_a_gain(dtype, tol, width):
    from inferx_amd import ops
    T = 7
    h, delta = rnd((T, width), 1, 2.0), rnd((T, width), 2, 1.0, dtype)
    gain, w, b = rnd((width,), 3) + 1.0, rnd((width,), 4) + 1.0, rnd((width,), 5, 0.3)
    alpha = 0.7
    want_h = h.to(F64) + gain.to(F64) * delta.to(F64)
    want = pp.dynamic_tanh(want_h, w.to(F64), b.to(F64), alpha)
    hd = h.to(DEV)
    out = torch.empty((T, width), dtype=dtype, device=DEV)
    ops.add_dyt(hd, delta.to(DEV), gain.to(DEV), w.to(DEV), b.to(DEV), alpha, out)
    close(out, want, tol, "normalised rows")
    close(hd, want_h, 1e-6, "the stream after the add")
    # picked rows: the stream stays as it is
    hd = h.to(DEV)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    out = torch.empty((3, width), dtype=dtype, device=DEV)
    ops.add_dyt(hd, delta.to(DEV), gain.to(DEV), w.to(DEV), b.to(DEV), alpha, out, rows)
    close(out, want[[5, 0, 5]], tol, "picked rows")
    assert torch.equal(hd.cpu(), h)
    # no delta, no gain, no bias
    out = torch.empty((T, width), dtype=dtype, device=DEV)
    ops.add_dyt(hd, None, None, w.to(DEV), None, alpha, out)
    close(out, torch.tanh(alpha * h.to(F64)) * w.to(F64), tol, "without delta and bias")


def test_gain_alone():
    from inferx_amd import ops
    for dtype, tol in TYPES:
        x, gain = rnd((5, 72), 1, 1.0, dtype), rnd((72,), 2)
        out = torch.empty_like(x, device=DEV)
        ops.scale_columns(x.to(DEV), gain.to(DEV), out)
        close(out, x.to(F64) * gain.to(F64), tol, "gain")


# ---- the token shift: alone and inside the norm's kernel, over steps -----------------------------------------
def shift_reference(rows_by_request, mix):
    return [pp.token_shift(x, mix) for x in rows_by_request]


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("dtype,tol", TYPES)
def test_token_shift_over_steps(dtype, tol, fused):
    """Three requests whose rows come in steps of unequal portions (one token, two, many; a request left out of a
    step; a request that starts later in a slot that another one used).  Whatever the cut, row t is blended with the
    original row t-1 of its own sequence, and the first row with zeros."""
    from inferx_amd import ops
    W = 136
    mix = torch.rand(W, generator=torch.Generator().manual_seed(5))
    lengths = [9, 4, 6]
    w, b, alpha = rnd((W,), 7) + 1.0, rnd((W,), 8, 0.2), 0.9
    streams = [rnd((n, W), 10 + i, 1.5) for i, n in enumerate(lengths)]
    if fused:
        normal = [pp.dynamic_tanh(s.to(F64), w.to(F64), b.to(F64), alpha) for s in streams]
    else:
        streams = [s.to(dtype) for s in streams]
        normal = [s.to(F64) for s in streams]
    want = shift_reference(normal, mix.to(F64))
    state = torch.full((2, W), float("nan"), device=DEV)  # two slots; what they hold at a start must not matter
    slot_of = {0: 0, 1: 1, 2: 1}  # request 2 takes request 1's slot after it ended
    # (request, rows) per step
    steps = [[(0, 2), (1, 1)], [(0, 1), (1, 3)], [(0, 5), (2, 2)], [(2, 1)], [(0, 1), (2, 3)]]
    fed = {0: 0, 1: 0, 2: 0}
    got = {r: [] for r in fed}
    for step in steps:
        reqs = [r for r, _ in step]
        new = [n for _, n in step]
        seq, pos, q_start = step_arrays(new, [fed[r] for r in reqs])
        slots = torch.tensor([slot_of[r] for r in reqs], dtype=torch.int32, device=DEV)
        x = torch.cat([streams[r][fed[r]:fed[r] + n] for r, n in step]).to(DEV)
        operands = ops.ShiftOperands(mix.to(DEV), state, seq, q_start, slots, pos)
        out = torch.empty((x.shape[0], W), dtype=dtype, device=DEV)
        if fused:
            moved = torch.empty_like(x)
            ops.add_dyt(x, None, None, w.to(DEV), b.to(DEV), alpha, out, None, h_out=moved, shift=operands)
            assert torch.equal(moved, x)
        else:
            ops.token_shift(x, out, operands)
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n].cpu())
            at += n
            fed[r] += n
    for r in got:
        close(torch.cat(got[r]), want[r], tol, f"request {r}")


# ---- after the product: whole-projection norm, value blend, cache append --------------------------------------
@pytest.mark.parametrize("dtype,tol", TYPES)
@pytest.mark.parametrize("H,G,d,e", [(6, 3, 32, 16), (4, 1, 24, 40), (2, 2, 64, 64)])
def test_norm_blend_and_append(dtype, tol, H, G, d, e):
    from inferx_amd import ops
    T, page, pages = 11, 8, 6
    width = H * d + G * d + G * e
    stride = -(-(width + H) // 16) * 16
    qkv = rnd((T, stride), 1, 1.0, dtype)
    qn, kn = rnd((H * d,), 2) + 1.0, rnd((G * d,), 3) + 1.0
    v_first = rnd((T, G * e), 4, 1.0, dtype)
    lam, eps = 0.3, 1e-3
    slots = torch.randperm(page * pages, generator=torch.Generator().manual_seed(9))[:T].to(torch.int32)
    k_cache = torch.zeros((pages, G, page, d), dtype=dtype, device=DEV)
    v_cache = torch.zeros((pages, G, e, page), dtype=dtype, device=DEV)
    q_out = torch.empty((T, H, d), dtype=dtype, device=DEV)
    v_out = torch.empty((T, G * e), dtype=dtype, device=DEV)
    ops.qk_norm_append(qkv.to(DEV), qn.to(DEV), kn.to(DEV), eps, v_first.to(DEV), lam, v_out, slots.to(DEV), q_out,
                       k_cache, v_cache, H, G, d, e)
    x = qkv.to(F64)
    want_q = pp.rms_norm_whole(x[:, :H * d], qn.to(F64), eps)
    want_k = pp.rms_norm_whole(x[:, H * d:H * d + G * d], kn.to(F64), eps)
    want_v = pp.blend_values(x[:, H * d + G * d:width], v_first.to(F64), lam)
    close(q_out.view(T, -1), want_q, tol, "queries")
    close(v_out, want_v, tol, "blended values")
    got_k = torch.stack([k_cache[int(s) // page, :, int(s) % page, :].reshape(-1) for s in slots])
    got_v = torch.stack([v_cache[int(s) // page, :, :, int(s) % page].reshape(-1) for s in slots])
    close(got_k, want_k, tol, "cached keys")
    close(got_v, want_v, tol, "cached values")
    # without norm and blend the numbers pass through
    ops.qk_norm_append(qkv.to(DEV), None, None, eps, None, 0.0, None, slots.to(DEV), q_out, k_cache, v_cache, H, G, d, e)
    close(q_out.view(T, -1), x[:, :H * d], tol, "queries as they are")


# ---- attention ------------------------------------------------------------------------------------------------
def paged(keys, values, page, seed, dtype):
    """Lay the sequences' keys [T, G, d] and values [T, G, e] into shuffled pages; returns the caches and the table."""
    need = [-(-k.shape[0] // page) for k in keys]
    total = sum(need) + 3
    order = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
    G, d, e = keys[0].shape[1], keys[0].shape[2], values[0].shape[2]
    k_cache = torch.full((total, G, page, d), float("nan"), dtype=dtype)
    v_cache = torch.full((total, G, e, page), float("nan"), dtype=dtype)
    table = torch.full((len(keys), max(need) + 1), -1, dtype=torch.int32)
    for s, (k, v) in enumerate(zip(keys, values)):
        for j in range(need[s]):
            pg = order.pop()
            table[s, j] = pg
            n = min(page, k.shape[0] - j * page)
            k_cache[pg, :, :n, :] = k[j * page:j * page + n].transpose(0, 1).to(dtype)
            v_cache[pg, :, :, :n] = v[j * page:j * page + n].permute(1, 2, 0).to(dtype)
            # what lies behind a sequence's end in its last page is never read: NaN stays there
    return k_cache.to(DEV), v_cache.to(DEV), table.to(DEV)


def attention_reference(q, k, v, talk, sink, gate, scale):
    """All rows of one sequence: q [T, H, d] (float64) -> [T, H, e]."""
    s = pp.raw_scores(q, k, scale)
    if talk is not None:
        s = pp.mix_heads(s, talk)
    out = pp.weighted_values(pp.softmax_with_sink(s, sink), v)
    if gate is not None:
        out = out * torch.sigmoid(gate).unsqueeze(-1)
    return out


def run_attention(kernel, q_rows, k_cache, v_cache, table, seq, pos, talk, sink, gate, scale, e, q_start=None):
    from inferx_amd import ops
    T, H, _ = q_rows.shape
    out = torch.empty((T, H, e), dtype=q_rows.dtype, device=DEV)
    dev = lambda t: None if t is None else t.to(DEV)
    if kernel == "plain":
        ops.attention_talk_plain(q_rows.to(DEV), k_cache, v_cache, table, seq, pos, out, dev(talk), dev(sink), dev(gate),
                                 scale)
    else:
        starts = q_start.tolist()
        tiles = [(s, r0, min(16, starts[s + 1] - r0)) for s in range(len(starts) - 1)
                 for r0 in range(starts[s], starts[s + 1], 16)]
        tiles = torch.tensor(tiles, dtype=torch.int32).T.contiguous().to(DEV)
        outs = []
        for n_splits in (1, 4):  # the keys whole, and in slices whose parts a second kernel merges
            work = torch.empty(T * H * n_splits * (e + 2), dtype=torch.float32, device=DEV) if n_splits > 1 else None
            o = torch.full_like(out, float("nan"))
            ops.attention_talk_mfma(q_rows.to(DEV), k_cache, v_cache, table, tiles, pos, o, n_splits, work, dev(talk),
                                    dev(sink), dev(gate), scale)
            outs.append(o.cpu())
        return outs
    return [out.cpu()]


KERNELS = [("plain", torch.float32, 3e-6), ("plain", torch.bfloat16, 8e-3), ("mfma", torch.bfloat16, 8e-3)]
SHAPES = [(6, 3, 32, 16), (4, 1, 16, 48), (2, 2, 64, 64), (8, 2, 128, 128), (1, 1, 16, 16), (5, 5, 24, 40),
          (16, 4, 128, 128), (32, 8, 64, 32), (12, 12, 48, 80), (4, 4, 256, 64)]


def mfma_takes(H, G, d, e, page):
    from inferx_amd import ops
    return ops.attention_talk_mfma_heads_per_wave(H, G, d, e, page) > 0


@pytest.mark.parametrize("kernel,dtype,tol", KERNELS)
@pytest.mark.parametrize("H,G,d,e", SHAPES)
@pytest.mark.parametrize("options", ["all", "none", "talk", "sink", "gate"])
def test_attention_of_a_step(kernel, dtype, tol, H, G, d, e, options):
    """Two prompt portions on contexts (one starts at 0, one ends inside a page), and three single tokens, one of
    them a sequence's very first token, in one step; every option alone and all together."""
    page = 16
    if kernel == "mfma" and not mfma_takes(H, G, d, e, page):
        pytest.skip("sizes that the matrix-core kernel leaves to the plain one")
    lengths, new = [37, 150, 1, 64, 90], [37, 21, 1, 1, 1]
    scale = 1.0 / math.sqrt(d)
    qs = [rnd((n, H, d), 20 + i, 1.0, dtype) for i, n in enumerate(lengths)]
    ks = [rnd((n, G, d), 30 + i, 1.0, dtype) for i, n in enumerate(lengths)]
    vs = [rnd((n, G, e), 40 + i, 1.0, dtype) for i, n in enumerate(lengths)]
    gs = [rnd((n, H), 50 + i, 2.0, dtype) for i, n in enumerate(lengths)]
    talk = (torch.eye(H) + rnd((H, H), 3, 0.4)) if options in ("all", "talk") else None
    sink = rnd((H,), 4, 1.5) if options in ("all", "sink") else None
    use_gate = options in ("all", "gate")
    k_cache, v_cache, table = paged(ks, vs, page, 1, dtype)
    seq, pos, q_start = step_arrays(new, [l - n for l, n in zip(lengths, new)])
    q_rows = torch.cat([q[l - n:] for q, l, n in zip(qs, lengths, new)])
    gate = torch.cat([g[l - n:] for g, l, n in zip(gs, lengths, new)]) if use_gate else None
    wants = [attention_reference(qs[i].to(F64), ks[i].to(F64), vs[i].to(F64), None if talk is None else talk.to(F64),
                                 None if sink is None else sink.to(F64), gs[i].to(F64) if use_gate else None, scale)
             for i in range(len(lengths))]
    for got in run_attention(kernel, q_rows, k_cache, v_cache, table, seq, pos, talk, sink, gate, scale, e, q_start):
        at = 0
        for i, (l, n) in enumerate(zip(lengths, new)):
            close(got[at:at + n], wants[i][l - n:], tol, f"request {i}")
            at += n


@pytest.mark.parametrize("kernel,dtype,tol", KERNELS)
@pytest.mark.parametrize("where", [0, 1, 15, 16, 17, 127, 128, 511, 512, 900, 1022, 1023])
def test_one_key_that_must_be_found(kernel, dtype, tol, where):
    """Among 1,024 keys one lines up with the query of head 1 (its score stands out by far) and carries a value that
    no other key has; the sink is small.  Whichever key it is -- the first, the last, the query's own, at the edge of
    a page or of a chunk of keys -- head 1's result is that value, as a single token and as the last row of a portion.
    The mixing matrix hands head 1's score on to head 0 and leaves head 2 alone."""
    H, G, d, e, page, T = 3, 1, 32, 16, 16, 1024
    k = rnd((T, G, d), 1, 0.05, dtype)
    q = rnd((T, H, d), 2, 0.05, dtype)
    v = rnd((T, G, e), 3, 0.1, dtype)
    direction = torch.nn.functional.normalize(rnd((d,), 4), dim=0)
    k[where, 0] = (direction * 6.0).to(dtype)
    q[T - 1, 1] = (direction * 6.0).to(dtype)
    v[where, 0] = torch.full((e,), 3.0).to(dtype)
    talk = torch.tensor([[0.0, 1.0, 0.0], [0.0, 1.0, 0.0], [0.0, 0.0, 1.0]])
    sink = torch.tensor([-2.0, -2.0, -2.0])
    k_cache, v_cache, table = paged([k], [v], page, 2, dtype)
    want = attention_reference(q.to(F64), k.to(F64), v.to(F64), talk.to(F64), sink.to(F64), None, 1.0)
    assert float(want[T - 1, 1].min()) > 2.9 and float(want[T - 1, 0].min()) > 2.9 and float(want[T - 1, 2].abs().max()) < 0.5
    for new in (1, 40):
        seq, pos, q_start = step_arrays([new], [T - new])
        for got in run_attention(kernel, q[T - new:], k_cache, v_cache, table, seq, pos, talk, sink, None, 1.0, e, q_start):
            close(got, want[T - new:], tol, f"{new} rows")
            assert float(got[-1, 1].min()) > 2.9 and float(got[-1, 0].min()) > 2.9


@pytest.mark.parametrize("kernel,dtype,tol", KERNELS)
def test_a_sink_that_outweighs_every_key(kernel, dtype, tol):
    """With a large sink a head's weights add up to far less than one; leaving the sink out, or counting it per key,
    would show at once.  Head 0 has the large sink, head 1 a very small one."""
    H, G, d, e, page = 2, 1, 16, 16, 16
    for T in (1, 5, 33):
        q, k = rnd((T, H, d), 1, 0.3, dtype), rnd((T, G, d), 2, 0.3, dtype)
        v = torch.ones((T, G, e), dtype=dtype)
        sink = torch.tensor([4.0, -30.0])
        k_cache, v_cache, table = paged([k], [v], page, 3, dtype)
        seq, pos, q_start = step_arrays([T], [0])
        want = attention_reference(q.to(F64), k.to(F64), v.to(F64), None, sink.to(F64), None, 1.0)
        for got in run_attention(kernel, q, k_cache, v_cache, table, seq, pos, None, sink, None, 1.0, e, q_start):
            close(got, want, tol, f"{T} rows")
            assert float(got[-1, 0].max()) < 0.5 and abs(float(got[-1, 1].mean()) - 1.0) < 1e-2
