"""Every mechanism of the Dezudra design alone: the framework's kernels against the plain functions of
`plain_dezudra.py`, on sizes and inputs made here."""
import math

import numpy as np
import pytest
import torch

import plain_dezudra as pd

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64
TYPES = [(torch.float32, 3e-6), (torch.bfloat16, 8e-3)]


def rnd(shape, seed, std=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def f64(t):
    return t.detach().cpu().to(F64).numpy()


def close(got, want, tol, what):
    want = np.asarray(want)
    scale = max(float(np.abs(want).max()), 1e-6)
    err = float(np.abs(f64(got) - want).max()) / scale
    assert err <= tol, f"{what}: error {err:.3e} of the largest value, tolerance {tol:.1e}"


def i32(a):
    return torch.tensor(a, dtype=torch.int32, device=DEV)


def step_arrays(new, cached):
    """The device arrays of a step in which request s brings new[s] tokens after cached[s]."""
    seq, pos, q_start = [], [], [0]
    for s, (n, c) in enumerate(zip(new, cached)):
        seq += [s] * n
        pos += list(range(c, c + n))
        q_start.append(q_start[-1] + n)
    return i32(seq), i32(pos), i32(q_start)


# requests 0, 1, 2 in steps of unequal portions: one token, two, many; a request left out of a step; request 2 starts
# later, in the slot that request 1 used
STEPS = [[(0, 2), (1, 1)], [(0, 1), (1, 3)], [(0, 7), (2, 2)], [(2, 1)], [(0, 1), (2, 3)], [(0, 2), (2, 9)]]
LENGTHS = [13, 4, 15]
SLOT_OF = {0: 0, 1: 1, 2: 1}


def run_in_steps(run_step, state_tensors):
    """Feeds the three requests through `run_step(step rows by request, seq, pos, q_start, slots)` and returns
    what it gave, put together per request."""
    fed = {0: 0, 1: 0, 2: 0}
    got = {r: [] for r in fed}
    for step in STEPS:
        reqs, new = [r for r, _ in step], [n for _, n in step]
        for r in reqs:
            if fed[r] == 0:  # what the runner does for a request that starts: its slot is cleared
                for st in state_tensors:
                    st[SLOT_OF[r]].zero_()
        seq, pos, q_start = step_arrays(new, [fed[r] for r in reqs])
        out = run_step([(r, fed[r], n) for r, n in step], seq, pos, q_start, i32([SLOT_OF[r] for r in reqs]))
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n])
            at += n
            fed[r] += n
    assert [fed[r] for r in range(3)] == LENGTHS
    return {r: torch.cat(v) for r, v in got.items()}


# ---- the norm of a branch's result, the add and the next norm in one kernel --------------------------------------
@pytest.mark.parametrize("dtype,tol", TYPES)
@pytest.mark.parametrize("width", [40, 258, 1000])
def test_normed_branch_add_and_norm(dtype, tol, width):
    from inferx_amd import ops
    T = 7
    h, delta = rnd((T, width), 1, 2.0), rnd((T, width), 2, 3.0, dtype)
    wd, w = rnd((width,), 3) + 1.0, rnd((width,), 4) + 1.0
    eps_d, eps = 1e-5, 1e-3
    want_h = f64(h) + pd.rms_norm(f64(delta), f64(wd), eps_d)
    want = pd.rms_norm(want_h, f64(w), eps)
    hd = h.to(DEV)
    out = torch.empty((T, width), dtype=dtype, device=DEV)
    ops.add_normed_rmsnorm(hd, delta.to(DEV), wd.to(DEV), eps_d, w.to(DEV), out, eps)
    close(out, want, tol, "normalised rows")
    close(hd, want_h, 2e-6, "the stream after the add")
    hd = h.to(DEV)
    rows = i32([5, 0, 5])
    out = torch.empty((3, width), dtype=dtype, device=DEV)
    ops.add_normed_rmsnorm(hd, delta.to(DEV), wd.to(DEV), eps_d, w.to(DEV), out, eps, rows)
    close(out, want[[5, 0, 5]], tol, "picked rows")
    assert torch.equal(hd.cpu(), h)
    hd = h.to(DEV)
    ops.add_normed_rmsnorm(hd, delta.to(DEV), wd.to(DEV), eps_d, None, None, eps)
    close(hd, want_h, 2e-6, "the add alone")


@pytest.mark.parametrize("dtype,tol", TYPES)
@pytest.mark.parametrize("width,k", [(40, 1), (258, 3), (1000, 4)])
def test_experts_sum_normed_added_and_normed(dtype, tol, width, k):
    """The weighted sum of the chosen experts' rows, its own norm, the add and the next norm in one kernel."""
    from inferx_amd import ops
    T = 6
    h = rnd((T, width), 1, 2.0)
    y = rnd((T * k, width), 2, 1.0, dtype)
    g = torch.Generator().manual_seed(3)
    dest = torch.randperm(T * k, generator=g).to(torch.int32)
    topk_w = torch.rand((T, k), generator=g)
    wd, w = rnd((width,), 4) + 1.0, rnd((width,), 5) + 1.0
    eps_d, eps = 1e-5, 1e-4
    f = np.einsum("tk,tkw->tw", f64(topk_w), f64(y)[dest.long().numpy()].reshape(T, k, width))
    want_h = f64(h) + pd.rms_norm(f, f64(wd), eps_d)
    want = pd.rms_norm(want_h, f64(w), eps)
    hd = h.to(DEV)
    out = torch.empty((T, width), dtype=dtype, device=DEV)
    ops.moe_combine_add_rmsnorm(hd, y.to(DEV), dest.to(DEV), topk_w.to(DEV), None, None, w.to(DEV), out, eps,
                                sum_weight=wd.to(DEV), sum_eps=eps_d)
    close(out, want, tol, "normalised rows")
    close(hd, want_h, 2e-6, "the stream after the add")
    hd = h.to(DEV)
    rows = i32([4, 1])
    out = torch.empty((2, width), dtype=dtype, device=DEV)
    ops.moe_combine_add_rmsnorm(hd, y.to(DEV), dest.to(DEV), topk_w.to(DEV), None, None, w.to(DEV), out, eps, rows,
                                sum_weight=wd.to(DEV), sum_eps=eps_d)
    close(out, want[[4, 1]], tol, "picked rows")
    assert torch.equal(hd.cpu(), h)


# ---- the short convolution over steps, with silu, with rotation, into pages --------------------------------------
@pytest.mark.parametrize("eights", [False, True])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("dtype,tol", TYPES)
def test_short_convolution_over_steps(dtype, tol, taps, eights):
    """Whatever the cut, row t reads the rows t - taps + 1 .. t of its own sequence and zeros before its start; the
    state starts as not-a-number and is cleared when a request starts."""
    from inferx_amd import ops
    # q: two heads of 12, k: one, v: three of 20; or everything in eights (the kernel's 16-byte form in bfloat16)
    sizes = (2 * 16, 16, 3 * 24, 16, 24) if eights else (2 * 12, 12, 3 * 20, 12, 20)
    C = sizes[0] + sizes[1] + sizes[2]
    extra = 8 if eights else 5  # the projection's rows are wider than the convolved channels
    w = rnd((C, taps), 3, 0.5, dtype)
    bias = rnd((C,), 4, 0.5, dtype)
    xs = [rnd((n, C + extra), 10 + r, 1.0, dtype) for r, n in enumerate(LENGTHS)]
    state = torch.full((2, max(1, (taps - 1) * C) + (4 if eights else 3)), float("nan"), device=DEV)
    want = {r: pd.silu(pd.short_conv(f64(xs[r])[:, :C] + f64(bias), f64(w))) for r in range(3)}
    fast = dict(weight_t=w.to(DEV).float().t().contiguous(), bias_f32=bias.to(DEV).float()) if eights else {}

    def run_step(parts, seq, pos, q_start, slots):
        x = torch.cat([xs[r][a:a + n] for r, a, n in parts]).to(DEV)
        T = x.shape[0]
        q, k, v = (torch.empty((T, c), dtype=dtype, device=DEV) for c in sizes[:3])
        ops.short_conv(x, bias.to(DEV), w.to(DEV), state, ops.StepRows(seq, q_start, slots), sizes, q, k, v, silu=True,
                       **fast)
        return torch.cat([q, k, v], dim=1).cpu()

    got = run_in_steps(run_step, [state])
    for r in range(3):
        close(got[r], want[r], tol, f"request {r}, {taps} taps")


@pytest.mark.parametrize("D,V,rot", [(12, 20, 0), (12, 20, 4), (12, 20, 12), (16, 24, 0), (32, 8, 16), (32, 40, 32)])
@pytest.mark.parametrize("dtype,tol", TYPES)
def test_short_convolution_rotates_and_appends(dtype, tol, D, V, rot):
    """The convolved keys and values land in the request's pages (keys rotated, values transposed within a page),
    the queries in rows; pairs (i, i + rot / 2) of every head's first `rot` elements are rotated by the position."""
    from inferx_amd import ops
    page = 4
    sizes = (2 * D, 2 * D, V, D, V)  # (sizes in eights go through the kernel's 16-byte form in bfloat16)
    C, taps = sizes[0] + sizes[1] + sizes[2], 3
    w = rnd((C, taps), 3, 0.5, dtype)
    xs = [rnd((n, C), 20 + r, 1.0, dtype) for r, n in enumerate(LENGTHS)]
    state = torch.full((2, (taps - 1) * C), float("nan"), device=DEV)
    k_cache = torch.zeros((16, 2, page, D), dtype=dtype, device=DEV)
    v_cache = torch.zeros((16, 1, V, page), dtype=dtype, device=DEV)
    pages = {0: [5, 2, 9, 11], 1: [7], 2: [0, 7, 3, 14]}  # request 2 uses request 1's page again
    inv_freq = torch.tensor([50.0 ** (-2.0 * j / rot) for j in range(rot // 2)], dtype=torch.float32, device=DEV) if rot else None
    want = {}
    for r in range(3):
        y = pd.short_conv(f64(xs[r]), f64(w))
        posn = np.arange(LENGTHS[r])
        q = pd.rotate(y[:, :2 * D].reshape(-1, 2, D), posn, rot, 50.0).reshape(-1, 2 * D)
        k = pd.rotate(y[:, 2 * D:4 * D].reshape(-1, 2, D), posn, rot, 50.0).reshape(-1, 2 * D)
        want[r] = np.concatenate([q, k, y[:, 4 * D:]], axis=1)

    def run_step(parts, seq, pos, q_start, slots):
        x = torch.cat([xs[r][a:a + n] for r, a, n in parts]).to(DEV)
        T = x.shape[0]
        where = i32([pages[r][(a + i) // page] * page + (a + i) % page for r, a, n in parts for i in range(n)])
        table = None
        if rot:
            table = torch.empty((T, rot // 2, 2), dtype=torch.float32, device=DEV)
            ops.rope_table(table, pos, inv_freq)
        q = torch.empty((T, 2 * D), dtype=dtype, device=DEV)
        ops.short_conv(x, None, w.to(DEV), state, ops.StepRows(seq, q_start, slots), sizes, q, k_cache, v_cache,
                       slots=where, cos_sin=table, weight_t=w.to(DEV).float().t().contiguous())
        # read this step's keys and values back from the pages
        flat = where.long()
        k = k_cache.permute(0, 2, 1, 3).reshape(-1, 2 * D)[flat]
        v = v_cache.permute(0, 3, 1, 2).reshape(-1, V)[flat]
        return torch.cat([q, k, v], dim=1).cpu()

    got = run_in_steps(run_step, [state])
    for r in range(3):
        close(got[r], want[r], tol, f"request {r}, {rot} rotated")


# ---- the gated delta rule over steps ------------------------------------------------------------------------------
def plain_delta(q, k, v, a, b, a_log, dt_bias, heads, kv_heads, dim, vdim):
    """The recurrence of `plain_dezudra.delta_mixer`, on its operands (float64 arrays)."""
    T = q.shape[0]
    q = q.reshape(T, kv_heads, dim)
    k = k.reshape(T, kv_heads, dim)
    v = v.reshape(T, heads, vdim)
    q = q / np.sqrt(np.sum(q * q, axis=-1, keepdims=True) + 1e-6) * dim ** -0.5
    k = k / np.sqrt(np.sum(k * k, axis=-1, keepdims=True) + 1e-6)
    beta = 1.0 / (1.0 + np.exp(-b))
    g = np.exp(-np.exp(a_log)[None, :] * pd.softplus(a + dt_bias[None, :]))
    o = np.zeros((T, heads, vdim))
    for hd in range(heads):
        kv = hd // (heads // kv_heads)
        S = np.zeros((dim, vdim))
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + np.outer(k[t, kv], u)
            o[t, hd] = S.T @ q[t, kv]
    return o


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 32, 48), (3, 1, 20, 12), (1, 1, 128, 16), (2, 2, 7, 70),
                                                     (2, 1, 200, 17), (2, 1, 64, 40), (1, 1, 96, 32), (2, 2, 128, 20)])
@pytest.mark.parametrize("dtype,tol", TYPES)
def test_delta_rule_over_steps(dtype, tol, heads, kv_heads, dim, vdim):
    from inferx_amd import ops
    qs = [rnd((n, kv_heads * dim), 30 + r, 1.0, dtype) for r, n in enumerate(LENGTHS)]
    ks = [rnd((n, kv_heads * dim), 40 + r, 1.0, dtype) for r, n in enumerate(LENGTHS)]
    vs = [rnd((n, heads * vdim), 50 + r, 1.0, dtype) for r, n in enumerate(LENGTHS)]
    abs_ = [rnd((n, 2 * heads), 60 + r, 1.5) for r, n in enumerate(LENGTHS)]
    a_log, dt_bias = rnd((heads,), 5, 0.7), rnd((heads,), 6, 0.7)
    # (blocks of a multiple of four numbers let the kernel read the state in 16-byte pieces: both ways are run)
    state = torch.full((2, heads * dim * vdim + (12 if vdim % 16 == 0 else 11)), float("nan"), device=DEV)
    want = {r: plain_delta(f64(qs[r]), f64(ks[r]), f64(vs[r]), f64(abs_[r])[:, :heads], f64(abs_[r])[:, heads:],
                           f64(a_log), f64(dt_bias), heads, kv_heads, dim, vdim) for r in range(3)}

    def run_step(parts, seq, pos, q_start, slots):
        cat = lambda xs: torch.cat([xs[r][a:a + n] for r, a, n in parts]).to(DEV)
        q, k, v, ab = cat(qs), cat(ks), cat(vs), cat(abs_)
        out = torch.empty((q.shape[0], heads, vdim), dtype=torch.float32, device=DEV)
        ops.delta_rule(q, k, v, ab, a_log.to(DEV), dt_bias.to(DEV), state, ops.StepRows(seq, q_start, slots), out,
                       heads, kv_heads, dim, vdim)
        return out.cpu()

    got = run_in_steps(run_step, [state])
    for r in range(3):
        close(got[r], want[r], tol, f"request {r}")


def test_delta_rule_keeps_what_was_written_long_ago():
    """A key written at the first token and never touched again (all later keys are orthogonal to it, no decay) is
    read back 300 tokens later, through steps of one token; with a decay it has faded by exactly the product of the
    decays."""
    from inferx_amd import ops
    dim, vdim, T = 16, 8, 300
    k = torch.zeros((T, dim))
    k[0, 3] = 1.0
    k[1:, 5] = 1.0
    q = torch.zeros((T, dim))
    q[:, 3] = 1.0
    v = rnd((T, vdim), 1)
    for decay_logit, faded in ((-60.0, 1.0), (-5.0, None)):
        ab = torch.zeros((T, 2))
        ab[:, 0] = decay_logit   # softplus(-60) = 0: no decay
        ab[:, 1] = 60.0          # beta = 1
        a_log, dt_bias = torch.zeros(1), torch.zeros(1)
        state = torch.zeros((1, dim * vdim), device=DEV)
        outs = []
        for t in range(T):
            seq, pos, q_start = step_arrays([1], [t])
            out = torch.empty((1, 1, vdim), dtype=torch.float32, device=DEV)
            ops.delta_rule(q[t:t + 1].to(DEV), k[t:t + 1].to(DEV), v[t:t + 1].to(DEV), ab[t:t + 1].to(DEV),
                           a_log.to(DEV), dt_bias.to(DEV), state, ops.StepRows(seq, q_start, i32([0])), out, 1, 1, dim, vdim)
            outs.append(out.cpu()[0, 0])
        g = math.exp(-math.log1p(math.exp(decay_logit)))
        for t in (0, 1, 150, 299):
            factor = g ** t if faded is None else 1.0
            close(outs[t], f64(v[0]) * factor / math.sqrt(dim) * (1.0 / math.sqrt(1 + 1e-6)) ** 2, 1e-5, f"token {t}")


# ---- the norm per head, the gate, the difference --------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", TYPES)
@pytest.mark.parametrize("heads,vdim", [(3, 12), (2, 64), (1, 200)])
def test_head_norm_with_gate_and_with_difference(dtype, tol, heads, vdim):
    from inferx_amd import ops
    T = 9
    x, x2 = rnd((T, heads, vdim), 1), rnd((T, heads, vdim), 2)
    w = rnd((vdim,), 3, 0.3, dtype) + 1.0
    wide = rnd((T, heads * vdim + 6), 4, 1.0, dtype)
    gate = wide[:, 6:]
    out = torch.empty((T, heads * vdim), dtype=dtype, device=DEV)
    ops.head_norm_gate(x.to(DEV), out, 1e-5, weight=w.to(DEV), gate=wide.to(DEV)[:, 6:])
    want = pd.rms_norm(f64(x), f64(w), 1e-5) * pd.silu(f64(gate)).reshape(T, heads, vdim)
    close(out, want.reshape(T, -1), tol, "norm, weight and gate")
    ops.head_norm_gate(x.to(DEV), out, 1e-4, x2=x2.to(DEV), lam=0.37, mult=0.6)
    want = pd.rms_norm(f64(x) - 0.37 * f64(x2), None, 1e-4) * 0.6
    close(out, want.reshape(T, -1), tol, "difference and norm")


# ---- differential attention over pages --------------------------------------------------------------------------------
def plain_diff_attention(q, k, v, positions, scale, window, keep_first, lam, eps, mult):
    """q [T, H, 2, D] at `positions` of one sequence whose keys k [L, G, 2, D] and values v [L, G, V] are all there."""
    T, H, _, D = q.shape
    L, G, V = v.shape
    out = np.zeros((T, H, V))
    j = np.arange(L)
    for t in range(T):
        p = positions[t]
        see = (j <= p) & (((p - j < window) | (j < keep_first)) if window > 0 else True)
        for h in range(H):
            g = h // (H // G)
            a = []
            for m in range(2):
                s = k[:, g, m] @ q[t, h, m] * scale
                s = np.where(see, s, -np.inf)
                e = np.exp(s - s.max())
                a.append((e / e.sum()) @ v[:, g])
            o = a[0] - lam * a[1]
            out[t, h] = o / np.sqrt(np.mean(o * o) + eps) * mult
    return out


def paged(k, v, page, dtype, seed=0):
    """Keys [L, G2, D] and values [L, G, V] of one request in pages handed out in a shuffled order; what the pages
    hold elsewhere is not-a-number."""
    L = k.shape[0]
    n = -(-L // page)
    order = torch.randperm(n + 3, generator=torch.Generator().manual_seed(seed))[:n].tolist()
    kc = torch.full((n + 3, k.shape[1], page, k.shape[2]), float("nan"), dtype=dtype)
    vc = torch.full((n + 3, v.shape[1], v.shape[2], page), float("nan"), dtype=dtype)
    for j in range(L):
        kc[order[j // page], :, j % page] = k[j]
        vc[order[j // page], :, :, j % page] = v[j]
    return kc.to(DEV), vc.to(DEV), i32([order])


@pytest.mark.parametrize("dtype,tol", TYPES)
@pytest.mark.parametrize("H,G,D,V,window,keep", [(4, 2, 32, 32, 24, 3), (3, 1, 12, 20, 0, 0), (2, 2, 16, 48, 9, 0),
                                                 (1, 1, 16, 16, 1, 2), (4, 1, 64, 96, 33, 40), (6, 3, 20, 12, 17, 5)])
def test_differential_attention(dtype, tol, H, G, D, V, window, keep):
    """A portion of queries at the end of a context and single queries elsewhere, against attention over all keys."""
    from inferx_amd import ops
    L, page = 150, 16
    k, v = rnd((L, 2 * G, D), 1, 1.0, dtype), rnd((L, G, V), 2, 1.0, dtype)
    positions = [0, 1, keep, max(window - 1, 0), window, window + keep, 70, 99] + list(range(120, 150))
    q = rnd((len(positions), H, 2, D), 3, 1.0, dtype)
    kc, vc, table = paged(k, v, page, dtype)
    out = torch.empty((len(positions), H, V), dtype=dtype, device=DEV)
    lam, eps, mult = 0.45, 1e-5, 0.7
    ops.attention_diff_plain(q.to(DEV), kc, vc, table, i32([0] * len(positions)), i32(positions), out, 0.3, window, keep,
                             lam, eps, mult)
    want = plain_diff_attention(f64(q), f64(k).reshape(L, G, 2, D), f64(v), positions, 0.3, window, keep, lam, eps, mult)
    close(out, want, tol, "differential attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_key_stands_out_at_every_edge(dtype):
    """Map 0 of the queries points at ONE key with a score far above the others, so the result is that key's value
    (normalised) if the key is seen and something else if it is not: keys just inside and just outside the window,
    the kept first tokens and the ones after them, page borders, far keys; for queries at many positions."""
    from inferx_amd import ops
    H, G, D, V, L, page = 2, 1, 16, 24, 1100, 16
    window, keep = 37, 5
    k = rnd((L, 2 * G, D), 1, 0.05)
    v = rnd((L, G, V), 2, 1.0)
    mark = torch.zeros(D)
    mark[7] = 1.0
    lam, eps, mult = 0.0, 1e-6, 1.0  # lambda 0: the result is map 0's alone
    for pos in (36, 37, 38, 47, 48, 300, 1023, 1024, 1099):
        cases = {0: True, keep - 1: True, keep: pos - keep < window, 15: pos - 15 < window, 16: pos - 16 < window,
                 pos - window + 1: True, pos - window: pos - window < keep, pos - window - 1: pos - window - 1 < keep,
                 pos: True, (pos // page) * page: True, (pos // page) * page - 1: pos - ((pos // page) * page - 1) < window}
        for key, seen in cases.items():
            if key < 0:
                continue
            kk = k.clone()
            kk[key, 0] = mark * 40.0
            q = torch.zeros((1, H, 2, D))
            q[0, :, 0] = mark * 40.0
            kc, vc, table = paged(kk.to(dtype), v.to(dtype), page, dtype, seed=pos)
            out = torch.empty((1, H, V), dtype=dtype, device=DEV)
            ops.attention_diff_plain(q.to(dtype).to(DEV), kc, vc, table, i32([0]), i32([pos]), out, 1.0, window, keep, lam,
                                     eps, mult)
            target = f64(v.to(dtype))[key, 0]
            target = target / np.sqrt(np.mean(target * target) + eps)
            err = float(np.abs(f64(out)[0, 0] - target).max())
            assert (err < 2e-2) == seen, f"query {pos}, key {key}: {'not ' if seen else ''}found (error {err:.2e})"


# ---- experts of squared relu, chosen among groups ---------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", TYPES)
@pytest.mark.parametrize("tokens", [3, 16, 40, 300])
@pytest.mark.parametrize("E,top,groups,keep,ff,width", [(6, 2, 3, 2, 64, 96), (9, 3, 3, 1, 52, 72), (16, 4, 8, 3, 32, 128),
                                                        (4, 4, 2, 2, 40, 40), (5, 1, 1, 1, 36, 72), (2, 1, 2, 1, 24, 40),
                                                        (16, 6, 4, 2, 32, 128), (128, 5, 16, 3, 16, 64)])
def test_experts_chosen_among_groups(dtype, tol, tokens, E, top, groups, keep, ff, width):
    """The feed-forward part as the design builds it, against the plain one: choices (where no near tie), weights and
    the weighted sum; few tokens (the streaming kernels, and the router, selection and grouping in one launch: up to 64
    assignments in registers, more through LDS), some (16-row tiles) and many (tiles through LDS)."""
    from inferx_amd.engine.runtime import Runtime, StepContext
    from inferx_amd.parts.base import resolve_delta
    from inferx_amd.parts.moe import MoeFeedForward
    rt = Runtime("float32" if dtype == torch.float32 else "bfloat16")
    part = MoeFeedForward(width, E, top, ff, gated=False, activation="relu2", groups=groups, groups_keep=keep)
    W = {"router": rnd((E, width), 1, 0.5, dtype)}
    tensors = {"gate.weight": W["router"].to(DEV)}
    for e in range(E):
        W[f"e{e}.up"], W[f"e{e}.down"] = rnd((ff, width), 10 + e, 0.2, dtype), rnd((width, ff), 40 + e, 0.2, dtype)
        tensors[f"experts.{e}.up_proj.weight"] = W[f"e{e}.up"].to(DEV)
        tensors[f"experts.{e}.down_proj.weight"] = W[f"e{e}.down"].to(DEV)
    part.bind(tensors, rt)
    x = rnd((tokens, width), 2, 1.0, dtype)
    ctx = StepContext(rt=rt, num_tokens=tokens, num_requests=1, token_ids=None, positions=None, seq_of_token=None,
                      q_start=None, seq_lens=None, state_slots=None, logits_rows=None, slots=[], block_tables=[])
    topk_w, topk_e, _ = part.route(ctx, x.to(DEV))
    mlp = {"router": {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}}
    Wn = {n: f64(t) for n, t in W.items()}
    margins = []
    s, ids, wts = pd.route(f64(x), mlp["router"], Wn["router"], margins)
    sure = margins[0] > (1e-6 if dtype == torch.float32 else 3e-2)
    assert sure.sum() >= tokens // 3
    assert np.array_equal(topk_e.cpu().numpy()[sure], ids[sure]), "another choice of experts"
    close(topk_w.cpu()[torch.from_numpy(sure)], wts[sure], tol, "weights")
    got = resolve_delta(ctx, part.forward(ctx, x.to(DEV)))
    want = pd.moe(f64(x), mlp, Wn)
    scale = float(np.abs(want).max())
    err = np.abs(f64(got) - want).max(axis=1) / scale
    assert (err[sure] <= (2e-5 if dtype == torch.float32 else 2e-2)).all(), f"weighted sum: {err[sure].max():.2e}"


# ---- the matrix-core kernel of differential attention ----------------------------------------------------------------
def tiles_of(portions):
    """int32 [3, n]: request, first row, rows of tiles of up to 16 queries, for portions [(request, first row, rows)]."""
    t = []
    for req, row0, n in portions:
        for a in range(0, n, 16):
            t.append((req, row0 + a, min(16, n - a)))
    return torch.tensor(t, dtype=torch.int32, device=DEV).t().contiguous()


def mfma_attend(q, kc, vc, table, tiles, positions, n_splits, scale, window, keep, lam, eps, mult, grouped=False):
    from inferx_amd import ops
    T, H = q.shape[0], q.shape[1]
    V = vc.shape[2]
    out = torch.empty((T, H, V), dtype=torch.bfloat16, device=DEV)
    work = torch.full((T * H * 2 * n_splits * (V + 2),), float("nan"), dtype=torch.float32, device=DEV)
    ops.attention_diff_mfma(q.to(DEV), kc, vc, table, tiles, i32(positions), out, n_splits, work, scale, window, keep, lam,
                            eps, mult, grouped=grouped)
    return out


@pytest.mark.parametrize("n_splits", [1, 2, 8])
@pytest.mark.parametrize("H,G,D,V,window,keep", [(4, 2, 32, 32, 24, 3), (3, 1, 16, 48, 0, 0), (2, 2, 16, 48, 9, 0),
                                                 (1, 1, 16, 16, 1, 2), (4, 1, 64, 96, 33, 40), (4, 2, 128, 128, 70, 5),
                                                 (6, 3, 48, 16, 17, 35), (2, 1, 96, 64, 64, 32)])
def test_differential_attention_on_the_matrix_cores(H, G, D, V, window, keep, n_splits):
    """A portion of queries at the end of a context (tiles of 16 and a ragged one), a portion at its very start, and
    single queries elsewhere, with the keys in one slice and in several."""
    dtype = torch.bfloat16
    L, page = 150, 16
    k, v = rnd((L, 2 * G, D), 1, 1.0, dtype), rnd((L, G, V), 2, 1.0, dtype)
    singles = [keep, max(window - 1, 0), window, window + keep, 70, 99]
    positions = list(range(0, 21)) + singles + list(range(111, 150))
    portions = [(0, 0, 21)] + [(0, 21 + i, 1) for i in range(len(singles))] + [(0, 21 + len(singles), 39)]
    q = rnd((len(positions), H, 2, D), 3, 1.0, dtype)
    kc, vc, table = paged(k, v, page, dtype)
    lam, eps, mult = 0.45, 1e-5, 0.7
    out = mfma_attend(q, kc, vc, table, tiles_of(portions), positions, n_splits, 0.3, window, keep, lam, eps, mult)
    want = plain_diff_attention(f64(q), f64(k).reshape(L, G, 2, D), f64(v), positions, 0.3, window, keep, lam, eps, mult)
    close(out, want, 1.5e-2, "differential attention (matrix cores)")


@pytest.mark.parametrize("n_splits", [1, 4])
@pytest.mark.parametrize("H,G,D,V,window,keep", [(4, 2, 32, 32, 24, 3), (16, 1, 64, 32, 0, 0), (6, 2, 16, 96, 44, 3)])
def test_differential_attention_one_token_each_grouped(H, G, D, V, window, keep, n_splits):
    """Three requests of unequal contexts, one token each, the query heads of a key/value head side by side."""
    dtype = torch.bfloat16
    page, lens = 16, [150, 37, 1]
    ks = [rnd((n, 2 * G, D), 10 + i, 1.0, dtype) for i, n in enumerate(lens)]
    vs = [rnd((n, G, V), 20 + i, 1.0, dtype) for i, n in enumerate(lens)]
    pages = sum(-(-n // page) for n in lens)
    kc = torch.full((pages + 2, 2 * G, page, D), float("nan"), dtype=dtype)
    vc = torch.full((pages + 2, G, V, page), float("nan"), dtype=dtype)
    order = torch.randperm(pages + 2, generator=torch.Generator().manual_seed(3)).tolist()
    rows, at = [], 0
    for i, n in enumerate(lens):
        mine = order[at:at + -(-n // page)]
        at += len(mine)
        rows.append(mine + [-1] * (10 - len(mine)))
        for j in range(n):
            kc[mine[j // page], :, j % page] = ks[i][j]
            vc[mine[j // page], :, :, j % page] = vs[i][j]
    q = rnd((3, H, 2, D), 3, 1.0, dtype)
    positions = [n - 1 for n in lens]
    lam, eps, mult = 0.3, 1e-5, 0.5
    tiles = torch.tensor([[0, 1, 2], [0, 1, 2], [1, 1, 1]], dtype=torch.int32, device=DEV)
    out = mfma_attend(q, kc.to(DEV), vc.to(DEV), i32(rows), tiles, positions, n_splits, 0.3, window, keep, lam, eps, mult,
                      grouped=True)
    for i, n in enumerate(lens):
        want = plain_diff_attention(f64(q)[i:i + 1], f64(ks[i]).reshape(n, G, 2, D), f64(vs[i]), [n - 1], 0.3, window, keep,
                                    lam, eps, mult)
        close(out[i:i + 1], want, 1.5e-2, f"request {i}")


@pytest.mark.parametrize("grouped", [False, True])
def test_one_key_stands_out_at_every_edge_on_the_matrix_cores(grouped):
    """As the plain kernel's test: one key far above the others is found exactly where the window and the kept
    first tokens say, also when the pages between them hold not-a-number (they may have been given back)."""
    H, G, D, V, L, page = 2, 1, 16, 32, 1100, 16
    window, keep = 37, 5
    dtype = torch.bfloat16
    k = rnd((L, 2 * G, D), 1, 0.05)
    v = rnd((L, G, V), 2, 1.0)
    mark = torch.zeros(D)
    mark[7] = 1.0
    lam, eps, mult = 0.0, 1e-6, 1.0
    for pos in (36, 37, 38, 47, 48, 300, 1023, 1024, 1099):
        cases = {0: True, keep - 1: True, keep: pos - keep < window, 15: pos - 15 < window, 16: pos - 16 < window,
                 pos - window + 1: True, pos - window: pos - window < keep, pos - window - 1: pos - window - 1 < keep,
                 pos: True, (pos // page) * page: True, (pos // page) * page - 1: pos - ((pos // page) * page - 1) < window}
        for key, seen in cases.items():
            if key < 0:
                continue
            kk, vv = k.clone(), v.clone()
            kk[key, 0] = mark * 40.0
            # whole pages between the kept first tokens' page and the window hold not-a-number
            first_dead, last_dead = 2 * page, ((pos + 1 - window) // page) * page
            if last_dead > first_dead:
                kk[first_dead:last_dead] = float("nan")
                vv[first_dead:last_dead] = float("nan")
            q = torch.zeros((1, H, 2, D))
            q[0, :, 0] = mark * 40.0
            kc, vc, table = paged(kk.to(dtype), vv.to(dtype), page, dtype, seed=pos)
            tiles = torch.tensor([[0], [0], [1]], dtype=torch.int32, device=DEV)
            for n_splits in (1, 4):
                out = mfma_attend(q.to(dtype), kc, vc, table, tiles, [pos], n_splits, 1.0, window, keep, lam, eps, mult,
                                  grouped=grouped)
                target = f64(v.to(dtype))[key, 0]
                target = target / np.sqrt(np.mean(target * target) + eps)
                err = float(np.abs(f64(out)[0, 0] - target).max())
                assert np.isfinite(f64(out)).all(), f"query {pos}, key {key}: not-a-number read"
                assert (err < 3e-2) == seen, f"query {pos}, key {key}, {n_splits} slices: {'not ' if seen else ''}found (error {err:.2e})"


@pytest.mark.parametrize("kernel", ["plain", "matrix cores", "matrix cores, 4 slices"])
def test_one_key_stands_out_for_every_query_of_a_portion(kernel):
    """A prompt portion of 48 queries that all point at ONE key: every query finds it exactly if it sees it (at or
    before its own position, and within its own window or among the kept first tokens), whatever its place in its
    tile of 16; the portion ends at a page's edge, in the middle of a page, and right after the window has filled."""
    from inferx_amd import ops
    H, G, D, V, L, page = 2, 1, 16, 32, 400, 16
    window, keep = 37, 5
    dtype = torch.bfloat16
    k = rnd((L, 2 * G, D), 1, 0.05)
    v = rnd((L, G, V), 2, 1.0)
    mark = torch.zeros(D)
    mark[7] = 1.0
    eps = 1e-6
    for last in (47, 63, 100, 255, 399):
        positions = list(range(last - 47, last + 1))
        for key in (0, keep - 1, keep, last - 47 - window, last - 47 - window + 1, last - window, last - window + 1,
                    last - 60, last - 47, last - 20, last - 16, last - 15, last):
            if key < 0:
                continue
            kk = k.clone()
            kk[key, 0] = mark * 40.0
            q = torch.zeros((48, H, 2, D))
            q[:, :, 0] = mark * 40.0
            kc, vc, table = paged(kk.to(dtype), v.to(dtype), page, dtype, seed=last)
            if kernel == "plain":
                out = torch.empty((48, H, V), dtype=dtype, device=DEV)
                ops.attention_diff_plain(q.to(dtype).to(DEV), kc, vc, table, i32([0] * 48), i32(positions), out, 1.0, window,
                                         keep, 0.0, eps, 1.0)
            else:
                out = mfma_attend(q.to(dtype), kc, vc, table, tiles_of([(0, 0, 48)]), positions, 4 if "slices" in kernel else 1,
                                  1.0, window, keep, 0.0, eps, 1.0)
            target = f64(v.to(dtype))[key, 0]
            target = target / np.sqrt(np.mean(target * target) + eps)
            err = np.abs(f64(out)[:, 0] - target[None, :]).max(axis=1)
            seen = np.array([key <= p and (p - key < window or key < keep) for p in positions])
            assert np.array_equal(err < 3e-2, seen), \
                f"portion ending at {last}, key {key}: queries {np.flatnonzero((err < 3e-2) != seen).tolist()} of the portion are wrong"
