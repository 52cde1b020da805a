"""Per-kernel times of Numalorn's layer kernels at the sizes of a served model's steps
(``bench.py --arch-compare numalorn``): a prefill step of 4,096 rows and a decode step of 64
rows on 4096-wide layers (32 heads over a 512-wide cached latent, 64 recurrent heads of 64,
8 experts of width 14,336 with 2 per token), bf16, random inputs.

Each entry: time (HIP events, median of the repeats), the bytes the kernel has to move and
the arithmetic it has to do, and ``distance`` = time / max(bytes / 8 TB/s, flops / 2.5 PFLOP/s).
"""
from __future__ import annotations

import torch

from .. import ops

HBM, MFMA = 8e12, 2.5e15
DEV = "cuda"


def _time(fn, reps=20, warm=5):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        ts.append(a.elapsed_time(b) * 1e-3)
    ts.sort()
    return ts[len(ts) // 2]


def _entry(t, nbytes, flops):
    floor = max(nbytes / HBM, flops / MFMA)
    return {"us": round(t * 1e6, 1), "mbytes": round(nbytes / 1e6, 1), "gflop": round(flops / 1e9, 2),
            "floor_us": round(floor * 1e6, 2), "distance": round(t / floor, 1)}


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _runs(lens, slots, first=0):
    """Per-row state arrays of runs of the given lengths that start at position ``first``."""
    rs, rb, rf, pos = [], [], [], []
    for n, s in zip(lens, slots):
        rs += [2 * s] * n
        rb += list(range(n))
        rf += list(range(n - 1, -1, -1))
        pos += list(range(first, first + n))
    return _i32(rs), _i32(rb), _i32(rf), _i32(pos)


def _rows(T, d, lens, slots, out, first=0):
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn(T, d, generator=g, device=DEV)
    y = torch.randn(T, d, generator=g, device=DEV).bfloat16()
    w = torch.randn(d, generator=g, device=DEV) * 0.3
    cp = torch.empty(T, d, dtype=torch.bfloat16, device=DEV)
    out["post_norm_add"] = _entry(_time(lambda: ops.post_norm_add(y, x, w, 0.5, 1e-5, cp)), T * d * 12, 0)
    mu = torch.rand(5, d, generator=g, device=DEV)
    prev = torch.zeros(128, d, device=DEV)
    rows = _runs(lens, slots, first)
    mixes = torch.empty(5, T, d, dtype=torch.bfloat16, device=DEV)
    out["token_shift_mix"] = _entry(_time(lambda: ops.token_shift_mix(x, mu, prev, *rows, mixes)), T * d * 14, 0)
    return rows


def _wkv(T, H, N, rows, out, decode):
    g = torch.Generator(device=DEV).manual_seed(1)
    r, k, v, gate, zw = ((torch.randn(T, H * N, generator=g, device=DEV) * 0.5).bfloat16() for _ in range(5))
    w0 = torch.randn(H * N, generator=g, device=DEV) - 2
    u = torch.randn(H, N, generator=g, device=DEV) * 0.3
    nw = torch.ones(H * N, device=DEV)
    st = torch.zeros(128, H, N, N, device=DEV)
    y = torch.empty(T, H * N, dtype=torch.bfloat16, device=DEV)
    run = torch.nonzero(rows[1] == 0)[:, 0].to(torch.int32)       # the runs' first rows
    t = _time(lambda: ops.wkv_recurrence(r, k, v, zw, w0, u, gate, nw, 1e-5, st, *rows, y, run))
    seqs = int(run.numel())
    nbytes = T * H * N * 12 + (2 if decode else 1) * seqs * H * N * N * 4
    out["wkv_recurrence"] = _entry(t, nbytes, 6.0 * T * H * N * N)


def _attention(H, R, lens, q_lens, out, name, mfma=False):
    g = torch.Generator(device=DEV).manual_seed(2)
    BS = 32
    nblk = sum((n + BS - 1) // BS for n in lens) + 1
    pool = (torch.randn(nblk, 1, BS, R, generator=g, device=DEV) * 0.5).bfloat16()
    T = sum(q_lens)
    qa = torch.randn(T, H, R, generator=g, device=DEV) * R ** -0.5
    sink = torch.randn(H, generator=g, device=DEV)
    maxb = (max(lens) + BS - 1) // BS
    tables, at = [], 0
    for n in lens:
        nb = (n + BS - 1) // BS
        tables.append(list(range(at, at + nb)) + [nblk - 1] * (maxb - nb))
        at += nb
    starts = [sum(q_lens[:i]) for i in range(len(lens))]
    lat = torch.empty(T, H * R, dtype=torch.bfloat16, device=DEV)
    zero = torch.zeros(H, device=DEV)
    bt, qs, ql, kl = _i32(tables), _i32(starts), _i32(q_lens), _i32(lens)
    pairs = sum(q * (n - q) + q * (q + 1) // 2 for n, q in zip(lens, q_lens))
    flops = 4.0 * R * H * pairs
    work = [(s, b) for s, n in enumerate(q_lens) for b in range((n + 31) // 32)]
    ws, wq = _i32([w[0] for w in work]), _i32([w[1] for w in work])
    if mfma:
        qh = qa.bfloat16().transpose(0, 1).contiguous().transpose(0, 1)       # [H, T, R] in memory
        t = _time(lambda: ops.attn_latent_mfma(qh, pool, bt, qs, ql, kl, ws, wq, lat, sink, 1.0),
                  reps=10, warm=2)
        out[f"attn_latent_mfma ({name})"] = _entry(t, sum(lens) * R * 2 + T * H * R * 4, flops)
    elif name == "decode":
        t = _time(lambda: ops.attn_talk_decode(qa, pool, pool, bt, qs, ql, kl, lat, zero, None, sink, 1.0, 0))
        out["attn_talk_decode (latent, general FMA)"] = _entry(t, sum(lens) * R * 2 + T * H * R * 6, flops)
    else:
        t = _time(lambda: ops.attn_mixq_prefill(qa, pool, pool, bt, qs, ql, kl, ws, wq, lat, zero, sink, 0, 32),
                  reps=3, warm=1)
        out["attn_mixq_prefill (latent, general FMA)"] = _entry(t, sum(lens) * R * 2 + T * H * R * 6, flops)


def _experts(T, d, F, E, top, out):
    from ..models.moe import MoEBuffers, grouped_ok, moe_mlp

    g = torch.Generator(device=DEV).manual_seed(3)
    h = torch.randn(T, d, generator=g, device=DEV).bfloat16()
    w13 = (torch.randn(E, 2 * F, d, generator=g, device=DEV) * d ** -0.5).bfloat16()
    w2 = (torch.randn(E, d, F, generator=g, device=DEV) * F ** -0.5).bfloat16()
    z = torch.randn(T, E, generator=g, device=DEV) * 2
    corr = torch.randn(E, generator=g, device=DEV) * 0.3
    ids = torch.empty(T, top, dtype=torch.int32, device=DEV)
    wts = torch.empty(T, top, device=DEV)
    out["moe_route_grouped"] = _entry(_time(lambda: ops.moe_route_grouped(z, corr, top, 2, 1, ids, wts)),
                                      T * (E * 4 + top * 8), 0)
    if not grouped_ok(w13, w2):
        return
    bufs = MoEBuffers.allocate(T, top, E, d, F, DEV, torch.bfloat16)
    dummy = z.new_zeros(E, d)
    t = _time(lambda: moe_mlp(h, dummy, w13, w2, top, bufs,
                              routing=lambda w, i: ops.moe_route_grouped(z, corr, top, 2, 1, i, w)),
              reps=10, warm=2)
    used = min(E, T * top)
    out["experts (route + grouped GEMMs + combine)"] = _entry(
        t, used * 3 * d * F * 2 + T * d * 4, 6.0 * T * top * d * F)


def run(args) -> dict:
    torch.manual_seed(0)
    d, H, R, WH, N, E, top, F = 4096, 32, 512, 64, 64, 8, 2, 14336
    res = {"width": d, "heads": H, "latent": R, "recurrent_heads": [WH, N], "experts": [E, top, F]}
    pre = {}
    rows = _rows(4096, d, [2048, 2048], [0, 63], pre)
    _wkv(4096, WH, N, rows, pre, False)
    _attention(H, R, [2048, 600], [2048, 600], pre, "prefill", mfma=True)
    _attention(H, R, [2048, 600], [2048, 600], pre, "prefill")
    _experts(4096, d, F, E, top, pre)
    res["prefill_step_4096_rows"] = pre
    dec = {}
    rows = _rows(64, d, [1] * 64, list(range(64)), dec, first=600)
    _wkv(64, WH, N, rows, dec, True)
    _attention(H, R, [600] * 64, [1] * 64, dec, "decode", mfma=True)
    # the general kernel at 16 heads: its key tile still fits the LDS four times over
    _attention(16, R, [600] * 64, [1] * 64, dec, "decode")
    _experts(64, d, F, E, top, dec)
    res["decode_step_64_rows"] = dec
    return res


# ---------------------------------------------------------------------------
# Bilolix's layer kernels at the same step sizes (``bench.py --arch-compare bilolix``):
# 4096-wide layers, 32 heads with two 64-wide score maps over 8 key/value heads and 128-wide
# values, a window of 1,024 positions, 32 recurrent heads with 64 x 128 states, a convolution
# of 4 taps; beside them Numalorn's like kernels (the entries of ``run`` above).
def _b_rows(T, d, out):
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn(T, d, generator=g, device=DEV)
    y1 = torch.randn(T, d, generator=g, device=DEV).bfloat16()
    y2 = torch.randn(T, d, generator=g, device=DEV)
    w = torch.randn(d, generator=g, device=DEV) * 0.3
    h = torch.empty(T, d, dtype=torch.bfloat16, device=DEV)
    out["residual_add_norm"] = _entry(_time(lambda: ops.residual_add_norm(x, y1, y2, None, w, 1e-5, 1.0, h)),
                                      T * d * 16, 0)
    F = 14336
    u = torch.randn(T, F, generator=g, device=DEV).bfloat16()
    o = torch.empty_like(u)
    out["gelu_rows"] = _entry(_time(lambda: ops.gelu_rows(u, o)), T * F * 4, 0)
    z = torch.randn(T, 8, generator=g, device=DEV) * 2
    b = torch.randn(8, generator=g, device=DEV)
    ids = torch.empty(T, 2, dtype=torch.int32, device=DEV)
    wts = torch.empty(T, 2, device=DEV)
    out["moe_route_topk"] = _entry(_time(lambda: ops.moe_route_topk(z, b, 2, ids, wts)), T * (8 * 4 + 16), 0)


def _b_attention(H, G, dim, vdim, window, lens, q_lens, out, name):
    g = torch.Generator(device=DEV).manual_seed(2)
    BS = 32
    nblk = sum((n + BS - 1) // BS for n in lens) + 1
    kc = (torch.randn(nblk, G, BS, 2 * dim, generator=g, device=DEV) * 0.5).bfloat16()
    vc = (torch.randn(nblk, G, BS, vdim, generator=g, device=DEV) * 0.5).bfloat16()
    T = sum(q_lens)
    N = (H + G) * 2 * dim + G * vdim
    qkv = (torch.randn(T, N, generator=g, device=DEV) * 0.5).bfloat16()
    pos = torch.cat([torch.arange(n - q, n) for n, q in zip(lens, q_lens)]).to(torch.int32).to(DEV)
    maxb = (max(lens) + BS - 1) // BS
    tables, at, slots = [], 0, []
    for n, q in zip(lens, q_lens):
        nb = (n + BS - 1) // BS
        tables.append(list(range(at, at + nb)) + [nblk - 1] * (maxb - nb))
        slots += [(at + p // BS) * BS + p % BS for p in range(n - q, n)]
        at += nb
    inv = ops.rotary_inv_freq(dim, 5e5, DEV)
    q = torch.empty(T, H, 2 * dim, device=DEV)
    sl = _i32(slots)
    t = _time(lambda: ops.rotary_append(qkv, pos, inv, sl, kc, vc, H, G, 2, dim, vdim, q))
    out[f"rotary_append ({name})"] = _entry(t, T * N * 2 + T * H * 2 * dim * 4 + T * G * (2 * dim + vdim) * 2, 0)
    gate = torch.randn(T, H, generator=g, device=DEV).bfloat16()
    o = torch.empty(T, H * vdim, dtype=torch.bfloat16, device=DEV)
    starts = [sum(q_lens[:i]) for i in range(len(lens))]
    bt, qs, ql, kl = _i32(tables), _i32(starts), _i32(q_lens), _i32(lens)
    work = [(s, b) for s, n in enumerate(q_lens) for b in range((n + 31) // 32)]
    ws, wq = _i32([w[0] for w in work]), _i32([w[1] for w in work])
    pairs = 0
    for n, ql_ in zip(lens, q_lens):
        for p in range(n - ql_, n):
            pairs += min(p + 1, window)
    flops = (4.0 * dim + 4.0 * vdim) * H * pairs
    seen = sum(min(n, window + q - 1) for n, q in zip(lens, q_lens))
    nbytes = seen * G * (2 * dim + vdim) * 2 + T * H * (2 * dim * 4 + vdim * 2)
    short = ops.TALK_DECODE_MAX_ROWS if name == "decode" else 0
    t = _time(lambda: ops.attn_diff_window(q, kc, vc, bt, qs, ql, kl, ws, wq, gate, o, dim ** -0.5,
                                           window, 0.4, 1e-5, 0.4, short), reps=5, warm=2)
    out[f"attn_diff_window ({name})"] = _entry(t, nbytes, flops)


def _b_recurrence(T, H, dim, vdim, rows, out, decode):
    g = torch.Generator(device=DEV).manual_seed(1)
    run = torch.nonzero(rows[1] == 0)[:, 0].to(torch.int32)
    seqs = int(run.numel())
    q, k = ((torch.randn(T, H, dim, generator=g, device=DEV) * 0.5).bfloat16() for _ in range(2))
    v = (torch.randn(T, H, vdim, generator=g, device=DEV) * 0.5).bfloat16()
    gate = torch.randn(T, H * vdim, generator=g, device=DEV).bfloat16()
    z = torch.randn(T, H * dim, generator=g, device=DEV)
    rate = torch.full((H,), 1 / 16, device=DEV)
    zb = torch.randn(H * dim, generator=g, device=DEV) + 2
    nw = torch.ones(vdim, device=DEV)
    st = torch.zeros(128, H, dim, vdim, device=DEV)
    y = torch.empty(T, H * vdim, dtype=torch.bfloat16, device=DEV)
    state_bytes = (2 if decode else 1) * seqs * H * dim * vdim * 4
    t = _time(lambda: ops.gated_linear_recurrence(q, k, v, z, rate, zb, -1.0, None, gate, False, nw, 1e-5,
                                                  dim ** -0.5, st, *rows, y, run), reps=5, warm=2)
    out["gated_linear_recurrence (gla)"] = _entry(
        t, T * H * (2 * dim * 2 + dim * 4 + vdim * 6) + state_bytes, 6.0 * T * H * dim * vdim)
    # the delta rule: q, k, v come from the convolution in fp32
    C = 2 * H * dim + H * vdim
    x = (torch.randn(T, C, generator=g, device=DEV) * 0.5).bfloat16()
    cw = torch.randn(C, 4, generator=g, device=DEV) * 0.5
    cs = torch.zeros(128, 3, C, device=DEV)
    qkv = torch.empty(T, C, device=DEV)
    t = _time(lambda: ops.conv_act_heads(x, cw, cs, *rows, 2 * H, dim, 1e-6, qkv))
    out["conv_act_heads"] = _entry(t, T * C * 6 + (seqs * 3 * C * 8 if decode else 0), 0)
    beta = torch.randn(T, H, generator=g, device=DEV).bfloat16()
    qf, kf = qkv[:, :H * dim].unflatten(1, (H, dim)), qkv[:, H * dim:2 * H * dim].unflatten(1, (H, dim))
    vf = qkv[:, 2 * H * dim:].unflatten(1, (H, vdim))
    t = _time(lambda: ops.gated_linear_recurrence(qf, kf, vf, z, rate, zb, 1.0, beta, gate, True, nw, 1e-5,
                                                  dim ** -0.5, st, *rows, y, run), reps=5, warm=2)
    out["gated_linear_recurrence (delta rule)"] = _entry(
        t, T * H * (2 * dim * 4 + dim * 4 + vdim * 8) + state_bytes, 10.0 * T * H * dim * vdim)


def run_bilolix(args) -> dict:
    torch.manual_seed(0)
    d, H, G, dim, vdim, window, RH = 4096, 32, 8, 64, 128, 1024, 32
    res = {"width": d, "heads": [H, G], "maps": [2, dim], "vdim": vdim, "window": window,
           "recurrent_heads": [RH, dim, vdim]}
    pre, like_pre = {}, {}
    _b_rows(4096, d, pre)
    rows = _runs([2048, 2048], [0, 63])
    _b_recurrence(4096, RH, dim, vdim, rows, pre, False)
    _b_attention(H, G, dim, vdim, window, [2048, 600], [2048, 600], pre, "prefill")
    nrows = _rows(4096, d, [2048, 2048], [0, 63], like_pre)
    _wkv(4096, 64, 64, nrows, like_pre, False)
    _attention(32, 512, [2048, 600], [2048, 600], like_pre, "prefill", mfma=True)
    res["prefill_step_4096_rows"] = {"bilolix": pre, "numalorn": like_pre}
    dec, like_dec = {}, {}
    _b_rows(64, d, dec)
    rows = _runs([1] * 64, list(range(64)), first=600)
    _b_recurrence(64, RH, dim, vdim, rows, dec, True)
    _b_attention(H, G, dim, vdim, window, [600] * 64, [1] * 64, dec, "decode")
    nrows = _rows(64, d, [1] * 64, list(range(64)), like_dec, first=600)
    _wkv(64, 64, 64, nrows, like_dec, True)
    _attention(32, 512, [600] * 64, [1] * 64, like_dec, "decode", mfma=True)
    res["decode_step_64_rows"] = {"bilolix": dec, "numalorn": like_dec}
    return res


# ---------------------------------------------------------------------------
# Nutitar's kernels (``bench.py --arch-compare nutitar``) beside Bilolix's like kernels in the
# same run: 4096-wide layers, 32 heads over 8 key/value heads of 128, a 512-wide latent with a
# 64-wide rotated key part, window 1,024 with 64 kept tokens.
def _pages(lens, q_lens, G, kw, vw, g):
    BS = 32
    nblk = sum((n + BS - 1) // BS for n in lens) + 1
    kc = (torch.randn(nblk, G, BS, kw, generator=g, device=DEV) * 0.5).bfloat16()
    vc = None if vw == 0 else (torch.randn(nblk, G, BS, vw, generator=g, device=DEV) * 0.5).bfloat16()
    maxb = (max(lens) + BS - 1) // BS
    tables, at, slots = [], 0, []
    for n, q in zip(lens, q_lens):
        nb = (n + BS - 1) // BS
        tables.append(list(range(at, at + nb)) + [nblk - 1] * (maxb - nb))
        slots += [(at + p // BS) * BS + p % BS for p in range(n - q, n)]
        at += nb
    pos = torch.cat([torch.arange(n - q, n) for n, q in zip(lens, q_lens)]).to(torch.int32).to(DEV)
    starts = [sum(q_lens[:i]) for i in range(len(lens))]
    work = [(s, b) for s, n in enumerate(q_lens) for b in range((n + 31) // 32)]
    meta = (_i32(tables), _i32(starts), _i32(q_lens), _i32(lens), _i32([w[0] for w in work]),
            _i32([w[1] for w in work]))
    return kc, vc, pos, _i32(slots), meta


def _n_attention(kind, H, G, lens, q_lens, out, name, window=0, keep=0):
    """kind: "window" (sigmoid, biased, norm over the projection), "keyval" (softmax, head
    norms, values = keys) or "latent" (512 + 64 wide shared pages, sink, gate)."""
    g = torch.Generator(device=DEV).manual_seed(3)
    T = sum(q_lens)
    short = ops.TALK_DECODE_MAX_ROWS if name == "decode" else 0
    dim = 128
    if kind == "latent":
        R, rd = 512, 64
        E, vd, Gk = R + rd, R, 1
        kc, _, pos, sl, meta = _pages(lens, q_lens, 1, E, 0, g)
        vc = kc
        N = H * (dim + rd) + E + H
        pr = (torch.randn(T, N, generator=g, device=DEV) * 0.5).bfloat16()
        nw = torch.randn(R, generator=g, device=DEV)
        inv, mult = ops.rotary_scaled_freq(rd, 5e5, ("yarn", 4.0, 4096.0, 32.0, 1.0), DEV)
        qf = torch.empty(T, H, dim + rd, device=DEV)
        t = _time(lambda: ops.qk_norm_rotary_append(pr, None, None, nw, False, R, 1e-5, pos, inv, mult, dim,
                                                    R, sl, kc, None, H, 1, dim + rd, E, 0, 2, qf))
        out[f"qk_norm_rotary_append latent ({name})"] = _entry(
            t, T * (H * (dim + rd) + E) * 2 + T * H * (dim + rd) * 4 + T * E * 2, 0)
        q = torch.randn(T, H, E, generator=g, device=DEV) * 0.3
        bias = torch.randn(H, generator=g, device=DEV)
        gate = pr[:, N - H:]
        sig = False
    else:
        E, vd, Gk = dim, dim, G
        kc, vc, pos, sl, meta = _pages(lens, q_lens, G, dim, dim, g)
        second = kind == "keyval"
        N = (H + G) * dim + (0 if second else G * dim)
        pr = (torch.randn(T, N, generator=g, device=DEV) * 0.5).bfloat16()
        pb = None if second else torch.randn(N, generator=g, device=DEV)
        n = dim if second else H * dim
        qn = torch.randn(n, generator=g, device=DEV)
        kn = torch.randn(dim if second else G * dim, generator=g, device=DEV)
        inv, mult = ops.rotary_scaled_freq(64, 5e5, (), DEV)
        q = torch.empty(T, H, dim, device=DEV)
        t = _time(lambda: ops.qk_norm_rotary_append(pr, pb, qn, kn, not second, dim, 1e-5, pos, inv, mult, 0,
                                                    0, sl, kc, vc, H, G, dim, dim, dim, 1 if second else 0, q))
        out[f"qk_norm_rotary_append {kind} ({name})"] = _entry(
            t, T * N * 2 + T * H * dim * 4 + T * G * 2 * dim * 2, 0)
        bias = None if second else torch.randn(H, generator=g, device=DEV) - 3.0
        gate, sig = None, not second
    o = torch.empty(T, H * vd, dtype=torch.bfloat16, device=DEV)
    pairs = seen = 0
    for n_, q_ in zip(lens, q_lens):
        for p in range(n_ - q_, n_):
            pairs += p + 1 if window == 0 else min(p + 1, window + min(keep, max(0, p + 1 - window)))
        seen += n_ if window == 0 else min(n_, window + q_ - 1 + keep)
    flops = (2.0 * E + 2.0 * vd) * H * pairs
    nbytes = seen * Gk * (E + (0 if kind == "latent" else vd)) * 2 + T * H * (E * 4 + vd * 2)
    bt, qs, ql, kl, ws, wq = meta
    t = _time(lambda: ops.attn_keep_window(q, kc, vc, vd, bt, qs, ql, kl, ws, wq, bias, gate, o, E ** -0.5,
                                           window, keep, sig, short_rows=short), reps=5, warm=2)
    out[f"attn_keep_window {kind} ({name})"] = _entry(t, nbytes, flops)


def _n_rows(T, d, lens, slots, out, first=0):
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn(T, d, generator=g, device=DEV)
    y1 = torch.randn(T, d, generator=g, device=DEV).bfloat16()
    y2 = torch.randn(T, d, generator=g, device=DEV).bfloat16()
    w = torch.randn(d, generator=g, device=DEV) * 0.3
    hf = torch.empty(T, d, device=DEV)
    out["residual_add_norm"] = _entry(
        _time(lambda: ops.residual_add_norm(x, y1, y2, None, w, 1e-5, 1.0, hf, mult=0.5)), T * d * 16, 0)
    mu = torch.rand(2, d, generator=g, device=DEV)
    prev = torch.zeros(2 * 64, d, device=DEV)
    rows = _runs(lens, slots, first)
    mixes = torch.empty(2, T, d, dtype=torch.bfloat16, device=DEV)
    out["token_shift_mix"] = _entry(_time(lambda: ops.token_shift_mix(hf, mu, prev, *rows, mixes)),
                                    T * d * 8 + len(lens) * d * 8, 0)
    F = 14336
    u = torch.randn(T, F, generator=g, device=DEV).bfloat16()
    o = torch.empty_like(u)
    out["xielu_rows"] = _entry(_time(lambda: ops.xielu_rows(u, 0.8, 1.2, o)), T * F * 4, 0)


def run_nutitar(args) -> dict:
    torch.manual_seed(0)
    d, H, G, window, keep = 4096, 32, 8, 1024, 64
    res = {"width": d, "heads": [H, G], "head": 128, "latent": [512, 64], "window": [window, keep]}
    for name, lens, q_lens, key in (("prefill", [2048, 600], [2048, 600], "prefill_step_rows"),
                                    ("decode", [600] * 64, [1] * 64, "decode_step_64_rows")):
        mine, like = {}, {}
        T = sum(q_lens)
        rl = [2048, 2048] if name == "prefill" else [1] * 64
        sl = [0, 63] if name == "prefill" else list(range(64))
        _n_rows(sum(rl), d, rl, sl, mine, 0 if name == "prefill" else 600)
        _n_attention("window", H, G, lens, q_lens, mine, name, window, keep)
        _n_attention("keyval", H, G, lens, q_lens, mine, name)
        _n_attention("latent", H, G, lens, q_lens, mine, name)
        _b_rows(sum(rl), d, like)
        _b_attention(H, G, 64, 128, window, lens, q_lens, like, name)
        _attention(32, 512, lens, q_lens, like, name, mfma=True)
        res[key] = {"nutitar": mine, "bilolix": like, "rows": T}
    return res
