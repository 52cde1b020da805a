"""Each Nutitar mechanism alone (package op on CPU tensors or the gfx950 kernel) against the slow
oracle, with inputs made so that a key, a kept token, a sink or a state missed or wrongly seen
shows."""
import math

import pytest
import torch

from replisense_rfq_amd import ops

from . import oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BS = 32
D64 = torch.float64


def close(a, b, tol=2e-5):
    a, b = a.double().cpu(), b.double().cpu()
    assert float((a - b).abs().max()) <= tol * max(1.0, float(b.abs().max())), \
        float((a - b).abs().max())


def i32(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


# ------------------------------------------------------------------ stream, norm, embedding
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("d", [44, 256, 1030])
def test_scaled_residual_of_two_sublayers_and_next_norm(device, d):
    """x += m (y1 + y2), then the next layer's input rms(x) (1 + w) in fp32."""
    g = torch.Generator().manual_seed(1)
    T, eps, m = 5, 1e-3, 0.35
    x = torch.randn(T, d, generator=g) * 4
    y1, y2 = torch.randn(T, d, generator=g), torch.randn(T, d, generator=g) * 0.3
    w = torch.randn(d, generator=g) * 0.5
    for a, b in ((y1, y2), (y1, None), (None, y2)):
        want = x.double() + m * ((a.double() if a is not None else 0.0) + (b.double() if b is not None else 0.0))
        xd, out = x.clone().to(device), torch.empty(T, d, device=device)
        ops.residual_add_norm(xd, None if a is None else a.to(device), None if b is None else b.to(device),
                              None, w.to(device), eps, 1.0, out, mult=m)
        close(xd, want)
        close(out, oracle.norm_around_zero(want, w.double(), eps))
    # the multiplier is not applied to the stream itself
    xd = x.clone().to(device)
    ops.residual_add_norm(xd, y1.to(device).bfloat16(), None, mult=m)
    close(xd, x.double() + m * y1.bfloat16().double())


@pytest.mark.parametrize("device", DEVICES)
def test_scaled_embedding(device):
    g = torch.Generator().manual_seed(2)
    table = torch.randn(37, 50, generator=g).bfloat16()
    ids = [5, 0, 36, 5]
    got = ops.embed_rows(i32(ids, device), table.to(device), scale=7.5)
    close(got, table.double()[ids] * 7.5, 1e-6)


@pytest.mark.parametrize("device", DEVICES)
def test_xielu(device):
    x = torch.linspace(-9, 9, 3999).view(3, -1)
    p, q = 0.3, -0.8
    ap, an = oracle.softplus(p), 0.5 + oracle.softplus(q)
    close(ops.xielu_rows(x.to(device), ap, an), oracle.xielu(x.double(), p, q), 1e-6)
    wide = torch.randn(4, 70)
    close(ops.xielu_rows(wide.to(device)[:, 3:40], ap, an), oracle.xielu(wide[:, 3:40].double(), p, q), 1e-6)
    # both branches matter and the slope at zero is one half from either side
    y = oracle.xielu(torch.tensor([-1e-4, 1e-4], dtype=D64), p, q)
    assert abs(float(y[1] - y[0]) / 2e-4 - 0.5) < 1e-3
    assert float(oracle.xielu(torch.tensor([2.0], dtype=D64), p, q)) > 1.0 + 2.0 * ap


# ------------------------------------------------------------------ token shift through slots
@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_in_portions_through_slots_with_stale_contents(device):
    """Two sequences cut into runs; the row before a run comes from the sequence's slot half,
    zeros at position 0 whatever the slot holds; mix 0 (shift 0) is the row itself."""
    g = torch.Generator().manual_seed(3)
    d, slots = 40, 3
    shift = torch.rand(d, generator=g)
    mu = torch.stack([torch.zeros(d), shift]).to(device)
    hs = {0: torch.randn(11, d, generator=g), 2: torch.randn(7, d, generator=g)}
    want = {s: oracle.token_shift(h.double(), shift.double()) for s, h in hs.items()}
    prev = torch.full((2 * slots, d), 99.0, device=device)            # stale everywhere
    at, gen = {0: 0, 2: 0}, {0: 0, 2: 0}
    for runs in ([(0, 4), (2, 1)], [(2, 3), (0, 1)], [(0, 6), (2, 3)]):
        rows, rs, rb, rf, pos = [], [], [], [], []
        for s, n in runs:
            for i in range(n):
                rows.append(hs[s][at[s] + i])
                rs.append(2 * s + (gen[s] & 1))
                rb.append(i)
                rf.append(n - 1 - i)
                pos.append(at[s] + i)
        x = torch.stack(rows).to(device)
        out = torch.empty(2, len(rows), d, device=device)
        ops.token_shift_mix(x, mu, prev, i32(rs, device), i32(rb, device), i32(rf, device),
                            i32(pos, device), out)
        r = 0
        for s, n in runs:
            close(out[1, r:r + n], want[s][at[s]:at[s] + n])
            close(out[0, r:r + n], hs[s][at[s]:at[s] + n], 0)
            r += n
            at[s] += n
            gen[s] += 1


# ------------------------------------------------------------------ frequencies
def test_scaled_frequencies_against_the_oracle():
    cases = [
        ({"dims": 20, "base": 250000.0}, ()),
        ({"dims": 8, "base": 300.0, "scaling": {"factor": 3.0, "original": 40, "fast": 8.0, "slow": 1.0}},
         ("yarn", 3.0, 40.0, 8.0, 1.0)),
        # every dimension past the ramp, and none: lo = hi, and lo clamped to 0
        ({"dims": 6, "base": 50.0, "scaling": {"factor": 2.0, "original": 1000, "fast": 0.5, "slow": 0.4}},
         ("yarn", 2.0, 1000.0, 0.5, 0.4)),
        ({"dims": 12, "base": 10000.0, "scaling": {"factor": 5.0, "original": 6, "fast": 64.0, "slow": 32.0}},
         ("yarn", 5.0, 6.0, 64.0, 32.0)),
        ({"dims": 40, "base": 30000.0, "scaling": {"factor": 6.0, "original": 96, "low": 1.0, "high": 8.0}},
         ("banded", 6.0, 96.0, 1.0, 8.0)),
        ({"dims": 10, "base": 100.0, "scaling": {"factor": 8.0, "original": 20, "low": 2.0, "high": 3.0}},
         ("banded", 8.0, 20.0, 2.0, 3.0)),
    ]
    for rot, scaling in cases:
        f, mult = ops.rotary_scaled_freq(rot["dims"], rot["base"], scaling)
        wf, wm = oracle.frequencies(rot)
        close(f, wf, 1e-7)
        assert abs(mult - wm) < 1e-12
    # the banded rule has all three bands in the first banded case
    f, _ = ops.rotary_scaled_freq(40, 30000.0, ("banded", 6.0, 96.0, 1.0, 8.0))
    r = f.double() / oracle.base_frequencies(40, 30000.0)
    assert float(r.max()) == 1.0 and abs(float(r.min()) - 1 / 6) < 1e-6 and ((r > 0.18) & (r < 0.99)).any()


# ------------------------------------------------------------------ norms, rotation, pages
POS = [0, 1, 2, 40, 41, 500, 31, 32, 33]
SLOTS = [5 * BS + 0, 5 * BS + 1, 2 * BS + 31, 0, 1, -1, 3 * BS + 7, 4 * BS + 30, BS + 2]


def _pages_hold(cache, rows, slots, tol=1e-5):
    for t, s in enumerate(slots):
        if s >= 0:
            close(cache[s // BS, :, s % BS], rows[t], tol)
    written = {s for s in slots if s >= 0}
    for s in range(cache.shape[0] * BS):
        if s not in written:
            assert float(cache[s // BS, :, s % BS].min()) == 9.0 == float(cache[s // BS, :, s % BS].max())


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,dim,rot", [(4, 2, 16, 8), (3, 1, 10, 10), (2, 2, 8, 0), (1, 1, 6, 2), (8, 4, 64, 32)])
def test_head_norms_half_split_rotation_and_keys_as_values(device, H, G, dim, rot):
    """Per-head norms with one shared weight, rotation of entry i with entry i + rot / 2, the
    rest of a head unchanged; the value pages receive the keys as projected."""
    g = torch.Generator().manual_seed(4)
    T, eps = len(POS), 1e-4
    N = (H + G) * dim
    wide = torch.randn(T, N + 5, generator=g)
    qw_, kw_ = torch.randn(dim, generator=g), torch.randn(dim, generator=g)
    rcfg = {"dims": rot, "base": 777.0, "scaling": {"factor": 3.0, "original": 16, "low": 1.0, "high": 5.0}}
    f, mult = ops.rotary_scaled_freq(rot, 777.0, ("banded", 3.0, 16.0, 1.0, 5.0), device)
    kc = torch.full((6, G, BS, dim), 9.0, device=device)
    vc = torch.full((6, G, BS, dim), 9.0, device=device)
    q = torch.empty(T, H, dim, device=device)
    ops.qk_norm_rotary_append(wide.to(device)[:, :N], None, qw_.to(device), kw_.to(device), False, dim, eps,
                              i32(POS, device), f, mult, 0, 0, i32(SLOTS, device), kc, vc, H, G, dim,
                              dim, dim, 1, q)
    x = wide[:, :N].double()
    pos = torch.tensor(POS)
    wf, wm = oracle.frequencies(rcfg)
    rq = x[:, :H * dim].reshape(T, H, dim)
    rk = x[:, H * dim:].reshape(T, G, dim)
    wq = oracle.rotate_half(oracle.rms_unit(rq, eps) * qw_.double(), pos, wf, wm)
    wk = oracle.rotate_half(oracle.rms_unit(rk, eps) * kw_.double(), pos, wf, wm)
    close(q, wq, 1e-5)
    _pages_hold(kc, wk, SLOTS)
    _pages_hold(vc, rk, SLOTS, 0)
    if rot >= 4:                                       # entry 1 turns with entry 1 + rot / 2
        n = oracle.rms_unit(rq, eps) * qw_.double()
        ang = float(pos[3]) * float(wf[1])
        close(q[3, 0, 1], n[3, 0, 1] * math.cos(ang) - n[3, 0, 1 + rot // 2] * math.sin(ang), 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,dim,vdim,rot", [(4, 2, 16, 8, 8), (3, 3, 10, 6, 4), (8, 2, 64, 64, 16)])
def test_whole_projection_norms_with_biases(device, H, G, dim, vdim, rot):
    """One root mean square over all heads of q (and of k) with a weight per entry; biases are
    added before the norm; v gets its bias and no norm or rotation."""
    g = torch.Generator().manual_seed(5)
    T, eps = len(POS), 1e-4
    N = (H + G) * dim + G * vdim
    proj = torch.randn(T, N, generator=g)
    bias = torch.randn(N, generator=g)
    qw_, kw_ = torch.randn(H * dim, generator=g), torch.randn(G * dim, generator=g)
    f, mult = ops.rotary_scaled_freq(rot, 1e6, (), device)
    kc = torch.full((6, G, BS, dim), 9.0, device=device)
    vc = torch.full((6, G, BS, vdim), 9.0, device=device)
    q = torch.empty(T, H, dim, device=device)
    ops.qk_norm_rotary_append(proj.to(device), bias.to(device), qw_.to(device), kw_.to(device), True, dim,
                              eps, i32(POS, device), f, mult, 0, 0, i32(SLOTS, device), kc, vc, H, G,
                              dim, dim, vdim, 0, q)
    x = proj.double() + bias.double()
    pos = torch.tensor(POS)
    wf = oracle.base_frequencies(rot, 1e6)
    wq = oracle.rotate_half((oracle.rms_unit(x[:, :H * dim], eps) * qw_.double()).view(T, H, dim), pos, wf)
    wk = oracle.rotate_half((oracle.rms_unit(x[:, H * dim:(H + G) * dim], eps) * kw_.double()).view(T, G, dim),
                            pos, wf)
    close(q, wq, 1e-5)
    _pages_hold(kc, wk, SLOTS)
    _pages_hold(vc, x[:, (H + G) * dim:].view(T, G, vdim), SLOTS, 1e-6)
    per_head = oracle.rms_unit(x[:, :H * dim].view(T, H, dim), eps)
    assert float((per_head - oracle.rms_unit(x[:, :H * dim], eps).view(T, H, dim)).abs().max()) > 1e-2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,dim,rd,R", [(3, 12, 8, 24), (2, 6, 6, 14), (8, 32, 16, 64)])
def test_latent_row_norm_and_rotated_key_part(device, H, dim, rd, R):
    """q: no norm, only the trailing rot_dim of every head rotated (with the YaRN factor on cos and
    sin); the page row is [normed latent | rotated key part]; a layer without latent of its own
    writes nothing."""
    g = torch.Generator().manual_seed(6)
    T, eps = len(POS), 1e-4
    N = H * (dim + rd) + R + rd
    proj = torch.randn(T, N + H, generator=g)
    nw = torch.randn(R, generator=g)
    rcfg = {"dims": rd, "base": 300.0, "scaling": {"factor": 3.0, "original": 40, "fast": 8.0, "slow": 1.0}}
    f, mult = ops.rotary_scaled_freq(rd, 300.0, ("yarn", 3.0, 40.0, 8.0, 1.0), device)
    assert mult > 1.05
    pool = torch.full((6, 1, BS, R + rd), 9.0, device=device)
    q = torch.empty(T, H, dim + rd, device=device)
    ops.qk_norm_rotary_append(proj.to(device), None, None, nw.to(device), False, R, eps, i32(POS, device),
                              f, mult, dim, R, i32(SLOTS, device), pool, None, H, 1, dim + rd, R + rd, 0,
                              2, q)
    x = proj.double()
    pos = torch.tensor(POS)
    wf, wm = oracle.frequencies(rcfg)
    rq = x[:, :H * (dim + rd)].view(T, H, dim + rd)
    wq = torch.cat([rq[..., :dim], oracle.rotate_half(rq[..., dim:], pos, wf, wm)], -1)
    dkv = x[:, H * (dim + rd):N]
    row = torch.cat([oracle.rms_unit(dkv[:, :R], eps) * nw.double(),
                     oracle.rotate_half(dkv[:, R:], pos, wf, wm)], -1)
    close(q, wq, 1e-5)
    _pages_hold(pool, row.view(T, 1, R + rd), SLOTS)
    q2 = torch.empty(T, H, dim + rd, device=device)
    ops.qk_norm_rotary_append(proj.to(device), None, None, None, False, R, eps, i32(POS, device), f, mult,
                              dim, R, i32(SLOTS, device), None, None, H, 0, dim + rd, R + rd, 0, 2, q2)
    close(q2, wq, 1e-5)


# ------------------------------------------------------------------ attention
def _paged(k, v, order, device, dtype=torch.float32):
    """k [L, G, E], v [L, G, vdim] (or None: the values are the keys' leading entries) into
    pools whose pages lie in the given order."""
    L, G = k.shape[:2]
    nb = (L + BS - 1) // BS
    blocks = max(order) + 2
    kc = torch.full((blocks, G, BS, k.shape[2]), 7.0, dtype=dtype)
    vc = None if v is None else torch.full((blocks, G, BS, v.shape[2]), 7.0, dtype=dtype)
    for j in range(L):
        kc[order[j // BS], :, j % BS] = k[j].to(dtype)
        if v is not None:
            vc[order[j // BS], :, j % BS] = v[j].to(dtype)
    bt = order[:nb] + [blocks - 1] * 3
    kc = kc.to(device)
    return kc, (kc if v is None else vc.to(device)), bt


def _attend(device, q, k, v, vdim, sections, scale, window=0, keep=0, bias=None, gate=None,
            sigmoid=False, dtype=torch.float32, mfma=None, short=False):
    """sections: [(first row, rows)] of ONE sequence of L rows, each run as its own launch with
    everything before it already cached; returns out [L, H vdim]."""
    L, H = q.shape[:2]
    order = [4, 0, 9, 2, 7, 1, 8, 3, 6, 5, 10, 11, 12, 13, 14][: (L + BS - 1) // BS]
    kc, vc, bt = _paged(k, v, order, device, dtype)
    out = torch.zeros(L, H * vdim, dtype=dtype, device=device)
    hb = None if bias is None else bias.float().to(device)
    for lo, n in sections:
        nblk = (n + ops.KEEP_QBLK - 1) // ops.KEEP_QBLK
        ops.attn_keep_window(q[lo:lo + n].float().contiguous().to(device), kc, vc, vdim, i32([bt], device),
                             i32([0], device), i32([n], device), i32([lo + n], device),
                             i32([0] * nblk, device), i32(list(range(nblk)), device), hb,
                             None if gate is None else gate[lo:lo + n].to(dtype).to(device),
                             out[lo:lo + n], scale, window, keep, sigmoid,
                             short_rows=32 if (short and n <= 32) else 0, mfma=mfma)
    return out


def _dense(q, k, v, scale, window, keep, bias, gate, sigmoid):
    """The oracle's masks and weights on whole tensors: q [L, H, E], k [L, G, E], v [L, G, vdim]."""
    L, H = q.shape[:2]
    G = k.shape[1]
    pos = torch.arange(L)
    ok = oracle.visible(pos, pos, window, keep)
    out = torch.zeros(L, H, v.shape[2], dtype=D64)
    for h in range(H):
        c = h // (H // G)
        s = (q[:, h].double() @ k[:, c].double().T) * scale
        if sigmoid:
            p = oracle.sigmoid_weights(s, ok, bias[h].double())
        else:
            p = oracle.softmax_weights(s, ok, None if bias is None else bias[h].double())
        out[:, h] = p @ v[:, c].double()
        if gate is not None:
            out[:, h] *= oracle.sigmoid(gate[:, h:h + 1].double())
    return out.reshape(L, -1)


SECTIONS = [(0, 70), (70, 3), (73, 45)] + [(118 + i, 1) for i in range(32)]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,dim,vdim", [(4, 2, 16, 8), (3, 3, 40, 24), (2, 1, 8, 72), (8, 2, 64, 64)])
@pytest.mark.parametrize("window,keep", [(0, 0), (1, 0), (5, 2), (32, 32), (33, 7), (100, 40), (20, 200)])
@pytest.mark.parametrize("kind", ["softmax", "sink", "sigmoid"])
def test_attention_in_sections(device, H, G, dim, vdim, window, keep, kind):
    """A prompt portion (several query blocks), a short extend and single decoded rows (through
    the work-item kernel and the grouped decode kernel) over pages in odd order equal the dense
    computation of the whole sequence, for every kind of weights."""
    g = torch.Generator().manual_seed(7)
    L, scale = 150, 0.4
    q = torch.randn(L, H, dim, generator=g)
    k = torch.randn(L, G, dim, generator=g)
    v = torch.randn(L, G, vdim, generator=g)
    bias = None if kind == "softmax" else torch.randn(H, generator=g)
    gate = torch.randn(L, H, generator=g) if kind == "sink" else None
    want = _dense(q, k, v, scale, window, keep, bias, gate, kind == "sigmoid")
    for short in (False, True):
        got = _attend(device, q, k, v, vdim, SECTIONS, scale, window, keep, bias, gate, kind == "sigmoid",
                      short=short)
        close(got, want, 5e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("R,rd,H", [(24, 8, 3), (16, 16, 5), (64, 32, 8)])
def test_values_are_the_leading_part_of_the_key_pages(device, R, rd, H):
    """Latent attention: one key head of R + rd entries whose first R are also the values; sink
    and output gate."""
    g = torch.Generator().manual_seed(8)
    L = 150
    q = torch.randn(L, H, R + rd, generator=g)
    k = torch.randn(L, 1, R + rd, generator=g)
    sink, gate = torch.randn(H, generator=g), torch.randn(L, H, generator=g)
    want = _dense(q, k, k[..., :R], 0.3, 0, 0, sink, gate, False)
    for short in (False, True):
        close(_attend(device, q, k, None, R, SECTIONS, 0.3, bias=sink, gate=gate, short=short), want, 5e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window", [1, 2, 31, 32, 33, 64, 65, 97])
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("sigmoid", [False, True])
def test_a_key_at_the_window_edge_stands_out(device, window, decoded, sigmoid):
    """One key matches the last query and carries a value far from the others: on the window's
    last position inside it shows in the output, one position further out it must not."""
    g = torch.Generator().manual_seed(9)
    L, H, G, dim, vdim = 140, 2, 1, 16, 8
    bias = torch.full((H,), -4.0) if sigmoid else None
    for inside in (True, False):
        q = torch.randn(L, H, dim, generator=g) * 0.1
        k = torch.randn(L, G, dim, generator=g) * 0.1
        v = torch.randn(L, G, vdim, generator=g)
        j = L - 1 - (window - 1) - (0 if inside else 1)
        q[L - 1, :, 0] = 3.0
        k[j, 0, 0] = 3.0
        v[j, 0] = 100.0
        want = _dense(q, k, v, 1.0, window, 0, bias, None, sigmoid)
        sections = [(0, L - 1), (L - 1, 1)] if decoded else [(0, L)]
        got = _attend(device, q, k, v, vdim, sections, 1.0, window, 0, bias, None, sigmoid, short=decoded)
        close(got, want, 5e-5)
        assert (float(got[L - 1, 0]) > 50.0) == inside, (window, inside, float(got[L - 1, 0]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("keep", [1, 2, 31, 32, 33, 70])
@pytest.mark.parametrize("decoded", [False, True])
def test_the_last_kept_token_and_the_one_after_it(device, keep, decoded):
    """Far outside the window, token keep - 1 is seen and token keep is not, whatever page it
    lies in; kept tokens keep their true positions."""
    g = torch.Generator().manual_seed(10)
    L, H, G, dim, vdim, window = 150, 2, 2, 8, 8, 9
    for j in (keep - 1, keep):
        q = torch.randn(L, H, dim, generator=g) * 0.1
        k = torch.randn(L, G, dim, generator=g) * 0.1
        v = torch.randn(L, G, vdim, generator=g)
        q[L - 1, :, 1] = 3.0
        k[j, :, 1] = 3.0
        v[j, :] = 100.0
        want = _dense(q, k, v, 1.0, window, keep, None, None, False)
        sections = [(0, L - 1), (L - 1, 1)] if decoded else [(0, 100), (100, 50)]
        got = _attend(device, q, k, v, vdim, sections, 1.0, window, keep, short=decoded)
        close(got, want, 5e-5)
        assert (float(got[L - 1, 0]) > 50.0) == (j < keep), (keep, j)


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds_and_the_sink(device):
    g = torch.Generator().manual_seed(11)
    L, H, G, dim, vdim = 450, 2, 2, 8, 8
    q = torch.randn(L, H, dim, generator=g) * 0.1
    k = torch.randn(L, G, dim, generator=g) * 0.1
    v = torch.randn(L, G, vdim, generator=g)
    q[L - 1, 1, 1] = 4.0
    k[3, 1, 1] = 4.0                                         # head 1 finds token 3
    v[3, 1] = 50.0
    for sections, short in (([(0, L)], False), ([(0, L - 1), (L - 1, 1)], True), ([(0, L - 1), (L - 1, 1)], False)):
        want = _dense(q, k, v, 1.0, 0, 0, None, None, False)
        close(_attend(device, q, k, v, vdim, sections, 1.0, short=short), want, 5e-5)
        assert float(want[L - 1, vdim:].min()) > 45.0
        # a sink as large as the found key's score takes half of the weight, once
        sink = torch.tensor([0.0, 16.0])
        want = _dense(q, k, v, 1.0, 0, 0, sink, None, False)
        got = _attend(device, q, k, v, vdim, sections, 1.0, bias=sink, short=short)
        close(got, want, 5e-5)
        assert 20.0 < float(got[L - 1, vdim]) < 30.0


@pytest.mark.parametrize("device", DEVICES)
def test_sigmoid_weights_are_not_normalised(device):
    """Equal scores on n visible keys: the output grows with n (a softmax's would not)."""
    L, H, dim, vdim = 40, 1, 4, 4
    q, k = torch.zeros(L, H, dim), torch.zeros(L, 1, dim)
    v = torch.ones(L, 1, vdim)
    bias = torch.tensor([0.5])
    got = _attend(device, q, k, v, vdim, [(0, L)], 1.0, 0, 0, bias, None, True)
    w = 1.0 / (1.0 + math.exp(-0.5))
    close(got[:, 0], torch.arange(1, L + 1, dtype=D64) * w, 1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_two_sequences_one_launch(device):
    """Work items of two sequences of unequal length in one launch, prompt rows and the grouped
    decode kernel."""
    g = torch.Generator().manual_seed(12)
    H, G, dim, vdim, scale = 3, 1, 8, 8, 0.5
    lens, news = (50, 9), (40, 9)                              # (kv length, new rows) of the two
    qs = [torch.randn(L, H, dim, generator=g) for L in lens]
    ks = [torch.randn(L, G, dim, generator=g) for L in lens]
    vs = [torch.randn(L, G, vdim, generator=g) for L in lens]
    kc = torch.full((8, G, BS, dim), 7.0)
    vc = torch.full((8, G, BS, vdim), 7.0)
    tables = [[5, 1, 7, 7], [2, 6, 7, 7]]
    for s in range(2):
        for j in range(lens[s]):
            kc[tables[s][j // BS], :, j % BS] = ks[s][j]
            vc[tables[s][j // BS], :, j % BS] = vs[s][j]
    q = torch.cat([qs[0][-news[0]:], qs[1][-news[1]:]]).to(device)
    for short in (0, 32):
        out = torch.zeros(sum(news), H * vdim, device=device)
        ops.attn_keep_window(q, kc.to(device), vc.to(device), vdim, i32(tables, device),
                             i32([0, news[0]], device), i32(list(news), device), i32(list(lens), device),
                             i32([1, 0, 0], device), i32([0, 0, 1], device), None, None, out, scale, 7, 2,
                             False, short_rows=short)
        r = 0
        for s in range(2):
            want = _dense(qs[s], ks[s], vs[s], scale, 7, 2, None, None, False)[-news[s]:]
            close(out[r:r + news[s]], want, 5e-5)
            r += news[s]


# ------------------------------------------------------------------ MFMA tiles
@pytest.mark.gpu
@pytest.mark.parametrize("H,G,E,vdim,shared", [(4, 2, 32, 32, False), (2, 1, 64, 128, False),
                                               (8, 2, 128, 64, False), (3, 3, 64, 64, False),
                                               (4, 1, 96, 64, True), (8, 1, 160, 128, True),
                                               (3, 1, 576, 512, True), (16, 1, 96, 64, True),
                                               (40, 2, 64, 64, False), (48, 1, 160, 128, True)])
@pytest.mark.parametrize("window,keep", [(0, 0), (1, 0), (31, 3), (32, 33), (33, 1), (100, 40)])
@pytest.mark.parametrize("kind", ["softmax", "sink", "sigmoid"])
def test_attention_on_mfma_tiles(H, G, E, vdim, shared, window, keep, kind):
    """bf16 pages with sizes of the MFMA tiles: prompt portions cut inside pages and query blocks
    and decoded rows against the dense computation on the same (rounded) keys and values, and
    against the FMA kernels to within the output's rounding."""
    assert ops.keep_mfma_ok(E, vdim, shared=shared)
    g = torch.Generator().manual_seed(30)
    L, scale = 200, E ** -0.5 * 2
    q = torch.randn(L, H, E, generator=g)
    k = torch.randn(L, G, E, generator=g).bfloat16().float()
    v = k[..., :vdim] if shared else torch.randn(L, G, vdim, generator=g).bfloat16().float()
    bias = None if kind == "softmax" else torch.randn(H, generator=g)
    gate = torch.randn(L, H, generator=g).bfloat16().float() if kind == "sink" else None
    want = _dense(q, k, v, scale, window, keep, bias, gate, kind == "sigmoid")
    sections = [(0, 70), (70, 33), (103, 60), (163, 30)] + [(193 + i, 1) for i in range(7)]
    args = (q, k, None if shared else v, vdim, sections, scale, window, keep, bias, gate, kind == "sigmoid")
    got = _attend("cuda", *args, dtype=torch.bfloat16, mfma=True)
    fma = _attend("cuda", *args, dtype=torch.bfloat16, mfma=False)
    # decoded rows of groups of 16 heads or more: the tiles' columns are heads
    dec = _attend("cuda", *args, dtype=torch.bfloat16, mfma=True, short=True)
    close(dec, want, 6e-3 * (2.0 if E > 320 else 1.0))
    close(got, want, 6e-3 * (2.0 if E > 320 else 1.0))       # bf16 output
    # keys wider than 320 entries meet queries rounded to bf16 (no lo part)
    loose = 4.0 if E > 320 else 1.0
    assert float((got.double() - fma.double()).abs().max()) <= loose * 2.0 ** -7 * float(want.abs().max())
    assert float((got.double() - fma.double()).abs().mean()) <= loose * 2e-4 * float(want.abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("window", [33, 64, 65])
@pytest.mark.parametrize("sigmoid", [False, True])
def test_mfma_tiles_see_the_window_edge_and_the_kept_tokens(window, sigmoid):
    g = torch.Generator().manual_seed(31)
    L, H, G, dim, vdim, keep = 140, 2, 1, 32, 32, 5
    bias = torch.full((H,), -4.0) if sigmoid else None
    for j, seen in ((L - window, True), (L - window - 1, False), (keep - 1, True), (keep, False)):
        q = torch.randn(L, H, dim, generator=g) * 0.1
        k = (torch.randn(L, G, dim, generator=g) * 0.1).bfloat16().float()
        v = torch.randn(L, G, vdim, generator=g).bfloat16().float()
        q[L - 1, :, 0] = 3.0
        k[j, 0, 0] = 3.0
        v[j, 0] = 100.0
        got = _attend("cuda", q, k, v, vdim, [(0, L)], 1.0, window, keep, bias, None, sigmoid,
                      dtype=torch.bfloat16, mfma=True)
        assert (float(got[L - 1, 0]) > 50.0) == seen, (window, j, float(got[L - 1, 0]))
    # the same through the decode rows' form (16 heads of one key head are the columns)
    H = 16
    for j, seen in ((L - window, True), (L - window - 1, False), (keep - 1, True), (keep, False)):
        q = torch.randn(L, H, dim, generator=g) * 0.1
        k = (torch.randn(L, G, dim, generator=g) * 0.1).bfloat16().float()
        v = torch.randn(L, G, vdim, generator=g).bfloat16().float()
        q[L - 1, :, 0] = 3.0
        k[j, 0, 0] = 3.0
        v[j, 0] = 100.0
        hb = torch.full((H,), -4.0) if sigmoid else None
        got = _attend("cuda", q, k, v, vdim, [(0, L - 1), (L - 1, 1)], 1.0, window, keep, hb, None, sigmoid,
                      dtype=torch.bfloat16, mfma=True, short=True)
        assert (float(got[L - 1, 0]) > 50.0) == seen and (float(got[L - 1, 15 * vdim]) > 50.0) == seen
