"""Each Bilolix mechanism alone (package op on CPU tensors or the gfx950 kernel) against the
slow oracle, with inputs made so that a key, a state or a choice missed or wrongly seen shows."""
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


# ------------------------------------------------------------------ residual and norm
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("d", [44, 256, 1030])
def test_residual_of_two_sublayers_step_vector_and_next_norm(device, d):
    """x += y1 + y2 + step, then the next layer's input rms(x) (1 + w): one norm, stored around
    zero; either sublayer output may be absent, and they may come in different types."""
    g = torch.Generator().manual_seed(1)
    T, eps = 5, 1e-3
    x = torch.randn(T, d, generator=g) * 4
    y1, y2 = torch.randn(T, d, generator=g), torch.randn(T, d, generator=g) * 0.3
    step, w = torch.randn(d, generator=g), torch.randn(d, generator=g) * 0.5
    for a, b, s in ((y1, y2, step), (y1, None, None), (None, None, step), (y1, y2, None)):
        want = x.double()
        for t in (a, b, s):
            want = want + (t.double() if t is not None else 0.0)
        xd, out = x.clone().to(device), torch.empty(T, d, device=device)
        dev = [t.to(device) if t is not None else None for t in (a, b, s)]
        ops.residual_add_norm(xd, dev[0], dev[1], dev[2], w.to(device), eps, 1.0, out)
        close(xd, want)
        close(out, oracle.norm_around_zero(want, w.double(), eps))
    # no norm: only the sum; a bf16 mixer output beside an fp32 expert sum, bf16 result
    xd = x.clone().to(device)
    ops.residual_add_norm(xd, y1.to(device).bfloat16(), y2.to(device))
    want = x.double() + y1.bfloat16().double() + y2.double()
    close(xd, want)
    out = torch.empty(T, d, device=device, dtype=torch.bfloat16)
    ops.residual_add_norm(xd, None, None, None, w.to(device), eps, 1.0, out)
    close(out, oracle.norm_around_zero(want, w.double(), eps), 1e-2)


@pytest.mark.parametrize("device", DEVICES)
def test_exact_gelu(device):
    x = torch.linspace(-6, 6, 3999).view(3, -1)
    close(ops.gelu_rows(x.to(device)), oracle.gelu_erf(x.double()), 1e-6)
    wide = torch.randn(4, 70)
    close(ops.gelu_rows(wide.to(device)[:, 3:40]), oracle.gelu_erf(wide[:, 3:40].double()), 1e-6)
    # not the tanh form
    assert float((oracle.gelu_erf(x.double()) - torch.nn.functional.gelu(x.double(), approximate="tanh")).abs().max()) > 1e-4


# ------------------------------------------------------------------ rotation and pages
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,dim,vdim,rot", [(4, 2, 16, 8, 8), (3, 1, 10, 6, 10), (2, 2, 8, 8, 0),
                                              (1, 1, 6, 5, 2), (8, 4, 64, 64, 32), (2, 1, 24, 16, 10)])
@pytest.mark.parametrize("pad", [5, 0])
def test_rotation_of_both_maps_and_cache_append(device, H, G, dim, vdim, rot, pad):
    """Each map of each head is rotated on its own leading dimensions, in neighbouring pairs,
    by the row's position; the rest passes unchanged; v is not rotated; k and v land in the
    page and row that the slot names, wherever that page lies."""
    g = torch.Generator().manual_seed(2)
    T, base, blocks = 9, 777.0, 6
    N = (H + G) * 2 * dim + G * vdim
    wide = torch.randn(T, N + pad, generator=g)          # pad 0: rows the 16-byte kernel takes
    pos = torch.tensor([0, 1, 2, 40, 41, 500, 31, 32, 33])
    slots = torch.tensor([5 * BS + 0, 5 * BS + 1, 2 * BS + 31, 0, 1, -1, 3 * BS + 7, 4 * BS + 30, BS + 2])
    kc = torch.full((blocks, G, BS, 2 * dim), 9.0, device=device)
    vc = torch.full((blocks, G, BS, vdim), 9.0, device=device)
    q = torch.empty(T, H, 2 * dim, device=device)
    ops.rotary_append(wide.to(device)[:, :N], i32(pos.tolist(), device),
                      ops.rotary_inv_freq(rot, base, device), i32(slots.tolist(), device), kc, vc,
                      H, G, 2, dim, vdim, q)
    x = wide[:, :N].double()
    wq = oracle.rotate(x[:, :H * 2 * dim].reshape(T, H, 2, dim), pos, rot, base)
    wk = oracle.rotate(x[:, H * 2 * dim:(H + G) * 2 * dim].reshape(T, G, 2, dim), pos, rot, base)
    wv = x[:, (H + G) * 2 * dim:].reshape(T, G, vdim)
    close(q, wq.reshape(T, H, 2 * dim), 1e-5)
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            close(kc[s // BS, :, s % BS], wk[t].reshape(G, 2 * dim), 1e-5)
            close(vc[s // BS, :, s % BS], wv[t], 0)
    written = {int(s) for s in slots if s >= 0}
    for s in range(blocks * BS):
        if s not in written:
            assert float(kc[s // BS, :, s % BS].min()) == 9.0 and float(vc[s // BS, :, s % BS].max()) == 9.0
    if rot:                                          # the rotation is interleaved, not half-split
        half = x[:, :H * 2 * dim].reshape(T, H, 2, dim).clone()
        assert float((wq - half).abs().max()) > 1e-2


def _paged(k, v, order, device, dtype=torch.float32):
    """k [L, G, 2 dim], v [L, G, vdim] into pools whose pages lie in the given order."""
    L, G = k.shape[:2]
    nb = (L + BS - 1) // BS
    blocks = max(order) + 2
    kc = torch.full((blocks, G, BS, k.shape[2]), 7.0, dtype=dtype)
    vc = torch.full((blocks, G, BS, v.shape[2]), 7.0, dtype=dtype)
    for j in range(L):
        kc[order[j // BS], :, j % BS] = k[j].to(dtype)
        vc[order[j // BS], :, j % BS] = v[j].to(dtype)
    bt = order[:nb] + [blocks - 1] * 3
    return kc.to(device), vc.to(device), bt


def _attend(device, q, k, v, gate, sections, scale, window, lam, eps, mult, dtype=torch.float32,
            mfma=None):
    """sections: [(first row, rows)] of ONE sequence of L rows, each run as its own launch with
    everything before it already cached; returns out [L, H vdim]."""
    L, H = q.shape[:2]
    order = [4, 0, 9, 2, 7, 1, 8, 3, 6, 5, 10, 11, 12, 13, 14][: (L + BS - 1) // BS]
    kc, vc, bt = _paged(k, v, order, device, dtype)
    out = torch.zeros(L, H * v.shape[2], dtype=dtype, device=device)
    for lo, n in sections:
        nblk = (n + ops.DIFF_QBLK - 1) // ops.DIFF_QBLK
        ops.attn_diff_window(q[lo:lo + n].float().contiguous().to(device), kc, vc, i32([bt], device),
                             i32([0], device), i32([n], device), i32([lo + n], device),
                             i32([0] * nblk, device), i32(list(range(nblk)), device),
                             gate[lo:lo + n].to(dtype).to(device), out[lo:lo + n], scale, window,
                             lam, eps, mult, 0, mfma)
    return out


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,dim,vdim", [(4, 2, 16, 8), (3, 3, 40, 24), (2, 1, 8, 72), (8, 2, 64, 64)])
@pytest.mark.parametrize("window", [0, 1, 5, 32, 33, 100])
def test_differential_attention_in_sections(device, H, G, dim, vdim, window):
    """A prompt portion (several query blocks), a short extend and single decoded rows over
    pages that lie in odd order equal the dense computation of the whole sequence."""
    g = torch.Generator().manual_seed(3)
    L, scale, lam, diff, eps = 150, 0.4, 0.37, 0.55, 1e-4
    q = torch.randn(L, H, 2, dim, generator=g)
    k = torch.randn(L, G, 2, dim, generator=g)
    v = torch.randn(L, G, vdim, generator=g)
    gate = torch.randn(L, H, generator=g)
    want = oracle.diff_attention(q.double(), k.double(), v.double(), scale, window, lam, diff, eps,
                                 gate.double()).reshape(L, H * vdim)
    sections = [(0, 70), (70, 3), (73, 45)] + [(118 + i, 1) for i in range(32)]
    got = _attend(device, q.reshape(L, H, 2 * dim), k.reshape(L, G, 2 * dim), v, gate, sections,
                  scale, window, lam, eps, 1.0 - diff)
    close(got, want, 5e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window", [1, 2, 31, 32, 33, 64, 65, 97])
@pytest.mark.parametrize("decoded", [False, True])
def test_a_key_at_the_window_edge_stands_out(device, window, decoded):
    """One key is made to match the last query of map 1 and carries a value far from the
    others: placed on the window's last position inside it owns the output, one position
    further out it must not be seen at all."""
    g = torch.Generator().manual_seed(4)
    L, H, G, dim, vdim, scale, eps = 140, 2, 1, 16, 8, 1.0, 1e-6
    for inside in (True, False):
        q = torch.randn(L, H, 2, dim, generator=g) * 0.1
        k = torch.randn(L, G, 2, dim, generator=g) * 0.1
        v = torch.randn(L, G, vdim, generator=g)
        gate = torch.zeros(L, H)
        j = L - 1 - (window - 1) - (0 if inside else 1)      # just inside / just outside
        q[L - 1, :, 0] = 3.0
        k[j, 0, 0] = 3.0                                     # score 3 * 3 * dim: dominates map 1
        v[j, 0] = 100.0
        want = oracle.diff_attention(q.double(), k.double(), v.double(), scale, window, 0.0, 0.0, eps,
                                     gate.double()).reshape(L, H * vdim)
        # without the head norm the row would be ~100 (seen) or ~1 (not seen); normed, a seen
        # key makes every channel equal, an unseen one leaves the random values' spread
        sections = [(0, L - 1), (L - 1, 1)] if decoded else [(0, L)]
        got = _attend(device, q.reshape(L, H, 2 * dim), k.reshape(L, G, 2 * dim), v, gate, sections,
                      scale, window, 0.0, eps, 1.0)
        close(got, want, 5e-5)
        spread = float(got[L - 1, :vdim].double().std())
        assert (spread < 0.05) == inside, (window, inside, spread)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dim,vdim", [(4, 2, 32, 32), (2, 1, 64, 128), (8, 2, 128, 64), (3, 3, 64, 64)])
@pytest.mark.parametrize("window", [0, 1, 31, 32, 33, 100])
def test_differential_attention_on_mfma_tiles(H, G, dim, vdim, window):
    """bf16 pages with sizes of the MFMA tiles: prompt portions cut inside pages and query
    blocks against the dense computation on the same (rounded) keys and values, and against
    the FMA kernel to within the output's rounding."""
    assert ops.diff_mfma_ok(dim, vdim)
    g = torch.Generator().manual_seed(30)
    L, scale, lam, diff, eps = 200, dim ** -0.5 * 2, 0.37, 0.55, 1e-4
    q = torch.randn(L, H, 2, dim, generator=g)
    k = torch.randn(L, G, 2, dim, generator=g).bfloat16().float()
    v = torch.randn(L, G, vdim, generator=g).bfloat16().float()
    gate = torch.randn(L, H, generator=g).bfloat16().float()
    want = oracle.diff_attention(q.double(), k.double(), v.double(), scale, window, lam, diff, eps,
                                 gate.double()).reshape(L, H * vdim)
    sections = [(0, 70), (70, 33), (103, 97)]
    args = (q.reshape(L, H, 2 * dim), k.reshape(L, G, 2 * dim), v, gate, sections, scale, window,
            lam, eps, 1.0 - diff)
    got = _attend("cuda", *args, dtype=torch.bfloat16, mfma=True)
    fma = _attend("cuda", *args, dtype=torch.bfloat16, mfma=False)
    close(got, want, 6e-3)                                   # bf16 output
    assert float((got.double() - fma.double()).abs().max()) <= 2.0 ** -7 * float(want.abs().max())
    assert float((got.double() - fma.double()).abs().mean()) <= 2e-4 * float(want.abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("window", [33, 64, 65])
def test_mfma_tiles_see_the_window_edge(window):
    """The standing-out key just inside / just outside the window, on the MFMA tiles."""
    g = torch.Generator().manual_seed(31)
    L, H, G, dim, vdim, eps = 140, 2, 1, 32, 32, 1e-6
    for inside in (True, False):
        q = torch.randn(L, H, 2, dim, generator=g) * 0.1
        k = (torch.randn(L, G, 2, dim, generator=g) * 0.1).bfloat16().float()
        v = torch.randn(L, G, vdim, generator=g).bfloat16().float()
        j = L - 1 - (window - 1) - (0 if inside else 1)
        q[L - 1, :, 0] = 3.0
        k[j, 0, 0] = 3.0
        v[j, 0] = 100.0
        got = _attend("cuda", q.reshape(L, H, 2 * dim), k.reshape(L, G, 2 * dim), v, torch.zeros(L, H),
                      [(0, L)], 1.0, window, 0.0, eps, 1.0, dtype=torch.bfloat16, mfma=True)
        spread = float(got[L - 1, :vdim].double().std())
        assert (spread < 0.05) == inside, (window, inside, spread)


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds_without_window(device):
    g = torch.Generator().manual_seed(5)
    L, H, G, dim, vdim = 450, 2, 2, 8, 8
    q = torch.randn(L, H, 2, dim, generator=g) * 0.1
    k = torch.randn(L, G, 2, dim, generator=g) * 0.1
    v = torch.randn(L, G, vdim, generator=g)
    q[L - 1, 1, 1] = 4.0
    k[3, 1, 1] = 4.0                                         # map 2 of head 1 finds token 3
    v[3, 1] = 50.0
    gate = torch.randn(L, H, generator=g)
    want = oracle.diff_attention(q.double(), k.double(), v.double(), 1.0, 0, 0.5, 0.1, 1e-5,
                                 gate.double()).reshape(L, H * vdim)
    for sections in ([(0, L)], [(0, L - 1), (L - 1, 1)]):
        got = _attend(device, q.reshape(L, H, 2 * dim), k.reshape(L, G, 2 * dim), v, gate, sections,
                      1.0, 0, 0.5, 1e-5, 0.9)
        close(got, want, 5e-5)
    assert float(want[L - 1, vdim:].std()) < 0.05           # the far value owns head 1's output


@pytest.mark.parametrize("device", DEVICES)
def test_two_sequences_one_launch_and_lambda(device):
    """Work items of two sequences of unequal length in one launch; lambda weighs map 2."""
    g = torch.Generator().manual_seed(6)
    H, G, dim, vdim, scale, eps = 3, 1, 8, 8, 0.5, 1e-5
    lens, news = (50, 9), (40, 9)                              # kv lengths, new rows
    qs, outs_want, kcs, vcs, bts = [], [], [], [], []
    lam = oracle.diff_lambda(torch.full((dim,), 0.2, dtype=D64), torch.full((dim,), 0.3, dtype=D64),
                             torch.full((dim,), -0.1, dtype=D64), torch.full((dim,), 0.4, dtype=D64), 0.8)
    assert abs(lam - (math.exp(0.48) - math.exp(-0.32) + 0.8)) < 1e-12
    kc = torch.zeros(8, G, BS, 2 * dim)
    vc = torch.zeros(8, G, BS, vdim)
    tables = [[5, 1, 7, 7], [3, 6, 7, 7]]
    gate_all = []
    for s, (L, n) in enumerate(zip(lens, news)):
        q = torch.randn(L, H, 2, dim, generator=g)
        k = torch.randn(L, G, 2, dim, generator=g)
        v = torch.randn(L, G, vdim, generator=g)
        gate = torch.randn(L, H, generator=g)
        for j in range(L):
            kc[tables[s][j // BS], :, j % BS] = k[j].reshape(G, 2 * dim)
            vc[tables[s][j // BS], :, j % BS] = v[j]
        w = oracle.diff_attention(q.double(), k.double(), v.double(), scale, 12, lam, 0.8, eps, gate.double())
        outs_want.append(w[L - n:].reshape(n, H * vdim))
        qs.append(q[L - n:].reshape(n, H, 2 * dim))
        gate_all.append(gate[L - n:])
    qd = torch.cat(qs).to(device)
    out = torch.zeros(sum(news), H * vdim, device=device)
    nblk = [(n + ops.DIFF_QBLK - 1) // ops.DIFF_QBLK for n in news]
    ops.attn_diff_window(qd, kc.to(device), vc.to(device), i32(tables, device), i32([0, news[0]], device),
                         i32(list(news), device), i32(list(lens), device),
                         i32([0] * nblk[0] + [1] * nblk[1], device),
                         i32(list(range(nblk[0])) + list(range(nblk[1])), device),
                         torch.cat(gate_all).to(device), out, scale, 12, lam, eps, 0.2)
    close(out, torch.cat(outs_want), 5e-5)


# ------------------------------------------------------------------ state slots
def run_rows(cuts, slot, gen0=0, pos0=0):
    """row_state / row_back / row_fwd / positions of a sequence's portions, one launch each."""
    at, gen = pos0, gen0
    for n in cuts:
        yield at - pos0, n, ([slot * 2 + (gen & 1)] * n, list(range(n)), list(range(n - 1, -1, -1)),
                             list(range(at, at + n)))
        at += n
        gen += 1


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 4, 5])
@pytest.mark.parametrize("cuts", [[50], [1] * 50, [2, 1, 3, 44], [3, 3, 1, 1, 2, 40]])
def test_convolution_in_portions(device, taps, cuts):
    """silu(conv) in portions through a slot with another sequence's rest equals the whole
    sequence's; the first tokens see zeros; the leading heads come out as unit vectors."""
    g = torch.Generator().manual_seed(7)
    T, S, slot, dim, n_unit = sum(cuts), 3, 2, 6, 3
    C = n_unit * dim + 11
    wide = torch.randn(T, C + 4, generator=g)
    x = wide[:, 2:2 + C]
    w = torch.randn(C, taps, generator=g)
    y = oracle.silu(oracle.causal_conv(x.double(), w.double()))
    want = y.clone()
    want[:, :n_unit * dim] = oracle.unit_vectors(y[:, :n_unit * dim].reshape(T, n_unit, dim)).reshape(T, -1)
    state = (torch.randn(2 * S, taps - 1, C, generator=g) * 100).to(device)
    outs = []
    for lo, n, rows in run_rows(cuts, slot):
        out = torch.empty(n, C, device=device)
        ops.conv_act_heads(wide.to(device)[lo:lo + n, 2:2 + C], w.to(device), state,
                           *(i32(r, device) for r in rows), n_unit, dim, 1e-6, out)
        outs.append(out.cpu())
    close(torch.cat(outs), want)


def _scan_inputs(g, T, H, Hq, dim, vdim):
    q = torch.randn(T, Hq, dim, generator=g)
    k = torch.randn(T, Hq, dim, generator=g) * 0.5
    v = torch.randn(T, H, vdim, generator=g)
    z = torch.randn(T, H * dim, generator=g) * 2
    gate = torch.randn(T, H * vdim, generator=g)
    beta = torch.randn(T, H, generator=g)
    return q, k, v, z, gate, beta


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,Hq,dim,vdim", [(2, 2, 32, 64), (3, 3, 16, 24), (1, 1, 7, 5), (2, 1, 64, 32),
                                           (4, 2, 128, 16), (2, 2, 40, 100)])
@pytest.mark.parametrize("cuts", [[40], [1] * 40, [2, 1, 33, 4], [17, 2, 2, 19], [150, 3, 1]])
@pytest.mark.parametrize("mode", ["gla", "delta"])
def test_linear_recurrence_in_portions(device, H, Hq, dim, vdim, cuts, mode):
    """The recurrence in portions through a state slot with stale contents equals the scan of
    the whole sequence: the decay acts on key channels, the read-out sees the token's own
    write, the delta rule subtracts what the state already holds for the key.  (A long portion
    has its decays formed ahead of the scan on the GPU, short ones inside it.)"""
    g = torch.Generator().manual_seed(8)
    T, S, slot, eps, scale = sum(cuts), 2, 1, 1e-4, dim ** -0.5
    q, k, v, z, gate, beta = _scan_inputs(g, T, H, Hq, dim, vdim)
    zb = torch.randn(H * dim, generator=g)
    nw = torch.randn(vdim, generator=g)
    rep = H // Hq
    qq, kk = q.double().repeat_interleave(rep, 1), k.double().repeat_interleave(rep, 1)
    if mode == "gla":
        tau = 4.0
        rate, sign = torch.full((H,), 1.0 / tau), -1.0
        a = oracle.decay_sigmoid_pow(z.double() + zb.double(), tau).view(T, H, dim)
        o, _ = oracle.linear_scan(qq * scale, kk, v.double(), a)
        act = oracle.silu(gate.double())
    else:
        a_log = torch.randn(H, generator=g) * 0.5 - 0.5
        rate, sign = torch.exp(a_log.double()).float(), 1.0
        kk = oracle.unit_vectors(kk)
        k = oracle.unit_vectors(k.double()).float()
        a = oracle.decay_softplus((z.double() + zb.double()).view(T, H, dim), a_log.double())
        o, _ = oracle.linear_scan(qq * scale, kk, v.double(), a, torch.sigmoid(beta.double()))
        act = torch.sigmoid(gate.double())
    want = (oracle.rms_unit(o, eps) * nw.double()).reshape(T, H * vdim) * act
    state = (torch.randn(2 * S, H, dim, vdim, generator=g) * 50).to(device)
    outs = []
    for lo, n, rows in run_rows(cuts, slot):
        out = torch.empty(n, H * vdim, device=device)
        r = [i32(x, device) for x in rows]
        ops.gated_linear_recurrence(
            q[lo:lo + n].to(device), k[lo:lo + n].to(device), v[lo:lo + n].to(device),
            z[lo:lo + n].to(device), rate.to(device), zb.to(device), sign,
            beta[lo:lo + n].to(device) if mode == "delta" else None, gate[lo:lo + n].to(device),
            mode == "delta", nw.to(device), eps, scale, state, *r, out,
            i32([0], device) if device != "cpu" else None)
        outs.append(out.cpu())
    close(torch.cat(outs), want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_recurrence_two_sequences_one_launch_and_strided_inputs(device):
    """Two runs in one launch (one continues from its slot, one starts), operands that are
    column slices of one wide matrix; the new states land in the other halves."""
    g = torch.Generator().manual_seed(9)
    H, dim, vdim, eps = 2, 8, 12, 1e-5
    na, nb = 5, 3
    T = na + nb
    N = 2 * H * dim + 2 * H * vdim + 3
    wide = torch.randn(T, N, generator=g)
    z = torch.randn(T, H * dim, generator=g)
    rate, zb, nw = torch.rand(H, generator=g) + 0.1, torch.randn(H * dim, generator=g), torch.randn(vdim, generator=g)
    prev = torch.randn(H, dim, vdim, generator=g)
    state = torch.zeros(4, H, dim, vdim)
    state[0] = prev                                       # slot 0, half 0: a's state so far
    state[1] = 99.0                                       # slot 1, half 0: stale, b starts anew
    rs = [0] * na + [2] * nb
    rb = list(range(na)) + list(range(nb))
    rf = list(range(na - 1, -1, -1)) + list(range(nb - 1, -1, -1))
    pos = list(range(7, 7 + na)) + list(range(nb))
    wd = wide.to(device)
    cols = lambda a, n, h: wd[:, a:a + n].unflatten(1, (h, n // h))      # noqa: E731
    sd = state.to(device)
    out = torch.empty(T, H * vdim, device=device)
    ops.gated_linear_recurrence(cols(0, H * dim, H), cols(H * dim, H * dim, H), cols(2 * H * dim, H * vdim, H),
                                z.to(device), rate.to(device), zb.to(device), -1.0, None,
                                wd[:, 2 * H * dim + H * vdim:2 * H * dim + 2 * H * vdim], False,
                                nw.to(device), eps, 1.0, sd, *(i32(r, device) for r in (rs, rb, rf, pos)),
                                out, i32([0, na], device) if device != "cpu" else None)
    x = wide.double()
    qq = x[:, :H * dim].reshape(T, H, dim)
    kk = x[:, H * dim:2 * H * dim].reshape(T, H, dim)
    vv = x[:, 2 * H * dim:2 * H * dim + H * vdim].reshape(T, H, vdim)
    gg = x[:, 2 * H * dim + H * vdim:2 * H * dim + 2 * H * vdim]
    a = torch.exp(-rate.double()[None, :, None] * torch.log1p(torch.exp(-(z.double() + zb.double()))).view(T, H, dim))
    oa, sa = oracle.linear_scan(qq[:na], kk[:na], vv[:na], a[:na], state=prev.double())
    ob, sb = oracle.linear_scan(qq[na:], kk[na:], vv[na:], a[na:])
    want = (oracle.rms_unit(torch.cat([oa, ob]), eps) * nw.double()).reshape(T, H * vdim) * oracle.silu(gg)
    close(out, want, 1e-4)
    close(sd[2], sa, 1e-4)                                 # other half of slot 0
    close(sd[3], sb, 1e-4)                                 # other half of slot 1
    close(sd[0], prev, 0)                                  # the read halves are untouched


# ------------------------------------------------------------------ routing
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top", [(12, 2), (5, 5), (7, 1), (64, 6)])
def test_routing_softmax_over_the_chosen(device, E, top):
    g = torch.Generator().manual_seed(10)
    T = 37
    z = torch.randn(T, E, generator=g) * 2
    b = torch.randn(E, generator=g)
    z[0] = 1.0                                                 # all tied: the lowest indices win
    b0 = b.clone()
    ids = torch.empty(T, top, dtype=torch.int32, device=device)
    wts = torch.empty(T, top, device=device)
    ops.moe_route_topk(z.to(device), b.to(device), top, ids, wts)
    wi, ww = oracle.route_top(z.double() + b0.double(), top)
    assert torch.equal(ids.cpu().long(), wi)
    close(wts, ww, 1e-6)
    close(wts.sum(-1), torch.ones(T), 1e-6)
    # the weights are NOT the softmax over all experts
    if top < E:
        full = torch.softmax(z.double() + b0.double(), -1).gather(1, wi)
        assert float((full - ww).abs().max()) > 1e-3
    ops.moe_route_topk(z.to(device), None, top, ids, wts)
    assert torch.equal(ids.cpu().long(), oracle.route_top(z.double(), top)[0])
    assert ids[0].tolist() == list(range(top))
