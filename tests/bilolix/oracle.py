"""A slow float64 implementation of Bilolix written from its equations, one function per
mechanism.  It shares no code with the package: tensors come by their checkpoint names, whole
sequences are computed at once with dense masks and token-by-token scans."""
import math

import torch

D64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w)


def silu(x):
    return x / (1.0 + torch.exp(-x))


def gelu_erf(x):
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def rotate(x, positions, rot_dims, base):
    """x [T, ..., dim]: entries (2i, 2i+1), i < rot_dims / 2, turn by positions * base^(-2i / rot_dims)."""
    if rot_dims == 0:
        return x
    i = torch.arange(rot_dims // 2, dtype=D64)
    ang = positions.to(D64)[:, None] * base ** (-2.0 * i / rot_dims)[None]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (rot_dims // 2,)
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    y = x.clone()
    u, v = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
    y[..., 0:rot_dims:2] = u * c - v * s
    y[..., 1:rot_dims:2] = v * c + u * s
    return y


def window_mask(T, window):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < window) if window > 0 else (j >= 0))


def diff_lambda(lq1, lk1, lq2, lk2, diff):
    return math.exp(float(lq1 @ lk1)) - math.exp(float(lq2 @ lk2)) + diff


def diff_attention(q, k, v, scale, window, lam, diff, eps, gate_logits):
    """q [T, H, 2, dim], k [T, G, 2, dim] (rotated), v [T, G, vdim], gate_logits [T, H]."""
    T, H = q.shape[:2]
    G = k.shape[1]
    ok = window_mask(T, window)
    out = torch.zeros(T, H, v.shape[-1], dtype=D64)
    for h in range(H):
        c = h // (H // G)
        a = []
        for mp in range(2):
            s = (q[:, h, mp] @ k[:, c, mp].T) * scale
            s = s.masked_fill(~ok, float("-inf"))
            a.append(torch.softmax(s, -1) @ v[:, c])
        o = rms_unit(a[0] - lam * a[1], eps) * (1.0 - diff)
        out[:, h] = o * torch.sigmoid(gate_logits[:, h:h + 1])
    return out


def decay_sigmoid_pow(z, tau):
    return torch.sigmoid(z) ** (1.0 / tau)


def decay_softplus(z, a_log):
    """z [T, H, dim], a_log [H]."""
    return torch.exp(-torch.exp(a_log)[None, :, None] * torch.log1p(torch.exp(z)))


def linear_scan(q, k, v, a, beta=None, state=None):
    """q, k [T, H, dim], v [T, H, vdim], a [T, H, dim], beta [T, H] or None.
    S <- diag(a) S; u = beta (v - S^T k) or v; S <- S + k u^T; o = S^T q."""
    T, H, dim = q.shape
    S = torch.zeros(H, dim, v.shape[-1], dtype=D64) if state is None else state.clone()
    o = torch.zeros(T, H, v.shape[-1], dtype=D64)
    for t in range(T):
        for h in range(H):
            S[h] = a[t, h][:, None] * S[h]
            u = v[t, h] if beta is None else beta[t, h] * (v[t, h] - S[h].T @ k[t, h])
            S[h] = S[h] + torch.outer(k[t, h], u)
            o[t, h] = S[h].T @ q[t, h]
    return o, S


def causal_conv(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] x_(t - (taps-1-j)), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=D64), x], 0)
    y = torch.zeros(T, C, dtype=D64)
    for j in range(taps):
        y += xp[j:j + T] * w[:, j]
    return y


def unit_vectors(x, eps=1e-6):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def route_top(z, top):
    """The top largest logits per row (ties to the lower index) and the softmax over them."""
    order = torch.argsort(z, dim=-1, descending=True, stable=True)[:, :top]
    return order, torch.softmax(torch.gather(z, 1, order), -1)


# ------------------------------------------------------------------ whole model
def _mixer_attention(W, p, m, h, eps):
    T = h.shape[0]
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate((h @ W[p + "q"].T).view(T, H, 2, dim), pos, rot["dims"], rot["base"])
    k = rotate((h @ W[p + "k"].T).view(T, G, 2, dim), pos, rot["dims"], rot["base"])
    v = (h @ W[p + "v"].T).view(T, G, vd)
    lam = diff_lambda(W[p + "lq1"], W[p + "lk1"], W[p + "lq2"], W[p + "lk2"], m["diff"])
    o = diff_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size", 0), lam, m["diff"],
                       eps, h @ W[p + "g"].T)
    return o.reshape(T, H * vd) @ W[p + "o"].T


def _mixer_gla(W, p, m, h, eps):
    T = h.shape[0]
    H, dim, vd = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, dim) * dim ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, dim)
    v = (h @ W[p + "v"].T).view(T, H, vd)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    o, _ = linear_scan(q, k, v, decay_sigmoid_pow(z, m["tau"]).view(T, H, dim))
    o = rms_unit(o, eps) * W[p + "norm"]
    return (o.reshape(T, H * vd) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def _mixer_delta(W, p, m, h, eps):
    T = h.shape[0]
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rep = H // G
    q = silu(causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, dim)
    k = silu(causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, dim)
    v = silu(causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, vd)
    q = (unit_vectors(q) * dim ** -0.5).repeat_interleave(rep, 1)
    k = unit_vectors(k).repeat_interleave(rep, 1)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    z = ((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]).view(T, H, dim)
    o, _ = linear_scan(q, k, v, decay_softplus(z, W[p + "A_log"]), beta)
    o = rms_unit(o, eps) * W[p + "norm"]
    gate = torch.sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T)
    return (o.reshape(T, H * vd) * gate) @ W[p + "o"].T


def _mlp(W, p, f, h):
    if f["kind"] == "dense":
        return gelu_erf(h @ W[p + "up"].T) @ W[p + "down"].T
    ids, wts = route_top(h @ W[p + "router"].T + W[p + "router.b"], f["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t].tolist(), wts[t]):
            pe = f"{p}e{e}."
            out[t] += wt * ((silu(h[t] @ W[pe + "gate"].T) * (h[t] @ W[pe + "up"].T)) @ W[pe + "down"].T)
    return out


def layer_runs(cfg):
    """[(layer index, pass number or None)] in execution order; the pass number is set on the
    first layer of a pass of the looped span."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp or lp["stop"] <= lp["start"]:
        return [(i, None) for i in range(n)]
    out = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        out += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return out + [(i, None) for i in range(lp["stop"], n)]


def forward(cfg, full, tokens, taps=None):
    """Logits [T, vocab] (float64) of one whole sequence; ``taps`` receives the residual
    stream after every layer run."""
    W = {k: v.to(D64) for k, v in full.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    for li, t in layer_runs(cfg):
        if t is not None:
            x = x + W["loop.step"][t]
        ly, p = cfg["layers"][li], f"l{li}."
        h = norm_around_zero(x, W[p + "norm1"], eps)
        mix = {"attention": _mixer_attention, "gla": _mixer_gla, "channel_delta": _mixer_delta}[ly["type"]]
        y = mix(W, p + "mix.", ly["mixer"], h, eps)
        if ly.get("mlp") is not None:
            y = y + _mlp(W, p + "mlp.", ly["mlp"], h)
        x = x + y
        if taps is not None:
            taps.append(x.clone())
    return norm_around_zero(x, W["final.norm"], eps) @ W["head"].T


def greedy(cfg, full, prompt, n):
    """n greedily chosen tokens after the prompt (the whole sequence is recomputed each time)."""
    seq, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(forward(cfg, full, seq)[-1]))
        seq.append(nxt)
        out.append(nxt)
    return out
