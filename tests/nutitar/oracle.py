"""A slow float64 implementation of Nutitar written from its equations, one function per
mechanism.  It shares no code with the package: the configuration comes as the dictionary of a
checkpoint's config.json, tensors by their checkpoint names, and whole sequences are computed at
once with dense masks."""
import math

import torch

D64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w)


def softplus(x):
    return math.log1p(math.exp(x))


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z / 2."""
    ap, an = softplus(float(p)), 0.5 + softplus(float(q))
    zn = torch.clamp(z, max=0.0)
    return torch.where(z > 0, ap * z * z + 0.5 * z, an * (torch.exp(zn) - 1.0 - zn) + 0.5 * zn)


def token_shift(h, shift, before=None):
    """h [T, d] -> h + (h' - h) shift with h' the row above (``before`` or zeros for row 0)."""
    first = torch.zeros_like(h[:1]) if before is None else before.view(1, -1)
    prev = torch.cat([first, h[:-1]], 0)
    return h + (prev - h) * shift


# ------------------------------------------------------------------ rotation
def base_frequencies(dims, base):
    i = torch.arange(dims // 2, dtype=D64)
    return base ** (-2.0 * i / dims)


def yarn_frequencies(dims, base, factor, original, fast, slow):
    """Returns (frequencies, multiplier of cos and sin)."""
    f = base_frequencies(dims, base)

    def dim_of(t):
        return dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(fast)), 0)
    hi = min(math.ceil(dim_of(slow)), dims - 1)
    i = torch.arange(dims // 2, dtype=D64)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def banded_frequencies(dims, base, factor, low, high, original):
    """Long wavelengths are stretched by ``factor``, short ones kept, a blend between."""
    f = base_frequencies(dims, base)
    out = f.clone()
    for n in range(f.numel()):
        fi = float(f[n])
        wl = 2.0 * math.pi / fi
        if wl < original / high:
            out[n] = fi
        elif wl > original / low:
            out[n] = fi / factor
        else:
            s = (original / wl - low) / (high - low)
            out[n] = (1.0 - s) * fi / factor + s * fi
    return out


def frequencies(rot):
    """rot: the ``rot`` entry of a mixer's configuration."""
    sc = rot.get("scaling")
    if not sc:
        return base_frequencies(rot["dims"], rot["base"]), 1.0
    if "fast" in sc:
        return yarn_frequencies(rot["dims"], rot["base"], sc["factor"], sc["original"], sc["fast"],
                                sc["slow"])
    return banded_frequencies(rot["dims"], rot["base"], sc["factor"], sc["low"], sc["high"],
                              sc["original"]), 1.0


def rotate_half(x, positions, freq, mult=1.0):
    """x [T, ..., n]: entry i pairs with entry i + dims/2 (dims = 2 len(freq) <= n)."""
    half = freq.numel()
    if half == 0:
        return x
    ang = positions.to(D64)[:, None] * freq[None]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (half,)
    c, s = (torch.cos(ang) * mult).view(shape), (torch.sin(ang) * mult).view(shape)
    y = x.clone()
    u, v = x[..., :half], x[..., half:2 * half]
    y[..., :half] = u * c - v * s
    y[..., half:2 * half] = v * c + u * s
    return y


# ------------------------------------------------------------------ masks and weights
def visible(pos_q, pos_k, window=0, keep_first=0):
    i, j = pos_q[:, None], pos_k[None, :]
    ok = j <= i
    if window > 0:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def softmax_weights(scores, ok, sink=None):
    """scores [T, S]; the denominator also holds exp(sink) when a sink is given."""
    s = scores.masked_fill(~ok, -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.clamp(m, min=float(sink))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink - m)
    return e / den


def sigmoid_weights(scores, ok, bias):
    return sigmoid(scores + bias) * ok.to(D64)


# ------------------------------------------------------------------ mixers
def latent_kv(m, w, pre, h, pos, eps):
    """What a latent-attention layer caches per token: (c [T, R], rotated shared key [T, rot_dim])."""
    R = m["kv_rank"]
    d = h @ w[pre + "dkv"].T
    c = rms_unit(d[:, :R], eps) * w[pre + "dkv.norm"]
    f, mult = frequencies(m["rot"])
    return c, rotate_half(d[:, R:], pos, f, mult)


def latent_attention(m, w, pre, h, pos, eps, kv):
    T = h.shape[0]
    H, dim, rd, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, kr = kv
    q = (h @ w[pre + "q"].T).view(T, H, dim + rd)
    f, mult = frequencies(m["rot"])
    qn, qr = q[..., :dim], rotate_half(q[..., dim:], pos, f, mult)
    kn = (c @ w[pre + "uk"].T).view(T, H, dim)
    v = (c @ w[pre + "uv"].T).view(T, H, vd)
    gate = sigmoid(h @ w[pre + "g"].T)                               # [T, H]
    ok = visible(pos, pos)
    out = torch.zeros(T, H, vd, dtype=D64)
    for hh in range(H):
        s = (qn[:, hh] @ kn[:, hh].T + qr[:, hh] @ kr.T) * m["scale"]
        out[:, hh] = softmax_weights(s, ok, w[pre + "sink"][hh]) @ v[:, hh]
        out[:, hh] *= gate[:, hh:hh + 1]
    return out.reshape(T, H * vd) @ w[pre + "o"].T


def gated_window_attention(m, w, pre, h, pos, eps):
    """'attention': biased projections, norms over the whole projection, plain rotation,
    sliding window with kept first tokens, sigmoid weights."""
    T = h.shape[0]
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[pre + "q"].T + w[pre + "q.b"]
    k = h @ w[pre + "k"].T + w[pre + "k.b"]
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).view(T, G, vd)
    q = (rms_unit(q, eps) * w[pre + "q.norm"]).view(T, H, dim)
    k = (rms_unit(k, eps) * w[pre + "k.norm"]).view(T, G, dim)
    f, mult = frequencies(m["rot"])
    q, k = rotate_half(q, pos, f, mult), rotate_half(k, pos, f, mult)
    mask = m.get("mask") or {}
    ok = visible(pos, pos, mask.get("size", 0), mask.get("keep_first", 0))
    out = torch.zeros(T, H, vd, dtype=D64)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"]
        out[:, hh] = sigmoid_weights(s, ok, w[pre + "pb"][hh]) @ v[:, g]
    return out.reshape(T, H * vd) @ w[pre + "o"].T + w[pre + "o.b"]


def key_value_attention(m, w, pre, h, pos, eps):
    """'attention_2': values are the keys as projected, per-head norms, banded frequencies,
    causal softmax."""
    T = h.shape[0]
    H, G, dim = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[pre + "q"].T).view(T, H, dim)
    k = (h @ w[pre + "k"].T).view(T, G, dim)
    v = k.clone()
    q = rms_unit(q, eps) * w[pre + "q.norm"]
    k = rms_unit(k, eps) * w[pre + "k.norm"]
    f, mult = frequencies(m["rot"])
    q, k = rotate_half(q, pos, f, mult), rotate_half(k, pos, f, mult)
    ok = visible(pos, pos)
    out = torch.zeros(T, H, dim, dtype=D64)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"]
        out[:, hh] = softmax_weights(s, ok) @ v[:, g]
    return out.reshape(T, H * dim) @ w[pre + "o"].T


def feed_forward(w, pre, h):
    p, q = w[pre + "act"]
    return xielu(h @ w[pre + "up"].T, p, q) @ w[pre + "down"].T


# ------------------------------------------------------------------ model
def forward(cfg, weights, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence; ``layers_out`` receives the stream after every
    layer."""
    w = {k: v.to(D64) for k, v in weights.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(ids.numel())
    x = w["embed"][ids] * cfg["embedding"]["scale"]
    cached = {}
    for i, ly in enumerate(cfg["layers"]):
        L = "l%d." % i
        m = ly["mixer"]
        h = norm_around_zero(x, w[L + "norm1"], eps)
        hs = token_shift(h, w[L + "shift"]) if L + "shift" in w else h
        if ly["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                cached[i] = latent_kv(m, w, L + "mix.", hs, pos, eps)
                src = i
            y = latent_attention(m, w, L + "mix.", hs, pos, eps, cached[src])
        elif ly["type"] == "attention":
            y = gated_window_attention(m, w, L + "mix.", hs, pos, eps)
        elif ly["type"] == "attention_2":
            y = key_value_attention(m, w, L + "mix.", hs, pos, eps)
        else:
            raise ValueError(ly["type"])
        if ly.get("mlp") is not None:
            y = y + feed_forward(w, L + "mlp.", h)
        x = x + mult * y
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_around_zero(x, w["final.norm"], eps) @ w["head"].T


def greedy(cfg, weights, prompt, n):
    """n tokens after the prompt, each the largest logit of the sequence so far."""
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(cfg, weights, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
