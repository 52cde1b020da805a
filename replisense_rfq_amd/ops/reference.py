"""Plain PyTorch (fp32-accumulating) reference implementations of every HIP op.

These are (a) the numerics oracles the kernel tests compare against and (b) the
CPU execution path used by the engine when no GPU is present (unit tests of the
scheduler / grammar / service layers run the whole model on CPU through them).
They mirror the kernels' exact contracts: paged KV layout
``[num_blocks, Hkv, BS, D]``, in-place q rotation inside the fused QKV buffer,
Gumbel-max sampling with the same counter-based hash, etc.
"""
from __future__ import annotations

import math

import torch

MASK64 = (1 << 64) - 1


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_((xf * r * w.float()).to(out.dtype))


def fused_add_rms_norm(x, residual, w, eps, out) -> None:
    s = (x.float() + residual.float()).to(residual.dtype)
    residual.copy_(s)
    rms_norm(s, w, eps, out)


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    F = out.shape[1]
    g, u = gate_up[:, :F], gate_up[:, F:]
    out.copy_((torch.nn.functional.silu(g.float()).to(g.dtype).float() * u.float()).to(out.dtype))


def embed(ids, table, out, vocab_start: int = 0) -> None:
    V = table.shape[0]
    local = ids.long() - vocab_start
    ok = (local >= 0) & (local < V)
    rows = table[local.clamp(0, V - 1)]
    out.copy_(torch.where(ok[:, None], rows, torch.zeros_like(rows)))


def rope_cos_sin(max_pos: int, head_dim: int, theta: float, device="cpu") -> torch.Tensor:
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv)
    return torch.cat([f.cos(), f.sin()], dim=-1).float().to(device)


def rope_kv(qkv, positions, cos_sin, slot_mapping, k_cache, v_cache, Hq: int, Hkv: int) -> None:
    D = 128
    T = qkv.shape[0]
    if T == 0:
        return
    BS = k_cache.shape[2]
    cs = cos_sin[positions[:T].long()]
    c, s = cs[:, None, : D // 2], cs[:, None, D // 2:]

    def rot(x):
        x1, x2 = x[..., : D // 2].float(), x[..., D // 2:].float()
        return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1).to(x.dtype)

    q = qkv[:, : Hq * D].view(T, Hq, D)
    k = qkv[:, Hq * D:(Hq + Hkv) * D].view(T, Hkv, D)
    v = qkv[:, (Hq + Hkv) * D:(Hq + 2 * Hkv) * D].view(T, Hkv, D)
    q.copy_(rot(q))
    kr = rot(k)
    slots = slot_mapping[:T].long()
    ok = slots >= 0
    if ok.any():
        sl = slots[ok]
        blk, off = sl // BS, sl % BS
        k_cache[blk, :, off] = kr[ok]
        v_cache[blk, :, off] = v[ok]


def _gather_kv(cache, block_table, n: int):
    BS = cache.shape[2]
    nb = (n + BS - 1) // BS
    pages = cache[block_table[:nb].long()]             # [nb, Hkv, BS, D]
    return pages.permute(1, 0, 2, 3).reshape(cache.shape[1], nb * BS, -1)[:, :n]


def attn_prefill(q, k_cache, v_cache, block_tables, seq_q_start, seq_q_len, seq_kv_len,
                 work_seq, work_qblk, out, Hq: int, Hkv: int, scale: float) -> None:
    G = Hq // Hkv
    for b in range(seq_q_len.shape[0]):
        ql, kl, t0 = int(seq_q_len[b]), int(seq_kv_len[b]), int(seq_q_start[b])
        if ql == 0:
            continue
        k = _gather_kv(k_cache, block_tables[b], kl).float()
        v = _gather_kv(v_cache, block_tables[b], kl).float()
        k = k.repeat_interleave(G, 0)
        v = v.repeat_interleave(G, 0)
        qb = q[t0:t0 + ql, : Hq * 128].view(ql, Hq, 128).permute(1, 0, 2).float()
        s = torch.einsum("hqd,hkd->hqk", qb, k) * scale
        qpos = torch.arange(kl - ql, kl, device=q.device)[:, None]
        kpos = torch.arange(kl, device=q.device)[None, :]
        s = s.masked_fill(kpos > qpos, float("-inf"))
        o = torch.einsum("hqk,hkd->hqd", torch.softmax(s, -1), v)
        out[t0:t0 + ql, : Hq * 128].copy_(o.permute(1, 0, 2).reshape(ql, -1).to(out.dtype))


def _mix64(x: torch.Tensor) -> torch.Tensor:
    """splitmix-style finaliser on int64 tensors (wrapping arithmetic)."""
    def lsr(v, n):
        return (v >> n) & ((1 << (64 - n)) - 1)
    x = x ^ lsr(x, 33)
    x = x * torch.tensor(0xff51afd7ed558ccd - (1 << 64), dtype=torch.int64)
    x = x ^ lsr(x, 33)
    x = x * torch.tensor(0xc4ceb9fe1a85ec53 - (1 << 64), dtype=torch.int64)
    x = x ^ lsr(x, 33)
    return x


def gumbel_noise(seed: int, cols: torch.Tensor) -> torch.Tensor:
    """Same noise as the kernel's hash_u32(seed, 0x9e3779b9, col) -> Gumbel(0,1)."""
    s = seed & MASK64
    s = s - (1 << 64) if s >= (1 << 63) else s
    base = (0x9E3779B9 << 32)
    base = base - (1 << 64) if base >= (1 << 63) else base
    x = torch.tensor(s, dtype=torch.int64) ^ (torch.tensor(base, dtype=torch.int64) | cols.long())
    h = _mix64(x) & 0xFFFFFFFF
    u = ((h >> 8).double() + 0.5) * (1.0 / 16777216.0)
    return (-torch.log(-torch.log(u))).float()


def sample(logits: torch.Tensor, mask_table: torch.Tensor | None, mask_idx: torch.Tensor,
           temps: torch.Tensor, seeds: torch.Tensor, v0: int = 0):
    """Returns (best_val[B], best_idx[B]) over the local vocab shard (global ids)."""
    B, Vl = logits.shape
    cols = torch.arange(v0, v0 + Vl)
    vals = torch.empty(B)
    idxs = torch.empty(B, dtype=torch.int32)
    for b in range(B):
        sc = logits[b].float().cpu()
        t = float(temps[b])
        if t > 0:
            sc = sc / t + gumbel_noise(int(seeds[b]), cols)
        mi = int(mask_idx[b])
        if mask_table is not None and mi >= 0:
            words = mask_table[mi].cpu().long() & 0xFFFFFFFF
            bits = (words[cols >> 5] >> (cols & 31)) & 1
            sc = sc.masked_fill(bits == 0, float("-inf"))
        j = int(torch.argmax(sc))
        vals[b] = sc[j]
        idxs[b] = v0 + j
    return vals, idxs


def moe_topk(router_logits, topk: int, renorm: bool):
    p = torch.softmax(router_logits.float(), -1)
    # ties (equal bf16 logits) go to the lower expert index, as in moe_topk_kernel
    order = torch.sort(router_logits.float(), dim=-1, descending=True, stable=True).indices
    ids = order[..., :topk]
    w = p.gather(-1, ids)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return w, ids.int()


def moe_forward(x, w13, w2, router_logits, topk: int, expert_offset: int = 0):
    """Mixtral sparse MLP oracle: x [T,d], w13 [E, 2F, d], w2 [E, d, F].  With expert
    parallelism w13/w2 hold experts [expert_offset, expert_offset + E) only and the
    result is this rank's partial sum."""
    w, ids = moe_topk(router_logits, topk, True)
    out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
    F = w2.shape[2]
    for e in range(w13.shape[0]):
        tok, slot = torch.nonzero(ids == e + expert_offset, as_tuple=True)
        if tok.numel() == 0:
            continue
        h = x[tok].float() @ w13[e].float().t()
        a = torch.nn.functional.silu(h[:, :F]) * h[:, F:]
        y = a.to(x.dtype).float() @ w2[e].float().t()
        out.index_add_(0, tok, y * w[tok, slot, None])
    return out.to(x.dtype)


def softmax_scale(head_dim: int = 128) -> float:
    return 1.0 / math.sqrt(head_dim)


# --------------------------------------------------------------------------
# Ops of the layer-list models (fp32 residual stream, sandwich norms, short causal
# input convolutions with per-sequence state, biased / mixed-head / sink attention).
def embed_sinusoid(ids, positions, table, inv_freq, scale: float, out) -> None:
    """out[t] = table[ids[t]] * scale + pe(positions[t]) in fp32, with
    pe[2i] = sin(p * inv_freq[i]), pe[2i+1] = cos of the same angle."""
    d = table.shape[1]
    x = table[ids.long()].float() * scale
    ang = positions.float()[:, None] * inv_freq.float()[None]
    x[:, 0::2] += torch.sin(ang)[:, : (d + 1) // 2]
    x[:, 1::2] += torch.cos(ang)[:, : d // 2]
    out.copy_(x)


def _rms(x, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def sandwich_norm(y, residual, w_post, gain, w_pre, eps: float, out) -> None:
    """residual += rms(y) * w_post * gain (skipped when y is None); out = rms(residual) * w_pre."""
    if y is not None:
        residual.add_(_rms(y.float(), eps) * w_post.float() * gain.float())
    out.copy_(_rms(residual, eps) * w_pre.float())


def canon_conv(h, w, state, row_state, row_back, row_fwd, positions, out) -> None:
    """out[t] = h[t] + sum_j w[:, j] h[t - (taps-1-j)] over the sequence of row t; inputs
    before the scheduled run come from the sequence's state half (its last taps-1
    inputs), inputs before position 0 are zero.  The other half receives the run's last
    taps-1 inputs.  state: [2 * slots, taps-1, d] fp32; row_state = slot * 2 + read half."""
    T, d = h.shape
    taps = w.shape[1]
    K = taps - 1
    S = state.shape[0] // 2
    hf = h.float()
    wf = w.float()
    acc = hf.clone()
    new = {}
    for t in range(T):
        code, i, f, p = int(row_state[t]), int(row_back[t]), int(row_fwd[t]), int(positions[t])
        rd = (code & 1) * S + (code >> 1) if code >= 0 else -1
        for dl in range(taps):                      # delay dl uses tap j = taps-1-dl
            if dl == 0:
                src = hf[t]
            elif dl <= i:
                src = hf[t - dl]
            elif p - dl >= 0 and rd >= 0:
                src = state[rd, K + i - dl]
            else:
                continue
            acc[t] += wf[:, taps - 1 - dl] * src
        if code >= 0:
            wr = (1 - (code & 1)) * S + (code >> 1)
            q = i + f + 1
            if f < K:
                new[(wr, K - 1 - f)] = hf[t]
            if i == 0:
                for e in range(0, K - q):            # run shorter than the state: shift
                    new[(wr, e)] = state[rd, e + q].clone()
    for (wr, e), v in new.items():
        state[wr, e] = v
    out.copy_(acc.to(out.dtype))


def head_norm_append(qkv, q_w, k_w, eps: float, slot_mapping, k_cache, v_cache, H: int, G: int,
                     dim: int, vdim: int, qn, talk_scaled, qmix, mix_from: int) -> None:
    """Per head: q <- rms(q) * q_w (into qn, fp32), k <- rms(k) * k_w and v <- v / rms(v)
    into the paged caches [blocks, G, BS, dim | vdim].  Rows >= mix_from also get mixed
    queries qmix[t - mix_from, h, c*dim:(c+1)*dim] = sum_{g in group c} talk_scaled[h, g] qn[t, g]
    (talk_scaled = score scale * head-mixing matrix), so that mixed scores are one product
    with the concatenated key heads."""
    T = qkv.shape[0]
    if T == 0:
        return
    BS = k_cache.shape[2]
    q = qkv[:, : H * dim].float().view(T, H, dim)
    k = qkv[:, H * dim:(H + G) * dim].float().view(T, G, dim)
    v = qkv[:, (H + G) * dim:(H + G) * dim + G * vdim].float().view(T, G, vdim)
    qf = _rms(q, eps) * q_w.float()
    qn.copy_(qf)
    kf = _rms(k, eps) * k_w.float()
    vf = _rms(v, eps)
    slots = slot_mapping[:T].long()
    ok = slots >= 0
    if ok.any():
        sl = slots[ok]
        blk, off = sl // BS, sl % BS
        k_cache[blk, :, off] = kf[ok].to(k_cache.dtype)
        v_cache[blk, :, off] = vf[ok].to(v_cache.dtype)
    if qmix is not None and mix_from < T:
        rep = H // G
        ts = talk_scaled.float().view(H, G, rep)
        qg = qf[mix_from:].view(T - mix_from, G, rep, dim)
        qmix.copy_(torch.einsum("hcr,tcrd->thcd", ts, qg).reshape(T - mix_from, H, G * dim))


def _sink_softmax(s, ok, sink):
    s = s.masked_fill(~ok, float("-inf"))
    m = s.max(-1).values
    if sink is not None:
        m = torch.maximum(m, sink.float()[:, None])
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    e = torch.exp(s - m[..., None])
    den = e.sum(-1)
    if sink is not None:
        den = den + torch.exp(sink.float()[:, None] - m)
    return e / den.clamp_min(1e-38)[..., None]


def attn_talk_decode(qn, k_cache, v_cache, block_tables, q_start, q_len, kv_len, out, slopes,
                     talk, sink, scale: float, chunk: int) -> None:
    """Decode / short-extend rows: score_g = scale q_g.k - slopes[g] (i - j), mixed over
    heads by ``talk`` [H, H] (None = no mixing), masked to j <= i inside i's block of
    ``chunk`` positions (0 = causal), softmax with a per-head sink logit in the denominator."""
    H, dim = qn.shape[1], qn.shape[2]
    G = k_cache.shape[1]
    rep = H // G
    for b in range(q_len.shape[0]):
        ql, kl, t0 = int(q_len[b]), int(kv_len[b]), int(q_start[b])
        if ql == 0:
            continue
        k = _gather_kv(k_cache, block_tables[b], kl).float().repeat_interleave(rep, 0)
        v = _gather_kv(v_cache, block_tables[b], kl).float().repeat_interleave(rep, 0)
        q = qn[t0:t0 + ql].permute(1, 0, 2)
        i = torch.arange(kl - ql, kl, device=qn.device)[:, None]
        j = torch.arange(kl, device=qn.device)[None, :]
        s = torch.einsum("hqd,hkd->hqk", q, k) * scale - slopes.float()[:, None, None] * (i - j).float()
        if talk is not None:
            s = torch.einsum("hg,gqk->hqk", talk.float(), s)
        ok = j <= i
        if chunk > 0:
            ok = ok & ((i // chunk) == (j // chunk))
        p = _sink_softmax(s, ok[None], sink)
        o = torch.einsum("hqk,hkd->qhd", p, v)
        out[t0:t0 + ql].copy_(o.reshape(ql, -1).to(out.dtype))


def attn_mixq_prefill(qmix, k_cache, v_cache, block_tables, q_start, q_len, kv_len, out, slopes,
                      sink, chunk: int) -> None:
    """Prefill rows on pre-mixed, pre-scaled queries [T, H, G*dim]: every head's score is
    one product with the concatenation of all G key heads, minus slopes[h] (i - j) (the
    slopes already mixed); values come from the head's own key/value head."""
    H = qmix.shape[1]
    G = k_cache.shape[1]
    rep = H // G
    for b in range(q_len.shape[0]):
        ql, kl, t0 = int(q_len[b]), int(kv_len[b]), int(q_start[b])
        if ql == 0:
            continue
        k = _gather_kv(k_cache, block_tables[b], kl).float()            # [G, kl, dim]
        kc = k.permute(1, 0, 2).reshape(kl, -1)                          # [kl, G*dim]
        v = _gather_kv(v_cache, block_tables[b], kl).float().repeat_interleave(rep, 0)
        i = torch.arange(kl - ql, kl, device=qmix.device)[:, None]
        j = torch.arange(kl, device=qmix.device)[None, :]
        s = torch.einsum("qhe,ke->hqk", qmix[t0:t0 + ql].float(), kc)
        s = s - slopes.float()[:, None, None] * (i - j).float()
        ok = j <= i
        if chunk > 0:
            ok = ok & ((i // chunk) == (j // chunk))
        p = _sink_softmax(s, ok[None], sink)
        o = torch.einsum("hqk,hkd->qhd", p, v)
        out[t0:t0 + ql].copy_(o.reshape(ql, -1).to(out.dtype))


def glu_clamped(gate_up, limit: float, alpha: float, out) -> None:
    """g = min(gate, limit), u = clamp(up, -limit, limit); out = g sigmoid(alpha g) (u + 1)."""
    F = out.shape[1]
    g = gate_up[:, :F].float().clamp(max=limit)
    u = gate_up[:, F:].float().clamp(-limit, limit)
    out.copy_((g * torch.sigmoid(alpha * g) * (u + 1)).to(out.dtype))


# --------------------------------------------------------------------------
# Post-norm residual layers, latent attention, wkv recurrence, grouped sigmoid routing.
def embed_rows(ids, table, out, scale: float = 1.0) -> None:
    """out[t] = table[ids[t]] * scale in fp32."""
    out.copy_(table[ids.long()].float() * scale)


def post_norm_add(y, residual, w, mult: float, eps: float, out) -> None:
    """residual (fp32, in place) += mult * rms(y) * (1 + w); out (any dtype, may be None)
    receives the updated residual: the next sublayer reads the stream itself."""
    residual.add_(_rms(y.float(), eps) * (1.0 + w.float()) * mult)
    if out is not None:
        out.copy_(residual.to(out.dtype))


def rms_norm_rows(x, w, eps: float, out, offset: float = 0.0) -> None:
    """out = rms(x) * (w + offset) per row, computed in fp32; x may be a column slice."""
    out.copy_((_rms(x.float(), eps) * (w.float() + offset)).to(out.dtype))


def latent_norm_append(x, w, eps: float, slot_mapping, pool) -> None:
    """c = rms(x) * w per row (fp32) into the paged latent pool [blocks, 1, BS, R] at the
    rows' slots (slot < 0: dropped)."""
    T = x.shape[0]
    if T == 0:
        return
    BS = pool.shape[2]
    c = _rms(x.float(), eps) * w.float()
    slots = slot_mapping[:T].long()
    ok = slots >= 0
    if ok.any():
        sl = slots[ok]
        pool[sl // BS, 0, sl % BS] = c[ok].to(pool.dtype)


def _state_rows(code: int, S: int):
    """(read row, write row) of a state pool [2 * S, ...] for row_state code slot*2+half."""
    return (code & 1) * S + (code >> 1), (1 - (code & 1)) * S + (code >> 1)


def token_shift_mix(x, mu, prev, row_state, row_back, row_fwd, positions, out) -> None:
    """out[s, t] = x[t] + (x'[t] - x[t]) * mu[s] for each of the mu rows, x' the previous
    token's row of the same sequence: the row above inside a scheduled run, the sequence's
    state half (prev [2 * slots, d] fp32) at the run's start, zeros at position 0.  The
    run's last row goes to the other half."""
    T, d = x.shape
    if T == 0:
        return
    S = prev.shape[0] // 2
    xf = x.float()
    before = torch.zeros_like(xf)
    new = []
    for t in range(T):
        code, i, f, p = int(row_state[t]), int(row_back[t]), int(row_fwd[t]), int(positions[t])
        if i > 0:
            before[t] = xf[t - 1]
        elif p > 0 and code >= 0:
            before[t] = prev[_state_rows(code, S)[0]]
        if f == 0 and code >= 0:
            new.append((_state_rows(code, S)[1], xf[t].clone()))
    for wr, v in new:
        prev[wr] = v
    out.copy_((xf[None] + (before - xf)[None] * mu.float()[:, None, :]).to(out.dtype))


def wkv_recurrence(r, k, v, zw, w0, u, gate, norm_w, eps: float, state, row_state, row_back,
                   row_fwd, positions, out) -> None:
    """Per head (N key x N value channels), token by token inside each scheduled run:
        w_t = exp(-exp(zw_t + w0));  o_t = (S + diag(u) k_t v_t^T)^T r_t;  S <- diag(w_t) S + k_t v_t^T
    then out_t = o_t / rms_head(o_t) * norm_w * silu(gate_t).  state: [2 * slots, H, N, N]
    fp32, read from the row's half at the run's start (zeros at position 0), the run's last
    state written to the other half.  Decay, state and output norm in fp32."""
    T = r.shape[0]
    if T == 0:
        return
    H, N = u.shape
    S_ = state.shape[0] // 2
    rf, kf, vf = (a.float().reshape(T, H, N) for a in (r, k, v))
    w = torch.exp(-torch.exp(zw.float() + w0.float())).reshape(T, H, N)
    uf = u.float()
    o = torch.zeros(T, H, N)
    cur = None
    for t in range(T):
        code, i, f, p = int(row_state[t]), int(row_back[t]), int(row_fwd[t]), int(positions[t])
        if i == 0:
            cur = state[_state_rows(code, S_)[0]].clone() if p > 0 and code >= 0 \
                else torch.zeros(H, N, N)
        kv = kf[t][:, :, None] * vf[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", cur + uf[:, :, None] * kv, rf[t])
        cur = w[t][:, :, None] * cur + kv
        if f == 0 and code >= 0:
            state[_state_rows(code, S_)[1]] = cur
    y = _rms(o, eps).reshape(T, H * N) * norm_w.float() * torch.nn.functional.silu(gate.float())
    out.copy_(y.to(out.dtype))


def moe_route_grouped(z, correction, top: int, groups: int, keep: int, ids, weights) -> None:
    """Sigmoid routing: s = sigmoid(z); experts are chosen by s + correction, only inside the
    ``keep`` groups (of ``groups`` equal groups of neighbours; 0 = no limit) whose two largest
    choice scores sum highest; weights = s of the chosen / (their sum + 1e-20).  Ties go to the
    lower index."""
    T, E = z.shape
    s = torch.sigmoid(z.float())
    choice = s + correction.float()
    if groups > 0:
        per = E // groups
        grp = choice.view(T, groups, per)
        gs = grp.topk(min(2, per), -1).values.sum(-1)
        kept = torch.zeros(T, groups, dtype=torch.bool)
        order = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep]
        kept.scatter_(1, order, True)
        choice = torch.where(kept[:, :, None].expand(T, groups, per), grp,
                             torch.full_like(grp, float("-inf"))).reshape(T, E)
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    wt = s.gather(1, idx)
    ids.copy_(idx.to(ids.dtype))
    weights.copy_(wt / (wt.sum(-1, keepdim=True) + 1e-20))


def silu_mul_any(gate_up, out) -> None:
    """out = silu(gate) * up for gate_up = [gate | up] columns, any dtype and width."""
    F = out.shape[1]
    out.copy_((torch.nn.functional.silu(gate_up[:, :F].float()) * gate_up[:, F:].float()).to(out.dtype))


def softcap(x, cap: float) -> None:
    """x <- cap * tanh(x / cap), in place (fp32)."""
    x.copy_(cap * torch.tanh(x / cap))


def moe_experts(h, ids, weights, w13, w2, base, out) -> None:
    """out (fp32) = base + sum_k weights[t, k] * W2[e] (silu(Wg[e] h_t) * (Wu[e] h_t)) with
    e = ids[t, k]; w13 [E, 2F, d] holds gate | up rows, w2 [E, d, F].  Products in h's dtype
    with fp32 accumulation, the weighted sum in fp32."""
    T, F = h.shape[0], w2.shape[2]
    acc = torch.zeros((T, w2.shape[1]), dtype=torch.float32) if base is None else base.float().clone()
    for e in range(w13.shape[0]):
        hit = (ids == e)
        rows = hit.any(-1).nonzero()[:, 0]
        if rows.numel() == 0:
            continue
        x = h[rows]
        gu = x @ w13[e].t()
        a = (torch.nn.functional.silu(gu[:, :F].float()) * gu[:, F:].float()).to(h.dtype)
        y = (a @ w2[e].t()).float()
        wt = (weights[rows] * hit[rows]).sum(-1)
        acc[rows] += wt[:, None] * y
    out.copy_(acc)


# ---------------------------------------------------------------------------
# Parallel-sublayer residual, rotary windowed differential attention, gated linear
# recurrences (plain and delta rule), activated causal convolutions, softmax top-k routing.
def residual_add_norm(x, y1, y2, shift, w, eps: float, offset: float, out,
                      mult: float = 1.0) -> None:
    """x (fp32, in place) += mult * (y1 + y2) + shift (each optional; shift is one row for
    all); with ``w``: out = x / sqrt(mean(x^2) + eps) * (w + offset) in out's dtype."""
    if y1 is not None or y2 is not None:
        y = (y1.float() if y1 is not None else 0.0) + (y2.float() if y2 is not None else 0.0)
        x.add_(y * mult if mult != 1.0 else y)
    if shift is not None:
        x.add_(shift.float())
    if w is not None:
        out.copy_((_rms(x, eps) * (w.float() + offset)).to(out.dtype))


def rotary_inv_freq(rot_dims: int, base: float, device="cpu") -> torch.Tensor:
    """f_i = base^(-2i / rot_dims), i < rot_dims / 2, rounded once from float64."""
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / max(1, rot_dims)) \
        .float().to(device)


def _rotate_pairs(x, positions, inv_freq):
    """Rotates the leading 2 * len(inv_freq) entries of the last axis of x [T, ..., w]:
    entries (2i, 2i+1) by the angle position * f_i (angles, sines and cosines in fp32)."""
    n = inv_freq.numel()
    if n == 0:
        return x
    ang = positions.float()[:, None] * inv_freq.float()[None]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (n,)
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    x = x.clone()
    u, v = x[..., 0:2 * n:2].clone(), x[..., 1:2 * n:2].clone()
    x[..., 0:2 * n:2] = u * c - v * s
    x[..., 1:2 * n:2] = v * c + u * s
    return x


def rotary_append(qkv, positions, inv_freq, slot_mapping, k_cache, v_cache, H: int, G: int,
                  maps: int, dim: int, vdim: int, q_out) -> None:
    """Rows of qkv are q [H, maps, dim] | k [G, maps, dim] | v [G, vdim].  The first
    2 * len(inv_freq) dimensions of every map of q and k are rotated by the row's position;
    q goes to q_out [T, H, maps * dim] fp32, k and v into their pages (slot < 0: nowhere)."""
    T = qkv.shape[0]
    if T == 0:
        return
    nq, nk = H * maps * dim, G * maps * dim
    x = qkv.float()
    q = _rotate_pairs(x[:, :nq].reshape(T, H, maps, dim), positions[:T], inv_freq)
    k = _rotate_pairs(x[:, nq:nq + nk].reshape(T, G, maps, dim), positions[:T], inv_freq)
    v = x[:, nq + nk:nq + nk + G * vdim].reshape(T, G, vdim)
    q_out.copy_(q.reshape(T, H, maps * dim))
    BS = k_cache.shape[2]
    for t in range(T):
        s = int(slot_mapping[t])
        if s >= 0:
            k_cache[s // BS, :, s % BS] = k[t].reshape(G, maps * dim).to(k_cache.dtype)
            v_cache[s // BS, :, s % BS] = v[t].to(v_cache.dtype)


def attn_diff_window(q, k_cache, v_cache, block_tables, q_start, q_len, kv_len, gate, out,
                     scale: float, window: int, lam: float, eps: float, out_mult: float) -> None:
    """Differential attention inside a sliding window.  q [T, H, 2 dim] fp32 (rotated),
    k_cache [blocks, G, BS, 2 dim], v_cache [blocks, G, BS, vdim]; per head two softmax
    attentions a1, a2 (the two halves of q and k) over the same values; position i sees
    j <= i with i - j < window (0: all).  o = a1 - lam a2, divided by its root mean square
    over vdim (+ eps), times out_mult, times sigmoid(gate[t, h]); out [T, H vdim]."""
    H, dim = q.shape[1], q.shape[2] // 2
    G = k_cache.shape[1]
    rep = H // G
    for b in range(q_len.shape[0]):
        ql, kl, t0 = int(q_len[b]), int(kv_len[b]), int(q_start[b])
        if ql == 0:
            continue
        lo = max(0, kl - ql - window + 1) if window > 0 else 0
        k = _gather_kv(k_cache, block_tables[b], kl).float()[:, lo:].repeat_interleave(rep, 0)
        v = _gather_kv(v_cache, block_tables[b], kl).float()[:, lo:].repeat_interleave(rep, 0)
        i = torch.arange(kl - ql, kl)[:, None]
        j = torch.arange(lo, kl)[None, :]
        ok = (j <= i) & ((i - j < window) if window > 0 else (j >= 0))
        qq = q[t0:t0 + ql].float()
        a = []
        for mp in range(2):
            s = torch.einsum("qhe,hke->hqk", qq[:, :, mp * dim:(mp + 1) * dim],
                             k[:, :, mp * dim:(mp + 1) * dim]) * scale
            s = s.masked_fill(~ok[None], float("-inf"))
            a.append(torch.einsum("hqk,hkd->qhd", torch.softmax(s, -1), v))
        o = _rms(a[0] - lam * a[1], eps) * out_mult
        o = o * torch.sigmoid(gate[t0:t0 + ql].float())[:, :, None]
        out[t0:t0 + ql].copy_(o.reshape(ql, -1).to(out.dtype))


def conv_act_heads(x, w, state, row_state, row_back, row_fwd, positions, n_unit: int, dim: int,
                   unit_eps: float, out) -> None:
    """out[t] = silu(sum_j w[:, j] x[t - (taps-1-j)]) over the sequence of row t (inputs
    before the run from the state half, zeros before position 0; the run's last taps-1
    inputs go to the other half; state [2 * slots, taps-1, C] fp32).  The first ``n_unit``
    heads of ``dim`` channels are then made unit vectors: y / sqrt(sum(y^2) + unit_eps).
    out [T, C] fp32."""
    T, C = x.shape
    if T == 0:
        return
    taps = w.shape[1]
    K = taps - 1
    S = state.shape[0] // 2
    xf, wf = x.float(), w.float()
    acc = torch.zeros(T, C)
    new = {}
    for t in range(T):
        code, i, f, p = int(row_state[t]), int(row_back[t]), int(row_fwd[t]), int(positions[t])
        rd, wr = _state_rows(code, S) if code >= 0 else (-1, -1)
        for dl in range(taps):
            if dl <= i:
                src = xf[t - dl]
            elif p - dl >= 0 and rd >= 0:
                src = state[rd, K + i - dl]
            else:
                continue
            acc[t] += wf[:, taps - 1 - dl] * src
        if code >= 0:
            n = i + f + 1
            if f < K:
                new[(wr, K - 1 - f)] = xf[t].clone()
            if i == 0:
                for e in range(0, K - n):
                    new[(wr, e)] = state[rd, e + n].clone()
    for (wr, e), v in new.items():
        state[wr, e] = v
    y = torch.nn.functional.silu(acc)
    if n_unit > 0:
        u = y[:, :n_unit * dim].reshape(T, n_unit, dim)
        y[:, :n_unit * dim] = (u / torch.sqrt((u * u).sum(-1, keepdim=True) + unit_eps)).reshape(T, -1)
    out.copy_(y)


def gated_linear_recurrence(q, k, v, z, rate, zbias, zsign: float, beta, gate, gate_sigmoid: bool,
                            norm_w, eps: float, q_scale: float, state, row_state, row_back,
                            row_fwd, positions, out) -> None:
    """Per head a dim x vdim state S (fp32), token by token inside each scheduled run:
        a_t = exp(-rate_h softplus(zsign (z_t + zbias)))            decay per key channel
        S <- diag(a_t) S
        u_t = beta_t (v_t - S^T k_t)   (delta rule; without beta: u_t = v_t)
        S <- S + k_t u_t^T ;  o_t = q_scale S^T q_t
    out_t = o_t / rms(o_t) * norm_w * act(gate_t), act = sigmoid or silu.  q, k
    [T, Hq, dim] (head h reads head h // (H / Hq)), v [T, H, vdim], z [T, H dim], beta
    [T, H] logits (sigmoid applied here) or None, gate [T, H vdim], norm_w [vdim].
    state [2 * slots, H, dim, vdim]: read at the run's start (zeros at position 0), the
    run's last state written to the other half."""
    T = q.shape[0]
    if T == 0:
        return
    H, dim, vdim = state.shape[1], state.shape[2], state.shape[3]
    Hq = q.shape[1]
    rep = H // Hq
    S_ = state.shape[0] // 2
    qf = q.float().repeat_interleave(rep, 1)
    kf = k.float().repeat_interleave(rep, 1)
    vf = v.float().reshape(T, H, vdim)
    zz = zsign * (z.float() + zbias.float())
    a = torch.exp(-rate.float()[None, :, None] * torch.nn.functional.softplus(zz).reshape(T, H, dim))
    bt = torch.sigmoid(beta.float()) if beta is not None else None
    o = torch.zeros(T, H, vdim)
    cur = None
    for t in range(T):
        code, i, f, p = int(row_state[t]), int(row_back[t]), int(row_fwd[t]), int(positions[t])
        if i == 0:
            cur = state[_state_rows(code, S_)[0]].clone() if p > 0 and code >= 0 \
                else torch.zeros(H, dim, vdim)
        cur = a[t][:, :, None] * cur
        u = vf[t]
        if bt is not None:
            u = bt[t][:, None] * (u - torch.einsum("hkv,hk->hv", cur, kf[t]))
        cur = cur + kf[t][:, :, None] * u[:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", cur, qf[t]) * q_scale
        if f == 0 and code >= 0:
            state[_state_rows(code, S_)[1]] = cur
    g = gate.float().reshape(T, H, vdim)
    g = torch.sigmoid(g) if gate_sigmoid else torch.nn.functional.silu(g)
    y = _rms(o, eps) * norm_w.float() * g
    out.copy_(y.reshape(T, H * vdim).to(out.dtype))


def moe_route_topk(z, bias, top: int, ids, weights) -> None:
    """The ``top`` largest of z + bias per row (ties to the lower index), weighted by the
    softmax over the chosen logits only."""
    zz = z.float() + (bias.float() if bias is not None else 0.0)
    T, E = zz.shape
    order = torch.argsort(zz, dim=-1, descending=True, stable=True)[:, :top]
    val = torch.gather(zz, 1, order)
    ids.copy_(order.to(ids.dtype))
    weights.copy_(torch.softmax(val, -1))


def gelu_rows(x, out) -> None:
    """out = 0.5 x (1 + erf(x / sqrt 2)), computed in fp32."""
    xf = x.float()
    out.copy_((0.5 * xf * (1.0 + torch.erf(xf * 0.7071067811865476))).to(out.dtype))


# ---------------------------------------------------------------------------
# Scaled half-split rotation, projection norms, attention with a sliding window that keeps
# the first tokens and softmax / sink / sigmoid weights, the xIELU unit.
def rotary_scaled_freq(rot_dims: int, base: float, scaling: tuple = (), device="cpu"):
    """(f [rot_dims / 2] fp32, multiplier of cos and sin).  f_i = base^(-2i / rot_dims), then by
    ``scaling``:
      ("yarn", factor, original, fast, slow): with dim(t) = rot_dims ln(original / (2 pi t)) /
        (2 ln base), lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), rot_dims - 1) and
        r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1): f_i (r_i / factor + 1 - r_i); the
        multiplier is 0.1 ln(factor) + 1;
      ("banded", factor, original, low, high): wavelengths 2 pi / f below original / high keep
        f, above original / low get f / factor, between them the blend
        (1 - s) f / factor + s f with s = (original f / (2 pi) - low) / (high - low).
    Everything in float64, rounded once."""
    n = rot_dims // 2
    i = torch.arange(n, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / max(1, rot_dims))
    mult = 1.0
    if scaling and scaling[0] == "yarn":
        _, factor, original, fast, slow = scaling

        def dim_of(t):
            return rot_dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))

        lo = max(math.floor(dim_of(fast)), 0)
        hi = min(math.ceil(dim_of(slow)), rot_dims - 1)
        r = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * r + f * (1.0 - r)
        mult = 0.1 * math.log(factor) + 1.0
    elif scaling and scaling[0] == "banded":
        _, factor, original, low, high = scaling
        wl = 2.0 * math.pi / f
        s = (original / wl - low) / (high - low)
        mid = (1.0 - s) * f / factor + s * f
        f = torch.where(wl < original / high, f, torch.where(wl > original / low, f / factor, mid))
    elif scaling:
        raise ValueError(f"unknown frequency scaling {scaling[0]!r}")
    return f.float().to(device), float(mult)


def _rotate_halves(x, positions, inv_freq, mult: float, off: int):
    """Entries off + i and off + i + n (n = len(inv_freq)) of the last axis of x [T, ..., w]
    turn by the angle position * f_i; cos and sin carry the factor ``mult`` (all fp32)."""
    n = inv_freq.numel()
    if n == 0:
        return x
    ang = positions.float()[:, None] * inv_freq.float()[None]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (n,)
    c, s = (torch.cos(ang) * mult).view(shape), (torch.sin(ang) * mult).view(shape)
    y = x.clone()
    u, v = x[..., off:off + n], x[..., off + n:off + 2 * n]
    y[..., off:off + n] = u * c - v * s
    y[..., off + n:off + 2 * n] = v * c + u * s
    return y


def qk_norm_rotary_append(proj, bias, q_norm_w, k_norm_w, norm_all: bool, k_norm_n: int, eps: float,
                          positions, inv_freq, rot_mult: float, q_rot_off: int, k_rot_off: int,
                          slot_mapping, k_cache, v_cache, H: int, G: int, qw: int, kw: int, vdim: int,
                          v_mode: int, q_out) -> None:
    """Rows of proj are q [H, qw] | k [G, kw] (| v [G, vdim] with v_mode 0); ``bias`` (fp32, the
    row's width) is added first.  RMS norms with plain weights: over the whole q and the whole k
    projection (``norm_all``; weights [H qw], [G kw]) or per head, q over its qw entries
    (weight [qw]) and k over its leading ``k_norm_n`` entries (weight [k_norm_n]); a weight of
    None means no norm.  Then the half-split rotation of entries rot_off .. rot_off + 2 n of
    every head.  q goes to q_out [T, H, qw] fp32; k rows into k_cache [blocks, G, BS, kw];
    values into v_cache [blocks, G, BS, vdim]: v_mode 0 the v columns, 1 the keys as projected
    (before norm and rotation), 2 none."""
    T = proj.shape[0]
    if T == 0:
        return
    x = proj.float()
    if bias is not None:
        x = x + bias.float()
    nq, nk = H * qw, G * kw
    q, k = x[:, :nq], x[:, nq:nq + nk]
    raw_k = k.reshape(T, G, kw)
    if norm_all:
        if q_norm_w is not None:
            q = _rms(q, eps) * q_norm_w.float()
        if k_norm_w is not None:
            k = _rms(k, eps) * k_norm_w.float()
        q, k = q.reshape(T, H, qw), k.reshape(T, G, kw)
    else:
        q, k = q.reshape(T, H, qw), k.reshape(T, G, kw).clone()
        if q_norm_w is not None:
            q = _rms(q, eps) * q_norm_w.float()
        if k_norm_w is not None:
            k[..., :k_norm_n] = _rms(k[..., :k_norm_n], eps) * k_norm_w.float()
    q = _rotate_halves(q, positions[:T], inv_freq, rot_mult, q_rot_off)
    k = _rotate_halves(k, positions[:T], inv_freq, rot_mult, k_rot_off)
    q_out.copy_(q)
    if k_cache is None or G == 0:
        return
    v = x[:, nq + nk:nq + nk + G * vdim].reshape(T, G, vdim) if v_mode == 0 else raw_k
    BS = k_cache.shape[2]
    for t in range(T):
        s = int(slot_mapping[t])
        if s >= 0:
            k_cache[s // BS, :, s % BS] = k[t].to(k_cache.dtype)
            if v_mode != 2:
                v_cache[s // BS, :, s % BS] = v[t].to(v_cache.dtype)


def attn_keep_window(q, k_cache, v_cache, vdim: int, block_tables, q_start, q_len, kv_len, head_bias,
                     gate, out, scale: float, window: int, keep_first: int, sigmoid: bool) -> None:
    """q [T, H, E] fp32; k_cache [blocks, G, BS, E]; the values are the first ``vdim`` entries
    of v_cache's rows (which may be the key pages themselves).  Position i sees j <= i with
    i - j < window or j < keep_first (window 0: every j <= i).  Weights: softmax over the
    visible keys, with exp(head_bias[h]) added to the denominator when head_bias is given; or
    (``sigmoid``) sigmoid(score + head_bias[h]) per visible key, not normalised.  ``gate``
    [T, H]: the head's output is multiplied by sigmoid(gate).  out [T, H vdim]."""
    H = q.shape[1]
    G = k_cache.shape[1]
    rep = H // G
    for b in range(q_len.shape[0]):
        ql, kl, t0 = int(q_len[b]), int(kv_len[b]), int(q_start[b])
        if ql == 0:
            continue
        k = _gather_kv(k_cache, block_tables[b], kl).float().repeat_interleave(rep, 0)
        v = _gather_kv(v_cache, block_tables[b], kl).float()[..., :vdim].repeat_interleave(rep, 0)
        i = torch.arange(kl - ql, kl)[:, None]
        j = torch.arange(kl)[None, :]
        ok = j <= i
        if window > 0:
            ok = ok & ((i - j < window) | (j < keep_first))
        s = torch.einsum("qhe,hke->hqk", q[t0:t0 + ql].float(), k) * scale
        if sigmoid:
            p = torch.sigmoid(s + head_bias.float()[:, None, None]) * ok[None]
        else:
            s = s.masked_fill(~ok[None], float("-inf"))
            if head_bias is not None:
                s = torch.cat([s, head_bias.float()[:, None, None].expand(H, ql, 1)], -1)
            p = torch.softmax(s, -1)[..., :kl]
        o = torch.einsum("hqk,hkd->qhd", p, v)
        if gate is not None:
            o = o * torch.sigmoid(gate[t0:t0 + ql].float())[:, :, None]
        out[t0:t0 + ql].copy_(o.reshape(ql, -1).to(out.dtype))


def xielu_rows(x, alpha_p: float, alpha_n: float, out) -> None:
    """z > 0: alpha_p z^2 + z / 2;  z <= 0: alpha_n (exp(z) - 1 - z) + z / 2, in fp32."""
    z = x.float()
    zn = torch.clamp(z, max=0.0)
    out.copy_(torch.where(z > 0, alpha_p * z * z + 0.5 * z,
                          alpha_n * (torch.expm1(zn) - zn) + 0.5 * zn).to(out.dtype))
