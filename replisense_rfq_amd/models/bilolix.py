"""Bilolix: parallel-sublayer layers of windowed differential attention, gated linear
attention or the channel-wise gated delta rule, with dense or routed feed-forwards and a
looped span of layers, on the kernels of csrc/kernels/mix_*.hip.

The residual stream x is fp32.  One zero-centred RMS norm per layer feeds both sublayers:

  x = embed[token]
  per layer run r (a looped layer runs once per pass, with pages and state of its own):
    x += step[t]                       before the first layer of pass t of the loop
    h = rms(x) (1 + w)
    x += mixer(h) + ff(h)
  logits = head . (rms(x) (1 + w_final))

The residual update, the step vector and the next run's norm are one kernel
(residual_add_norm).  Mixers:

differential attention   q | k | v in one product; q and k hold two score maps per head
  ([map 1 | map 2], each ``dim`` wide); the first rot_dims dimensions of every map are
  rotated in interleaved pairs; k (both maps side by side) and v go to the run's pages.
  Per head two softmax attentions inside the sliding window over the same values,
  o = a1 - lambda a2 with lambda = exp(lq1.lk1) - exp(lq2.lk2) + diff (one float per layer,
  formed at load time), o / rms(o) (1 - diff), times sigmoid of a per-head gate logit.
gla   q | k | v | gate | decay-inner in one product; decay logits z = W_a2 (inner) in fp32;
  a = sigmoid(z + b)^(1 / tau) = exp(-(1 / tau) softplus(-(z + b))); S <- diag(a) S + k v^T,
  o = dim^-1/2 S^T q; o / rms(o) * w * silu(gate).
channel_delta   q | k | v | beta | decay-inner | gate-inner in one product; q, k, v pass a
  causal convolution + silu (the last taps - 1 inputs are per-sequence state), q and k become
  unit vectors; a = exp(-exp(A_log) softplus(z + dt_bias)); S <- diag(a) S,
  u = beta (v - S^T k), S <- S + k u^T, o = dim^-1/2 S^T q; o / rms(o) * w * sigmoid(gate).
  Both recurrences are one kernel (gated_linear_recurrence): a = exp(-rate softplus(sign (z + bias))).
feed-forward   W_down gelu(W_up h), or experts W_down (silu(W_gate h) * W_up h) chosen by the
  top router logits (fp32, with a bias) and weighted by the softmax over the chosen ones.
"""
from __future__ import annotations

import torch

from .. import ops
from ..parallel.tp import SINGLE, TPContext
from .config import LayeredConfig
from .moe import MoEBuffers, grouped_ok, moe_mlp
from .weights import init_bilolix_weights

UNIT_EPS = 1e-6            # q, k of the delta rule: y / sqrt(sum(y^2) + UNIT_EPS)
MAPS = 2                   # score maps per head of the differential attention


class BilolixLM:
    stateful = True            # sequences own a state slot (recurrent matrices, convolution inputs)

    def __init__(self, cfg: LayeredConfig, device, tp: TPContext = SINGLE, seed: int = 0,
                 weights: dict | None = None, dtype=torch.bfloat16, moe_ep: bool = False):
        if tp.enabled:
            raise ValueError("layer-list models run at TP = 1")
        self.cfg = cfg
        self.tp = tp
        self.device = torch.device(device)
        self.dtype = dtype
        self.w = weights if weights is not None else init_bilolix_weights(cfg, self.device, dtype, seed)
        self.vocab_start = 0
        self.vocab_local = self.w["lm_head"].shape[0]
        # the kernels of this model take no per-head decode work list: one entry per row
        self.hq = self.hkv = 1
        self.kv_k = self.kv_v = self.layer_state = None
        self.norms_folded = False
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False
        self._moe_bufs: dict = {}
        self._seq_ids = None
        self.runs = cfg.runs
        self.pass_starts = cfg.pass_starts
        for ly, lw in zip(cfg.layers, self.w["layers"]):
            m = ly.mixer
            if m.kind == "diff_attention":
                lw["inv_freq"] = ops.rotary_inv_freq(m.rot_dims, m.rot_base, self.device)
            lw["grouped"] = bool(ly.mlp is not None and ly.mlp.kind == "moe"
                                 and self.device.type == "cuda" and dtype == torch.bfloat16
                                 and grouped_ok(lw["w13"], lw["w2e"]))

    # engine hooks shared with the other decoders
    def fold_norms(self) -> bool:
        return False

    def tile_decode_weights(self, mode: str | None = None) -> int:
        return 0

    def attach_kv_cache(self, k_pools, v_pools, state=None, layer_state=None) -> None:
        """Per layer run: K pool [num_blocks, G, block, 2 dim] and V pool [.., vdim] for the
        attention runs; layer_state[r]: "S" [2*slots, H, dim, vdim] for the recurrent runs and
        "conv" [2*slots, taps-1, channels] for the delta rule's convolutions, fp32."""
        assert len(k_pools) == len(self.runs)
        self.kv_k, self.kv_v, self.layer_state = k_pools, v_pools, layer_state

    def _decode_work(self, n: int):
        """(sequence index, query block 0) per decode-section sequence; views of two tensors
        that only grow (never inside a graph capture: the warm-up run sizes them)."""
        if self._seq_ids is None or self._seq_ids[0].numel() < n:
            size = max(1024, 2 * n)
            self._seq_ids = (torch.arange(size, dtype=torch.int32, device=self.device),
                             torch.zeros(size, dtype=torch.int32, device=self.device))
        return self._seq_ids[0][:n], self._seq_ids[1][:n]

    def _run_rows(self, m):
        """First row of every scheduled run of the step (decode section, then prefill section;
        -1 for a sequence without rows: padding of a graph step), for the recurrences' grid."""
        if self.device.type != "cuda" or \
                not any(ly.mixer.kind in ("gla", "channel_delta") for ly in self.cfg.layers):
            return None
        parts = []
        if m.dec_q_len is not None and m.dec_q_len.numel():
            parts.append(torch.where(m.dec_q_len > 0, m.dec_q_start, -1))
        if m.pf_q_len is not None and m.pf_q_len.numel():
            parts.append(torch.where(m.pf_q_len > 0, m.pf_q_start + m.num_decode, -1))
        if not parts:
            return None
        return (parts[0] if len(parts) == 1 else torch.cat(parts)).to(torch.int32)

    def weight_bytes(self) -> int:
        tot = sum(v.numel() * v.element_size() for v in self.w.values() if isinstance(v, torch.Tensor))
        for lw in self.w["layers"]:
            tot += sum(t.numel() * t.element_size() for t in lw.values() if isinstance(t, torch.Tensor))
        return tot

    # ------------------------------------------------------------------ mixers
    def _diff_attention(self, ri, mx, lw, h, m):
        T, D, dt, dev = m.num_tokens, m.num_decode, self.dtype, h.device
        H, G, dim, vd = mx.heads, mx.kv_heads, mx.dim, mx.vdim
        kc, vc = self.kv_k[ri], self.kv_v[ri]
        qkv = ops.matmul_nt(h, lw["qkv"])
        gate = ops.matmul_nt(h, lw["g"])                       # [T, H] logits
        q = torch.empty((T, H, MAPS * dim), dtype=torch.float32, device=dev)
        ops.rotary_append(qkv, m.positions[:T], lw["inv_freq"], m.slot_mapping[:T], kc, vc, H, G,
                          MAPS, dim, vd, q)
        attn = torch.empty((T, H * vd), dtype=dt, device=dev)
        eps, keep = self.cfg.rms_eps, 1.0 - mx.diff
        if D > 0:
            ids, zeros = self._decode_work(m.dec_q_len.shape[0])
            ops.attn_diff_window(q[:D], kc, vc, m.dec_block_tables, m.dec_q_start, m.dec_q_len,
                                 m.dec_kv_len, ids, zeros, gate[:D], attn[:D], mx.scale, mx.window,
                                 lw["lam"], eps, keep, short_rows=ops.TALK_DECODE_MAX_ROWS)
        if T > D:
            ops.attn_diff_window(q[D:], kc, vc, m.pf_block_tables, m.pf_q_start, m.pf_q_len,
                                 m.pf_kv_len, m.work_seq, m.work_qblk, gate[D:T], attn[D:T],
                                 mx.scale, mx.window, lw["lam"], eps, keep)
        return ops.matmul_nt(attn, lw["o"])

    @staticmethod
    def _cols(pr, seg, name, heads=0):
        a, n = seg[name]
        x = pr[:, a:a + n]
        return x.unflatten(1, (heads, n // heads)) if heads else x

    def _gla(self, ri, mx, lw, h, m, rows):
        T = m.num_tokens
        H, seg = mx.heads, lw["seg"]
        rs, rb, rf, pos, runs = rows
        pr = ops.matmul_nt(h, lw["proj"])
        z = ops.matmul_nt(self._cols(pr, seg, "a1"), lw["a2"], out_dtype=torch.float32)
        y = torch.empty((T, H * mx.vdim), dtype=self.dtype, device=h.device)
        ops.gated_linear_recurrence(
            self._cols(pr, seg, "q", H), self._cols(pr, seg, "k", H), self._cols(pr, seg, "v", H),
            z, lw["rate"], lw["zbias"], -1.0, None, self._cols(pr, seg, "g"), False, lw["gn"],
            self.cfg.rms_eps, mx.scale, self.layer_state[ri]["S"], rs, rb, rf, pos, y, runs)
        return ops.matmul_nt(y, lw["o"])

    def _channel_delta(self, ri, mx, lw, h, m, rows):
        T = m.num_tokens
        H, G, dim, vd, seg = mx.heads, mx.kv_heads, mx.dim, mx.vdim, lw["seg"]
        rs, rb, rf, pos, runs = rows
        st = self.layer_state[ri]
        pr = ops.matmul_nt(h, lw["proj"])
        C = 2 * G * dim + H * vd
        qkv = torch.empty((T, C), dtype=torch.float32, device=h.device)
        ops.conv_act_heads(pr[:, :C], lw["conv_w"], st["conv"], rs, rb, rf, pos, 2 * G, dim,
                           UNIT_EPS, qkv)
        z = ops.matmul_nt(self._cols(pr, seg, "a1"), lw["a2"], out_dtype=torch.float32)
        gate = ops.matmul_nt(self._cols(pr, seg, "g1"), lw["g2"])
        y = torch.empty((T, H * vd), dtype=self.dtype, device=h.device)
        ops.gated_linear_recurrence(
            qkv[:, :G * dim].unflatten(1, (G, dim)), qkv[:, G * dim:2 * G * dim].unflatten(1, (G, dim)),
            qkv[:, 2 * G * dim:].unflatten(1, (H, vd)), z, lw["rate"], lw["zbias"], 1.0,
            self._cols(pr, seg, "b"), gate, True, lw["gn"], self.cfg.rms_eps, mx.scale, st["S"],
            rs, rb, rf, pos, y, runs)
        return ops.matmul_nt(y, lw["o"])

    # ------------------------------------------------------------ feed-forward
    def _moe_buffers(self, T: int, f, d: int) -> MoEBuffers:
        cap = 1
        while cap < T:
            cap *= 2
        key = (cap, f.top, f.experts, f.ff)
        if key not in self._moe_bufs:
            self._moe_bufs[key] = MoEBuffers.allocate(cap, f.top, f.experts, d, f.ff, self.device,
                                                      self.dtype)
        return self._moe_bufs[key]

    def _moe(self, f, lw, h):
        T, dev = h.shape[0], h.device
        z = ops.matmul_nt(h, lw["router"], out_dtype=torch.float32)
        if lw["grouped"]:
            # the sparse decoder's alignment, grouped MFMA GEMMs and combine behind this router
            return moe_mlp(h, lw["router"], lw["w13"], lw["w2e"], f.top,
                           self._moe_buffers(T, f, h.shape[1]),
                           routing=lambda w, i: ops.moe_route_topk(z, lw["router_b"], f.top, i, w))
        ids = torch.empty((T, f.top), dtype=torch.int32, device=dev)
        wts = torch.empty((T, f.top), dtype=torch.float32, device=dev)
        ops.moe_route_topk(z, lw["router_b"], f.top, ids, wts)
        return ops.moe_experts(h, ids, wts, lw["w13"], lw["w2e"], None,
                               torch.empty((T, h.shape[1]), dtype=torch.float32, device=dev))

    def _mlp(self, f, lw, h):
        if f.kind == "moe":
            return self._moe(f, lw, h)
        return ops.matmul_nt(ops.gelu_rows(ops.matmul_nt(h, lw["up"])), lw["down"])

    # ------------------------------------------------------------------ forward
    def forward(self, m, taps: list | None = None) -> torch.Tensor:
        """Logits [rows, V] (fp32) of the step.  ``taps``: a list that receives the residual
        stream after every layer run (debugging / layer-wise tests)."""
        cfg, w = self.cfg, self.w
        T, eps, dt = m.num_tokens, cfg.rms_eps, self.dtype
        pos = m.positions[:T]
        rows = (m.extra["row_state"], m.extra["row_back"], m.extra["row_fwd"], pos,
                self._run_rows(m))
        runs, starts = self.runs, self.pass_starts
        step = w.get("loop_step")
        x = ops.embed_rows(m.input_ids[:T], w["embed"])
        h = torch.empty((T, cfg.hidden), dtype=dt, device=x.device)
        ops.residual_add_norm(x, None, None, step[starts[0]] if 0 in starts else None,
                              w["layers"][runs[0]]["norm1"], eps, 1.0, h)
        for ri, li in enumerate(runs):
            ly, lw = cfg.layers[li], w["layers"][li]
            mx = ly.mixer
            if mx.kind == "diff_attention":
                y1 = self._diff_attention(ri, mx, lw, h, m)
            elif mx.kind == "gla":
                y1 = self._gla(ri, mx, lw, h, m, rows)
            else:
                y1 = self._channel_delta(ri, mx, lw, h, m, rows)
            y2 = self._mlp(ly.mlp, lw, h) if ly.mlp is not None else None
            last = ri + 1 == len(runs)
            nw = None if last else w["layers"][runs[ri + 1]]["norm1"]
            shift = step[starts[ri + 1]] if ri + 1 in starts else None
            if taps is not None:
                ops.residual_add_norm(x, y1, y2)
                taps.append(x.clone())
                if not last:
                    ops.residual_add_norm(x, None, None, shift, nw, eps, 1.0, h)
            else:
                ops.residual_add_norm(x, y1, y2, shift, nw, eps, 1.0, None if last else h)
        xs = x if m.logits_idx is None else x.index_select(0, m.logits_idx.long())
        hn = ops.rms_norm_rows(xs, w["final_norm"], eps,
                               torch.empty(xs.shape, dtype=dt, device=x.device), 1.0)
        return ops.matmul_nt(hn, w["lm_head"], out_dtype=torch.float32)
