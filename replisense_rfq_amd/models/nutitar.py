"""Nutitar: parallel-sublayer layers whose mixer reads a token-shifted input, with latent
attention that carries a rotated key part, windowed sigmoid attention and softmax attention
whose values are its keys, and xIELU feed-forwards, on the kernels of csrc/kernels/mix_*.hip.

The residual stream x is fp32.  One zero-centred RMS norm per layer feeds both sublayers; the
mixer reads the normed row mixed with the previous token's normed row:

  x = embed[token] * embed_scale
  per layer:
    h  = rms(x) (1 + w)
    hs = h + (h' - h) * shift          h' = h of the previous token (per-sequence state; zeros
                                       before the first token)
    x += m * (mixer(hs) + ff(h))
  logits = head . (rms(x) (1 + w_final))

The residual update and the next layer's norm are one kernel (residual_add_norm, fp32 out);
the token shift (token_shift_mix) turns that row into the two GEMM inputs.  Mixers:

rope_latent_attention   q | dkv | gate in one product.  q holds per head ``dim`` plain and
  ``rot_dim`` rotated dimensions; dkv holds the latent (RMS-normed, ``kv_rank`` wide) and one
  rotated key part shared by all heads; the page row is [latent | key part] (a layer with
  kv_from reads another layer's pages and projects no dkv).  Keys and values are per-head
  up-projections of the latent, so both products run in the latent space: the plain query part
  is carried there (q W_uk per head) and meets the latent, the rotated part meets the key part:
  one (kv_rank + rot_dim)-wide key "head" whose first kv_rank entries are also the values.
  Softmax with a per-head sink logit in the denominator; o = W_uv o' per head, times the
  sigmoid of the head's gate logit.
window_attention   q | k (| v) in one product (+ bias); RMS norm of q and k per head or over
  the whole projection; half-split rotation of the leading rot_dims of every head with plain,
  YaRN or banded frequencies; the values are projected or are the keys as projected.  Position
  i sees j <= i with i - j < window or j < keep_first; weights are a softmax over the visible
  keys or sigmoid(score + bias_h) per visible key.
feed-forward   W_down xielu(W_up h).
"""
from __future__ import annotations

import torch

from .. import ops
from ..parallel.tp import SINGLE, TPContext
from .config import LayeredConfig
from .weights import init_nutitar_weights


class NutitarLM:
    stateful = True            # sequences own a state slot (every layer's previous normed row)

    def __init__(self, cfg: LayeredConfig, device, tp: TPContext = SINGLE, seed: int = 0,
                 weights: dict | None = None, dtype=torch.bfloat16, moe_ep: bool = False):
        if tp.enabled:
            raise ValueError("layer-list models run at TP = 1")
        self.cfg = cfg
        self.tp = tp
        self.device = torch.device(device)
        self.dtype = dtype
        self.w = weights if weights is not None else init_nutitar_weights(cfg, self.device, dtype, seed)
        self.vocab_start = 0
        self.vocab_local = self.w["lm_head"].shape[0]
        # the kernels of this model take no per-head decode work list: one entry per row
        self.hq = self.hkv = 1
        self.kv_k = self.kv_v = self.layer_state = None
        self.norms_folded = False
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False
        self._seq_ids = None
        for ly, lw in zip(cfg.layers, self.w["layers"]):
            m = ly.mixer
            lw["inv_freq"], lw["rot_mult"] = ops.rotary_scaled_freq(m.rot_dims, m.rot_base,
                                                                    m.rot_scaling, self.device)

    # engine hooks shared with the other decoders
    def fold_norms(self) -> bool:
        return False

    def tile_decode_weights(self, mode: str | None = None) -> int:
        return 0

    def attach_kv_cache(self, k_pools, v_pools, state=None, layer_state=None) -> None:
        """Per layer: K pool [num_blocks, G, block, dim] and V pool [.., vdim] for windowed
        attention; one pool [num_blocks, 1, block, kv_rank + rot_dim] for latent attention (the
        same tensor where a layer reads another's); layer_state[i]["prev"] [2*slots, d] fp32."""
        assert len(k_pools) == self.cfg.n_layers
        self.kv_k, self.kv_v, self.layer_state = k_pools, v_pools, layer_state

    def _decode_work(self, n: int):
        """(sequence index, query block 0) per decode-section sequence; views of two tensors
        that only grow (never inside a graph capture: the warm-up run sizes them)."""
        if self._seq_ids is None or self._seq_ids[0].numel() < n:
            size = max(1024, 2 * n)
            self._seq_ids = (torch.arange(size, dtype=torch.int32, device=self.device),
                             torch.zeros(size, dtype=torch.int32, device=self.device))
        return self._seq_ids[0][:n], self._seq_ids[1][:n]

    def weight_bytes(self) -> int:
        tot = sum(v.numel() * v.element_size() for v in self.w.values() if isinstance(v, torch.Tensor))
        for lw in self.w["layers"]:
            tot += sum(t.numel() * t.element_size() for t in lw.values() if isinstance(t, torch.Tensor))
        return tot

    # ------------------------------------------------------------------ mixers
    def _attend(self, m, q, kc, vc, vdim, bias, gate, out, mx, sigmoid=False):
        """Both sections of the step through attn_keep_window."""
        T, D = m.num_tokens, m.num_decode
        if D > 0:
            ids, zeros = self._decode_work(m.dec_q_len.shape[0])
            ops.attn_keep_window(q[:D], kc, vc, vdim, m.dec_block_tables, m.dec_q_start, m.dec_q_len,
                                 m.dec_kv_len, ids, zeros, bias, None if gate is None else gate[:D],
                                 out[:D], mx.scale, mx.window, mx.keep_first, sigmoid,
                                 short_rows=ops.TALK_DECODE_MAX_ROWS)
        if T > D:
            ops.attn_keep_window(q[D:], kc, vc, vdim, m.pf_block_tables, m.pf_q_start, m.pf_q_len,
                                 m.pf_kv_len, m.work_seq, m.work_qblk, bias,
                                 None if gate is None else gate[D:T], out[D:T], mx.scale, mx.window,
                                 mx.keep_first, sigmoid)

    def _window_attention(self, li, mx, lw, hs, m):
        T, dt, dev = m.num_tokens, self.dtype, hs.device
        H, G, dim, vd = mx.heads, mx.kv_heads, mx.dim, mx.vdim
        kc, vc = self.kv_k[li], self.kv_v[li]
        pr = ops.matmul_nt(hs, lw["proj"])
        q = torch.empty((T, H, dim), dtype=torch.float32, device=dev)
        ops.qk_norm_rotary_append(pr, lw["proj_b"], lw["qn"], lw["kn"], mx.qk_norm == "all", dim,
                                  self.cfg.rms_eps, m.positions[:T], lw["inv_freq"], lw["rot_mult"],
                                  0, 0, m.slot_mapping[:T], kc, vc, H, G, dim, dim, vd,
                                  1 if mx.v_is_k else 0, q)
        attn = torch.empty((T, H * vd), dtype=dt, device=dev)
        self._attend(m, q, kc, vc, vd, lw["pb"], None, attn, mx, sigmoid=mx.weights == "sigmoid")
        if lw["o_b"] is not None:
            return torch.addmm(lw["o_b"], attn, lw["o"].t())
        return ops.matmul_nt(attn, lw["o"])

    def _latent_attention(self, li, mx, lw, hs, m):
        T, dt, dev = m.num_tokens, self.dtype, hs.device
        H, dim, rd, R, vd = mx.heads, mx.dim, mx.rot_dim, mx.kv_rank, mx.vdim
        pool = self.kv_k[li]
        own = mx.kv_from < 0
        pr = ops.matmul_nt(hs, lw["proj"])                  # q | dkv | gate  (or q | gate)
        nq = H * (dim + rd)
        gate = pr[:, nq + (R + rd if own else 0):]
        qf = torch.empty((T, H, dim + rd), dtype=torch.float32, device=dev)
        ops.qk_norm_rotary_append(pr, None, None, lw["dkv_norm"] if own else None, False, R,
                                  self.cfg.rms_eps, m.positions[:T], lw["inv_freq"], lw["rot_mult"],
                                  dim, R, m.slot_mapping[:T], pool if own else None, None, H,
                                  1 if own else 0, dim + rd, R + rd, 0, 2, qf)
        # the plain query part (untouched by the kernel above: read as the projection left it)
        # carried into the latent space, fp32 (a score operand), beside the rotated part: one
        # (R + rd)-wide query per head
        qn = pr[:, :nq].unflatten(1, (H, dim + rd))[:, :, :dim].transpose(0, 1)
        qa = ops.bmm_f32(qn, lw["uk"])                                              # [H, T, R]
        qfull = torch.cat([qa.transpose(0, 1), qf[:, :, dim:]], -1)
        lat = torch.empty((T, H * R), dtype=dt, device=dev)
        self._attend(m, qfull, pool, pool, R, lw["sink"], gate, lat, mx)
        ov = torch.bmm(lat.view(T, H, R).transpose(0, 1), lw["uv_t"])               # [H, T, vdim]
        return ops.matmul_nt(ov.transpose(0, 1).reshape(T, H * vd), lw["o"])

    def _mlp(self, lw, h):
        ap, an = lw["xi"]
        return ops.matmul_nt(ops.xielu_rows(ops.matmul_nt(h, lw["up"]), ap, an), lw["down"])

    # ------------------------------------------------------------------ forward
    def forward(self, m, taps: list | None = None) -> torch.Tensor:
        """Logits [rows, V] (fp32) of the step.  ``taps``: a list that receives the residual
        stream after every layer (debugging / layer-wise tests)."""
        cfg, w = self.cfg, self.w
        T, eps, dt, mult = m.num_tokens, cfg.rms_eps, self.dtype, cfg.residual_mult
        pos = m.positions[:T]
        rs, rb, rf = m.extra["row_state"], m.extra["row_back"], m.extra["row_fwd"]
        f32 = dt == torch.float32
        x = ops.embed_rows(m.input_ids[:T], w["embed"], scale=cfg.embed_scale)
        hf = torch.empty((T, cfg.hidden), dtype=torch.float32, device=x.device)
        ops.residual_add_norm(x, None, None, None, w["layers"][0]["norm1"], eps, 1.0, hf)
        n = cfg.n_layers
        for li, ly in enumerate(cfg.layers):
            lw, mx = w["layers"][li], ly.mixer
            # fp32 model: the normed row itself feeds the feed-forward, one mix is formed;
            # bf16: mix 0 (shift 0) is the row in bf16, mix 1 the shifted row
            mu = lw["mu"][1:] if f32 else lw["mu"]
            mixes = ops.token_shift_mix(hf, mu, self.layer_state[li]["prev"], rs, rb, rf, pos,
                                        torch.empty((mu.shape[0], T, cfg.hidden), dtype=dt,
                                                    device=x.device))
            h, hs = (hf, mixes[0]) if f32 else (mixes[0], mixes[1])
            if mx.kind == "rope_latent_attention":
                y1 = self._latent_attention(li, mx, lw, hs, m)
            else:
                y1 = self._window_attention(li, mx, lw, hs, m)
            y2 = self._mlp(lw, h) if ly.mlp is not None else None
            last = li + 1 == n
            nw = None if last else w["layers"][li + 1]["norm1"]
            if taps is not None:
                ops.residual_add_norm(x, y1, y2, mult=mult)
                taps.append(x.clone())
                if not last:
                    ops.residual_add_norm(x, None, None, None, nw, eps, 1.0, hf)
            else:
                ops.residual_add_norm(x, y1, y2, None, nw, eps, 1.0, None if last else hf, mult=mult)
        xs = x if m.logits_idx is None else x.index_select(0, m.logits_idx.long())
        hn = ops.rms_norm_rows(xs, w["final_norm"], eps,
                               torch.empty(xs.shape, dtype=dt, device=x.device), 1.0)
        return ops.matmul_nt(hn, w["lm_head"], out_dtype=torch.float32)
