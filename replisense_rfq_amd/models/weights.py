"""Seeded random-init weights, generated directly as this rank's TP shard.

BASELINE.json runs the benchmark on random-init weights of the real
architectures (no checkpoints, no network).  Each tensor is drawn on the target
device from a generator seeded by (seed, layer, name, tp_rank), so TP workers
build their shards independently with no weight broadcast
and a replica restart regenerates identical weights.

Layout (torch Linear convention, out = x @ W^T):
  qkv     [(Hq + 2 Hkv)/TP * 128, d]      column-parallel (q heads | k heads | v heads)
  o       [d, Hq/TP * 128]                row-parallel
  gate_up [2 F/TP, d]                     column-parallel (gate | up)
  down    [d, F/TP]                       row-parallel
  MoE:    router [E, d]; w13 [E, 2F/TP, d]; w2 [E, d, F/TP]
  embed   [V, d] replicated; lm_head [V/TP, d] vocab-parallel

A safetensors loader with the same names is provided for real checkpoints.
"""
from __future__ import annotations

import hashlib

import torch

from ..parallel.tp import TPContext
from .config import ModelConfig


def _seed(*parts) -> int:
    h = hashlib.blake2b(repr(parts).encode(), digest_size=8).digest()
    return int.from_bytes(h, "little") & ((1 << 63) - 1)


def _randn(shape, std, seed_parts, device, dtype):
    g = torch.Generator(device=device)
    g.manual_seed(_seed(*seed_parts))
    t = torch.empty(shape, dtype=torch.float32, device=device)
    t.normal_(0.0, std, generator=g)
    return t.to(dtype)


class LayerWeights(dict):
    __getattr__ = dict.__getitem__


def init_weights(cfg: ModelConfig, tp: TPContext, device, dtype=torch.bfloat16, seed: int = 0,
                 moe_ep: bool = False):
    """moe_ep: experts are split across the TP group (each rank holds E/TP whole
    experts) instead of every expert's FFN being column/row split."""
    d, D = cfg.hidden, cfg.head_dim
    R = tp.world
    if cfg.n_heads % R or cfg.n_kv_heads % R or cfg.ffn % R or cfg.vocab_size % R:
        raise ValueError(f"{cfg.name} is not divisible by TP={R}")
    if moe_ep and cfg.n_experts % R:
        raise ValueError(f"{cfg.n_experts} experts are not divisible by EP={R}")
    hq, hkv, F = cfg.n_heads // R, cfg.n_kv_heads // R, cfg.ffn // R
    std = cfg.init_std
    r = tp.rank
    ones = lambda n: torch.ones(n, dtype=dtype, device=device)  # noqa: E731
    layers = []
    for li in range(cfg.n_layers):
        lw = LayerWeights(
            attn_norm=ones(d),
            mlp_norm=ones(d),
            qkv=_randn(((hq + 2 * hkv) * D, d), std, (seed, li, "qkv", r), device, dtype),
            o=_randn((d, hq * D), std, (seed, li, "o", r), device, dtype),
        )
        if cfg.is_moe:
            E = cfg.n_experts
            lw["router"] = _randn((E, d), std, (seed, li, "router"), device, dtype)
            if moe_ep:
                El, Ff = E // R, cfg.ffn
                lw["w13"] = _randn((El, 2 * Ff, d), std, (seed, li, "w13e", r), device, dtype)
                lw["w2"] = _randn((El, d, Ff), std, (seed, li, "w2e", r), device, dtype)
            else:
                lw["w13"] = _randn((E, 2 * F, d), std, (seed, li, "w13", r), device, dtype)
                lw["w2"] = _randn((E, d, F), std, (seed, li, "w2", r), device, dtype)
        else:
            lw["gate_up"] = _randn((2 * F, d), std, (seed, li, "gate_up", r), device, dtype)
            lw["down"] = _randn((d, F), std, (seed, li, "down", r), device, dtype)
        layers.append(lw)
    v0, v1 = tp.shard(cfg.vocab_size)
    return dict(
        embed=_randn((cfg.vocab_size, d), std, (seed, "embed"), device, dtype),
        final_norm=ones(d),
        lm_head=_randn((v1 - v0, d), std, (seed, "lm_head", r), device, dtype),
        layers=layers,
        vocab_start=v0,
    )


class _LazyCheckpoint:
    """Tensor name -> file index over a set of safetensors files; reads only the
    requested slice of each tensor (memory-mapped), so a TP rank of a 141 GB
    Llama-3-70B checkpoint touches ~1/8 of it and never holds the whole file."""

    def __init__(self, files):
        from safetensors import safe_open

        self._handles = [safe_open(f, framework="pt", device="cpu") for f in files]
        self._where = {}
        for h in self._handles:
            for k in h.keys():
                self._where[k] = h

    def __contains__(self, name):
        return name in self._where

    def full(self, name):
        return self._where[name].get_tensor(name)

    def rows(self, name, a, b):          # W[a:b]
        return self._where[name].get_slice(name)[a:b]

    def cols(self, name, a, b):          # W[:, a:b]
        return self._where[name].get_slice(name)[:, a:b]


def load_safetensors(path: str, cfg: ModelConfig, tp: TPContext, device, dtype=torch.bfloat16,
                     moe_ep: bool = False):
    """Load HF-style Llama/Mixtral safetensors shards into this rank's layout
    (Megatron TP split, or whole experts per rank with moe_ep), reading only this
    rank's slices; each layer is moved to the device as it is assembled."""
    import glob
    import os

    files = sorted(glob.glob(os.path.join(path, "*.safetensors"))) if os.path.isdir(path) else [path]
    ck = _LazyCheckpoint(files)

    def cols(name, n):        # column-parallel: this rank's rows of W
        a, b = tp.shard(n)
        return ck.rows(name, a, b)

    def rows(name, n):        # row-parallel: this rank's columns of W
        a, b = tp.shard(n)
        return ck.cols(name, a, b)

    D, F = cfg.head_dim, cfg.ffn
    layers = []
    for li in range(cfg.n_layers):
        p = f"model.layers.{li}."
        q = cols(p + "self_attn.q_proj.weight", cfg.n_heads * D)
        k = cols(p + "self_attn.k_proj.weight", cfg.n_kv_heads * D)
        v = cols(p + "self_attn.v_proj.weight", cfg.n_kv_heads * D)
        lw = LayerWeights(
            attn_norm=ck.full(p + "input_layernorm.weight"),
            mlp_norm=ck.full(p + "post_attention_layernorm.weight"),
            qkv=torch.cat([q, k, v]),
            o=rows(p + "self_attn.o_proj.weight", cfg.n_heads * D),
        )
        if cfg.is_moe and moe_ep and tp.world > 1:
            ex = p + "block_sparse_moe."
            El = cfg.n_experts // tp.world
            mine = range(tp.rank * El, (tp.rank + 1) * El)
            lw["router"] = ck.full(ex + "gate.weight")
            lw["w13"] = torch.stack([torch.cat([ck.full(f"{ex}experts.{e}.w1.weight"),
                                                ck.full(f"{ex}experts.{e}.w3.weight")])
                                     for e in mine])
            lw["w2"] = torch.stack([ck.full(f"{ex}experts.{e}.w2.weight") for e in mine])
        elif cfg.is_moe:
            ex = p + "block_sparse_moe."
            lw["router"] = ck.full(ex + "gate.weight")
            lw["w13"] = torch.stack([torch.cat([cols(f"{ex}experts.{e}.w1.weight", F),
                                                cols(f"{ex}experts.{e}.w3.weight", F)])
                                     for e in range(cfg.n_experts)])
            lw["w2"] = torch.stack([rows(f"{ex}experts.{e}.w2.weight", F)
                                    for e in range(cfg.n_experts)])
        else:
            lw["gate_up"] = torch.cat([cols(p + "mlp.gate_proj.weight", F),
                                       cols(p + "mlp.up_proj.weight", F)])
            lw["down"] = rows(p + "mlp.down_proj.weight", F)
        layers.append(LayerWeights({k: t.to(device=device, dtype=dtype).contiguous()
                                    for k, t in lw.items()}))
    v0, v1 = tp.shard(cfg.vocab_size)
    head_name = "lm_head.weight" if "lm_head.weight" in ck else "model.embed_tokens.weight"
    return dict(
        embed=ck.full("model.embed_tokens.weight").to(device=device, dtype=dtype),
        final_norm=ck.full("model.norm.weight").to(device=device, dtype=dtype),
        lm_head=ck.rows(head_name, v0, v1).to(device=device, dtype=dtype).contiguous(),
        layers=layers,
        vocab_start=v0,
    )


def shard_weights(full: dict, cfg: ModelConfig, tp: TPContext, moe_ep: bool = False) -> dict:
    """Slice full (TP=1) weights into this rank's Megatron shard (same layout as
    init_weights), e.g. to check TP numerics against the single-device model.
    moe_ep: whole experts per rank instead of FFN-split experts."""
    D, R, r = cfg.head_dim, tp.world, tp.rank
    hq, hkv, F = cfg.n_heads // R, cfg.n_kv_heads // R, cfg.ffn // R
    Hq, Hkv = cfg.n_heads, cfg.n_kv_heads
    layers = []
    for lw in full["layers"]:
        q = lw["qkv"][: Hq * D][r * hq * D:(r + 1) * hq * D]
        k = lw["qkv"][Hq * D:(Hq + Hkv) * D][r * hkv * D:(r + 1) * hkv * D]
        v = lw["qkv"][(Hq + Hkv) * D:][r * hkv * D:(r + 1) * hkv * D]
        out = LayerWeights(attn_norm=lw["attn_norm"], mlp_norm=lw["mlp_norm"],
                           qkv=torch.cat([q, k, v]).contiguous(),
                           o=lw["o"][:, r * hq * D:(r + 1) * hq * D].contiguous())
        if cfg.is_moe and moe_ep:
            El = cfg.n_experts // R
            out["router"] = lw["router"]
            out["w13"] = lw["w13"][r * El:(r + 1) * El].contiguous()
            out["w2"] = lw["w2"][r * El:(r + 1) * El].contiguous()
        elif cfg.is_moe:
            Ff = cfg.ffn
            out["router"] = lw["router"]
            out["w13"] = torch.cat([lw["w13"][:, r * F:(r + 1) * F],
                                    lw["w13"][:, Ff + r * F:Ff + (r + 1) * F]], 1).contiguous()
            out["w2"] = lw["w2"][:, :, r * F:(r + 1) * F].contiguous()
        else:
            Ff = cfg.ffn
            out["gate_up"] = torch.cat([lw["gate_up"][r * F:(r + 1) * F],
                                        lw["gate_up"][Ff + r * F:Ff + (r + 1) * F]]).contiguous()
            out["down"] = lw["down"][:, r * F:(r + 1) * F].contiguous()
        layers.append(out)
    v0, v1 = tp.shard(cfg.vocab_size)
    return dict(embed=full["embed"], final_norm=full["final_norm"],
                lm_head=full["lm_head"][v0:v1].contiguous(), layers=layers, vocab_start=v0)


def export_hf(full: dict, cfg: ModelConfig) -> dict[str, torch.Tensor]:
    """Inverse of load_safetensors for TP=1 weights: HF tensor names -> tensors
    (used to write test checkpoints and to round-trip the loader)."""
    D, F, Hq, Hkv = cfg.head_dim, cfg.ffn, cfg.n_heads, cfg.n_kv_heads
    out = {"model.embed_tokens.weight": full["embed"], "model.norm.weight": full["final_norm"],
           "lm_head.weight": full["lm_head"]}
    from .. import ops

    for li, lw in enumerate(full["layers"]):
        p = f"model.layers.{li}."
        # an engine's in-place decode-tiled projections (DecoderLM.tile_decode_weights)
        lw = {k: ops.untile_weight(v) if isinstance(v, torch.Tensor) and ops.tiled_only(v)
              else v for k, v in lw.items()}
        out[p + "input_layernorm.weight"] = lw["attn_norm"]
        out[p + "post_attention_layernorm.weight"] = lw["mlp_norm"]
        out[p + "self_attn.q_proj.weight"] = lw["qkv"][: Hq * D]
        out[p + "self_attn.k_proj.weight"] = lw["qkv"][Hq * D:(Hq + Hkv) * D]
        out[p + "self_attn.v_proj.weight"] = lw["qkv"][(Hq + Hkv) * D:]
        out[p + "self_attn.o_proj.weight"] = lw["o"]
        if cfg.is_moe:
            ex = p + "block_sparse_moe."
            out[ex + "gate.weight"] = lw["router"]
            for e in range(cfg.n_experts):
                out[f"{ex}experts.{e}.w1.weight"] = lw["w13"][e, :F]
                out[f"{ex}experts.{e}.w3.weight"] = lw["w13"][e, F:]
                out[f"{ex}experts.{e}.w2.weight"] = lw["w2"][e]
        else:
            out[p + "mlp.gate_proj.weight"] = lw["gate_up"][:F]
            out[p + "mlp.up_proj.weight"] = lw["gate_up"][F:]
            out[p + "mlp.down_proj.weight"] = lw["down"]
    return {k: v.contiguous() for k, v in out.items()}


# --------------------------------------------------------------------------
# Layer-list models (LayeredConfig).  Tensor names are the checkpoint's own:
#   embed, head [V, d]; final.norm [d]
#   l<i>.norm1 | norm1b | norm2 | norm2b | ls1 | ls2 [d]; l<i>.canon1 | canon2 [d, taps]
#   l<i>.mix.q [H*dim, d]  .k [G*dim, d]  .v [G*vdim, d]  .o [d, H*vdim]
#   l<i>.mix.q.norm | k.norm [dim]; l<i>.mix.talk [H, H]; l<i>.mix.sink [H]
#   l<i>.mlp.gate | up [F, d]; l<i>.mlp.down [d, F]
# Loaded layout per layer: qkv = q|k|v rows and gate_up = gate|up rows in the model's
# dtype; norm weights, layer scales, convolution taps, talk and sink in fp32.
LAYERED_F32 = ("norm1", "norm1b", "norm2", "norm2b", "ls1", "ls2", "canon1", "canon2")


def _assemble_layer(get, ly, has, dtype, device):
    lw = LayerWeights()
    for k in LAYERED_F32:
        if has(k):
            lw[k] = get(k).float().contiguous().to(device)
    lw["qkv"] = torch.cat([get("mix.q"), get("mix.k"), get("mix.v")], 0).to(dtype).contiguous().to(device)
    lw["o"] = get("mix.o").to(dtype).contiguous().to(device)
    lw["q_norm"] = get("mix.q.norm").float().to(device)
    lw["k_norm"] = get("mix.k.norm").float().to(device)
    lw["talk"] = get("mix.talk").float().contiguous().to(device)
    lw["sink"] = get("mix.sink").float().to(device)
    if ly.mlp is not None:
        lw["gate_up"] = torch.cat([get("mlp.gate"), get("mlp.up")], 0).to(dtype).contiguous().to(device)
        lw["down"] = get("mlp.down").to(dtype).contiguous().to(device)
    m = ly.mixer
    shapes = {"qkv": (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim),), "talk": (m.heads, m.heads),
              "sink": (m.heads,), "q_norm": (m.dim,), "k_norm": (m.dim,)}
    for k, shp in shapes.items():
        if tuple(lw[k].shape[:len(shp)]) != shp:
            raise ValueError(f"tensor {k}: shape {tuple(lw[k].shape)} does not fit the configuration")
    return lw


def load_layered_safetensors(path: str, cfg, device, dtype=torch.bfloat16) -> dict:
    import glob
    import os

    files = sorted(glob.glob(os.path.join(path, "*.safetensors"))) if os.path.isdir(path) else [path]
    ck = _LazyCheckpoint(files)
    if cfg.architecture == "Numalorn":
        return _numalorn_assemble(ck.full, lambda k: k in ck, cfg, device, dtype)
    if cfg.architecture == "Bilolix":
        return _bilolix_assemble(ck.full, lambda k: k in ck, cfg, device, dtype)
    if cfg.architecture == "Nutitar":
        return _nutitar_assemble(ck.full, lambda k: k in ck, cfg, device, dtype)
    w = {"embed": ck.full("embed").to(dtype).to(device), "lm_head": ck.full("head").to(dtype).to(device),
         "final_norm": ck.full("final.norm").float().to(device), "vocab_start": 0, "layers": []}
    for i, ly in enumerate(cfg.layers):
        pre = f"l{i}."
        w["layers"].append(_assemble_layer(lambda k: ck.full(pre + k), ly, lambda k: pre + k in ck,
                                           dtype, device))
    return w


def init_layered_weights(cfg, device, dtype=torch.bfloat16, seed: int = 0) -> dict:
    """Seeded random weights of a layer-list model (tests and benchmarks): projections
    N(0, init_std) scaled so that activations stay O(1), norm weights near one, layer
    scales, taps, sinks and the head-mixing matrix away from their neutral values so
    that each of them shows in the logits."""
    d = cfg.hidden
    full = {}

    def rnd(name, shape, std, mean=0.0):
        t = _randn(shape, std, (seed, name), "cpu", torch.float32) + mean
        full[name] = t.to(torch.bfloat16).float()      # checkpoint precision
        return full[name]

    rnd("embed", (cfg.vocab_size, d), 1.0)
    rnd("head", (cfg.vocab_size, d), d ** -0.5)
    rnd("final.norm", (d,), 0.1, 1.0)
    for i, ly in enumerate(cfg.layers):
        m, p = ly.mixer, f"l{i}."
        for k in ("norm1", "norm1b", "norm2", "norm2b"):
            rnd(p + k, (d,), 0.1, 1.0)
        rnd(p + "ls1", (d,), 0.1, 0.5)
        rnd(p + "ls2", (d,), 0.1, 0.5)
        rnd(p + "canon1", (d, cfg.canon_taps), 0.3)
        rnd(p + "canon2", (d, cfg.canon_taps), 0.3)
        rnd(p + "mix.q", (m.heads * m.dim, d), d ** -0.5)
        rnd(p + "mix.k", (m.kv_heads * m.dim, d), d ** -0.5)
        rnd(p + "mix.v", (m.kv_heads * m.vdim, d), d ** -0.5)
        rnd(p + "mix.o", (d, m.heads * m.vdim), (m.heads * m.vdim) ** -0.5)
        rnd(p + "mix.q.norm", (m.dim,), 0.1, 1.0)
        rnd(p + "mix.k.norm", (m.dim,), 0.1, 1.0)
        full[p + "mix.talk"] = (torch.eye(m.heads) + rnd(p + "mix.talk", (m.heads, m.heads), 0.2)
                                ).to(torch.bfloat16).float()
        rnd(p + "mix.sink", (m.heads,), 1.0)
        if ly.mlp is not None:
            rnd(p + "mlp.gate", (ly.mlp.ff, d), d ** -0.5)
            rnd(p + "mlp.up", (ly.mlp.ff, d), d ** -0.5)
            rnd(p + "mlp.down", (d, ly.mlp.ff), ly.mlp.ff ** -0.5)
    return layered_from_full(full, cfg, device, dtype)


def layered_from_full(full: dict, cfg, device, dtype=torch.bfloat16) -> dict:
    """Loaded layout from a name -> tensor dict under the checkpoint's names."""
    w = {"embed": full["embed"].to(dtype).to(device), "lm_head": full["head"].to(dtype).to(device),
         "final_norm": full["final.norm"].float().to(device), "vocab_start": 0, "layers": [],
         "full": full}
    for i, ly in enumerate(cfg.layers):
        pre = f"l{i}."
        w["layers"].append(_assemble_layer(lambda k: full[pre + k], ly, lambda k: pre + k in full,
                                           dtype, device))
    return w


# --------------------------------------------------------------------------
# Numalorn.  Checkpoint names:
#   embed, head [V, d]; final.norm [d]; l<i>.norm1 | norm2 [d] (stored around zero)
#   latent attention: l<i>.mix.dq [q_rank, d]  .dq.norm [q_rank]  .uq [H*dim, q_rank]
#     .dkv [kv_rank, d]  .dkv.norm [kv_rank] (absent with kv_from)  .uk [H*dim, kv_rank]
#     .uv [H*vdim, kv_rank]  .sink [H]  .o [d, H*vdim]
#   wkv: l<i>.mix.mu.{r,k,v,g,w} [d]  .r | .k | .v | .g [H*N, d]  .w1 [rank, d]  .w2 [H*N, rank]
#     .w0 [H*N]  .u [H, N]  .norm [H*N]  .o [d, H*N]
#   moe: l<i>.mlp.router [E, d]  .correction [E]  .e<j>.gate | up [F, d]  .e<j>.down [d, F]
#     .shared.gate | up [Fs, d]  .shared.down [d, Fs]
# Loaded layout per layer: "down" = dq | dkv rows, uk [H, dim, R] and uv^T [H, R, vdim] for the
# absorbed products, "rkvg" [4, H*N, d], w13 [E, 2F, d] gate | up rows, w2 [E, d, F]; norm
# weights, mu, w0, u, sink, router and correction in fp32.
def _numalorn_assemble(get, has, cfg, device, dtype) -> dict:
    d = cfg.hidden

    def mat(name, rows, cols):
        t = get(name)
        if tuple(t.shape) != (rows, cols):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, expected {(rows, cols)}")
        return t.to(dtype)

    def vec(name, *shape):
        t = get(name)
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t.float().contiguous().to(device)

    V = cfg.vocab_size
    w = {"embed": mat("embed", V, d).to(device), "lm_head": mat("head", V, d).to(device),
         "final_norm": vec("final.norm", d), "vocab_start": 0, "layers": []}
    for i, ly in enumerate(cfg.layers):
        p, m, lw = f"l{i}.", ly.mixer, LayerWeights()
        lw["norm1"] = vec(p + "norm1", d)
        if m.kind == "latent_attention":
            H, R = m.heads, m.kv_rank
            rows = [mat(p + "mix.dq", m.q_rank, d)]
            if m.kv_from < 0:
                rows.append(mat(p + "mix.dkv", R, d))
                lw["dkv_norm"] = vec(p + "mix.dkv.norm", R)
            lw["down"] = torch.cat(rows, 0).contiguous().to(device)
            lw["dq_norm"] = vec(p + "mix.dq.norm", m.q_rank)
            lw["uq"] = mat(p + "mix.uq", H * m.dim, m.q_rank).contiguous().to(device)
            lw["uk"] = mat(p + "mix.uk", H * m.dim, R).view(H, m.dim, R).contiguous().to(device)
            lw["uv_t"] = mat(p + "mix.uv", H * m.vdim, R).view(H, m.vdim, R).transpose(1, 2) \
                .contiguous().to(device)
            lw["sink"] = vec(p + "mix.sink", H)
            lw["o"] = mat(p + "mix.o", d, H * m.vdim).contiguous().to(device)
        else:
            HN = m.heads * m.dim
            lw["mu"] = torch.stack([vec(p + "mix.mu." + s, d) for s in "rkvgw"]).contiguous()
            lw["rkvg"] = torch.stack([mat(p + "mix." + s, HN, d) for s in "rkvg"]).contiguous().to(device)
            w1 = get(p + "mix.w1")
            rank = w1.shape[0]                       # the decay's inner size is the tensor's
            if tuple(w1.shape) != (rank, d):
                raise ValueError(f"tensor {p}mix.w1: shape {tuple(w1.shape)}, expected (rank, {d})")
            lw["w1"] = w1.to(dtype).contiguous().to(device)
            lw["w2"] = mat(p + "mix.w2", HN, rank).contiguous().to(device)
            lw["w0"] = vec(p + "mix.w0", HN)
            lw["u"] = vec(p + "mix.u", m.heads, m.dim)
            lw["gn"] = vec(p + "mix.norm", HN)
            lw["o"] = mat(p + "mix.o", d, HN).contiguous().to(device)
        f = ly.mlp
        if f is not None:
            q = p + "mlp."
            lw["norm2"] = vec(p + "norm2", d)
            # the router's product accumulates and leaves in fp32; its operands are the
            # checkpoint's weights in the model's dtype (exact: they are stored in bf16)
            lw["router"] = mat(q + "router", f.experts, d).contiguous().to(device)
            lw["correction"] = vec(q + "correction", f.experts)
            lw["w13"] = torch.stack([torch.cat([mat(f"{q}e{e}.gate", f.ff, d), mat(f"{q}e{e}.up", f.ff, d)], 0)
                                     for e in range(f.experts)]).contiguous().to(device)
            lw["w2e"] = torch.stack([mat(f"{q}e{e}.down", d, f.ff) for e in range(f.experts)]) \
                .contiguous().to(device)
            if f.shared_ff:
                lw["shared_gu"] = torch.cat([mat(q + "shared.gate", f.shared_ff, d),
                                             mat(q + "shared.up", f.shared_ff, d)], 0).contiguous().to(device)
                lw["shared_down"] = mat(q + "shared.down", d, f.shared_ff).contiguous().to(device)
        w["layers"].append(lw)
    return w


def init_numalorn_weights(cfg, device, dtype=torch.bfloat16, seed: int = 0,
                          keep_full: bool = True) -> dict:
    """Seeded random Numalorn weights under the checkpoint's names (tests and benchmarks):
    projections scaled so that activations stay O(1); sinks, corrections, bonuses, decays and
    zero-centred norm weights away from their neutral values so that each shows in the logits.
    ``keep_full`` False (benchmark sizes): drawn on the device, the name -> tensor dict is not
    kept."""
    d, full = cfg.hidden, {}

    def rnd(name, shape, std, mean=0.0):
        if keep_full:
            t = _randn(shape, std, (seed, name), "cpu", torch.float32) + mean
            full[name] = t.to(torch.bfloat16).float()
        else:
            full[name] = (_randn(shape, std, (seed, name), device, torch.float32) + mean).to(torch.bfloat16)
        return full[name]

    rnd("embed", (cfg.vocab_size, d), 1.0)
    rnd("head", (cfg.vocab_size, d), 2.0 * d ** -0.5)
    rnd("final.norm", (d,), 0.2)
    for i, ly in enumerate(cfg.layers):
        p, m = f"l{i}.", ly.mixer
        rnd(p + "norm1", (d,), 0.2)
        if m.kind == "latent_attention":
            H, R = m.heads, m.kv_rank
            rnd(p + "mix.dq", (m.q_rank, d), d ** -0.5)
            rnd(p + "mix.dq.norm", (m.q_rank,), 0.1, 1.0)
            rnd(p + "mix.uq", (H * m.dim, m.q_rank), 1.5 * m.q_rank ** -0.5)
            if m.kv_from < 0:
                rnd(p + "mix.dkv", (R, d), d ** -0.5)
                rnd(p + "mix.dkv.norm", (R,), 0.1, 1.0)
            rnd(p + "mix.uk", (H * m.dim, R), 1.5 * R ** -0.5)
            rnd(p + "mix.uv", (H * m.vdim, R), R ** -0.5)
            rnd(p + "mix.sink", (H,), 1.0)
            rnd(p + "mix.o", (d, H * m.vdim), (H * m.vdim) ** -0.5)
        else:
            HN = m.heads * m.dim
            for s in "rkvgw":
                rnd(p + "mix.mu." + s, (d,), 0.25, 0.5)
            for s in "rkvg":
                rnd(p + "mix." + s, (HN, d), d ** -0.5)
            rnd(p + "mix.w1", (cfg.decay_rank, d), d ** -0.5)
            rnd(p + "mix.w2", (HN, cfg.decay_rank), cfg.decay_rank ** -0.5)
            rnd(p + "mix.w0", (HN,), 1.0, -2.0)
            rnd(p + "mix.u", (m.heads, m.dim), 0.5)
            rnd(p + "mix.norm", (HN,), 0.1, 1.0)
            rnd(p + "mix.o", (d, HN), HN ** -0.5)
        f = ly.mlp
        if f is not None:
            q = p + "mlp."
            rnd(p + "norm2", (d,), 0.2)
            rnd(q + "router", (f.experts, d), 2.0 * d ** -0.5)
            rnd(q + "correction", (f.experts,), 0.3)
            for e in range(f.experts):
                rnd(f"{q}e{e}.gate", (f.ff, d), d ** -0.5)
                rnd(f"{q}e{e}.up", (f.ff, d), d ** -0.5)
                rnd(f"{q}e{e}.down", (d, f.ff), f.ff ** -0.5)
            if f.shared_ff:
                rnd(q + "shared.gate", (f.shared_ff, d), d ** -0.5)
                rnd(q + "shared.up", (f.shared_ff, d), d ** -0.5)
                rnd(q + "shared.down", (d, f.shared_ff), f.shared_ff ** -0.5)
    if not keep_full:
        return _numalorn_assemble(lambda k: full.pop(k), lambda k: k in full, cfg, device, dtype)
    return numalorn_from_full(full, cfg, device, dtype)


def numalorn_from_full(full: dict, cfg, device, dtype=torch.bfloat16) -> dict:
    w = _numalorn_assemble(lambda k: full[k], lambda k: k in full, cfg, device, dtype)
    w["full"] = full
    return w


# --------------------------------------------------------------------------
# Bilolix.  Checkpoint names:
#   embed, head [V, d]; final.norm [d]; loop.step [times, d]; l<i>.norm1 [d] (stored around zero)
#   attention: l<i>.mix.q [H*2*dim, d]  .k [G*2*dim, d]  .v [G*vdim, d]  .g [H, d]  .o [d, H*vdim]
#     .lq1 | .lk1 | .lq2 | .lk2 [dim]
#   gla: l<i>.mix.q | .k [H*dim, d]  .v | .g [H*vdim, d]  .a1 [rank, d]  .a2 [H*dim, rank]
#     .a2.b [H*dim]  .norm [vdim]  .o [d, H*vdim]
#   channel_delta: l<i>.mix.q | .k [G*dim, d]  .v [H*vdim, d]  .q.conv | .k.conv | .v.conv
#     [channels, taps]  .b [H, d]  .A_log [H]  .a1 [rank, d]  .a2 [H*dim, rank]  .dt_bias [H*dim]
#     .g1 [grank, d]  .g2 [H*vdim, grank]  .norm [vdim]  .o [d, H*vdim]
#   dense: l<i>.mlp.up [F, d]  .down [d, F]
#   moe: l<i>.mlp.router [E, d]  .router.b [E]  .e<j>.gate | up [F, d]  .e<j>.down [d, F]
# Loaded layout per layer: attention "qkv" = q | k | v rows; the recurrent mixers' input
# projections are ONE matrix "proj" whose row segments (each padded with zero rows to a
# multiple of 8, so that every column slice of the product starts 16-byte aligned) are listed
# in "seg": name -> (first column, width); inner ranks come from the tensors' shapes; the
# attention's lambda = exp(lq1.lk1) - exp(lq2.lk2) + diff is one float ("lam"); the delta
# rule's rate exp(A_log) and the gla rate 1 / tau are "rate" [H] fp32; norm weights, biases
# and convolution taps in fp32.
SEG_ALIGN = 8


def _stack_segments(parts, d, dtype):
    """[(name, tensor [n, d], pad)] -> (matrix of the segments in order, {name: (first row,
    n)}); after a segment with ``pad`` zero rows bring the next one to a multiple of
    SEG_ALIGN (segments that only this package's kernels read need none)."""
    rows, seg, at = [], {}, 0
    for name, t, pad in parts:
        n = t.shape[0]
        seg[name] = (at, n)
        rows.append(t.to(dtype))
        at += n
        if pad and at % SEG_ALIGN:
            z = (-at) % SEG_ALIGN
            rows.append(torch.zeros((z, d), dtype=dtype, device=t.device))
            at += z
    return torch.cat(rows, 0).contiguous(), seg


def _bilolix_assemble(get, has, cfg, device, dtype) -> dict:
    import math

    d = cfg.hidden

    def mat(name, rows, cols):
        t = get(name)
        if tuple(t.shape) != (rows, cols):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, expected {(rows, cols)}")
        return t.to(dtype)

    def lowrank(name, cols):
        t = get(name)
        if t.dim() != 2 or t.shape[1] != cols:
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, expected (rank, {cols})")
        return t.to(dtype)

    def vec(name, *shape):
        t = get(name)
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t.float().contiguous().to(device)

    V = cfg.vocab_size
    w = {"embed": mat("embed", V, d).to(device), "lm_head": mat("head", V, d).to(device),
         "final_norm": vec("final.norm", d), "vocab_start": 0, "layers": []}
    a, b, times = cfg.loop
    if b > a:
        w["loop_step"] = vec("loop.step", times, d)
    for i, ly in enumerate(cfg.layers):
        p, m, lw = f"l{i}.mix.", ly.mixer, LayerWeights()
        lw["norm1"] = vec(f"l{i}.norm1", d)
        H, G, dim, vd = m.heads, m.kv_heads, m.dim, m.vdim
        if m.kind == "diff_attention":
            lw["qkv"] = torch.cat([mat(p + "q", H * 2 * dim, d), mat(p + "k", G * 2 * dim, d),
                                   mat(p + "v", G * vd, d)], 0).contiguous().to(device)
            lw["g"] = mat(p + "g", H, d).contiguous().to(device)
            lv = [vec(p + n, dim).double().cpu() for n in ("lq1", "lk1", "lq2", "lk2")]
            lw["lam"] = math.exp(float((lv[0] * lv[1]).sum())) - math.exp(float((lv[2] * lv[3]).sum())) \
                + m.diff
        elif m.kind == "gla":
            a1 = lowrank(p + "a1", d)
            proj, seg = _stack_segments([("q", mat(p + "q", H * dim, d), 0), ("k", mat(p + "k", H * dim, d), 0),
                                         ("v", mat(p + "v", H * vd, d), 0), ("g", mat(p + "g", H * vd, d), 1),
                                         ("a1", a1, 1)], d, dtype)
            lw["proj"], lw["seg"] = proj.to(device), seg
            lw["a2"] = mat(p + "a2", H * dim, a1.shape[0]).contiguous().to(device)
            lw["zbias"] = vec(p + "a2.b", H * dim)
            lw["rate"] = torch.full((H,), 1.0 / m.tau, dtype=torch.float32, device=device)
            lw["gn"] = vec(p + "norm", vd)
        elif m.kind == "channel_delta":
            a1, g1 = lowrank(p + "a1", d), lowrank(p + "g1", d)
            proj, seg = _stack_segments([("q", mat(p + "q", G * dim, d), 0), ("k", mat(p + "k", G * dim, d), 0),
                                         ("v", mat(p + "v", H * vd, d), 0), ("b", mat(p + "b", H, d), 1),
                                         ("a1", a1, 1), ("g1", g1, 1)], d, dtype)
            lw["proj"], lw["seg"] = proj.to(device), seg
            taps = m.conv
            lw["conv_w"] = torch.cat([vec(p + "q.conv", G * dim, taps), vec(p + "k.conv", G * dim, taps),
                                      vec(p + "v.conv", H * vd, taps)], 0).contiguous()
            lw["a2"] = mat(p + "a2", H * dim, a1.shape[0]).contiguous().to(device)
            lw["zbias"] = vec(p + "dt_bias", H * dim)
            lw["rate"] = torch.exp(vec(p + "A_log", H).double()).float()
            lw["g2"] = mat(p + "g2", H * vd, g1.shape[0]).contiguous().to(device)
            lw["gn"] = vec(p + "norm", vd)
        else:
            raise ValueError(f"layer {i}: no weights known for mixer {m.kind!r}")
        lw["o"] = mat(p + "o", d, H * vd).contiguous().to(device)
        f, q = ly.mlp, f"l{i}.mlp."
        if f is not None and f.kind == "moe":
            lw["router"] = mat(q + "router", f.experts, d).contiguous().to(device)
            lw["router_b"] = vec(q + "router.b", f.experts)
            lw["w13"] = torch.stack([torch.cat([mat(f"{q}e{e}.gate", f.ff, d), mat(f"{q}e{e}.up", f.ff, d)], 0)
                                     for e in range(f.experts)]).contiguous().to(device)
            lw["w2e"] = torch.stack([mat(f"{q}e{e}.down", d, f.ff) for e in range(f.experts)]) \
                .contiguous().to(device)
        elif f is not None:
            lw["up"] = mat(q + "up", f.ff, d).contiguous().to(device)
            lw["down"] = mat(q + "down", d, f.ff).contiguous().to(device)
        w["layers"].append(lw)
    return w


def init_bilolix_weights(cfg, device, dtype=torch.bfloat16, seed: int = 0,
                         keep_full: bool = True) -> dict:
    """Seeded random Bilolix weights under the checkpoint's names (tests and benchmarks):
    projections scaled so that activations stay O(1); lambda vectors, decay biases, step
    vectors, router biases and zero-centred norm weights away from their neutral values so
    that each shows in the logits.  ``keep_full`` False (benchmark sizes): drawn on the device,
    the name -> tensor dict is not kept."""
    d, full = cfg.hidden, {}

    def rnd(name, shape, std, mean=0.0):
        if keep_full:
            t = _randn(shape, std, (seed, name), "cpu", torch.float32) + mean
            full[name] = t.to(torch.bfloat16).float()
        else:
            full[name] = (_randn(shape, std, (seed, name), device, torch.float32) + mean).to(torch.bfloat16)
        return full[name]

    rnd("embed", (cfg.vocab_size, d), 1.0)
    rnd("head", (cfg.vocab_size, d), 2.0 * d ** -0.5)
    rnd("final.norm", (d,), 0.2)
    if cfg.loop[1] > cfg.loop[0]:
        rnd("loop.step", (cfg.loop[2], d), 0.5)
    for i, ly in enumerate(cfg.layers):
        p, m = f"l{i}.mix.", ly.mixer
        H, G, dim, vd = m.heads, m.kv_heads, m.dim, m.vdim
        rnd(f"l{i}.norm1", (d,), 0.2)
        if m.kind == "diff_attention":
            rnd(p + "q", (H * 2 * dim, d), 2.0 * d ** -0.5)
            rnd(p + "k", (G * 2 * dim, d), 2.0 * d ** -0.5)
            rnd(p + "v", (G * vd, d), d ** -0.5)
            rnd(p + "g", (H, d), 2.0 * d ** -0.5)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                rnd(p + n, (dim,), 0.5 * dim ** -0.5)
        elif m.kind == "gla":
            rnd(p + "q", (H * dim, d), 2.0 * d ** -0.5)
            rnd(p + "k", (H * dim, d), d ** -0.5)
            rnd(p + "v", (H * vd, d), d ** -0.5)
            rnd(p + "g", (H * vd, d), 2.0 * d ** -0.5)
            rnd(p + "a1", (cfg.decay_rank, d), d ** -0.5)
            rnd(p + "a2", (H * dim, cfg.decay_rank), 2.0 * cfg.decay_rank ** -0.5)
            rnd(p + "a2.b", (H * dim,), 1.0, 2.0)
            rnd(p + "norm", (vd,), 0.1, 1.0)
        else:
            rnd(p + "q", (G * dim, d), 2.0 * d ** -0.5)
            rnd(p + "k", (G * dim, d), 2.0 * d ** -0.5)
            rnd(p + "v", (H * vd, d), 2.0 * d ** -0.5)
            for n, c in (("q", G * dim), ("k", G * dim), ("v", H * vd)):
                rnd(p + n + ".conv", (c, m.conv), 0.5)
            rnd(p + "b", (H, d), 2.0 * d ** -0.5)
            rnd(p + "A_log", (H,), 0.5, -1.0)
            rnd(p + "a1", (cfg.decay_rank, d), d ** -0.5)
            rnd(p + "a2", (H * dim, cfg.decay_rank), 2.0 * cfg.decay_rank ** -0.5)
            rnd(p + "dt_bias", (H * dim,), 1.0, -1.0)
            rnd(p + "g1", (cfg.gate_rank, d), d ** -0.5)
            rnd(p + "g2", (H * vd, cfg.gate_rank), 2.0 * cfg.gate_rank ** -0.5)
            rnd(p + "norm", (vd,), 0.1, 1.0)
        rnd(p + "o", (d, H * vd), (H * vd) ** -0.5)
        f, q = ly.mlp, f"l{i}.mlp."
        if f is not None and f.kind == "moe":
            rnd(q + "router", (f.experts, d), 2.0 * d ** -0.5)
            rnd(q + "router.b", (f.experts,), 0.5)
            for e in range(f.experts):
                rnd(f"{q}e{e}.gate", (f.ff, d), d ** -0.5)
                rnd(f"{q}e{e}.up", (f.ff, d), d ** -0.5)
                rnd(f"{q}e{e}.down", (d, f.ff), f.ff ** -0.5)
        elif f is not None:
            rnd(q + "up", (f.ff, d), d ** -0.5)
            rnd(q + "down", (d, f.ff), f.ff ** -0.5)
    if not keep_full:
        return _bilolix_assemble(lambda k: full.pop(k), lambda k: k in full, cfg, device, dtype)
    return bilolix_from_full(full, cfg, device, dtype)


def bilolix_from_full(full: dict, cfg, device, dtype=torch.bfloat16) -> dict:
    w = _bilolix_assemble(lambda k: full[k], lambda k: k in full, cfg, device, dtype)
    w["full"] = full
    return w


# --------------------------------------------------------------------------
# Nutitar.  Checkpoint names:
#   embed, head [V, d]; final.norm [d]; l<i>.norm1 [d] (stored around zero); l<i>.shift [d]
#   latent attention: l<i>.mix.q [H*(dim+rot_dim), d]  .dkv [kv_rank+rot_dim, d]  .dkv.norm [kv_rank]
#     (both absent with kv_from)  .uk [H*dim, kv_rank]  .uv [H*vdim, kv_rank]  .sink [H]  .g [H, d]
#     .o [d, H*vdim]
#   attention: l<i>.mix.q | k | v (+ .b)  .q.norm [H*dim]  .k.norm [G*dim]  .pb [H]  .o (+ .b)
#   attention_2: l<i>.mix.q | k  .q.norm | .k.norm [dim]  .o
#   feed-forward: l<i>.mlp.up [F, d]  .down [d, F]  .act [2]
# Loaded layout per layer: one fused input projection "proj" (its bias "proj_b" in fp32), for
# latent attention q | dkv | g rows with uk [H, dim, R] and uv^T [H, R, vdim] for the products
# in the latent space; "mu" [2, d] = (0, shift): the token shift's mixes (the row itself in the
# model's dtype, and the shifted row); "xi": the unit's two coefficients, formed once in float64.
def _nutitar_assemble(get, has, cfg, device, dtype) -> dict:
    import math

    d = cfg.hidden

    def mat(name, rows, cols):
        t = get(name)
        if tuple(t.shape) != (rows, cols):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, expected {(rows, cols)}")
        return t.to(dtype)

    def vec(name, *shape):
        t = get(name)
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"tensor {name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t.float().contiguous().to(device)

    def softplus(v):
        return max(v, 0.0) + math.log1p(math.exp(-abs(v)))

    V = cfg.vocab_size
    w = {"embed": mat("embed", V, d).to(device), "lm_head": mat("head", V, d).to(device),
         "final_norm": vec("final.norm", d), "vocab_start": 0, "layers": []}
    for i, ly in enumerate(cfg.layers):
        p, m, lw = f"l{i}.mix.", ly.mixer, LayerWeights()
        lw["norm1"] = vec(f"l{i}.norm1", d)
        shift = vec(f"l{i}.shift", d) if has(f"l{i}.shift") else torch.zeros(d, device=device)
        lw["mu"] = torch.stack([torch.zeros_like(shift), shift]).contiguous()
        H, G, dim, vd = m.heads, m.kv_heads, m.dim, m.vdim
        if m.kind == "rope_latent_attention":
            R, rd = m.kv_rank, m.rot_dim
            parts = [mat(p + "q", H * (dim + rd), d)]
            if m.kv_from < 0:
                parts.append(mat(p + "dkv", R + rd, d))
                lw["dkv_norm"] = vec(p + "dkv.norm", R)
            parts.append(mat(p + "g", H, d))
            lw["proj"] = torch.cat(parts, 0).contiguous().to(device)
            lw["proj_b"] = None
            lw["uk"] = mat(p + "uk", H * dim, R).view(H, dim, R).contiguous().to(device)
            lw["uv_t"] = mat(p + "uv", H * vd, R).view(H, vd, R).transpose(1, 2).contiguous().to(device)
            lw["sink"] = vec(p + "sink", H)
            lw["o_b"] = None
        elif m.kind == "window_attention":
            names = ["q", "k"] + ([] if m.v_is_k else ["v"])
            rows = {"q": H * dim, "k": G * dim, "v": G * vd}
            lw["proj"] = torch.cat([mat(p + n, rows[n], d) for n in names], 0).contiguous().to(device)
            lw["proj_b"] = torch.cat([vec(p + n + ".b", rows[n]) for n in names]).contiguous() \
                if m.bias else None
            if m.qk_norm == "all":
                lw["qn"], lw["kn"] = vec(p + "q.norm", H * dim), vec(p + "k.norm", G * dim)
            elif m.qk_norm == "head":
                lw["qn"], lw["kn"] = vec(p + "q.norm", dim), vec(p + "k.norm", dim)
            else:
                lw["qn"] = lw["kn"] = None
            lw["pb"] = vec(p + "pb", H) if m.weights == "sigmoid" else None
            lw["o_b"] = vec(p + "o.b", d).to(dtype) if m.bias else None
        else:
            raise ValueError(f"layer {i}: no weights known for mixer {m.kind!r}")
        lw["o"] = mat(p + "o", d, H * vd).contiguous().to(device)
        f, q = ly.mlp, f"l{i}.mlp."
        if f is not None:
            lw["up"] = mat(q + "up", f.ff, d).contiguous().to(device)
            lw["down"] = mat(q + "down", d, f.ff).contiguous().to(device)
            a = vec(q + "act", 2).double().cpu()
            lw["xi"] = (softplus(float(a[0])), 0.5 + softplus(float(a[1])))
        w["layers"].append(lw)
    return w


def init_nutitar_weights(cfg, device, dtype=torch.bfloat16, seed: int = 0,
                         keep_full: bool = True) -> dict:
    """Seeded random Nutitar weights under the checkpoint's names (tests and benchmarks):
    projections scaled so that activations stay O(1); shifts, sinks, biases, norm weights and
    the unit's numbers away from their neutral values so that each shows in the logits.
    ``keep_full`` False (benchmark sizes): drawn on the device, the name -> tensor dict is not
    kept."""
    d, full = cfg.hidden, {}

    def rnd(name, shape, std, mean=0.0):
        if keep_full:
            t = _randn(shape, std, (seed, name), "cpu", torch.float32) + mean
            full[name] = t.to(torch.bfloat16).float()
        else:
            full[name] = (_randn(shape, std, (seed, name), device, torch.float32) + mean).to(torch.bfloat16)
        return full[name]

    rnd("embed", (cfg.vocab_size, d), 1.0 / max(1.0, cfg.embed_scale))
    rnd("head", (cfg.vocab_size, d), 2.0 * d ** -0.5)
    rnd("final.norm", (d,), 0.2)
    for i, ly in enumerate(cfg.layers):
        p, m = f"l{i}.mix.", ly.mixer
        H, G, dim, vd = m.heads, m.kv_heads, m.dim, m.vdim
        rnd(f"l{i}.norm1", (d,), 0.2)
        rnd(f"l{i}.shift", (d,), 0.25, 0.4)
        if m.kind == "rope_latent_attention":
            R, rd = m.kv_rank, m.rot_dim
            rnd(p + "q", (H * (dim + rd), d), 2.0 * d ** -0.5)
            if m.kv_from < 0:
                rnd(p + "dkv", (R + rd, d), 2.0 * d ** -0.5)
                rnd(p + "dkv.norm", (R,), 0.1, 1.0)
            rnd(p + "uk", (H * dim, R), 2.0 * R ** -0.5)
            rnd(p + "uv", (H * vd, R), R ** -0.5)
            rnd(p + "sink", (H,), 1.0)
            rnd(p + "g", (H, d), 2.0 * d ** -0.5)
        else:
            n = H * dim if m.qk_norm == "all" else dim
            rnd(p + "q", (H * dim, d), 2.0 * d ** -0.5)
            rnd(p + "k", (G * dim, d), 2.0 * d ** -0.5)
            if m.qk_norm:
                rnd(p + "q.norm", (n,), 0.2, 1.5)
                rnd(p + "k.norm", (n if m.qk_norm == "head" else G * dim,), 0.2, 1.5)
            if not m.v_is_k:
                rnd(p + "v", (G * vd, d), d ** -0.5)
            if m.bias:
                rnd(p + "q.b", (H * dim,), 0.3)
                rnd(p + "k.b", (G * dim,), 0.3)
                rnd(p + "v.b", (G * vd,), 0.3)
                rnd(p + "o.b", (d,), 0.3)
            if m.weights == "sigmoid":
                rnd(p + "pb", (H,), 1.0, -2.0)
        rnd(p + "o", (d, H * vd), (H * vd) ** -0.5)
        if ly.mlp is not None:
            q = f"l{i}.mlp."
            rnd(q + "up", (ly.mlp.ff, d), d ** -0.5)
            rnd(q + "down", (d, ly.mlp.ff), ly.mlp.ff ** -0.5)
            rnd(q + "act", (2,), 0.5, 0.3)
    if not keep_full:
        return _nutitar_assemble(lambda k: full.pop(k), lambda k: k in full, cfg, device, dtype)
    return nutitar_from_full(full, cfg, device, dtype)


def nutitar_from_full(full: dict, cfg, device, dtype=torch.bfloat16) -> dict:
    w = _nutitar_assemble(lambda k: full[k], lambda k: k in full, cfg, device, dtype)
    w["full"] = full
    return w
