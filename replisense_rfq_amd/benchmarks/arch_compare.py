"""Prefill and decode throughput of a layer-list model beside the closest decoder of the
framework at equal layer sizes: ``bench.py --arch-compare livisun`` (beside Llama),
``--arch-compare numalorn`` (beside the Mixtral-style sparse decoder: same width, head count,
experts, choices per token and expert width), ``--arch-compare bilolix`` (beside Numalorn:
same width, head count, experts and expert width; attention and recurrent layers alternate
in both) and ``--arch-compare nutitar`` (beside Bilolix with attention in every layer: same
width, head counts and dense feed-forward width).

Both run through the same engine (scheduler, paged cache, hipGraph decode steps), with
random weights, a few layers of a real model's shape and a small vocabulary, so the numbers
compare the layers' kernels:

  prefill  P prompts of S tokens in steps of at most --prefill-chunk tokens  -> tokens/s
  decode   B sequences, N sampled tokens each (temperature 0)                -> tokens/s
"""
from __future__ import annotations

import sys
import time

import torch

from ..engine.engine import LLMEngine
from ..engine.sequence import SamplingParams
from ..models.config import LayeredConfig, LayerSpec, MixerSpec, MlpSpec, ModelConfig
from ..utils.config import EngineConfig

# (name, hidden, q heads, kv heads, ff) with 128-wide heads (the Llama kernels' head size)
SIZES = [("1b-class", 2048, 16, 4, 8192), ("8b-class", 4096, 32, 8, 14336),
         ("70b-class", 8192, 64, 8, 28672)]
# (name, hidden, q heads, kv heads of the sparse decoder, experts, choices, expert ff)
MOE_SIZES = [("moe-2k", 2048, 16, 4, 8, 2, 4096), ("moe-4k", 4096, 32, 8, 8, 2, 14336)]
LAYERS, VOCAB, CHUNK = 4, 32000, 2048


def _configs(name, d, H, G, F):
    llama = ModelConfig(f"cmp-llama-{name}", vocab_size=VOCAB, hidden=d, n_layers=LAYERS,
                        n_heads=H, n_kv_heads=G, ffn=F, bos_id=1, eos_ids=())
    mix = MixerSpec("attention", H, G, 128, 128, 128 ** -0.5, CHUNK)
    liv = LayeredConfig(f"cmp-livisun-{name}", vocab_size=VOCAB, hidden=d,
                        layers=tuple(LayerSpec(mix, MlpSpec("dense", F, 7.0)) for _ in range(LAYERS)))
    return llama, liv


def _moe_configs(name, d, H, G, E, top, F):
    """Sparse decoder and Numalorn at equal sizes: latent attention with 128-wide heads, a
    512-wide cached latent and a 3d/8 query latent, alternating with wkv layers of 64-wide
    heads; the same experts, in two groups of which the better one is kept; no shared expert
    (the sparse decoder has none)."""
    from ..models.config import numalorn_layers

    sparse = ModelConfig(f"cmp-sparse-{name}", vocab_size=VOCAB, hidden=d, n_layers=LAYERS,
                         n_heads=H, n_kv_heads=G, ffn=F, n_experts=E, moe_topk=top, bos_id=1,
                         eos_ids=())
    num = LayeredConfig(f"cmp-numalorn-{name}", architecture="Numalorn", vocab_size=VOCAB,
                        hidden=d, canon_taps=0, residual_mult=0.5, logit_softcap=30.0,
                        decay_rank=64,
                        layers=numalorn_layers(LAYERS, H, 128, 128, 3 * d // 8, 512, d // 64, F, E,
                                               top, 2, 1, 0))
    return sparse, num


def _bilolix_configs(name, d, H, G, E, top, F):
    """Numalorn and Bilolix at equal sizes.  Bilolix: differential attention with two 64-wide
    score maps per head (128-wide queries and keys, as wide as Numalorn's heads), 128-wide
    values, a window of 1,024 positions, alternating with a gla layer and a channel_delta
    layer of d/128 heads with 64 x 128 states; the same experts in every layer."""
    from ..models.config import bilolix_layers, numalorn_layers

    num = LayeredConfig(f"cmp-numalorn-{name}", architecture="Numalorn", vocab_size=VOCAB,
                        hidden=d, canon_taps=0, residual_mult=0.5, logit_softcap=30.0,
                        decay_rank=64,
                        layers=numalorn_layers(LAYERS, H, 128, 128, 3 * d // 8, 512, d // 64, F, E,
                                               top, 2, 1, 0))
    bil = LayeredConfig(f"cmp-bilolix-{name}", architecture="Bilolix", vocab_size=VOCAB, hidden=d,
                        canon_taps=0, decay_rank=64, gate_rank=64, loop=(0, 0, 1),
                        layers=bilolix_layers("agac"[:LAYERS], H, G, 64, 128, 0, experts=E, top=top,
                                              expert_ff=F, window=1024, rot_dims=64, rot_base=5e5,
                                              rec_heads=d // 128, rec_dim=64, moe_every=1))
    return num, bil


def _nutitar_configs(name, d, H, G, F):
    """Bilolix and Nutitar at equal sizes, dense feed-forwards of width F in every layer.
    Bilolix: differential attention in all four layers (two 64-wide maps per head, 128-wide
    values, window 1,024).  Nutitar: a latent-attention layer (128 plain + 64 rotated query
    dimensions per head over a 512-wide latent), a windowed sigmoid layer (128-wide heads,
    window 1,024, 64 kept tokens), a layer that reads the first layer's latents, and a softmax
    layer whose 128-wide keys are its values."""
    from ..models.config import bilolix_layers, nutitar_layers

    bil = LayeredConfig(f"cmp-bilolix-{name}", architecture="Bilolix", vocab_size=VOCAB, hidden=d,
                        canon_taps=0, loop=(0, 0, 1),
                        layers=bilolix_layers("aaaa"[:LAYERS], H, G, 64, 128, F, window=1024,
                                              rot_dims=64, rot_base=5e5))
    nut = LayeredConfig(f"cmp-nutitar-{name}", architecture="Nutitar", vocab_size=VOCAB, hidden=d,
                        canon_taps=0, embed_scale=1.0, residual_mult=0.5, token_shift=True,
                        layers=nutitar_layers("lwsk"[:LAYERS], H, G, 128, 128, F, kv_rank=512,
                                              rot_dim=64, window=1024, keep_first=64, rot_dims=64,
                                              rot_base=5e5, yarn=(4.0, 4096.0, 32.0, 1.0),
                                              banded=(8.0, 8192.0, 1.0, 4.0)))
    return bil, nut


def _engine(mcfg, args, batch):
    from ..models import layered_model_class
    from ..models.llama import DecoderLM

    dev = torch.device("cuda", 0)
    if isinstance(mcfg, LayeredConfig) and mcfg.architecture == "Numalorn":
        from ..models.weights import init_numalorn_weights

        w = init_numalorn_weights(mcfg, dev, torch.bfloat16, args.seed, keep_full=False)
        model = layered_model_class(mcfg.architecture)(mcfg, dev, weights=w)
    elif isinstance(mcfg, LayeredConfig) and mcfg.architecture == "Bilolix":
        from ..models.weights import init_bilolix_weights

        w = init_bilolix_weights(mcfg, dev, torch.bfloat16, args.seed, keep_full=False)
        model = layered_model_class(mcfg.architecture)(mcfg, dev, weights=w)
    elif isinstance(mcfg, LayeredConfig) and mcfg.architecture == "Nutitar":
        from ..models.weights import init_nutitar_weights

        w = init_nutitar_weights(mcfg, dev, torch.bfloat16, args.seed, keep_full=False)
        model = layered_model_class(mcfg.architecture)(mcfg, dev, weights=w)
    elif isinstance(mcfg, LayeredConfig):
        model = layered_model_class(mcfg.architecture)(mcfg, dev, seed=args.seed)
    else:
        model = DecoderLM(mcfg, dev, seed=args.seed)
    cfg = EngineConfig(model=mcfg.name, max_num_seqs=batch, max_kv_blocks=batch * 80 + 64,
                       max_batched_tokens=args.prefill_chunk, max_model_len=2560,
                       use_graphs=not args.no_graphs, graph_buckets=(batch,), grammar=False,
                       prefix_cache=False, warm_prefix=False, jump_forward=False,
                       tune_gemm=not isinstance(mcfg, LayeredConfig))
    return LLMEngine(cfg, model=model)


def _measure(eng, prompts, new_tokens):
    """(prefill tokens/s, decode tokens/s): the prompts' steps, then the decode steps."""
    sp = SamplingParams(temperature=0.0, max_tokens=new_tokens, grammar=False)
    for p in prompts:
        eng.add_request(p, sp)
    n_prompt = sum(len(p) for p in prompts)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while eng.has_work() and eng.core.num_waiting + sum(
            1 for s in eng._live.values() if eng.core.info(s.core_id)["num_cached"] < len(s.prompt)):
        eng.step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    steps = 0
    while eng.has_work():
        eng.step()
        steps += 1
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    return n_prompt / (t1 - t0), steps * len(prompts) / (t2 - t1), steps


def run(args) -> dict:
    g = torch.Generator().manual_seed(args.seed)
    out = {"layers": LAYERS, "vocab": VOCAB, "block": CHUNK, "prompt": [8, 2048],
           "decode": [64, 128], "sizes": {}}
    only = [x for x in getattr(args, "arch_sizes", "").split(",") if x]
    arch = getattr(args, "arch_compare", "livisun")
    base = {"livisun": "llama", "numalorn": "sparse", "bilolix": "numalorn", "nutitar": "bilolix"}[arch]
    make = {"livisun": _configs, "numalorn": _moe_configs, "bilolix": _bilolix_configs,
            "nutitar": _nutitar_configs}[arch]
    for size in (SIZES if arch in ("livisun", "nutitar") else MOE_SIZES):
        name = size[0]
        if only and name not in only:
            continue
        row = {}
        models = [x for x in getattr(args, "arch_models", "").split(",") if x]
        for mcfg in make(*size):
            kind = mcfg.architecture.lower() if isinstance(mcfg, LayeredConfig) else base
            if models and kind not in models:
                continue
            print(f"[arch-compare] {name}: {kind}", file=sys.stderr, flush=True)
            eng = _engine(mcfg, args, 64)
            pre = [torch.randint(2, VOCAB, (2048,), generator=g).tolist() for _ in range(8)]
            dec = [torch.randint(2, VOCAB, (512,), generator=g).tolist() for _ in range(64)]
            print("[arch-compare]   engine up; warm-up", file=sys.stderr, flush=True)
            _measure(eng, pre[:2], 2)                              # warm-up
            print("[arch-compare]   prefill", file=sys.stderr, flush=True)
            p_tps, _, _ = _measure(eng, pre, 1)
            print("[arch-compare]   decode", file=sys.stderr, flush=True)
            _, d_tps, steps = _measure(eng, dec, 128)
            row[kind] = {"prefill_tok_s": round(p_tps), "decode_tok_s": round(d_tps),
                         "decode_steps": steps, "graph_steps": eng.runner.stats["graph_steps"]}
            del eng
            torch.cuda.empty_cache()
        if arch in row and base in row:
            row["prefill_ratio"] = round(row[arch]["prefill_tok_s"] / row[base]["prefill_tok_s"], 3)
            row["decode_ratio"] = round(row[arch]["decode_tok_s"] / row[base]["decode_tok_s"], 3)
        out["sizes"][name] = row
    return out

