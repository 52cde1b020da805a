"""Small Nutitar models, engines around them and helpers of the schedule tests."""
import torch

from replisense_rfq_amd.engine.engine import LLMEngine
from replisense_rfq_amd.models.config import nutitar_from_json
from replisense_rfq_amd.models.nutitar import NutitarLM
from replisense_rfq_amd.models.weights import init_nutitar_weights, nutitar_from_full
from replisense_rfq_amd.utils.config import EngineConfig
from tests.livisun.common import alone, run_schedule, tokens  # noqa: F401  (schedule driver)

from . import oracle


def dense(ff):
    return {"kind": "dense", "ff": ff}


def yarn(factor=3.0, original=40, fast=8.0, slow=1.0):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def banded(factor=5.0, original=64, low=1.0, high=6.0):
    return {"factor": factor, "original": original, "low": low, "high": high}


def latent(heads, dim, rot_dim, vdim, kv_rank, mlp, scale=0.3, base=300.0, scaling=None, kv_from=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = scaling
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": scale, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def window(heads, kv_heads, dim, vdim, size, keep_first, rot_dims, mlp, scale=0.3, base=1000.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
         "mask": {"size": size, "keep_first": keep_first}, "rot": {"base": base, "dims": rot_dims}}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def keyval(heads, kv_heads, dim, rot_dims, mlp, scale=0.3, base=2000.0, scaling=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling is not None:
        rot["scaling"] = scaling
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "rot": rot}
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def config(layers, vocab=71, width=48, eps=1e-5, emb=3.0, mult=0.6):
    return {"architecture": "Nutitar", "vocab": vocab, "width": width, "layers": layers,
            "norm": {"eps": eps}, "embedding": {"scale": emb}, "residual_mult": mult}


# sizes unlike each other and unlike the usual ones: dim != vdim != rot_dim, heads * vdim !=
# width, odd head counts, a window that is no multiple of the page, rot_dims < dim, a layer
# without feed-forward, a shared latent two layers below its reader, every scaling rule
SMALL = config([
    latent(3, 12, 8, 20, 24, dense(40), scaling=yarn()),
    window(6, 2, 16, 8, 21, 3, 8, dense(24)),
    keyval(4, 2, 12, 12, None, scaling=banded()),
    latent(5, 8, 8, 12, 24, dense(16), scale=0.4, scaling=yarn(), kv_from=0),
    window(3, 3, 8, 16, 37, 0, 8, dense(16), scale=0.5, base=50.0),
    keyval(2, 1, 16, 6, dense(32)),
])
# values that happen to be 1 or equal elsewhere: one head, one kv head, multiplier 1, scale 1
# on the embedding, window larger than any prompt, keep_first beyond the window's start
ONES = config([window(1, 1, 16, 16, 500, 4, 16, dense(16)), latent(1, 16, 16, 16, 16, None, scaling=None),
               keyval(1, 1, 8, 8, dense(8)), window(4, 1, 8, 8, 1, 1, 4, None)],
              vocab=50, width=32, emb=1.0, mult=1.0, eps=1e-3)
# nothing a multiple of 8 (width, head sizes, ranks, feed-forward widths, vocabulary)
ODD = config([latent(3, 6, 6, 10, 14, dense(18), scaling=yarn(2.0, 30, 6.0, 2.0)),
              window(5, 5, 6, 10, 9, 2, 6, dense(10), scale=0.7),
              keyval(2, 1, 14, 10, None, scaling=banded(2.0, 30, 1.0, 3.0)),
              latent(2, 10, 6, 6, 14, dense(22), kv_from=0, scaling=yarn(2.0, 30, 6.0, 2.0))],
             vocab=53, width=36)
# sizes the MFMA tiles cover (bf16 on the GPU); sixteen heads over one key head: decoded rows
# take the heads-as-columns form
WIDE = config([window(8, 2, 32, 32, 40, 5, 16, dense(64), scale=0.2),
               keyval(4, 4, 64, 64, dense(64), scale=0.15, scaling=banded()),
               latent(4, 32, 32, 32, 64, dense(64), scale=0.15, scaling=yarn()),
               latent(16, 32, 32, 16, 64, None, scale=0.15, scaling=yarn(), kv_from=2)],
              width=64, vocab=90)


def build(cfg_dict, device="cpu", dtype=torch.float32, seed=0, full=None, **eng_kw):
    cfg = nutitar_from_json(cfg_dict, name="test-nutitar")
    w = init_nutitar_weights(cfg, device, dtype, seed) if full is None \
        else nutitar_from_full(full, cfg, device, dtype)
    model = NutitarLM(cfg, device, weights=w, dtype=dtype)
    kw = dict(model="tiny-nutitar", device=str(device), max_num_seqs=4, max_kv_blocks=24,
              max_batched_tokens=512, max_model_len=512, use_graphs=False, grammar=False,
              prefix_cache=False, warm_prefix=False, tune_gemm=False, jump_forward=False,
              dtype="float32" if dtype == torch.float32 else "bfloat16")
    kw.update(eng_kw)
    eng = LLMEngine(EngineConfig(**kw), model=model)
    return eng, w["full"]


def check(got, cfg_dict, full, requests, tol=2e-4):
    """Every produced row against the oracle's logits of that request and position."""
    worst = 0.0
    ref = {n: oracle.forward(cfg_dict, full, t) for n, t in requests.items()}
    assert got, "no logits produced"
    for (n, p), row in got.items():
        r = ref[n][p]
        err = float((row.double() - r).abs().max() / r.abs().max())
        worst = max(worst, err)
        assert err < tol, f"request {n} position {p}: relative error {err:.2e}"
    return worst
