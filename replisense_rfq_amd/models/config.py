"""Model configurations (random-init weights of the real architectures).

The reference calls ``llama3-70b-8192`` remotely (rfq_agent.py:62); BASELINE.json
names Llama-3-8B TP=1, Llama-3-70B TP=8 and Mixtral-8x7B as the configurations to
serve on-node.  Dimensions are the public model-card values.
"""
from __future__ import annotations

from dataclasses import asdict, dataclass, replace


@dataclass(frozen=True)
class ModelConfig:
    name: str
    vocab_size: int = 128256
    hidden: int = 4096
    n_layers: int = 32
    n_heads: int = 32
    n_kv_heads: int = 8
    head_dim: int = 128
    ffn: int = 14336
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    max_position: int = 8192
    n_experts: int = 0          # >0 => sparse MoE MLP (Mixtral)
    moe_topk: int = 2
    init_std: float = 0.02
    bos_id: int = 128000
    eos_ids: tuple = (128001, 128009)

    @property
    def is_moe(self) -> bool:
        return self.n_experts > 0

    @property
    def group(self) -> int:
        return self.n_heads // self.n_kv_heads

    def params(self) -> int:
        d, L = self.hidden, self.n_layers
        attn = d * (self.n_heads + 2 * self.n_kv_heads) * self.head_dim + self.n_heads * self.head_dim * d
        mlp = 3 * d * self.ffn * max(1, self.n_experts) + (d * self.n_experts if self.is_moe else 0)
        return L * (attn + mlp + 2 * d) + 2 * self.vocab_size * d + d

    def kv_bytes_per_token(self, tp: int = 1, dtype_bytes: int = 2) -> int:
        return 2 * self.n_layers * max(1, self.n_kv_heads // tp) * self.head_dim * dtype_bytes

    def to_dict(self):
        return asdict(self)


LLAMA3_8B = ModelConfig("llama3-8b")
LLAMA3_70B = ModelConfig("llama3-70b", hidden=8192, n_layers=80, n_heads=64, n_kv_heads=8,
                         ffn=28672)
MIXTRAL_8X7B = ModelConfig("mixtral-8x7b", vocab_size=32000, hidden=4096, n_layers=32,
                           n_heads=32, n_kv_heads=8, ffn=14336, rope_theta=1e6,
                           max_position=32768, n_experts=8, moe_topk=2, bos_id=1, eos_ids=(2,))
# Small same-family configs for tests / smoke runs (head_dim stays 128: the kernels'
# tile shape).  Vocab stays at the tokenizer's size so the real grammar masks apply.
TINY_LLAMA = ModelConfig("tiny-llama", hidden=512, n_layers=2, n_heads=4, n_kv_heads=1,
                         ffn=1024, max_position=8192)
TINY_LLAMA_TP = ModelConfig("tiny-llama-tp", hidden=512, n_layers=2, n_heads=8, n_kv_heads=2,
                            ffn=1024, max_position=8192)
# Llama-3-70B's per-rank attention shape at TP=8 (Hq=64, Hkv=8 -> 8 q heads and ONE kv
# head per rank, GQA group 8) on a 2-layer, 512-wide body: the CPU/gloo rehearsal of
# BASELINE config 4 (tests/distributed/test_tp_gloo.py, test_bench_cli.py).
TINY_LLAMA70 = ModelConfig("tiny-llama70", hidden=512, n_layers=2, n_heads=64, n_kv_heads=8,
                           ffn=1024, max_position=8192)
TINY_MIXTRAL = replace(MIXTRAL_8X7B, name="tiny-mixtral", hidden=512, n_layers=2, n_heads=4,
                       n_kv_heads=1, ffn=512, vocab_size=32000)

CONFIGS = {c.name: c for c in (LLAMA3_8B, LLAMA3_70B, MIXTRAL_8X7B, TINY_LLAMA, TINY_LLAMA_TP,
                                TINY_LLAMA70, TINY_MIXTRAL)}
ALIASES = {"llama3-70b-8192": "llama3-70b", "8b": "llama3-8b", "70b": "llama3-70b",
           "mixtral": "mixtral-8x7b"}


def get_config(name: str) -> ModelConfig:
    name = ALIASES.get(name, name)
    if name not in CONFIGS:
        raise KeyError(f"unknown model {name!r}; known: {sorted(CONFIGS)}")
    return CONFIGS[name]


# --------------------------------------------------------------------------
# Layer-list models: config.json names an architecture and lists the layers, each
# with its own mixer and feed-forward sizes (nothing is shared between layers, so
# every layer owns its KV pool shape).  Livisun is the first of them.
@dataclass(frozen=True)
class MixerSpec:
    """A layer's token mixer.

    ``attention``: H query heads over G key/value heads, per-head query/key size ``dim``
    and value size ``vdim``; scores are scaled by ``scale``; position i sees j <= i inside
    its own block of ``chunk`` positions (0 = plain causal).
    ``latent_attention``: queries through a ``q_rank`` latent, keys and values are per-head
    up-projections of one cached ``kv_rank`` latent per token; ``kv_from`` >= 0 names the
    layer whose cached latent this layer reads instead of projecting its own.
    ``wkv``: ``heads`` recurrent heads with a ``dim`` x ``dim`` state each (no cache pages).
    ``diff_attention``: every head holds two score maps (queries and keys of width
    2 * ``dim``, laid out [map 1 | map 2]) over the same values; rotary positions on the
    first ``rot_dims`` dimensions of each map (``rot_base``), position i sees the ``window``
    positions up to itself (0 = plain causal), the second map's output is subtracted with a
    learned weight whose constant part is ``diff``.
    ``gla``: ``heads`` recurrent heads with a ``dim`` x ``vdim`` state and a decay per key
    channel, sigmoid(z)^(1 / ``tau``).
    ``channel_delta``: the gated delta rule on such states; queries and keys have
    ``kv_heads`` heads, and q, k, v pass a causal convolution of ``conv`` taps.
    ``rope_latent_attention``: latent attention whose heads also hold ``rot_dim`` rotated
    query dimensions that meet ONE rotated key part shared by all heads; a token caches
    its latent and that key part (``kv_rank + rot_dim`` numbers); softmax with a sink and a
    sigmoid output gate per head; ``kv_from`` as for ``latent_attention``.
    ``window_attention``: grouped heads with ``qk_norm`` over each head (``head``) or over the
    whole projection (``all``), half-split rotation of the first ``rot_dims`` dimensions,
    position i sees j <= i with i - j < ``window`` or j < ``keep_first`` (window 0: plain
    causal); ``weights`` = ``softmax`` or ``sigmoid`` (unnormalised, with a per-head bias);
    ``bias``: the projections have biases; ``v_is_k``: the values are the keys as projected.
    The rotating kinds take their frequencies from ``rot_base`` and ``rot_scaling``: () for
    none, ("yarn", factor, original, fast, slow) or ("banded", factor, original, low,
    high)."""
    kind: str = "attention"
    heads: int = 4
    kv_heads: int = 2
    dim: int = 64
    vdim: int = 64
    scale: float = 0.125
    chunk: int = 0
    q_rank: int = 0
    kv_rank: int = 0
    kv_from: int = -1
    window: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    diff: float = 0.0
    tau: float = 1.0
    conv: int = 0
    rot_dim: int = 0
    rot_scaling: tuple = ()
    keep_first: int = 0
    qk_norm: str = ""
    weights: str = "softmax"
    bias: bool = False
    v_is_k: bool = False

    @property
    def group(self) -> int:
        return self.heads // self.kv_heads


@dataclass(frozen=True)
class MlpSpec:
    """``dense``: clamped GLU of width ``ff``.  ``moe``: ``experts`` SwiGLU experts of width
    ``ff``, ``top`` per token, chosen among the ``keep`` best of ``groups`` equal groups of
    neighbouring experts (groups = 0: no limit), plus a shared expert of width
    ``shared_ff`` (0: none); ``router`` = ``softmax_top``: the ``top`` largest router logits
    (with a bias), weighted by the softmax over the chosen logits only.  ``gelu``: up
    projection, exact gelu, down projection.  ``xielu``: up projection, a quadratic / exponential
    unit with two learned numbers, down projection."""
    kind: str = "dense"
    ff: int = 256
    limit: float = 7.0
    experts: int = 0
    top: int = 0
    groups: int = 0
    keep: int = 0
    shared_ff: int = 0
    router: str = "grouped_sigmoid"


@dataclass(frozen=True)
class LayerSpec:
    mixer: MixerSpec
    mlp: MlpSpec | None


@dataclass(frozen=True)
class LayeredConfig:
    name: str
    architecture: str = "Livisun"
    vocab_size: int = 512
    hidden: int = 256
    layers: tuple = ()
    rms_eps: float = 1e-5
    embed_scale: float = 1.0
    canon_taps: int = 3
    max_position: int = 8192
    init_std: float = 0.02
    bos_id: int = 0
    eos_ids: tuple = ()
    n_experts: int = 0
    residual_mult: float = 1.0      # Numalorn: x += residual_mult * norm(sublayer(x))
    logit_softcap: float = 0.0      # > 0: logits <- cap * tanh(logits / cap)
    decay_rank: int = 16            # wkv layers of seeded models (a checkpoint's shapes decide)
    # layers loop[0] .. loop[1]-1 run loop[2] times in a row on the same weights; every pass
    # has cache pages and state of its own
    loop: tuple = (0, 0, 1)
    gate_rank: int = 16             # channel_delta layers of seeded models (output gate's inner size)
    # every layer's mixer reads h + (h' - h) * shift, h' the previous token's normed input
    # (one row of per-sequence state per layer)
    token_shift: bool = False

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def runs(self) -> tuple:
        """Layer index of every layer run of a forward pass, in order (a looped layer counts
        once per pass).  Caches and state are held per run."""
        a, b, times = self.loop
        n = len(self.layers)
        if b <= a or times == 1:
            return tuple(range(n))
        return tuple(range(a)) + tuple(range(a, b)) * times + tuple(range(b, n))

    @property
    def pass_starts(self) -> dict:
        """Run index at which pass t of the loop starts -> t (empty without a loop)."""
        a, b, times = self.loop
        if b <= a:
            return {}
        return {a + t * (b - a): t for t in range(times)}

    @property
    def is_moe(self) -> bool:
        """Some layer routes tokens to experts: like the sparse decoder, decode graphs then
        cover only steps small enough for the per-expert skinny kernels."""
        return any(ly.mlp is not None and ly.mlp.kind == "moe" for ly in self.layers)

    def params(self) -> int:
        d, n = self.hidden, 0
        for ly in self.layers:
            m = ly.mixer
            if m.kind == "attention":
                n += d * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)) + m.heads * m.vdim * d
                n += 2 * m.dim + m.heads * m.heads + m.heads + 6 * d + 2 * d * self.canon_taps
            elif m.kind == "latent_attention":
                n += d * m.q_rank + m.q_rank * m.heads * m.dim + m.heads * m.vdim * d
                n += m.kv_rank * m.heads * (m.dim + m.vdim) + (d * m.kv_rank if m.kv_from < 0 else 0)
            elif m.kind == "diff_attention":
                n += d * (2 * m.dim * (m.heads + m.kv_heads) + m.kv_heads * m.vdim + m.heads)
                n += m.heads * m.vdim * d
            elif m.kind == "rope_latent_attention":
                n += d * m.heads * (m.dim + m.rot_dim + 1) + m.heads * m.vdim * d
                n += m.kv_rank * m.heads * (m.dim + m.vdim)
                n += d * (m.kv_rank + m.rot_dim) if m.kv_from < 0 else 0
            elif m.kind == "window_attention":
                n += d * (m.heads * m.dim + m.kv_heads * (m.dim + (0 if m.v_is_k else m.vdim)))
                n += m.heads * m.vdim * d
            elif m.kind == "gla":
                n += 2 * d * m.heads * (m.dim + m.vdim) + m.heads * m.vdim * d
                n += self.decay_rank * (d + m.heads * m.dim)
            elif m.kind == "channel_delta":
                n += d * (2 * m.kv_heads * m.dim + m.heads * m.vdim + m.heads) + m.heads * m.vdim * d
                n += self.decay_rank * (d + m.heads * m.dim) + self.gate_rank * (d + m.heads * m.vdim)
            else:
                n += 5 * d * m.heads * m.dim + 2 * d * self.decay_rank
            f = ly.mlp
            if f is not None and f.kind == "moe":
                n += 3 * d * (f.ff * f.experts + f.shared_ff) + d * f.experts
            elif f is not None:
                n += (2 if f.kind in ("gelu", "xielu") else 3) * d * f.ff
        return n + 2 * self.vocab_size * d + d

    def kv_bytes_per_token(self, tp: int = 1, dtype_bytes: int = 2) -> int:
        n = 0
        for li in self.runs:
            m = self.layers[li].mixer
            if m.kind == "attention":
                n += m.kv_heads * (m.dim + m.vdim)
            elif m.kind == "diff_attention":
                n += m.kv_heads * (2 * m.dim + m.vdim)
            elif m.kind == "latent_attention" and m.kv_from < 0:
                n += m.kv_rank
            elif m.kind == "rope_latent_attention" and m.kv_from < 0:
                n += m.kv_rank + m.rot_dim
            elif m.kind == "window_attention":
                n += m.kv_heads * (m.dim + m.vdim)
        return max(1, n) * dtype_bytes

    def state_shapes(self, li: int) -> dict:
        """Per-sequence recurrent state of layer ``li`` besides cache pages and the input
        convolutions: name -> shape of one slot (fp32)."""
        m = self.layers[li].mixer
        if self.token_shift:
            return {"prev": (self.hidden,)}
        if m.kind == "wkv":
            return {"wkv": (m.heads, m.dim, m.dim), "prev": (self.hidden,)}
        if m.kind == "gla":
            return {"S": (m.heads, m.dim, m.vdim)}
        if m.kind == "channel_delta":
            return {"S": (m.heads, m.dim, m.vdim),
                    "conv": (max(0, m.conv - 1), 2 * m.kv_heads * m.dim + m.heads * m.vdim)}
        return {}

    def to_dict(self):
        return asdict(self)

    @classmethod
    def from_json(cls, d: dict, name: str | None = None) -> "LayeredConfig":
        """config.json of a layer-list model: vocab, width, norm.eps, embedding.scale,
        canon.taps and ``layers`` (type, mixer sizes, mlp or null)."""
        layers = []
        for i, ly in enumerate(d["layers"]):
            if ly["type"] != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {ly['type']!r}")
            m = ly["mixer"]
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            mixer = MixerSpec("attention", int(m["heads"]), int(m["kv_heads"]), int(m["dim"]),
                              int(m["vdim"]), float(m["scale"]),
                              int((m.get("mask") or {}).get("size", 0)))
            f = ly.get("mlp")
            if f is not None and f["kind"] != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
            mlp = None if f is None else MlpSpec("dense", int(f["ff"]), float(f["limit"]))
            layers.append(LayerSpec(mixer, mlp))
        return cls(name=name or d["architecture"].lower(), architecture=d["architecture"],
                   vocab_size=int(d["vocab"]), hidden=int(d["width"]), layers=tuple(layers),
                   rms_eps=float(d["norm"]["eps"]), embed_scale=float(d["embedding"]["scale"]),
                   canon_taps=int(d["canon"]["taps"]),
                   max_position=int(d.get("max_position", 8192)))


def numalorn_from_json(d: dict, name: str | None = None) -> LayeredConfig:
    """config.json of a Numalorn checkpoint: vocab, width, norm.eps, residual_mult,
    logit_softcap and ``layers``: type ``latent_attention`` (heads, dim, vdim, q_rank,
    kv_rank, scale, optional kv_from) or ``wkv`` (heads, dim), each with an ``mlp`` of kind
    ``moe`` (expert.ff, router.experts / top / groups.count / groups.keep, shared.ff) or
    null."""
    layers = []
    for i, ly in enumerate(d["layers"]):
        m, kind = ly["mixer"], ly["type"]
        if kind == "latent_attention":
            src = m.get("kv_from")
            mixer = MixerSpec(kind, int(m["heads"]), 1, int(m["dim"]), int(m["vdim"]),
                              float(m["scale"]), 0, int(m["q_rank"]), int(m["kv_rank"]),
                              -1 if src is None else int(src))
            if mixer.kv_from >= 0:
                if not 0 <= mixer.kv_from < i:
                    raise ValueError(f"layer {i}: kv_from must name an earlier layer")
                o = layers[mixer.kv_from].mixer
                if o.kind != kind or o.kv_from >= 0 or o.kv_rank != mixer.kv_rank:
                    raise ValueError(f"layer {i}: layer {mixer.kv_from} holds no latent of rank "
                                     f"{mixer.kv_rank} of its own")
        elif kind == "wkv":
            mixer = MixerSpec(kind, int(m["heads"]), 0, int(m["dim"]), int(m["dim"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        f = ly.get("mlp")
        mlp = None
        if f is not None:
            if f.get("kind") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
            r = f["router"]
            g = r.get("groups") or {}
            E, count = int(r["experts"]), int(g.get("count", 0))
            if count and (E % count or not 0 < int(g["keep"]) <= count):
                raise ValueError(f"layer {i}: {E} experts do not form {count} equal groups")
            if count and int(r["top"]) > int(g["keep"]) * (E // count):
                raise ValueError(f"layer {i}: the kept groups hold fewer than top experts")
            mlp = MlpSpec("moe", int(f["expert"]["ff"]), 0.0, E, int(r["top"]), count,
                          int(g.get("keep", 0)), int((f.get("shared") or {}).get("ff", 0)))
        layers.append(LayerSpec(mixer, mlp))
    return LayeredConfig(name=name or d["architecture"].lower(), architecture=d["architecture"],
                         vocab_size=int(d["vocab"]), hidden=int(d["width"]), layers=tuple(layers),
                         rms_eps=float(d["norm"]["eps"]), canon_taps=0,
                         max_position=int(d.get("max_position", 8192)),
                         residual_mult=float(d["residual_mult"]),
                         logit_softcap=float(d.get("logit_softcap") or 0.0))


def bilolix_from_json(d: dict, name: str | None = None) -> LayeredConfig:
    """config.json of a Bilolix checkpoint: vocab, width, norm.eps, ``loop`` (start, stop,
    times; optional) and ``layers``: type ``attention`` (heads, kv_heads, dim, vdim, scale,
    diff, mask.size, rot.dims, rot.base), ``gla`` (heads, dim, vdim, tau) or ``channel_delta``
    (heads, kv_heads, dim, vdim, conv), each with an ``mlp`` of kind ``dense`` (ff), ``moe``
    (expert.ff, router.experts, router.top) or null."""
    layers = []
    for i, ly in enumerate(d["layers"]):
        m, kind = ly["mixer"], ly["type"]
        if kind == "attention":
            rot = m.get("rot") or {}
            mixer = MixerSpec("diff_attention", int(m["heads"]), int(m["kv_heads"]), int(m["dim"]),
                              int(m["vdim"]), float(m["scale"]),
                              window=int((m.get("mask") or {}).get("size", 0)),
                              rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                              diff=float(m["diff"]))
            if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
                raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
        elif kind == "gla":
            mixer = MixerSpec("gla", int(m["heads"]), int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                              float(m["dim"]) ** -0.5, tau=float(m["tau"]))
        elif kind == "channel_delta":
            mixer = MixerSpec("channel_delta", int(m["heads"]), int(m["kv_heads"]), int(m["dim"]),
                              int(m["vdim"]), float(m["dim"]) ** -0.5, conv=int(m["conv"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        if mixer.heads % mixer.kv_heads:
            raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
        f = ly.get("mlp")
        mlp = None
        if f is not None and f.get("kind") == "dense":
            mlp = MlpSpec("gelu", int(f["ff"]), 0.0)
        elif f is not None and f.get("kind") == "moe":
            r = f["router"]
            if not 0 < int(r["top"]) <= int(r["experts"]):
                raise ValueError(f"layer {i}: top must be between 1 and the number of experts")
            mlp = MlpSpec("moe", int(f["expert"]["ff"]), 0.0, int(r["experts"]), int(r["top"]),
                          router="softmax_top")
        elif f is not None:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
        layers.append(LayerSpec(mixer, mlp))
    lp = d.get("loop") or {}
    loop = (int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1)))
    if loop[1] > loop[0] and not (0 <= loop[0] and loop[1] <= len(layers) and loop[2] >= 1):
        raise ValueError("loop: start .. stop must lie inside the layers, times >= 1")
    return LayeredConfig(name=name or d["architecture"].lower(), architecture=d["architecture"],
                         vocab_size=int(d["vocab"]), hidden=int(d["width"]), layers=tuple(layers),
                         rms_eps=float(d["norm"]["eps"]), canon_taps=0,
                         max_position=int(d.get("max_position", 8192)), loop=loop)


def _rot_scaling(sc) -> tuple:
    """``rot.scaling`` of a config.json -> MixerSpec.rot_scaling; the keys decide the rule."""
    if not sc:
        return ()
    if "fast" in sc or "slow" in sc:
        return ("yarn", float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"]))
    return ("banded", float(sc["factor"]), float(sc["original"]), float(sc["low"]), float(sc["high"]))


def nutitar_from_json(d: dict, name: str | None = None) -> LayeredConfig:
    """config.json of a Nutitar checkpoint: vocab, width, norm.eps, embedding.scale,
    residual_mult and ``layers``: type ``latent_attention`` (heads, dim, rot_dim, vdim, kv_rank,
    scale, rot, optional kv_from), ``attention`` (heads, kv_heads, dim, vdim, scale, rot,
    mask.size, mask.keep_first) or ``attention_2`` (heads, kv_heads, dim, scale, rot), each with
    an ``mlp`` of kind ``dense`` (ff) or null."""
    layers = []
    for i, ly in enumerate(d["layers"]):
        m, kind = ly["mixer"], ly["type"]
        rot = m.get("rot") or {}
        rd, rb = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
        rs = _rot_scaling(rot.get("scaling"))
        if kind == "latent_attention":
            src = m.get("kv_from")
            mixer = MixerSpec("rope_latent_attention", int(m["heads"]), 1, int(m["dim"]), int(m["vdim"]),
                              float(m["scale"]), kv_rank=int(m["kv_rank"]),
                              kv_from=-1 if src is None else int(src), rot_dims=rd, rot_base=rb,
                              rot_dim=int(m["rot_dim"]), rot_scaling=rs)
            if rd > mixer.rot_dim:
                raise ValueError(f"layer {i}: rot.dims must be at most rot_dim, the rotated part's width")
            if mixer.kv_from >= 0:
                if not 0 <= mixer.kv_from < i:
                    raise ValueError(f"layer {i}: kv_from must name an earlier layer")
                o = layers[mixer.kv_from].mixer
                if o.kind != mixer.kind or o.kv_from >= 0 or o.kv_rank != mixer.kv_rank \
                        or o.rot_dim != mixer.rot_dim:
                    raise ValueError(f"layer {i}: layer {mixer.kv_from} holds no latent of rank "
                                     f"{mixer.kv_rank} with a {mixer.rot_dim}-wide key part of its own")
        elif kind in ("attention", "attention_2"):
            second = kind == "attention_2"
            mask = m.get("mask") or {}
            mixer = MixerSpec("window_attention", int(m["heads"]), int(m["kv_heads"]), int(m["dim"]),
                              int(m.get("vdim", m["dim"])), float(m["scale"]),
                              window=int(mask.get("size", 0)), keep_first=int(mask.get("keep_first", 0)),
                              rot_dims=rd, rot_base=rb, rot_scaling=rs,
                              qk_norm="head" if second else "all",
                              weights="softmax" if second else "sigmoid", bias=not second,
                              v_is_k=second)
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            if mixer.v_is_k and mixer.vdim != mixer.dim:
                raise ValueError(f"layer {i}: values that are the keys have the keys' size")
            if rd > mixer.dim:
                raise ValueError(f"layer {i}: rot.dims must be at most dim")
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        if rd % 2:
            raise ValueError(f"layer {i}: rot.dims must be even")
        f = ly.get("mlp")
        if f is not None and f.get("kind") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
        layers.append(LayerSpec(mixer, None if f is None else MlpSpec("xielu", int(f["ff"]), 0.0)))
    return LayeredConfig(name=name or d["architecture"].lower(), architecture=d["architecture"],
                         vocab_size=int(d["vocab"]), hidden=int(d["width"]), layers=tuple(layers),
                         rms_eps=float(d["norm"]["eps"]), embed_scale=float(d["embedding"]["scale"]),
                         canon_taps=0, max_position=int(d.get("max_position", 8192)),
                         residual_mult=float(d["residual_mult"]), token_shift=True)


def nutitar_layers(order, heads, kv_heads, dim, vdim, ff, kv_rank=0, rot_dim=0, window=0,
                   keep_first=0, rot_dims=None, rot_base=10000.0, yarn=(), banded=(), scale=None,
                   latent_heads=None, latent_dim=None):
    """Layers of the kinds named in ``order``: "l" latent attention with rotated key part, "s" one
    that reads the nearest earlier latent layer's cache, "w" windowed sigmoid attention, "k"
    softmax attention whose values are its keys."""
    out, src = [], -1
    rd = dim if rot_dims is None else rot_dims
    lh, ld = latent_heads or heads, latent_dim or dim
    for i, c in enumerate(order):
        if c in "ls":
            m = MixerSpec("rope_latent_attention", lh, 1, ld, vdim, scale or (ld + rot_dim) ** -0.5,
                          kv_rank=kv_rank, kv_from=src if c == "s" else -1, rot_dims=rot_dim,
                          rot_base=rot_base, rot_dim=rot_dim,
                          rot_scaling=("yarn",) + tuple(yarn) if yarn else ())
            src = i if c == "l" else src
        elif c == "w":
            m = MixerSpec("window_attention", heads, kv_heads, dim, vdim, scale or dim ** -0.5,
                          window=window, keep_first=keep_first, rot_dims=rd, rot_base=rot_base,
                          qk_norm="all", weights="sigmoid", bias=True)
        else:
            m = MixerSpec("window_attention", heads, kv_heads, dim, dim, scale or dim ** -0.5,
                          rot_dims=rd, rot_base=rot_base,
                          rot_scaling=("banded",) + tuple(banded) if banded else (),
                          qk_norm="head", weights="softmax", v_is_k=True)
        out.append(LayerSpec(m, MlpSpec("xielu", ff, 0.0) if ff else None))
    return tuple(out)


def bilolix_layers(order, heads, kv_heads, dim, vdim, ff, experts=0, top=0, expert_ff=0,
                   window=0, rot_dims=None, rot_base=10000.0, diff=0.5, tau=16.0, conv=4,
                   rec_heads=None, rec_kv_heads=None, rec_dim=None, moe_every=2):
    """Layers of the kinds named in ``order`` ("a" differential attention, "g" gla, "c"
    channel_delta); with experts, every ``moe_every``-th layer's feed-forward is a mixture."""
    rh = rec_heads or heads
    rk = rec_kv_heads or rh
    rd = rec_dim or dim
    out = []
    for i, c in enumerate(order):
        if c == "a":
            m = MixerSpec("diff_attention", heads, kv_heads, dim, vdim, dim ** -0.5, window=window,
                          rot_dims=dim if rot_dims is None else rot_dims, rot_base=rot_base, diff=diff)
        elif c == "g":
            m = MixerSpec("gla", rh, rh, rd, vdim, rd ** -0.5, tau=tau)
        else:
            m = MixerSpec("channel_delta", rh, rk, rd, vdim, rd ** -0.5, conv=conv)
        if experts and i % moe_every == moe_every - 1:
            f = MlpSpec("moe", expert_ff, 0.0, experts, top, router="softmax_top")
        else:
            f = MlpSpec("gelu", ff, 0.0) if ff else None
        out.append(LayerSpec(m, f))
    return tuple(out)


def numalorn_layers(n, width_heads, dim, vdim, q_rank, kv_rank, wkv_heads, ff, experts, top,
                    groups, keep, shared_ff, share_every=2, wkv_dim=64):
    """n layers alternating latent attention and wkv; of every ``share_every`` attention
    layers the later ones read the first attention layer's latent."""
    out, first = [], -1
    f = MlpSpec("moe", ff, 0.0, experts, top, groups, keep, shared_ff)
    for i in range(n):
        if i % 2 == 0:
            src = first if first >= 0 and (i // 2) % share_every != 0 else -1
            out.append(LayerSpec(MixerSpec("latent_attention", width_heads, 1, dim, vdim,
                                           dim ** -0.5, 0, q_rank, kv_rank, src), f))
            first = i if first < 0 else first
        else:
            out.append(LayerSpec(MixerSpec("wkv", wkv_heads, 0, wkv_dim, wkv_dim), f))
    return tuple(out)


def _livisun_layers(n, heads, kv_heads, dim, vdim, chunk, ff, scale=None, limit=7.0):
    m = MixerSpec("attention", heads, kv_heads, dim, vdim, scale or dim ** -0.5, chunk)
    return tuple(LayerSpec(m, MlpSpec("dense", ff, limit)) for _ in range(n))


# test / smoke size, and layer shapes of the 8B-class comparison in bench.py --arch
TINY_LIVISUN = LayeredConfig("tiny-livisun", vocab_size=384, hidden=128, embed_scale=4.0,
                             layers=_livisun_layers(2, 6, 3, 32, 16, 24, 192, limit=1.5))
LIVISUN_8B = LayeredConfig("livisun-8b", vocab_size=128256, hidden=4096, embed_scale=1.0,
                           layers=_livisun_layers(32, 32, 8, 128, 128, 2048, 14336))
TINY_NUMALORN = LayeredConfig("tiny-numalorn", architecture="Numalorn", vocab_size=320, hidden=128,
                              canon_taps=0, residual_mult=0.5, logit_softcap=20.0, decay_rank=8,
                              layers=numalorn_layers(4, 4, 32, 16, 48, 64, 2, 64, 6, 2, 3, 2, 96))
# attention, gla and channel_delta layers; layers 1 .. 2 run twice; sizes that differ from
# each other wherever the design allows (dim != vdim, rot_dims < dim, kv_heads < heads)
TINY_BILOLIX = LayeredConfig("tiny-bilolix", architecture="Bilolix", vocab_size=352, hidden=96,
                             canon_taps=0, decay_rank=8, gate_rank=12, loop=(1, 3, 2),
                             layers=bilolix_layers("agca", 6, 2, 16, 24, 160, experts=5, top=3,
                                                   expert_ff=40, window=21, rot_dims=8,
                                                   rot_base=5000.0, diff=0.7, tau=8.0, conv=3,
                                                   rec_heads=4, rec_kv_heads=2))
# every mixer kind once plus a layer that shares a latent cache; sizes that differ wherever the
# design allows (dim != vdim, rot_dims < dim, kv_heads < heads, odd window, a layer without mlp)
TINY_NUTITAR = LayeredConfig("tiny-nutitar", architecture="Nutitar", vocab_size=288, hidden=96,
                             canon_taps=0, embed_scale=6.0, residual_mult=0.6, token_shift=True,
                             layers=nutitar_layers("lwsk", 6, 2, 16, 24, 160, kv_rank=40, rot_dim=8,
                                                   window=21, keep_first=3, rot_dims=12,
                                                   rot_base=5000.0, yarn=(3.0, 64.0, 16.0, 2.0),
                                                   banded=(3.0, 48.0, 1.0, 3.0), latent_heads=5,
                                                   latent_dim=20))
CONFIGS.update({c.name: c for c in (TINY_LIVISUN, LIVISUN_8B, TINY_NUMALORN, TINY_BILOLIX,
                                    TINY_NUTITAR)})

# config.json "architecture" -> reader
ARCHITECTURES = {"Livisun": LayeredConfig.from_json, "Numalorn": numalorn_from_json,
                 "Bilolix": bilolix_from_json, "Nutitar": nutitar_from_json}


def load_config(path: str):
    """Model configuration from a checkpoint folder's config.json, chosen by its
    ``architecture`` key; None when the folder names no architecture known here."""
    import json
    import os

    f = os.path.join(path, "config.json") if os.path.isdir(path) else ""
    if not f or not os.path.exists(f):
        return None
    with open(f) as fh:
        d = json.load(fh)
    reader = ARCHITECTURES.get(d.get("architecture", ""))
    return reader(d) if reader else None
