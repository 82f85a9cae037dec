"""Model architecture configs.

Dimensions are the public model-card values the reference's model names imply
(SURVEY.md §2.C): the reference only names the models (``meta/llama3-8b-instruct``,
``meta/llama3-70b-instruct`` — deploy/compose/docker-compose-nim-ms.yaml:4,
rag-app-api-catalog-text-chatbot.yaml:14; ``snowflake/arctic-embed-l`` — compose.env:25-27).
Weights are random-initialised (no checkpoints are reachable), so every benchmark runs the
real architecture on synthetic inputs.
"""
from __future__ import annotations

from dataclasses import asdict, dataclass, field, replace
from typing import Optional, Sequence


@dataclass(frozen=True)
class LlamaConfig:
    """Decoder-only LM config. The defaults are Llama-3-8B; the architecture switches below
    cover every decoder family the reference names:

    * ``mistral`` — Llama layout, optional sliding-window attention (Mistral-7B NIM config,
      experimental/fm-asr-streaming-rag/nim/configs/mistral-7b.yaml:3);
    * ``mixtral`` — sparse MoE MLP, ``num_experts`` SwiGLU experts, top-``experts_per_tok``
      softmax routing (the reference's default chat model ``ai-mixtral-8x7b-instruct``,
      RetrievalAugmentedGeneration/common/configuration.py:75);
    * ``gemma`` — GeGLU (tanh GELU), RMSNorm with a (1 + w) scale, sqrt(hidden) embedding
      scale, tied embeddings, head_dim 256 (models/Gemma/*.ipynb, models/Codegemma/lora.ipynb);
    * ``starcoder2`` — LayerNorm with bias, biased projections, non-gated tanh-GELU MLP,
      sliding-window attention (models/StarCoder2/*.ipynb)."""

    name: str = "llama3-8b"
    vocab_size: int = 128256
    hidden: int = 4096
    layers: int = 32
    heads: int = 32
    kv_heads: int = 8
    head_dim: int = 128
    ffn: int = 14336
    rope_theta: float = 500000.0
    rope_scaling: Optional[dict] = None
    eps: float = 1e-5
    max_position: int = 8192
    bos_id: int = 128000
    eos_ids: tuple = (128001, 128009)
    arch: str = "llama"            # llama | mistral | mixtral | gemma | starcoder2
    norm: str = "rms"              # rms | layer (LayerNorm with bias)
    act: str = "silu"              # silu | gelu_tanh
    gated_mlp: bool = True         # act(gate) * up  (False: act(fc(x) + b) -> proj)
    attn_bias: bool = False        # q/k/v/o projection biases
    mlp_bias: bool = False
    embed_scale: float = 1.0       # Gemma multiplies the embedding by sqrt(hidden)
    tie_embeddings: bool = False
    sliding_window: int = 0        # 0: full causal attention; W: key j visible to query i iff i - W < j <= i
    num_experts: int = 0           # > 0: sparse MoE MLP
    experts_per_tok: int = 2
    chat_format: str = "llama3"    # llama3 | mistral | gemma | plain

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    @property
    def qkv_dim(self) -> int:
        return (self.heads + 2 * self.kv_heads) * self.head_dim

    def num_params(self) -> int:
        mlp = (3 if self.gated_mlp else 2) * self.hidden * self.ffn
        if self.is_moe:
            mlp = mlp * self.num_experts + self.num_experts * self.hidden
        per_layer = (self.hidden * self.qkv_dim + self.heads * self.head_dim * self.hidden
                     + mlp + 2 * self.hidden)
        heads = 1 if self.tie_embeddings else 2
        return per_layer * self.layers + heads * self.vocab_size * self.hidden + self.hidden

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return 2 * self.layers * self.kv_heads * self.head_dim * dtype_bytes

    def to_dict(self):
        return asdict(self)


@dataclass(frozen=True)
class EncoderConfig:
    """BERT-large-class bidirectional encoder (snowflake-arctic-embed-l shape)."""

    name: str = "arctic-embed-l"
    vocab_size: int = 30522
    hidden: int = 1024
    layers: int = 24
    heads: int = 16
    ffn: int = 4096
    max_position: int = 512
    type_vocab: int = 2
    eps: float = 1e-12
    pooling: str = "cls"  # "cls" | "mean"
    normalize: bool = True
    query_prefix: str = "Represent this sentence for searching relevant passages: "
    passage_prefix: str = ""
    num_labels: int = 0  # >0: cross-encoder / reranker head on the pooled output

    @property
    def head_dim(self) -> int:
        return self.hidden // self.heads

    def to_dict(self):
        return asdict(self)


LLAMA_PRESETS = {
    "llama3-8b": LlamaConfig(),
    "llama3-70b": LlamaConfig(name="llama3-70b", hidden=8192, layers=80, heads=64, kv_heads=8,
                              ffn=28672),
    # small language model (models/NeMo/slm/slm_pretraining_sft.ipynb#cell 18: 12 layers,
    # hidden 768) in this architecture, for training/pretrain.py
    "slm-125m": LlamaConfig(name="slm-125m", hidden=768, layers=12, heads=12, kv_heads=12,
                            head_dim=64, ffn=2048, rope_theta=10000.0, max_position=2048),
    # ---- other decoder families (public model-card dimensions)
    # Mistral-7B-Instruct v0.3 (32768-token vocabulary, full attention, theta 1e6)
    "mistral-7b": LlamaConfig(name="mistral-7b", arch="mistral", vocab_size=32768, rope_theta=1e6,
                              max_position=32768, bos_id=1, eos_ids=(2,), chat_format="mistral"),
    # Mistral-7B v0.1: 4096-token sliding window
    "mistral-7b-v0.1": LlamaConfig(name="mistral-7b-v0.1", arch="mistral", vocab_size=32000,
                                   rope_theta=10000.0, sliding_window=4096, max_position=32768,
                                   bos_id=1, eos_ids=(2,), chat_format="mistral"),
    "mixtral-8x7b": LlamaConfig(name="mixtral-8x7b", arch="mixtral", vocab_size=32000,
                                rope_theta=1e6, max_position=32768, num_experts=8,
                                experts_per_tok=2, bos_id=1, eos_ids=(2,), chat_format="mistral"),
    "gemma-7b": LlamaConfig(name="gemma-7b", arch="gemma", vocab_size=256000, hidden=3072,
                            layers=28, heads=16, kv_heads=16, head_dim=256, ffn=24576,
                            rope_theta=10000.0, eps=1e-6, act="gelu_tanh",
                            embed_scale=3072 ** 0.5, tie_embeddings=True, bos_id=2, eos_ids=(1, 107),
                            chat_format="gemma"),
    "gemma-2b": LlamaConfig(name="gemma-2b", arch="gemma", vocab_size=256000, hidden=2048,
                            layers=18, heads=8, kv_heads=1, head_dim=256, ffn=16384,
                            rope_theta=10000.0, eps=1e-6, act="gelu_tanh",
                            embed_scale=2048 ** 0.5, tie_embeddings=True, bos_id=2, eos_ids=(1, 107),
                            chat_format="gemma"),
    "codegemma-7b": LlamaConfig(name="codegemma-7b", arch="gemma", vocab_size=256000, hidden=3072,
                                layers=28, heads=16, kv_heads=16, head_dim=256, ffn=24576,
                                rope_theta=10000.0, eps=1e-6, act="gelu_tanh",
                                embed_scale=3072 ** 0.5, tie_embeddings=True, bos_id=2,
                                eos_ids=(1, 107), chat_format="gemma"),
    "starcoder2-3b": LlamaConfig(name="starcoder2-3b", arch="starcoder2", vocab_size=49152,
                                 hidden=3072, layers=30, heads=24, kv_heads=2, ffn=12288,
                                 rope_theta=999999.4, norm="layer", act="gelu_tanh",
                                 gated_mlp=False, attn_bias=True, mlp_bias=True,
                                 tie_embeddings=True, sliding_window=4096, max_position=16384,
                                 bos_id=0, eos_ids=(0,), chat_format="plain"),
    "starcoder2-7b": LlamaConfig(name="starcoder2-7b", arch="starcoder2", vocab_size=49152,
                                 hidden=4608, layers=32, heads=36, kv_heads=4, ffn=18432,
                                 rope_theta=1e6, norm="layer", act="gelu_tanh", gated_mlp=False,
                                 attn_bias=True, mlp_bias=True, tie_embeddings=True,
                                 sliding_window=4096, max_position=16384, bos_id=0, eos_ids=(0,),
                                 chat_format="plain"),
    "starcoder2-15b": LlamaConfig(name="starcoder2-15b", arch="starcoder2", vocab_size=49152,
                                  hidden=6144, layers=40, heads=48, kv_heads=4, ffn=24576,
                                  rope_theta=100000.0, norm="layer", act="gelu_tanh",
                                  gated_mlp=False, attn_bias=True, mlp_bias=True,
                                  sliding_window=4096, max_position=16384, bos_id=0, eos_ids=(0,),
                                  chat_format="plain"),
    # nv-rerank-qa-mistral-4b: Mistral-7B v0.1 cut to its first 16 layers (bidirectional)
    "mistral-4b-rerank": LlamaConfig(name="mistral-4b-rerank", arch="mistral", vocab_size=32000,
                                     layers=16, rope_theta=10000.0, max_position=4096, bos_id=1,
                                     eos_ids=(2,), chat_format="mistral"),
    # LLaVA-1.5's language model (Vicuna-7B = Llama-2-7B dims) and the NeVA-22B-class decoder
    "vicuna-7b": LlamaConfig(name="vicuna-7b", vocab_size=32000, hidden=4096, layers=32, heads=32,
                             kv_heads=32, ffn=11008, rope_theta=10000.0, max_position=4096,
                             bos_id=1, eos_ids=(2,), chat_format="plain"),
    "neva-22b-llm": LlamaConfig(name="neva-22b-llm", vocab_size=32768, hidden=6144, layers=40,
                                heads=48, kv_heads=8, ffn=24576, rope_theta=10000.0,
                                max_position=4096, bos_id=1, eos_ids=(2,), chat_format="plain"),
    # small configs with the same structure for CPU tests / smoke runs
    "llama-tiny": LlamaConfig(name="llama-tiny", vocab_size=32768, hidden=256, layers=2, heads=4,
                              kv_heads=2, head_dim=64, ffn=512, max_position=2048,
                              bos_id=1, eos_ids=(2,)),
    # Llama-3-70B's attention layout (64 q : 8 kv heads: at TP=8 one KV head per rank) at tiny width
    "llama70b-tiny": LlamaConfig(name="llama70b-tiny", vocab_size=32768, hidden=256, layers=2, heads=64,
                                 kv_heads=8, head_dim=16, ffn=512, max_position=2048,
                                 bos_id=1, eos_ids=(2,)),
    # Llama-3-70B's attention layout with its real head_dim 128 at a small width: at TP=8 each
    # rank holds 8 q heads and 1 KV head and the q/k/v shard is 1280 wide (as 70B's), so the
    # one-GPU TP=8 rehearsal runs the GPU kernels of a 70B rank; hidden 2048 makes a 256-token
    # step's all-reduce 1 MiB, past the two-shot threshold
    "llama70b-small": LlamaConfig(name="llama70b-small", vocab_size=32768, hidden=2048, layers=2, heads=64,
                                  kv_heads=8, head_dim=128, ffn=4096, max_position=8192, bos_id=1,
                                  eos_ids=(2,)),
    # Llama-3-8B's attention layout (32 q : 8 kv heads of 128) at a small width: the headline's
    # GQA group and work-item counts in step-graph GPU tests
    "llama3-gqa-small": LlamaConfig(name="llama3-gqa-small", vocab_size=32768, hidden=1024, layers=2, heads=32,
                                    kv_heads=8, head_dim=128, ffn=2816, max_position=8192, bos_id=1,
                                    eos_ids=(2,)),
    "llama-small": LlamaConfig(name="llama-small", vocab_size=32768, hidden=1024, layers=4,
                               heads=8, kv_heads=2, head_dim=128, ffn=2816,
                               max_position=8192, bos_id=1, eos_ids=(2,)),
    "mistral-tiny": LlamaConfig(name="mistral-tiny", arch="mistral", vocab_size=32768, hidden=256,
                                layers=2, heads=4, kv_heads=2, head_dim=64, ffn=512,
                                rope_theta=1e6, sliding_window=96, max_position=2048, bos_id=1,
                                eos_ids=(2,), chat_format="mistral"),
    "mixtral-tiny": LlamaConfig(name="mixtral-tiny", arch="mixtral", vocab_size=32768, hidden=256,
                                layers=2, heads=4, kv_heads=2, head_dim=64, ffn=384,
                                rope_theta=1e6, num_experts=4, experts_per_tok=2,
                                max_position=2048, bos_id=1, eos_ids=(2,), chat_format="mistral"),
    "gemma-tiny": LlamaConfig(name="gemma-tiny", arch="gemma", vocab_size=32768, hidden=256,
                              layers=2, heads=2, kv_heads=1, head_dim=256, ffn=512,
                              rope_theta=10000.0, eps=1e-6, act="gelu_tanh", embed_scale=16.0,
                              tie_embeddings=True, max_position=2048, bos_id=1, eos_ids=(2,),
                              chat_format="gemma"),
    "starcoder2-tiny": LlamaConfig(name="starcoder2-tiny", arch="starcoder2", vocab_size=32768,
                                   hidden=256, layers=2, heads=4, kv_heads=2, head_dim=64, ffn=512,
                                   rope_theta=1e5, norm="layer", act="gelu_tanh", gated_mlp=False,
                                   attn_bias=True, mlp_bias=True, tie_embeddings=True,
                                   sliding_window=96, max_position=2048, bos_id=1, eos_ids=(2,),
                                   chat_format="plain"),
    # small models of the real families' shapes for GPU kernel tests (head_dim 128 / 256)
    "mixtral-small": LlamaConfig(name="mixtral-small", arch="mixtral", vocab_size=32768,
                                 hidden=1024, layers=2, heads=8, kv_heads=2, head_dim=128,
                                 ffn=1792, rope_theta=1e6, num_experts=8, experts_per_tok=2,
                                 max_position=8192, bos_id=1, eos_ids=(2,), chat_format="mistral"),
    "mistral-small": LlamaConfig(name="mistral-small", arch="mistral", vocab_size=32768,
                                 hidden=1024, layers=2, heads=8, kv_heads=2, head_dim=128,
                                 ffn=2816, rope_theta=1e6, sliding_window=200, max_position=8192,
                                 bos_id=1, eos_ids=(2,), chat_format="mistral"),
    "starcoder2-small": LlamaConfig(name="starcoder2-small", arch="starcoder2", vocab_size=32768,
                                    hidden=1024, layers=2, heads=8, kv_heads=2, head_dim=128,
                                    ffn=4096, rope_theta=1e5, norm="layer", act="gelu_tanh",
                                    gated_mlp=False, attn_bias=True, mlp_bias=True,
                                    tie_embeddings=True, sliding_window=200, max_position=8192,
                                    bos_id=1, eos_ids=(2,), chat_format="plain"),
    "gemma-small": LlamaConfig(name="gemma-small", arch="gemma", vocab_size=32768, hidden=1024,
                               layers=2, heads=8, kv_heads=1, head_dim=256, ffn=2048,
                               rope_theta=10000.0, eps=1e-6, act="gelu_tanh", embed_scale=32.0,
                               tie_embeddings=True, max_position=8192, bos_id=1, eos_ids=(2,),
                               chat_format="gemma"),
}

# DecoderConfig is the family-neutral name of the same dataclass
DecoderConfig = LlamaConfig

ENCODER_PRESETS = {
    "arctic-embed-l": EncoderConfig(),
    "nv-embed-qa": EncoderConfig(name="nv-embed-qa"),
    "e5-large-v2": EncoderConfig(name="e5-large-v2", pooling="mean", query_prefix="query: ",
                                 passage_prefix="passage: "),
    "all-minilm-l6-v2": EncoderConfig(name="all-minilm-l6-v2", hidden=384, layers=6, heads=12,
                                      ffn=1536, pooling="mean", query_prefix=""),
    "bge-reranker-large": EncoderConfig(name="bge-reranker-large", num_labels=1,
                                        normalize=False, query_prefix=""),
    "encoder-tiny": EncoderConfig(name="encoder-tiny", vocab_size=30522, hidden=128, layers=2,
                                  heads=2, ffn=256, max_position=512),
    "reranker-tiny": EncoderConfig(name="reranker-tiny", vocab_size=30522, hidden=128, layers=2,
                                   heads=2, ffn=256, max_position=512, num_labels=1,
                                   normalize=False, query_prefix=""),
}


def llama_config(name_or_cfg, **overrides) -> LlamaConfig:
    cfg = LLAMA_PRESETS[name_or_cfg] if isinstance(name_or_cfg, str) else name_or_cfg
    return replace(cfg, **overrides) if overrides else cfg


def encoder_config(name_or_cfg, **overrides) -> EncoderConfig:
    cfg = ENCODER_PRESETS[name_or_cfg] if isinstance(name_or_cfg, str) else name_or_cfg
    return replace(cfg, **overrides) if overrides else cfg


# ---------------------------------------------------------------------------------------------
# Layer-list decoders: config.json lists the blocks one by one, each with its own mixer sizes.
@dataclass(frozen=True)
class SigmoidAttentionSpec:
    """Mixer ``attention`` of the Bidasun design: un-normalised sigmoid attention with a
    logarithmic distance term, a sliding window that keeps the first tokens, whole-projection
    q / k RMS norm and an output gate (``ops.sigmoid_attention``)."""

    heads: int
    kv_heads: int
    dim: int            # per-head q / k size
    vdim: int           # per-head v size
    scale: float
    window: int         # i sees j when i - j < window ...
    keep_first: int     # ... or j < keep_first


@dataclass(frozen=True)
class DenseMlpSpec:
    ff: int
    kind: str = "dense"     # down(gelu_tanh(gate x) * (up x))


@dataclass(frozen=True)
class BlockSpec:
    type: str                              # mixer kind; "attention" -> SigmoidAttentionSpec
    mixer: SigmoidAttentionSpec
    mlp: Optional[DenseMlpSpec] = None     # None: the block has no feed-forward


@dataclass(frozen=True)
class BidasunConfig:
    """Bidasun: post-norm blocks (x += norm(mixer(shift(x))), x += norm(ff(x))) on an fp32
    residual stream, learned positions, token shift in front of every mixer. Every size and
    constant comes from the model folder's config.json (:meth:`from_dict`)."""

    name: str = "bidasun"
    vocab_size: int = 512
    hidden: int = 128
    max_position: int = 1024
    eps: float = 1e-5
    blocks: tuple = ()
    arch: str = "bidasun"
    bos_id: int = 0
    eos_ids: tuple = ()
    chat_format: str = "plain"
    is_moe: bool = False

    @property
    def layers(self) -> int:
        return len(self.blocks)

    @classmethod
    def from_dict(cls, d: dict, name: str = "bidasun") -> "BidasunConfig":
        blocks = []
        for i, b in enumerate(d["layers"]):
            if b["type"] != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {b['type']!r}")
            m = b["mixer"]
            mixer = SigmoidAttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                         vdim=int(m["vdim"]), scale=float(m["scale"]),
                                         window=int(m["mask"]["size"]), keep_first=int(m["mask"]["keep_first"]))
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"layer {i}: {mixer.heads} heads over {mixer.kv_heads} kv heads")
            mlp = b.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
                mlp = DenseMlpSpec(ff=int(mlp["ff"]))
            blocks.append(BlockSpec(type="attention", mixer=mixer, mlp=mlp))
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]),
                   max_position=int(d["max_positions"]), eps=float(d["norm"]["eps"]), blocks=tuple(blocks))

    def to_json_dict(self) -> dict:
        """The config.json form (inverse of :meth:`from_dict`)."""
        return {"architecture": "Bidasun", "vocab": self.vocab_size, "width": self.hidden,
                "max_positions": self.max_position, "norm": {"eps": self.eps},
                "layers": [{"type": b.type,
                            "mixer": {"heads": b.mixer.heads, "kv_heads": b.mixer.kv_heads, "dim": b.mixer.dim,
                                      "vdim": b.mixer.vdim, "scale": b.mixer.scale,
                                      "mask": {"size": b.mixer.window, "keep_first": b.mixer.keep_first}},
                            "mlp": None if b.mlp is None else {"kind": b.mlp.kind, "ff": b.mlp.ff}}
                           for b in self.blocks]}

    def num_params(self) -> int:
        n = (2 * self.vocab_size + self.max_position + 1) * self.hidden
        for b in self.blocks:
            m = b.mixer
            nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            n += self.hidden * (nq + nk + nv + 2 * m.heads * m.vdim) + nq + nk + 3 * m.heads + 2 * self.hidden
            if b.mlp is not None:
                n += 3 * self.hidden * b.mlp.ff + self.hidden
        return n

    def to_dict(self):
        return asdict(self)


def bidasun_uniform(layers: int, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, ff: int,
                    window: int, keep_first: int, vocab_size: int = 32768, max_position: int = 8192,
                    scale: Optional[float] = None, eps: float = 1e-5, name: str = "bidasun") -> BidasunConfig:
    """A Bidasun config whose blocks are all alike (benchmarks, tests)."""
    m = SigmoidAttentionSpec(heads, kv_heads, dim, vdim, dim ** -0.5 if scale is None else scale, window, keep_first)
    blk = BlockSpec("attention", m, DenseMlpSpec(ff) if ff else None)
    return BidasunConfig(name=name, vocab_size=vocab_size, hidden=hidden, max_position=max_position, eps=eps,
                         blocks=(blk,) * layers)


# ---------------------------------------------------------------------------------------------
# Biruvik: a layer list whose entries choose between three mixers.
@dataclass(frozen=True)
class DiffAttentionSpec:
    """Mixer ``attention`` of the Biruvik design: differential softmax attention. Every head has
    two score maps (own q and k halves, shared v); ``o = a1 - lam * a2`` with one ``lam`` per
    layer, unit RMS per head, times ``1 - diff``. Causal, GQA, per head-and-map RMS norm of q
    and k, biases on q / k / v, no rotation; the query is scaled by
    ``1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1)`` at position p."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    q_temp_coef: float
    q_temp_every: int


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Mixer ``latent_attention``: keys and values are linear maps of one RMS-normed latent per
    token (only the latent is cached), softmax over a sliding window (``window`` keys, the
    query's own included; 0 = no limit), sigmoid output gate per head, no positions."""

    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int


@dataclass(frozen=True)
class Hgrn2Spec:
    """Mixer ``hgrn2``: per head ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T q`` with
    ``q = silu(W_q h)`` and the forget gate ``f = l + (1 - l) sigmoid(W_f h + b)`` bounded from
    below by ``l``; RMS norm of every head's output; fp32 state [heads, dim, vdim] per sequence."""

    heads: int
    dim: int
    vdim: int


@dataclass(frozen=True)
class ReluSqMlpSpec:
    ff: int
    kind: str = "dense"     # down(relu(up x)^2)


@dataclass(frozen=True)
class BiruvikLayer:
    type: str                 # "attention" | "latent_attention" | "hgrn2"
    mixer: object
    mlp: Optional[ReluSqMlpSpec] = None


_BIRUVIK_MIXERS = ("attention", "latent_attention", "hgrn2")


@dataclass(frozen=True)
class BiruvikConfig:
    """Biruvik: pre- and post-normed sub-layers on an fp32 residual stream
    (``x += norm_b(sub(norm_a(x)))``, every norm an RMS norm with one gain), a scaled embedding,
    no position table, a tanh soft cap on the logits. Every size and constant that can differ
    between models comes from config.json (:meth:`from_dict`)."""

    name: str = "biruvik"
    vocab_size: int = 512
    hidden: int = 128
    eps: float = 1e-5
    embed_scale: float = 1.0
    logit_softcap: float = 0.0      # 0: none
    blocks: tuple = ()
    max_position: int = 1 << 20     # no position table: only the engine's bookkeeping is bounded
    arch: str = "biruvik"
    bos_id: int = 0
    eos_ids: tuple = ()
    chat_format: str = "plain"
    is_moe: bool = False

    @property
    def layers(self) -> int:
        return len(self.blocks)

    @classmethod
    def from_dict(cls, d: dict, name: str = "biruvik") -> "BiruvikConfig":
        blocks = []
        for i, b in enumerate(d["layers"]):
            t, m = b["type"], b["mixer"]
            if t == "attention":
                mixer = DiffAttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                          vdim=int(m["vdim"]), scale=float(m["scale"]), diff=float(m["diff"]),
                                          q_temp_coef=float(m["q_temp"]["coef"]),
                                          q_temp_every=int(m["q_temp"]["every"]))
                if mixer.heads % mixer.kv_heads:
                    raise ValueError(f"layer {i}: {mixer.heads} heads over {mixer.kv_heads} kv heads")
                if mixer.q_temp_every < 1:
                    raise ValueError(f"layer {i}: q_temp.every must be at least 1")
            elif t == "latent_attention":
                mixer = LatentAttentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                            kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                                            window=int(m["mask"]["size"]))
                if mixer.window < 1:
                    raise ValueError(f"layer {i}: a window holds at least the query's own position")
            elif t == "hgrn2":
                mixer = Hgrn2Spec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {t!r} (known: {_BIRUVIK_MIXERS})")
            mlp = b.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
                mlp = ReluSqMlpSpec(ff=int(mlp["ff"]))
            blocks.append(BiruvikLayer(type=t, mixer=mixer, mlp=mlp))
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), eps=float(d["norm"]["eps"]),
                   embed_scale=float(d["embedding"]["scale"]), logit_softcap=float(d.get("logit_softcap") or 0.0),
                   blocks=tuple(blocks))

    def to_json_dict(self) -> dict:
        """The config.json form (inverse of :meth:`from_dict`)."""
        layers = []
        for b in self.blocks:
            m = b.mixer
            if b.type == "attention":
                mx = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                      "diff": m.diff, "q_temp": {"coef": m.q_temp_coef, "every": m.q_temp_every}}
            elif b.type == "latent_attention":
                mx = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                      "mask": {"size": m.window}}
            else:
                mx = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim}
            layers.append({"type": b.type, "mixer": mx,
                           "mlp": None if b.mlp is None else {"kind": b.mlp.kind, "ff": b.mlp.ff}})
        return {"architecture": "Biruvik", "vocab": self.vocab_size, "width": self.hidden,
                "embedding": {"scale": self.embed_scale}, "norm": {"eps": self.eps},
                "logit_softcap": self.logit_softcap, "layers": layers}

    def num_params(self) -> int:
        H = self.hidden
        n = 2 * self.vocab_size * H + 1
        for b in self.blocks:
            m = b.mixer
            n += 2
            if b.type == "attention":
                n += (H + 1) * (2 * m.heads * m.dim + 2 * m.kv_heads * m.dim + m.kv_heads * m.vdim) + 6 * m.dim
                n += H * m.heads * m.vdim
            elif b.type == "latent_attention":
                n += H * (m.heads * m.dim + m.kv_rank + m.heads) + m.kv_rank
                n += m.kv_rank * m.heads * (m.dim + m.vdim) + H * m.heads * m.vdim
            else:
                n += H * (2 * m.heads * m.dim + m.heads * m.vdim) + 2 * m.heads * m.dim + m.vdim
                n += H * m.heads * m.vdim
            if b.mlp is not None:
                n += 2 * H * b.mlp.ff + 2
        return n

    def to_dict(self):
        return asdict(self)


def biruvik_layers(pattern: Sequence[str], hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, ff: int,
                   window: int = 1024, kv_rank: int = 512, diff: float = 0.25, q_temp=(0.1, 1024),
                   vocab_size: int = 32768, embed_scale: float = 1.0, logit_softcap: float = 30.0,
                   eps: float = 1e-5, name: str = "biruvik") -> BiruvikConfig:
    """A Biruvik config from a pattern of mixer types with the same sizes in every layer
    (benchmarks, tests)."""
    blocks = []
    for t in pattern:
        if t == "attention":
            m = DiffAttentionSpec(heads, kv_heads, dim, vdim, dim ** -0.5, diff, float(q_temp[0]), int(q_temp[1]))
        elif t == "latent_attention":
            m = LatentAttentionSpec(heads, dim, vdim, kv_rank, dim ** -0.5, window)
        elif t == "hgrn2":
            m = Hgrn2Spec(heads, dim, vdim)
        else:
            raise ValueError(f"unknown mixer type {t!r}")
        blocks.append(BiruvikLayer(t, m, ReluSqMlpSpec(ff) if ff else None))
    return BiruvikConfig(name=name, vocab_size=vocab_size, hidden=hidden, eps=eps, embed_scale=embed_scale,
                         logit_softcap=logit_softcap, blocks=tuple(blocks))


# ---------------------------------------------------------------------------------------------
# Lumepel: pre-norm layers whose mixers are latent attention with a rotated key part.
@dataclass(frozen=True)
class RotarySpec:
    """Rotary positions on the first ``dims`` elements of a vector: pair i turns by
    ``p * f_i`` at position p, ``f_i = base^(-2i / dims)``. ``interleaved``: pair i is elements
    (2i, 2i + 1), else (i, i + dims / 2). ``yarn`` = (factor, original, fast, slow) or None: the
    frequencies of slow pairs are divided by ``factor`` along a linear ramp over the pair index,
    and cos / sin are multiplied by ``0.1 ln(factor) + 1`` (:func:`ops.rotary_frequencies`)."""

    dims: int
    base: float
    interleaved: bool = False
    yarn: Optional[tuple] = None


@dataclass(frozen=True)
class RotaryLatentAttentionSpec:
    """Mixers ``latent_attention`` / ``latent_attention_2``: causal softmax attention whose keys
    and values are linear maps of one RMS-normed latent of ``kv_rank`` elements per token, plus
    one rotated key part of ``rot_dim`` elements shared by all heads; a query head is ``dim``
    unrotated and ``rot_dim`` rotated elements. Only the latent and the rotated key part are
    cached. ``q_rank`` > 0: the query goes through an RMS-normed latent of its own."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: RotarySpec
    q_rank: int = 0


@dataclass(frozen=True)
class ClampedGluSpec:
    """down(g * sigmoid(1.702 g) * (u + 1)) with g = min(gate x, limit), u = clamp(up x, +-limit)."""

    ff: int
    limit: float
    kind: str = "dense"


@dataclass(frozen=True)
class SigmoidMoeSpec:
    """``experts`` clamped-GLU experts of which a token uses the ``top`` with the largest
    ``sigmoid(router x)``; the scores are the weights as they are (not renormalised) and multiply
    the expert's *input*. ``shared``: an expert every token uses, times ``sigmoid(sg . x)``."""

    experts: int
    top: int
    expert: ClampedGluSpec
    shared: Optional[ClampedGluSpec] = None
    kind: str = "moe"


@dataclass(frozen=True)
class LumepelLayer:
    type: str                 # "latent_attention" | "latent_attention_2"
    mixer: RotaryLatentAttentionSpec
    mlp: object = None        # ClampedGluSpec | SigmoidMoeSpec | None


_LUMEPEL_MIXERS = ("latent_attention", "latent_attention_2")


@dataclass(frozen=True)
class LumepelConfig:
    """Lumepel: pre-norm layers on an fp32 residual stream (``x += mixer(norm1(x))``,
    ``x += ff(norm2(x))``), a scaled embedding, scaled and soft-capped logits. Every size and
    every constant that can differ between models comes from config.json (:meth:`from_dict`)."""

    name: str = "lumepel"
    vocab_size: int = 512
    hidden: int = 128
    eps: float = 1e-5
    embed_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0      # 0: none
    blocks: tuple = ()
    max_position: int = 1 << 20     # no position table: only the engine's bookkeeping is bounded
    arch: str = "lumepel"
    bos_id: int = 0
    eos_ids: tuple = ()
    chat_format: str = "plain"

    @property
    def layers(self) -> int:
        return len(self.blocks)

    @property
    def is_moe(self) -> bool:
        return any(isinstance(b.mlp, SigmoidMoeSpec) for b in self.blocks)

    @property
    def experts_per_tok(self) -> int:
        """Largest top-k of any layer (sizes the engine's routing workspace)."""
        return max([b.mlp.top for b in self.blocks if isinstance(b.mlp, SigmoidMoeSpec)] or [1])

    @property
    def num_experts(self) -> int:
        return max([b.mlp.experts for b in self.blocks if isinstance(b.mlp, SigmoidMoeSpec)] or [0])

    @staticmethod
    def _glu(d: dict, what: str) -> ClampedGluSpec:
        s = ClampedGluSpec(ff=int(d["ff"]), limit=float(d["limit"]))
        if s.ff < 1 or not s.limit > 0:
            raise ValueError(f"{what}: ff and limit must be positive")
        return s

    @classmethod
    def from_dict(cls, d: dict, name: str = "lumepel") -> "LumepelConfig":
        blocks = []
        for i, b in enumerate(d["layers"]):
            t, m = b["type"], b["mixer"]
            if t not in _LUMEPEL_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {t!r} (known: {_LUMEPEL_MIXERS})")
            r = m["rot"]
            sc = r.get("scaling")
            rot = RotarySpec(dims=int(r["dims"]), base=float(r["base"]), interleaved=t == "latent_attention",
                             yarn=None if not sc else (float(sc["factor"]), float(sc["original"]),
                                                       float(sc["fast"]), float(sc["slow"])))
            mixer = RotaryLatentAttentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]),
                                              vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                                              rot=rot, q_rank=int(m["q_rank"]) if t == "latent_attention" else 0)
            if rot.dims % 2 or not 0 < rot.dims <= mixer.rot_dim:
                raise ValueError(f"layer {i}: rot.dims must be even and at most rot_dim")
            if t == "latent_attention" and mixer.q_rank < 1:
                raise ValueError(f"layer {i}: latent_attention needs q_rank")
            mlp = b.get("mlp")
            if mlp is not None:
                kind = mlp.get("kind", "dense")
                if kind == "dense":
                    mlp = cls._glu(mlp, f"layer {i} feed-forward")
                elif kind == "moe":
                    sh = mlp.get("shared")
                    mlp = SigmoidMoeSpec(experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                                         expert=cls._glu(mlp["expert"], f"layer {i} experts"),
                                         shared=None if not sh else cls._glu(sh, f"layer {i} shared expert"))
                    if not 1 <= mlp.top <= mlp.experts:
                        raise ValueError(f"layer {i}: top {mlp.top} of {mlp.experts} experts")
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
            blocks.append(LumepelLayer(type=t, mixer=mixer, mlp=mlp))
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), eps=float(d["norm"]["eps"]),
                   embed_scale=float(d["embedding"]["scale"]), logit_scale=float(d.get("logit_scale", 1.0)),
                   logit_softcap=float(d.get("logit_softcap") or 0.0), blocks=tuple(blocks))

    def to_json_dict(self) -> dict:
        """The config.json form (inverse of :meth:`from_dict`)."""
        layers = []
        for b in self.blocks:
            m = b.mixer
            rot = {"base": m.rot.base, "dims": m.rot.dims}
            if m.rot.yarn:
                rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), m.rot.yarn))
            mx = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                  "scale": m.scale, "rot": rot}
            if b.type == "latent_attention":
                mx["q_rank"] = m.q_rank
            f = b.mlp
            if isinstance(f, SigmoidMoeSpec):
                ff = {"kind": "moe", "router": {"experts": f.experts, "top": f.top},
                      "expert": {"ff": f.expert.ff, "limit": f.expert.limit}}
                if f.shared is not None:
                    ff["shared"] = {"ff": f.shared.ff, "limit": f.shared.limit}
            elif f is not None:
                ff = {"kind": "dense", "ff": f.ff, "limit": f.limit}
            else:
                ff = None
            layers.append({"type": b.type, "mixer": mx, "mlp": ff})
        return {"architecture": "Lumepel", "vocab": self.vocab_size, "width": self.hidden,
                "embedding": {"scale": self.embed_scale}, "norm": {"eps": self.eps},
                "logit_scale": self.logit_scale, "logit_softcap": self.logit_softcap, "layers": layers}

    def num_params(self) -> int:
        H = self.hidden
        n = 2 * self.vocab_size * H + H
        for b in self.blocks:
            m = b.mixer
            nq = m.heads * (m.dim + m.rot_dim)
            n += H + (H * m.q_rank + m.q_rank + m.q_rank * nq if m.q_rank else H * nq)
            n += H * (m.kv_rank + m.rot_dim) + m.kv_rank + m.kv_rank * m.heads * (m.dim + m.vdim) + H * m.heads * m.vdim
            f = b.mlp
            if isinstance(f, SigmoidMoeSpec):
                n += H + f.experts * (3 * H * f.expert.ff + H)
                if f.shared is not None:
                    n += 3 * H * f.shared.ff + H
            elif f is not None:
                n += H + 3 * H * f.ff
        return n

    def to_dict(self):
        return asdict(self)


def lumepel_layers(pattern: Sequence[str], hidden: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                   q_rank: int, ff: int, experts: int = 0, top: int = 2, expert_ff: int = 0, shared_ff: int = 0,
                   limit: float = 7.0, rot_base: float = 10000.0, yarn: Optional[tuple] = None,
                   vocab_size: int = 32768, embed_scale: float = 1.0, logit_scale: float = 1.0,
                   logit_softcap: float = 30.0, eps: float = 1e-5, name: str = "lumepel") -> LumepelConfig:
    """A Lumepel config from a pattern of mixer types with the same sizes in every layer
    (benchmarks, tests). ``experts`` > 0: every feed-forward is a mixture of ``experts`` experts of
    ``expert_ff`` (plus a shared one of ``shared_ff``), else dense of ``ff`` (0: none)."""
    blocks = []
    for t in pattern:
        if t not in _LUMEPEL_MIXERS:
            raise ValueError(f"unknown mixer type {t!r}")
        lat = t == "latent_attention"
        rot = RotarySpec(rot_dim, rot_base, interleaved=lat, yarn=yarn if lat else None)
        m = RotaryLatentAttentionSpec(heads, dim, rot_dim, vdim, kv_rank, (dim + rot_dim) ** -0.5, rot,
                                      q_rank if lat else 0)
        if experts:
            mlp = SigmoidMoeSpec(experts, top, ClampedGluSpec(expert_ff, limit),
                                 ClampedGluSpec(shared_ff, limit) if shared_ff else None)
        else:
            mlp = ClampedGluSpec(ff, limit) if ff else None
        blocks.append(LumepelLayer(t, m, mlp))
    return LumepelConfig(name=name, vocab_size=vocab_size, hidden=hidden, eps=eps, embed_scale=embed_scale,
                         logit_scale=logit_scale, logit_softcap=logit_softcap, blocks=tuple(blocks))


# ---------------------------------------------------------------------------------------------
# Lizezen: parallel layers behind one dynamic-tanh norm, mLSTM and rotary attention mixers, a
# repeated span of layers with an input injection in front of every pass.
@dataclass(frozen=True)
class MlstmSpec:
    """Mixer ``mlstm``: a matrix memory per head, ``S <- a S + b k v^T`` and a normaliser
    ``n <- a n + b k`` with log-domain gates kept stable by a running maximum m; log input gate
    ``cap tanh(z_i / cap)``, log forget gate ``logsigmoid(cap tanh(z_f / cap))``; every head's
    output is brought to unit RMS, weighted, and gated by ``sigmoid(W_g h)``."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class RotaryAttentionSpec:
    """Mixers ``attention`` / ``attention_2``: causal softmax attention with GQA and rotary
    positions (pairs (i, i + dims / 2)) on the first ``rot.dims`` elements of q and k heads.
    ``qk_norm``: RMS norm of every q and k head (one weight of ``dim`` elements each) before the
    rotation; ``values_from_keys``: the values are the key projections as they leave W_k (no
    W_v; ``vdim`` = ``dim``); ``softcap`` > 0: scores go through ``softcap tanh(s / softcap)``;
    ``head_gate``: every head's output is multiplied by ``sigmoid(W_g h)_head``."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotarySpec
    softcap: float = 0.0
    qk_norm: bool = False
    values_from_keys: bool = False
    head_gate: bool = False


@dataclass(frozen=True)
class GeluMlpSpec:
    """down(gelu_tanh(up x + b_up)) + b_down."""

    ff: int
    kind: str = "dense"


@dataclass(frozen=True)
class SwigluSpec:
    """down(silu(gate x) * (up x)), no biases."""

    ff: int


@dataclass(frozen=True)
class GroupedMoeSpec:
    """``experts`` SwiGLU experts plus ``identity`` experts that return their input. Scores are a
    softmax over all ``experts + identity`` router outputs; experts are chosen by score plus a
    per-expert ``correction`` among the ``keep`` best of ``groups`` equal groups of neighbours (a
    group's rank is its largest corrected score); the weights are the uncorrected scores of the
    ``top`` chosen, divided by their sum, times ``scale``. ``shared``: an expert every token uses,
    times ``sigmoid(sg . x)``."""

    experts: int
    top: int
    expert: SwigluSpec
    identity: int = 0
    scale: float = 1.0
    groups: int = 1
    keep: int = 1
    shared: Optional[SwigluSpec] = None
    kind: str = "moe"

    @property
    def routed(self) -> int:
        return self.experts + self.identity


@dataclass(frozen=True)
class LoopSpec:
    """Layers ``start .. stop - 1`` run ``times`` times in a row with the same weights (every
    pass with a cache / state of its own); in front of every pass the stream is replaced by
    ``W_in [x ; x0]`` with x0 the embedding output."""

    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class LizezenLayer:
    type: str                 # "mlstm" | "attention" | "attention_2"
    mixer: object
    mlp: object = None        # GeluMlpSpec | GroupedMoeSpec | None


_LIZEZEN_MIXERS = ("mlstm", "attention", "attention_2")


@dataclass(frozen=True)
class LizezenConfig:
    """Lizezen: parallel layers on an fp32 residual stream, ``h = dyt(x)``,
    ``x += mixer(h) + ff(h)`` with ``dyt(x) = tanh(alpha x) * w + b`` (no statistics). Every size
    and every constant that can differ between models comes from config.json
    (:meth:`from_dict`)."""

    name: str = "lizezen"
    vocab_size: int = 512
    hidden: int = 128
    eps: float = 1e-5
    blocks: tuple = ()
    loop: Optional[LoopSpec] = None
    max_position: int = 1 << 20     # no position table: only the engine's bookkeeping is bounded
    arch: str = "lizezen"
    bos_id: int = 0
    eos_ids: tuple = ()
    chat_format: str = "plain"

    @property
    def layers(self) -> int:
        return len(self.blocks)

    @property
    def runs(self) -> tuple:
        """The order the layers run in: ((layer index, first of a pass of the loop), ...)."""
        n, lp = len(self.blocks), self.loop
        if lp is None:
            return tuple((i, False) for i in range(n))
        out = [(i, False) for i in range(lp.start)]
        for _ in range(lp.times):
            out += [(i, i == lp.start) for i in range(lp.start, lp.stop)]
        return tuple(out + [(i, False) for i in range(lp.stop, n)])

    @property
    def is_moe(self) -> bool:
        return any(isinstance(b.mlp, GroupedMoeSpec) for b in self.blocks)

    @property
    def experts_per_tok(self) -> int:
        """Largest top-k of any layer (sizes the engine's routing workspace)."""
        return max([b.mlp.top for b in self.blocks if isinstance(b.mlp, GroupedMoeSpec)] or [1])

    @property
    def num_experts(self) -> int:
        return max([b.mlp.experts for b in self.blocks if isinstance(b.mlp, GroupedMoeSpec)] or [0])

    @staticmethod
    def _rot(r: dict, what: str, dim: int) -> RotarySpec:
        sc = r.get("scaling")
        rot = RotarySpec(dims=int(r["dims"]), base=float(r["base"]), interleaved=False,
                         yarn=None if not sc else (float(sc["factor"]), float(sc["original"]),
                                                   float(sc["fast"]), float(sc["slow"])))
        if rot.dims % 2 or not 0 < rot.dims <= dim:
            raise ValueError(f"{what}: rot.dims must be even and at most dim")
        return rot

    @classmethod
    def from_dict(cls, d: dict, name: str = "lizezen") -> "LizezenConfig":
        blocks = []
        for i, b in enumerate(d["layers"]):
            t, m = b["type"], b["mixer"]
            if t == "mlstm":
                mixer = MlstmSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                  gate_cap=float(m["gate_cap"]))
                if not mixer.gate_cap > 0:
                    raise ValueError(f"layer {i}: gate_cap must be positive")
            elif t in ("attention", "attention_2"):
                second = t == "attention_2"
                dim = int(m["dim"])
                # (values that are the keys have the keys' size, whatever the config says about vdim)
                mixer = RotaryAttentionSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=dim,
                                            vdim=dim if second else int(m.get("vdim", dim)), scale=float(m["scale"]),
                                            rot=cls._rot(m["rot"], f"layer {i}", dim),
                                            softcap=float(m.get("softcap") or 0.0), qk_norm=second,
                                            values_from_keys=second, head_gate=second)
                if mixer.heads % mixer.kv_heads:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            else:
                raise ValueError(f"layer {i}: unknown mixer type {t!r} (known: {_LIZEZEN_MIXERS})")
            if min(mixer.heads, mixer.dim, mixer.vdim) < 1:
                raise ValueError(f"layer {i}: sizes must be positive")
            mlp = b.get("mlp")
            if mlp is not None:
                kind = mlp.get("kind", "dense")
                if kind == "dense":
                    mlp = GeluMlpSpec(ff=int(mlp["ff"]))
                elif kind == "moe":
                    r, sh, g = mlp["router"], mlp.get("shared"), mlp["router"].get("groups")
                    mlp = GroupedMoeSpec(experts=int(r["experts"]), top=int(r["top"]),
                                         expert=SwigluSpec(int(mlp["expert"]["ff"])),
                                         identity=int(r.get("identity") or 0), scale=float(r.get("scale", 1.0)),
                                         groups=int(g["count"]) if g else 1, keep=int(g["keep"]) if g else 1,
                                         shared=None if not sh else SwigluSpec(int(sh["ff"])))
                    if mlp.routed % mlp.groups or not 1 <= mlp.keep <= mlp.groups:
                        raise ValueError(f"layer {i}: {mlp.routed} routed outputs in {mlp.groups} groups, keep {mlp.keep}")
                    if not 1 <= mlp.top <= mlp.keep * (mlp.routed // mlp.groups):
                        raise ValueError(f"layer {i}: top {mlp.top} does not fit the kept groups")
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
            blocks.append(LizezenLayer(type=t, mixer=mixer, mlp=mlp))
        lp = d.get("loop")
        loop = None
        if lp:
            loop = LoopSpec(start=int(lp["start"]), stop=int(lp["stop"]), times=int(lp["times"]))
            if not (0 <= loop.start < loop.stop <= len(blocks)) or loop.times < 1:
                raise ValueError(f"loop {lp} does not fit {len(blocks)} layers")
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), eps=float(d["norm"]["eps"]),
                   blocks=tuple(blocks), loop=loop)

    def to_json_dict(self) -> dict:
        """The config.json form (inverse of :meth:`from_dict`)."""
        layers = []
        for b in self.blocks:
            m = b.mixer
            if b.type == "mlstm":
                mx = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap}
            else:
                rot = {"base": m.rot.base, "dims": m.rot.dims}
                if m.rot.yarn:
                    rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), m.rot.yarn))
                mx = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale, "rot": rot}
                if m.softcap:
                    mx["softcap"] = m.softcap
            f = b.mlp
            if isinstance(f, GroupedMoeSpec):
                router = {"experts": f.experts, "top": f.top, "identity": f.identity, "scale": f.scale}
                if f.groups > 1:
                    router["groups"] = {"count": f.groups, "keep": f.keep}
                ff = {"kind": "moe", "router": router, "expert": {"ff": f.expert.ff}}
                if f.shared is not None:
                    ff["shared"] = {"ff": f.shared.ff}
            elif f is not None:
                ff = {"kind": "dense", "ff": f.ff}
            else:
                ff = None
            layers.append({"type": b.type, "mixer": mx, "mlp": ff})
        out = {"architecture": "Lizezen", "vocab": self.vocab_size, "width": self.hidden, "norm": {"eps": self.eps},
               "layers": layers}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out

    def to_dict(self):
        return asdict(self)


def lizezen_layers(pattern: Sequence[str], hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, ff: int,
                   mlstm_heads: int = 0, mlstm_dim: int = 0, mlstm_vdim: int = 0, experts: int = 0, top: int = 2,
                   expert_ff: int = 0, shared_ff: int = 0, identity: int = 0, groups: int = 1, keep: int = 1,
                   route_scale: float = 1.0, softcap: float = 0.0, gate_cap: float = 15.0, rot_base: float = 10000.0,
                   rot_dims: int = 0, yarn: Optional[tuple] = None, loop: Optional[tuple] = None,
                   vocab_size: int = 32768, eps: float = 1e-5, name: str = "lizezen") -> LizezenConfig:
    """A Lizezen config from a pattern of mixer types with the same sizes in every layer of a
    kind (benchmarks, tests). ``experts`` > 0: every second feed-forward is a mixture (the others
    dense of ``ff``; ``ff`` 0: none). ``loop`` = (start, stop, times)."""
    blocks = []
    for i, t in enumerate(pattern):
        if t == "mlstm":
            m = MlstmSpec(mlstm_heads or heads, mlstm_dim or dim, mlstm_vdim or vdim, gate_cap)
        elif t in ("attention", "attention_2"):
            second = t == "attention_2"
            rot = RotarySpec(rot_dims or dim, rot_base, False, yarn if second else None)
            m = RotaryAttentionSpec(heads, kv_heads, dim, dim if second else vdim, dim ** -0.5, rot,
                                    softcap if second else 0.0, second, second, second)
        else:
            raise ValueError(f"unknown mixer type {t!r}")
        if experts and i % 2:
            mlp = GroupedMoeSpec(experts, top, SwigluSpec(expert_ff), identity, route_scale, groups, keep,
                                 SwigluSpec(shared_ff) if shared_ff else None)
        else:
            mlp = GeluMlpSpec(ff) if ff else None
        blocks.append(LizezenLayer(t, m, mlp))
    return LizezenConfig(name=name, vocab_size=vocab_size, hidden=hidden, eps=eps, blocks=tuple(blocks),
                         loop=None if not loop else LoopSpec(*loop))
