"""Model and engine configuration.

The reference serves ``meta-llama/Llama-3.1-8B-Instruct`` through vLLM with the knobs in
infra/docker-compose.yml:16-27 (dtype float16, max_num_seqs 12, max_num_batched_tokens
8192, gpu_memory_utilization 0.90, max_model_len 4096) and KV blocks of 16 tokens
(llm/serve_llm.py:325).  ``EngineConfig`` keeps those names and defaults; the MI355X
specific additions (tensor/data parallel degree, hipGraph buckets, decode partitioning)
default to values sized for 288 GB of HBM3E per GPU.
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, field, replace
from pathlib import Path

LLAMA3_ROPE_SCALING = {
    "rope_type": "llama3",
    "factor": 8.0,
    "low_freq_factor": 1.0,
    "high_freq_factor": 4.0,
    "original_max_position_embeddings": 8192,
}


@dataclass(frozen=True)
class ModelConfig:
    name: str = "llama-3.1-8b"
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: dict | None = field(default_factory=lambda: dict(LLAMA3_ROPE_SCALING))
    max_position_embeddings: int = 131072
    tie_word_embeddings: bool = False
    bos_token_id: int = 128000
    eos_token_ids: tuple = (128001, 128008, 128009)
    family: str = "llama"

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def num_params(self) -> int:
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        per_layer = h * (self.q_size + 2 * self.kv_size) + self.q_size * h + 3 * h * i + 2 * h
        emb = v * h * (1 if self.tie_word_embeddings else 2)
        return self.num_layers * per_layer + emb + h

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return self.num_layers * 2 * self.num_kv_heads * self.head_dim * dtype_bytes


MODEL_PRESETS: dict[str, ModelConfig] = {
    "llama-3.1-8b": ModelConfig(),
    "llama-3-8b": ModelConfig(name="llama-3-8b", rope_scaling=None, max_position_embeddings=8192,
                              eos_token_ids=(128001, 128009)),
    "llama-3-70b": ModelConfig(name="llama-3-70b", hidden_size=8192, intermediate_size=28672,
                               num_layers=80, num_heads=64, num_kv_heads=8, rope_scaling=None,
                               max_position_embeddings=8192, eos_token_ids=(128001, 128009)),
    "llama-3.1-70b": ModelConfig(name="llama-3.1-70b", hidden_size=8192, intermediate_size=28672,
                                 num_layers=80, num_heads=64, num_kv_heads=8),
    "llama-3.2-3b": ModelConfig(name="llama-3.2-3b", hidden_size=3072, intermediate_size=8192,
                                num_layers=28, num_heads=24, num_kv_heads=8,
                                tie_word_embeddings=True,
                                rope_scaling=dict(LLAMA3_ROPE_SCALING, factor=32.0)),
    "llama-3.2-1b": ModelConfig(name="llama-3.2-1b", hidden_size=2048, intermediate_size=8192,
                                num_layers=16, num_heads=32, num_kv_heads=8, head_dim=64,
                                tie_word_embeddings=True,
                                rope_scaling=dict(LLAMA3_ROPE_SCALING, factor=32.0)),
    # small shapes for tests / CPU plumbing runs (head_dim 128 like every Llama-3 >= 3B)
    "tiny": ModelConfig(name="tiny", vocab_size=4096, hidden_size=256, intermediate_size=512,
                        num_layers=2, num_heads=4, num_kv_heads=2, max_position_embeddings=4096,
                        bos_token_id=3840, eos_token_ids=(3841, 3849)),
    "small": ModelConfig(name="small", vocab_size=32768, hidden_size=1024, intermediate_size=2816,
                         num_layers=4, num_heads=8, num_kv_heads=2, max_position_embeddings=8192,
                         bos_token_id=32512, eos_token_ids=(32513, 32521)),
    # long-context tests: the "small" shape with a 32k RoPE table (reference .env runs 11k)
    "small-32k": ModelConfig(name="small-32k", vocab_size=32768, hidden_size=1024,
                             intermediate_size=2816, num_layers=4, num_heads=8, num_kv_heads=2,
                             max_position_embeddings=32768, bos_token_id=32512,
                             eos_token_ids=(32513, 32521)),
    # TP rehearsal shape: 8 q heads over 2 KV heads, so TP=4/8 replicate KV heads (kv_rep > 1)
    "tiny-tp8": ModelConfig(name="tiny-tp8", vocab_size=4096, hidden_size=256,
                            intermediate_size=512, num_layers=2, num_heads=8, num_kv_heads=2,
                            max_position_embeddings=4096, bos_token_id=3840,
                            eos_token_ids=(3841, 3849)),
    # 70B attention geometry (GQA 8:1, hidden 8192) with few layers / a small FFN and vocab:
    # the G=8 decode path and 8192-wide GEMVs on one GPU in seconds
    # Llama-3.2-3B geometry (reference infra/.env.example:116): hidden 3072, 24 q / 8 kv heads
    # (GQA G = 3), tied embeddings - 2 layers and a small vocab for GPU tests
    "llama-3b-slice": ModelConfig(name="llama-3b-slice", vocab_size=16384, hidden_size=3072,
                                  intermediate_size=8192, num_layers=2, num_heads=24,
                                  num_kv_heads=8, tie_word_embeddings=True,
                                  rope_scaling=dict(LLAMA3_ROPE_SCALING, factor=32.0),
                                  bos_token_id=16000, eos_token_ids=(16001, 16009)),
    # the Llama-3.1-8B layer geometry (hidden 4096, 32 q / 8 kv heads, FFN 14336) with 2
    # layers and a small vocab: the persistent decode step's shapes on one GPU in seconds
    "llama-8b-slice": ModelConfig(name="llama-8b-slice", vocab_size=16384, hidden_size=4096,
                                  intermediate_size=14336, num_layers=2, num_heads=32,
                                  num_kv_heads=8, max_position_embeddings=16384,
                                  bos_token_id=16000, eos_token_ids=(16001, 16009)),
    # the Llama-3-70B TP=8 per-rank geometry (one KV head and 8 q heads per rank, hidden 8192)
    # with an FFN that stays fused-decode-shaped at TP=2/4/8 (7168 / 8 = 896 = 7 x 128): the
    # one-GPU TP rehearsal of graph-captured decode
    "llama-70b-tp-slice": ModelConfig(name="llama-70b-tp-slice", vocab_size=16384,
                                      hidden_size=8192, intermediate_size=7168, num_layers=2,
                                      num_heads=64, num_kv_heads=8, rope_scaling=None,
                                      max_position_embeddings=16384, bos_token_id=16000,
                                      eos_token_ids=(16001, 16009)),
    # the same per-rank geometry for fp8 weights (BASELINE config 5): the fp8 GEMVs stream K in
    # 256-wide steps (4 waves x 64), so the FFN shard must be a multiple of 256 at TP=8 - the
    # real 70B's 28672 / 8 = 3584 is; this slice's 14336 / 8 = 1792 = 7 x 256 is too
    "llama-70b-tp-slice-fp8": ModelConfig(name="llama-70b-tp-slice-fp8", vocab_size=16384,
                                          hidden_size=8192, intermediate_size=14336,
                                          num_layers=2, num_heads=64, num_kv_heads=8,
                                          rope_scaling=None, max_position_embeddings=16384,
                                          bos_token_id=16000, eos_token_ids=(16001, 16009)),
    "llama-70b-slice": ModelConfig(name="llama-70b-slice", vocab_size=16384, hidden_size=8192,
                                   intermediate_size=3584, num_layers=2, num_heads=64,
                                   num_kv_heads=8, rope_scaling=None,
                                   max_position_embeddings=16384, bos_token_id=16000,
                                   eos_token_ids=(16001, 16009)),
}


# ---------------------------------------------------------------------------------------
# Hybrid decoders: per-layer lists of sequence mixers (softmax attention over the paged KV
# cache and / or a recurrent gated delta rule with per-sequence state slots).

@dataclass(frozen=True)
class SoftmaxMixerConfig:
    """Grouped-query softmax attention with per-head q/k RMS norm, interleaved-pair rotary
    positions on the first ``rot_dims`` channels and (``sink``) one extra zero-score,
    value-less key in every softmax denominator."""
    heads: int
    kv_heads: int
    dim: int          # per-head query / key width
    vdim: int         # per-head value width
    rot_dims: int
    rot_base: float
    scale: float
    sink: bool = True


@dataclass(frozen=True)
class DeltaMixerConfig:
    """Gated delta rule: ``kv_heads`` query / key heads of ``dim`` channels shared by groups of
    ``heads`` value heads of ``vdim`` channels, short causal convolutions of ``conv`` taps on
    q, k and v.  ``channel_decay``: one decay per head and key channel from a low-rank pair of
    projections (and a low-rank sigmoid output gate); otherwise one decay per head and a
    full-rank SiLU output gate."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    channel_decay: bool = False
    decay_rank: int = 0   # rows of the first low-rank decay projection (channel_decay)
    gate_rank: int = 0    # rows of the first low-rank gate projection (channel_decay)


@dataclass(frozen=True)
class HybridLayerConfig:
    kind: str                                  # "delta" | "parallel"
    softmax: SoftmaxMixerConfig | None = None
    delta: DeltaMixerConfig | None = None
    softmax_scale: float = 1.0                 # weights of the two branches of a parallel layer
    delta_scale: float = 1.0
    ff: int = 0                                # feed-forward width, 0 = no feed-forward
    ff_kind: str = "dense"


@dataclass(frozen=True)
class LedazenConfig:
    """Ledazen: parallel-residual decoder (one norm per layer feeding the mixer and a
    squared-ReLU feed-forward side by side), hashed token-pair embedding added to the token
    embedding, fp32 residual stream."""
    name: str = "ledazen"
    vocab_size: int = 1024
    hidden_size: int = 256
    layers: tuple = ()
    rms_norm_eps: float = 1e-5
    pair_buckets: int = 0
    pair_mul_prev: int = 0
    pair_mul_cur: int = 0
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    max_position_embeddings: int = 1 << 20
    family: str = "ledazen"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def from_dict(c: dict, name: str = "ledazen") -> "LedazenConfig":
        """Parse the checkpoint's config.json (keys: vocab, width, norm.eps,
        embedding.bigram.{buckets,mul_prev,mul_cur}, layers[].{type,mixer,mlp})."""

        def delta(m: dict, channel: bool) -> DeltaMixerConfig:
            return DeltaMixerConfig(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                                    dim=int(m["dim"]), vdim=int(m["vdim"]),
                                    conv=int(m["conv"]), channel_decay=channel)

        def softmax(m: dict) -> SoftmaxMixerConfig:
            return SoftmaxMixerConfig(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                                      dim=int(m["dim"]), vdim=int(m["vdim"]),
                                      rot_dims=int(m["rot"]["dims"]),
                                      rot_base=float(m["rot"]["base"]), scale=float(m["scale"]))

        layers = []
        for L in c["layers"]:
            mlp = L.get("mlp")
            ff, kind = (int(mlp["ff"]), str(mlp.get("kind", "dense"))) if mlp else (0, "dense")
            if kind != "dense":
                raise ValueError(f"unsupported feed-forward kind {kind!r}")
            m = L["mixer"]
            if L["type"] == "delta":
                layers.append(HybridLayerConfig("delta", delta=delta(m, False), ff=ff))
            elif L["type"] == "parallel":
                layers.append(HybridLayerConfig(
                    "parallel", softmax=softmax(m["left"]), delta=delta(m["right"], True),
                    softmax_scale=float(m["left_scale"]), delta_scale=float(m["right_scale"]),
                    ff=ff))
            else:
                raise ValueError(f"unknown layer type {L['type']!r}")
        bg = c["embedding"]["bigram"]
        return LedazenConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                             layers=tuple(layers), rms_norm_eps=float(c["norm"]["eps"]),
                             pair_buckets=int(bg["buckets"]), pair_mul_prev=int(bg["mul_prev"]),
                             pair_mul_cur=int(bg["mul_cur"]))


def ledazen_preset(name: str, vocab: int, width: int, ff: int, pattern: str, heads: int,
                   kv_heads: int, dim: int, vdim: int, delta_heads: int, delta_kv_heads: int,
                   delta_dim: int, delta_vdim: int, low_rank: int = 0) -> LedazenConfig:
    """A Ledazen shape for benchmarks and tests: ``pattern`` is one letter per layer, ``p`` a
    parallel layer (softmax + channel-decay delta branch), ``d`` a delta layer."""
    sm = SoftmaxMixerConfig(heads, kv_heads, dim, vdim, rot_dims=dim, rot_base=1000000.0,
                            scale=dim ** -0.5)
    rank = low_rank or max(16, width // 16)
    layers = []
    for ch in pattern:
        if ch == "p":
            layers.append(HybridLayerConfig(
                "parallel", softmax=sm,
                delta=DeltaMixerConfig(delta_heads, delta_kv_heads, delta_dim, delta_vdim, 4, True,
                                       rank, rank),
                softmax_scale=0.75, delta_scale=0.6, ff=ff))
        else:
            layers.append(HybridLayerConfig(
                "delta", delta=DeltaMixerConfig(delta_heads, delta_kv_heads, delta_dim,
                                                delta_vdim, 4, False), ff=ff))
    return LedazenConfig(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers),
                         pair_buckets=max(7, vocab // 2 - 1), pair_mul_prev=37, pair_mul_cur=11)


HYBRID_PRESETS: dict[str, LedazenConfig] = {
    # plumbing shape for the CPU tier (odd group sizes, value width != key width)
    "ledazen-tiny": ledazen_preset("ledazen-tiny", 512, 128, 192, "pdp", 4, 2, 32, 16, 4, 2, 16,
                                   32, low_rank=8),
    # the "small" Llama preset's geometry (width 1024, 8 q / 2 kv heads of 128, FFN 2816, 4 layers)
    "ledazen-small": ledazen_preset("ledazen-small", 32768, 1024, 2816, "pdpd", 8, 2, 128, 128,
                                    8, 2, 128, 128),
    # Llama-3.2-3B layer geometry (width 3072, 24 q / 8 kv heads of 128, FFN 8192), 2 layers
    "ledazen-3b-slice": ledazen_preset("ledazen-3b-slice", 16384, 3072, 8192, "pd", 24, 8, 128,
                                       128, 24, 8, 128, 128),
    # Llama-3.1-8B layer geometry (width 4096, 32 q / 8 kv heads of 128, FFN 14336), 2 layers
    "ledazen-8b-slice": ledazen_preset("ledazen-8b-slice", 16384, 4096, 14336, "pd", 32, 8, 128,
                                       128, 32, 8, 128, 128),
}

# config.json "architecture" -> parser of that design's configuration
ARCHITECTURES = {"Ledazen": LedazenConfig.from_dict}


# ---------------------------------------------------------------------------------------
# Soselix: pre-norm decoder whose layers pick one of three mixers - latent attention over a
# compressed, optionally shared K / V cache, an HGRN2 forget-gate recurrence or a Mamba-2
# state-space recurrence - followed by a biased xIELU feed-forward.

@dataclass(frozen=True)
class LatentAttentionConfig:
    """Softmax attention whose keys and values are up-projected from one cached latent of
    ``kv_rank`` channels per token plus ``rot_dim`` rotated key channels shared by all heads;
    queries go through a ``q_rank`` latent; a learned sink score per head; a sigmoid output
    gate per head.  ``kv_from`` >= 0: the layer has no down-projection and reads that layer's
    cached latent and rotated key."""
    heads: int
    dim: int          # unrotated query / key channels per head
    rot_dim: int      # rotated query / key channels per head
    vdim: int
    kv_rank: int
    q_rank: int
    rot_dims: int     # leading channels of the rotated part that actually rotate
    rot_base: float
    scale: float
    kv_from: int = -1


@dataclass(frozen=True)
class Hgrn2Config:
    """Linear attention with a per-channel forget gate that is also the write gate."""
    heads: int
    dim: int
    vdim: int


@dataclass(frozen=True)
class Mamba2Config:
    """State-space duality layer: ``heads`` of ``vdim`` channels, ``state`` rows per head, B / C
    shared by ``groups``, a causal convolution of ``conv`` taps, output norm in ``norm_groups``."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass(frozen=True)
class SoselixLayerConfig:
    kind: str                 # "latent_attention" | "hgrn2" | "mamba2"
    mixer: object = None
    ff: int = 0               # feed-forward width, 0 = no feed-forward
    ff_kind: str = "dense"


@dataclass(frozen=True)
class SoselixConfig:
    name: str = "soselix"
    vocab_size: int = 1024
    hidden_size: int = 256
    layers: tuple = ()
    rms_norm_eps: float = 1e-6
    embed_scale: float = 1.0
    residual_mult: float = 1.0
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    max_position_embeddings: int = 1 << 20
    family: str = "soselix"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def from_dict(c: dict, name: str = "soselix") -> "SoselixConfig":
        """Parse the checkpoint's config.json (keys: vocab, width, norm.eps, embedding.scale,
        residual_mult, layers[].{type,mixer,mlp})."""
        layers = []
        for i, L in enumerate(c["layers"]):
            mlp = L.get("mlp")
            ff, kind = (int(mlp["ff"]), str(mlp.get("kind", "dense"))) if mlp else (0, "dense")
            if kind != "dense":
                raise ValueError(f"unsupported feed-forward kind {kind!r}")
            m, t = L["mixer"], L["type"]
            if t == "latent_attention":
                rot = m.get("rot") or {}
                rot_dim = int(m["rot_dim"])
                mc = LatentAttentionConfig(
                    heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim,
                    vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]), q_rank=int(m.get("q_rank", 0)),
                    rot_dims=int(rot.get("dims", rot_dim)), rot_base=float(rot.get("base", 10000.0)),
                    scale=float(m["scale"]), kv_from=int(m["kv_from"]) if "kv_from" in m else -1)
                if mc.rot_dims > mc.rot_dim or mc.rot_dims % 2:
                    raise ValueError(f"layer {i}: rot.dims must be even and <= rot_dim")
                if mc.kv_from >= 0:
                    src = layers[mc.kv_from].mixer if mc.kv_from < i else None
                    if not isinstance(src, LatentAttentionConfig) or src.kv_from >= 0 or \
                            (src.kv_rank, src.rot_dim, src.rot_dims, src.rot_base) != \
                            (mc.kv_rank, mc.rot_dim, mc.rot_dims, mc.rot_base):
                        raise ValueError(f"layer {i}: kv_from must name an earlier latent-attention "
                                         "layer with its own cache and the same latent geometry")
            elif t == "hgrn2":
                mc = Hgrn2Config(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]))
            elif t == "mamba2":
                mc = Mamba2Config(heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]),
                                  groups=int(m.get("groups", 1)), conv=int(m["conv"]),
                                  norm_groups=int(m.get("norm_groups", 1)))
                if mc.heads % mc.groups or mc.inner % mc.norm_groups:
                    raise ValueError(f"layer {i}: heads % groups and inner % norm_groups must be 0")
            else:
                raise ValueError(f"unknown layer type {t!r}")
            layers.append(SoselixLayerConfig(t, mc, ff, kind))
        return SoselixConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                             layers=tuple(layers), rms_norm_eps=float(c["norm"]["eps"]),
                             embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                             residual_mult=float(c.get("residual_mult", 1.0)))


def soselix_preset(name: str, vocab: int, width: int, ff: int, pattern: str, heads: int,
                   head_dim: int, kv_rank: int, q_rank: int, rot_dim: int = 64,
                   state: int = 128) -> SoselixConfig:
    """A Soselix shape for benchmarks and tests: one letter per layer, ``a`` latent attention,
    ``s`` latent attention on the first ``a`` layer's cache, ``h`` HGRN2, ``m`` Mamba-2."""
    layers, first_a = [], -1
    for i, ch in enumerate(pattern):
        if ch in "as":
            share = first_a if ch == "s" else -1
            mc = LatentAttentionConfig(heads, head_dim, rot_dim, head_dim, kv_rank, q_rank, rot_dim,
                                       10000.0, (head_dim + rot_dim) ** -0.5, share)
            if ch == "a" and first_a < 0:
                first_a = i
            layers.append(SoselixLayerConfig("latent_attention", mc, ff))
        elif ch == "h":
            layers.append(SoselixLayerConfig("hgrn2", Hgrn2Config(heads, head_dim, head_dim), ff))
        else:
            mh = max(1, 2 * width // 64)
            layers.append(SoselixLayerConfig(
                "mamba2", Mamba2Config(mh, 64, state, max(1, min(8, mh // 8)), 4, 1), ff))
    return SoselixConfig(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers),
                         embed_scale=1.0, residual_mult=1.0)


HYBRID_PRESETS.update({
    "soselix-tiny": soselix_preset("soselix-tiny", 512, 128, 192, "mahs", 4, 16, 32, 48, 8, 16),
    # the "small" Llama preset's geometry (width 1024, 8 heads of 128, FFN 2816, 4 layers)
    "soselix-small": soselix_preset("soselix-small", 32768, 1024, 2816, "mahs", 8, 128, 192, 384),
    # Llama-3.2-3B / Llama-3.1-8B layer geometry, one layer per mixer
    "soselix-3b-slice": soselix_preset("soselix-3b-slice", 16384, 3072, 8192, "mah", 24, 128, 192,
                                       768),
    "soselix-8b-slice": soselix_preset("soselix-8b-slice", 16384, 4096, 14336, "mah", 32, 128,
                                       192, 1024),
})
ARCHITECTURES["Soselix"] = SoselixConfig.from_dict


# ---------------------------------------------------------------------------------------
# Semezen: pre-norm decoder on several residual streams (hyper-connections) whose mixers read a
# token-shifted input; a layer's mixer is sliding-window attention whose values are its keys, or
# a minGRU recurrence; its feed-forward is a dense GELU layer or a mixture of clamped-GLU experts.

@dataclass(frozen=True)
class WindowAttentionConfig:
    """Grouped-query softmax attention with biased q / k projections, values = the projected
    keys (before rotation and norm), rotate-half positions on the first ``rot_dims`` channels with
    optional wavelength-dependent frequency scaling ``rot_scaling`` = (factor, low, high,
    original), weightless per-head RMS norm of q and k after the rotation, a sliding window of
    ``window`` keys (0: all earlier keys) and an element-wise sigmoid output gate."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: tuple | None = None


@dataclass(frozen=True)
class MinGruConfig:
    """Element-wise gated recurrence of ``width`` channels whose gates read only the current
    token."""
    width: int


@dataclass(frozen=True)
class MoeConfig:
    """``experts`` clamped-GLU feed-forward layers of width ``ff``; a token runs its ``top`` best
    by sigmoid router score, the score scaling the expert's input."""
    experts: int
    top: int
    ff: int
    limit: float
    act_alpha: float = 1.702


@dataclass(frozen=True)
class SemezenLayerConfig:
    kind: str                 # "attention" | "mingru"
    mixer: object = None
    ff: int = 0               # dense feed-forward width (0: none, or see ``moe``)
    moe: MoeConfig | None = None
    ff_act: str = "gelu"      # dense activation: "gelu" (erf) or "gelu_tanh"


@dataclass(frozen=True)
class SemezenConfig:
    name: str = "semezen"
    vocab_size: int = 1024
    hidden_size: int = 256
    layers: tuple = ()
    rms_norm_eps: float = 1e-6
    streams: int = 1
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    max_position_embeddings: int = 1 << 20
    family: str = "semezen"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def from_dict(c: dict, name: str = "semezen") -> "SemezenConfig":
        """Parse the checkpoint's config.json (keys: vocab, width, norm.eps, streams,
        layers[].{type, mixer, mlp}; attention: heads, kv_heads, dim, vdim, scale, mask.size,
        rot.{dims, base, scaling.{factor, low, high, original}}; mingru: width; mlp: kind dense
        {ff} or moe {expert.{ff, limit}, router.{experts, top}})."""
        layers = []
        for i, L in enumerate(c["layers"]):
            m, t = L["mixer"], L["type"]
            if t == "attention":
                rot = m.get("rot") or {}
                sc = rot.get("scaling")
                mc = WindowAttentionConfig(
                    heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                    dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                    window=int((m.get("mask") or {}).get("size") or 0),
                    rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                    rot_scaling=(float(sc["factor"]), float(sc["low"]), float(sc["high"]),
                                 float(sc["original"])) if sc else None)
                if mc.heads % mc.kv_heads:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                if mc.vdim != mc.dim:
                    raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
                if mc.rot_dims % 2 or mc.rot_dims > mc.dim:
                    raise ValueError(f"layer {i}: rot.dims must be even and <= dim")
            elif t == "mingru":
                mc = MinGruConfig(width=int(m["width"]))
            else:
                raise ValueError(f"unknown layer type {t!r}")
            mlp = L.get("mlp")
            ff, moe, act = 0, None, "gelu"
            if mlp:
                kind = str(mlp.get("kind", "dense"))
                if kind == "dense":
                    ff, act = int(mlp["ff"]), str(mlp.get("act", "gelu"))
                    if act not in ("gelu", "gelu_tanh"):
                        raise ValueError(f"layer {i}: unknown activation {act!r}")
                elif kind == "moe":
                    moe = MoeConfig(experts=int(mlp["router"]["experts"]),
                                    top=int(mlp["router"]["top"]), ff=int(mlp["expert"]["ff"]),
                                    limit=float(mlp["expert"]["limit"]))
                    if not 1 <= moe.top <= moe.experts:
                        raise ValueError(f"layer {i}: router.top must be in [1, experts]")
                else:
                    raise ValueError(f"unsupported feed-forward kind {kind!r}")
            layers.append(SemezenLayerConfig(t, mc, ff, moe, act))
        return SemezenConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                             layers=tuple(layers), rms_norm_eps=float(c["norm"]["eps"]),
                             streams=int(c.get("streams", 1)))


def semezen_preset(name: str, vocab: int, width: int, ff: int, pattern: str, heads: int,
                   kv_heads: int, dim: int, window: int, experts: int = 8, top: int = 2,
                   expert_ff: int = 0, streams: int = 2) -> SemezenConfig:
    """A Semezen shape for benchmarks and tests: two letters per layer, mixer (``a`` window
    attention, ``g`` minGRU) then feed-forward (``d`` dense, ``e`` experts, ``-`` none)."""
    layers = []
    for j in range(0, len(pattern), 2):
        mx_, f = pattern[j], pattern[j + 1]
        mc = (WindowAttentionConfig(heads, kv_heads, dim, dim, dim ** -0.5, window, dim // 2,
                                    500000.0, (8.0, 1.0, 4.0, 8192.0))
              if mx_ == "a" else MinGruConfig(heads * dim))
        layers.append(SemezenLayerConfig(
            "attention" if mx_ == "a" else "mingru", mc, ff if f == "d" else 0,
            MoeConfig(experts, top, expert_ff or max(8, ff // max(1, top)), 7.0)
            if f == "e" else None))
    return SemezenConfig(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers),
                         streams=streams)


HYBRID_PRESETS.update({
    "semezen-tiny": semezen_preset("semezen-tiny", 512, 128, 192, "adgeae", 4, 2, 32, 24, 6, 2,
                                   48, 3),
    # the "small" Llama preset's geometry (width 1024, 8 q / 2 kv heads of 128, FFN 2816, 4 layers)
    "semezen-small": semezen_preset("semezen-small", 32768, 1024, 2816, "adgeadge", 8, 2, 128,
                                    1024, 8, 2, 1408),
    # Llama-3.2-3B / Llama-3.1-8B layer geometry, one attention + dense and one minGRU + experts
    "semezen-3b-slice": semezen_preset("semezen-3b-slice", 16384, 3072, 8192, "adge", 24, 8, 128,
                                       1024, 8, 2, 4096),
    "semezen-8b-slice": semezen_preset("semezen-8b-slice", 16384, 4096, 14336, "adge", 32, 8, 128,
                                       1024, 8, 2, 7168),
})
ARCHITECTURES["Semezen"] = SemezenConfig.from_dict


# ---------------------------------------------------------------------------------------
# Lovapel: decoder with a layer norm before AND after every sub-layer, sliding-window attention
# with a learned sink per head and q / k norms over the whole projection, dense GELU-GLU layers or
# grouped-choice routed experts (with identity experts and a shared expert), a span of layers
# that runs several times with the same weights, tied and soft-capped output logits.

@dataclass(frozen=True)
class SinkWindowAttentionConfig:
    """Grouped-query softmax attention: q and k RMS-normed over their WHOLE projection (all heads
    at once, one weight per row of the projection) before the rotation, rotate-half positions on
    the first ``rot_dims`` channels of every head, a sliding window of ``window`` keys (0: all
    earlier keys) and one learned sink score per query head in the softmax denominator."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0


@dataclass(frozen=True)
class GroupedMoeConfig:
    """``experts`` SiLU-GLU feed-forward layers of width ``ff`` plus ``identity`` experts without
    weights that return their input.  The router's softmax scores (plus a stored correction,
    used for the choice only) pick ``top`` experts inside the ``keep`` best of ``groups`` equal
    runs of neighbours; the chosen scores, normalised to sum 1, weight the outputs.  A shared
    expert of width ``shared_ff`` (0: none) runs for every token."""
    experts: int
    top: int
    ff: int
    identity: int = 0
    groups: int = 1
    keep: int = 1
    shared_ff: int = 0

    @property
    def routes(self) -> int:
        return self.experts + self.identity


@dataclass(frozen=True)
class LovapelLayerConfig:
    kind: str                 # "attention"
    mixer: object = None
    ff: int = 0               # dense GELU-GLU width (0: none, or see ``moe``)
    moe: GroupedMoeConfig | None = None


@dataclass(frozen=True)
class LovapelConfig:
    name: str = "lovapel"
    vocab_size: int = 1024
    hidden_size: int = 256
    layers: tuple = ()
    norm_eps: float = 1e-5
    loop_start: int = 0       # layers [loop_start, loop_stop) run loop_times times in a row
    loop_stop: int = 0
    loop_times: int = 1
    logit_scale: float = 1.0
    logit_softcap: float = 0.0   # 0: none
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    max_position_embeddings: int = 1 << 20
    family: str = "lovapel"

    @property
    def runs(self) -> tuple:
        """Layer index of every layer run, in order; a run has a cache of its own."""
        a, b = self.loop_start, self.loop_stop
        n = len(self.layers)
        return tuple(range(a)) + tuple(range(a, b)) * self.loop_times + tuple(range(b, n))

    @property
    def num_layers(self) -> int:
        return len(self.runs)

    @property
    def rms_norm_eps(self) -> float:
        return self.norm_eps

    def __post_init__(self):
        n = len(self.layers)
        if not (0 <= self.loop_start <= self.loop_stop <= n) or self.loop_times < 1:
            raise ValueError("loop: need 0 <= start <= stop <= layers and times >= 1")

    @staticmethod
    def from_dict(c: dict, name: str = "lovapel") -> "LovapelConfig":
        """Parse the checkpoint's config.json (keys: vocab, width, norm.eps, logit_scale,
        logit_softcap, loop.{start, stop, times}, layers[].{type, mixer, mlp}; attention: heads,
        kv_heads, dim, vdim, scale, mask.size, rot.{dims, base}; mlp: kind dense {ff} or moe
        {expert.ff, router.{experts, identity, top, groups.{count, keep}}, shared.ff}).  An absent
        loop, mask, rot, softcap, groups, identity or shared means none."""
        layers = []
        for i, L in enumerate(c["layers"]):
            m, t = L["mixer"], L["type"]
            if t != "attention":
                raise ValueError(f"unknown layer type {t!r}")
            rot = m.get("rot") or {}
            mc = SinkWindowAttentionConfig(
                heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                window=int((m.get("mask") or {}).get("size") or 0),
                rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)))
            if mc.heads % mc.kv_heads:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            if mc.rot_dims % 2 or mc.rot_dims > mc.dim:
                raise ValueError(f"layer {i}: rot.dims must be even and <= dim")
            mlp = L.get("mlp")
            ff, moe = 0, None
            if mlp:
                kind = str(mlp.get("kind", "dense"))
                if kind == "dense":
                    ff = int(mlp["ff"])
                elif kind == "moe":
                    r = mlp["router"]
                    g = r.get("groups") or {}
                    groups = int(g.get("count", 1))
                    moe = GroupedMoeConfig(
                        experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                        identity=int(r.get("identity", 0)), groups=groups,
                        keep=int(g.get("keep", groups)),
                        shared_ff=int((mlp.get("shared") or {}).get("ff", 0)))
                    if moe.groups < 1 or moe.routes % moe.groups:
                        raise ValueError(f"layer {i}: the experts do not split into equal groups")
                    if not 1 <= moe.keep <= moe.groups:
                        raise ValueError(f"layer {i}: groups.keep must be in [1, groups.count]")
                    if not 1 <= moe.top <= moe.keep * (moe.routes // moe.groups):
                        raise ValueError(f"layer {i}: router.top exceeds the experts of the kept groups")
                else:
                    raise ValueError(f"unsupported feed-forward kind {kind!r}")
            layers.append(LovapelLayerConfig(t, mc, ff, moe))
        loop = c.get("loop") or {}
        return LovapelConfig(
            name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
            layers=tuple(layers), norm_eps=float(c["norm"]["eps"]),
            loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
            loop_times=int(loop.get("times", 1)), logit_scale=float(c.get("logit_scale", 1.0)),
            logit_softcap=float(c.get("logit_softcap") or 0.0))


def lovapel_preset(name: str, vocab: int, width: int, ff: int, pattern: str, heads: int,
                   kv_heads: int, dim: int, window: int, experts: int = 8, top: int = 2,
                   expert_ff: int = 0, identity: int = 0, groups: int = 1, keep: int = 1,
                   shared_ff: int = 0, loop: tuple = (0, 0, 1)) -> LovapelConfig:
    """A Lovapel shape for benchmarks and tests: one letter per layer for its feed-forward
    (``d`` dense, ``e`` experts, ``-`` none); every mixer is the sink-window attention."""
    mc = SinkWindowAttentionConfig(heads, kv_heads, dim, dim, dim ** -0.5, window, dim // 2,
                                   500000.0)
    layers = tuple(LovapelLayerConfig(
        "attention", mc, ff if f == "d" else 0,
        GroupedMoeConfig(experts, top, expert_ff or max(8, ff // max(1, top)), identity, groups,
                         keep, shared_ff) if f == "e" else None) for f in pattern)
    return LovapelConfig(name=name, vocab_size=vocab, hidden_size=width, layers=layers,
                         loop_start=loop[0], loop_stop=loop[1], loop_times=loop[2],
                         logit_scale=0.5, logit_softcap=30.0)


HYBRID_PRESETS.update({
    "lovapel-tiny": lovapel_preset("lovapel-tiny", 512, 128, 192, "ded", 4, 2, 32, 24, 6, 2, 48,
                                   2, 4, 2, 40, (1, 3, 2)),
    # the "small" Llama preset's geometry (width 1024, 8 q / 2 kv heads of 128, FFN 2816, 4 layers)
    "lovapel-small": lovapel_preset("lovapel-small", 32768, 1024, 2816, "dede", 8, 2, 128, 1024,
                                    8, 2, 1408, 0, 2, 1, 704),
    # Llama-3.2-3B / Llama-3.1-8B layer geometry, one dense layer and one with experts
    "lovapel-3b-slice": lovapel_preset("lovapel-3b-slice", 16384, 3072, 8192, "de", 24, 8, 128,
                                       1024, 8, 2, 4096, 0, 2, 1, 2048),
    "lovapel-8b-slice": lovapel_preset("lovapel-8b-slice", 16384, 4096, 14336, "de", 32, 8, 128,
                                       1024, 8, 2, 7168, 0, 2, 1, 3584),
})
ARCHITECTURES["Lovapel"] = LovapelConfig.from_dict


def resolve_model(model: str) -> tuple[ModelConfig, str | None]:
    """Map a reference-style model id (``meta-llama/Llama-3.1-8B-Instruct``), a preset name
    or a local HF directory (config.json [+ *.safetensors]) to a ModelConfig.
    Returns (config, weights_dir or None)."""
    p = Path(model)
    if p.is_dir() and (p / "config.json").exists():
        c = json.loads((p / "config.json").read_text())
        arch = c.get("architecture")
        if arch in ARCHITECTURES:
            return ARCHITECTURES[arch](c, name=p.name or arch.lower()), str(p)
        return config_from_hf(p / "config.json"), str(p)
    key = model.lower().split("/")[-1]
    if key in HYBRID_PRESETS:
        return HYBRID_PRESETS[key], None
    if key in MODEL_PRESETS:
        return MODEL_PRESETS[key], None
    for k in ("3.1-70b", "3.2-3b", "3.2-1b", "3-70b", "3.1-8b", "3-8b"):
        if k in key:
            name = "llama-" + k
            return MODEL_PRESETS[name], None
    if "70b" in key:
        return MODEL_PRESETS["llama-3-70b"], None
    if "opt-125m" in key or "tiny" in key:
        return MODEL_PRESETS["tiny"], None
    return MODEL_PRESETS["llama-3.1-8b"], None


def config_from_hf(path: Path) -> ModelConfig:
    c = json.loads(Path(path).read_text())
    eos = c.get("eos_token_id", 128009)
    eos = tuple(eos) if isinstance(eos, list) else (eos,)
    hd = c.get("head_dim") or c["hidden_size"] // c["num_attention_heads"]
    return ModelConfig(
        name=c.get("_name_or_path", Path(path).parent.name) or "hf-model",
        vocab_size=c["vocab_size"], hidden_size=c["hidden_size"],
        intermediate_size=c["intermediate_size"], num_layers=c["num_hidden_layers"],
        num_heads=c["num_attention_heads"],
        num_kv_heads=c.get("num_key_value_heads", c["num_attention_heads"]), head_dim=hd,
        rms_norm_eps=c.get("rms_norm_eps", 1e-5), rope_theta=c.get("rope_theta", 10000.0),
        rope_scaling=c.get("rope_scaling"),
        max_position_embeddings=c.get("max_position_embeddings", 8192),
        tie_word_embeddings=c.get("tie_word_embeddings", False),
        bos_token_id=c.get("bos_token_id", 128000), eos_token_ids=eos)


def _env_int(name, default):
    v = os.environ.get(name)
    try:
        return int(v) if v not in (None, "") else default
    except ValueError:
        return default


@dataclass
class EngineConfig:
    model: str = "meta-llama/Llama-3.1-8B-Instruct"
    dtype: str = "bfloat16"              # reference default float16; both supported
    # Limit: the flash prefill kernel stages a sequence's whole block-table row in LDS (2048
    # entries = 32k tokens at block_size 16).  max_model_len beyond that sends EVERY prefill
    # to the slower v1 kernel (ops.prefill_impl picks by table width, not by the batch) -
    # raise block_size with it (block_size 32 keeps flash up to 64k).
    max_model_len: int = 4096
    max_num_seqs: int = 12
    max_num_batched_tokens: int = 8192
    gpu_memory_utilization: float = 0.90
    block_size: int = 16                 # VLLM_BLOCK_SIZE default (serve_llm.py:325)
    enable_prefix_caching: bool = True
    tensor_parallel_size: int = 1
    seed: int = 0
    device: str = "cuda"
    # hipGraph capture of decode steps (padded batch buckets)
    use_graphs: bool = True
    graph_batch_sizes: tuple = (1, 2, 4, 8, 16, 32, 64, 128, 256)
    # decode split-K partition size (tokens) for the paged attention kernel
    decode_partition_tokens: int = 256
    # finer split for small decode batches (<= decode_small_batch_max sequences): a partition
    # is one workgroup's K/V stream, and at B <= 8 the attention is bound by per-CU bandwidth
    # x latency (256 tokens = 128 KB per workgroup, ~2.5 us to land: the timeline of
    # scripts/gpu/trace_decode_attention.py), so 128-token partitions put twice the CUs on it;
    # with the one-round-trip merge and partition-bucket graphs this wins in situ (bench
    # 760.5 -> 765.5 tok/s; r1 measured it losing with the old 4-per-round-trip merge).
    # Falls back to decode_partition_tokens when max_model_len needs > 64 partitions.
    decode_partition_tokens_small: int = 128
    # decode hipGraphs per partition bucket (attention grid sized to the step's longest
    # context, not max_model_len); buckets above max_model_len's count are dropped
    graph_parts_buckets: tuple = (1, 2, 4, 6, 8, 12, 16, 24, 32, 48, 64)
    decode_small_batch_max: int = 8
    # optional finest tier: B <= decode_tiny_batch_max splits into 64-token partitions
    # (0 = off, the default: faster in isolation - B = 1 at 0.6-3.5k context 7.3 / 8.8 us vs
    # 8.4 / 10.7 at 128 - but it lost in situ, bench 751.9 vs 756.9 tok/s on one box:
    # profiles/r5_attention_partitions.txt)
    decode_partition_tokens_tiny: int = 64
    decode_tiny_batch_max: int = 0
    # chunked prefill: max prompt tokens of one sequence per step (0 = max_num_batched_tokens)
    long_prefill_token_threshold: int = 0
    # fused native decode path (GEMV kernels) when available
    fused_decode: bool = True
    # burst-aware admission (engine/async_engine.py): requests that announce their fan-out
    # (X-Task-ID + x-fanout headers) are held up to this long for their siblings so the
    # burst shares one prefill; 0 disables.  Requests without the headers are never held.
    burst_window_ms: float = 10.0
    # ... and the window closes early once this long has passed since the burst's latest
    # arrival (a LAN fan-out lands inside ~1 ms; under netem skew early arrivals go ahead)
    burst_gap_ms: float = 4.0
    # prefill projection GEMMs: "hipblaslt", "atta" (hand-written CDNA4 Stream-K GEMM with
    # fused residual-add / SiLU-mul epilogues, bf16 and fp8: ops/csrc/prefill_gemm.hip, for
    # steps of >= prefill_gemm_min_rows tokens) or "auto" (each projection on whichever won
    # the measured A/B at that size: models/llama.py LlamaModel._PG_AUTO - with a shipped
    # tuned table the library wins every shape the workload reaches, round 5)
    prefill_gemm: str = "auto"
    prefill_gemm_min_rows: int = 128
    # prefill steps of <= 32 rows (cached-prompt planning prefills, short chunks) on the fused
    # decode kernels (norm-folded skinny GEMVs, RoPE / KV write / SiLU epilogues)
    small_prefill_fused: bool = True
    # library prefill GEMMs from a TunableOp solution table (rocBLAS / hipBLASLt solution per
    # exact shape, tuned cold on MI355X by scripts/gpu/tune_prefill_gemms.py): "auto" = the
    # table shipped for this GPU (agentic_traffic_testing_amd/tuning/), "" = off, else a path.
    # With a table, prefill steps pad their row count to the table's buckets
    # (tuning.bucket_rows) - padding rows carry slot -1 and are never written to the KV cache
    # or sampled
    gemm_tuning: str = "auto"
    # async look-ahead decode: launch the next decode graph step before waiting for the
    # current one's tokens (llm_engine.LLMEngine.step)
    async_decode: bool = True
    # keep a pre-shuffled copy of the decode-GEMV weights (contiguous 1 KiB wave loads)
    preshuffle_decode_weights: bool = True
    # GPU engine start: run every tuned library GEMM shape once and serve a few throw-away
    # requests of the workload's step shapes (prefix cache dropped after), so no code object
    # (HIP translation unit, rocBLAS / hipBLASLt solution, PyTorch kernel) loads inside a
    # timed request (bench/coldstart.py: first 560-row prefill 1157 ms -> 11.5 ms without)
    startup_warmup: bool = True
    # "" = 16-bit weights; "fp8" = OCP e4m3fn weight-only quantisation with per-row scales
    # (decode: fp8 GEMV kernels; prefill: hipBLASLt fp8 GEMM) - BASELINE config 5
    quantization: str = ""
    num_kv_blocks: int = 0               # 0 = size from gpu_memory_utilization
    load_format: str = "auto"            # auto | dummy (random init) | safetensors
    # tensor parallelism: "auto" = RCCL ("nccl") on GPUs, gloo on CPU; "gloo" forces the
    # host path (e.g. several ranks rehearsing on one GPU); tp_same_device puts every rank
    # on the first device (single-GPU rehearsal of the TP protocol)
    tp_backend: str = "auto"
    tp_same_device: bool = False
    tp_allreduce: str = "auto"           # auto | rccl | ipc (custom one-shot all-reduce)
    # IPC path: the row-parallel o / down decode GEMVs push their partial products straight
    # into the peers' receive slots (all-reduce push fused into the GEMV epilogue)
    tp_fused_push: bool = True
    dist_port: int = 0                   # 0 = pick a free port
    # a TP worker that has not registered on the step channel this long after rank 0
    # created it is reported dead (covers workers that die while loading weights)
    tp_register_timeout_s: float = 900.0

    def replace(self, **kw) -> "EngineConfig":
        return replace(self, **kw)

    def as_dict(self) -> dict:
        return asdict(self)

    @staticmethod
    def from_env(**overrides) -> "EngineConfig":
        """Engine knobs from the reference's env variables (infra/docker-compose.yml:16-27)."""
        cfg = EngineConfig()
        env = os.environ
        kw = {}
        if env.get("LLM_MODEL"):
            kw["model"] = env["LLM_MODEL"]
        if env.get("LLM_DTYPE"):
            kw["dtype"] = env["LLM_DTYPE"]
        n = _env_int("LLM_MAX_NUM_SEQS", -1)
        if n > 0:
            kw["max_num_seqs"] = n
        n = _env_int("LLM_MAX_NUM_BATCHED_TOKENS", -1)
        if n > 0:
            kw["max_num_batched_tokens"] = n
        if env.get("LLM_GPU_MEMORY_UTILIZATION"):
            kw["gpu_memory_utilization"] = float(env["LLM_GPU_MEMORY_UTILIZATION"])
        n = _env_int("LLM_MAX_MODEL_LEN", 0)
        if n > 0:
            kw["max_model_len"] = n
        n = _env_int("VLLM_BLOCK_SIZE", 0)
        if n > 0:
            kw["block_size"] = n
        n = _env_int("LLM_TENSOR_PARALLEL_SIZE", 0)
        if n > 0:
            kw["tensor_parallel_size"] = n
        if env.get("LLM_QUANTIZATION"):
            kw["quantization"] = env["LLM_QUANTIZATION"].strip().lower()
        kw.update({k: v for k, v in overrides.items() if v is not None})
        return cfg.replace(**kw)
