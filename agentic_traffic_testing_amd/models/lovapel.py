"""Lovapel decoder over the mixer op layer (``ops.mixers``).

Sandwich-norm layers on an fp32 residual stream: ``x += ln1b(mixer(ln1(x)))`` then
``x += ln2b(ff(ln2(x)))`` with weight-only layer norms.  A span of layers can run several times
in a row with the same weights; every run has pages of its own.

* mixer - grouped-query softmax attention inside a sliding window; q and k are RMS-normed over
  the WHOLE projection (all heads at once) before the rotate-half positions on the leading
  channels of every head; one learned sink score per query head in the denominator;
* feed-forward - dense GLU with the tanh-form GELU, or routed SiLU-GLU experts: softmax router in
  fp32, a stored correction added for the choice only, choice restricted to the best groups of
  neighbouring experts, identity experts without weights, normalised weights on the experts'
  outputs, plus a shared expert for every token;
* output - the embedding table as the head, logits scaled and soft-capped with tanh.

MI355X layout: q | k | v are one fused library GEMM and gate | up another (blocks padded to 8 rows
so kernels read 16-byte aligned slices in place); the post-norm of a branch, the residual sum and
the next pre-norm are one kernel; the inverse RMS of the q and k projections comes from a
one-wave-per-row pass, then one kernel norms, rotates and writes the K pages (V pages
channel-major for the P.V matrix-core operand); the experts run as two grouped matrix-core
products over rows sorted by expert on the device and a combine kernel that applies the weights,
the identity experts and the shared expert in fp32, so a decode step stays capturable as a
hipGraph.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path

import torch
import torch.nn.functional as F

from ..config import LovapelConfig
from ..engine.state_cache import HybridCache, LayerCacheSpec
from ..ops import mixers as mx


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


@dataclass
class LovapelLayerWeights:
    norm1: torch.Tensor
    norm1b: torch.Tensor
    w_in: torch.Tensor = None                  # fused q | k | v projections
    seg: dict = field(default_factory=dict)    # block name -> (column offset, width)
    q_norm: torch.Tensor | None = None         # [heads * dim]
    k_norm: torch.Tensor | None = None         # [kv_heads * dim]
    sink: torch.Tensor | None = None           # fp32 [heads]
    w_o: torch.Tensor | None = None
    inv_freq: torch.Tensor | None = None
    # feed-forward
    norm2: torch.Tensor | None = None
    norm2b: torch.Tensor | None = None
    gu: torch.Tensor | None = None             # dense: fused gate | up
    gu_seg: dict = field(default_factory=dict)
    down: torch.Tensor | None = None
    router: torch.Tensor | None = None         # fp32 [E + identity, W]
    correction: torch.Tensor | None = None     # fp32 [E + identity]
    e_gu: torch.Tensor | None = None           # [E, 2 ff, W]: gate rows, then up rows
    e_down: torch.Tensor | None = None         # [E, W, ff]
    s_gu: torch.Tensor | None = None           # shared expert: fused gate | up
    s_seg: dict = field(default_factory=dict)
    s_down: torch.Tensor | None = None


class LovapelModel:
    family = "lovapel"
    has_state = True     # served through the hybrid cache (pages per layer run, state slots unused)

    def __init__(self, cfg: LovapelConfig, dtype=torch.bfloat16, device="cuda", tp_rank: int = 0,
                 tp_size: int = 1, tp_group=None, quantization: str = ""):
        if tp_size != 1:
            raise ValueError("Lovapel runs on one GPU per replica (tensor_parallel_size 1)")
        if quantization:
            raise ValueError("Lovapel weights are 16-bit or 32-bit; no quantization")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Lovapel activations are bfloat16 or float32")
        self.cfg = cfg
        self.dtype = dtype
        self.device = torch.device(device)
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        self.layers: list[LovapelLayerWeights] = []
        self.embed = self.final_norm = None
        self.vocab_shard = cfg.vocab_size
        if self.dtype == torch.float32 and self.device.type == "cuda":
            # fp32 serving is exact fp32: no reduced-precision matrix mode
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False

    # ---------------------------------------------------------------------------------
    def tensor_shapes(self) -> dict:
        """Checkpoint tensor name -> shape for this configuration."""
        c = self.cfg
        W = c.hidden_size
        out = {"embed": (c.vocab_size, W), "final.norm": (W,)}
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.", L.mixer
            x = p + "mix."
            nq, nk = m.heads * m.dim, m.kv_heads * m.dim
            out.update({p + "norm1": (W,), p + "norm1b": (W,), x + "q": (nq, W), x + "k": (nk, W),
                        x + "v": (m.kv_heads * m.vdim, W), x + "q.norm": (nq,),
                        x + "k.norm": (nk,), x + "sink": (m.heads,),
                        x + "o": (W, m.heads * m.vdim)})
            if L.ff or L.moe:
                out.update({p + "norm2": (W,), p + "norm2b": (W,)})
            f = p + "mlp."
            if L.ff:
                out.update({f + "gate": (L.ff, W), f + "up": (L.ff, W), f + "down": (W, L.ff)})
            if L.moe:
                mo = L.moe
                out.update({f + "router": (mo.routes, W), f + "correction": (mo.routes,)})
                for e in range(mo.experts):
                    out.update({f"{f}e{e}.gate": (mo.ff, W), f"{f}e{e}.up": (mo.ff, W),
                                f"{f}e{e}.down": (W, mo.ff)})
                if mo.shared_ff:
                    out.update({f + "shared.gate": (mo.shared_ff, W),
                                f + "shared.up": (mo.shared_ff, W),
                                f + "shared.down": (W, mo.shared_ff)})
        return out

    def random_state(self, seed: int = 0) -> dict:
        """Seeded random tensors under the checkpoint's names (bf16-representable values)."""
        g = torch.Generator().manual_seed(97531 + seed)
        st = {}
        for name, shape in self.tensor_shapes().items():
            r = torch.randn(shape, generator=g)
            leaf = name.split(".")[-1]
            if name == "embed":
                t = r
            elif leaf.startswith("norm"):
                t = 1.0 + 0.1 * r
            elif leaf == "sink":
                t = r
            elif leaf == "correction":
                t = 0.02 * r
            elif leaf == "router":
                t = 4.0 * r / math.sqrt(shape[-1])
            else:
                t = r / math.sqrt(shape[-1])
            st[name] = t.to(torch.bfloat16)
        return st

    def init_random(self, seed: int = 0):
        return self.load_state(self.random_state(seed))

    def load_safetensors(self, path: str):
        from safetensors import safe_open

        files = sorted(Path(path).glob("*.safetensors"))
        if not files:
            raise FileNotFoundError(f"no safetensors in {path}")
        st = {}
        for f in files:
            with safe_open(str(f), framework="pt") as sf:
                for k in sf.keys():
                    st[k] = sf.get_tensor(k)
        return self.load_state(st)

    def load_state(self, st: dict):
        """Build the fused device weights from checkpoint-named tensors."""
        c, dev, dt = self.cfg, self.device, self.dtype
        W = c.hidden_size

        def get(name, shape):
            t = st[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, configuration wants {shape}")
            return t

        def act(name, shape):
            return get(name, shape).to(dt).to(dev).contiguous()

        def f32(name, shape):
            return get(name, shape).float().to(dev).contiguous()

        def fuse(seg, blocks):
            rows, off = [], 0
            for name, t in blocks:
                n = t.shape[0]
                seg[name] = (off, n)
                rows.append(t)
                if _pad8(n) != n:
                    rows.append(torch.zeros(_pad8(n) - n, W, dtype=dt, device=dev))
                off += _pad8(n)
            return torch.cat(rows).contiguous()

        self.embed = act("embed", (c.vocab_size, W))
        self.final_norm = act("final.norm", (W,))
        self.layers = []
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.", L.mixer
            x = p + "mix."
            nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            lw = LovapelLayerWeights(norm1=act(p + "norm1", (W,)), norm1b=act(p + "norm1b", (W,)))
            lw.w_in = fuse(lw.seg, [("q", act(x + "q", (nq, W))), ("k", act(x + "k", (nk, W))),
                                    ("v", act(x + "v", (nv, W)))])
            lw.q_norm = act(x + "q.norm", (nq,))
            lw.k_norm = act(x + "k.norm", (nk,))
            lw.sink = f32(x + "sink", (m.heads,))
            lw.w_o = act(x + "o", (W, m.heads * m.vdim))
            if m.rot_dims:
                lw.inv_freq = mx.inv_freq(m.rot_dims, m.rot_base, dev)
            if L.ff or L.moe:
                lw.norm2 = act(p + "norm2", (W,))
                lw.norm2b = act(p + "norm2b", (W,))
            f = p + "mlp."
            if L.ff:
                lw.gu = fuse(lw.gu_seg, [("gate", act(f + "gate", (L.ff, W))),
                                         ("up", act(f + "up", (L.ff, W)))])
                lw.down = act(f + "down", (W, L.ff))
            if L.moe:
                mo = L.moe
                lw.router = f32(f + "router", (mo.routes, W))
                lw.correction = (f32(f + "correction", (mo.routes,)) if f + "correction" in st
                                 else torch.zeros(mo.routes, dtype=torch.float32, device=dev))
                lw.e_gu = torch.stack([torch.cat([act(f"{f}e{e}.gate", (mo.ff, W)),
                                                  act(f"{f}e{e}.up", (mo.ff, W))])
                                       for e in range(mo.experts)])
                lw.e_down = torch.stack([act(f"{f}e{e}.down", (W, mo.ff))
                                         for e in range(mo.experts)])
                if mo.shared_ff:
                    lw.s_gu = fuse(lw.s_seg, [("gate", act(f + "shared.gate", (mo.shared_ff, W))),
                                              ("up", act(f + "shared.up", (mo.shared_ff, W)))])
                    lw.s_down = act(f + "shared.down", (W, mo.shared_ff))
            self.layers.append(lw)
        return self

    def prepare_decode_weights(self):
        return self

    def decode_copy_bytes(self) -> int:
        return 0

    def weight_bytes(self) -> int:
        ts = [self.embed, self.final_norm]
        for L in self.layers:
            ts += [v for v in vars(L).values() if isinstance(v, torch.Tensor)]
        return sum(t.numel() * t.element_size() for t in ts if t is not None)

    # ---------------------------------------------------------------------------------
    def cache_specs(self) -> list[LayerCacheSpec]:
        """One entry per layer RUN: a layer inside the repeated span owns pages per pass."""
        specs = []
        for li in self.cfg.runs:
            m = self.cfg.layers[li].mixer
            specs.append(LayerCacheSpec(kv_heads=m.kv_heads, kdim=m.dim, vdim=m.vdim))
        return specs

    @property
    def attn_tile_tokens(self) -> int:
        return mx.ATTN_TILE_TOKENS

    # ---------------------------------------------------------------------------------
    def _attention(self, h, lw, m, md, lc, tables):
        T = h.shape[0]
        P = F.linear(h, lw.w_in)
        (oq, nq), (ok, nk), (ov, nv) = lw.seg["q"], lw.seg["k"], lw.seg["v"]
        key = (m.rot_dims, m.rot_base)
        if key not in tables:   # cos / sin of the step's positions, once per rotary setting
            tables[key] = (mx.rotary_table(md.positions, lw.inv_freq) if m.rot_dims else
                           torch.zeros(T, 0, dtype=torch.float32, device=h.device))
        q = mx.qk_norm_rope_cache(P[:, oq:oq + nq], P[:, ok:ok + nk], P[:, ov:ov + nv], lw.q_norm,
                                  lw.k_norm, self.cfg.norm_eps, md.positions, md.slot_mapping,
                                  tables[key], lc.k, lc.v, m.heads, m.kv_heads, m.dim, m.vdim,
                                  rotate_half_pairs=True, whole_norm=True)
        a = mx.sink_attention(q, lc.k, lc.v, md.block_tables, md.seq_kvlen, md.seq_qstart,
                              md.tile_seq, md.tile_qoff, m.scale, True, md.num_decode,
                              md.max_decode_kv, sink_values=lw.sink, window=m.window)
        return F.linear(a.view(T, m.heads * m.vdim), lw.w_o)

    @staticmethod
    def _glu(h, w_gu, seg, w_down, act):
        P = F.linear(h, w_gu)
        (og, n), (ou, _) = seg["gate"], seg["up"]
        return F.linear(mx.gate_mul(P[:, ou:ou + n], P[:, og:og + n], act), w_down)

    def _experts(self, h, lw, mo):
        logits = F.linear(h.float(), lw.router)       # fp32 router on the (rounded) input
        idx, wts = mx.moe_route(logits, mo.top, "softmax", lw.correction, mo.groups, mo.keep,
                                renorm=True)
        shared = self._glu(h, lw.s_gu, lw.s_seg, lw.s_down, "silu") if mo.shared_ff else None
        return mx.moe_experts(h, idx, wts, lw.e_gu, lw.e_down, glu="silu", addend=shared)

    def forward(self, input_ids, md, cache: HybridCache, rows=None, layer_out=None):
        """One step over a decode-first batch of portions; returns the final-normed hidden rows
        (all, or ``rows``).  ``layer_out``: a list that receives a copy of the fp32 residual
        stream after every layer run (debugging / tests)."""
        c = self.cfg
        eps, runs = c.norm_eps, c.runs
        x = mx.embed_scale(self.embed, input_ids, 1.0)            # [T, W] fp32
        h = (mx.norm_add_norm(x, None, None, self.layers[runs[0]].norm1, eps, "layer", self.dtype)
             if runs else None)
        tables = {}
        for r, li in enumerate(runs):
            L, lw = c.layers[li], self.layers[li]
            y = self._attention(h, lw, L.mixer, md, cache.layers[r], tables)
            post = lw.norm1b
            if L.ff or L.moe:   # post-norm, residual sum and the feed-forward's norm in one kernel
                h2 = mx.norm_add_norm(x, y, post, lw.norm2, eps, "layer", self.dtype)
                y = (self._glu(h2, lw.gu, lw.gu_seg, lw.down, "gelu_tanh") if L.ff else
                     self._experts(h2, lw, L.moe))
                post = lw.norm2b
            nxt = self.layers[runs[r + 1]].norm1 if r + 1 < len(runs) else None
            h = mx.norm_add_norm(x, y, post, nxt, eps, "layer", self.dtype)
            if layer_out is not None:
                layer_out.append(x.clone())
        if rows is not None:
            x = x.index_select(0, rows)
        return mx.norm_add_norm(x, None, None, self.final_norm, eps, "layer", self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        c = self.cfg
        return mx.scale_softcap(F.linear(hidden, self.embed), c.logit_scale, c.logit_softcap)
