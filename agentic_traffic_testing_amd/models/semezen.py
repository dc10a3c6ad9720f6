"""Semezen decoder over the mixer op layer (``ops.mixers``).

Pre-norm layers on ``streams`` fp32 residual streams (hyper-connections): a sub-layer reads the
RMS norm of a weighted sum of the streams, and its output is added to every stream with a
weight of its own after the streams were mixed by a small matrix.  The mixer's input is token
shifted: every channel moves towards the previous token's normed row by a learned amount (that
row is per-sequence state in every layer).  Mixers:

* ``attention`` - grouped-query softmax attention inside a sliding window; biased q / k
  projections, the values ARE the projected keys (before rotation and norm), rotate-half
  positions with wavelength-dependent frequency scaling on the leading channels, weightless
  per-head RMS norm of q and k after the rotation, an element-wise sigmoid output gate;
* ``mingru`` - an element-wise gated recurrence with fp32 state per sequence.

Feed-forward: dense GELU, or routed experts (sigmoid router in fp32, the score scales the
expert's input, clamped GLU activation).

MI355X layout: the projections that read a mixer's input are one fused library GEMM with the
biases in its epilogue (blocks padded to 8 rows so kernels read 16-byte aligned slices in
place); the stream update and the next sub-layer's norm are one kernel; K pages hold the
rotated and normed keys, the channel-major V pages the raw projected keys; the experts run as
two grouped matrix-core products over rows sorted by expert on the device, so a decode step
stays capturable as a hipGraph.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path

import torch
import torch.nn.functional as F

from ..config import MinGruConfig, SemezenConfig, WindowAttentionConfig
from ..engine.state_cache import HybridCache, LayerCacheSpec
from ..ops import mixers as mx


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


@dataclass
class HyperWeights:
    """One sub-layer's stream weights (fp32): read-in [s], write-out [s], mix [s, s] (from, to)."""
    w_in: torch.Tensor
    w_out: torch.Tensor
    mix: torch.Tensor


@dataclass
class SemezenLayerWeights:
    norm1: torch.Tensor
    shift: torch.Tensor                        # fp32 [W]
    hc1: HyperWeights
    w_in: torch.Tensor = None                  # fused projections of the mixer's input
    b_in: torch.Tensor | None = None
    seg: dict = field(default_factory=dict)    # block name -> (column offset, width)
    w_o: torch.Tensor | None = None
    inv_freq: torch.Tensor | None = None
    # feed-forward
    norm2: torch.Tensor | None = None
    hc2: HyperWeights | None = None
    up: torch.Tensor | None = None
    down: torch.Tensor | None = None
    router: torch.Tensor | None = None         # fp32 [E, W]
    e_gu: torch.Tensor | None = None           # [E, 2 ff, W]: gate rows, then up rows
    e_down: torch.Tensor | None = None         # [E, W, ff]


class SemezenModel:
    family = "semezen"
    has_state = True

    def __init__(self, cfg: SemezenConfig, dtype=torch.bfloat16, device="cuda", tp_rank: int = 0,
                 tp_size: int = 1, tp_group=None, quantization: str = ""):
        if tp_size != 1:
            raise ValueError("Semezen runs on one GPU per replica (tensor_parallel_size 1)")
        if quantization:
            raise ValueError("Semezen weights are 16-bit or 32-bit; no quantization")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Semezen activations are bfloat16 or float32")
        self.cfg = cfg
        self.dtype = dtype
        self.device = torch.device(device)
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        self.layers: list[SemezenLayerWeights] = []
        self.embed = self.final_norm = self.head = self.ones = None
        self.vocab_shard = cfg.vocab_size
        if self.dtype == torch.float32 and self.device.type == "cuda":
            # fp32 serving is exact fp32: no reduced-precision matrix mode
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False

    # ---------------------------------------------------------------------------------
    def tensor_shapes(self) -> dict:
        """Checkpoint tensor name -> shape for this configuration."""
        c = self.cfg
        W, s = c.hidden_size, c.streams
        out = {"embed": (c.vocab_size, W), "final.norm": (W,), "head": (c.vocab_size, W)}
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.", L.mixer
            x = p + "mix."
            out.update({p + "norm1": (W,), p + "shift": (W,), p + "hc1.in": (s,),
                        p + "hc1.out": (s,), p + "hc1.mix": (s, s)})
            if L.kind == "attention":
                out.update({x + "q": (m.heads * m.dim, W), x + "q.b": (m.heads * m.dim,),
                            x + "k": (m.kv_heads * m.dim, W), x + "k.b": (m.kv_heads * m.dim,),
                            x + "g": (m.heads * m.vdim, W), x + "o": (W, m.heads * m.vdim)})
            else:
                out.update({x + "z": (m.width, W), x + "z.b": (m.width,), x + "x": (m.width, W),
                            x + "x.b": (m.width,), x + "g": (m.width, W), x + "o": (W, m.width)})
            if L.ff or L.moe:
                out.update({p + "norm2": (W,), p + "hc2.in": (s,), p + "hc2.out": (s,),
                            p + "hc2.mix": (s, s)})
            if L.ff:
                out.update({p + "mlp.up": (L.ff, W), p + "mlp.down": (W, L.ff)})
            if L.moe:
                out[p + "mlp.router"] = (L.moe.experts, W)
                for e in range(L.moe.experts):
                    out.update({f"{p}mlp.e{e}.gate": (L.moe.ff, W), f"{p}mlp.e{e}.up": (L.moe.ff, W),
                                f"{p}mlp.e{e}.down": (W, L.moe.ff)})
        return out

    def random_state(self, seed: int = 0) -> dict:
        """Seeded random tensors under the checkpoint's names (bf16-representable values)."""
        g = torch.Generator().manual_seed(24681357 + seed)
        s = self.cfg.streams
        st = {}
        for name, shape in self.tensor_shapes().items():
            r = torch.randn(shape, generator=g)
            parts = name.split(".")
            leaf = parts[-1]
            if name == "embed":
                t = r
            elif leaf in ("norm1", "norm2", "norm"):
                t = 1.0 + 0.1 * r
            elif leaf == "shift":
                t = torch.rand(shape, generator=g)
            elif leaf == "b":
                t = 0.3 * r
            elif len(parts) > 1 and parts[1] in ("hc1", "hc2"):
                if leaf == "in":
                    t = 1.0 / s + 0.2 * r
                elif leaf == "out":
                    t = 0.7 + 0.2 * r
                else:
                    t = torch.eye(s) * 0.8 + 0.15 * r
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
        W, s = c.hidden_size, c.streams

        def get(name, shape):
            t = st[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, configuration wants {shape}")
            return t

        def act(name, shape):
            return get(name, shape).to(dt).to(dev).contiguous()

        def f32(name, shape):
            return get(name, shape).float().to(dev).contiguous()

        def hyper(p):
            return HyperWeights(f32(p + "in", (s,)), f32(p + "out", (s,)), f32(p + "mix", (s, s)))

        def fuse(lw, blocks):
            rows, bias, off = [], [], 0
            for name, t, b in blocks:
                n = t.shape[0]
                lw.seg[name] = (off, n)
                rows.append(t)
                bias.append(b if b is not None else torch.zeros(n, dtype=dt, device=dev))
                if _pad8(n) != n:
                    rows.append(torch.zeros(_pad8(n) - n, W, dtype=dt, device=dev))
                    bias.append(torch.zeros(_pad8(n) - n, dtype=dt, device=dev))
                off += _pad8(n)
            lw.w_in = torch.cat(rows).contiguous()
            lw.b_in = torch.cat(bias).contiguous()

        self.embed = act("embed", (c.vocab_size, W))
        self.final_norm = act("final.norm", (W,))
        self.head = act("head", (c.vocab_size, W))
        self.ones = torch.ones(s, dtype=torch.float32, device=dev)
        self.layers = []
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.", L.mixer
            x = p + "mix."
            lw = SemezenLayerWeights(norm1=act(p + "norm1", (W,)), shift=f32(p + "shift", (W,)),
                                     hc1=hyper(p + "hc1."))
            if L.kind == "attention":
                nq, nk = m.heads * m.dim, m.kv_heads * m.dim
                fuse(lw, [("q", act(x + "q", (nq, W)), act(x + "q.b", (nq,))),
                          ("k", act(x + "k", (nk, W)), act(x + "k.b", (nk,))),
                          ("g", act(x + "g", (m.heads * m.vdim, W)), None)])
                lw.w_o = act(x + "o", (W, m.heads * m.vdim))
                if m.rot_dims:
                    lw.inv_freq = mx.scaled_inv_freq(m.rot_dims, m.rot_base, m.rot_scaling, dev)
            elif L.kind == "mingru":
                n = m.width
                fuse(lw, [("z", act(x + "z", (n, W)), act(x + "z.b", (n,))),
                          ("x", act(x + "x", (n, W)), act(x + "x.b", (n,))),
                          ("g", act(x + "g", (n, W)), None)])
                lw.w_o = act(x + "o", (W, n))
            else:
                raise ValueError(L.kind)
            if L.ff or L.moe:
                lw.norm2 = act(p + "norm2", (W,))
                lw.hc2 = hyper(p + "hc2.")
            if L.ff:
                lw.up = act(p + "mlp.up", (L.ff, W))
                lw.down = act(p + "mlp.down", (W, L.ff))
            if L.moe:
                E, ff = L.moe.experts, L.moe.ff
                lw.router = f32(p + "mlp.router", (E, W))
                lw.e_gu = torch.stack([torch.cat([act(f"{p}mlp.e{e}.gate", (ff, W)),
                                                  act(f"{p}mlp.e{e}.up", (ff, W))])
                                       for e in range(E)])
                lw.e_down = torch.stack([act(f"{p}mlp.e{e}.down", (W, ff)) for e in range(E)])
            self.layers.append(lw)
        return self

    def prepare_decode_weights(self):
        return self

    def decode_copy_bytes(self) -> int:
        return 0

    def weight_bytes(self) -> int:
        ts = [self.embed, self.final_norm, self.head]
        for L in self.layers:
            for v in vars(L).values():
                if isinstance(v, torch.Tensor):
                    ts.append(v)
                elif isinstance(v, HyperWeights):
                    ts += [v.w_in, v.w_out, v.mix]
        return sum(t.numel() * t.element_size() for t in ts if t is not None)

    # ---------------------------------------------------------------------------------
    def cache_specs(self) -> list[LayerCacheSpec]:
        W = self.cfg.hidden_size
        specs = []
        for L in self.cfg.layers:
            m = L.mixer
            if isinstance(m, WindowAttentionConfig):
                specs.append(LayerCacheSpec(kv_heads=m.kv_heads, kdim=m.dim, vdim=m.vdim,
                                            shift_channels=W))
            elif isinstance(m, MinGruConfig):
                specs.append(LayerCacheSpec(state_heads=1, state_dim=1, state_vdim=m.width,
                                            shift_channels=W))
        return specs

    @property
    def attn_tile_tokens(self) -> int:
        return mx.ATTN_TILE_TOKENS

    # ---------------------------------------------------------------------------------
    def _attention(self, h, lw, m, md, lc, tables):
        T = h.shape[0]
        P = F.linear(h, lw.w_in, lw.b_in)
        (oq, nq), (ok, nk), (og, ng) = lw.seg["q"], lw.seg["k"], lw.seg["g"]
        key = (m.rot_dims, m.rot_base, m.rot_scaling)
        if key not in tables:   # cos / sin of the step's positions, once per rotary setting
            tables[key] = (mx.rotary_table(md.positions, lw.inv_freq) if m.rot_dims else
                           torch.zeros(T, 0, dtype=torch.float32, device=h.device))
        kx = P[:, ok:ok + nk]
        # the value rows are the key projection as it is; K pages get rotation, then the norm
        q = mx.qk_norm_rope_cache(P[:, oq:oq + nq], kx, kx, None, None, self.cfg.rms_norm_eps,
                                  md.positions, md.slot_mapping, tables[key], lc.k, lc.v, m.heads,
                                  m.kv_heads, m.dim, m.vdim, rotate_half_pairs=True,
                                  norm_last=True)
        a = mx.sink_attention(q, lc.k, lc.v, md.block_tables, md.seq_kvlen, md.seq_qstart,
                              md.tile_seq, md.tile_qoff, m.scale, False, md.num_decode,
                              md.max_decode_kv, window=m.window)
        a = mx.gate_mul(a.view(T, m.heads * m.vdim), P[:, og:og + ng], "sigmoid")
        return F.linear(a, lw.w_o)

    def _mingru(self, h, lw, m, md, lc):
        P = F.linear(h, lw.w_in, lw.b_in)
        (oz, nz), (ox, nx), (og, ng) = lw.seg["z"], lw.seg["x"], lw.seg["g"]
        y = mx.mingru_scan(P[:, oz:oz + nz], P[:, ox:ox + nx], P[:, og:og + ng], lc.state,
                           md.positions, md.seq_qstart, md.seq_slot, self.dtype)
        return F.linear(y, lw.w_o)

    def _experts(self, h, lw, moe):
        logits = F.linear(h.float(), lw.router)       # fp32 router on the (rounded) input
        idx, wts = mx.moe_route(logits, moe.top)
        return mx.moe_experts(h, idx, wts, lw.e_gu, lw.e_down, moe.limit, moe.act_alpha)

    def forward(self, input_ids, md, cache: HybridCache, rows=None, layer_out=None):
        """One step over a decode-first batch of portions; returns the final-normed hidden rows
        (all, or ``rows``).  ``layer_out``: a list that receives a copy of the fp32 sum of the
        streams after every layer (debugging / tests)."""
        c = self.cfg
        eps, s = c.rms_norm_eps, c.streams
        xs = mx.embed_scale(self.embed, input_ids, 1.0, copies=s)   # [T, s, W] fp32
        n = (mx.hyper_norm(xs, self.layers[0].hc1.w_in, self.layers[0].norm1, eps, torch.float32)
             if self.layers else None)
        last = len(self.layers) - 1
        tables = {}
        for li, (L, lw) in enumerate(zip(c.layers, self.layers)):
            lc = cache.layers[li]
            h = mx.token_shift(n, lw.shift, lc.shift, md.positions, md.seq_qstart, md.seq_slot,
                               self.dtype)
            if L.kind == "attention":
                y = self._attention(h, lw, L.mixer, md, lc, tables)
            else:
                y = self._mingru(h, lw, L.mixer, md, lc)
            hc = lw.hc1
            if L.ff or L.moe:   # stream update and the feed-forward's norm in one kernel
                h2 = mx.hyper_update_norm(xs, y, hc.mix, hc.w_out, lw.hc2.w_in, lw.norm2, eps,
                                          self.dtype)
                if L.ff:
                    y = F.linear(mx.gelu(F.linear(h2, lw.up), L.ff_act == "gelu_tanh"), lw.down)
                else:
                    y = self._experts(h2, lw, L.moe)
                hc = lw.hc2
            if li < last:
                nx = self.layers[li + 1]
                n = mx.hyper_update_norm(xs, y, hc.mix, hc.w_out, nx.hc1.w_in, nx.norm1, eps,
                                         torch.float32)
            else:
                mx.hyper_update_norm(xs, y, hc.mix, hc.w_out, None, None, eps)
            if layer_out is not None:
                layer_out.append(xs.sum(1))
        if rows is not None:
            xs = xs.index_select(0, rows)
        return mx.hyper_norm(xs, self.ones, self.final_norm, eps, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.head).float()
