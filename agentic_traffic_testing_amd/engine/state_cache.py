"""Device side of the hybrid cache: per layer, paged K / V pools for softmax mixers and
(V pages are stored channel-major, [vdim, block], so the P.V matrix-core operand reads keys
contiguously) and fixed-size per-sequence state (recurrent matrix state in fp32, convolution tails) for
recurrent mixers, the previous token's mixer input of token-shifted layers (fp32), plus the
per-sequence previous token.  The host side - which pages and
which state slot a sequence owns - is the native ``BlockManager`` (state slots are handed
out at admission and returned with the pages).

A model describes what each layer needs with ``LayerCacheSpec``; the model runner sizes the
page pool from free memory and allocates a ``HybridCache``.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass(frozen=True)
class LayerCacheSpec:
    kv_heads: int = 0          # > 0: paged K [nb, kv_heads, BS, kdim] and V [nb, kv_heads, vdim, BS]
    kdim: int = 0
    vdim: int = 0
    state_heads: int = 0       # > 0: fp32 state [slots, state_heads, state_dim, state_vdim]
    state_dim: int = 0
    state_vdim: int = 0
    conv_channels: int = 0     # > 0: tails [slots, conv_taps - 1, conv_channels]
    conv_taps: int = 0
    kv_from: int = -1          # >= 0: no pages of its own, the layer reads that layer's K / V
    shift_channels: int = 0    # > 0: fp32 [slots, shift_channels], the previous token's mixer input

    def page_bytes(self, block_size: int, itemsize: int) -> int:
        if self.kv_from >= 0:
            return 0
        return self.kv_heads * block_size * (self.kdim + self.vdim) * itemsize

    def slot_bytes(self, itemsize: int) -> int:
        return (self.state_heads * self.state_dim * self.state_vdim * 4
                + max(0, self.conv_taps - 1) * self.conv_channels * itemsize
                + self.shift_channels * 4)


@dataclass
class LayerCache:
    k: torch.Tensor | None = None
    v: torch.Tensor | None = None
    state: torch.Tensor | None = None
    conv: torch.Tensor | None = None
    shift: torch.Tensor | None = None


@dataclass
class HybridCache:
    layers: list = field(default_factory=list)
    prev_token: torch.Tensor | None = None   # int32 [slots]
    num_blocks: int = 0
    num_slots: int = 0
    block_size: int = 0

    @staticmethod
    def allocate(specs, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        layers = []
        for sp in specs:
            lc = LayerCache()
            if sp.kv_from >= 0:
                if not 0 <= sp.kv_from < len(layers) or layers[sp.kv_from].k is None:
                    raise ValueError("kv_from must name an earlier layer with pages of its own")
                lc.k, lc.v = layers[sp.kv_from].k, layers[sp.kv_from].v
            elif sp.kv_heads:
                lc.k = torch.zeros(num_blocks, sp.kv_heads, block_size, sp.kdim, dtype=dtype,
                                   device=device)
                lc.v = torch.zeros(num_blocks, sp.kv_heads, sp.vdim, block_size, dtype=dtype,
                                   device=device)
            if sp.state_heads:
                lc.state = torch.zeros(num_slots, sp.state_heads, sp.state_dim, sp.state_vdim,
                                       dtype=torch.float32, device=device)
            if sp.conv_channels and sp.conv_taps > 1:
                lc.conv = torch.zeros(num_slots, sp.conv_taps - 1, sp.conv_channels, dtype=dtype,
                                      device=device)
            if sp.shift_channels:
                lc.shift = torch.zeros(num_slots, sp.shift_channels, dtype=torch.float32,
                                       device=device)
            layers.append(lc)
        return HybridCache(layers, torch.zeros(max(1, num_slots), dtype=torch.int32,
                                               device=device), num_blocks, num_slots, block_size)

    def nbytes(self) -> int:
        seen = {}
        for lc in self.layers:
            for t in (lc.k, lc.v, lc.state, lc.conv, lc.shift):
                if t is not None:
                    seen[t.data_ptr()] = t.numel() * t.element_size()
        return sum(seen.values())
