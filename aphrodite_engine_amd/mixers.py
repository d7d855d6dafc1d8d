"""Sequence-mixer building blocks beside the rotary softmax attention of ``attention/``: each is a mechanism with its
constants as parameters, says what cache it needs per layer run (``cache_spec``), and runs on a ``StepBatch`` -- prompt
portions and decoded tokens in one launch -- through the kernels of ``mixer_ops``.

  DistanceBiasAttention   grouped-query softmax attention over a token-major paged cache; no rotation: positions enter as
                          an additive per-head bias looked up by (bucketed) distance and as a query temperature that
                          grows with the logarithm of the position; optional per-head sigmoid output gate
  OuterProductMemory      a matrix state per head in a per-request slot: decay linear attention (fixed per-head decay) or
                          the mLSTM cell (exponential gating under a running maximum, normaliser vector)
  LayerNormParams, GatedMLP  the norm with weight and bias around an fp32 residual stream; gate * up feed-forward
"""
import math
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
from torch import nn

from . import mixer_ops as mops
from .step_batch import StepBatch


@dataclass(frozen=True)
class PagedKVSpec:
    """A token-major paged key / value cache: K [blocks, block, kv_heads, dim], V [blocks, block, kv_heads, vdim]."""
    kv_heads: int
    dim: int
    vdim: int

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return (torch.zeros(num_blocks, block_size, self.kv_heads, self.dim, dtype=dtype, device=device),
                torch.zeros(num_blocks, block_size, self.kv_heads, self.vdim, dtype=dtype, device=device))


@dataclass(frozen=True)
class MemoryStateSpec:
    """fp32 state of an OuterProductMemory, one entry per request slot."""
    heads: int
    dim: int
    vdim: int
    mode: int

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return tuple(torch.zeros(s, dtype=torch.float32, device=device)
                     for s in mops.memory_state_shapes(num_slots, self.heads, self.dim, self.vdim, self.mode))


def log_distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of a [rows, heads] bias table for a key ``n`` positions back: exact rows below rows // 2, then rows that widen
    geometrically and reach the last one at distance ``far``."""
    half = rows // 2
    if n < half or rows == 1:
        return min(n, rows - 1)
    if far <= half:
        return rows - 1
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


class LayerNormParams(nn.Module):
    def __init__(self, width: int, dtype):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(width, dtype=dtype), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(width, dtype=dtype), requires_grad=False)

    def pair(self) -> Tuple[torch.Tensor, torch.Tensor]:
        return self.weight, self.bias


class DistanceBiasAttention(nn.Module):
    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, bias_rows: int = 0,
                 bias_far: float = 0.0, temp_coef: float = 0.0, temp_every: int = 1):
        super().__init__()
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads over {kv_heads} key/value heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.bias_far = float(scale), float(bias_far)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        # the learned table stays fp32 (it is added to fp32 scores); ``finalize`` tabulates it by distance
        self.rel = nn.Parameter(torch.zeros(bias_rows, heads, dtype=torch.float32), requires_grad=False) if bias_rows else None
        self.bias_lut = None

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.kv_heads, self.dim, self.vdim)

    def finalize(self) -> None:
        """bias_lut[h, n] = rel[bucket(n), h] up to the first distance of the last row; farther keys clamp to it."""
        if self.rel is None:
            return
        rows = self.rel.shape[0]
        reach = max(rows // 2, int(math.ceil(self.bias_far))) + 1
        idx = torch.tensor([log_distance_bucket(n, rows, self.bias_far) for n in range(reach + 1)], device=self.rel.device)
        if int(idx[-1]) != rows - 1:
            raise ValueError("the distance bias does not reach its last row")
        self.bias_lut = self.rel.index_select(0, idx).t().contiguous()

    def forward(self, out: torch.Tensor, q, k, v, gate, cache, batch: StepBatch, out_scale: float = 1.0) -> None:
        k_cache, v_cache = cache
        mops.paged_kv_write(k_cache, v_cache, k, v, batch.slot_mapping)
        mops.distance_bias_attention(out, q, gate, k_cache, v_cache, batch.block_tables, batch.q_start, batch.q_len,
                                     batch.ctx_len, batch.seq_of_token, (min(batch.q_lens), max(batch.q_lens)), self.heads,
                                     self.scale, self.bias_lut, self.temp_coef, self.temp_every, out_scale,
                                     max_kv_len=max(c + n for c, n in zip(batch.ctx_lens, batch.q_lens)))


class OuterProductMemory(nn.Module):
    def __init__(self, mode: int, heads: int, dim: int, vdim: int, decay: Optional[List[float]] = None,
                 q_scale: float = 1.0, gate_cap: float = 1.0):
        super().__init__()
        self.mode, self.heads, self.dim, self.vdim = mode, heads, dim, vdim
        self.q_scale, self.gate_cap = float(q_scale), float(gate_cap)
        if mode == mops.MEMORY_DECAY:
            if decay is None or len(decay) != heads:
                raise ValueError("decay linear attention takes one decay per head")
            self.register_buffer("decay", torch.tensor(decay, dtype=torch.float32), persistent=False)
        else:
            self.decay = None

    def cache_spec(self) -> MemoryStateSpec:
        return MemoryStateSpec(self.heads, self.dim, self.vdim, self.mode)

    def forward(self, q, k, v, state, batch: StepBatch, gate_i=None, gate_f=None) -> torch.Tensor:
        return mops.outer_memory_scan(q, k, v, state, batch.state_slots, batch.q_start, batch.q_len, batch.ctx_len,
                                      self.heads, self.mode, self.decay, gate_i, gate_f, self.q_scale, self.gate_cap,
                                      max_q_len=max(batch.q_lens))


class GatedMLP(nn.Module):
    """down(act(gate x) * (up x)) with gate and up as one product."""

    def __init__(self, width: int, ff: int, act: int, dtype, prefix: str = ""):
        super().__init__()
        from .model import QuantLinear
        self.act = act
        self.gate_up = QuantLinear(width, [ff, ff], None, dtype, prefix=prefix + "gate_up")
        self.down = QuantLinear(ff, [width], None, dtype, prefix=prefix + "down")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(mops.act_and_mul(self.gate_up(h), self.act))
