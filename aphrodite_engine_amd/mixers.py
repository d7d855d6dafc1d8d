"""Sequence-mixer building blocks beside the rotary softmax attention of ``attention/``: each is a mechanism with its
constants as parameters, says what cache it needs per layer run (``cache_spec``), and runs on a ``StepBatch`` -- prompt
portions and decoded tokens in one launch -- through the kernels of ``mixer_ops``.

  DistanceBiasAttention   grouped-query softmax attention over a token-major paged cache; no rotation: positions enter as
                          an additive per-head bias looked up by (bucketed) distance and as a query temperature that
                          grows with the logarithm of the position; optional per-head sigmoid output gate
  OuterProductMemory      a matrix state per head in a per-request slot: decay linear attention (fixed per-head decay) or
                          the mLSTM cell (exponential gating under a running maximum, normaliser vector)
  LayerNormParams, GatedMLP  the norm with weight and bias around an fp32 residual stream; gate * up feed-forward
  WindowedMapsAttention   softmax attention under a sliding window that keeps the sequence's first tokens, no rotation, with a
                          short causal convolution over time on q, k and v (its last inputs in a per-request slot) and
                          several maps per head over shared values, joined differentially (a_1 - lambda a_2), unit RMS per
                          head, elementwise sigmoid gate; may read another layer's keys and values instead of its own
  PolyNormMLP             down(a N(z) + b N(z^2) + c N(z^3) + e), z = up(x), N = division by the row's root mean square
  RoutedExperts           softmax router with a choice correction, clamped gated experts, identity experts, gated shared expert
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
    """A token-major paged key / value cache: K [blocks, block, kv_heads * maps, dim], V [blocks, block, kv_heads, vdim]
    (``maps`` key rows per kv head share one value row: the maps of differential attention)."""
    kv_heads: int
    dim: int
    vdim: int
    maps: int = 1

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return (torch.zeros(num_blocks, block_size, self.kv_heads * self.maps, self.dim, dtype=dtype, device=device),
                torch.zeros(num_blocks, block_size, self.kv_heads, self.vdim, dtype=dtype, device=device))


@dataclass(frozen=True)
class ConvStateSpec:
    """The last taps - 1 inputs of a short causal convolution over ``channels`` channels, one entry per request slot."""
    channels: int
    taps: int

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return torch.zeros(num_slots, max(self.taps - 1, 0), self.channels, dtype=dtype, device=device)


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


class WindowedMapsAttention(nn.Module):
    """The mechanism only: takes the rows of the fused input product [q | k | v | ...] and leaves the gated, normed head
    outputs; the projections around it belong to the model.  ``own_kv`` False: the layer has queries only and attends over
    the cache another layer wrote (same head counts and sizes)."""

    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int, keep_first: int, taps: int,
                 diff: float, eps: float, dtype, maps: int = 2, own_kv: bool = True):
        super().__init__()
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads over {kv_heads} key/value heads")
        if maps not in (1, 2):
            raise ValueError("one map (plain attention) or two (differential attention)")
        if taps < 1:
            raise ValueError("a convolution has at least one tap")
        self.heads, self.kv_heads, self.dim, self.vdim, self.maps = heads, kv_heads, dim, vdim, maps
        self.scale, self.window, self.keep_first, self.taps = float(scale), int(window), int(keep_first), int(taps)
        self.diff, self.eps, self.own_kv = float(diff), float(eps), own_kv
        self.cq = heads * maps * dim
        self.ck = kv_heads * maps * dim if own_kv else 0
        self.cv = kv_heads * vdim if own_kv else 0
        self.channels = self.cq + self.ck + self.cv
        self.conv = nn.Parameter(torch.zeros(self.channels, taps, dtype=dtype), requires_grad=False)
        # lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number per layer, fp32 (finalize)
        self.lq1, self.lk1, self.lq2, self.lk2 = (nn.Parameter(torch.zeros(dim, dtype=torch.float32), requires_grad=False)
                                                  for _ in range(4))
        self.lam = 0.0

    def kv_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.kv_heads, self.dim, self.vdim, self.maps)

    def state_spec(self) -> ConvStateSpec:
        return ConvStateSpec(self.channels, self.taps)

    def finalize(self) -> None:
        if self.maps == 2:
            self.lam = float(torch.exp(torch.dot(self.lq1.float(), self.lk1.float()))
                             - torch.exp(torch.dot(self.lq2.float(), self.lk2.float()))) + self.diff

    def forward(self, out: torch.Tensor, qkv: torch.Tensor, gate: Optional[torch.Tensor], kv_cache, conv_state,
                batch: StepBatch) -> None:
        """qkv [T, channels] rows of the input product (q only for a layer that shares another's cache); gate [T, heads * vdim]
        raw; out [T, heads * vdim]."""
        k_cache, v_cache = kv_cache
        q = mops.short_conv(qkv, self.conv, conv_state, batch.state_slots, batch.q_start, batch.q_len, batch.ctx_len,
                            batch.seq_of_token, self.cq, self.ck, self.cv, k_cache if self.own_kv else None,
                            v_cache if self.own_kv else None, batch.slot_mapping if self.own_kv else None)
        lens = (min(batch.q_lens), max(batch.q_lens))
        if self.maps == 2 and mops.differential_window_attention_supported(self.heads, self.kv_heads, self.dim, self.vdim, q.dtype) \
                and (gate is None or gate.stride(0) % 4 == 0):
            mops.differential_window_attention(out, q, gate, k_cache, v_cache, batch.block_tables, batch.q_start, batch.q_len,
                                               batch.ctx_len, batch.seq_of_token, lens, self.heads, self.scale, self.window,
                                               self.keep_first, self.lam, 1.0 - self.diff, self.eps,
                                               max_kv_len=max(c + n for c, n in zip(batch.ctx_lens, batch.q_lens)))
            return
        a = mops.windowed_attention(q, k_cache, v_cache, batch.block_tables, batch.q_start, batch.q_len, batch.ctx_len,
                                    batch.seq_of_token, (min(batch.q_lens), max(batch.q_lens)), self.heads, self.maps, self.scale,
                                    self.window, self.keep_first,
                                    max_kv_len=max(c + n for c, n in zip(batch.ctx_lens, batch.q_lens)))
        mops.differential_norm_gate(out, a, gate, self.heads, self.maps, self.vdim, self.lam,
                                    1.0 - self.diff if self.maps == 2 else 1.0, self.eps)


class PolyNormMLP(nn.Module):
    def __init__(self, width: int, ff: int, eps: float, dtype, prefix: str = ""):
        super().__init__()
        from .model import QuantLinear
        self.eps = float(eps)
        self.up = QuantLinear(width, [ff], None, dtype, prefix=prefix + "up")
        self.down = QuantLinear(ff, [width], None, dtype, prefix=prefix + "down")
        self.act = nn.Parameter(torch.zeros(4, dtype=torch.float32), requires_grad=False)
        self.coef = (0.0, 0.0, 0.0, 0.0)

    def finalize(self) -> None:
        self.coef = tuple(float(c) for c in self.act.tolist())

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(mops.poly_norm(self.up(h), self.coef, self.eps))


class RoutedExperts(nn.Module):
    """``experts`` clamped gated feed-forwards of which a token uses ``top``, chosen by softmax score plus a correction and
    weighted by the score itself; the last ``identity`` router outputs stand for experts that return their input; an optional
    shared expert runs for every token, times sigmoid of a one-row product.  The router runs in fp32."""

    def __init__(self, width: int, ff: int, experts: int, top: int, identity: int, limit: float, dtype, shared_ff: int = 0,
                 shared_limit: float = 0.0, alpha: float = 1.702, prefix: str = ""):
        super().__init__()
        from .model import QuantLinear
        self.width, self.ff, self.experts, self.top, self.identity = width, ff, experts, top, identity
        self.limit, self.alpha, self.shared_ff, self.shared_limit = float(limit), float(alpha), shared_ff, float(shared_limit)
        if not 0 < top <= experts + identity:
            raise ValueError(f"top {top} of {experts} + {identity} experts")
        self.router = nn.Parameter(torch.zeros(experts + identity, width, dtype=torch.float32), requires_grad=False)
        self.correction = nn.Parameter(torch.zeros(experts + identity, dtype=torch.float32), requires_grad=False)
        self.w_gate_up = nn.Parameter(torch.zeros(experts, 2 * ff, width, dtype=dtype), requires_grad=False)
        self.w_down = nn.Parameter(torch.zeros(experts, width, ff, dtype=dtype), requires_grad=False)
        if shared_ff:
            # [gate | up | the one-row gate | zero rows up to a multiple of 8]: one product for everything that reads h
            self.shared_splits = [shared_ff, shared_ff, 1, (-(2 * shared_ff + 1)) % 8 or 8]
            self.shared_in = QuantLinear(width, self.shared_splits, None, dtype, prefix=prefix + "shared.in")
            self.shared_in.weight.data.zero_()
            self.shared_down = QuantLinear(shared_ff, [width], None, dtype, prefix=prefix + "shared.down")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        z = torch.nn.functional.linear(h.float(), self.router)
        ids, w = mops.experts_route(z, self.correction, self.top)
        shared = gate = None
        if self.shared_ff:
            s_in = self.shared_in(h)
            shared = self.shared_down(mops.clamped_glu(s_in, self.shared_ff, self.shared_limit, self.alpha))
            gate = s_in[:, 2 * self.shared_ff:2 * self.shared_ff + 1]
        return mops.experts_forward(h, ids, w, self.w_gate_up, self.w_down, self.limit, self.alpha, shared, gate)
