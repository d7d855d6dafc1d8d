"""Fatudra: a decoder built from the mixers of ``mixers.py`` around an fp32 residual stream.

  x = embed[token] * scale
  per layer run:   x += LN_1b(mixer(LN_1(x)));   x += LN_2b(mlp(LN_2(x)))   (the second only if the layer has an mlp)
  logits = head LN_final(x)

A layer's mixer is either ``parallel`` -- DistanceBiasAttention and a decay-linear-attention memory side by side on the same
input, summed with fixed weights -- or ``mlstm``.  A contiguous range of layers may be looped: it runs ``times`` times with
the same weights, every pass with its own cache / state and a learned per-pass vector added to x before its first layer.
So the unit that owns a cache is the LAYER RUN, not the layer (``FatudraConfig.schedule``).

Everything the checkpoint's config.json can vary is read from it; nothing here depends on particular sizes.  The fused
projections (one product for every matrix that reads the mixer's input, one for the output projections of both branches)
are assembled at load time.  Norm statistics, scores, gates, states and the residual are fp32 also in a bfloat16 model."""
from dataclasses import dataclass
from typing import Any, Dict, Iterable, List, Optional, Tuple

import torch
from torch import nn
from torch.nn import functional as F

from . import mixer_ops as mops
from .mixers import DistanceBiasAttention, GatedMLP, LayerNormParams, OuterProductMemory
from .step_batch import StepBatch


@dataclass
class FatudraConfig:
    vocab: int
    width: int
    eps: float
    embed_scale: float
    layers: List[Dict[str, Any]]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0

    @staticmethod
    def from_dict(c: Dict[str, Any]) -> "FatudraConfig":
        loop = c.get("loop") or {}
        cfg = FatudraConfig(vocab=int(c["vocab"]), width=int(c["width"]), eps=float(c["norm"]["eps"]),
                            embed_scale=float(c["embedding"]["scale"]), layers=list(c["layers"]),
                            loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                            loop_times=int(loop.get("times", 0)))
        for i, lc in enumerate(cfg.layers):
            if lc["type"] not in ("parallel", "mlstm"):
                raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
            if lc.get("mlp") is not None and lc["mlp"].get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {lc['mlp'].get('kind')!r}")
        if cfg.looped and not (0 <= cfg.loop_start < cfg.loop_stop <= len(cfg.layers)):
            raise ValueError("loop range outside the layers")
        return cfg

    @property
    def looped(self) -> bool:
        return self.loop_times > 0 and self.loop_stop > self.loop_start

    def schedule(self) -> List[Tuple[int, Optional[int]]]:
        """(layer, pass) of every layer run in execution order; pass is None outside the loop."""
        n = len(self.layers)
        if not self.looped:
            return [(i, None) for i in range(n)]
        runs: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            runs += [(i, t) for i in range(self.loop_start, self.loop_stop)]
        return runs + [(i, None) for i in range(self.loop_stop, n)]


def _linear(width_in: int, outs: List[int], dtype, bias: bool, prefix: str):
    from .loader import merged_plan
    from .model import QuantLinear
    lin = QuantLinear(width_in, outs, None, dtype, prefix=prefix, plan=merged_plan(outs), bias=bias)
    lin.weight.data.zero_()
    return lin


def _padded(splits: List[int]) -> List[int]:
    """A last, never-loaded all-zero partition that makes the fused product's rows a multiple of 16 bytes: the column
    slices handed to the kernels then keep 16-byte-aligned rows whenever their own offsets do."""
    pad = -sum(splits) % 8
    return splits + [pad] if pad else list(splits)


class ParallelMixer(nn.Module):
    """left: DistanceBiasAttention with biased projections and a per-head output gate; right: decay linear attention with
    silu on q / k / v, a joint RMS norm over its heads and an elementwise sigmoid gate.  One input product
    [q k v g | q k v g], one output product over the concatenated, pre-scaled branch outputs."""

    def __init__(self, width: int, mc: Dict[str, Any], eps: float, dtype, prefix: str):
        super().__init__()
        L, R = mc["left"], mc["right"]
        self.eps = eps
        self.left_scale, self.right_scale = float(mc["left_scale"]), float(mc["right_scale"])
        H, G, d, e = int(L["heads"]), int(L["kv_heads"]), int(L["dim"]), int(L["vdim"])
        temp = L.get("q_temp") or {}
        self.attn = DistanceBiasAttention(H, G, d, e, float(L["scale"]), bias_rows=1, bias_far=float(L["bias_max"]),
                                          temp_coef=float(temp.get("coef", 0.0)), temp_every=int(temp.get("every", 1)))
        Hr, dr, er = int(R["heads"]), int(R["dim"]), int(R["vdim"])
        self.memory = OuterProductMemory(mops.MEMORY_DECAY, Hr, dr, er, decay=[float(x) for x in R["decay"]])
        self.splits = [H * d, G * d, G * e, H, Hr * dr, Hr * dr, Hr * er, Hr * er]
        self.names = ["left.q", "left.k", "left.v", "left.g", "right.q", "right.k", "right.v", "right.g"]
        self.splits = _padded(self.splits)
        self.in_proj = _linear(width, self.splits, dtype, True, prefix + "in_proj")
        self.left_out, self.right_out = H * e, Hr * er
        self.out_proj = _linear(self.left_out + self.right_out, [width], dtype, False, prefix + "out_proj")
        self.right_norm = nn.Parameter(torch.ones(self.right_out, dtype=dtype), requires_grad=False)
        self.left_out_bias = nn.Parameter(torch.zeros(width, dtype=torch.float32), requires_grad=False)
        self.out_bias = None        # fp32 left_scale * left_out_bias (finalize)

    def cache_specs(self):
        return [self.attn.cache_spec(), self.memory.cache_spec()]

    def finalize(self) -> None:
        self.attn.finalize()
        self.out_bias = (self.left_out_bias.float() * self.left_scale).contiguous()

    def forward(self, h: torch.Tensor, caches, batch: StepBatch) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        lq, lk, lv, lg, rq, rk, rv, rg = self.in_proj(h).split(self.splits, dim=-1)[:8]
        cat = torch.empty(h.shape[0], self.left_out + self.right_out, dtype=h.dtype, device=h.device)
        self.attn(cat[:, :self.left_out], lq, lk, lv, lg, caches[0], batch, out_scale=self.left_scale)
        o = self.memory(rq, rk, rv, caches[1], batch)
        mops.gated_group_rms_norm(cat[:, self.left_out:], o, self.right_norm, rg, self.right_out, self.eps, self.right_scale)
        return self.out_proj(cat), self.out_bias


class MLSTMMixer(nn.Module):
    """mLSTM cell: one input product [q k v g i f], per-head unit RMS, weight, sigmoid gate, output product."""

    def __init__(self, width: int, mc: Dict[str, Any], eps: float, dtype, prefix: str):
        super().__init__()
        H, d, e = int(mc["heads"]), int(mc["dim"]), int(mc["vdim"])
        self.eps, self.vdim = eps, e
        self.memory = OuterProductMemory(mops.MEMORY_MLSTM, H, d, e, q_scale=d ** -0.5, gate_cap=float(mc["gate_cap"]))
        self.splits = [H * d, H * d, H * e, H * e, H, H]
        self.names = ["q", "k", "v", "g", "i", "f"]
        self.splits = _padded(self.splits)
        self.in_proj = _linear(width, self.splits, dtype, True, prefix + "in_proj")
        self.out_proj = _linear(H * e, [width], dtype, False, prefix + "out_proj")
        self.norm = nn.Parameter(torch.ones(H * e, dtype=dtype), requires_grad=False)

    def cache_specs(self):
        return [self.memory.cache_spec()]

    def finalize(self) -> None:
        pass

    def forward(self, h: torch.Tensor, caches, batch: StepBatch) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        q, k, v, g, gi, gf = self.in_proj(h).split(self.splits, dim=-1)[:6]
        o = self.memory(q, k, v, caches[0], batch, gate_i=gi, gate_f=gf)
        normed = torch.empty(h.shape[0], o.shape[1], dtype=h.dtype, device=h.device)
        mops.gated_group_rms_norm(normed, o, self.norm, g, self.vdim, self.eps)
        return self.out_proj(normed), None


class FatudraLayer(nn.Module):
    def __init__(self, cfg: FatudraConfig, index: int, dtype):
        super().__init__()
        lc = cfg.layers[index]
        pfx = f"l{index}."
        kind = {"parallel": ParallelMixer, "mlstm": MLSTMMixer}[lc["type"]]
        self.mix = kind(cfg.width, lc["mixer"], cfg.eps, dtype, pfx + "mix.")
        self.norm1, self.norm1b = LayerNormParams(cfg.width, dtype), LayerNormParams(cfg.width, dtype)
        self.mlp = None
        if lc.get("mlp") is not None:
            self.mlp = GatedMLP(cfg.width, int(lc["mlp"]["ff"]), mops.ACT_GELU_TANH, dtype, pfx + "mlp.")
            self.norm2, self.norm2b = LayerNormParams(cfg.width, dtype), LayerNormParams(cfg.width, dtype)


class FatudraForCausalLM(nn.Module):
    def __init__(self, cfg: FatudraConfig, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        from .distributed import get_tensor_model_parallel_world_size
        if get_tensor_model_parallel_world_size() != 1:
            raise ValueError("Fatudra runs on one rank (its recurrent states are not sharded)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Fatudra runs in bfloat16 or float32")
        self.cfg, self.dtype = cfg, dtype
        self.embed = nn.Parameter(torch.empty(cfg.vocab, cfg.width, dtype=dtype), requires_grad=False)
        self.layers = nn.ModuleList([FatudraLayer(cfg, i, dtype) for i in range(len(cfg.layers))])
        self.loop_step = (nn.Parameter(torch.zeros(cfg.loop_times, cfg.width, dtype=dtype), requires_grad=False)
                          if cfg.looped else None)
        self.final_norm = LayerNormParams(cfg.width, dtype)
        self.head = nn.Parameter(torch.empty(cfg.vocab, cfg.width, dtype=dtype), requires_grad=False)
        self.runs = cfg.schedule()
        # cache index of every layer run: each run owns the caches its mixer names
        self.run_caches: List[List[int]] = []
        self.specs = []
        for li, _ in self.runs:
            idx = []
            for spec in self.layers[li].mix.cache_specs():
                idx.append(len(self.specs))
                self.specs.append(spec)
            self.run_caches.append(idx)
        self.residual_trace: Optional[List[torch.Tensor]] = None     # set to [] to record x after every layer run

    # ---- what the engine asks of a model ---------------------------------------------------------------------------
    @property
    def vocab_size(self) -> int:
        return self.cfg.vocab

    def make_caches(self, num_blocks: int, block_size: int, num_slots: int, device):
        return [s.allocate(num_blocks, block_size, num_slots, self.dtype, device) for s in self.specs]

    def finalize(self):
        for layer in self.layers:
            layer.mix.finalize()
        return self

    @torch.no_grad()
    def step(self, batch: StepBatch, caches, rows: torch.Tensor) -> torch.Tensor:
        """One engine step: run the batch's rows through every layer run (caches and states advance), return the fp32
        logits of ``rows`` (int64 indices into the batch)."""
        x, pend = self.forward(batch, caches)
        xs = x.index_select(0, rows)
        y, post, yb = pend
        h = mops.residual_layer_norm(xs, y=y.index_select(0, rows), post=post, y_bias=yb, pre=self.final_norm.pair(),
                                     eps=self.cfg.eps)
        return F.linear(h, self.head).float()

    def forward(self, batch: StepBatch, caches):
        """Returns the residual stream and the last sublayer's still-unadded output (y, its norm, its fp32 bias): every
        ``x += LN(y)`` rides in the launch that also produces the next sublayer's normed input."""
        cfg, eps = self.cfg, self.cfg.eps
        x = mops.embed_scale(self.embed, batch.input_ids, cfg.embed_scale)
        pend = None
        for run, (li, t) in enumerate(self.runs):
            layer = self.layers[li]
            add = self.loop_step[t] if (t is not None and li == cfg.loop_start) else None
            y, post, yb = pend if pend is not None else (None, None, None)
            h = mops.residual_layer_norm(x, y=y, post=post, y_bias=yb, add_vec=add, pre=layer.norm1.pair(), eps=eps,
                                         dtype=self.dtype)
            y, yb = layer.mix(h, [caches[i] for i in self.run_caches[run]], batch)
            pend = (y, layer.norm1b.pair(), yb)
            if layer.mlp is not None:
                h = mops.residual_layer_norm(x, y=y, post=pend[1], y_bias=yb, pre=layer.norm2.pair(), eps=eps)
                pend = (layer.mlp(h), layer.norm2b.pair(), None)
            if self.residual_trace is not None:
                mops.residual_layer_norm(x, y=pend[0], post=pend[1], y_bias=pend[2], eps=eps)
                self.residual_trace.append(x.clone())
                pend = None
        if pend is None:      # only when tracing: nothing left to add
            z = torch.zeros(x.shape[0], cfg.width, dtype=self.dtype, device=x.device)
            zero = (torch.zeros(cfg.width, dtype=self.dtype, device=x.device), ) * 2
            pend = (z, zero, None)
        return x, pend

    # ---- checkpoint ----------------------------------------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> None:
        """Checkpoint names: embed, head, final.norm[.b], loop.step, l<i>.norm{1,1b,2,2b}[.b], l<i>.mix.*, l<i>.mlp.*."""
        from .loader import default_weight_loader
        seen = set()
        expected = set(self.expected_names())
        for name, t in weights:
            if name not in expected:
                raise ValueError(f"unexpected tensor {name!r} in a Fatudra checkpoint")
            seen.add(name)
            self._load_one(name, t, default_weight_loader)
        missing = sorted(expected - seen)
        if missing:
            raise ValueError(f"checkpoint lacks {len(missing)} tensors, e.g. {missing[:4]}")

    def expected_names(self) -> List[str]:
        names = ["embed", "head", "final.norm", "final.norm.b"] + (["loop.step"] if self.loop_step is not None else [])
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            norms = ["norm1", "norm1b"] + (["norm2", "norm2b"] if layer.mlp is not None else [])
            names += [p + n + s for n in norms for s in ("", ".b")]
            if isinstance(layer.mix, ParallelMixer):
                names += [p + "mix." + n for n in layer.mix.names + ["left.q.b", "left.k.b", "left.v.b", "left.rel",
                                                                      "left.o", "left.o.b", "right.o", "right.norm"]]
            else:
                names += [p + "mix." + n for n in layer.mix.names + ["i.b", "f.b", "o", "norm"]]
            if layer.mlp is not None:
                names += [p + "mlp." + n for n in ("gate", "up", "down")]
        return names

    def _load_one(self, name: str, t: torch.Tensor, copy) -> None:
        def cast(p):
            return t.to(p.dtype)
        if name in ("embed", "head"):
            return copy(getattr(self, name), cast(getattr(self, name)))
        if name == "loop.step":
            return copy(self.loop_step, cast(self.loop_step))
        if name.startswith("final.norm"):
            p = self.final_norm.bias if name.endswith(".b") else self.final_norm.weight
            return copy(p, cast(p))
        head, rest = name.split(".", 1)
        layer = self.layers[int(head[1:])]
        if rest.startswith("norm"):
            ln = getattr(layer, rest[:-2] if rest.endswith(".b") else rest)
            p = ln.bias if rest.endswith(".b") else ln.weight
            return copy(p, cast(p))
        if rest.startswith("mlp."):
            key = rest[4:]
            if key == "down":
                return layer.mlp.down.weight_loader(layer.mlp.down.weight, cast(layer.mlp.down.weight), 0)
            lin = layer.mlp.gate_up
            return lin.weight_loader(lin.weight, cast(lin.weight), {"gate": 0, "up": 1}[key])
        key, mix = rest[4:], layer.mix
        is_bias = key.endswith(".b")
        base = key[:-2] if is_bias else key
        if base in mix.names:
            lin = mix.in_proj
            p = lin.bias if is_bias else lin.weight
            return lin.weight_loader(p, cast(p), mix.names.index(base))
        if isinstance(mix, ParallelMixer):
            if key == "left.rel":
                if t.dim() != 2 or t.shape[1] != mix.attn.heads:
                    raise ValueError(f"{name}: a [rows, heads] table expected, got {tuple(t.shape)}")
                mix.attn.rel = nn.Parameter(t.float().clone(), requires_grad=False)
                return None
            if key == "left.o.b":
                return copy(mix.left_out_bias, t.float())
            if key == "right.norm":
                return copy(mix.right_norm, cast(mix.right_norm))
            w = mix.out_proj.weight
            part = w.data[:, :mix.left_out] if key == "left.o" else w.data[:, mix.left_out:]
            if part.shape != t.shape:
                raise ValueError(f"{name}: checkpoint tensor {tuple(t.shape)} does not fit {tuple(part.shape)}")
            part.copy_(t.to(w.dtype))
            return None
        if key == "norm":
            return copy(mix.norm, cast(mix.norm))
        if key == "o":
            return mix.out_proj.weight_loader(mix.out_proj.weight, cast(mix.out_proj.weight), 0)
        raise ValueError(f"unexpected tensor {name!r}")

    @torch.no_grad()
    def init_synthetic(self, device, seed: int = 0, bias_rows: int = 32):
        """Random weights of the checkpoint's scale on the device (benchmarks, tests)."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        for layer in self.layers:
            if isinstance(layer.mix, ParallelMixer):
                layer.mix.attn.rel = nn.Parameter(torch.zeros(bias_rows, layer.mix.attn.heads), requires_grad=False)
        self.to(device)
        for name, p in self.named_parameters():
            if p.dim() >= 2:
                std = 1.0 if name == "embed" else p.shape[-1] ** -0.5
                p.copy_((torch.randn(p.shape, generator=g) * std).to(p.dtype))
            elif "norm" in name and not name.endswith("bias"):
                p.copy_((1.0 + 0.1 * torch.randn(p.shape, generator=g)).to(p.dtype))
            else:
                p.copy_((0.1 * torch.randn(p.shape, generator=g)).to(p.dtype))
        return self.finalize()


def load_fatudra(model_dir: str, hf: Dict[str, Any], dtype: torch.dtype, device, **_unused) -> FatudraForCausalLM:
    from .loader import iter_safetensors
    model = FatudraForCausalLM(FatudraConfig.from_dict(hf), dtype)
    model.load_weights(iter_safetensors(model_dir))
    model.to(device)
    return model.finalize()
