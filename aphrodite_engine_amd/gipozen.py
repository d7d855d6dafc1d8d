"""Gipozen: a pre-norm decoder around an fp32 residual stream whose layers are joined by a learned average over depth.

  X_0 = embed[token]
  layer i:   x += mixer(norm1(x));  x += ff(norm2(x))  (the second only if the layer has a feed-forward);  X_(i+1) = x
             x = sum_{j <= i+1} dwa_i[j] X_j           -- what the next layer (and, after the last one, the output) reads
  logits = head norm_final(x) * logit_scale

Every norm is an RMS norm with ONE learned number as its gain.  The mixer is ``WindowedMapsAttention`` (mixers.py): differential
attention without rotation under a sliding window that keeps the first tokens, a short causal convolution on q, k and v, unit
RMS per head and an elementwise sigmoid gate; a layer may read another layer's keys and values.  The feed-forward is
``PolyNormMLP`` or ``RoutedExperts``.  Everything the checkpoint's config.json can vary is read from it; nothing here depends on
particular sizes.  Norm statistics, scores, the router, the depth average and the residual are fp32 also in a bfloat16 model.

One launch (``depth_residual_rms_norm``) folds a sublayer's residual add, the depth average at a layer's end and the RMS norm
that feeds the next sublayer.  The projections that read a mixer's input -- q, k, v and the output gate -- are one product."""
from dataclasses import dataclass
from typing import Any, Dict, Iterable, List, Optional, Tuple

import torch
from torch import nn
from torch.nn import functional as F

from . import mixer_ops as mops
from .mixers import PolyNormMLP, RoutedExperts, WindowedMapsAttention
from .step_batch import StepBatch


@dataclass
class GipozenConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: List[Dict[str, Any]]

    @staticmethod
    def from_dict(c: Dict[str, Any]) -> "GipozenConfig":
        cfg = GipozenConfig(vocab=int(c["vocab"]), width=int(c["width"]), eps=float(c["norm"]["eps"]),
                            logit_scale=float(c.get("logit_scale", 1.0)), layers=list(c["layers"]))
        for i, lc in enumerate(cfg.layers):
            if lc["type"] != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            src = lc["mixer"].get("kv_from")
            if src is not None:
                src = int(src)
                if not 0 <= src < i or cfg.layers[src]["mixer"].get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from {src} is not an earlier layer with keys and values of its own")
                a, b = lc["mixer"], cfg.layers[src]["mixer"]
                if any(int(a[k]) != int(b[k]) for k in ("kv_heads", "dim", "vdim")):
                    raise ValueError(f"layer {i}: its key / value sizes differ from layer {src}'s")
        return cfg


def _linear(width_in: int, outs: List[int], dtype, prefix: str):
    from .loader import merged_plan
    from .model import QuantLinear
    lin = QuantLinear(width_in, outs, None, dtype, prefix=prefix, plan=merged_plan(outs))
    lin.weight.data.zero_()
    return lin


class GipozenMixer(nn.Module):
    """[q | k | v | g] (or [q | g] over another layer's cache) as one input product, WindowedMapsAttention, output product."""

    def __init__(self, width: int, mc: Dict[str, Any], eps: float, dtype, prefix: str):
        super().__init__()
        H, G, d, e = int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"])
        mask = mc.get("mask") or {}
        self.kv_from = None if mc.get("kv_from") is None else int(mc["kv_from"])
        self.attn = WindowedMapsAttention(H, G, d, e, float(mc["scale"]), int(mask.get("size", 0)), int(mask.get("keep_first", 0)),
                                          int(mc.get("conv", 1)), float(mc["diff"]), eps, dtype, maps=2,
                                          own_kv=self.kv_from is None)
        a = self.attn
        self.names = ["q"] + (["k", "v"] if a.own_kv else []) + ["g"]
        self.splits = [a.cq] + ([a.ck, a.cv] if a.own_kv else []) + [H * e]
        pad = -sum(self.splits) % 8               # rows of the fused product stay 16-byte multiples
        if pad:
            self.splits.append(pad)
        self.in_proj = _linear(width, self.splits, dtype, prefix + "in_proj")
        self.out_proj = _linear(H * e, [width], dtype, prefix + "out_proj")
        self.gate_at = a.channels

    def forward(self, h: torch.Tensor, kv_cache, conv_state, batch: StepBatch) -> torch.Tensor:
        a = self.attn
        proj = self.in_proj(h)
        o = torch.empty(h.shape[0], a.heads * a.vdim, dtype=h.dtype, device=h.device)
        a(o, proj[:, :a.channels], proj[:, self.gate_at:self.gate_at + a.heads * a.vdim], kv_cache, conv_state, batch)
        return self.out_proj(o)


class GipozenLayer(nn.Module):
    def __init__(self, cfg: GipozenConfig, index: int, dtype):
        super().__init__()
        lc = cfg.layers[index]
        pfx = f"l{index}."
        self.mix = GipozenMixer(cfg.width, lc["mixer"], cfg.eps, dtype, pfx + "mix.")
        self.norm1 = nn.Parameter(torch.ones((), dtype=torch.float32), requires_grad=False)
        self.norm2 = nn.Parameter(torch.ones((), dtype=torch.float32), requires_grad=False)
        self.dwa = nn.Parameter(torch.zeros(index + 2, dtype=torch.float32), requires_grad=False)
        mlp = lc.get("mlp")
        self.mlp = None
        if mlp is not None and mlp["kind"] == "dense":
            self.mlp = PolyNormMLP(cfg.width, int(mlp["ff"]), cfg.eps, dtype, pfx + "mlp.")
        elif mlp is not None:
            r, sh = mlp["router"], mlp.get("shared")
            self.mlp = RoutedExperts(cfg.width, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), int(r.get("identity", 0)),
                                     float(mlp["expert"]["limit"]), dtype, shared_ff=int(sh["ff"]) if sh else 0,
                                     shared_limit=float(sh["limit"]) if sh else 0.0, prefix=pfx + "mlp.")
        self.gain1 = self.gain2 = 1.0


class GipozenForCausalLM(nn.Module):
    def __init__(self, cfg: GipozenConfig, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        from .distributed import get_tensor_model_parallel_world_size
        if get_tensor_model_parallel_world_size() != 1:
            raise ValueError("Gipozen runs on one rank")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Gipozen runs in bfloat16 or float32")
        self.cfg, self.dtype = cfg, dtype
        self.embed = nn.Parameter(torch.empty(cfg.vocab, cfg.width, dtype=dtype), requires_grad=False)
        self.layers = nn.ModuleList([GipozenLayer(cfg, i, dtype) for i in range(len(cfg.layers))])
        self.final_norm = nn.Parameter(torch.ones((), dtype=torch.float32), requires_grad=False)
        self.head = nn.Parameter(torch.empty(cfg.vocab, cfg.width, dtype=dtype), requires_grad=False)
        self.final_gain = 1.0
        # caches: a layer owns its convolution state; its paged keys and values are its own or an earlier layer's
        self.specs, self.kv_index, self.state_index = [], [], []
        for i, layer in enumerate(self.layers):
            a = layer.mix.attn
            if a.own_kv:
                self.kv_index.append(len(self.specs))
                self.specs.append(a.kv_spec())
            else:
                self.kv_index.append(self.kv_index[layer.mix.kv_from])
            self.state_index.append(len(self.specs))
            self.specs.append(a.state_spec())
        self.residual_trace: Optional[List[torch.Tensor]] = None     # set to [] to record x after every layer

    # ---- what the engine asks of a model ---------------------------------------------------------------------------
    @property
    def vocab_size(self) -> int:
        return self.cfg.vocab

    def make_caches(self, num_blocks: int, block_size: int, num_slots: int, device):
        return [s.allocate(num_blocks, block_size, num_slots, self.dtype, device) for s in self.specs]

    def finalize(self):
        for layer in self.layers:
            layer.mix.attn.finalize()
            if isinstance(layer.mlp, PolyNormMLP):
                layer.mlp.finalize()
            layer.gain1, layer.gain2 = float(layer.norm1), float(layer.norm2)
        self.final_gain = float(self.final_norm)
        return self

    @torch.no_grad()
    def step(self, batch: StepBatch, caches, rows: torch.Tensor) -> torch.Tensor:
        """One engine step: run the batch's rows through every layer (caches and states advance), return the fp32 logits of
        ``rows`` (int64 indices into the batch)."""
        h = self.forward(batch, caches)
        return self.logits(h.index_select(0, rows))

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.head).float() * self.cfg.logit_scale

    def forward(self, batch: StepBatch, caches) -> torch.Tensor:
        """The final norm's output for every row of the batch."""
        cfg, eps, T = self.cfg, self.cfg.eps, batch.num_tokens
        L = len(self.layers)
        dev = batch.input_ids.device
        history = torch.empty(L + 1, T, cfg.width, dtype=torch.float32, device=dev)
        x = torch.empty(T, cfg.width, dtype=torch.float32, device=dev)
        mops.embed_scale(self.embed, batch.input_ids, 1.0, out=history[0])
        h = mops.depth_residual_rms_norm(history[0], x_out=x, gain=self.layers[0].gain1, eps=eps, dtype=self.dtype)
        for i, layer in enumerate(self.layers):
            y = layer.mix(h, caches[self.kv_index[i]], caches[self.state_index[i]], batch)
            if layer.mlp is not None:
                h = mops.depth_residual_rms_norm(x, x_out=x, y=y, gain=layer.gain2, eps=eps)
                y = layer.mlp(h)
            gain = self.layers[i + 1].gain1 if i + 1 < L else self.final_gain
            h = mops.depth_residual_rms_norm(x, x_out=x, y=y, history=history, n_hist=i + 1, depth_w=layer.dwa, gain=gain, eps=eps)
            if self.residual_trace is not None:
                self.residual_trace.append(x.clone())
        return h

    # ---- checkpoint ----------------------------------------------------------------------------------------------------
    def expected_names(self) -> List[str]:
        names = ["embed", "head", "final.norm"]
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            names += [p + "norm1", p + "dwa"] + [p + "mix." + n for n in layer.mix.names + ["o", "lq1", "lk1", "lq2", "lk2"]]
            names += [p + "mix." + n + ".conv" for n in layer.mix.names if n != "g"]
            m = layer.mlp
            if m is not None:
                names.append(p + "norm2")
            if isinstance(m, PolyNormMLP):
                names += [p + "mlp." + n for n in ("up", "down", "act")]
            elif isinstance(m, RoutedExperts):
                names += [p + "mlp.router", p + "mlp.correction"]
                names += [f"{p}mlp.e{e}.{n}" for e in range(m.experts) for n in ("gate", "up", "down")]
                if m.shared_ff:
                    names += [p + "mlp.shared." + n for n in ("gate", "up", "down", "sg")]
        return names

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> None:
        """Checkpoint names: embed, head, final.norm, l<i>.norm{1,2}, l<i>.dwa, l<i>.mix.{q,k,v}[.conv], l<i>.mix.{g,o,lq1,lk1,
        lq2,lk2}, l<i>.mlp.{up,down,act} or l<i>.mlp.{router,correction,e<j>.{gate,up,down},shared.{gate,up,down,sg}}."""
        expected, seen = set(self.expected_names()), set()
        # a second norm's gain of a layer that has no feed-forward is never used: accepted and left aside
        unused = {f"l{i}.norm2" for i, layer in enumerate(self.layers) if layer.mlp is None}
        for name, t in weights:
            if name in unused:
                continue
            if name not in expected:
                raise ValueError(f"unexpected tensor {name!r} in a Gipozen checkpoint")
            seen.add(name)
            self._load_one(name, t)
        missing = expected - seen
        if "head" in missing:                    # no output matrix of its own: the embedding's
            self.head = self.embed
            missing.discard("head")
        missing -= {n for n in missing if n.endswith(".mlp.correction")}      # no correction: the scores alone choose
        if missing:
            raise ValueError(f"checkpoint lacks {len(missing)} tensors, e.g. {sorted(missing)[:4]}")

    @staticmethod
    def _put(dst: torch.Tensor, t: torch.Tensor, name: str) -> None:
        if tuple(dst.shape) != tuple(t.shape):
            raise ValueError(f"{name}: checkpoint tensor {tuple(t.shape)} does not fit {tuple(dst.shape)}")
        dst.copy_(t.to(dst.dtype))

    def _load_one(self, name: str, t: torch.Tensor) -> None:
        put = self._put
        if name in ("embed", "head"):
            return put(getattr(self, name).data, t, name)
        if name == "final.norm":
            return put(self.final_norm.data, t.reshape(()), name)
        first, rest = name.split(".", 1)
        layer = self.layers[int(first[1:])]
        if rest in ("norm1", "norm2"):
            return put(getattr(layer, rest).data, t.reshape(()), name)
        if rest == "dwa":
            return put(layer.dwa.data, t, name)
        if rest.startswith("mix."):
            key, mix = rest[4:], layer.mix
            a = mix.attn
            if key.endswith(".conv"):
                at = sum(mix.splits[:mix.names.index(key[:-5])])
                n = mix.splits[mix.names.index(key[:-5])]
                if t.dim() != 2 or t.shape[1] != a.taps:
                    raise ValueError(f"{name}: {tuple(t.shape)} is not [channels, {a.taps} taps]")
                return put(a.conv.data[at:at + n], t, name)
            if key in mix.names:
                lin = mix.in_proj
                return lin.weight_loader(lin.weight, t.to(lin.weight.dtype), mix.names.index(key))
            if key == "o":
                return mix.out_proj.weight_loader(mix.out_proj.weight, t.to(mix.out_proj.weight.dtype), 0)
            return put(getattr(a, key).data, t, name)
        key, m = rest[4:], layer.mlp
        if isinstance(m, PolyNormMLP):
            if key == "act":
                return put(m.act.data, t, name)
            lin = getattr(m, key)
            return lin.weight_loader(lin.weight, t.to(lin.weight.dtype), 0)
        if key in ("router", "correction"):
            return put(getattr(m, key).data, t, name)
        who, part = key.split(".", 1)
        if who == "shared":
            if part == "down":
                return m.shared_down.weight_loader(m.shared_down.weight, t.to(m.shared_down.weight.dtype), 0)
            lin = m.shared_in
            return lin.weight_loader(lin.weight, t.to(lin.weight.dtype), {"gate": 0, "up": 1, "sg": 2}[part])
        e = int(who[1:])
        if part == "down":
            return put(m.w_down.data[e], t, name)
        return put(m.w_gate_up.data[e, :m.ff] if part == "gate" else m.w_gate_up.data[e, m.ff:], t, name)

    @torch.no_grad()
    def init_synthetic(self, device, seed: int = 0):
        """Random weights of a checkpoint's scale on the device (benchmarks, tests)."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        self.to(device)
        for name, p in self.named_parameters():
            if p.dim() >= 2 and not name.endswith("attn.conv"):
                std = 1.0 if name == "embed" else p.shape[-1] ** -0.5
                p.copy_((torch.randn(p.shape, generator=g) * std).to(p.dtype))
            elif name.endswith("attn.conv"):
                p.copy_((torch.randn(p.shape, generator=g) * p.shape[1] ** -0.5).to(p.dtype))
            elif "norm" in name:
                p.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
            elif name.endswith("dwa"):
                w = 0.1 * torch.randn(p.shape, generator=g)
                w[-1] += 1.0
                p.copy_(w)
            elif name.endswith("mlp.act"):
                p.copy_(torch.tensor([1.0, 0.5, 0.25, 0.0]) + 0.1 * torch.randn(4, generator=g))
            else:
                p.copy_((0.1 * torch.randn(p.shape, generator=g)).to(p.dtype))
        for layer in self.layers:               # the fused products' padding rows stay zero
            lin = layer.mix.in_proj
            lin.weight.data[sum(layer.mix.splits[:len(layer.mix.names)]):].zero_()
            if isinstance(layer.mlp, RoutedExperts) and layer.mlp.shared_ff:
                layer.mlp.shared_in.weight.data[2 * layer.mlp.shared_ff + 1:].zero_()
        return self.finalize()


def load_gipozen(model_dir: str, hf: Dict[str, Any], dtype: torch.dtype, device, **_unused) -> GipozenForCausalLM:
    from .loader import iter_safetensors
    model = GipozenForCausalLM(GipozenConfig.from_dict(hf), dtype)
    model.load_weights(iter_safetensors(model_dir))
    model.to(device)
    return model.finalize()
