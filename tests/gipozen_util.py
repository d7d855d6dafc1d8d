"""Small random Gipozen checkpoints for the tests: a config dict, numpy weights named as in a checkpoint, and a writer of
config.json + model.safetensors.  Sizes are deliberately unlike one another (dim != vdim, heads != kv heads, a width that is no
power of two, layers that differ in window, kept tokens, taps and constants) so that a swapped size or a constant taken from
the wrong layer shows."""
import json
import os

import numpy as np
import torch

from fatudra_util import bf16_round, logit_errors  # noqa: F401


def attention_layer(heads=6, kv_heads=2, dim=24, vdim=40, window=23, keep_first=3, taps=3, diff=0.2, scale=None, kv_from=None,
                    mlp="dense", ff=88, experts=5, identity=1, top=2, limit=1.25, shared_ff=56, shared_limit=2.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps, "diff": diff,
         "mask": {"size": window, "keep_first": keep_first}, "scale": scale if scale is not None else dim ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    if mlp == "dense":
        f = {"kind": "dense", "ff": ff}
    elif mlp == "moe":
        f = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "identity": identity, "top": top}}
        if shared_ff:
            f["shared"] = {"ff": shared_ff, "limit": shared_limit}
    else:
        f = None
    return {"type": "attention", "mixer": m, "mlp": f}


def make_config(layers, vocab=131, width=72, eps=1e-5, logit_scale=0.7):
    return {"architecture": "Gipozen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "layers": layers}


def make_weights(cfg, seed=0, round_bf16=True):
    rng = np.random.default_rng(seed)
    W, width = {}, cfg["width"]

    def mat(o, i, gain=1.0):
        return rng.standard_normal((o, i)) * gain / np.sqrt(i)

    W["embed"] = rng.standard_normal((cfg["vocab"], width))
    W["head"] = mat(cfg["vocab"], width)
    W["final.norm"] = np.array(0.8 + 0.4 * rng.random())
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = lc["mixer"]
        H, G, d, e, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        W[p + "norm1"] = np.array(0.8 + 0.4 * rng.random())
        W[p + "mix.q"] = mat(H * 2 * d, width, 2.5)
        W[p + "mix.q.conv"] = rng.standard_normal((H * 2 * d, taps)) / np.sqrt(taps)
        if m.get("kv_from") is None:
            W[p + "mix.k"], W[p + "mix.v"] = mat(G * 2 * d, width, 2.5), mat(G * e, width)
            W[p + "mix.k.conv"] = rng.standard_normal((G * 2 * d, taps)) / np.sqrt(taps)
            W[p + "mix.v.conv"] = rng.standard_normal((G * e, taps)) / np.sqrt(taps)
        for n in ("lq1", "lk1", "lq2", "lk2"):
            W[p + "mix." + n] = rng.standard_normal(d) * 0.3
        W[p + "mix.g"], W[p + "mix.o"] = mat(H * e, width), mat(width, H * e)
        f = lc["mlp"]
        if f is not None:
            W[p + "norm2"] = np.array(0.8 + 0.4 * rng.random())
        if f is not None and f["kind"] == "dense":
            W[p + "mlp.up"], W[p + "mlp.down"] = mat(f["ff"], width), mat(width, f["ff"])
            W[p + "mlp.act"] = np.array([0.7, 0.5, 0.3, 0.1]) + 0.1 * rng.standard_normal(4)
        elif f is not None:
            r = f["router"]
            E, R = r["experts"], r["experts"] + r.get("identity", 0)
            W[p + "mlp.router"] = mat(R, width, 3.0)
            W[p + "mlp.correction"] = rng.standard_normal(R) * 0.1
            for j in range(E):
                pe = f"{p}mlp.e{j}."
                W[pe + "gate"], W[pe + "up"] = mat(f["expert"]["ff"], width, 2.0), mat(f["expert"]["ff"], width, 2.0)
                W[pe + "down"] = mat(width, f["expert"]["ff"])
            if f.get("shared"):
                sf = f["shared"]["ff"]
                W[p + "mlp.shared.gate"], W[p + "mlp.shared.up"] = mat(sf, width, 2.0), mat(sf, width, 2.0)
                W[p + "mlp.shared.down"], W[p + "mlp.shared.sg"] = mat(width, sf), mat(1, width, 2.0)
        w = rng.standard_normal(i + 2) * 0.15
        w[-1] += 1.0
        W[p + "dwa"] = w
    if round_bf16:
        W = {k: bf16_round(v) for k, v in W.items()}
    return {k: np.asarray(v, np.float32) for k, v in W.items()}


def write_checkpoint(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: torch.from_numpy(np.ascontiguousarray(v)).to(torch.bfloat16).contiguous() for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
    return path


def assert_logits(got, want, sharp, what=""):
    """``sharp`` (float32 runs): every position within 2e-4 of the logits' spread.  bfloat16 against the unrounded restatement:
    the typical position within the rounding of a few bfloat16 layers and no more than a tenth of them far off -- with random
    weights a router's choice now and then rests on a margin smaller than that rounding, and the other expert's output is a
    different one; a bound on the worst position cannot tell that from a fault, the float32 run of the same test can."""
    e = logit_errors(got, want)
    assert np.isfinite(e).all(), what
    if sharp:
        assert e.max() < 2e-4, (what, float(e.max()), int(e.argmax()))
    else:
        assert np.median(e) < 0.04 and np.quantile(e, 0.9) < 0.15, (what, float(np.median(e)), float(np.quantile(e, 0.9)))
