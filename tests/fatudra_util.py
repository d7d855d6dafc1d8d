"""Small random Fatudra checkpoints for the tests: a config dict, numpy weights named as in a checkpoint, and a writer
of config.json + model.safetensors.  Sizes are deliberately unlike one another (dim != vdim, heads != kv heads, width
not a power of two) so that a swapped size shows."""
import json
import os

import numpy as np
import torch


def bf16_round(a):
    return torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16).float().numpy()


def parallel_layer(heads=4, kv_heads=2, dim=24, vdim=40, rheads=3, rdim=20, rvdim=72, ff=96, bias_max=50, every=16, coef=0.5,
                   decay=None, scale=None, left_scale=1.3, right_scale=0.8, mlp=True):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "bias_max": bias_max,
                               "scale": scale if scale is not None else dim ** -0.5, "q_temp": {"coef": coef, "every": every}},
                      "right": {"heads": rheads, "dim": rdim, "vdim": rvdim,
                                "decay": decay or [0.5 + 0.499 * i / max(1, rheads - 1) for i in range(rheads)]},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": {"kind": "dense", "ff": ff} if mlp else None}


def mlstm_layer(heads=3, dim=20, vdim=36, cap=9.0, ff=80, mlp=True):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": {"kind": "dense", "ff": ff} if mlp else None}


def make_config(layers, vocab=97, width=72, loop=None, eps=1e-5, embed_scale=7.0):
    c = {"architecture": "Fatudra", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "embedding": {"scale": embed_scale}, "layers": layers}
    if loop is not None:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def make_weights(cfg, seed=0, bias_rows=12, round_bf16=True):
    rng = np.random.default_rng(seed)
    W, width = {}, cfg["width"]

    def mat(o, i, gain=1.0):
        return rng.standard_normal((o, i)) * gain / np.sqrt(i)

    def vec(n, mean=0.0, std=0.3):
        return mean + std * rng.standard_normal(n)

    W["embed"] = rng.standard_normal((cfg["vocab"], width)) / np.sqrt(width)
    W["head"] = mat(cfg["vocab"], width)
    W["final.norm"], W["final.norm.b"] = vec(width, 1.0, 0.2), vec(width)
    if cfg.get("loop"):
        W["loop.step"] = rng.standard_normal((cfg["loop"]["times"], width)) * 0.5
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        for n in ["norm1", "norm1b"] + (["norm2", "norm2b"] if lc["mlp"] else []):
            W[p + n], W[p + n + ".b"] = vec(width, 1.0, 0.2), vec(width)
        m = lc["mixer"]
        if lc["type"] == "parallel":
            L, R = m["left"], m["right"]
            H, G, d, e = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
            W[p + "mix.left.q"], W[p + "mix.left.q.b"] = mat(H * d, width, 2.0), vec(H * d)
            W[p + "mix.left.k"], W[p + "mix.left.k.b"] = mat(G * d, width, 2.0), vec(G * d)
            W[p + "mix.left.v"], W[p + "mix.left.v.b"] = mat(G * e, width), vec(G * e)
            W[p + "mix.left.rel"] = rng.standard_normal((bias_rows, H)) * 1.5
            W[p + "mix.left.g"] = mat(H, width)
            W[p + "mix.left.o"], W[p + "mix.left.o.b"] = mat(width, H * e), vec(width)
            Hr, dr, er = R["heads"], R["dim"], R["vdim"]
            W[p + "mix.right.q"], W[p + "mix.right.k"] = mat(Hr * dr, width), mat(Hr * dr, width)
            W[p + "mix.right.v"], W[p + "mix.right.g"] = mat(Hr * er, width), mat(Hr * er, width)
            W[p + "mix.right.o"], W[p + "mix.right.norm"] = mat(width, Hr * er), vec(Hr * er, 1.0, 0.2)
        else:
            H, d, e = m["heads"], m["dim"], m["vdim"]
            W[p + "mix.q"], W[p + "mix.k"] = mat(H * d, width), mat(H * d, width)
            W[p + "mix.v"], W[p + "mix.g"] = mat(H * e, width), mat(H * e, width)
            W[p + "mix.o"], W[p + "mix.norm"] = mat(width, H * e), vec(H * e, 1.0, 0.2)
            W[p + "mix.i"], W[p + "mix.i.b"] = mat(H, width, 2.0), vec(H, 0.0, 1.0)
            W[p + "mix.f"], W[p + "mix.f.b"] = mat(H, width, 2.0), vec(H, 2.0, 1.0)
        if lc["mlp"]:
            ff = lc["mlp"]["ff"]
            W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"] = mat(ff, width), mat(ff, width), mat(width, ff)
    if round_bf16:
        W = {k: bf16_round(v) for k, v in W.items()}
    return {k: np.asarray(v, np.float32) for k, v in W.items()}


def write_checkpoint(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: torch.from_numpy(v).to(torch.bfloat16).contiguous() for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
    return path


def logit_errors(got, want):
    """Per position: root mean square of the centred difference over the vocabulary, relative to the spread of the
    expected logits."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / want.std()


def assert_logits(got, want, sharp, what=""):
    """``sharp`` (float32 runs): every position within 2e-4.  Otherwise (bfloat16 against the unrounded restatement): the
    typical position within rounding, and no more than a tenth of them far off -- a position where the mLSTM normaliser
    passes through zero amplifies rounding by orders of magnitude, which a fixed bound on the worst position cannot
    tell from a fault; the float32 run of the same test can."""
    e = logit_errors(got, want)
    assert np.isfinite(e).all(), what
    if sharp:
        assert e.max() < 2e-4, (what, float(e.max()), int(e.argmax()))
    else:
        assert np.median(e) < 0.06 and np.quantile(e, 0.9) < 0.2, (what, float(np.median(e)), float(np.quantile(e, 0.9)))
