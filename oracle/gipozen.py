"""Plain, slow restatement of the Gipozen decoder, one function per mechanism (test infrastructure only: nothing under
aphrodite_engine_amd/ imports this, and this imports nothing from there).  float64 numpy, token by token, no cache: every
call recomputes a whole sequence.

Notation: x [T, W] is the residual stream of one sequence, positions 0 .. T-1.  Weights come as a dict name -> array, named as
in the checkpoint; the configuration is the checkpoint's config.json as a dict."""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def scalar_rms_norm(x, g, eps):
    """RMS norm whose learned gain is ONE number for all coordinates."""
    return rms_unit(x, eps) * float(g)


def depth_average(history, weights):
    """history: [X_0, ..., X_n] (each [T, W]); weights [n + 1] -> sum_j weights[j] X_j."""
    assert len(history) == len(weights)
    out = np.zeros_like(history[0])
    for w, X in zip(weights, history):
        out = out + float(w) * X
    return out


def short_causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the sequence's start."""
    T, C = u.shape
    taps = w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def visible(i, j, window, keep_first):
    """Sliding window that also keeps the sequence's first tokens."""
    return j <= i and (i - j < window or j < keep_first)


def windowed_softmax_attention(q, k, v, scale, window, keep_first):
    """q [T, d], k [T, d], v [T, e] of ONE map of one head -> [T, e]; no rotation, ordinary softmax over the visible keys."""
    T = q.shape[0]
    out = np.zeros((T, v.shape[1]))
    for i in range(T):
        js = [j for j in range(i + 1) if visible(i, j, window, keep_first)]
        s = k[js] @ q[i] * scale
        p = np.exp(s - s.max())
        out[i] = (p / p.sum()) @ v[js]
    return out


def differential_lambda(lq1, lk1, lq2, lk2, diff):
    return math.exp(float(np.dot(lq1, lk1))) - math.exp(float(np.dot(lq2, lk2))) + diff


def differential_attention(q, k, v, heads, kv_heads, dim, vdim, scale, window, keep_first, lam, diff, eps):
    """q [T, H * 2 * d] and k [T, G * 2 * d] laid out head by head as [map 1, map 2]; v [T, G * e].  Each map is an attention
    of its own over the same values: o = a1 - lam * a2, brought to unit RMS over the head's values, times (1 - diff).
    -> [T, H * e]"""
    T = q.shape[0]
    q = q.reshape(T, heads, 2, dim)
    k = k.reshape(T, kv_heads, 2, dim)
    v = v.reshape(T, kv_heads, vdim)
    out = np.zeros((T, heads, vdim))
    for h in range(heads):
        g = h // (heads // kv_heads)
        a1 = windowed_softmax_attention(q[:, h, 0], k[:, g, 0], v[:, g], scale, window, keep_first)
        a2 = windowed_softmax_attention(q[:, h, 1], k[:, g, 1], v[:, g], scale, window, keep_first)
        out[:, h] = rms_unit(a1 - lam * a2, eps) * (1.0 - diff)
    return out.reshape(T, heads * vdim)


def poly_norm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e with N = division by the root mean square over the token's vector."""
    a, b, c, e = (float(t) for t in coef)
    return a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z ** 3, eps) + e


def dense_ff(h, W, p, eps):
    return poly_norm(h @ W[p + "up"].T, W[p + "act"], eps) @ W[p + "down"].T


def clamped_glu_expert(h, gate, up, down, limit):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h, router, correction, top):
    """-> (chosen expert indices [T, top], their weights [T, top]): softmax over all router outputs, choice by score plus
    correction, weight = the score itself, not renormalised."""
    z = h @ router.T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s = s / s.sum(-1, keepdims=True)
    order = np.argsort(-(s + correction), axis=-1, kind="stable")[:, :top]
    return order, np.take_along_axis(s, order, -1)


def moe_ff(h, W, p, mc):
    r = mc["router"]
    E, top, ident = int(r["experts"]), int(r["top"]), int(r.get("identity", 0))
    assert W[p + "router"].shape[0] == E + ident
    idx, wts = route(h, W[p + "router"], W[p + "correction"], top)
    out = np.zeros_like(h)
    limit = float(mc["expert"]["limit"])
    for t in range(h.shape[0]):
        for e, w in zip(idx[t], wts[t]):
            if e >= E:                       # identity expert
                out[t] += w * h[t]
            else:
                pe = f"{p}e{e}."
                out[t] += w * clamped_glu_expert(h[t:t + 1], W[pe + "gate"], W[pe + "up"], W[pe + "down"], limit)[0]
    if mc.get("shared") is not None:
        ps = p + "shared."
        y = clamped_glu_expert(h, W[ps + "gate"], W[ps + "up"], W[ps + "down"], float(mc["shared"]["limit"]))
        out += y * sigmoid(h @ W[ps + "sg"].T)
    return out


def forward(cfg, W, tokens, trace=None):
    """Logits [T, vocab] of one sequence.  ``trace``: a list that receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    W = {k: np.asarray(v, np.float64) for k, v in W.items()}
    x = W["embed"][np.asarray(tokens)]
    history = [x]
    kv = {}
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        mc = lc["mixer"]
        assert lc["type"] == "attention"
        H, G, d, e = int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"])
        h = scalar_rms_norm(x, W[p + "norm1"], eps)
        q = short_causal_conv(h @ W[p + "mix.q"].T, W[p + "mix.q.conv"])
        if mc.get("kv_from") is None:
            k = short_causal_conv(h @ W[p + "mix.k"].T, W[p + "mix.k.conv"])
            v = short_causal_conv(h @ W[p + "mix.v"].T, W[p + "mix.v.conv"])
            kv[i] = (k, v)
        else:
            k, v = kv[int(mc["kv_from"])]
        diff = float(mc["diff"])
        lam = differential_lambda(W[p + "mix.lq1"], W[p + "mix.lk1"], W[p + "mix.lq2"], W[p + "mix.lk2"], diff)
        o = differential_attention(q, k, v, H, G, d, e, float(mc["scale"]), int(mc["mask"]["size"]),
                                   int(mc["mask"]["keep_first"]), lam, diff, eps)
        o = o * sigmoid(h @ W[p + "mix.g"].T)
        x = x + o @ W[p + "mix.o"].T
        if lc.get("mlp") is not None:
            h = scalar_rms_norm(x, W[p + "norm2"], eps)
            if lc["mlp"]["kind"] == "dense":
                x = x + dense_ff(h, W, p + "mlp.", eps)
            else:
                x = x + moe_ff(h, W, p + "mlp.", lc["mlp"])
        history.append(x)
        x = depth_average(history, W[p + "dwa"])
        if trace is not None:
            trace.append(x.copy())
    head = W["head"] if "head" in W else W["embed"]
    return scalar_rms_norm(x, W["final.norm"], eps) @ head.T * float(cfg["logit_scale"])
