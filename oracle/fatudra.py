"""Plain, slow restatement of the Fatudra decoder, one function per mechanism (test infrastructure only: nothing under
aphrodite_engine_amd/ imports this, and this imports nothing from there).  float64 numpy, token by token where the design
is a recurrence, no cache: every call recomputes a whole sequence.

Notation: x [T, W] is the residual stream; a "layer run" is one execution of a layer (a looped layer runs several times,
each run with its own history).  Weights come as a dict name -> array, named as in the checkpoint."""
import math

import numpy as np


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def rms_unit(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def distance_bucket(n, rows, far):
    """Row of the distance-bias table for a key n >= 0 positions back: one row per distance below rows // 2, then
    logarithmically wider rows that reach the last one at distance ``far``."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def query_temperature(p, coef, every):
    return 1.0 + coef * math.log((p + 1) // every + 1)


def biased_softmax_attention(q, k, v, rel, scale, far, coef, every):
    """q [T, H, d], k [T, G, d], v [T, G, e], rel [rows, H] -> [T, H, e]; causal, grouped heads, per-position query
    temperature, additive bias by distance bucket (not multiplied by ``scale``)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    row_of = np.array([distance_bucket(n, rel.shape[0], far) for n in range(T)])
    for i in range(T):
        temp = query_temperature(i, coef, every)
        rows = row_of[i::-1]                      # distances i, i-1, ..., 0 for keys 0..i
        for h in range(H):
            g = h // (H // G)
            s = k[:i + 1, g] @ (q[i, h] * temp) * scale + rel[rows, h]
            p = np.exp(s - s.max())
            out[i, h] = (p / p.sum()) @ v[:i + 1, g]
    return out


def decay_linear_attention(q, k, v, decay):
    """q, k [T, H, d], v [T, H, e], decay [H]: S <- decay S + k v^T, o = S^T q."""
    T, H, d = q.shape
    S = np.zeros((H, d, v.shape[2]))
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        for h in range(H):
            S[h] = decay[h] * S[h] + np.outer(k[t, h], v[t, h])
            out[t, h] = S[h].T @ q[t, h]
    return out


def mlstm_memory(q, k, v, ig, fg):
    """Stabilised matrix memory.  q (already scaled), k [T, H, d], v [T, H, e]; ig, fg [T, H] are the LOG input and
    forget gates.  The running maximum starts at zero."""
    T, H, d = q.shape
    S = np.zeros((H, d, v.shape[2]))
    n = np.zeros((H, d))
    m = np.zeros(H)
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        for h in range(H):
            m_new = max(fg[t, h] + m[h], ig[t, h])
            a, b = math.exp(fg[t, h] + m[h] - m_new), math.exp(ig[t, h] - m_new)
            S[h] = a * S[h] + b * np.outer(k[t, h], v[t, h])
            n[h] = a * n[h] + b * k[t, h]
            m[h] = m_new
            out[t, h] = S[h].T @ q[t, h] / (max(abs(n[h] @ q[t, h]), math.exp(-m_new)) + 1e-6)
    return out


def parallel_mixer(h, W, pfx, mc, eps):
    """A softmax-attention branch and a decay-linear-attention branch on the same input, summed with fixed weights."""
    T = h.shape[0]
    L, R = mc["left"], mc["right"]
    lp, rp = pfx + "left.", pfx + "right."
    H, G, d, e = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
    q = (h @ W[lp + "q"].T + W[lp + "q.b"]).reshape(T, H, d)
    k = (h @ W[lp + "k"].T + W[lp + "k.b"]).reshape(T, G, d)
    v = (h @ W[lp + "v"].T + W[lp + "v.b"]).reshape(T, G, e)
    o = biased_softmax_attention(q, k, v, W[lp + "rel"], L["scale"], L["bias_max"], L["q_temp"]["coef"], L["q_temp"]["every"])
    o = o * sigmoid(h @ W[lp + "g"].T)[:, :, None]
    left = o.reshape(T, H * e) @ W[lp + "o"].T + W[lp + "o.b"]
    Hr, dr, er = R["heads"], R["dim"], R["vdim"]
    q = silu(h @ W[rp + "q"].T).reshape(T, Hr, dr)
    k = silu(h @ W[rp + "k"].T).reshape(T, Hr, dr)
    v = silu(h @ W[rp + "v"].T).reshape(T, Hr, er)
    o = decay_linear_attention(q, k, v, np.asarray(R["decay"], np.float64)).reshape(T, Hr * er)
    o = rms_unit(o, eps) * W[rp + "norm"] * sigmoid(h @ W[rp + "g"].T)
    right = o @ W[rp + "o"].T
    return mc["left_scale"] * left + mc["right_scale"] * right


def mlstm_mixer(h, W, pfx, mc, eps):
    T = h.shape[0]
    H, d, e, cap = mc["heads"], mc["dim"], mc["vdim"], mc["gate_cap"]
    q = (h @ W[pfx + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ W[pfx + "k"].T).reshape(T, H, d)
    v = (h @ W[pfx + "v"].T).reshape(T, H, e)
    ig = cap * np.tanh((h @ W[pfx + "i"].T + W[pfx + "i.b"]) / cap)
    fg = log_sigmoid(cap * np.tanh((h @ W[pfx + "f"].T + W[pfx + "f.b"]) / cap))
    o = rms_unit(mlstm_memory(q, k, v, ig, fg), eps).reshape(T, H * e)
    o = o * W[pfx + "norm"] * sigmoid(h @ W[pfx + "g"].T)
    return o @ W[pfx + "o"].T


def gated_mlp(h, W, pfx):
    return (gelu_tanh(h @ W[pfx + "gate"].T) * (h @ W[pfx + "up"].T)) @ W[pfx + "down"].T


def layer_schedule(cfg):
    """[(layer index, pass number or None)] in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 0}
    a, b, times = loop["start"], loop["stop"], loop["times"]
    if b <= a or times <= 0:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def forward(cfg, W, tokens, trace=None):
    """Logits [T, vocab] of one whole sequence; ``trace`` (a list) receives the residual stream after every layer run."""
    W = {k: np.asarray(v, np.float64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    loop = cfg.get("loop") or {}
    for li, t in layer_schedule(cfg):
        if t is not None and li == loop["start"]:
            x = x + W["loop.step"][t]
        lc, p = cfg["layers"][li], f"l{li}."
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        mix = {"parallel": parallel_mixer, "mlstm": mlstm_mixer}[lc["type"]](h, W, p + "mix.", lc["mixer"], eps)
        x = x + layer_norm(mix, W[p + "norm1b"], W[p + "norm1b.b"], eps)
        if lc.get("mlp") is not None:
            if lc["mlp"]["kind"] != "dense":
                raise ValueError("feed-forward kind " + str(lc["mlp"]["kind"]))
            h = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps)
            x = x + layer_norm(gated_mlp(h, W, p + "mlp."), W[p + "norm2b"], W[p + "norm2b.b"], eps)
        if trace is not None:
            trace.append(x.copy())
    x = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return x @ W["head"].T
