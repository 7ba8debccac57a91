"""Plain, slow Nabelix forward used as the numerics oracle by the tests.

Written directly from the design's equations in float64, one function per
mechanism, whole sequences only (no cache, no batching). It shares no code
with the package: weights come in as a flat ``{tensor name: tensor}`` dict
with the checkpoint's own names and the config as the parsed ``config.json``
dict.
"""

import math

import torch

F64 = torch.float64


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def causal_conv(h, w):
    """h (T, C), w (C, taps): y_t = sum_j w[:, j] * h_{t - (taps-1) + j}."""
    T, C = h.shape
    taps = w.shape[1]
    y = torch.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += w[:, j] * h[s]
    return y


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def visible(i, j, size, keep_first):
    return j <= i and (i - j < size or j < keep_first)


def biased_window_attention(h, W, pre, c):
    """Softmax attention without rotation: log-distance penalty, sliding
    window plus always-visible first tokens, sigmoid output gate."""
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    size, keep = c["mask"]["size"], c["mask"]["keep_first"]
    q = (h @ W[pre + "q"].T).view(T, H, D)
    k = (h @ W[pre + "k"].T).view(T, G, D)
    v = (h @ W[pre + "v"].T).view(T, G, Dv)
    r1, r2 = W[pre + "r1"], W[pre + "r2"]
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j, size, keep)]
            jt = torch.tensor(js)
            s = (k[jt, g] @ q[i, hd]) * c["scale"]
            s = s - r1[hd] * torch.log1p(r2[hd] * (i - jt).to(F64))
            p = torch.softmax(s, 0)
            out[i, hd] = p @ v[jt, g]
    gate = torch.sigmoid(h @ W[pre + "g"].T)
    return (out.reshape(T, H * Dv) * gate) @ W[pre + "o"].T


def gated_delta_rule(h, W, pre, c, eps):
    """Delta-rule linear recurrence with a per-key-channel decay."""
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    silu = torch.nn.functional.silu

    def proj(name):
        return silu(causal_conv(h @ W[pre + name].T, W[pre + name + ".conv"]))

    q = proj("q").view(T, G, D)
    k = proj("k").view(T, G, D)
    v = proj("v").view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[pre + "b"].T)                       # (T, H)
    dt = torch.nn.functional.softplus(
        (h @ W[pre + "a1"].T) @ W[pre + "a2"].T + W[pre + "dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(W[pre + "A_log"]).view(1, H, 1) * dt)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = decay[t, hd].view(D, 1) * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * W[pre + "norm"]
    gate = torch.sigmoid((h @ W[pre + "g1"].T) @ W[pre + "g2"].T)
    return (o.reshape(T, H * Dv) * gate) @ W[pre + "o"].T


def feed_forward(h, W, pre):
    return (gelu_tanh(h @ W[pre + "gate"].T) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def layer(x, W, i, lc, eps):
    pre = "l%d." % i
    h = layer_norm(x, W[pre + "norm1"], eps)
    h = h + causal_conv(h, W[pre + "canon1"])
    m = lc["mixer"]
    assert lc["type"] == "parallel"
    mix = m["left_scale"] * biased_window_attention(h, W, pre + "mix.left.", m["left"]) \
        + m["right_scale"] * gated_delta_rule(h, W, pre + "mix.right.", m["right"], eps)
    x = x + mix
    if lc.get("mlp"):
        x = x + feed_forward(layer_norm(x, W[pre + "norm2"], eps), W, pre + "mlp.")
    return x


def run_order(cfg):
    """Layer indices in execution order, with a flag on the first layer of
    every repeated pass after the first."""
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    order = [(i, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        for i in range(lp["start"], lp["stop"]):
            order.append((i, t > 0 and i == lp["start"]))
    order += [(i, False) for i in range(lp["stop"], n)]
    return order


def forward(tokens, W, cfg, want_streams=False):
    """tokens: list of ids. Returns logits (T, vocab) [, residual streams]."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x0 = W["embed"][torch.tensor(tokens)]
    x = x0.clone()
    streams = []
    for i, readd in run_order(cfg):
        if readd:
            x = x + x0
        x = layer(x, W, i, cfg["layers"][i], eps)
        streams.append(x.clone())
    logits = layer_norm(x, W["final.norm"], eps) @ W["embed"].T
    cap = cfg["logit_softcap"]
    logits = cap * torch.tanh(logits / cap)
    return (logits, torch.stack(streams)) if want_streams else logits
