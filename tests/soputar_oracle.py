"""Plain, slow, whole-sequence Soputar in float64, one function per
mechanism, written from the equations. Shares no code with the package:
it is the yardstick the engine, its cache/state handling and its kernels are
compared with.

A model is ``(cfg, weights)``: ``cfg`` the checkpoint's config dictionary,
``weights`` a dict of tensors under the checkpoint's names. Every function
takes the full token sequence of ONE request; nothing is cached.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def _w(weights, name):
    return weights[name].to(F64)


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def silu(x):
    return x * torch.sigmoid(x)


def causal_conv(x, taps_w):
    """x (T, C), taps_w (C, K): y_t = sum_j w[:, j] x_{t-(K-1)+j}, zeros
    before the start."""
    T, C = x.shape
    K = taps_w.shape[1]
    xp = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros(T, C, dtype=x.dtype)
    for j in range(K):
        y = y + taps_w[:, j] * xp[j:j + T]
    return y


def delta_mixer(h, weights, pre, mc, eps):
    """Gated delta rule with one decay per head. h (T, W)."""
    T = h.shape[0]
    H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = silu(causal_conv(h @ _w(weights, pre + "q").T, _w(weights, pre + "q.conv"))).view(T, G, D)
    k = silu(causal_conv(h @ _w(weights, pre + "k").T, _w(weights, pre + "k.conv"))).view(T, G, D)
    v = silu(causal_conv(h @ _w(weights, pre + "v").T, _w(weights, pre + "v.conv"))).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ _w(weights, pre + "b").T)                      # (T, H)
    dt = torch.nn.functional.softplus(h @ _w(weights, pre + "a").T + _w(weights, pre + "dt_bias"))
    decay = torch.exp(-torch.exp(_w(weights, pre + "A_log")) * dt)         # (T, H)
    rep = H // G
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // rep
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = decay[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hd] = S.T @ q[t, g]
    out = rms(out, eps) * _w(weights, pre + "norm")
    gate = silu(h @ _w(weights, pre + "g").T).view(T, H, Dv)
    return (out * gate).reshape(T, H * Dv) @ _w(weights, pre + "o").T


def attention_keys_values(h, weights, pre, mc, eps):
    """Keys (after their norm) and values of a softmax-attention layer."""
    T = h.shape[0]
    G, D, Dv = mc["kv_heads"], mc["dim"], mc["vdim"]
    k = rms(h @ _w(weights, pre + "k").T, eps) * _w(weights, pre + "k.norm")
    v = h @ _w(weights, pre + "v").T
    return k.view(T, G, D), v.view(T, G, Dv)


def attention_mixer(h, weights, pre, mc, eps, kv):
    """Softmax attention without rotation: whole-projection q norm, query
    temperature, tanh score cap, causal. ``kv`` = (k, v) from this layer or
    from the layer it borrows them from."""
    T = h.shape[0]
    H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    k, v = kv
    q = rms(h @ _w(weights, pre + "q").T, eps) * _w(weights, pre + "q.norm")
    qt = mc.get("q_temp")
    if qt:
        p = torch.arange(T, dtype=F64)
        q = q * (1.0 + qt["coef"] * torch.log(torch.floor((p + 1) / qt["every"]) + 1.0)).view(T, 1)
    q = q.view(T, H, D)
    rep = H // G
    cap = mc.get("softcap")
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // rep
        s = (q[:, hd] @ k[:, g].T) * mc["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~causal, -math.inf)
        out[:, hd] = torch.softmax(s, -1) @ v[:, g]
    return out.reshape(T, H * Dv) @ _w(weights, pre + "o").T


def rotate_pairs(x, pos, base, dims):
    """Interleaved rotary on the first `dims` channels of the last axis:
    channels (2i, 2i+1) turn by pos * base^(-2i/dims). x (T, ..., C)."""
    T = x.shape[0]
    i = torch.arange(dims // 2, dtype=F64)
    ang = pos.to(F64).view(T, 1) * base ** (-2.0 * i / dims)            # (T, dims/2)
    shape = [T] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def latent_mixer(h, weights, pre, mc, eps):
    """Latent attention: keys/values expanded from a normed low-rank
    latent, one shared rotated key part, softmax with a per-head sink."""
    T = h.shape[0]
    H, D, R, Dv, C = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    pos = torch.arange(T)
    q = (h @ _w(weights, pre + "q").T).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    dkv = h @ _w(weights, pre + "dkv").T
    c = rms(dkv[:, :C], eps) * _w(weights, pre + "dkv.norm")
    k_rot = dkv[:, C:]
    rot = mc["rot"]
    q_rot = rotate_pairs(q_rot, pos, rot["base"], rot["dims"])
    k_rot = rotate_pairs(k_rot, pos, rot["base"], rot["dims"])
    k_plain = (c @ _w(weights, pre + "uk").T).view(T, H, D)
    v = (c @ _w(weights, pre + "uv").T).view(T, H, Dv)
    sink = _w(weights, pre + "sink")
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        s = (q_plain[:, hd] @ k_plain[:, hd].T + q_rot[:, hd] @ k_rot.T) * mc["scale"]
        s = s.masked_fill(~causal, -math.inf)
        m = torch.maximum(s.max(-1, keepdim=True).values, sink[hd])
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True) + torch.exp(sink[hd] - m)
        out[:, hd] = (e / den) @ v[:, hd]
    return out.reshape(T, H * Dv) @ _w(weights, pre + "o").T


def feed_forward(h, weights, pre, fc):
    lim = fc["limit"]
    g = torch.clamp(h @ _w(weights, pre + "gate").T, max=lim)
    u = torch.clamp(h @ _w(weights, pre + "up").T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ _w(weights, pre + "down").T


def forward(cfg, weights, tokens, return_layers=False):
    """Logits (T, vocab) in float64 (and the stream after every layer)."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = _w(weights, "embed")[tokens] * cfg["embedding"]["scale"]
    kvs = {}
    streams = []
    for i, lc in enumerate(cfg["layers"]):
        pre = f"l{i}.mix."
        mc = lc["mixer"]
        if lc["type"] == "delta":
            y = delta_mixer(x, weights, pre, mc, eps)
        elif lc["type"] == "attention":
            src = mc.get("kv_from")
            if src is None:
                kvs[i] = attention_keys_values(x, weights, pre, mc, eps)
                src = i
            y = attention_mixer(x, weights, pre, mc, eps, kvs[src])
        elif lc["type"] == "latent_attention":
            y = latent_mixer(x, weights, pre, mc, eps)
        else:
            raise ValueError(lc["type"])
        x = x + norm_one_plus(y, _w(weights, f"l{i}.norm1"), eps)
        if lc.get("mlp"):
            y = feed_forward(x, weights, f"l{i}.mlp.", lc["mlp"])
            x = x + norm_one_plus(y, _w(weights, f"l{i}.norm2"), eps)
        streams.append(x)
    logits = norm_one_plus(x, _w(weights, "final.norm"), eps) @ _w(weights, "head").T
    if return_layers:
        return logits, torch.stack(streams)
    return logits
