"""Plain, slow oracle for the Povazen design: one function per mechanism,
written as token-by-token loops in float64 straight from the equations. It
shares no code with the engine, its ops or its kernels; the tests compare
the framework against it.

Weights are a dict of tensors under the checkpoint's names ('embed',
'l<i>.norm1', 'l<i>.mix.q', ...); cfg is the parsed config.json dict.
A whole sequence is run at once: x is [T, width].
"""

import math

import torch

F64 = torch.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """RMS norm in `groups` equal consecutive parts, then times w."""
    T, C = x.shape
    parts = x.reshape(T, groups, C // groups)
    return rms(parts, eps).reshape(T, C) * w


def causal_conv(x, w):
    """y_t = sum_j w[:, j] * x_(t - taps + 1 + j); zeros before the start.
    x [T, C], w [C, taps]."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def attention_mixer(h, W, p, m, eps):
    """Softmax attention with whole-projection q/k norm, per-head value
    norm, a linear distance penalty per head and a per-head output gate."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ W[p + "q"].T + W[p + "q.b"]
    k = h @ W[p + "k"].T + W[p + "k.b"]
    v = h @ W[p + "v"].T + W[p + "v.b"]
    q = rms(q, eps) * W[p + "q.norm"]
    k = rms(k, eps) * W[p + "k.norm"]
    q = q.reshape(T, H, D)
    k = k.reshape(T, G, D)
    v = rms(v.reshape(T, G, Dv), eps)
    gate = torch.sigmoid(h @ W[p + "g"].T)            # [T, H]
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hd in range(H):
        kv = hd // (H // G)
        slope = 2.0 ** (-8.0 * (hd + 1) / H)
        for i in range(T):
            j = torch.arange(i + 1, dtype=h.dtype)
            s = (k[: i + 1, kv] @ q[i, hd]) * m["scale"] - slope * (i - j)
            a = torch.softmax(s, 0)
            out[i, hd] = (a[:, None] * v[: i + 1, kv]).sum(0) * gate[i, hd]
    return out.reshape(T, H * Dv) @ W[p + "o"].T


def channel_delta_mixer(h, W, p, m, eps):
    """Gated delta rule with one decay per head and key channel."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])).reshape(T, G, D)
    k = silu(causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])).reshape(T, G, D)
    v = silu(causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).reshape(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)                                  # [T, H]
    a = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]
    decay = torch.exp(-torch.exp(W[p + "A_log"])[None, :, None] * softplus(a).reshape(T, H, D))
    og = torch.sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T).reshape(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hd in range(H):
        kv = hd // (H // G)
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(T):
            S = decay[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, hd] = S.T @ q[t, kv]
    out = rms(out, eps) * W[p + "norm"] * og
    return out.reshape(T, H * Dv) @ W[p + "o"].T


def dense_mlp(x, W, p):
    return (silu(x @ W[p + "gate"].T) * (x @ W[p + "up"].T)) @ W[p + "down"].T


def forward(tokens, weights, cfg, dtype=F64):
    """Returns (logits [T, vocab], residual stream after every layer [L, T, width])."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        h = x + causal_conv(x, W[p + "canon1"])
        if layer["type"] == "attention":
            y = attention_mixer(h, W, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "channel_delta":
            y = channel_delta_mixer(h, W, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + group_norm(y, W[p + "norm1"], groups, eps)
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            x = x + group_norm(dense_mlp(x, W, p + "mlp."), W[p + "norm2"], groups, eps)
        after.append(x)
    x = group_norm(x, W["final.norm"], groups, eps)
    logits = x @ W["head"].T
    cap = cfg["logit_softcap"]
    logits = cap * torch.tanh(logits / cap)
    return logits, torch.stack(after)


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Random weights of the design's shapes for a config dict."""
    g = torch.Generator().manual_seed(seed)
    C = cfg["width"]

    def lin(o, i, s=1.0):
        return torch.randn(o, i, generator=g) * (s / math.sqrt(i))

    W = {"embed": torch.randn(cfg["vocab"], C, generator=g), "head": lin(cfg["vocab"], C),
         "final.norm": 1 + 0.1 * torch.randn(C, generator=g)}
    taps = cfg["canon"]["taps"]
    for i, layer in enumerate(cfg["layers"]):
        p, m = "l%d." % i, layer["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "norm1"] = 1 + 0.1 * torch.randn(C, generator=g)
        W[p + "canon1"] = 0.3 * torch.randn(C, taps, generator=g)
        if layer["type"] == "attention":
            W[p + "mix.q"], W[p + "mix.q.b"] = lin(H * D, C), 0.1 * torch.randn(H * D, generator=g)
            W[p + "mix.k"], W[p + "mix.k.b"] = lin(G * D, C), 0.1 * torch.randn(G * D, generator=g)
            W[p + "mix.v"], W[p + "mix.v.b"] = lin(G * Dv, C), 0.1 * torch.randn(G * Dv, generator=g)
            W[p + "mix.q.norm"] = 1 + 0.2 * torch.randn(H * D, generator=g)
            W[p + "mix.k.norm"] = 1 + 0.2 * torch.randn(G * D, generator=g)
            W[p + "mix.g"] = lin(H, C)
            W[p + "mix.o"] = lin(C, H * Dv)
        else:
            r = max(4, C // 16)
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                W[p + "mix." + n] = lin(rows, C)
                W[p + "mix." + n + ".conv"] = 0.5 * torch.randn(rows, m["conv"], generator=g)
            W[p + "mix.b"] = lin(H, C)
            W[p + "mix.A_log"] = torch.randn(H, generator=g) * 0.5 - 1.0
            W[p + "mix.norm"] = 1 + 0.1 * torch.randn(Dv, generator=g)
            W[p + "mix.a1"], W[p + "mix.a2"] = lin(r, C), lin(H * D, r)
            W[p + "mix.dt_bias"] = torch.randn(H * D, generator=g) - 2.0
            W[p + "mix.g1"], W[p + "mix.g2"] = lin(r, C), lin(H * Dv, r)
            W[p + "mix.o"] = lin(C, H * Dv)
        if layer.get("mlp") is not None:
            W[p + "norm2"] = 1 + 0.1 * torch.randn(C, generator=g)
            ff = layer["mlp"]["ff"]
            W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"] = lin(ff, C), lin(ff, C), lin(C, ff)
    return {k: v.to(dtype) for k, v in W.items()}
