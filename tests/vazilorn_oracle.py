"""Plain, slow float64 implementation of the Vazilorn design, one function
per mechanism, written from its equations. It shares no code with the engine
or its ops and keeps no cache: every call recomputes a whole sequence.

A model is (cfg, tensors): cfg is the config.json dictionary, tensors maps
checkpoint names to torch tensors. Notation: n tokens, C width, H query
heads, G key/value heads, D key size, E value size.
"""

import math

import torch

F64 = torch.float64


def dyt(x, w, b, alpha):
    """Dynamic tanh norm: tanh(alpha x) * w + b, elementwise over channels."""
    return torch.tanh(alpha * x) * w + b


def rms_unit(x, eps):
    """x over the root of its mean square (eps inside the root), last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2, then the wavelength-dependent
    rescaling: short waves stay, long waves are slowed by `factor`, the band
    between is blended linearly in original/wavelength."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling:
            fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wl = 2.0 * math.pi / f
            if wl < orig / hi:
                pass
            elif wl > orig / lo:
                f = f / fac
            else:
                s = (orig / wl - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate_pairs(x, positions, freqs):
    """x [n, heads, D]; the first 2*len(freqs) channels of every head are
    rotated, channel 2i with channel 2i+1, by the angle position * f_i."""
    n, _, D = x.shape
    r = 2 * freqs.numel()
    out = x.clone()
    if r == 0:
        return out
    ang = positions.to(F64)[:, None] * freqs[None, :]          # [n, r/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:r:2], x[..., 1:r:2]
    out[..., 0:r:2] = a * c - b * s
    out[..., 1:r:2] = b * c + a * s
    return out


def windowed_sink_attention(q, k, v, scale, window, sink):
    """q [n,H,D], k [n,G,D], v [n,G,E]. Query i sees keys j with
    0 <= i - j < window (window None: all j <= i). Every head's softmax
    denominator holds one more term exp(sink_h) that carries no value."""
    n, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(n, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale                      # [n, n]
        i = torch.arange(n)[:, None]
        j = torch.arange(n)[None, :]
        ok = (j <= i)
        if window is not None:
            ok = ok & (i - j < window)
        s = s.masked_fill(~ok, -math.inf)
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].expand_as(m))
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def attention_mixer(h, positions, m, tn, prefix, eps):
    """The whole mixer on its input h [n, C]. m is the layer's 'mixer'
    dictionary, tn its tensors (prefix + 'q', ...)."""
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    t = lambda name: tn[prefix + name].to(F64)
    q = (h @ t("q").T).view(n, H, D)
    k = (h @ t("k").T).view(n, G, D)
    v = (h @ t("v").T).view(n, G, E)
    q = rms_unit(q, eps) * t("q.norm")
    k = rms_unit(k, eps) * t("k.norm")
    rot = m.get("rot")
    if rot:
        fr = rotary_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q = rotate_pairs(q, positions, fr)
        k = rotate_pairs(k, positions, fr)
    mask = m.get("mask")
    window = int(mask["size"]) if mask else None
    sink = t("sink") if (prefix + "sink") in tn else None
    o = windowed_sink_attention(q, k, v, float(m["scale"]), window, sink)
    return o.reshape(n, H * E) @ t("o").T


def gated_ff(h, tn, prefix, act):
    t = lambda name: tn[prefix + name].to(F64)
    return (act(h @ t("gate").T) * (h @ t("up").T)) @ t("down").T


def route(h, tn, prefix, r):
    """Returns (chosen experts [n, top], weights [n, top]).
    s = sigmoid(W h); c = s + correction ranks; a group is rated by
    max1(c) + max2(c) and only the `keep` top-rated groups may be picked
    from; w_j = scale * s_j / (sum_k s_k + 1e-20)."""
    E, top = int(r["experts"]), int(r["top"])
    z = h @ tn[prefix + "router"].to(F64).T
    s = torch.sigmoid(z)
    choice = s + tn[prefix + "correction"].to(F64)
    grp = r.get("groups")
    if grp:
        cnt, keep = int(grp["count"]), int(grp["keep"])
        per = E // cnt
        gs = choice.view(-1, cnt, per).topk(min(2, per), dim=-1).values.sum(-1)   # [n, cnt]
        best = gs.topk(keep, dim=-1).indices
        allowed = torch.zeros(choice.shape[0], cnt, dtype=torch.bool)
        allowed.scatter_(1, best, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), -math.inf)
    idx = choice.topk(top, dim=-1).indices
    w = s.gather(1, idx)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * float(r["scale"])
    return idx, w


def moe_ff(h, mlp, tn, prefix):
    idx, w = route(h, tn, prefix, mlp["router"])
    out = torch.zeros(h.shape[0], tn[prefix + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            out[t] += w[t, j] * gated_ff(h[t : t + 1], tn, f"{prefix}e{e}.", silu)[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, tn, prefix + "shared.", silu)
    return out


def norm_of(x, tn, name):
    return dyt(x, tn[name].to(F64), tn[name + ".b"].to(F64), tn[name + ".alpha"].to(F64))


def forward(cfg, tn, tokens, layers_out=None):
    """Logits [n, vocab] (float64) of one whole sequence from position 0."""
    ids = torch.as_tensor(tokens, dtype=torch.int64)
    pos = torch.arange(ids.numel())
    eps = float(cfg["norm"]["eps"])
    x = tn["embed"].to(F64)[ids]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        assert layer["type"] == "attention"
        y = attention_mixer(norm_of(x, tn, p + "norm1"), pos, layer["mixer"], tn, p + "mix.", eps)
        x = x + norm_of(y, tn, p + "norm1b")
        mlp = layer.get("mlp")
        if mlp is not None:
            hin = norm_of(x, tn, p + "norm2")
            if mlp["kind"] == "dense":
                y = gated_ff(hin, tn, p + "mlp.", gelu_tanh)
            else:
                y = moe_ff(hin, mlp, tn, p + "mlp.")
            x = x + norm_of(y, tn, p + "norm2b")
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_of(x, tn, "final.norm") @ tn["head"].to(F64).T


def greedy(cfg, tn, prompt, steps):
    toks = list(prompt)
    for _ in range(steps):
        toks.append(int(forward(cfg, tn, toks)[-1].argmax()))
    return toks[len(prompt):]


def random_weights(cfg, seed=0):
    """Random tensors under the checkpoint's names for a config dictionary."""
    g = torch.Generator().manual_seed(seed)
    C, V = cfg["width"], cfg["vocab"]
    rn = lambda *s, std=1.0: torch.randn(*s, generator=g) * std
    W = {"embed": rn(V, C), "head": rn(V, C, std=C ** -0.5)}

    def norm(name):
        W[name] = 1.0 + 0.2 * rn(C)
        W[name + ".b"] = 0.1 * rn(C)
        W[name + ".alpha"] = torch.tensor(0.4 + 0.4 * float(torch.rand((), generator=g)))

    def ff(prefix, inner):
        W[prefix + "gate"] = rn(inner, C, std=C ** -0.5)
        W[prefix + "up"] = rn(inner, C, std=C ** -0.5)
        W[prefix + "down"] = rn(C, inner, std=inner ** -0.5)

    norm("final.norm")
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        norm(p + "norm1")
        norm(p + "norm1b")
        W[p + "mix.q"] = rn(H * D, C, std=C ** -0.5)
        W[p + "mix.k"] = rn(G * D, C, std=C ** -0.5)
        W[p + "mix.v"] = rn(G * E, C, std=C ** -0.5)
        W[p + "mix.q.norm"] = 1.0 + 0.2 * rn(D)
        W[p + "mix.k.norm"] = 1.0 + 0.2 * rn(D)
        W[p + "mix.sink"] = rn(H)
        W[p + "mix.o"] = rn(C, H * E, std=(H * E) ** -0.5)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        norm(p + "norm2")
        norm(p + "norm2b")
        if mlp["kind"] == "dense":
            ff(p + "mlp.", mlp["ff"])
        else:
            n = mlp["router"]["experts"]
            W[p + "mlp.router"] = rn(n, C, std=2.0 * C ** -0.5)
            W[p + "mlp.correction"] = 0.3 * rn(n)
            for e in range(n):
                ff(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            if mlp.get("shared"):
                ff(p + "mlp.shared.", mlp["shared"]["ff"])
    return W
