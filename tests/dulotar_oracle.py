"""Plain, slow oracle for the Dulotar design (hybrid recurrent / chunked-attention
decoder). Everything here is whole-sequence, token-by-token torch code in one
floating type, written from the design's equations; it shares nothing with
the engine's ops, kernels, loader or cache. Tests compare the engine to it.

Weights are a flat dict name -> tensor using the checkpoint's own names
("l<i>.mix.z", "l<i>.norm1.b", "embed", "head", ...). `cfg` is the parsed
config.json dict.
"""
from __future__ import annotations

import math

import torch


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal_conv(u, w):
    """u [T, C], w [C, taps]; y_t = sum_j w[:, j] * u_(t - taps + 1 + j)."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def silu(x):
    return x * torch.sigmoid(x)


def mingru(h, W, p):
    """minGRU: elementwise state, gate and candidate depend on the input at t alone
    (no path from the state into the gates)."""
    z = torch.sigmoid(h @ W[p + "z"].T + W[p + "z.b"])
    u = h @ W[p + "x"].T + W[p + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = silu(h @ W[p + "g"].T)
    S = torch.zeros(z.shape[1], dtype=h.dtype)
    out = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * cand[t]
        out.append(S * g[t])
    return torch.stack(out) @ W[p + "o"].T


def wkv(h, W, p, heads, dim, eps):
    """Matrix-state time mixing with per-channel data-dependent decay."""
    T = h.shape[0]
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    mix = {s: h + (prev - h) * W[p + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ W[p + "r"].T).view(T, heads, dim)
    k = (mix["k"] @ W[p + "k"].T).view(T, heads, dim)
    v = (mix["v"] @ W[p + "v"].T).view(T, heads, dim)
    gate = silu(mix["g"] @ W[p + "g"].T)
    dec = torch.exp(
        -torch.exp(torch.tanh(mix["w"] @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])
    ).view(T, heads, dim)
    u = W[p + "u"]  # [heads, dim]
    S = torch.zeros(heads, dim, dim, dtype=h.dtype)  # [head, key ch, value ch]
    out = []
    for t in range(T):
        kv = k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o = torch.einsum("hkv,hk->hv", S + u.unsqueeze(-1) * kv, r[t])
        S = dec[t].unsqueeze(-1) * S + kv
        out.append(rms_unit(o, eps).reshape(-1))
    o = torch.stack(out) * W[p + "norm"] * gate
    return o @ W[p + "o"].T


def rotate_interleaved(x, pos, base, dims):
    """x [T, heads, dim]; pairs (2i, 2i+1) of the first `dims` dims."""
    x = x.clone()
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    f = base ** (-2.0 * i / dims)
    a = pos.to(x.dtype).unsqueeze(-1) * f  # [T, half]
    c, s = torch.cos(a).unsqueeze(1), torch.sin(a).unsqueeze(1)
    u = x[..., 0:dims:2].clone()
    v = x[..., 1:dims:2].clone()
    x[..., 0:dims:2] = u * c - v * s
    x[..., 1:dims:2] = v * c + u * s
    return x


def chunk_softmax(q, k, v, scale, cap, size):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv]; position t sees
    j <= t with floor(j / size) == floor(t / size)."""
    T, H, _ = q.shape
    G, Dv = k.shape[1], v.shape[2]
    out = torch.zeros(T, H, Dv, dtype=q.dtype)
    for t in range(T):
        lo = (t // size) * size
        for hd in range(H):
            g = hd // (H // G)
            s = (k[lo : t + 1, g] @ q[t, hd]) * scale
            s = cap * torch.tanh(s / cap)
            out[t, hd] = torch.softmax(s, 0) @ v[lo : t + 1, g]
    return out


def chunked_attention(h, W, p, m):
    """Softmax attention inside position-aligned chunks, with short
    convolutions on q/k/v, partial rotary and a tanh cap on the scores."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, H, D)
    k = causal_conv(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, G, D)
    v = causal_conv(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, G, Dv)
    pos = torch.arange(T)
    q = rotate_interleaved(q, pos, m["rot"]["base"], m["rot"]["dims"])
    k = rotate_interleaved(k, pos, m["rot"]["base"], m["rot"]["dims"])
    out = chunk_softmax(q, k, v, m["scale"], m["softcap"], m["mask"]["size"])
    return out.reshape(T, H * Dv) @ W[p + "o"].T


def lightning(h, W, p, m, eps):
    """Linear attention with a constant per-head decay of the state."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).view(T, H, D)
    k = silu(h @ W[p + "k"].T).view(T, H, D)
    v = silu(h @ W[p + "v"].T).view(T, H, Dv)
    dec = torch.tensor(m["decay"], dtype=h.dtype).view(H, 1, 1)
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    out = []
    for t in range(T):
        S = dec * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out.append(torch.einsum("hkv,hk->hv", S, q[t]).reshape(-1))
    o = rms_unit(torch.stack(out), eps) * W[p + "norm"]
    o = o * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def parallel(h, W, p, m, eps):
    left = chunked_attention(h, W, p + "left.", m["left"])
    right = lightning(h, W, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def dense_ff(h, W, p):
    a = torch.relu(h @ W[p + "up"].T)
    return (a * a) @ W[p + "down"].T


def forward(cfg, W, tokens, dtype=torch.float64, return_layers=False):
    """Whole-sequence logits [T, vocab] (and the residual after every layer)."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    layers = []
    for i, L in enumerate(cfg["layers"]):
        src = L.get("weights_of", i)
        p = "l%d." % src
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        h = h + causal_conv(h, W[p + "canon1"])
        m = L["mixer"]
        if L["type"] == "mingru":
            y = mingru(h, W, p + "mix.")
        elif L["type"] == "wkv":
            y = wkv(h, W, p + "mix.", m["heads"], m["dim"], eps)
        elif L["type"] == "parallel":
            y = parallel(h, W, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        x = x + y
        if L.get("mlp") is not None:
            assert L["mlp"]["kind"] == "dense"
            h = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps)
            x = x + dense_ff(h, W, p + "mlp.")
        layers.append(x)
    h = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    logits = h @ W["head"].T
    if return_layers:
        return logits, torch.stack(layers)
    return logits


def random_weights(cfg, seed=0, dtype=torch.bfloat16, scale=1.0):
    """Random checkpoint for a config: name -> tensor, shapes as the design
    stores them (linear weights [out, in])."""
    g = torch.Generator().manual_seed(seed)
    Wd = cfg["width"]
    taps = cfg["canon"]["taps"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s * scale).to(dtype)

    def lin(o, i):
        return rnd(o, i, s=1.0 / math.sqrt(i))

    W = {"embed": rnd(cfg["vocab"], Wd, s=0.5), "head": lin(cfg["vocab"], Wd)}
    W["final.norm"] = (1 + rnd(Wd, s=0.1)).to(dtype)
    W["final.norm.b"] = rnd(Wd, s=0.1)
    for i, L in enumerate(cfg["layers"]):
        if "weights_of" in L:
            continue
        p = "l%d." % i
        W[p + "norm1"] = (1 + rnd(Wd, s=0.1)).to(dtype)
        W[p + "norm1.b"] = rnd(Wd, s=0.1)
        W[p + "canon1"] = rnd(Wd, taps, s=0.3)
        m = L["mixer"]
        q = p + "mix."
        if L["type"] == "mingru":
            n = m["width"]
            for s in "zxg":
                W[q + s] = lin(n, Wd)
            W[q + "z.b"] = rnd(n, s=0.5)
            W[q + "x.b"] = rnd(n, s=0.5)
            W[q + "o"] = lin(Wd, n)
        elif L["type"] == "wkv":
            n = m["heads"] * m["dim"]
            for s in "rkvgw":
                W[q + "mu." + s] = torch.rand(Wd, generator=g).to(dtype)
            for s in "rkvg":
                W[q + s] = lin(n, Wd)
            lr = max(4, Wd // 16)
            W[q + "w1"] = lin(lr, Wd)
            W[q + "w2"] = lin(n, lr)
            W[q + "w0"] = (rnd(n, s=1.0) - 1.0).to(dtype)
            W[q + "u"] = rnd(m["heads"], m["dim"], s=0.5)
            W[q + "norm"] = (1 + rnd(n, s=0.1)).to(dtype)
            W[q + "o"] = lin(Wd, n)
        elif L["type"] == "parallel":
            a, b = m["left"], m["right"]
            sizes = {"q": a["heads"] * a["dim"], "k": a["kv_heads"] * a["dim"],
                     "v": a["kv_heads"] * a["vdim"]}
            for s, n in sizes.items():
                W[q + "left." + s] = lin(n, Wd)
                W[q + "left." + s + ".conv"] = rnd(n, a["conv"], s=0.5)
            W[q + "left.o"] = lin(Wd, a["heads"] * a["vdim"])
            for s in "qkg":
                n = b["heads"] * (b["vdim"] if s == "g" else b["dim"])
                W[q + "right." + s] = lin(n, Wd)
            W[q + "right.v"] = lin(b["heads"] * b["vdim"], Wd)
            W[q + "right.norm"] = (1 + rnd(b["heads"] * b["vdim"], s=0.1)).to(dtype)
            W[q + "right.o"] = lin(Wd, b["heads"] * b["vdim"])
        if L.get("mlp") is not None:
            W[p + "norm2"] = (1 + rnd(Wd, s=0.1)).to(dtype)
            W[p + "norm2.b"] = rnd(Wd, s=0.1)
            W[p + "mlp.up"] = lin(L["mlp"]["ff"], Wd)
            W[p + "mlp.down"] = lin(Wd, L["mlp"]["ff"])
    return W
