"""Plain whole-sequence implementation of the Nugopel decoder, one function
per mechanism, float64 throughout, no cache and no batching. It exists to be
compared with the engine and shares no code with it.

A model is (cfg, W): cfg the parsed config.json, W {tensor name: float64
array}. Every function takes whole-sequence arrays [n, ...].
"""
from __future__ import annotations

import math

import numpy as np


def rms_unit(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def norm_one_plus(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def rotary_frequencies(dims, base, scaling):
    """Per-pair frequencies, wavelength-dependent rescaling applied."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f
    factor, low, high = scaling["factor"], scaling["low"], scaling["high"]
    orig = scaling["original"]
    out = f.copy()
    for i, fi in enumerate(f):
        lam = 2.0 * math.pi / fi
        if lam < orig / high:
            continue
        if lam > orig / low:
            out[i] = fi / factor
        else:
            s = (orig / lam - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate_half(x, pos, freqs):
    """x [n, heads, dim]; the first 2*len(freqs) dims of each head rotate,
    dimension i paired with i + len(freqs)."""
    half = len(freqs)
    a = pos[:, None].astype(np.float64) * freqs[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half : 2 * half]
    out = x.copy()
    out[..., :half] = u * c - v * s
    out[..., half : 2 * half] = v * c + u * s
    return out


def softmax_visible(scores, visible, sink):
    """scores [n, n] for one head; rows are queries. With sink, one is added
    to the denominator (a key of score 0 that carries no value)."""
    s = np.where(visible, scores, -np.inf)
    m = s.max(-1, keepdims=True)
    if sink:
        m = np.maximum(m, 0.0)
    e = np.exp(s - m)
    d = e.sum(-1, keepdims=True)
    if sink:
        d = d + np.exp(-m)
    return e / d


def windowed_attention(h, W, p, mx, eps):
    n = h.shape[0]
    H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = h @ W[p + "q"].T
    k = h @ W[p + "k"].T
    v = h @ W[p + "v"].T
    q = norm_plain(q, W[p + "q.norm"], eps).reshape(n, H, D)
    k = norm_plain(k, W[p + "k.norm"], eps).reshape(n, G, D)
    v = v.reshape(n, G, Dv)
    rot = mx.get("rot")
    pos = np.arange(n)
    if rot and rot.get("dims", 0) > 0:
        fr = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_half(q, pos, fr), rotate_half(k, pos, fr)
    i, j = pos[:, None], pos[None, :]
    vis = j <= i
    size = (mx.get("mask") or {}).get("size", 0)
    if size:
        vis &= (i - j) < size
    out = np.zeros((n, H, Dv))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * mx["scale"]
        out[:, hd] = softmax_visible(s, vis, sink=True) @ v[:, g]
    return out.reshape(n, H * Dv) @ W[p + "o"].T


def latent_of(h, W, p, eps):
    return norm_plain(h @ W[p + "dkv"].T, W[p + "dkv.norm"], eps)


def latent_attention(h, c, W, p, mx):
    """c [n, kv_rank]: this layer's latent, or the one of the layer it
    takes its keys and values from."""
    n = h.shape[0]
    H, D, Dv = mx["heads"], mx["dim"], mx["vdim"]
    q = (h @ W[p + "q"].T).reshape(n, H, D)
    k = (c @ W[p + "uk"].T).reshape(n, H, D)
    v = (c @ W[p + "uv"].T).reshape(n, H, Dv)
    pos = np.arange(n)
    vis = pos[None, :] <= pos[:, None]
    out = np.zeros((n, H, Dv))
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd].T) * mx["scale"]
        out[:, hd] = softmax_visible(s, vis, sink=False) @ v[:, hd]
    gate = 1.0 / (1.0 + np.exp(-(h @ W[p + "g"].T)))
    return (out.reshape(n, H * Dv) * gate) @ W[p + "o"].T


def expert(h, up, down):
    a = np.maximum(h @ up.T, 0.0)
    return (a * a) @ down.T


def routed_feed_forward(h, W, p, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ W[p + "router"].T
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        order = np.argsort(-z[t], kind="stable")[:top]
        w = np.exp(z[t, order] - z[t, order].max())
        w /= w.sum()
        for e, we in zip(order, w):
            out[t] += we * expert(h[t : t + 1], W[f"{p}e{e}.up"], W[f"{p}e{e}.down"])[0]
    if mlp.get("shared"):
        out += expert(h, W[p + "shared.up"], W[p + "shared.down"])
    return out


def forward(cfg, W, tokens, capture=None):
    """Logits [n, vocab]; capture (a list) receives the residual stream
    after every layer."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)]
    latents = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = norm_one_plus(x, W[p + "norm1"], eps)
        mx = L["mixer"]
        if L["type"] == "attention":
            y = windowed_attention(h, W, p + "mix.", mx, eps)
        elif L["type"] == "latent_attention":
            src = mx.get("kv_from")
            if src is None:
                latents[i] = latent_of(h, W, p + "mix.", eps)
                src = i
            y = latent_attention(h, latents[src], W, p + "mix.", mx)
        else:
            raise ValueError(L["type"])
        x = x + norm_one_plus(y, W[p + "norm1b"], eps)
        if L.get("mlp") is not None:
            h = norm_one_plus(x, W[p + "norm2"], eps)
            y = routed_feed_forward(h, W, p + "mlp.", L["mlp"])
            x = x + norm_one_plus(y, W[p + "norm2b"], eps)
        if capture is not None:
            capture.append(x.copy())
    x = norm_one_plus(x, W["final.norm"], eps)
    return x @ W["head"].T


def random_weights(cfg, seed):
    """{name: bfloat16 torch tensor} for a config; norm offsets around zero,
    plain norm weights around one."""
    import torch

    g = torch.Generator().manual_seed(seed)
    W = {}

    def mat(name, n_out, n_in, gain=1.0):
        W[name] = (torch.randn(n_out, n_in, generator=g) * gain * n_in ** -0.5).bfloat16()

    def vec(name, n, center):
        W[name] = (center + 0.2 * torch.randn(n, generator=g)).bfloat16()

    width, vocab = cfg["width"], cfg["vocab"]
    W["embed"] = torch.randn(vocab, width, generator=g).bfloat16()
    mat("head", vocab, width)
    vec("final.norm", width, 0.0)
    for i, L in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", L["mixer"]
        vec(p + "norm1", width, 0.0)
        vec(p + "norm1b", width, 0.0)
        if L["type"] == "attention":
            H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            mat(p + "mix.q", H * D, width)
            mat(p + "mix.k", G * D, width)
            mat(p + "mix.v", G * Dv, width)
            vec(p + "mix.q.norm", H * D, 1.0)
            vec(p + "mix.k.norm", G * D, 1.0)
            mat(p + "mix.o", width, H * Dv)
        else:
            H, D, Dv, R = mx["heads"], mx["dim"], mx["vdim"], mx["kv_rank"]
            mat(p + "mix.q", H * D, width, 2.0)
            if mx.get("kv_from") is None:
                mat(p + "mix.dkv", R, width)
                vec(p + "mix.dkv.norm", R, 1.0)
            mat(p + "mix.uk", H * D, R, 2.0)
            mat(p + "mix.uv", H * Dv, R)
            mat(p + "mix.g", H * Dv, width)
            mat(p + "mix.o", width, H * Dv)
        mlp = L.get("mlp")
        if mlp is not None:
            vec(p + "norm2", width, 0.0)
            vec(p + "norm2b", width, 0.0)
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                mat(f"{p}mlp.e{e}.up", ff, width)
                mat(f"{p}mlp.e{e}.down", width, ff)
            mat(p + "mlp.router", mlp["router"]["experts"], width, 3.0)
            if mlp.get("shared"):
                mat(p + "mlp.shared.up", mlp["shared"]["ff"], width)
                mat(p + "mlp.shared.down", width, mlp["shared"]["ff"])
    return W


def as_float64(W):
    return {k: v.double().numpy() for k, v in W.items()}
