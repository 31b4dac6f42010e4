"""Nugopel: a decoder whose layers alternate, in the order the config lists,
between sliding-window attention (whole-projection q/k norm, split-half
rotary with wavelength-scaled frequencies, sink softmax) and latent
attention (a cached low-rank latent, optionally the one another layer
cached), each followed by a routed mixture of squared-ReLU experts with a
shared expert. Every sublayer is normalised on both sides:
x <- x + norm_b(sublayer(norm_a(x))), RMS norms with weights stored as
offsets from one.

Same execution model as the other decoder families: one token-packed
forward per engine step over the ForwardBatch, GEMMs through the BLAS
library in the serving dtype, everything else in the gfx950 kernels of
kubeai_amd.ops.seq. The residual stream is fp32; a sublayer's post-norm,
the residual add and the next sublayer's pre-norm are one kernel.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from kubeai_amd.engine.batch import ForwardBatch
from kubeai_amd.ops import seq as sops
from .config import HybridLayerSpec, ModelArchConfig
from .mixers import LatentAttention, RoutedSquaredReluMoE, SinkWindowAttention, _f32


def build_mixer(spec: HybridLayerSpec, width: int, eps: float) -> nn.Module:
    m = spec.mixer
    if spec.type == "attention":
        rot = m.get("rot") or {}
        return SinkWindowAttention(
            width, heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
            dim=int(m["dim"]), vdim=int(m["vdim"]), scale=m["scale"],
            window=int((m.get("mask") or {}).get("size", 0)), sink=True,
            qk_norm=True, rot_dims=int(rot.get("dims", 0)),
            rot_base=float(rot.get("base", 1.0)), rot_scaling=rot.get("scaling"),
            eps=eps,
        )
    if spec.type == "latent_attention":
        return LatentAttention(
            width, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
            kv_rank=int(m["kv_rank"]), scale=m["scale"],
            own_latent=m.get("kv_from") is None, eps=eps,
        )
    raise ValueError(f"unknown mixer type {spec.type!r}")


def build_mlp(mlp: dict | None, width: int):
    if mlp is None:
        return None
    if mlp.get("kind", "moe") != "moe":
        raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
    return RoutedSquaredReluMoE(
        width, experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
        ff=int(mlp["expert"]["ff"]),
        shared_ff=int((mlp.get("shared") or {}).get("ff", 0)),
    )


class NugopelLayer(nn.Module):
    def __init__(self, spec: HybridLayerSpec, width: int, eps: float):
        super().__init__()
        self.mixer = build_mixer(spec, width, eps)
        self.mlp = build_mlp(spec.mlp, width)
        # multipliers (1 + stored weight), fp32
        self.norm1, self.norm1b = _f32(width), _f32(width)
        nn.init.ones_(self.norm1)
        nn.init.ones_(self.norm1b)
        if self.mlp is not None:
            self.norm2, self.norm2b = _f32(width), _f32(width)
            nn.init.ones_(self.norm2)
            nn.init.ones_(self.norm2b)


class NugopelForCausalLM(nn.Module):
    #: attention-only: no per-sequence state slots, but the kernels take the
    #: packed runs (SeqMeta), so the engine builds fb.seq
    has_seq_state = False
    uses_seq_meta = True

    def __init__(self, cfg: ModelArchConfig, device=None, dtype=torch.bfloat16):
        super().__init__()
        assert cfg.hybrid is not None
        self.cfg = cfg
        self.dtype = dtype
        hs = cfg.hybrid
        W = cfg.hidden_size
        self.eps = hs.norm_eps
        prev_dtype = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            with torch.device(device if device is not None else "cpu"):
                self.embed_tokens = nn.Embedding(cfg.vocab_size, W)
                self.layers = nn.ModuleList(
                    [NugopelLayer(spec, W, hs.norm_eps) for spec in hs.layers]
                )
                self.final_norm = _f32(W)
                nn.init.ones_(self.final_norm)
                self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W),
                                            requires_grad=False)
                nn.init.normal_(self.lm_head, std=W ** -0.5)
        finally:
            torch.set_default_dtype(prev_dtype)
        # which layer's cache every layer reads: its own, or the one of the
        # layer whose latents it takes
        self.cache_of = []
        for i, spec in enumerate(hs.layers):
            src = spec.mixer.get("kv_from") if spec.type == "latent_attention" else None
            if src is None:
                self.cache_of.append(i)
                continue
            src = int(src)
            if not 0 <= src < i:
                raise ValueError(f"layer {i}: kv_from must name an earlier layer")
            other = hs.layers[src]
            if other.type != "latent_attention" or other.mixer.get("kv_from") is not None:
                raise ValueError(f"layer {i}: kv_from layer {src} caches no latent")
            if int(other.mixer["kv_rank"]) != int(spec.mixer["kv_rank"]):
                raise ValueError(f"layer {i}: kv_rank differs from layer {src}'s")
            self.cache_of.append(src)
        self.capture_layers = None  # set to a list to record per-layer residuals

    def kv_cache_specs(self):
        return [layer.mixer.kv_spec() for layer in self.layers]

    def bind_kv_caches(self, kv_caches):
        self.kv_caches = [kv_caches[j] for j in self.cache_of]

    @torch.inference_mode()
    def forward(self, fb: ForwardBatch) -> torch.Tensor:
        residual = self.embed_tokens(fb.input_ids.long()).float()
        n = len(self.layers)
        h = sops.sandwich_rmsnorm(None, None, residual, self.layers[0].norm1,
                                  self.eps, self.dtype)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            y = layer.mixer(h, fb, None, self.kv_caches[i])
            if layer.mlp is not None:
                h = sops.sandwich_rmsnorm(y, layer.norm1b, residual, layer.norm2,
                                          self.eps, self.dtype)
                y = layer.mlp(h)
                h = sops.sandwich_rmsnorm(y, layer.norm2b, residual, nxt,
                                          self.eps, self.dtype)
            else:
                h = sops.sandwich_rmsnorm(y, layer.norm1b, residual, nxt,
                                          self.eps, self.dtype)
            if self.capture_layers is not None:
                self.capture_layers.append(residual.clone())
        return h

    @torch.inference_mode()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.lm_head).float()

    # -- checkpoint names -> fused engine layout -----------------------------
    def load_named_tensors(self, tensors) -> int:
        """tensors: iterable of (name, tensor) with the design's names
        ('embed', 'l<i>.norm1', 'l<i>.mix.q', 'l<i>.mlp.e<k>.up', 'final.norm',
        'head', ...)."""
        W = {k: v for k, v in tensors}
        used = set()

        def get(name):
            used.add(name)
            return W[name]

        def put(param, value):
            value = value.to(device=param.device, dtype=param.dtype)
            if param.shape != value.shape:
                raise ValueError(
                    f"checkpoint tensor of shape {tuple(value.shape)} does not fit "
                    f"{tuple(param.shape)}")
            param.data.copy_(value)

        def one_plus(name):
            return 1.0 + get(name).float()

        put(self.embed_tokens.weight, get("embed"))
        put(self.lm_head, get("head"))
        put(self.final_norm, one_plus("final.norm"))
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            put(layer.norm1, one_plus(p + "norm1"))
            put(layer.norm1b, one_plus(p + "norm1b"))
            m, q = layer.mixer, p + "mix."
            if isinstance(m, SinkWindowAttention):
                put(m.in_proj.weight, torch.cat([get(q + "q"), get(q + "k"), get(q + "v")]))
                if m.q_norm is not None:
                    put(m.q_norm, get(q + "q.norm"))
                    put(m.k_norm, get(q + "k.norm"))
                put(m.o_proj.weight, get(q + "o"))
            else:
                parts = [get(q + "q"), get(q + "g")]
                if m.own_latent:
                    parts.append(get(q + "dkv"))
                    put(m.latent_norm, get(q + "dkv.norm"))
                put(m.in_proj.weight, torch.cat(parts))
                H, D, Dv, R = m.heads, m.dim, m.vdim, m.rank
                put(m.uk_r, get(q + "uk").reshape(H, D, R).transpose(1, 2))
                put(m.uv, get(q + "uv").reshape(H, Dv, R))
                put(m.o_proj.weight, get(q + "o"))
            if layer.mlp is not None:
                put(layer.norm2, one_plus(p + "norm2"))
                put(layer.norm2b, one_plus(p + "norm2b"))
                f, q = layer.mlp, p + "mlp."
                ups = [get(f"{q}e{e}.up") for e in range(f.experts)]
                downs = [get(f"{q}e{e}.down") for e in range(f.experts)]
                if f.shared_ff:
                    ups.append(get(q + "shared.up"))
                    downs.append(get(q + "shared.down"))
                put(f.up.weight, torch.cat(ups, dim=0))
                put(f.down.weight, torch.cat(downs, dim=1))
                put(f.router, get(q + "router"))
        missing = set(W) - used
        if missing:
            raise ValueError(f"checkpoint tensors not consumed: {sorted(missing)[:8]}")
        return len(used)
