"""Dulotar: a hybrid decoder whose layers pick their mixer from the config —
minGRU recurrence, WKV time mixing, or chunked softmax attention in parallel
with lightning attention — each behind a LayerNorm and a per-layer causal
input convolution, with optional squared-ReLU feed-forwards and layers that
reuse another layer's tensors (with state of their own).

Execution model matches the other decoder families: one token-packed forward
per engine step over the ForwardBatch; GEMMs through the BLAS library in the
serving dtype; everything else in hand-written gfx950 kernels
(kubeai_amd.ops.seq). The residual stream is fp32 throughout: each sublayer's
branch output is added to it inside the next LayerNorm kernel.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from kubeai_amd.engine.batch import ForwardBatch
from kubeai_amd.ops import seq as sops
from .config import HybridLayerSpec, ModelArchConfig
from .mixers import (
    CausalConvTails,
    ChunkedAttention,
    LightningAttention,
    MinGRUMixer,
    ParallelMixer,
    SquaredReluMLP,
    WKVMixer,
    _f32,
)


def build_mixer(spec: HybridLayerSpec, width: int, eps: float) -> nn.Module:
    m = spec.mixer
    if spec.type == "mingru":
        return MinGRUMixer(width, int(m["width"]))
    if spec.type == "wkv":
        return WKVMixer(width, int(m["heads"]), int(m["dim"]),
                        int(m.get("lowrank", max(4, width // 16))), eps)
    if spec.type == "parallel":
        a, b = m["left"], m["right"]
        rot = a.get("rot") or {}
        left = ChunkedAttention(
            heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]),
            vdim=int(a["vdim"]), conv_taps=int(a.get("conv") or 0),
            rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 1.0)),
            scale=a["scale"], softcap=a.get("softcap") or 0.0,
            chunk=int((a.get("mask") or {}).get("size", 0)),
        )
        right = LightningAttention(int(b["heads"]), int(b["dim"]), int(b["vdim"]),
                                   b["decay"], eps)
        return ParallelMixer(width, left, right, m["left_scale"], m["right_scale"])
    raise ValueError(f"unknown mixer type {spec.type!r}")


class HybridLayer(nn.Module):
    def __init__(self, spec: HybridLayerSpec, width: int, eps: float, taps: int):
        super().__init__()
        self.eps = eps
        self.norm1_w, self.norm1_b = _f32(width), _f32(width)
        nn.init.ones_(self.norm1_w)
        self.canon = CausalConvTails(width, taps, residual=True) if taps > 0 else None
        self.mixer = build_mixer(spec, width, eps)
        self.mlp = None
        if spec.mlp is not None:
            if spec.mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {spec.mlp['kind']!r}")
            self.norm2_w, self.norm2_b = _f32(width), _f32(width)
            nn.init.ones_(self.norm2_w)
            self.mlp = SquaredReluMLP(width, int(spec.mlp["ff"]))

    def state_spec(self):
        spec = dict(self.mixer.state_spec())
        if self.canon is not None:
            spec["canon"] = self.canon.state_shape()
        return spec

    def forward(self, branch, residual, fb, state, kv_cache, dtype):
        h = sops.add_layernorm(branch, residual, self.norm1_w, self.norm1_b,
                               self.eps, dtype)
        if self.canon is not None:
            h = self.canon(h, fb, state["canon"])
        branch = self.mixer(h, fb, state, kv_cache)
        if self.mlp is not None:
            h = sops.add_layernorm(branch, residual, self.norm2_w, self.norm2_b,
                                   self.eps, dtype)
            branch = self.mlp(h)
        return branch


class DulotarForCausalLM(nn.Module):
    #: the engine gives every live sequence a state slot and builds fb.seq
    has_seq_state = True

    def __init__(self, cfg: ModelArchConfig, device=None, dtype=torch.bfloat16):
        super().__init__()
        assert cfg.hybrid is not None
        self.cfg = cfg
        self.dtype = dtype
        hs = cfg.hybrid
        W = cfg.hidden_size
        prev_dtype = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            with torch.device(device if device is not None else "cpu"):
                self.embed_tokens = nn.Embedding(cfg.vocab_size, W)
                own = {}
                for i, spec in enumerate(hs.layers):
                    if not 0 <= spec.weights_of < len(hs.layers):
                        raise ValueError(f"layer {i}: weights_of out of range")
                    if spec.weights_of == i:
                        own[i] = HybridLayer(spec, W, hs.norm_eps, hs.canon_taps)
                self.layers = nn.ModuleDict({str(i): m for i, m in own.items()})
                self.final_w, self.final_b = _f32(W), _f32(W)
                nn.init.ones_(self.final_w)
                self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W),
                                            requires_grad=False)
                nn.init.normal_(self.lm_head, std=W ** -0.5)
        finally:
            torch.set_default_dtype(prev_dtype)
        # layer runs in execution order: a layer that uses another's tensors
        # runs that module with its own state / cache index
        def owner(i: int) -> int:
            seen = set()
            while hs.layers[i].weights_of != i:  # a shared layer may itself share
                if i in seen:
                    raise ValueError("weights_of forms a cycle")
                seen.add(i)
                i = hs.layers[i].weights_of
            return i

        self.runs = [self.layers[str(owner(i))] for i in range(len(hs.layers))]
        self.capture_layers = None  # set to a list to record per-layer residuals

    # -- what the runner allocates per layer run -------------------------
    def kv_cache_specs(self):
        return [m.mixer.kv_spec() for m in self.runs]

    def state_specs(self):
        return [m.state_spec() for m in self.runs]

    def bind_kv_caches(self, kv_caches):
        self.kv_caches = kv_caches

    def bind_states(self, states):
        self.states = states

    # --------------------------------------------------------------------
    @torch.inference_mode()
    def forward(self, fb: ForwardBatch) -> torch.Tensor:
        hs = self.cfg.hybrid
        residual = self.embed_tokens(fb.input_ids.long()).float() * hs.embedding_scale
        branch = None
        for i, layer in enumerate(self.runs):
            branch = layer(branch, residual, fb, self.states[i], self.kv_caches[i],
                           self.dtype)
            if self.capture_layers is not None:
                self.capture_layers.append(residual + branch.float())
        return sops.add_layernorm(branch, residual, self.final_w, self.final_b,
                                  hs.norm_eps, self.dtype)

    @torch.inference_mode()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.lm_head).float()

    # -- checkpoint names -> fused engine layout -----------------------------
    def load_named_tensors(self, tensors) -> int:
        """tensors: iterable of (name, tensor) with the design's names
        ('l<i>.mix.z', 'l<i>.norm1.b', 'embed', 'head', 'final.norm', ...)."""
        W = {k: v for k, v in tensors}
        used = set()

        def get(name):
            used.add(name)
            return W[name]

        def put(param, value):
            value = value.to(device=param.device, dtype=param.dtype)
            if param.shape != value.shape:
                param.data = value.contiguous()
            else:
                param.data.copy_(value)

        def cat(names):
            return torch.cat([get(n) for n in names], dim=0)

        put(self.embed_tokens.weight, get("embed"))
        put(self.lm_head, get("head"))
        put(self.final_w, get("final.norm"))
        put(self.final_b, get("final.norm.b"))
        for key, layer in self.layers.items():
            p = f"l{key}."
            put(layer.norm1_w, get(p + "norm1"))
            put(layer.norm1_b, get(p + "norm1.b"))
            if layer.canon is not None:
                put(layer.canon.weight, get(p + "canon1"))
            if layer.mlp is not None:
                put(layer.norm2_w, get(p + "norm2"))
                put(layer.norm2_b, get(p + "norm2.b"))
                put(layer.mlp.up.weight, get(p + "mlp.up"))
                put(layer.mlp.down.weight, get(p + "mlp.down"))
            m, q = layer.mixer, p + "mix."
            if isinstance(m, MinGRUMixer):
                put(m.in_proj.weight, cat([q + "z", q + "x", q + "g"]))
                put(m.bias_z, get(q + "z.b"))
                put(m.bias_x, get(q + "x.b"))
                put(m.o_proj.weight, get(q + "o"))
            elif isinstance(m, WKVMixer):
                put(m.mu, torch.stack([get(q + "mu." + s) for s in m.STREAMS]))
                put(m.rkvg, torch.stack([get(q + s) for s in "rkvg"]))
                put(m.w1.weight, get(q + "w1"))
                put(m.w2.weight, get(q + "w2"))
                put(m.w0, get(q + "w0"))
                put(m.u, get(q + "u"))
                put(m.norm, get(q + "norm"))
                put(m.o_proj.weight, get(q + "o"))
            elif isinstance(m, ParallelMixer):
                l, r = q + "left.", q + "right."
                put(m.in_proj.weight,
                    cat([l + "q", l + "k", l + "v", r + "q", r + "k", r + "v", r + "g"]))
                if m.left.conv is not None:
                    put(m.left.conv.weight,
                        cat([l + "q.conv", l + "k.conv", l + "v.conv"]))
                put(m.right.norm, get(r + "norm"))
                put(m.o_proj.weight,
                    torch.cat([get(l + "o"), get(r + "o")], dim=1))
        missing = set(W) - used
        if missing:
            raise ValueError(f"checkpoint tensors not consumed: {sorted(missing)[:8]}")
        return len(used)
