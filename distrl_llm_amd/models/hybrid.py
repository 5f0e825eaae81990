"""Layer-list ("hybrid") decoder models: every layer names its own mixer.

The dense families in ``model.py`` repeat one block; the models here are
described by a list of layers, each with a token mixer of some kind
(windowed latent attention, a minGRU recurrence, ...) and an optional
mixture-of-experts feed-forward. A design is a small table that maps its
``config.json`` onto these generic layer specs and its tensor names onto
the packed weights the engine's step function reads; the mechanisms
themselves (``ops/seqmix.py``) take every size and constant as a
parameter, so another design can reuse them in another order.

``Nibalix`` is the first design of this kind:

* residual stream in fp32; one offset-weight RMS norm per layer feeds both
  sublayers (parallel arrangement), ``x += m * (g1*mixer + g2*ff)`` with
  sigmoid gates read from the normed input;
* the mixer reads ``h + conv(h)``, a short causal depthwise convolution;
* mixers: latent attention (a low-rank latent plus one rotated key part
  shared by the heads is all that is cached; sliding window; a layer may
  read another layer's cache) and minGRU (gates depend on the current
  token only; fp32 state carried per sequence);
* feed-forward: top-k mixture of SiLU-gated experts, softmax over the
  chosen logits.

``Nedasun`` is the second:

* residual stream in fp32; sequential sublayers, each with an offset RMS
  norm before and after it (sandwich arrangement),
  ``x += norm_b(mixer(norm_a(x)))`` then the same around the feed-forward;
* mixers: grouped-query softmax attention over a paged K/V cache
  (interleaved-pair rotary on part of each head, tanh-capped scores, a
  learned per-head sink in the softmax denominator, the heads' weights
  mixed by a learned matrix, values blended with the first such layer's
  values) and the gated delta rule (short causal convolutions with SiLU on
  q/k/v, unit-norm q/k, per-head decay and write strength, fp32 matrix
  state per head and sequence, gated RMS norm on the read-out);
* feed-forward: a clamped GLU, dense or as a mixture of experts whose
  router takes a softmax over all outputs, chooses with an added
  correction, scales the unnormalised scores, may name identity experts
  and adds an always-on shared expert.
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn


# ------------------------------------------------------------------ specs

@dataclass(frozen=True)
class LatentAttentionSpec:
    heads: int
    dim: int            # unrotated q/k dims per head
    rot_dim: int        # rotated q/k dims per head (the key part is shared)
    vdim: int
    kv_rank: int
    scale: float
    rope_base: float
    rope_dims: int      # how many of the rot_dim entries are rotated
    window: int         # 0 = unbounded causal
    kv_from: Optional[int] = None   # layer whose cache this layer reads

    kind = "latent_attention"

    @property
    def q_size(self) -> int:
        return self.heads * (self.dim + self.rot_dim)

    @property
    def cache_width(self) -> int:
        return self.kv_rank + self.rot_dim


@dataclass(frozen=True)
class MinGRUSpec:
    width: int
    kind = "mingru"

    @property
    def state_size(self) -> int:
        return self.width


@dataclass(frozen=True)
class SinkAttentionSpec:
    """Grouped-query softmax attention over paged K/V rows."""
    heads: int
    kv_heads: int
    dim: int            # q/k dims per head
    vdim: int
    scale: float
    softcap: float      # 0 = scores are not capped
    rope_base: float
    rope_dims: int      # leading dims of each head rotated as (2i, 2i+1) pairs
    v_first: Optional[int] = None   # layer whose fresh values are blended in
    v_mix: bool = False             # this layer takes part in value mixing

    kind = "sink_attention"

    @property
    def q_size(self) -> int:
        return self.heads * self.dim

    @property
    def k_size(self) -> int:
        return self.kv_heads * self.dim

    @property
    def v_size(self) -> int:
        return self.kv_heads * self.vdim

    @property
    def cache_width(self) -> int:      # one cache row = [k heads | v heads]
        return self.k_size + self.v_size


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Gated delta rule with short convolutions on q, k and v."""
    heads: int          # value heads (one state matrix each)
    kv_heads: int       # q/k heads, shared by heads // kv_heads value heads
    dim: int
    vdim: int
    taps: int

    kind = "delta_rule"

    @property
    def qk_size(self) -> int:
        return self.kv_heads * self.dim

    @property
    def v_size(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:    # q | k | v, convolved together
        return 2 * self.qk_size + self.v_size

    @property
    def state_size(self) -> int:
        return self.heads * self.dim * self.vdim


@dataclass(frozen=True)
class GluSpec:
    """Clamped GLU: g = min(gate, limit), u = clamp(up, +-limit),
    y = g * sigmoid(1.702 g) * (u + 1)."""
    ff: int
    limit: float


@dataclass(frozen=True)
class MoESpec:
    experts: int
    top: int
    ff: int
    # routing "chosen": softmax over the chosen logits; "all": softmax over
    # every router output, choice by score + correction, weight = score * scale
    routing: str = "chosen"
    identity: int = 0       # trailing router outputs that pass the input through
    scale: float = 1.0
    limit: float = 0.0      # 0: SiLU-gated experts; > 0: clamped GLU experts
    shared: Optional[GluSpec] = None


@dataclass(frozen=True)
class LayerSpec:
    mixer: object
    mlp: object         # MoESpec, GluSpec or None


@dataclass(frozen=True)
class HybridSpec:
    name: str
    vocab_size: int
    width: int
    norm_eps: float
    residual_mult: float
    conv_taps: int
    layers: tuple = field(default_factory=tuple)
    # "parallel_gated": one norm feeds mixer and feed-forward, gated sum;
    # "sandwich": norm before and after each sublayer, one after the other
    block: str = "parallel_gated"
    design: str = "nibalix"

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def nibalix_spec_from_config(cfg: dict, name: str = "nibalix") -> HybridSpec:
    """Map a Nibalix ``config.json`` onto the generic layer specs."""
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        mc = lc["mixer"]
        if lc["type"] == "latent_attention":
            rot = mc.get("rot") or {}
            mixer = LatentAttentionSpec(
                heads=int(mc["heads"]), dim=int(mc["dim"]),
                rot_dim=int(mc["rot_dim"]), vdim=int(mc["vdim"]),
                kv_rank=int(mc["kv_rank"]),
                scale=float(mc["scale"] if mc.get("scale") is not None
                            else (int(mc["dim"]) + int(mc["rot_dim"])) ** -0.5),
                rope_base=float(rot.get("base") or 10000.0),
                rope_dims=int(rot["dims"] if rot.get("dims") is not None
                              else mc["rot_dim"]),
                window=int((mc.get("mask") or {}).get("size") or 0),
                kv_from=(int(mc["kv_from"]) if mc.get("kv_from") is not None
                         else None))
            if mixer.rope_dims > mixer.rot_dim or mixer.rope_dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and "
                                 f"<= rot_dim")
        elif lc["type"] == "mingru":
            mixer = MinGRUSpec(width=int(mc["width"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
        fc = lc.get("mlp")
        mlp = None
        if fc is not None:
            if fc.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: unknown mlp kind {fc['kind']!r}")
            mlp = MoESpec(experts=int(fc["router"]["experts"]),
                          top=int(fc["router"]["top"]),
                          ff=int(fc["expert"]["ff"]))
            if not 1 <= mlp.top <= mlp.experts:
                raise ValueError(f"layer {i}: top must be in [1, experts]")
        layers.append(LayerSpec(mixer, mlp))
    for i, ls in enumerate(layers):
        m = ls.mixer
        if isinstance(m, LatentAttentionSpec) and m.kv_from is not None:
            src = layers[m.kv_from].mixer if 0 <= m.kv_from < i else None
            if (not isinstance(src, LatentAttentionSpec)
                    or src.kv_from is not None
                    or src.cache_width != m.cache_width
                    or src.kv_rank != m.kv_rank):
                raise ValueError(f"layer {i}: kv_from must name an earlier "
                                 f"latent layer with a cache of its own and "
                                 f"equal kv_rank/rot_dim")
    return HybridSpec(name=name, vocab_size=int(cfg["vocab"]),
                      width=int(cfg["width"]),
                      norm_eps=float(cfg["norm"]["eps"]),
                      residual_mult=float(cfg["residual_mult"]),
                      conv_taps=int((cfg.get("canon") or {}).get("taps") or 0),
                      layers=tuple(layers))


def nibalix_config_from_spec(spec: HybridSpec) -> dict:
    """Inverse of :func:`nibalix_spec_from_config` (checkpoint saving)."""
    layers = []
    for ls in spec.layers:
        m = ls.mixer
        if isinstance(m, LatentAttentionSpec):
            mc = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
                  "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                  "rot": {"base": m.rope_base, "dims": m.rope_dims}}
            if m.window:
                mc["mask"] = {"size": m.window}
            if m.kv_from is not None:
                mc["kv_from"] = m.kv_from
            typ = "latent_attention"
        else:
            mc, typ = {"width": m.width}, "mingru"
        fc = None
        if ls.mlp is not None:
            fc = {"kind": "moe", "expert": {"ff": ls.mlp.ff},
                  "router": {"experts": ls.mlp.experts, "top": ls.mlp.top}}
        layers.append({"type": typ, "mixer": mc, "mlp": fc})
    out = {"architecture": "Nibalix", "layers": layers,
           "norm": {"eps": spec.norm_eps},
           "residual_mult": spec.residual_mult, "vocab": spec.vocab_size,
           "width": spec.width}
    if spec.conv_taps:
        out["canon"] = {"taps": spec.conv_taps}
    return out


# ---------------------------------------------------------------- weights

class HybridLayer(nn.Module):
    """Packed inference weights of one layer.

    Projections that read the same input are stacked along the output
    axis so each input feeds one GEMM: ``in_w`` = [q; dkv] (latent),
    [z; x; g] (minGRU), [q; k; v] (sink attention) or [q; k; v; g] (delta
    rule); ``exp_gu``/``gu_w`` = [gate; up]. The block arrangement adds its
    own tensors: ``gate_w`` = [rg1; rg2] on the normed input (parallel
    gated), or the norms before/after each sublayer (sandwich)."""

    def __init__(self, spec: HybridSpec, ls: LayerSpec, dtype, device):
        super().__init__()
        D = spec.width

        def P(*shape, dt=dtype):
            return nn.Parameter(torch.zeros(*shape, dtype=dt, device=device),
                                requires_grad=False)

        f32 = torch.float32
        self.norm_w = P(D, dt=f32)
        if spec.block == "sandwich":
            self.post_w = P(D, dt=f32)
            if ls.mlp is not None:
                self.ff_norm_w, self.ff_post_w = P(D, dt=f32), P(D, dt=f32)
        else:
            if spec.conv_taps:  # 0: the mixer reads the normed input as it is
                self.conv_w = P(D, spec.conv_taps, dt=f32)
            n_gate = 2 * D if ls.mlp is not None else D
            self.gate_w, self.gate_b = P(n_gate, D), P(n_gate, dt=f32)
        m = ls.mixer
        if isinstance(m, LatentAttentionSpec):
            own = m.kv_from is None
            self.in_w = P(m.q_size + (m.cache_width if own else 0), D)
            if own:
                self.latent_norm_w = P(m.kv_rank, dt=f32)
            self.uk = P(m.heads, m.dim, m.kv_rank)
            self.uv = P(m.heads, m.vdim, m.kv_rank)
            self.out_w = P(D, m.heads * m.vdim)
        elif isinstance(m, SinkAttentionSpec):
            self.in_w = P(m.q_size + m.cache_width, D)
            self.talk = P(m.heads, m.heads, dt=f32)
            self.sink = P(m.heads, dt=f32)
            self.vmix = P(1, dt=f32)
            self.out_w = P(D, m.heads * m.vdim)
        elif isinstance(m, DeltaRuleSpec):
            self.in_w = P(m.conv_channels + m.v_size, D)
            self.conv_w = P(m.conv_channels, m.taps, dt=f32)
            self.ab_w = P(2 * m.heads, D, dt=f32)       # [write strength; step]
            self.a_log, self.dt_bias = P(m.heads, dt=f32), P(m.heads, dt=f32)
            self.onorm_w = P(m.vdim, dt=f32)
            self.out_w = P(D, m.v_size)
        else:
            self.in_w, self.in_b = P(3 * m.width, D), P(3 * m.width, dt=f32)
            self.out_w = P(D, m.width)
        f = ls.mlp
        if isinstance(f, GluSpec):
            self.gu_w, self.down_w = P(2 * f.ff, D), P(D, f.ff)
        elif f is not None:
            n = f.experts + f.identity
            self.router_w, self.router_b = P(n, D, dt=f32), P(n, dt=f32)
            if f.routing == "all":
                self.correction = P(n, dt=f32)
            self.exp_gu = P(f.experts, 2 * f.ff, D)
            self.exp_down = P(f.experts, D, f.ff)
            if f.shared is not None:
                self.shared_gu = P(2 * f.shared.ff, D)
                self.shared_down = P(D, f.shared.ff)


class HybridLM(nn.Module):
    """Inference weights of a layer-list model. ``dtype`` is the matrix
    dtype (bf16 or fp32); norm, conv, bias and router tensors stay fp32."""

    def __init__(self, spec: HybridSpec, dtype: torch.dtype = torch.bfloat16,
                 device=None):
        super().__init__()
        self.spec = spec
        self.dtype_ = dtype
        D = spec.width
        f32 = torch.float32

        def P(*shape, dt=dtype):
            return nn.Parameter(torch.zeros(*shape, dtype=dt, device=device),
                                requires_grad=False)

        self.embed = P(spec.vocab_size, D)
        if spec.design == "nibalix":
            self.embed_norm_w = P(D, dt=f32)
        self.final_norm_w = P(D, dt=f32)
        self.head = P(spec.vocab_size, D)
        self.layers = nn.ModuleList(
            [HybridLayer(spec, ls, dtype, device) for ls in spec.layers])

    @property
    def device(self):
        return self.embed.device

    # ---- the design's tensor names <-> packed weights -------------------

    def _named_slices(self) -> Dict[str, tuple]:
        """{checkpoint tensor name: (packed parameter, row0, rows | None)}.
        ``rows`` None means the tensor fills the whole parameter; expert
        entries carry an index tuple instead of a row range."""
        if self.spec.design == "nedasun":
            return _nedasun_named_slices(self)
        out = {"embed": (self.embed, None), "embed.norm": (self.embed_norm_w, None),
               "final.norm": (self.final_norm_w, None), "head": (self.head, None)}
        D = self.spec.width
        for i, (ls, L) in enumerate(zip(self.spec.layers, self.layers)):
            p = f"l{i}."
            out[p + "norm1"] = (L.norm_w, None)
            if self.spec.conv_taps:
                out[p + "canon1"] = (L.conv_w, None)
            out[p + "rg1"], out[p + "rg1.b"] = (L.gate_w, (0, D)), (L.gate_b, (0, D))
            m = ls.mixer
            if isinstance(m, LatentAttentionSpec):
                out[p + "mix.q"] = (L.in_w, (0, m.q_size))
                if m.kv_from is None:
                    out[p + "mix.dkv"] = (L.in_w, (m.q_size, m.cache_width))
                    out[p + "mix.dkv.norm"] = (L.latent_norm_w, None)
                out[p + "mix.uk"] = (L.uk, "flat")
                out[p + "mix.uv"] = (L.uv, "flat")
            else:
                n = m.width
                for k, nm in enumerate(("z", "x", "g")):
                    out[p + "mix." + nm] = (L.in_w, (k * n, n))
                out[p + "mix.z.b"] = (L.in_b, (0, n))
                out[p + "mix.x.b"] = (L.in_b, (n, n))
            out[p + "mix.o"] = (L.out_w, None)
            if ls.mlp is not None:
                f = ls.mlp
                out[p + "rg2"], out[p + "rg2.b"] = (L.gate_w, (D, D)), (L.gate_b, (D, D))
                out[p + "mlp.router"] = (L.router_w, None)
                out[p + "mlp.router.b"] = (L.router_b, None)
                for e in range(f.experts):
                    out[f"{p}mlp.e{e}.gate"] = (L.exp_gu[e], (0, f.ff))
                    out[f"{p}mlp.e{e}.up"] = (L.exp_gu[e], (f.ff, f.ff))
                    out[f"{p}mlp.e{e}.down"] = (L.exp_down[e], None)
        return out

    @staticmethod
    def _view(param, where):
        if where is None:
            return param
        if where == "flat":
            return param.view(-1, param.shape[-1])
        r0, n = where
        return param[r0:r0 + n]

    @torch.no_grad()
    def load_tensors(self, tensors: Dict[str, torch.Tensor], strict=True) -> int:
        names = self._named_slices()
        for k, v in tensors.items():
            if k not in names:
                if strict:
                    raise ValueError(f"unexpected checkpoint tensor {k!r}")
                continue
            dst = self._view(*names[k])
            if v.dim() == 0 and dst.numel() == 1:
                v = v.reshape(dst.shape)
            if tuple(dst.shape) != tuple(v.shape):
                raise ValueError(f"shape mismatch for {k}: checkpoint "
                                 f"{tuple(v.shape)} vs model {tuple(dst.shape)}")
            dst.copy_(v.to(dst.dtype))
        missing = set(names) - set(tensors)
        if strict and missing:
            raise ValueError(f"checkpoint misses tensors: {sorted(missing)[:8]}")
        return len(names) - len(missing)

    def export_tensors(self, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
        scalars = _SCALAR_TENSORS.get(self.spec.design, ())
        out = {}
        for k, w in self._named_slices().items():
            t = self._view(*w).detach().to(dtype).contiguous().cpu()
            out[k] = t.reshape(()) if k.rsplit(".", 1)[-1] in scalars else t
        return out

    @torch.no_grad()
    def random_init(self, seed: int = 3407) -> "HybridLM":
        """Deterministic random weights (synthetic benches and tests)."""
        dev = self.device
        g = torch.Generator(device=dev).manual_seed(seed)
        for name, (param, where) in sorted(self._named_slices().items()):
            dst = self._view(param, where)
            r = torch.randn(dst.shape, generator=g, dtype=torch.float32, device=dev)
            last = name.rsplit(".", 1)[-1]
            if name == "embed":
                pass
            elif last == "talk":
                r = torch.eye(dst.shape[0], device=dev) + 0.2 * r
            elif last == "vmix":
                r = 0.3 + 0.1 * r
            elif last == "conv":
                r *= 0.5
            elif dst.dim() >= 2 and "canon" not in name:
                r *= 1.0 / math.sqrt(dst.shape[-1])
            elif name.endswith("dkv.norm") or name.endswith("mix.norm"):
                r = 1.0 + 0.1 * r
            else:
                r *= 0.1
            dst.copy_(r.to(dst.dtype))
        return self


# ------------------------------------------------------------ checkpoints

def load_nibalix_checkpoint(path: str, dtype=torch.bfloat16, device=None) -> HybridLM:
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    name = os.path.basename(os.path.normpath(path)) or "nibalix"
    model = HybridLM(nibalix_spec_from_config(cfg, name), dtype=dtype, device=device)
    tensors = load_file(os.path.join(path, "model.safetensors"))
    known = model._named_slices()
    extra = sorted(k for k in tensors if k not in known)
    if extra:
        import sys
        sys.stderr.write(f"[nibalix] ignoring {len(extra)} tensors the design "
                         f"does not name: {extra[:4]}\n")
    model.load_tensors({k: v for k, v in tensors.items() if k in known})
    return model


def save_nibalix_checkpoint(model: HybridLM, path: str) -> None:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file(model.export_tensors(), os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(nibalix_config_from_spec(model.spec), f, indent=1)


# ---------------------------------------------------------------- Nedasun

_SCALAR_TENSORS = {"nedasun": ("vmix",)}   # stored with shape ()


def _glu_from_config(fc: dict) -> GluSpec:
    return GluSpec(ff=int(fc["ff"]), limit=float(fc["limit"]))


def nedasun_spec_from_config(cfg: dict, name: str = "nedasun") -> HybridSpec:
    """Map a Nedasun ``config.json`` onto the generic layer specs."""
    layers, v_first = [], None
    for i, lc in enumerate(cfg["layers"]):
        mc = lc["mixer"]
        heads, kvh = int(mc["heads"]), int(mc["kv_heads"])
        if kvh < 1 or heads % kvh:
            raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
        if lc["type"] == "attention":
            rot = mc.get("rot") or {}
            mixes = bool(mc.get("v_mix"))
            mixer = SinkAttentionSpec(
                heads=heads, kv_heads=kvh, dim=int(mc["dim"]),
                vdim=int(mc["vdim"]), scale=float(mc["scale"]),
                softcap=float(mc.get("softcap") or 0.0),
                rope_base=float(rot.get("base") or 10000.0),
                rope_dims=int(rot.get("dims") or 0), v_mix=mixes,
                v_first=v_first if mixes else None)
            if mixer.rope_dims > mixer.dim or mixer.rope_dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and <= dim")
            if mixes and v_first is None:
                v_first = i
            elif mixes and ((layers[v_first].mixer.kv_heads, layers[v_first].mixer.vdim)
                            != (kvh, mixer.vdim)):
                raise ValueError(f"layer {i}: value mixing needs the first "
                                 f"mixing layer's kv_heads and vdim")
        elif lc["type"] == "delta":
            mixer = DeltaRuleSpec(heads=heads, kv_heads=kvh, dim=int(mc["dim"]),
                                  vdim=int(mc["vdim"]), taps=int(mc["conv"]))
            if mixer.taps < 1:
                raise ValueError(f"layer {i}: conv needs at least one tap")
        else:
            raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
        fc = lc.get("mlp")
        mlp = None
        if fc is not None and fc.get("kind") == "dense":
            mlp = _glu_from_config(fc)
        elif fc is not None and fc.get("kind") == "moe":
            rc = fc["router"]
            mlp = MoESpec(experts=int(rc["experts"]), top=int(rc["top"]),
                          ff=int(fc["expert"]["ff"]), routing="all",
                          identity=int(rc.get("identity") or 0),
                          scale=float(rc.get("scale", 1.0)),
                          limit=float(fc["expert"]["limit"]),
                          shared=(_glu_from_config(fc["shared"])
                                  if fc.get("shared") else None))
            if not 1 <= mlp.top <= mlp.experts + mlp.identity:
                raise ValueError(f"layer {i}: top must be in [1, experts + identity]")
            if mlp.limit <= 0:
                raise ValueError(f"layer {i}: expert limit must be positive")
        elif fc is not None:
            raise ValueError(f"layer {i}: unknown mlp kind {fc.get('kind')!r}")
        layers.append(LayerSpec(mixer, mlp))
    return HybridSpec(name=name, vocab_size=int(cfg["vocab"]),
                      width=int(cfg["width"]),
                      norm_eps=float(cfg["norm"]["eps"]), residual_mult=1.0,
                      conv_taps=0, layers=tuple(layers), block="sandwich",
                      design="nedasun")


def nedasun_config_from_spec(spec: HybridSpec) -> dict:
    """Inverse of :func:`nedasun_spec_from_config` (checkpoint saving)."""
    layers = []
    for ls in spec.layers:
        m = ls.mixer
        if isinstance(m, SinkAttentionSpec):
            mc = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                  "vdim": m.vdim, "scale": m.scale, "softcap": m.softcap,
                  "rot": {"base": m.rope_base, "dims": m.rope_dims},
                  "v_mix": m.v_mix}
            typ = "attention"
        else:
            mc = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                  "vdim": m.vdim, "conv": m.taps}
            typ = "delta"
        f, fc = ls.mlp, None
        if isinstance(f, GluSpec):
            fc = {"kind": "dense", "ff": f.ff, "limit": f.limit}
        elif f is not None:
            fc = {"kind": "moe", "expert": {"ff": f.ff, "limit": f.limit},
                  "router": {"experts": f.experts, "identity": f.identity,
                             "scale": f.scale, "top": f.top},
                  "shared": ({"ff": f.shared.ff, "limit": f.shared.limit}
                             if f.shared is not None else None)}
        layers.append({"type": typ, "mixer": mc, "mlp": fc})
    return {"architecture": "Nedasun", "layers": layers,
            "norm": {"eps": spec.norm_eps}, "vocab": spec.vocab_size,
            "width": spec.width}


def _nedasun_named_slices(model: "HybridLM") -> Dict[str, tuple]:
    out = {"embed": (model.embed, None), "final.norm": (model.final_norm_w, None),
           "head": (model.head, None)}

    def glu(pre, gu, down, ff):
        out[pre + "gate"], out[pre + "up"] = (gu, (0, ff)), (gu, (ff, ff))
        out[pre + "down"] = (down, None)

    for i, (ls, L) in enumerate(zip(model.spec.layers, model.layers)):
        p, m = f"l{i}.", ls.mixer
        out[p + "norm1"], out[p + "norm1b"] = (L.norm_w, None), (L.post_w, None)
        x = p + "mix."
        if isinstance(m, SinkAttentionSpec):
            out[x + "q"] = (L.in_w, (0, m.q_size))
            out[x + "k"] = (L.in_w, (m.q_size, m.k_size))
            out[x + "v"] = (L.in_w, (m.q_size + m.k_size, m.v_size))
            out[x + "vmix"], out[x + "talk"] = (L.vmix, None), (L.talk, None)
            out[x + "sink"] = (L.sink, None)
        else:
            n, nv = m.qk_size, m.v_size
            for nm, r0, rows in (("q", 0, n), ("k", n, n), ("v", 2 * n, nv)):
                out[x + nm] = (L.in_w, (r0, rows))
                out[x + nm + ".conv"] = (L.conv_w, (r0, rows))
            out[x + "g"] = (L.in_w, (2 * n + nv, nv))
            out[x + "b"] = (L.ab_w, (0, m.heads))
            out[x + "a"] = (L.ab_w, (m.heads, m.heads))
            out[x + "A_log"], out[x + "dt_bias"] = (L.a_log, None), (L.dt_bias, None)
            out[x + "norm"] = (L.onorm_w, None)
        out[x + "o"] = (L.out_w, None)
        f = ls.mlp
        if f is None:
            continue
        out[p + "norm2"], out[p + "norm2b"] = (L.ff_norm_w, None), (L.ff_post_w, None)
        x = p + "mlp."
        if isinstance(f, GluSpec):
            glu(x, L.gu_w, L.down_w, f.ff)
            continue
        out[x + "router"], out[x + "correction"] = (L.router_w, None), (L.correction, None)
        for e in range(f.experts):
            glu(f"{x}e{e}.", L.exp_gu[e], L.exp_down[e], f.ff)
        if f.shared is not None:
            glu(x + "shared.", L.shared_gu, L.shared_down, f.shared.ff)
    return out


def load_nedasun_checkpoint(path: str, dtype=torch.bfloat16, device=None) -> HybridLM:
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    name = os.path.basename(os.path.normpath(path)) or "nedasun"
    model = HybridLM(nedasun_spec_from_config(cfg, name), dtype=dtype, device=device)
    tensors = load_file(os.path.join(path, "model.safetensors"))
    known = model._named_slices()
    extra = sorted(k for k in tensors if k not in known)
    if extra:
        import sys
        sys.stderr.write(f"[nedasun] ignoring {len(extra)} tensors the design "
                         f"does not name: {extra[:4]}\n")
    # the blend factor is read only by mixing layers after the first one: a
    # checkpoint may leave it out elsewhere
    unused = {f"l{i}.mix.vmix" for i, ls in enumerate(model.spec.layers)
              if isinstance(ls.mixer, SinkAttentionSpec) and ls.mixer.v_first is None}
    have = {k: v for k, v in tensors.items() if k in known}
    missing = set(known) - set(have) - unused
    if missing:
        raise ValueError(f"checkpoint misses tensors: {sorted(missing)[:8]}")
    model.load_tensors(have, strict=False)
    return model


def save_nedasun_checkpoint(model: HybridLM, path: str) -> None:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file(model.export_tensors(), os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(nedasun_config_from_spec(model.spec), f, indent=1)
