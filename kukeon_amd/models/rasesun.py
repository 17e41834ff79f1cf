"""Rasesun: a decoder that mixes selective state-space layers with
latent-attention layers. Every sublayer is wrapped in two RMS norms,

    x <- x + norm_b(sublayer(norm_a(x)))

on an fp32 residual stream; the feed-forward is dense (xIELU) or a mixture
of experts picked by the token id; a span of layers may run several times in
a row with the same weights (each pass with its own cache pages and state);
the logits are soft-capped with tanh.

Everything a checkpoint's config.json states (sizes, layer order, the looped
span, constants) is read from it. Cache pages and state slots are per layer
RUN: a layer inside the looped span owns one set per pass.

Tensor parallelism is not implemented for this family (tp_size must be 1).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kukeon_amd import ops
from kukeon_amd import parallel
from kukeon_amd.models.feedforward import FFCfg, TableMoE, XieluFF
from kukeon_amd.models.mixers import (LatentAttention, LatentAttnCfg,
                                      StateSpaceCfg, StateSpaceMixer)
from kukeon_amd.models.rotary import angle_table

_DTYPES = {"bf16": torch.bfloat16, "bfloat16": torch.bfloat16,
           "fp32": torch.float32, "float32": torch.float32}

MIXERS = {"mamba2": StateSpaceMixer, "latent_attention": LatentAttention}
FEED_FORWARDS = {"dense": XieluFF, "moe": TableMoE}


@dataclass
class RasesunLayerCfg:
    type: str
    mixer: object
    mlp: Optional[FFCfg]


@dataclass
class RasesunConfig:
    family = "rasesun"
    name: str = "rasesun"
    width: int = 1024
    vocab_size: int = 32000
    embed_scale: float = 1.0
    rms_eps: float = 1e-6
    logit_softcap: float = 0.0
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    layers: List[RasesunLayerCfg] = field(default_factory=list)

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return False

    def runs(self) -> List[int]:
        """Layer indices in running order."""
        n = len(self.layers)
        a, b, k = self.loop_start, self.loop_stop, self.loop_times
        if k <= 1 or b <= a:
            return list(range(n))
        return list(range(a)) + list(range(a, b)) * k + list(range(b, n))

    @staticmethod
    def from_json(c: dict, name: str = "rasesun") -> "RasesunConfig":
        layers = []
        for i, L in enumerate(c["layers"]):
            kind = L.get("type")
            m = L["mixer"]
            if kind == "mamba2":
                mix = StateSpaceCfg(
                    heads=int(m["heads"]), vdim=int(m["vdim"]),
                    state=int(m["state"]), groups=int(m.get("groups", 1)),
                    conv=int(m["conv"]),
                    norm_groups=int(m.get("norm_groups", 1)))
            elif kind == "latent_attention":
                r = m["rot"]
                mix = LatentAttnCfg(
                    heads=int(m["heads"]), dim=int(m["dim"]),
                    rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                    q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]),
                    scale=float(m["scale"]),
                    window=int((m.get("mask") or {}).get("size", 0)),
                    rot_dims=int(r["dims"]), rot_base=float(r["base"]))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp = None
            if L.get("mlp"):
                f = L["mlp"]
                fk = f.get("kind", "dense")
                if fk == "dense":
                    mlp = FFCfg("dense", int(f["ff"]))
                elif fk == "moe":
                    mlp = FFCfg("moe", int(f["expert"]["ff"]),
                                experts=int(f["router"]["experts"]),
                                top=int(f["router"]["top"]))
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind "
                                     f"{fk!r}")
            layers.append(RasesunLayerCfg(kind, mix, mlp))
        lp = c.get("loop") or {}
        n = len(layers)
        a, b = int(lp.get("start", 0)), int(lp.get("stop", 0))
        if lp and not (0 <= a <= b <= n):
            raise ValueError("loop span outside the layer list")
        return RasesunConfig(
            name=name, width=int(c["width"]), vocab_size=int(c["vocab"]),
            embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
            rms_eps=float(c["norm"]["eps"]),
            logit_softcap=float(c.get("logit_softcap") or 0.0),
            loop_start=a, loop_stop=b, loop_times=int(lp.get("times", 1)),
            layers=layers)


def rasesun_bench(width=4096, layers=8, heads=32, ff=14336, vocab=128256,
                  attn_every=4, window=1024, experts=16, top=2,
                  name="rasesun-8b-like") -> RasesunConfig:
    """A layer stack at real-model sizes (random weights) for throughput
    runs: every `attn_every`-th layer is latent attention (heads of 128
    unrotated + 64 rotated entries, a 512-wide latent), the others are
    state-space layers of twice the width (64-channel heads, 128 state
    rows, 8 groups); feed-forwards alternate between dense and
    table-routed experts of the same total active size."""
    ls = []
    for i in range(layers):
        if i % attn_every == attn_every - 1:
            kind = "latent_attention"
            mix = LatentAttnCfg(heads=heads, dim=128, rot_dim=64, vdim=128,
                                q_rank=max(64, width * 3 // 8), kv_rank=512,
                                scale=192 ** -0.5, window=window,
                                rot_dims=64, rot_base=10000.0)
        else:
            kind = "mamba2"
            ssm_heads = max(1, 2 * width // 64)
            parts = 8 if ssm_heads % 8 == 0 else 1
            mix = StateSpaceCfg(heads=ssm_heads, vdim=64, state=128,
                                groups=parts, conv=4, norm_groups=parts)
        if i % 2:
            mlp = FFCfg("moe", max(8, ff // top // 8 * 8), experts=experts,
                        top=top)
        else:
            mlp = FFCfg("dense", ff)
        ls.append(RasesunLayerCfg(kind, mix, mlp))
    return RasesunConfig(name=name, width=width, vocab_size=vocab,
                         embed_scale=1.0, rms_eps=1e-6, logit_softcap=30.0,
                         layers=ls)


def tensor_shapes(cfg: RasesunConfig) -> Dict[str, tuple]:
    """Names and shapes of a checkpoint of this configuration."""
    W = cfg.width
    out = {"embed": (cfg.vocab_size, W)}
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        out[p + "norm1"] = (W,)
        out[p + "norm1b"] = (W,)
        for n, s in MIXERS[L.type].tensor_shapes(L.mixer, W).items():
            out[p + "mix." + n] = s
        if L.mlp is not None:
            out[p + "norm2"] = (W,)
            out[p + "norm2b"] = (W,)
            shapes = FEED_FORWARDS[L.mlp.kind].tensor_shapes(
                L.mlp, W, cfg.vocab_size)
            for n, s in shapes.items():
                out[p + "mlp." + n] = s
    out["final.norm"] = (W,)
    out["head"] = (cfg.vocab_size, W)
    return out


def random_tensors(cfg: RasesunConfig, seed: int = 0,
                   device="cpu") -> Dict[str, torch.Tensor]:
    """Random bf16 weights at a scale that keeps activations O(1)."""
    on_gpu = torch.device(device).type == "cuda"
    gdev = device if on_gpu else "cpu"
    g = torch.Generator(device=gdev).manual_seed(seed)
    out = {}
    for name, shp in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf == "table":
            i = int(name.split(".")[0][1:])
            E = cfg.layers[i].mlp.experts
            r = torch.rand(shp[0], E, generator=g, device=gdev)
            out[name] = r.argsort(1)[:, :shp[1]].to(torch.int32).to(device)
            continue
        if name.endswith("mix.conv"):
            t = torch.randn(shp, generator=g, device=gdev) * 0.4
        elif len(shp) == 2:
            std = shp[1] ** -0.5 if name != "embed" else 1.0
            t = torch.randn(shp, generator=g, device=gdev) * std
        elif leaf == "A_log":
            t = torch.rand(shp, generator=g, device=gdev) * 2.0 - 1.5
        elif leaf == "dt_bias":
            t = torch.rand(shp, generator=g, device=gdev) * 2.0 - 2.5
        elif leaf in ("norm", "norm1", "norm2", "norm1b", "norm2b", "D"):
            t = 1.0 + torch.randn(shp, generator=g, device=gdev) * 0.1
            if leaf in ("norm1b", "norm2b"):
                t = t * 0.5
        else:
            t = torch.randn(shp, generator=g, device=gdev) * 0.1
        out[name] = t.to(torch.bfloat16).to(device)
    return out


class RasesunLayer(nn.Module):
    def __init__(self, cfg: RasesunConfig, idx: int,
                 t: Dict[str, torch.Tensor], device, dtype):
        super().__init__()
        L = cfg.layers[idx]
        p = f"l{idx}."
        W = cfg.width
        self.idx = idx
        f32 = dict(device=device, dtype=torch.float32)
        self.norm1 = t[p + "norm1"].to(**f32).contiguous()
        self.norm1b = t[p + "norm1b"].to(**f32).contiguous()
        self.mixer = MIXERS[L.type](L.mixer, W, cfg.rms_eps, t, p + "mix.",
                                    device, dtype)
        self.ff = None
        if L.mlp is not None:
            self.norm2 = t[p + "norm2"].to(**f32).contiguous()
            self.norm2b = t[p + "norm2b"].to(**f32).contiguous()
            self.ff = FEED_FORWARDS[L.mlp.kind](L.mlp, W, t, p + "mlp.",
                                                device, dtype)


class RasesunModel(nn.Module):
    family = "rasesun"
    op_groups = ("recur",)      # kernel groups the forward pass needs

    def __init__(self, cfg: RasesunConfig, device="cuda", dtype="bf16",
                 tensors: Optional[Dict[str, torch.Tensor]] = None,
                 max_position: int = 4096, seed: int = 0):
        super().__init__()
        if parallel.tp_size() != 1:
            raise NotImplementedError("Rasesun runs with tp_size == 1 only")
        self.cfg = cfg
        self.device_ = torch.device(device)
        self.dtype = _DTYPES[dtype] if isinstance(dtype, str) else dtype
        if tensors is None:
            tensors = random_tensors(cfg, seed, device=self.device_)
        for name, shp in tensor_shapes(cfg).items():
            if name not in tensors:
                raise KeyError(f"checkpoint lacks tensor {name}")
            if tuple(tensors[name].shape) != tuple(shp):
                raise ValueError(f"{name}: shape {tuple(tensors[name].shape)}"
                                 f", configuration says {tuple(shp)}")
        dev, dt = self.device_, self.dtype
        self.embed = nn.Parameter(tensors["embed"].to(dev).to(dt),
                                  requires_grad=False)
        self.layers = nn.ModuleList(
            [RasesunLayer(cfg, i, tensors, dev, dt)
             for i in range(cfg.num_layers)])
        self.runs = cfg.runs()
        self.final_norm = tensors["final.norm"].to(dev).float().contiguous()
        self.lm_head = nn.Parameter(tensors["head"].to(dev).to(dt),
                                    requires_grad=False)
        self.set_max_position(max_position)

    @classmethod
    def from_checkpoint(cls, model_dir: str, device="cuda", dtype="bf16",
                        max_position: int = 4096):
        from kukeon_amd.models.weights import read_checkpoint
        config, tensors = read_checkpoint(model_dir)
        cfg = RasesunConfig.from_json(config)
        return cfg, cls(cfg, device=device, dtype=dtype, tensors=tensors,
                        max_position=max_position)

    def set_max_position(self, n: int) -> None:
        """(Re)build the angle tables for positions 0 .. n-1."""
        self.max_position = n
        tables: Dict[tuple, torch.Tensor] = {}
        for L in self.layers:
            mx = L.mixer
            if isinstance(mx, LatentAttention):
                key = (mx.m.rot_dims, mx.m.rot_base)
                if key not in tables:
                    tables[key] = angle_table(n, key[0], key[1]).to(
                        self.device_)
                mx.cs = tables[key]

    # ---- what the engine asks of a model with its own cache layout ----
    def kv_specs(self):
        return [self.layers[i].mixer.kv_spec() for i in self.runs]

    def state_shapes(self):
        return [self.layers[i].mixer.state_shape() for i in self.runs]

    def activation_dtype(self) -> torch.dtype:
        return self.dtype

    # ---- forward ----
    def forward(self, input_ids: torch.Tensor, kv_k, kv_v, meta,
                taps: Optional[list] = None) -> torch.Tensor:
        """-> final-normed hidden [T, W]. `taps`, if a list, receives the
        fp32 residual stream after every layer run."""
        cfg = self.cfg
        eps = cfg.rms_eps
        x = F.embedding(input_ids.long(), self.embed).float()
        if cfg.embed_scale != 1.0:
            x = x * cfg.embed_scale
        x = x.contiguous()
        h = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        ops.norm_only(x, self.layers[self.runs[0]].norm1, eps, h)
        n = len(self.runs)
        for r, li in enumerate(self.runs):
            layer = self.layers[li]
            nxt = (self.layers[self.runs[r + 1]].norm1 if r + 1 < n
                   else self.final_norm)
            st = meta.state[r] if meta.state is not None else None
            y = layer.mixer(h, kv_k[r], st, meta)
            h = torch.empty_like(h)
            if layer.ff is not None:
                ops.postnorm_residual_rmsnorm(x, y, layer.norm1b,
                                              layer.norm2, eps, h)
                y = layer.ff(h, input_ids, meta)
                h = torch.empty_like(h)
                ops.postnorm_residual_rmsnorm(x, y, layer.norm2b, nxt, eps, h)
            else:
                ops.postnorm_residual_rmsnorm(x, y, layer.norm1b, nxt, eps, h)
            if taps is not None:
                taps.append(x.clone())
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = ops.linear(hidden, self.lm_head).float()
        if self.cfg.logit_softcap > 0:
            ops.softcap_(logits, self.cfg.logit_softcap)
        return logits
