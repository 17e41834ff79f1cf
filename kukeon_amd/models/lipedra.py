"""Lipedra: a decoder of parallel layers — one RMS norm feeds a
differential-attention mixer and a clamped gated feed-forward, and both
results join the fp32 residual stream in one sum.

Per layer the compute path is three GEMMs and five kernels:

  h      = rmsnorm(x) * (1 + w)                    (fused with the previous
                                                    layer's residual sum)
  proj   = h @ [Wq | Wk | Wv | Wgate_out]^T
  pff    = h @ [Wff_gate | Wff_up]^T
  q,k,v  = rotary(conv(proj + bias))  -> q buffer / paged cache
  attn   = diff_attention(q, cache)   -> cat[:, :H*vdim]
  ff     = clamp_glu(pff + bias)      -> cat[:, H*vdim:]
  x     += cat @ [Wo | Wdown]^T + b_down           (one GEMM for both
                                                    sublayers' outputs)

A layer whose mixer names `kv_from` projects no keys or values and reads
the cache pages of that earlier layer. Everything the checkpoint's
config.json states (sizes, layer order, constants) is read from it.

Tensor parallelism is not implemented for this family (tp_size must be 1).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kukeon_amd import ops
from kukeon_amd import parallel
from kukeon_amd.engine.kv_cache import LayerKVSpec
from kukeon_amd.models.rotary import angle_table

_DTYPES = {"bf16": torch.bfloat16, "bfloat16": torch.bfloat16,
           "fp32": torch.float32, "float32": torch.float32}


@dataclass
class RotaryCfg:
    dims: int
    base: float
    scaling: Optional[dict] = None

    def key(self):
        sc = self.scaling
        return (self.dims, self.base,
                None if not sc else tuple(sorted(sc.items())))


@dataclass
class DiffAttnCfg:
    heads: int
    kv_heads: int
    dim: int                 # size of one score map of a head
    vdim: int
    conv: int                # taps of the short convolution
    diff: float
    scale: float
    rot: RotaryCfg
    kv_from: Optional[int] = None
    has_conv: bool = True    # False: the checkpoint has no '.conv' tensors


@dataclass
class GluCfg:
    ff: int
    limit: float
    kind: str = "dense"


@dataclass
class LipedraLayerCfg:
    mixer: DiffAttnCfg
    mlp: Optional[GluCfg]


@dataclass
class LipedraConfig:
    family = "lipedra"
    name: str = "lipedra"
    width: int = 1024
    vocab_size: int = 32000
    embed_scale: float = 1.0
    rms_eps: float = 1e-5
    layers: List[LipedraLayerCfg] = field(default_factory=list)

    # names the engine reads on every family
    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return False

    @staticmethod
    def from_json(c: dict, name: str = "lipedra") -> "LipedraConfig":
        layers = []
        for i, L in enumerate(c["layers"]):
            if L.get("type") != "attention":
                raise ValueError(f"layer {i}: unknown mixer type "
                                 f"{L.get('type')!r}")
            m = L["mixer"]
            r = m["rot"]
            rot = RotaryCfg(int(r["dims"]), float(r["base"]),
                            dict(r["scaling"]) if r.get("scaling") else None)
            mix = DiffAttnCfg(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                dim=int(m["dim"]), vdim=int(m["vdim"]),
                conv=int(m.get("conv") or 1),
                has_conv=bool(m.get("conv")), diff=float(m["diff"]),
                scale=float(m["scale"]), rot=rot,
                kv_from=(int(m["kv_from"]) if m.get("kv_from") is not None
                         else None))
            mlp = None
            if L.get("mlp"):
                f = L["mlp"]
                if f.get("kind", "dense") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind "
                                     f"{f.get('kind')!r}")
                mlp = GluCfg(ff=int(f["ff"]), limit=float(f["limit"]))
            layers.append(LipedraLayerCfg(mix, mlp))
        return LipedraConfig(
            name=name, width=int(c["width"]), vocab_size=int(c["vocab"]),
            embed_scale=float(c.get("embedding", {}).get("scale", 1.0)),
            rms_eps=float(c["norm"]["eps"]), layers=layers)


def lipedra_bench(width=4096, layers=8, heads=32, kv_heads=8, dim=64,
                  vdim=128, ff=14336, vocab=128256, share_every=2,
                  name="lipedra-8b-like") -> LipedraConfig:
    """A layer stack at real-model sizes (random weights) for throughput
    runs: every `share_every`-th layer reads its predecessor's cache."""
    rot = RotaryCfg(dims=dim, base=500000.0,
                    scaling={"factor": 4.0, "original": 4096, "fast": 16.0,
                             "slow": 2.0})
    ls = []
    for i in range(layers):
        shared = share_every > 1 and i % share_every == share_every - 1
        ls.append(LipedraLayerCfg(
            DiffAttnCfg(heads, kv_heads, dim, vdim, conv=4, diff=0.2,
                        scale=dim ** -0.5, rot=rot,
                        kv_from=(i - 1 if shared else None)),
            GluCfg(ff=ff, limit=7.0)))
    return LipedraConfig(name=name, width=width, vocab_size=vocab,
                         embed_scale=1.0, rms_eps=1e-5, layers=ls)


def tensor_shapes(cfg: LipedraConfig) -> Dict[str, tuple]:
    """Names and shapes of a checkpoint of this configuration."""
    W = cfg.width
    out = {"embed": (cfg.vocab_size, W)}
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        m = L.mixer
        out[p + "norm1"] = (W,)
        segs = [("q", m.heads * 2 * m.dim)]
        if m.kv_from is None:
            segs += [("k", m.kv_heads * 2 * m.dim),
                     ("v", m.kv_heads * m.vdim)]
        for n, c in segs:
            out[p + f"mix.{n}"] = (c, W)
            out[p + f"mix.{n}.b"] = (c,)
            if m.has_conv:
                out[p + f"mix.{n}.conv"] = (c, m.conv)
        for n in ("lq1", "lk1", "lq2", "lk2"):
            out[p + "mix." + n] = (m.dim,)
        out[p + "mix.g"] = (m.heads, W)
        out[p + "mix.o"] = (W, m.heads * m.vdim)
        if L.mlp is not None:
            ff = L.mlp.ff
            out[p + "mlp.gate"] = (ff, W)
            out[p + "mlp.gate.b"] = (ff,)
            out[p + "mlp.up"] = (ff, W)
            out[p + "mlp.up.b"] = (ff,)
            out[p + "mlp.down"] = (W, ff)
            out[p + "mlp.down.b"] = (W,)
    out["final.norm"] = (W,)
    out["head"] = (cfg.vocab_size, W)
    return out


def random_tensors(cfg: LipedraConfig, seed: int = 0,
                   device="cpu") -> Dict[str, torch.Tensor]:
    """Random bf16 weights at a scale that keeps activations O(1)."""
    on_gpu = torch.device(device).type == "cuda"
    g = torch.Generator(device=device if on_gpu else "cpu").manual_seed(seed)
    gdev = device if on_gpu else "cpu"
    out = {}
    for name, shp in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if len(shp) == 2 and leaf != "conv":
            std = shp[1] ** -0.5 if name != "embed" else 1.0
        elif leaf == "conv":
            std = 0.5
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            std = 0.3
        else:
            std = 0.1
        t = torch.randn(shp, generator=g, device=gdev) * std
        out[name] = t.to(torch.bfloat16).to(device)
    return out


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


class LipedraLayer(nn.Module):
    """One parallel layer; holds the fused weights and the column map of
    the fused input projection."""

    def __init__(self, cfg: LipedraConfig, idx: int,
                 t: Dict[str, torch.Tensor], device, dtype):
        super().__init__()
        L = cfg.layers[idx]
        m = L.mixer
        self.idx = idx
        self.m = m
        self.mlp = L.mlp
        self.eps = cfg.rms_eps
        p = f"l{idx}."
        W = cfg.width
        if m.heads % m.kv_heads:
            raise ValueError(f"layer {idx}: heads not a multiple of kv_heads")
        if m.rot.dims % 2 or m.rot.dims > m.dim:
            raise ValueError(f"layer {idx}: bad rotary dims")
        self.owns_kv = m.kv_from is None
        self.kv_layer = idx if self.owns_kv else m.kv_from
        self.Cq = m.heads * 2 * m.dim
        self.Ck = m.kv_heads * 2 * m.dim if self.owns_kv else 0
        self.Cv = m.kv_heads * m.vdim if self.owns_kv else 0

        def w(name):
            return t[p + name].to(device=device)

        # two input projections off the one normed input: the mixer's
        # [q | k | v | gate] and the feed-forward's [gate | up]; every
        # segment starts on a multiple of 8 columns
        def fuse(segs):
            col, rows, at = {}, [], 0
            for name, wt in segs:
                col[name] = at
                n = wt.shape[0]
                rows.append(wt.to(dtype))
                pad = _pad8(n) - n
                if pad:
                    rows.append(torch.zeros(pad, W, dtype=dtype,
                                            device=device))
                at += _pad8(n)
            return col, nn.Parameter(torch.cat(rows, 0).contiguous(),
                                     requires_grad=False)

        segs = [("q", w("mix.q"))]
        if self.owns_kv:
            segs += [("k", w("mix.k")), ("v", w("mix.v"))]
        segs.append(("g", w("mix.g")))
        self.col, self.w_mix = fuse(segs)
        self.w_ff = None
        if self.mlp is not None:
            self.ffcol, self.w_ff = fuse([("ffg", w("mlp.gate")),
                                          ("ffu", w("mlp.up"))])
        # fused output projection over [attention | feed-forward]
        outs = [w("mix.o").to(dtype)]
        self.attn_cols = m.heads * m.vdim
        self.ff_cols = 0
        self.b_down = None
        if self.mlp is not None:
            outs.append(w("mlp.down").to(dtype))
            self.ff_cols = self.mlp.ff
            self.b_down = w("mlp.down.b").float().contiguous()
            self.b_ffg = w("mlp.gate.b").float().contiguous()
            self.b_ffu = w("mlp.up.b").float().contiguous()
        self.w_out = nn.Parameter(torch.cat(outs, 1).contiguous(),
                                  requires_grad=False)
        # convolution taps and projection biases, fp32, channels [q|k|v]
        names = ["q"] + (["k", "v"] if self.owns_kv else [])
        if m.has_conv:
            self.conv_w = torch.cat(
                [w(f"mix.{n}.conv").float() for n in names],
                0).t().contiguous()                          # [taps, C]
        else:                   # no convolution: a single tap of weight 1
            self.conv_w = torch.ones(1, self.Cq + self.Ck + self.Cv,
                                     dtype=torch.float32, device=device)
        self.conv_b = torch.cat([w(f"mix.{n}.b").float() for n in names],
                                0).contiguous()
        if self.conv_w.shape[0] != m.conv:
            raise ValueError(f"layer {idx}: convolution taps differ from "
                             "the configuration")
        self.norm_w = w("norm1").float().contiguous()
        # lambda = exp(lq1.lk1) - exp(lq2.lk2) + diff, one number per layer
        d = lambda a, b: float((t[p + a].double() * t[p + b].double()).sum())
        self.lam = math.exp(d("mix.lq1", "mix.lk1")) - \
            math.exp(d("mix.lq2", "mix.lk2")) + m.diff
        self.cs = None      # angle table, set by the model

    def kv_spec(self) -> LayerKVSpec:
        m = self.m
        return LayerKVSpec(m.kv_heads, 2 * m.dim, m.vdim,
                           share_from=None if self.owns_kv else m.kv_from)

    def state_shape(self):
        back = self.m.conv - 1
        return (back, self.Cq + self.Ck + self.Cv)

    def forward(self, h: torch.Tensor, kc, vc, state, meta) -> torch.Tensor:
        """h: normed input [T, W] -> [T, W] sum of mixer and feed-forward
        (without the down-projection bias, which joins in the residual
        kernel)."""
        m = self.m
        T = h.shape[0]
        proj = ops.linear(h, self.w_mix)
        q = torch.empty(T, self.Cq, dtype=h.dtype, device=h.device)
        c = self.col
        shifted = ops.conv_rope_append(
            q, kc if self.owns_kv else None, vc if self.owns_kv else None,
            proj, self.conv_b, self.conv_w, state, self.cs, meta.positions,
            meta.row_seq, meta.cu_rows, meta.state_slots, meta.block_table,
            c["q"], c.get("k", 0), c.get("v", 0), self.Cq, self.Ck, self.Cv,
            m.dim, m.rot.dims, one_row_per_seq=(meta.max_rows == 1))
        if not shifted:
            ops.conv_state_update(state, proj, self.conv_b, meta.positions,
                                  meta.cu_rows, meta.state_slots, c["q"],
                                  c.get("k", 0), c.get("v", 0), self.Cq,
                                  self.Ck, self.Cv)
        cat = torch.empty(T, self.attn_cols + self.ff_cols, dtype=h.dtype,
                          device=h.device)
        gate = proj[:, c["g"]: c["g"] + m.heads]
        self._attend(cat, q, kc, vc, gate, meta)
        if self.mlp is not None:
            ff = self.mlp.ff
            fc = self.ffcol
            pff = ops.linear(h, self.w_ff)
            ops.clamp_glu(cat[:, self.attn_cols:],
                          pff[:, fc["ffg"]: fc["ffg"] + ff],
                          pff[:, fc["ffu"]: fc["ffu"] + ff],
                          self.b_ffg, self.b_ffu, self.mlp.limit, 1.702, 1.0)
        return ops.linear(cat, self.w_out)


    # ---- attention dispatch: three kernels, one interface ----
    _ws: Dict[tuple, tuple] = {}

    def _attend(self, cat, q, kc, vc, gate, meta) -> None:
        m = self.m
        tail = (m.heads, m.scale, self.lam, self.eps, 1.0 - m.diff)
        rows = q.shape[0]
        if (meta.mode == "decode" and
                ops.diff_decode_supported(q, m.heads, m.kv_heads, m.dim,
                                          m.vdim)):
            # split the keys so that a small batch still fills the chip
            ns = ops.diff_decode_splits(q, rows, m.heads, m.kv_heads, m.dim)
            key = (q.device, rows, m.heads, ns, m.vdim)
            ws = LipedraLayer._ws.get(key)
            if ws is None:
                ws = (torch.zeros(rows, m.heads, 2, ns, m.vdim,
                                  dtype=torch.float32, device=q.device),
                      torch.zeros(rows, m.heads, 2, ns, 2,
                                  dtype=torch.float32, device=q.device))
                LipedraLayer._ws[key] = ws
            ops.diff_attention_decode(cat, q, kc, vc, gate, meta.positions,
                                      meta.row_seq, meta.block_table, ws[0],
                                      ws[1], *tail)
            return
        if (meta.mode == "prefill" and meta.max_rows >= 16 and
                meta.chunk_lens is not None and
                cat.stride(0) % 4 == 0 and      # 8-byte output stores
                ops.diff_tiles_supported(q, m.dim, m.vdim)):
            hpg = m.heads // m.kv_heads
            hpw = 4 if hpg % 4 == 0 else 2 if hpg % 2 == 0 else 1
            ts, tr = _tile_map(meta, 32 * (4 // hpw), q.device)
            ops.diff_attention_tiles(cat, q, kc, vc, gate, meta.positions,
                                     meta.cu_rows, meta.block_table, ts, tr,
                                     m.heads, hpw, *tail[1:])
            return
        ops.diff_attention(cat, q, kc, vc, gate, meta.positions, meta.row_seq,
                           meta.block_table, *tail)


def _tile_map(meta, rows_per_wg: int, device):
    """(sequence, first local row) of every workgroup of the tile kernel,
    built once per step and granularity from the portions' lengths."""
    cache = meta.tile_maps
    if rows_per_wg not in cache:
        seq, row0 = [], []
        for s, n in enumerate(meta.chunk_lens):
            for r in range(0, n, rows_per_wg):
                seq.append(s)
                row0.append(r)
        cache[rows_per_wg] = (
            torch.tensor(seq, dtype=torch.int32, device=device),
            torch.tensor(row0, dtype=torch.int32, device=device))
    return cache[rows_per_wg]


class LipedraModel(nn.Module):
    family = "lipedra"
    op_groups = ("mix",)        # kernel groups the forward pass needs

    def __init__(self, cfg: LipedraConfig, device="cuda", dtype="bf16",
                 tensors: Optional[Dict[str, torch.Tensor]] = None,
                 max_position: int = 4096, seed: int = 0):
        super().__init__()
        if parallel.tp_size() != 1:
            raise NotImplementedError("Lipedra runs with tp_size == 1 only")
        self.cfg = cfg
        self.device_ = torch.device(device)
        self.dtype = _DTYPES[dtype] if isinstance(dtype, str) else dtype
        if tensors is None:
            tensors = random_tensors(cfg, seed, device=self.device_)
        want = tensor_shapes(cfg)
        for name, shp in want.items():
            if name not in tensors:
                raise KeyError(f"checkpoint lacks tensor {name}")
            if tuple(tensors[name].shape) != tuple(shp):
                raise ValueError(f"{name}: shape {tuple(tensors[name].shape)}"
                                 f", configuration says {tuple(shp)}")
        dev, dt = self.device_, self.dtype
        self.embed = nn.Parameter(tensors["embed"].to(dev).to(dt),
                                  requires_grad=False)
        self.layers = nn.ModuleList(
            [LipedraLayer(cfg, i, tensors, dev, dt)
             for i in range(cfg.num_layers)])
        for i, L in enumerate(self.layers):
            if not L.owns_kv:
                j = L.m.kv_from
                if not (0 <= j < i) or not self.layers[j].owns_kv:
                    raise ValueError(f"layer {i}: kv_from must name an "
                                     "earlier layer with its own keys")
        self.final_norm = tensors["final.norm"].to(dev).float().contiguous()
        self.lm_head = nn.Parameter(tensors["head"].to(dev).to(dt),
                                    requires_grad=False)
        self._tables: Dict[tuple, torch.Tensor] = {}
        self.set_max_position(max_position)

    # ---- construction helpers ----
    @classmethod
    def from_checkpoint(cls, model_dir: str, device="cuda", dtype="bf16",
                        max_position: int = 4096):
        from kukeon_amd.models.weights import read_checkpoint
        config, tensors = read_checkpoint(model_dir)
        cfg = LipedraConfig.from_json(config)
        return cfg, cls(cfg, device=device, dtype=dtype, tensors=tensors,
                        max_position=max_position)

    def set_max_position(self, n: int) -> None:
        """(Re)build the angle tables for positions 0 .. n-1."""
        self.max_position = n
        self._tables = {}
        for L in self.layers:
            r = L.m.rot
            if r.key() not in self._tables:
                self._tables[r.key()] = angle_table(
                    n, r.dims, r.base, r.scaling).to(self.device_)
            L.cs = self._tables[r.key()]

    # ---- what the engine asks of a model with its own cache layout ----
    def kv_specs(self) -> List[LayerKVSpec]:
        return [L.kv_spec() for L in self.layers]

    def state_shapes(self):
        return [L.state_shape() for L in self.layers]

    def activation_dtype(self) -> torch.dtype:
        return self.dtype

    # ---- forward ----
    def forward(self, input_ids: torch.Tensor, kv_k, kv_v, meta,
                taps: Optional[list] = None) -> torch.Tensor:
        """-> final-normed hidden [T, W]. `taps`, if a list, receives the
        fp32 residual stream after every layer (debugging, tests)."""
        cfg = self.cfg
        x = F.embedding(input_ids.long(), self.embed).float()
        if cfg.embed_scale != 1.0:
            x = x * cfg.embed_scale
        x = x.contiguous()
        h = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        n = len(self.layers)
        ops.residual_add_rmsnorm(x, None, None, self.layers[0].norm_w, 1.0,
                                 cfg.rms_eps, h)
        for i, layer in enumerate(self.layers):
            y = layer(h, kv_k[layer.kv_layer], kv_v[layer.kv_layer],
                      meta.state[i], meta)
            nw = self.layers[i + 1].norm_w if i + 1 < n else self.final_norm
            h = torch.empty_like(h)
            ops.residual_add_rmsnorm(x, y, layer.b_down, nw, 1.0,
                                     cfg.rms_eps, h)
            if taps is not None:
                taps.append(x.clone())
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear(hidden, self.lm_head)
