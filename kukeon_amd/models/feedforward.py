"""Feed-forward sublayers that are not gated linear units: a dense layer
with the xIELU activation, and a mixture of small experts chosen by a
per-token-id table (no learned router at run time)."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict

import torch
import torch.nn as nn

from kukeon_amd import ops


@dataclass
class FFCfg:
    kind: str                # "dense" | "moe"
    ff: int                  # hidden size (of one expert for "moe")
    experts: int = 0
    top: int = 0


def _softplus(x: float) -> float:
    return x if x > 30 else math.log1p(math.exp(x))


class XieluFF(nn.Module):
    """down(act(up h)) with act(z) = softplus(p) z^2 + z/2 for z > 0 and
    (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2 otherwise; (p, q) is the
    two-entry tensor `act`."""

    def __init__(self, f: FFCfg, width: int, t: Dict[str, torch.Tensor],
                 p: str, device, dtype):
        super().__init__()
        dev = dict(device=device, dtype=dtype)
        self.w_up = nn.Parameter(t[p + "up"].to(**dev).contiguous(),
                                 requires_grad=False)
        self.w_down = nn.Parameter(t[p + "down"].to(**dev).contiguous(),
                                   requires_grad=False)
        pq = t[p + "act"].double()
        self.ap = _softplus(float(pq[0]))
        self.aq = 0.5 + _softplus(float(pq[1]))

    @staticmethod
    def tensor_shapes(f: FFCfg, width: int, vocab: int) -> Dict[str, tuple]:
        return {"up": (f.ff, width), "down": (width, f.ff), "act": (2,)}

    def forward(self, h: torch.Tensor, ids: torch.Tensor,
                meta=None) -> torch.Tensor:
        z = ops.linear(h, self.w_up)
        a = torch.empty_like(z)
        ops.xielu(a, z, self.ap, self.aq)
        return ops.linear(a, self.w_down)


class TableMoE(nn.Module):
    """`experts` small feed-forward layers down(relu(up h)^2) without
    biases; token id v uses the `top` experts table[v] with weight 1/top
    each. The expert weights are stacked [E, ff, W] and [E, W, ff]."""

    def __init__(self, f: FFCfg, width: int, t: Dict[str, torch.Tensor],
                 p: str, device, dtype):
        super().__init__()
        dev = dict(device=device, dtype=dtype)
        self.f = f
        self.w_up = nn.Parameter(torch.stack(
            [t[p + f"e{e}.up"] for e in range(f.experts)]).to(**dev)
            .contiguous(), requires_grad=False)
        self.w_down = nn.Parameter(torch.stack(
            [t[p + f"e{e}.down"] for e in range(f.experts)]).to(**dev)
            .contiguous(), requires_grad=False)
        table = t[p + "table"].to(torch.int32)
        if table.dim() != 2 or table.shape[1] != f.top:
            raise ValueError(f"{p}table: shape {tuple(table.shape)}")
        if int(table.min()) < 0 or int(table.max()) >= f.experts:
            raise ValueError(f"{p}table names an expert that does not exist")
        self.table = table.to(device).contiguous()
        self.table_host = table.cpu().numpy()

    @staticmethod
    def tensor_shapes(f: FFCfg, width: int, vocab: int) -> Dict[str, tuple]:
        out = {"table": (vocab, f.top)}
        for e in range(f.experts):
            out[f"e{e}.up"] = (f.ff, width)
            out[f"e{e}.down"] = (width, f.ff)
        return out

    # portions of at least this many rows take the grouped form when the
    # step's token ids are known on the host
    grouped_min_rows = 64

    def forward(self, h: torch.Tensor, ids: torch.Tensor,
                meta=None) -> torch.Tensor:
        out = torch.empty_like(h)
        host_ids = getattr(meta, "host_ids", None)
        if host_ids is not None and h.shape[0] >= self.grouped_min_rows:
            return self._forward_grouped(out, h, host_ids, meta)
        ops.table_moe(out, h, ids, self.table, self.w_up, self.w_down)
        return out

    def _forward_grouped(self, out, h, host_ids, meta) -> torch.Tensor:
        """Rows sorted by expert on the host (the routing is a function of
        the token id, which the scheduler knows): no device round trip to
        learn the group sizes, and every expert runs plain GEMMs over its
        contiguous rows."""
        import numpy as np
        T, W = h.shape
        top, E = self.f.top, self.f.experts
        key = ("table_moe", id(self))
        maps = meta.tile_maps.get(key)
        if maps is None:
            flat = self.table_host[np.asarray(host_ids)].reshape(-1)
            order = np.argsort(flat, kind="stable")
            counts = np.bincount(flat, minlength=E)
            inv = np.empty_like(order)
            inv[order] = np.arange(order.size)
            dev = h.device
            maps = (torch.from_numpy((order // top).astype(np.int32)).to(dev),
                    torch.from_numpy(inv.astype(np.int32).reshape(T, top))
                    .to(dev), counts.tolist())
            meta.tile_maps[key] = maps
        row_map, inv, counts = maps
        rows = torch.empty(T * top, W, dtype=h.dtype, device=h.device)
        ops.gather_rows(rows, h, row_map)
        done = torch.empty_like(rows)
        at = 0
        for e in range(E):
            n = counts[e]
            if n == 0:
                continue
            a = ops.linear(rows[at: at + n], self.w_up[e])
            ops.relu_square_(a)
            done[at: at + n] = ops.linear(a, self.w_down[e])
            at += n
        ops.combine_rows(out, done, inv)
        return out
