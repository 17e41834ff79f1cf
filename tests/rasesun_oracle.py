"""A plain float64 Rasesun: one function per mechanism, whole sequences at a
time, no cache, no batching, no kernels. It shares no code with the package
and is what the package's results are compared with.

A model is (cfg, tensors): `cfg` is the dict of a config.json and `tensors`
maps names to torch tensors of any float type (integer tables as int)."""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def d(t):
    return t.to(F64)


# ---- small pieces ----------------------------------------------------------
def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * d(w)


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def xielu(z, p, q):
    """Piecewise activation: quadratic on the positive side, an exponential
    tail on the negative side, both meeting z / 2 at zero."""
    ap = float(softplus(torch.tensor(float(p), dtype=F64)))
    aq = 0.5 + float(softplus(torch.tensor(float(q), dtype=F64)))
    pos = ap * z * z + 0.5 * z
    neg = aq * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def rotate_pairs(v, pos, dims, base):
    """Rotate the first `dims` entries of the last axis, entry 2i with 2i+1,
    by the angle pos * base^(-2i/dims). v: [T, ..., n], pos: [T]."""
    out = v.clone()
    n = dims // 2
    i = torch.arange(n, dtype=F64)
    f = torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * i / dims)
    ang = d(pos)[:, None] * f[None, :]                    # [T, n]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [n]
    c, s = ang.cos().view(shape), ang.sin().view(shape)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ---- mixers ------------------------------------------------------------------
def causal_conv(u, w, b):
    """u [T, C]; w [C, taps] with the newest tap last; zeros before t = 0."""
    T, C = u.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), u], 0)
    out = torch.zeros(T, C, dtype=F64)
    for j in range(taps):
        out += pad[j: j + T] * d(w)[:, j][None, :]
    return out + d(b)[None, :]


def mamba2_mixer(h, m, t, p, eps):
    """Selective state-space mixer, token by token. h [T, W]."""
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    T = h.shape[0]
    proj = h @ d(t[p + "in"]).T
    z = proj[:, :inner]
    xbc = proj[:, inner: 2 * inner + 2 * G * N]
    dt = proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, t[p + "conv"], t[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner: inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + d(t[p + "dt_bias"])[None, :])          # [T, H]
    rate = torch.exp(d(t[p + "A_log"]))                        # [H]
    skip = d(t[p + "D"])
    y = torch.zeros(T, H, P, dtype=F64)
    per = H // G
    for hd in range(H):
        g = hd // per
        S = torch.zeros(N, P, dtype=F64)
        for i in range(T):
            S = math.exp(-float(rate[hd]) * float(dt[i, hd])) * S + \
                float(dt[i, hd]) * torch.outer(B[i, g], x[i, hd])
            y[i, hd] = S.T @ C[i, g] + skip[hd] * x[i, hd]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_unit(y.reshape(T, parts, inner // parts), eps).reshape(T, inner)
    return (y * d(t[p + "norm"])[None, :]) @ d(t[p + "o"]).T


def latent_attention_mixer(h, m, t, p, eps):
    """Attention whose keys and values are expanded from a shared low-rank
    latent, with a sliding causal window and a per-head output gate."""
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    R = m["kv_rank"]
    T = h.shape[0]
    pos = torch.arange(T)
    cq = rms_norm(h @ d(t[p + "dq"]).T, t[p + "dq.norm"], eps)
    q = (cq @ d(t[p + "uq"]).T).reshape(T, H, dn + dr)
    q_n, q_r = q[..., :dn], q[..., dn:]
    kv = h @ d(t[p + "dkv"]).T
    c = rms_norm(kv[:, :R], t[p + "dkv.norm"], eps)
    k_r = kv[:, R:]                                            # [T, dr]
    rot = m["rot"]
    q_r = rotate_pairs(q_r, pos, rot["dims"], rot["base"])
    k_r = rotate_pairs(k_r, pos, rot["dims"], rot["base"])
    k_n = (c @ d(t[p + "uk"]).T).reshape(T, H, dn)
    v = (c @ d(t[p + "uv"]).T).reshape(T, H, dv)
    s = torch.einsum("ihd,jhd->hij", q_n, k_n) + \
        torch.einsum("ihd,jd->hij", q_r, k_r)
    s = s * m["scale"]
    i = pos[:, None]
    j = pos[None, :]
    seen = (j <= i) & (i - j < m["mask"]["size"])
    s = s.masked_fill(~seen[None], float("-inf"))
    w = torch.softmax(s, -1)
    o = torch.einsum("hij,jhd->ihd", w, v)
    gate = torch.sigmoid(h @ d(t[p + "g"]).T)                  # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ d(t[p + "o"]).T


# ---- feed-forward ---------------------------------------------------------------
def dense_ff(h, t, p):
    pq = d(t[p + "act"])
    a = xielu(h @ d(t[p + "up"]).T, pq[0], pq[1])
    return a @ d(t[p + "down"]).T


def table_moe(h, ids, f, t, p):
    """Experts picked by the token id from a table, all with equal weight."""
    top = f["router"]["top"]
    table = t[p + "table"].long()
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e in table[int(ids[i])].tolist():
            a = torch.relu(d(t[p + f"e{e}.up"]) @ h[i]) ** 2
            out[i] += (d(t[p + f"e{e}.down"]) @ a) / top
    return out


# ---- the model ------------------------------------------------------------------
def layer_runs(cfg):
    """Layer indices in running order: the looped span repeated in place."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, k = lp["start"], lp["stop"], lp["times"]
    return list(range(a)) + list(range(a, b)) * k + list(range(b, n))


def forward(cfg, t, ids, taps=None):
    """ids: list of token ids -> logits [T, vocab] (float64). `taps`, if a
    list, receives the residual stream after every layer run."""
    eps = cfg["norm"]["eps"]
    ids = list(ids)
    x = d(t["embed"])[torch.tensor(ids)] * \
        (cfg.get("embedding") or {}).get("scale", 1.0)
    for li in layer_runs(cfg):
        L = cfg["layers"][li]
        p = f"l{li}."
        h = rms_norm(x, t[p + "norm1"], eps)
        if L["type"] == "mamba2":
            y = mamba2_mixer(h, L["mixer"], t, p + "mix.", eps)
        elif L["type"] == "latent_attention":
            y = latent_attention_mixer(h, L["mixer"], t, p + "mix.", eps)
        else:
            raise ValueError(L["type"])
        x = x + rms_norm(y, t[p + "norm1b"], eps)
        f = L.get("mlp")
        if f:
            h = rms_norm(x, t[p + "norm2"], eps)
            if f["kind"] == "dense":
                y = dense_ff(h, t, p + "mlp.")
            elif f["kind"] == "moe":
                y = table_moe(h, ids, f, t, p + "mlp.")
            else:
                raise ValueError(f["kind"])
            x = x + rms_norm(y, t[p + "norm2b"], eps)
        if taps is not None:
            taps.append(x.clone())
    h = rms_norm(x, t["final.norm"], eps)
    logits = h @ d(t["head"]).T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits


def greedy(cfg, t, prompt, n):
    """n greedy tokens after the prompt, by recomputing the whole sequence."""
    toks = list(prompt)
    out = []
    for _ in range(n):
        nxt = int(torch.argmax(forward(cfg, t, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out


def windowed_latent_rows(q_lat, q_rot, lat, k_rot, window, scale):
    """Attention of H heads over rows shared by all heads, by position:
    q_lat [T, H, R], q_rot [T, H, dr] (already rotated), lat [T, R],
    k_rot [T, dr] (already rotated) -> [T, H, R]: for position i the
    softmax over j in (i - window, i] of (q_lat.lat + q_rot.k_rot) * scale
    times lat."""
    T = lat.shape[0]
    out = torch.zeros_like(q_lat)
    for i in range(T):
        lo = max(0, i - window + 1) if window > 0 else 0
        s = (q_lat[i] @ lat[lo: i + 1].T + q_rot[i] @ k_rot[lo: i + 1].T)
        w = torch.softmax(s * scale, -1)
        out[i] = w @ lat[lo: i + 1]
    return out


def selective_scan(x, B, C, dt_raw, dt_bias, a_log, skip):
    """x [T, H, P], B, C [T, H, N] (already spread over heads), dt_raw
    [T, H] -> y [T, H, P] and the final state [H, N, P]."""
    T, H, P = x.shape
    N = B.shape[2]
    S = torch.zeros(H, N, P, dtype=F64)
    y = torch.zeros(T, H, P, dtype=F64)
    for i in range(T):
        step = softplus(dt_raw[i] + dt_bias)
        decay = torch.exp(-torch.exp(a_log) * step)
        S = decay[:, None, None] * S + \
            step[:, None, None] * B[i][:, :, None] * x[i][:, None, :]
        y[i] = (S * C[i][:, :, None]).sum(1) + skip[:, None] * x[i]
    return y, S
