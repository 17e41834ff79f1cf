"""Slow, plain model of the Lipedra design for the tests: one function per
mechanism, float64 on the CPU, whole sequences at once, no cache. It shares
no code with kukeon_amd; it reads the same config dictionary and tensor
names a checkpoint has."""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def zero_centred_norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def causal_short_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t-taps+1+j)."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros(T, C, dtype=u.dtype)
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                y[t] += w[:, j] * u[src]
    return y


def rotary_angles(rot, T):
    """-> (cos, sin) [T, dims/2] with the YaRN blend when `scaling` is set."""
    dims, base = rot["dims"], rot["base"]
    freqs = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    gain = 1.0
    sc = rot.get("scaling")
    if sc:
        def where(turns):
            return dims * math.log(sc["original"] / (2 * math.pi * turns)) \
                / (2 * math.log(base))
        lo = max(math.floor(where(sc["fast"])), 0)
        hi = min(math.ceil(where(sc["slow"])), dims - 1)
        out = []
        for i, f in enumerate(freqs):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(f / sc["factor"] * ramp + f * (1.0 - ramp))
        freqs = out
        gain = 0.1 * math.log(sc["factor"]) + 1.0
    cos = torch.zeros(T, dims // 2, dtype=F64)
    sin = torch.zeros(T, dims // 2, dtype=F64)
    for p in range(T):
        for i, f in enumerate(freqs):
            cos[p, i] = math.cos(p * f) * gain
            sin[p, i] = math.sin(p * f) * gain
    return cos, sin


def rotate_interleaved(x, cos, sin, dims):
    """x [T, n, dim]: pairs (2i, 2i+1) of the first `dims` entries."""
    y = x.clone()
    for i in range(dims // 2):
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        c, s = cos[:, i][:, None], sin[:, i][:, None]
        y[..., 2 * i] = a * c - b * s
        y[..., 2 * i + 1] = b * c + a * s
    return y


def diff_lambda(W, p, diff):
    return math.exp(float((W[p + "mix.lq1"] * W[p + "mix.lk1"]).sum())) - \
        math.exp(float((W[p + "mix.lq2"] * W[p + "mix.lk2"]).sum())) + diff


def softmax_attention(q, k, v, scale):
    """q, k [T, d], v [T, e]; causal."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for i in range(T):
        s = (k[: i + 1] @ q[i]) * scale
        w = torch.softmax(s, 0)
        out[i] = w @ v[: i + 1]
    return out


def diff_attention(q, k, v, H, G, scale, lam, diff, eps, gate):
    """q [T, H, 2, d], k [T, G, 2, d], v [T, G, e], gate [T, H] (logits)
    -> [T, H*e]."""
    T = q.shape[0]
    outs = []
    for h in range(H):
        g = h // (H // G)
        a1 = softmax_attention(q[:, h, 0], k[:, g, 0], v[:, g], scale)
        a2 = softmax_attention(q[:, h, 1], k[:, g, 1], v[:, g], scale)
        o = unit_rms(a1 - lam * a2, eps) * (1.0 - diff)
        outs.append(o * torch.sigmoid(gate[:, h])[:, None])
    return torch.cat(outs, -1)


def clamped_glu(g, u, limit):
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, -limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def mixer_qkv(W, p, m, h):
    """Projected, convolved and rotated q (and k, v if the layer has them)."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    cos, sin = rotary_angles(m["rot"], T)
    rd = m["rot"]["dims"]

    def proj(n):
        u = h @ W[p + "mix." + n].T + W[p + "mix." + n + ".b"]
        if not m.get("conv"):
            return u
        return causal_short_conv(u, W[p + "mix." + n + ".conv"])

    q = rotate_interleaved(proj("q").view(T, 2 * H, d), cos, sin, rd)
    q = q.view(T, H, 2, d)
    if m.get("kv_from") is not None:
        return q, None, None
    k = rotate_interleaved(proj("k").view(T, 2 * G, d), cos, sin, rd)
    return q, k.view(T, G, 2, d), proj("v").view(T, G, e)


def forward(config, tensors, tokens, residuals=None):
    """-> logits [T, vocab] (float64). `residuals`, if a list, gets the
    residual stream after every layer."""
    W = {k: v.to(F64) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * \
        config.get("embedding", {}).get("scale", 1.0)
    held = {}
    for i, L in enumerate(config["layers"]):
        p = "l%d." % i
        m = L["mixer"]
        h = zero_centred_norm(x, W[p + "norm1"], eps)
        q, k, v = mixer_qkv(W, p, m, h)
        if k is None:
            k, v = held[m["kv_from"]]
        else:
            held[i] = (k, v)
        a = diff_attention(q, k, v, m["heads"], m["kv_heads"], m["scale"],
                           diff_lambda(W, p, m["diff"]), m["diff"], eps,
                           h @ W[p + "mix.g"].T)
        y = a @ W[p + "mix.o"].T
        if L.get("mlp"):
            g = h @ W[p + "mlp.gate"].T + W[p + "mlp.gate.b"]
            u = h @ W[p + "mlp.up"].T + W[p + "mlp.up.b"]
            y = y + clamped_glu(g, u, L["mlp"]["limit"]) @ \
                W[p + "mlp.down"].T + W[p + "mlp.down.b"]
        x = x + y
        if residuals is not None:
            residuals.append(x.clone())
    x = zero_centred_norm(x, W["final.norm"], eps)
    return x @ W["head"].T


def greedy(config, tensors, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(config, tensors, toks)[-1].argmax()))
    return toks[len(prompt):]
