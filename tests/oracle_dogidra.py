"""Plain float64 oracle of the Dogidra design: one function per mechanism,
whole sequences, no cache, no state carried between calls, no code shared
with the engine. `cfg` is the checkpoint's config.json as a dict, `W` maps
checkpoint tensor names to tensors.

Notation: T tokens, H query heads, G key/value heads, D key width, DV value
width, P tokens per pooled block, K convolution taps.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def _w(W, name):
    return W[name].to(F64)


def lin(W, name, x, bias=False):
    y = x @ _w(W, name).t()
    if bias:
        y = y + _w(W, name + ".b")
    return y


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = (x - mu).pow(2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w.to(F64) + b.to(F64)


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def input_conv(h, w):
    """h [T, C] -> h + conv(h); w [C, K], the last column weighs the current
    token, zeros before the start."""
    T, C = h.shape
    K = w.shape[1]
    ext = torch.cat([torch.zeros(K - 1, C, dtype=F64), h], dim=0)
    y = h.clone()
    for j in range(K):
        y = y + ext[j:j + T] * w.to(F64)[:, j]
    return y


# ---------------------------------------------------------------------------
# left half: windowed attention with pooled blocks
# ---------------------------------------------------------------------------
def yarn_frequencies(rot):
    """Per-pair angular frequencies [dims/2] and the common magnitude of
    cos/sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = torch.pow(torch.tensor(base, dtype=F64), -2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (
            2 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


def rotate_half(x, pos, rot):
    """x [T, heads, D]: entry i of the first dims pairs with entry
    i + dims/2."""
    dims = int(rot["dims"])
    if dims <= 0:
        return x
    f, mag = yarn_frequencies(rot)
    a = pos.to(F64)[:, None] * f[None, :]
    c = (torch.cos(a) * mag)[:, None, :]
    s = (torch.sin(a) * mag)[:, None, :]
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    y = x.clone()
    y[..., :half] = u * c - v * s
    y[..., half:dims] = v * c + u * s
    return y


def pooled_window_attention(W, pre, m, h, eps):
    T = h.shape[0]
    H = m["heads"]
    G = m.get("kv_heads", H)
    D = m["dim"]
    DV = m.get("vdim", D)
    q = lin(W, pre + "q", h)
    k = lin(W, pre + "k", h)
    v = lin(W, pre + "v", h).view(T, G, DV)
    # one root mean square over the whole projection
    q = (unit_rms(q, eps) * _w(W, pre + "q.norm")).view(T, H, D)
    k = (unit_rms(k, eps) * _w(W, pre + "k.norm")).view(T, G, D)
    rot = m.get("rot")
    pos = torch.arange(T)
    if rot:
        q = rotate_half(q, pos, rot)
        k = rotate_half(k, pos, rot)
    mask = m.get("mask") or {}
    size = int(mask.get("size", 0))
    P = int(mask.get("pool", 0))
    cap = float(m.get("softcap") or 0.0)
    out = torch.zeros(T, H, DV, dtype=F64)
    rep = H // G
    for t in range(T):
        lo = max(0, t - size + 1) if size > 0 else 0
        nb = 0
        if size > 0 and P > 0:
            # blocks whose last token is at or before t - size
            nb = max(0, (t - size + 1) // P)
        for hh in range(H):
            g = hh // rep
            keys = [k[lo:t + 1, g]]
            vals = [v[lo:t + 1, g]]
            if nb:
                keys.insert(0, k[:nb * P, g].view(nb, P, D).mean(1))
                vals.insert(0, v[:nb * P, g].view(nb, P, DV).mean(1))
            kk, vv = torch.cat(keys), torch.cat(vals)
            s = (kk @ q[t, hh]) * m["scale"]
            if cap > 0:
                s = cap * torch.tanh(s / cap)
            out[t, hh] = torch.softmax(s, dim=0) @ vv
    return lin(W, pre + "o", out.reshape(T, H * DV))


# ---------------------------------------------------------------------------
# right half: minimal gated recurrent unit
# ---------------------------------------------------------------------------
def min_gru(W, pre, h):
    T = h.shape[0]
    z = torch.sigmoid(lin(W, pre + "z", h, True))
    u = lin(W, pre + "x", h, True)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(z.shape[1], dtype=F64)
    ys = []
    for t in range(T):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        ys.append(S)
    y = torch.stack(ys) * silu(lin(W, pre + "g", h))
    return lin(W, pre + "o", y)


def parallel_mixer(W, pre, m, h, eps):
    a = pooled_window_attention(W, pre + "left.", m["left"], h, eps)
    b = min_gru(W, pre + "right.", h)
    return m["left_scale"] * a + m["right_scale"] * b


# ---------------------------------------------------------------------------
# feed-forward
# ---------------------------------------------------------------------------
def relu2_mlp(W, pre, h):
    return lin(W, pre + "down", torch.relu(lin(W, pre + "up", h)).pow(2))


def routed_ff(W, pre, m, h):
    r = m["router"]
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(lin(W, pre + "router", h))
    choice = s + _w(W, pre + "correction")
    sel = torch.topk(choice, top, dim=-1).indices
    wts = s.gather(-1, sel) * float(r.get("scale", 1.0))
    out = torch.zeros_like(h)
    for e in range(E):
        hit = (sel == e)
        rows = hit.any(-1)
        if rows.any():
            we = (wts * hit).sum(-1)[rows]
            out[rows] += relu2_mlp(W, f"{pre}e{e}.", h[rows]) * we[:, None]
    if m.get("shared"):
        out = out + relu2_mlp(W, pre + "shared.", h)
    return out


# ---------------------------------------------------------------------------
# model
# ---------------------------------------------------------------------------
def layer_runs(cfg):
    """Order of layer indices, looped span repeated; the entries at which a
    pass begins."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n)), set()
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order, begins = list(range(a)), set()
    for _ in range(times):
        begins.add(len(order))
        order += list(range(a, b))
    order += list(range(b, n))
    return order, begins


def layer(W, cfg, i, x):
    spec = cfg["layers"][i]
    eps = cfg["norm"]["eps"]
    pre = f"l{i}."
    if spec["type"] != "parallel":
        raise ValueError(spec["type"])
    conv = bool((cfg.get("canon") or {}).get("taps"))
    h = layer_norm(x, W[pre + "norm1"], W[pre + "norm1.b"], eps)
    if conv:
        h = input_conv(h, W[pre + "canon1"])
    x = x + parallel_mixer(W, pre + "mix.", spec["mixer"], h, eps)
    if spec.get("mlp") is not None:
        h = layer_norm(x, W[pre + "norm2"], W[pre + "norm2.b"], eps)
        if conv:
            h = input_conv(h, W[pre + "canon2"])
        x = x + routed_ff(W, pre + "mlp.", spec["mlp"], h)
    return x


def forward(cfg, W, tokens, streams=None):
    """tokens: list of ids of one sequence. Returns float64 logits
    [T, vocab]; `streams` (a list) receives the residual stream after every
    layer run."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x0 = _w(W, "embed")[ids] * float(cfg["embedding"]["scale"])
    x = x0
    order, begins = layer_runs(cfg)
    for n, i in enumerate(order):
        if n in begins:
            x = torch.cat([x, x0], dim=-1) @ _w(W, "loop.in").t()
        x = layer(W, cfg, i, x)
        if streams is not None:
            streams.append(x.clone())
    eps = cfg["norm"]["eps"]
    h = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return h @ _w(W, "embed").t()
