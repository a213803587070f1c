"""Plain float64 oracle of the Bipulorn design: one function per mechanism,
whole sequences, no cache, no state carried between calls, no code shared
with the engine. `cfg` is the checkpoint's config.json as a dict, `W` maps
checkpoint tensor names to tensors.

Notation: T tokens, width the model width, H heads, G key/value heads or
groups, D key width, DV value width, N state size of the state-space mixer.
"""

from __future__ import annotations

import torch

F64 = torch.float64


def _w(W, name):
    return W[name].to(F64)


def lin(W, name, x, bias=False):
    y = x @ _w(W, name).t()
    if bias:
        y = y + _w(W, name + ".b")
    return y


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """Stack norm: the tensor holds the weight minus one."""
    return unit_rms(x, eps) * (1.0 + w.to(F64))


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w.to(F64)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ---------------------------------------------------------------------------
# mixers
# ---------------------------------------------------------------------------
def rotary(x, pos, dims, base, factor):
    """x [T, H, D]: interleaved pairs (2i, 2i+1) of the first dims entries
    turn by pos * base^(-2i/dims) / factor."""
    if dims <= 0:
        return x
    i = torch.arange(dims // 2, dtype=F64)
    f = torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * i / dims)
    f = f / factor
    a = pos.to(F64)[:, None] * f[None, :]             # [T, dims/2]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    y = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    y[..., 0:dims:2] = u * c - v * s
    y[..., 1:dims:2] = v * c + u * s
    return y


def window_attention(W, pre, m, h):
    """Grouped-query sliding-window softmax attention with partial rotary
    position code and a sigmoid output gate."""
    T = h.shape[0]
    H = m["heads"]
    G = m.get("kv_heads", H)
    D = m["dim"]
    DV = m.get("vdim", D)
    q = lin(W, pre + "q", h, True).view(T, H, D)
    k = lin(W, pre + "k", h, True).view(T, G, D)
    v = lin(W, pre + "v", h, True).view(T, G, DV)
    rot = m.get("rot")
    pos = torch.arange(T)
    if rot:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = rotary(q, pos, rot["dims"], rot["base"], factor)
        k = rotary(k, pos, rot["dims"], rot["base"], factor)
    size = int((m.get("mask") or {}).get("size", 0))
    out = torch.zeros(T, H, DV, dtype=F64)
    rep = H // G
    for t in range(T):
        lo = max(0, t - size + 1) if size > 0 else 0
        for hh in range(H):
            g = hh // rep
            s = (k[lo:t + 1, g] @ q[t, hh]) * m["scale"]
            p = torch.softmax(s, dim=0)
            out[t, hh] = p @ v[lo:t + 1, g]
    gate = torch.sigmoid(lin(W, pre + "g", h))
    return lin(W, pre + "o", out.reshape(T, H * DV) * gate, True)


def causal_conv_silu(x, w, b):
    """x [T, C]; w [C, K], last column weighs the current token; zeros
    before the start."""
    T, C = x.shape
    K = w.shape[1]
    ext = torch.cat([torch.zeros(K - 1, C, dtype=F64), x], dim=0)
    y = torch.zeros(T, C, dtype=F64) + b
    for j in range(K):
        y = y + ext[j:j + T] * w[:, j]
    return silu(y)


def ssd(W, pre, m, h, eps):
    """State-space duality mixer (scalar decay per head)."""
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    p = lin(W, pre + "in", h)
    z = p[:, :inner]
    xbc = p[:, inner:2 * inner + 2 * G * N]
    dt = p[:, 2 * inner + 2 * G * N:]
    assert dt.shape[1] == H
    xbc = causal_conv_silu(xbc, _w(W, pre + "conv"), _w(W, pre + "conv.b"))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + _w(W, pre + "dt_bias"))
    A = torch.exp(_w(W, pre + "A_log"))
    Dh = _w(W, pre + "D")
    rep = H // G
    S = torch.zeros(H, N, P, dtype=F64)
    y = torch.zeros(T, H, P, dtype=F64)
    for t in range(T):
        Bt = B[t].repeat_interleave(rep, dim=0)       # [H, N]
        Ct = C[t].repeat_interleave(rep, dim=0)
        S = torch.exp(-A * dt[t])[:, None, None] * S + dt[t][:, None, None] \
            * Bt[:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnp,hn->hp", S, Ct) + Dh[:, None] * x[t]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = unit_rms(y.view(T, ng, inner // ng), eps).reshape(T, inner)
    y = y * _w(W, pre + "norm")
    return lin(W, pre + "o", y)


def parallel_pair(W, pre, m, h, eps):
    a = window_attention(W, pre + "left.", m["left"], h)
    b = ssd(W, pre + "right.", m["right"], h, eps)
    return 0.5 * (norm_plain(a, W[pre + "left.out"], eps)
                  + norm_plain(b, W[pre + "right.out"], eps))


def gla(W, pre, m, h, eps):
    """Gated linear attention: a decay per key channel."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    DV = m.get("vdim", D)
    q = (lin(W, pre + "q", h) * D ** -0.5).view(T, H, D)
    k = lin(W, pre + "k", h).view(T, H, D)
    v = lin(W, pre + "v", h).view(T, H, DV)
    zz = lin(W, pre + "a2", lin(W, pre + "a1", h), True)
    alpha = torch.exp(torch.nn.functional.logsigmoid(zz) / m["tau"])
    alpha = alpha.view(T, H, D)
    S = torch.zeros(H, D, DV, dtype=F64)
    o = torch.zeros(T, H, DV, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o, eps) * _w(W, pre + "norm")
    o = o.reshape(T, H * DV) * silu(lin(W, pre + "g", h))
    return lin(W, pre + "o", o)


def mlstm(W, pre, m, h, eps):
    """Matrix memory with exponential gates and a running maximum."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    DV = m.get("vdim", D)
    cap = float(m["gate_cap"])
    q = (lin(W, pre + "q", h) * D ** -0.5).view(T, H, D)
    k = lin(W, pre + "k", h).view(T, H, D)
    v = lin(W, pre + "v", h).view(T, H, DV)
    ig = cap * torch.tanh(lin(W, pre + "i", h, True) / cap)        # [T, H]
    fg = torch.nn.functional.logsigmoid(
        cap * torch.tanh(lin(W, pre + "f", h, True) / cap))
    S = torch.zeros(H, D, DV, dtype=F64)
    n = torch.zeros(H, D, dtype=F64)
    mm = torch.zeros(H, dtype=F64)
    o = torch.zeros(T, H, DV, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(fg[t] + mm, ig[t])
        a = torch.exp(fg[t] + mm - m_new)
        b = torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] \
            * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mm = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mm)) + 1e-6
        o[t] = num / den[:, None]
    o = unit_rms(o, eps).reshape(T, H * DV) * _w(W, pre + "norm")
    o = o * torch.sigmoid(lin(W, pre + "g", h))
    return lin(W, pre + "o", o)


# ---------------------------------------------------------------------------
# feed-forward
# ---------------------------------------------------------------------------
def gated_expert(W, pre, x):
    return lin(W, pre + "down",
               silu(lin(W, pre + "gate", x)) * lin(W, pre + "up", x))


def router(W, pre, f, h):
    """(weights [T, top], chosen [T, top]) over experts + identity outputs."""
    r = f["router"]
    s = torch.softmax(lin(W, pre + "router", h), dim=-1)
    choice = s + _w(W, pre + "correction")
    sel = torch.topk(choice, r["top"], dim=-1).indices
    w = s.gather(-1, sel)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * r.get("scale", 1.0)
    return w, sel


def moe(W, pre, f, h):
    r = f["router"]
    E = r["experts"]
    w, sel = router(W, pre, f, h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(sel.shape[1]):
            e = int(sel[t, j])
            if e >= E:                     # identity expert
                out[t] += w[t, j] * h[t]
            else:
                out[t] += w[t, j] * gated_expert(W, f"{pre}e{e}.", h[t:t + 1])[0]
    if f.get("shared"):
        gate = torch.sigmoid(lin(W, pre + "shared.sg", h))        # [T, 1]
        out = out + gate * gated_expert(W, pre + "shared.", h)
    return out


# ---------------------------------------------------------------------------
# stack
# ---------------------------------------------------------------------------
def mixer(W, i, layer, h, eps):
    pre = f"l{i}.mix."
    kind = layer["type"]
    if kind == "parallel":
        return parallel_pair(W, pre, layer["mixer"], h, eps)
    if kind == "gla":
        return gla(W, pre, layer["mixer"], h, eps)
    if kind == "mlstm":
        return mlstm(W, pre, layer["mixer"], h, eps)
    raise ValueError(kind)


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] (float64) of one whole sequence; layers_out (a
    list) receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = _w(W, "embed")[torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = mixer(W, i, layer, norm_one_plus(x, W[p + "norm1"], eps), eps)
        x = x + norm_one_plus(y, W[p + "norm1b"], eps) * _w(W, p + "ls1")
        f = layer.get("mlp")
        if f is not None:
            y = moe(W, p + "mlp.", f, norm_one_plus(x, W[p + "norm2"], eps))
            x = x + norm_one_plus(y, W[p + "norm2b"], eps) * _w(W, p + "ls2")
        if layers_out is not None:
            layers_out.append(x.clone())
    x = norm_one_plus(x, W["final.norm"], eps)
    logits = lin(W, "head", x)
    cap = float(cfg.get("logit_softcap") or 0.0)
    if cap > 0:
        logits = cap * torch.tanh(logits / cap)
    return logits
