"""Pure-PyTorch reference implementations of the HIP kernels.

These serve two purposes:
  1. the fp32 ground truth that every GPU kernel unit test compares against
     (tests/test_kernels_gpu.py);
  2. the CPU execution path, so the whole engine runs (slowly) without a GPU
     for the CPU test tier (fake-engine/CPU tier first).

They intentionally mirror the kernel semantics exactly (paged cache layout
[num_blocks, kv_heads, block_size, head_dim], slot mapping, causal masking).
"""

from __future__ import annotations

import math

import torch


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps) * w.float()
    return out.to(x.dtype)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor, eps: float
) -> tuple[torch.Tensor, torch.Tensor]:
    """Returns (normed, new_residual). Matches the in-place kernel: the
    residual accumulator is stored in bf16 (summed in fp32, rounded once)."""
    summed = (x.float() + residual.float()).to(x.dtype)
    return rms_norm(summed, w, eps), summed


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    gate = x[..., :d].float()
    up = x[..., d:].float()
    return (torch.nn.functional.silu(gate) * up).to(x.dtype)


def rotary_embedding(
    positions: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    cos_sin: torch.Tensor,
    head_dim: int,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Neox-style rotation of the leading rot_dim dims of each head.

    q: [T, QH*HD] (or [T, QH, HD]); k analogous. cos_sin: [max_pos, rot_dim]
    laid out as cos[rot/2] || sin[rot/2]. Returns rotated copies.
    """
    T = positions.shape[0]
    rot = cos_sin.shape[-1]
    half = rot // 2
    cs = cos_sin[positions.long()]  # [T, rot]
    cos = cs[:, :half].view(T, 1, half)
    sin = cs[:, half:].view(T, 1, half)

    def rotate(t: torch.Tensor) -> torch.Tensor:
        shape = t.shape
        t = t.view(T, -1, head_dim)
        x1 = t[..., :half].float()
        x2 = t[..., half:rot].float()
        r1 = x1 * cos - x2 * sin
        r2 = x2 * cos + x1 * sin
        out = t.clone()
        out[..., :half] = r1.to(t.dtype)
        out[..., half:rot] = r2.to(t.dtype)
        return out.view(shape)

    return rotate(q), rotate(k)


def reshape_and_cache(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """k/v: [T, KH, HD]; caches: [NB, KH, BS, HD]; slot_mapping: [T] int64."""
    nb, kh, bs, hd = k_cache.shape
    mask = slot_mapping >= 0
    slots = slot_mapping[mask]
    blk = torch.div(slots, bs, rounding_mode="floor").long()
    off = (slots % bs).long()
    k_cache[blk, :, off] = k.view(-1, kh, hd)[mask].to(k_cache.dtype)
    v_cache[blk, :, off] = v.view(-1, kh, hd)[mask].to(v_cache.dtype)


def _gather_kv(
    cache: torch.Tensor, block_table: torch.Tensor, ctx: int
) -> torch.Tensor:
    """cache: [NB, KH, BS, HD] -> [ctx, KH, HD] for one sequence."""
    nb, kh, bs, hd = cache.shape
    nblocks = (ctx + bs - 1) // bs
    blocks = block_table[:nblocks].long()
    kv = cache[blocks]  # [nblocks, KH, BS, HD]
    kv = kv.permute(0, 2, 1, 3).reshape(nblocks * bs, kh, hd)
    return kv[:ctx]


def paged_attn_decode(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    """q: [S, QH, HD] -> out [S, QH, HD] (fp32 math, cast back).
    window > 0 = sliding-window attention over the last `window` keys."""
    S, QH, HD = q.shape
    KH = k_cache.shape[1]
    GQ = QH // KH
    out = torch.empty_like(q)
    for s in range(S):
        ctx = int(seq_lens[s])
        k = _gather_kv(k_cache, block_tables[s], ctx).float()  # [ctx, KH, HD]
        v = _gather_kv(v_cache, block_tables[s], ctx).float()
        if window and ctx > window:
            k = k[ctx - window:]
            v = v[ctx - window:]
        for h in range(QH):
            kvh = h // GQ
            qs = q[s, h].float()
            logits = (k[:, kvh] @ qs) * scale  # [ctx]
            p = torch.softmax(logits, dim=-1)
            out[s, h] = (p @ v[:, kvh]).to(q.dtype)
    return out


def paged_attn_prefill(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    token_seq: torch.Tensor,
    token_pos: torch.Tensor,
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    """q: [T, QH, HD]; each token t attends to cache[token_seq[t]][0..pos]
    (or the last `window` positions when window > 0)."""
    T, QH, HD = q.shape
    KH = k_cache.shape[1]
    GQ = QH // KH
    out = torch.empty_like(q)
    for t in range(T):
        s = int(token_seq[t])
        ctx = int(token_pos[t]) + 1
        k = _gather_kv(k_cache, block_tables[s], ctx).float()
        v = _gather_kv(v_cache, block_tables[s], ctx).float()
        if window and ctx > window:
            k = k[ctx - window:]
            v = v[ctx - window:]
        for h in range(QH):
            kvh = h // GQ
            qs = q[t, h].float()
            logits = (k[:, kvh] @ qs) * scale
            p = torch.softmax(logits, dim=-1)
            out[t, h] = (p @ v[:, kvh]).to(q.dtype)
    return out


def greedy_sample(logits: torch.Tensor) -> torch.Tensor:
    return logits.float().argmax(dim=-1)


def kv_quant(x: torch.Tensor) -> tuple:
    """Row-wise int8 quantization over the last dim. Returns (int8, scales)."""
    hd = x.shape[-1]
    rows = x.reshape(-1, hd).float()
    amax = rows.abs().amax(dim=-1)
    scales = torch.where(amax > 0, amax / 127.0, torch.ones_like(amax))
    q = torch.clamp(
        torch.round(rows / scales[:, None]), -127, 127
    ).to(torch.int8)
    return q.view(x.shape), scales


def kv_dequant(q: torch.Tensor, scales: torch.Tensor,
               dtype=torch.bfloat16) -> torch.Tensor:
    hd = q.shape[-1]
    rows = q.reshape(-1, hd).float() * scales[:, None]
    return rows.to(dtype).view(q.shape)


def lora_bgmv(out, x, A, B, scale, idx, col_off):
    """Reference BGMV: out[t, col_off:+W] += scale[s] * B[s] @ (A[s] @ x[t])
    for s = idx[t] >= 0."""
    import torch

    W = B.shape[1]
    for t in range(x.shape[0]):
        s = int(idx[t])
        if s < 0:
            continue
        y = (A[s].float() @ x[t].float()) * float(scale[s])
        out[t, col_off : col_off + W] += (B[s].float() @ y).to(out.dtype)


# ---------------------------------------------------------------------------
# fp32-residual stack ops (hybrid recurrent/attention models)
# ---------------------------------------------------------------------------
def embed_scale(tokens, embed, scale: float) -> torch.Tensor:
    """fp32 residual stream rows: embed[token] * scale."""
    return embed[tokens].float() * scale


def add_rms_norm32(x32, deltas, w32, eps: float, out_dtype, groups: int = 1,
                   out32=None):
    """out32 = x32 + sum(deltas) in fp32 (out32 defaults to x32: in place);
    returns norm(out32) * w32 in out_dtype. With groups > 1 every one of
    `groups` equal consecutive parts of a row is divided by its own root
    mean square."""
    if out32 is None:
        out32 = x32
    if deltas:
        acc = deltas[0].float()
        for d in deltas[1:]:
            acc = acc + d.float()
        torch.add(x32, acc, out=out32)
    elif out32 is not x32:
        out32.copy_(x32)
    return (_group_unit(out32, eps, groups) * w32).to(out_dtype)


def _group_unit(x32, eps: float, groups: int):
    T, W = x32.shape
    p = x32.view(T, groups, W // groups)
    return (p * torch.rsqrt(p.pow(2).mean(-1, keepdim=True) + eps)).view(T, W)


def group_norm_shift(x32, w32, eps: float, groups: int, out_dtype, shift,
                     state, seq_rows):
    """h = groupnorm(x32) * w32, then every row is blended with its
    predecessor's h: h + (h_prev - h) * shift (fp32, one rounding). The
    predecessor of a segment's first row is state[slot] (zeros when the
    segment starts at position 0); state[slot] becomes the h of the
    segment's last row. seq_rows [S, 4] = (first row, rows, first
    position, slot)."""
    h = _group_unit(x32, eps, groups) * w32
    out = torch.empty_like(h)
    for t0, n, p0, slot in seq_rows.tolist():
        prev = torch.empty_like(h[t0:t0 + n])
        prev[0] = state[slot] if p0 > 0 else 0.0
        prev[1:] = h[t0:t0 + n - 1]
        out[t0:t0 + n] = h[t0:t0 + n] + (prev - h[t0:t0 + n]) * shift
        state[slot] = h[t0 + n - 1]
    return out.to(out_dtype)


def depth_mix(hist, n: int, weights, base, delta):
    """hist fp32 [streams, T, W]. The newest stream hist[n-1] = base +
    delta (fp32) is stored, and sum_{j<n} weights[j] * hist[j] returned."""
    torch.add(base, delta.float(), out=hist[n - 1])
    return torch.einsum("j,jtw->tw", weights[:n].float(), hist[:n])


def gated_act(gate, up, kind: str, limit: float, out_dtype):
    """Gated-MLP inner activation, fp32 math, one rounding at the end.
    silu: silu(g)*u; gelu_tanh: gelu_tanh(g)*u; clamped_swish:
    g' = min(g, limit), u' = clamp(u, +-limit), g' sigmoid(1.702 g') (u'+1);
    sigmoid: sigmoid(g)*u (an output gate); relu2: relu(g)^2 * u. up None:
    the plain activation (u = 1).
    """
    g = gate.float()
    u = up.float() if up is not None else 1.0
    if kind == "relu2":
        y = torch.relu(g).pow(2) * u
    elif kind == "silu":
        y = torch.nn.functional.silu(g) * u
    elif kind == "gelu_tanh":
        y = torch.nn.functional.gelu(g, approximate="tanh") * u
    elif kind == "clamped_swish":
        g = torch.clamp(g, max=limit)
        u = (torch.clamp(u, min=-limit, max=limit) if up is not None
             else 0.0)
        y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    elif kind == "sigmoid":
        y = torch.sigmoid(g) * u
    else:
        raise ValueError(kind)
    return y.to(out_dtype)


def kv_append(k, v, k_cache, v_cache, slot_mapping) -> None:
    """k [T, G, D], v [T, G, DV] -> caches [NB, G, BS, D|DV] (k and v may
    differ in their last dim)."""
    bs = k_cache.shape[2]
    blk = (slot_mapping // bs).long()
    off = (slot_mapping % bs).long()
    k_cache[blk, :, off] = k.to(k_cache.dtype)
    v_cache[blk, :, off] = v.to(v_cache.dtype)


def talk_attention(q, k_cache, v_cache, block_tables, token_seq, token_pos,
                   scale: float, chunk: int, window: int, sink: bool,
                   talk, keep_first: int = 0, softcap: float = 0.0,
                   sink_vals=None, vdim: int = 0, pool=None):
    """Paged attention with optional head-mixed scores, aligned-chunk or
    trailing-window visibility (the first keep_first keys stay visible
    behind the window), capped scores and a denominator sink (score 0, or
    sink_vals[h]). q [T, H, D]; the values are the first vdim entries of
    v_cache rows (all of them when 0; v_cache may be k_cache). Returns
    [T, H, DV] in q's dtype; all score math in fp32. pool = (kp_cache,
    vp_cache, P): with a window, every block of P positions whose last
    position is at or before pos - window adds its pooled key/value (see
    pool_append) to the same softmax."""
    T, H, D = q.shape
    G, bs = v_cache.shape[1], v_cache.shape[2]
    DV = vdim or v_cache.shape[3]
    rep = H // G
    out = torch.zeros(T, H, DV, dtype=torch.float32)
    tk = talk.float() if talk is not None else None
    for t in range(T):
        pos = int(token_pos[t])
        lo = 0
        if chunk > 0:
            lo = (pos // chunk) * chunk
        if window > 0:
            lo = max(lo, pos - window + 1)
        idx = torch.arange(lo, pos + 1)
        if keep_first > 0 and lo > 0:
            idx = torch.cat([torch.arange(0, min(keep_first, lo)), idx])
        table = block_tables[int(token_seq[t])].long()
        blk = table[idx // bs]
        off = idx % bs
        kk = k_cache[blk, :, off].float()          # [n, G, D]
        vv = v_cache[blk, :, off][..., :DV].float()  # [n, G, DV]
        if pool is not None and window > 0:
            kp, vp, P = pool
            nb = max(0, (pos - window + 1) // P)
            if nb:
                first = torch.arange(nb) * P
                pb, po = table[first // bs], (first % bs) // P
                kk = torch.cat([kp[pb, :, po].float(), kk])
                vv = torch.cat([vp[pb, :, po][..., :DV].float(), vv])
        kk = kk.repeat_interleave(rep, dim=1)      # [n, H, D]
        vv = vv.repeat_interleave(rep, dim=1)
        s = torch.einsum("hd,nhd->hn", q[t].float(), kk) * scale
        if tk is not None:
            s = tk @ s
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        m = s.max(dim=-1, keepdim=True).values
        if sink:
            s0 = (sink_vals.float().view(H, 1) if sink_vals is not None
                  else torch.zeros(H, 1))
            m = torch.maximum(m, s0)
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink:
            den = den + torch.exp(s0 - m)
        out[t] = torch.einsum("hn,nhv->hv", e / den, vv)
    return out.to(q.dtype)


def attn_prep(q, k, v, q_w, k_w, eps: float, vmix, v_first, k_cache,
              v_cache, slot_mapping, heads: int, cos_sin=None,
              positions=None, rot_dims: int = 0, norm_all: bool = False,
              half: bool = False):
    """Query/key head norm, value blend and cache append of one attention
    layer. q [T, H*D] is normalised in place per head (x / rms(x) * q_w,
    fp32 math); k [T, G*D] likewise with k_w and appended; v [T, G*DV]
    becomes (1 - vmix) v + vmix v_first when v_first is given (vmix a
    0-dim fp32 tensor), is written back, and appended. q_w / k_w None:
    no norm. With cos_sin (fp32 [positions, rot_dims/2, 2]) the first
    rot_dims entries of every query and key head turn by the row of the
    token's position (interleaved pairs, or with `half` entry i paired
    with entry i + rot_dims/2), after the norm. norm_all: q_w [H*D] / k_w
    [G*D] and one root mean square over the whole projection."""
    T = q.shape[0]
    G, bs, D = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    DV = v_cache.shape[3]
    cs = cos_sin[positions.long()][:, None] if cos_sin is not None else None
    if q_w is not None or cs is not None:
        qf = q.float().view(T, heads, D)
        if q_w is not None:
            qf = _unit_heads(qf, eps, norm_all) * q_w.view(
                (1, heads, D) if norm_all else (1, 1, D))
        if cs is not None:
            qf = _rotate(qf, cs, rot_dims, half)
        q.copy_(qf.reshape(T, heads * D).to(q.dtype))
    kf = k.float().view(T, G, D)
    if k_w is not None:
        kf = _unit_heads(kf, eps, norm_all) * k_w.view(
            (1, G, D) if norm_all else (1, 1, D))
    if cs is not None:
        kf = _rotate(kf, cs, rot_dims, half)
    vf = v.float()
    if v_first is not None:
        lam = vmix.float()
        vf = (1.0 - lam) * vf + lam * v_first.float()
        v.copy_(vf.to(v.dtype))
    kv_append(kf, vf.view(T, G, DV), k_cache, v_cache, slot_mapping)


def _unit_heads(x, eps: float, whole: bool):
    """x fp32 [T, heads, D] over its root mean square per head, or over all
    heads at once."""
    ms = (x.pow(2).mean((-2, -1), keepdim=True) if whole
          else x.pow(2).mean(-1, keepdim=True))
    return x * torch.rsqrt(ms + eps)


def scaled_frequencies(dims: int, base: float, scaling=None):
    """float64 [dims/2] angular frequencies base^(-2i/dims) and the common
    magnitude of cos/sin. scaling = (factor, original, fast, slow): with
    d(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(
    d(fast)), 0), hi = min(ceil(d(slow)), dims - 1) and ramp_i =
    clamp((i - lo) / max(hi - lo, 0.001), 0, 1), frequency i becomes
    f_i / factor * ramp_i + f_i (1 - ramp_i); the magnitude is
    0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                  -2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original, fast, slow = (float(v) for v in scaling)

    def d_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (
            2.0 * math.log(base))

    lo = max(math.floor(d_of(fast)), 0)
    hi = min(math.ceil(d_of(slow)), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rope_table(max_pos: int, dims: int, base: float, device=None,
               factor: float = 1.0, scaling=None):
    """fp32 [max_pos, dims/2, 2] = (cos, sin) of position * base^(-2i/dims)
    / factor (linear position scaling); with `scaling` the frequencies and
    the magnitude of scaled_frequencies. The angles are formed in float64
    on the host, so an entry is the correctly rounded fp32 value."""
    f, mag = scaled_frequencies(dims, base, scaling)
    f = f / float(factor)
    a = torch.arange(max_pos, dtype=torch.float64)[:, None] * f
    t = (torch.stack([torch.cos(a), torch.sin(a)], dim=-1) * mag).float()
    return t.to(device).contiguous() if device is not None else t.contiguous()


def _rotate(x, cs, dims: int, half: bool = False):
    """x fp32 [..., n]; cs [..., dims/2, 2] broadcastable; pairs of the
    first dims entries turn: interleaved (2i, 2i+1), or (i, i + dims/2)
    with `half`."""
    x = x.clone()
    if half:
        a, b = slice(0, dims // 2), slice(dims // 2, dims)
    else:
        a, b = slice(0, dims, 2), slice(1, dims, 2)
    u, w = x[..., a].clone(), x[..., b].clone()
    c, s = cs[..., 0], cs[..., 1]
    x[..., a] = u * c - w * s
    x[..., b] = w * c + u * s
    return x


def pool_append(k_cache, v_cache, kp_cache, vp_cache, block_tables,
                seq_rows, pool: int) -> None:
    """Pooled keys/values of the blocks of `pool` consecutive positions
    that this step completes. Block b holds positions b*pool .. b*pool +
    pool - 1; once its last position is cached, the fp32 means of its keys
    and of its values, as the caches [NB, G, BS, D|DV] hold them, are
    stored (rounded to the cache dtype) in kp_cache / vp_cache [NB, G,
    ceil(BS / pool), D|DV]: in the page of the block's first position, at
    row (first position mod BS) div pool. seq_rows row i = (first batch
    row, rows, first position, slot) and block_tables row i belong to
    segment i."""
    bs = k_cache.shape[2]
    for i, (_, n, p0, _) in enumerate(seq_rows.tolist()):
        table = block_tables[i].long()
        # blocks whose last position lies in [p0, p0 + n)
        for b in range(p0 // pool, (p0 + n) // pool):
            idx = torch.arange(b * pool, (b + 1) * pool)
            blk, off = table[idx // bs], idx % bs
            page, row = table[(b * pool) // bs], ((b * pool) % bs) // pool
            kp_cache[page, :, row] = k_cache[blk, :, off].float().mean(0).to(
                kp_cache.dtype)
            vp_cache[page, :, row] = v_cache[blk, :, off].float().mean(0).to(
                vp_cache.dtype)


def add_layer_norm_conv32(x32, deltas, scales, w32, b32, eps: float,
                          conv_w, state, seq_rows, out_dtype):
    """Sublayer boundary of a stack with layer norms and input
    convolutions: x32 += sum_i scales[i] * deltas[i] (fp32, in place), y =
    (x32 - mean) / sqrt(var + eps) * w32 + b32 per row, and the returned
    h = y + conv(y) in out_dtype, conv(y)_t = sum_j conv_w[:, j] *
    y_(t - K + 1 + j) along each segment of seq_rows with the segment's
    previous K - 1 rows of y taken from state fp32 [slots, K-1, W] (zeros
    for a segment that starts at position 0); state receives the last K - 1
    rows. conv_w None: h = y."""
    if deltas:
        acc = None
        for d, sc in zip(deltas, scales):
            term = d.float() * sc
            acc = term if acc is None else acc + term
        x32.add_(acc)
    mu = x32.mean(-1, keepdim=True)
    var = (x32 - mu).pow(2).mean(-1, keepdim=True)
    y = (x32 - mu) * torch.rsqrt(var + eps) * w32 + b32
    if conv_w is None:
        return y.to(out_dtype)
    T, W = y.shape
    K = conv_w.shape[1]
    h = torch.empty_like(y)
    for t0, n, p0, slot in seq_rows.tolist():
        past = state[slot] if p0 > 0 else torch.zeros(K - 1, W)
        ext = torch.cat([past, y[t0:t0 + n]], dim=0)
        acc = y[t0:t0 + n].clone()
        for j in range(K):
            acc += ext[j:j + n] * conv_w[:, j]
        h[t0:t0 + n] = acc
        if K > 1:
            state[slot] = ext[n:]
    return h.to(out_dtype)


def mingru_scan(z, u, g, zb, ub, state, seq_rows, out_dtype):
    """Element-wise gated recurrence over a ragged batch. z / u / g [T, C]
    (gate, candidate and read-out projections), zb / ub fp32 [C] their
    biases; state fp32 [slots, C], updated in place, zeros for a segment
    that starts at position 0. Per token a = sigmoid(z + zb), c = u + ub +
    1/2 where u + ub >= 0 and sigmoid(u + ub) below, S <- (1 - a) S + a c;
    returns S * silu(g) in out_dtype. All arithmetic fp32."""
    a = torch.sigmoid(z.float() + zb)
    uu = u.float() + ub
    c = torch.where(uu >= 0, uu + 0.5, torch.sigmoid(uu))
    T, C = a.shape
    y = torch.empty(T, C, dtype=torch.float32)
    for t0, n, p0, slot in seq_rows.tolist():
        S = state[slot].clone() if p0 > 0 else torch.zeros(C)
        for t in range(t0, t0 + n):
            S = (1.0 - a[t]) * S + a[t] * c[t]
            y[t] = S
        state[slot] = S
    gf = g.float()
    return (y * gf * torch.sigmoid(gf)).to(out_dtype)


def latent_prep(q_lat, q, dkv, norm_w, eps: float, cos_sin, positions,
                cache, slot_mapping, heads: int, dim: int, rot_dim: int,
                rot_dims: int, out_dtype):
    """Inputs of latent attention for one step. q_lat [H, T, L]: the
    position-free query parts already mapped into the latent space; q
    [T, H*(dim+rot_dim)]: its rotated parts are taken and turned; dkv
    [T, L+rot_dim]: the first L entries are RMS-normalised (norm_w) into
    the latent, the rest is the shared rotated key part. The cache
    [NB, 1, BS, L+rot_dim] receives [latent | turned key part]; returns
    the queries [T, H*(L+rot_dim)] = per head [q_lat | turned part]."""
    H = heads
    T = q.shape[0]
    L = dkv.shape[1] - rot_dim
    cs = cos_sin[positions.long()]                        # [T, dims/2, 2]
    c = dkv[:, :L].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w
    kr = _rotate(dkv[:, L:].float(), cs, rot_dims)
    row = torch.cat([c, kr], dim=-1)
    bs = cache.shape[2]
    cache[(slot_mapping // bs).long(), 0, (slot_mapping % bs).long()] = \
        row.to(cache.dtype)
    qr = q.float().view(T, H, dim + rot_dim)[..., dim:]
    qr = _rotate(qr, cs[:, None], rot_dims)
    full = torch.cat([q_lat.float().transpose(0, 1), qr], dim=-1)
    return full.reshape(T, H * (L + rot_dim)).to(out_dtype)


def short_conv_silu(x, w, state, seq_rows, out_dtype, bias=None):
    """Causal per-channel convolution over time followed by silu. x [T, C];
    w fp32 [C, K] (last column weighs the current token); state
    [slots, K-1, C] holds a sequence's last K-1 inputs (oldest first) and is
    updated; a segment at position 0 starts from zeros. bias: optional
    fp32 [C] added before the silu."""
    T, C = x.shape
    K = w.shape[1]
    y = torch.empty(T, C, dtype=torch.float32)
    for t0, n, p0, slot in seq_rows.tolist():
        past = state[slot].float() if p0 > 0 else torch.zeros(K - 1, C)
        ext = torch.cat([past, x[t0:t0 + n].float()], dim=0)   # [K-1+n, C]
        acc = torch.zeros(n, C)
        if bias is not None:
            acc = acc + bias.float()
        for j in range(K):
            acc += ext[j:j + n] * w[:, j]
        y[t0:t0 + n] = acc
        if K > 1:
            state[slot] = ext[n:].to(state.dtype)
    return (y * torch.sigmoid(y)).to(out_dtype)


def gated_delta(q, k, v, beta, zdec, zgate, a_log, dt_bias, normw, state,
                seq_rows, heads: int, kv_heads: int, eps: float, out_dtype):
    """Gated delta rule with a per-(head, key channel) decay over a ragged
    batch. q/k [T, G, D], v [T, H, DV], beta [T, H] (pre-sigmoid), zdec
    [T, H, D] (pre-softplus, without dt_bias), zgate [T, H, DV]
    (pre-sigmoid); a_log fp32 [H], dt_bias fp32 [H*D], normw fp32 [DV];
    state fp32 [slots, H, D, DV] updated in place. Per token and head
      q, k <- unit vectors (q also times D^-1/2),
      g = exp(-exp(a_log) * softplus(zdec + dt_bias)),
      S <- diag(g) S;  u = sigmoid(beta) (v - S^T k);  S <- S + k u^T;
      o = S^T q,
    then o / rms(o) * normw * sigmoid(zgate)."""
    T, G, D = q.shape
    H = heads
    DV = v.shape[2]
    rep = H // G
    qf = q.float()
    kf = k.float()
    qf = qf * torch.rsqrt(qf.pow(2).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    kf = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + 1e-6)
    qf = qf.repeat_interleave(rep, dim=1)
    kf = kf.repeat_interleave(rep, dim=1)
    g = torch.exp(-torch.exp(a_log.float()).view(1, H, 1)
                  * torch.nn.functional.softplus(
                      zdec.float() + dt_bias.view(1, H, D)))
    b = torch.sigmoid(beta.float())
    out = torch.empty(T, H, DV, dtype=torch.float32)
    for t0, n, p0, slot in seq_rows.tolist():
        S = state[slot]
        if p0 == 0:
            S.zero_()
        for t in range(t0, t0 + n):
            S.mul_(g[t].unsqueeze(-1))
            sk = torch.einsum("hi,hij->hj", kf[t], S)
            u = b[t].unsqueeze(-1) * (v[t].float() - sk)
            S.add_(kf[t].unsqueeze(-1) * u.unsqueeze(1))
            out[t] = torch.einsum("hij,hi->hj", S, qf[t])
    y = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps)
    y = y * normw.view(1, 1, DV) * torch.sigmoid(zgate.float())
    return y.to(out_dtype)


def delta_rule(r, k, v, zw, za, g, w0, ab, normw, state, seq_rows,
               eps: float, decay_scale: float, out_dtype):
    """Gated delta-rule recurrence over a ragged batch.

    r/k/v/zw/za/g: [T, H, D] views (any float dtype); w0/ab/normw fp32
    [H*D]; state fp32 [slots, H, D, D] updated in place; seq_rows
    [S, 4] int (first row, rows, first position, state slot). Per token
      w = exp(-decay_scale * sigmoid(zw + w0)),  a = sigmoid(za + ab),
      u = k / sqrt(sum k^2 + 1e-6),
      S <- diag(w) S - (a*u)(u^T S) + k v^T,   o = S^T r,
    then o / rms(o) per head * normw * sigmoid(g). A segment whose first
    position is 0 starts from a zero state."""
    T, H, D = r.shape
    out = torch.empty(T, H, D, dtype=torch.float32)
    w0 = w0.view(H, D)
    ab = ab.view(H, D)
    for t0, n, p0, slot in seq_rows.tolist():
        S = state[slot]
        if p0 == 0:
            S.zero_()
        for t in range(t0, t0 + n):
            kk = k[t].float()
            w = torch.exp(-decay_scale * torch.sigmoid(zw[t].float() + w0))
            a = torch.sigmoid(za[t].float() + ab)
            u = kk * torch.rsqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
            sa = torch.einsum("hi,hij->hj", u, S)
            S.mul_(w.unsqueeze(-1))
            S.sub_((a * u).unsqueeze(-1) * sa.unsqueeze(1))
            S.add_(kk.unsqueeze(-1) * v[t].float().unsqueeze(1))
            out[t] = torch.einsum("hij,hi->hj", S, r[t].float())
    var = out.pow(2).mean(-1, keepdim=True)
    y = out * torch.rsqrt(var + eps) * normw.view(1, H, D)
    y = y * torch.sigmoid(g.float())
    return y.to(out_dtype)


def norm_sum32(inputs, weights, scale: float, eps: float):
    """fp32 [T, W] = scale * sum_i rmsnorm(inputs[i]) * weights[i]."""
    acc = None
    for x, w in zip(inputs, weights):
        xf = x.float()
        y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w
        acc = y if acc is None else acc + y
    return acc * scale


def post_norm_add_norm32(x32, delta, w_post, w_next, eps: float, out_dtype):
    """x32 += rmsnorm(delta) * w_post (fp32, in place); returns
    rmsnorm(x32) * w_next in out_dtype."""
    d = delta.float()
    x32.add_(d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w_post)
    return (x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps)
            * w_next).to(out_dtype)


def _log_sigmoid(z):
    return torch.clamp(z, max=0.0) - torch.log1p(torch.exp(-z.abs()))


def linear_scan(mode: str, q, k, v, dec, wr, gate, p0, p1, p2, normw, state,
                aux, seq_rows, heads: int, groups: int, eps: float,
                qscale: float, c0: float, out_dtype):
    """Gated linear recurrences S <- diag(a) S + w k v^T, o = S^T q over a
    ragged batch; S fp32 [slots, H, D, DV] updated in place, a segment at
    position 0 starts from zeros. q/k [T, G, D] (head h reads group
    h // (H / G)), v [T, H, DV], gate [T, H, DV].
    mode "gla": dec [T, H, D] raw, a = sigmoid(dec + p0)^c0 per key channel,
      w = 1, q *= qscale; result rmsnorm_DV(o) * normw[DV] * silu(gate).
    mode "ssd": dec [T, H] raw, dt = softplus(dec + p0[h]),
      a = exp(-exp(p1[h]) dt), w = dt; result (o + p2[h] v) * silu(gate),
      fp32.
    mode "mlstm": dec / wr [T, H] raw forget / input gates; f =
      logsigmoid(cap(dec + p1[h])), i = cap(wr + p0[h]), cap(z) = c0
      tanh(z / c0); running maximum m (aux[slot, h, D]) and normaliser n
      (aux[slot, h, :D]): m' = max(f + m, i), a = exp(f + m - m'), w =
      exp(i - m'), n <- a n + w k; o / (max(|n.q|, exp(-m')) + 1e-6),
      q *= qscale; result o / rms_DV(o) * normw[h, DV] * sigmoid(gate)."""
    T, G, D = q.shape
    H = heads
    DV = v.shape[2]
    rep = H // G
    qf = q.float().repeat_interleave(rep, dim=1) * qscale
    kf = k.float().repeat_interleave(rep, dim=1)
    vf = v.float()
    if mode == "gla":
        a_all = torch.exp(_log_sigmoid(dec.float() + p0.view(1, H, D)) * c0)
        w_all = torch.ones(T, H)
    elif mode == "ssd":
        dt = torch.nn.functional.softplus(dec.float() + p0.view(1, H),
                                          threshold=20.0)
        a_all = torch.exp(-torch.exp(p1.float()).view(1, H) * dt)
        w_all = dt
    elif mode == "mlstm":
        ig = c0 * torch.tanh((wr.float() + p0.view(1, H)) / c0)
        fg = _log_sigmoid(c0 * torch.tanh((dec.float() + p1.view(1, H)) / c0))
    else:
        raise ValueError(mode)
    out = torch.empty(T, H, DV, dtype=torch.float32)
    for t0, n, pos0, slot in seq_rows.tolist():
        S = state[slot]
        if pos0 == 0:
            S.zero_()
            if aux is not None:
                aux[slot].zero_()
        for t in range(t0, t0 + n):
            if mode == "mlstm":
                nv, m = aux[slot, :, :D], aux[slot, :, D]
                m_new = torch.maximum(fg[t] + m, ig[t])
                a = torch.exp(fg[t] + m - m_new)
                w = torch.exp(ig[t] - m_new)
                S.mul_(a.view(H, 1, 1))
                S.add_((w.view(H, 1) * kf[t]).unsqueeze(-1)
                       * vf[t].unsqueeze(1))
                nv.mul_(a.view(H, 1)).add_(w.view(H, 1) * kf[t])
                m.copy_(m_new)
                num = torch.einsum("hij,hi->hj", S, qf[t])
                den = torch.maximum((nv * qf[t]).sum(-1).abs(),
                                    torch.exp(-m_new)) + 1e-6
                out[t] = num / den.unsqueeze(-1)
                continue
            a = a_all[t]
            S.mul_(a.unsqueeze(-1) if mode == "gla" else a.view(H, 1, 1))
            S.add_((w_all[t].view(H, 1) * kf[t]).unsqueeze(-1)
                   * vf[t].unsqueeze(1))
            out[t] = torch.einsum("hij,hi->hj", S, qf[t])
    g = gate.float()
    if mode == "ssd":
        y = (out + p2.float().view(1, H, 1) * vf) * g * torch.sigmoid(g)
        return y
    y = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps)
    if mode == "gla":
        y = y * normw.view(1, 1, DV) * g * torch.sigmoid(g)
    else:
        y = y * normw.view(1, H, DV) * torch.sigmoid(g)
    return y.to(out_dtype)


def moe_route(x, router_w, top: int, score: str, renormalize: bool,
              correction, scale: float, renorm_eps: float):
    """Router of a routed feed-forward: fp32 logits, softmax | sigmoid
    scores, the `top` outputs with the largest score + correction (sigmoid
    scores without a correction are ranked by their logits), weights =
    chosen scores, divided by
    (their sum + renorm_eps) when renormalize, times scale. Returns
    (weights [T, top], indices [T, top], dense [T, n_out])."""
    logits = torch.nn.functional.linear(x.float(), router_w.float())
    if score == "softmax":
        probs = torch.softmax(logits, dim=-1)
        pick = probs + correction if correction is not None else probs
    else:
        probs = torch.sigmoid(logits)
        pick = probs + correction if correction is not None else logits
    sel = torch.topk(pick, top, dim=-1).indices
    w = probs.gather(-1, sel)
    if renormalize:
        w = w / (w.sum(-1, keepdim=True) + renorm_eps)
    w = w * scale
    dense = torch.zeros_like(probs).scatter_(1, sel, w)
    return w, sel, dense


def moe_combine(y, dense, x, experts: int, shared_y=None, shared_gate=None):
    """fp32 [T, W] = sum_e dense[:, e] y[e] over the experts + (sum of the
    identity outputs' weights) x + sigmoid(shared_gate) shared_y (shared_y
    alone when shared_gate is None)."""
    out = torch.einsum("te,etw->tw", dense[:, :experts], y.float())
    if dense.shape[1] > experts:
        out = out + dense[:, experts:].sum(-1, keepdim=True) * x.float()
    if shared_y is not None and shared_gate is not None:
        out = out + torch.sigmoid(shared_gate.float()) * shared_y.float()
    elif shared_y is not None:
        out = out + shared_y.float()
    return out
