"""Token mixers for heterogeneous (per-layer spec) models.

Each mixer exposes
  * in_params(): its input-projection parameters, so a layer can run ONE
                GEMM over [mixer rows | feed-forward rows] of the shared
                norm output;
  * cache_shape(): what the runner must allocate per layer — a paged KV
                pair for attention, a per-sequence fp32 state for the
                recurrence;
  * forward_from_proj(proj, meta, cache) -> the mixer's pre-output-projection
                activations [T, out_in], and out_weight [width, out_in];
  * forward(h, meta, cache, shared) -> the same from the layer input, for
                layers whose mixer does not share its input projection
                (`shared` is a per-step dict for tensors that later layers
                of the stack read, e.g. the first value-mixing layer's
                values).
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from production_stack_amd import ops
from production_stack_amd.engine.config import MixerSpec
from production_stack_amd.ops import gemm_policy

# decay = exp(-DECAY_SCALE * sigmoid(.)): the per-step decay stays in
# (exp(-DECAY_SCALE), 1)
DELTA_DECAY_SCALE = math.exp(-0.5)


class TalkAttention(nn.Module):
    """Grouped-query softmax attention over the paged KV cache with the
    MixerSpec's options: score mixing across heads, aligned-chunk /
    trailing-window visibility (with kept first keys), capped scores,
    denominator sink (fixed or learned), projection biases, per-head
    query/key norm, rotary position code on the leading entries of every
    head (interleaved or half-split pairs, linear position scaling or
    blended frequencies), value blending with the stack's first
    value-mixing layer, a sigmoid output gate on the concatenated heads;
    key and value widths may differ. `window_pool`: blocks of positions
    behind the window stay visible through one mean key/value each, kept in
    a pooled cache that shares the pages of the key/value cache;
    `qk_norm_all`: query and key are normalised over their whole
    projections."""

    kind = "attention"

    def __init__(self, width: int, spec: MixerSpec,
                 dtype: torch.dtype, eps: float = 1e-5,
                 max_pos: int = 8192) -> None:
        super().__init__()
        if spec.rope and spec.rot_dims <= 0:
            raise NotImplementedError(
                "rotary attention here turns pairs of the first rot_dims "
                "entries of a head; give rot_dims")
        self.spec = spec
        self.max_pos = max_pos
        self._cos_sin = None
        H, G = spec.heads, spec.kv_heads or spec.heads
        D, DV = spec.dim, spec.vdim or spec.dim
        if H % G:
            raise ValueError("heads must be a multiple of kv_heads")
        self.H, self.G, self.D, self.DV = H, G, D, DV
        # fused rows: q | k | v (| output gate)
        self.qkv_rows = H * D + G * D + G * DV
        self.qkv = nn.Parameter(torch.empty(
            self.qkv_rows + (H * DV if spec.out_gate else 0), width,
            dtype=dtype))
        self.out_weight = nn.Parameter(
            torch.empty(width, H * DV, dtype=dtype))
        self.out_bias = (nn.Parameter(torch.empty(width, dtype=dtype))
                         if spec.out_bias else None)
        self.talk = (
            nn.Parameter(torch.empty(H, H, dtype=torch.float32))
            if spec.talking_heads else None)
        self.scale = spec.scale or 1.0 / math.sqrt(D)
        self.eps = eps
        self.qkv_bias = (
            nn.Parameter(torch.empty(self.qkv.shape[0], dtype=dtype))
            if spec.bias else None)
        self.q_norm = self.k_norm = None
        if spec.qk_norm_all:
            self.q_norm = nn.Parameter(
                torch.empty(H * D, dtype=torch.float32))
            self.k_norm = nn.Parameter(
                torch.empty(G * D, dtype=torch.float32))
        elif spec.qk_norm:
            self.q_norm = nn.Parameter(torch.empty(D, dtype=torch.float32))
            self.k_norm = nn.Parameter(torch.empty(D, dtype=torch.float32))
        if spec.window_pool and not spec.window:
            raise ValueError("pooled blocks need a window")
        if spec.rot_layout not in ("interleaved", "half"):
            raise ValueError(f"unknown rotary layout {spec.rot_layout!r}")
        self.sink_vals = (
            nn.Parameter(torch.empty(H, dtype=torch.float32))
            if spec.learned_sink else None)
        self.vmix = (
            nn.Parameter(torch.empty((), dtype=torch.float32))
            if spec.v_mix else None)

    def in_params(self):
        return [self.qkv]

    def in_bias(self):
        return self.qkv_bias

    def cos_sin(self, device) -> Optional[torch.Tensor]:
        sp = self.spec
        if not sp.rope:
            return None
        cs = self._cos_sin
        if cs is None or cs.device != device:
            cs = ops.rope_table(self.max_pos, sp.rot_dims, sp.rot_base,
                                device, sp.rot_factor, sp.rot_scaling)
            self._cos_sin = cs
        return cs

    def project(self, o: torch.Tensor) -> torch.Tensor:
        if self.out_bias is not None:
            return torch.addmm(self.out_bias, o, self.out_weight.t())
        return gemm_policy.linear(o, self.out_weight)

    def forward(self, h: torch.Tensor, meta, cache, shared: dict,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self.qkv_bias is not None:
            # the bias joins the fp32 accumulator of the projection
            proj = torch.addmm(self.qkv_bias, h, self.qkv.t())
        else:
            proj = gemm_policy.linear(h, self.qkv)
        return self.forward_from_proj(proj, meta, cache, out, shared)

    @property
    def out_in(self) -> int:
        return self.H * self.DV

    def cache_shape(self):
        if self.spec.window_pool:
            return ("kvpool", self.G, self.D, self.DV,
                    self.spec.window_pool)
        return ("kv", self.G, self.D, self.DV)

    def forward_from_proj(self, proj: torch.Tensor, meta, cache,
                          out: Optional[torch.Tensor] = None,
                          shared: Optional[dict] = None) -> torch.Tensor:
        H, G, D, DV = self.H, self.G, self.D, self.DV
        sp = self.spec
        pool = None
        if sp.window_pool:
            k_cache, v_cache, kp_cache, vp_cache = cache
            pool = (kp_cache, vp_cache, sp.window_pool)
        else:
            k_cache, v_cache = cache
        q = proj[:, :H * D]
        k = proj[:, H * D:H * D + G * D]
        v = proj[:, H * D + G * D:self.qkv_rows]
        if sp.qk_norm or sp.qk_norm_all or sp.v_mix or sp.rope:
            # the first value-mixing layer of a step publishes its values;
            # later ones blend theirs with them before caching
            v_first = shared.get("v_first") if sp.v_mix else None
            ops.attn_prep(q, k, v, self.q_norm, self.k_norm, self.eps,
                          self.vmix, v_first, k_cache, v_cache,
                          meta.slot_mapping, H,
                          cos_sin=self.cos_sin(proj.device),
                          positions=meta.positions,
                          rot_dims=sp.rot_dims if sp.rope else 0,
                          norm_all=sp.qk_norm_all,
                          half=sp.rot_layout == "half")
            if sp.v_mix and v_first is None:
                shared["v_first"] = v
        else:
            ops.kv_append(k, v, k_cache, v_cache, meta.slot_mapping)
        T = proj.shape[0]
        if pool is not None:
            # blocks completed by this step's keys
            ops.pool_append(k_cache, v_cache, kp_cache, vp_cache,
                            meta.block_tables, meta.seq_rows,
                            sp.window_pool, T)
        if out is None:
            out = torch.empty((T, H * DV), dtype=proj.dtype,
                              device=proj.device)
        # batch rows: multi-token prompt portions first, single tokens
        # after them. Portions share key tiles between neighbouring rows
        # (tiled kernel); single tokens of different sequences share
        # nothing and take the split-key kernel, one workgroup per token.
        npt = min(getattr(meta, "num_prefill_tokens", T) or 0, T)
        for a, b, variant in ((0, npt, 0), (npt, T, 3)):
            if b > a:
                ops.talk_attention(
                    q[a:b], k_cache, v_cache, meta.block_tables,
                    meta.token_seq[a:b], meta.positions[a:b], self.scale, H,
                    chunk=sp.chunk, window=sp.window, sink=sp.sink,
                    talk=self.talk, out=out[a:b], variant=variant,
                    keep_first=sp.keep_first, softcap=sp.softcap,
                    sink_vals=self.sink_vals, pool=pool)
        if sp.out_gate:
            ops.gated_act(proj[:, self.qkv_rows:], out, "sigmoid", out=out)
        return out


class LatentAttention(nn.Module):
    """Multi-head attention whose keys and values are low-rank expansions
    of one cached latent per token. Per head the query has `dim`
    position-free entries and `rot_dim` rotary ones; the key's rotary part
    is one vector shared by all heads. The per-head up-projections are
    folded around the attention: the position-free query part is mapped
    into the latent space (q W_uk), attention runs as single-KV-head
    attention over cached rows [latent | rotary key part] whose values are
    the latent itself, and the result is expanded by W_uv. Only
    kv_rank + rot_dim numbers per token are cached."""

    kind = "latent_attention"

    def __init__(self, width: int, spec: MixerSpec, dtype: torch.dtype,
                 eps: float, max_pos: int) -> None:
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.max_pos = max_pos
        H, D, R, L = spec.heads, spec.dim, spec.rot_dim, spec.kv_rank
        DV = spec.vdim or D
        self.H, self.D, self.R, self.L, self.DV = H, D, R, L, DV
        # fused rows: q (per head [dim | rot_dim]) | latent | rotary key
        self.in_proj = nn.Parameter(
            torch.empty(H * (D + R) + L + R, width, dtype=dtype))
        self.latent_norm = nn.Parameter(torch.empty(L, dtype=torch.float32))
        self.uk = nn.Parameter(torch.empty(H, D, L, dtype=dtype))
        self.uv = nn.Parameter(torch.empty(H, DV, L, dtype=dtype))
        self.sink_vals = (
            nn.Parameter(torch.empty(H, dtype=torch.float32))
            if spec.learned_sink else None)
        self.out_weight = nn.Parameter(
            torch.empty(width, H * DV, dtype=dtype))
        self.scale = spec.scale or 1.0 / math.sqrt(D + R)
        self._cos_sin = None

    def in_params(self):
        return [self.in_proj]

    @property
    def out_in(self) -> int:
        return self.H * self.DV

    def cache_shape(self):
        return ("paged", 1, self.L + self.R)

    def cos_sin(self, device) -> torch.Tensor:
        cs = self._cos_sin
        if cs is None or cs.device != device:
            sp = self.spec
            cs = ops.rope_table(self.max_pos, sp.rot_dims or self.R,
                                sp.rot_base, device)
            self._cos_sin = cs
        return cs

    def forward(self, h: torch.Tensor, meta, cache, shared: dict,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        H, D, R, L, DV = self.H, self.D, self.R, self.L, self.DV
        sp = self.spec
        T = h.shape[0]
        proj = gemm_policy.linear(h, self.in_proj)
        q = proj[:, :H * (D + R)]
        dkv = proj[:, H * (D + R):]
        # position-free query part into the latent space: [H, T, L]
        q_lat = torch.bmm(q.view(T, H, D + R)[:, :, :D].transpose(0, 1),
                          self.uk)
        qf = ops.latent_prep(
            q_lat, q, dkv, self.latent_norm, self.eps,
            self.cos_sin(h.device), meta.positions, cache,
            meta.slot_mapping, H, D, R, sp.rot_dims or R)
        o_lat = torch.empty((T, H * L), dtype=h.dtype, device=h.device)
        npt = min(getattr(meta, "num_prefill_tokens", T) or 0, T)
        for a, b, variant in ((0, npt, 0), (npt, T, 3)):
            if b > a:
                ops.talk_attention(
                    qf[a:b], cache, cache, meta.block_tables,
                    meta.token_seq[a:b], meta.positions[a:b], self.scale, H,
                    sink=sp.sink, out=o_lat[a:b], variant=variant,
                    softcap=sp.softcap, sink_vals=self.sink_vals, vdim=L)
        # expand the attended latents per head: [H, T, L] x [H, L, DV]
        o = torch.bmm(o_lat.view(T, H, L).transpose(0, 1),
                      self.uv.transpose(1, 2))
        o = o.transpose(0, 1).reshape(T, H * DV)
        if out is not None:
            out.copy_(o)
            return out
        return o


class GeneralDelta(nn.Module):
    """Gated delta-rule linear recurrence ("generalized delta rule"): per
    head a dim x dim fp32 state with a per-channel data-dependent decay
    (low-rank projection) and a per-channel removal gate along the unit
    key; the read-out is RMS-normalised per head, channel-scaled and
    gated. State lives in a per-sequence slot of the runner's state
    cache."""

    kind = "general_delta"

    def __init__(self, width: int, spec: MixerSpec, eps: float,
                 dtype: torch.dtype) -> None:
        super().__init__()
        self.spec = spec
        self.eps = eps
        H, D, R = spec.heads, spec.dim, spec.decay_rank
        self.H, self.D, self.R = H, D, R
        HD = H * D
        # fused rows: r | k | v | g | a | w1
        self.in_proj = nn.Parameter(torch.empty(5 * HD + R, width,
                                                dtype=dtype))
        self.w2 = nn.Parameter(torch.empty(HD, R, dtype=dtype))
        self.w0 = nn.Parameter(torch.empty(HD, dtype=torch.float32))
        self.a_bias = nn.Parameter(torch.empty(HD, dtype=torch.float32))
        self.out_norm = nn.Parameter(torch.empty(HD, dtype=torch.float32))
        self.out_weight = nn.Parameter(torch.empty(width, HD, dtype=dtype))

    def in_params(self):
        return [self.in_proj]

    @property
    def out_in(self) -> int:
        return self.H * self.D

    def cache_shape(self):
        return ("state", self.H, self.D, self.D)

    def forward_from_proj(self, proj: torch.Tensor, meta, cache,
                          out: Optional[torch.Tensor] = None
                          ) -> torch.Tensor:
        HD = self.H * self.D
        r = proj[:, 0:HD]
        k = proj[:, HD:2 * HD]
        v = proj[:, 2 * HD:3 * HD]
        g = proj[:, 3 * HD:4 * HD]
        za = proj[:, 4 * HD:5 * HD]
        zw = gemm_policy.linear(torch.tanh(proj[:, 5 * HD:]), self.w2)
        return ops.delta_rule(
            r, k, v, zw, za, g, self.w0, self.a_bias, self.out_norm, cache,
            meta.seq_rows, self.H, self.eps, DELTA_DECAY_SCALE, out=out)


class ChannelDelta(nn.Module):
    """Gated delta rule with one decay per head and key channel. q, k
    (kv_heads x dim, shared by groups of heads) and v (heads x vdim) pass a
    short causal convolution and silu; q and k become unit vectors; the
    decay exp(-exp(A_log) softplus(.)) and the output gate come from
    low-rank projections, the write strength from a per-head sigmoid. The
    read-out is RMS-normalised per head and gated. Per sequence the runner
    keeps the fp32 state heads x dim x vdim and the convolution's last
    taps - 1 inputs."""

    kind = "channel_delta"

    def __init__(self, width: int, spec: MixerSpec, eps: float,
                 dtype: torch.dtype) -> None:
        super().__init__()
        self.spec = spec
        self.eps = eps
        H, G = spec.heads, spec.kv_heads or spec.heads
        D, DV = spec.dim, spec.vdim or spec.dim
        if H % G:
            raise ValueError("heads must be a multiple of kv_heads")
        self.H, self.G, self.D, self.DV = H, G, D, DV
        self.K = max(int(spec.conv), 1)
        ra, rg = spec.decay_rank, spec.gate_rank
        self.ra, self.rg = ra, rg
        self.C = 2 * G * D + H * DV          # convolved channels q | k | v
        # fused rows: q | k | v | write strength | decay rank | gate rank
        self.in_proj = nn.Parameter(
            torch.empty(self.C + H + ra + rg, width, dtype=dtype))
        self.conv_w = nn.Parameter(
            torch.empty(self.C, self.K, dtype=torch.float32))
        self.a2 = nn.Parameter(torch.empty(H * D, ra, dtype=dtype))
        self.g2 = nn.Parameter(torch.empty(H * DV, rg, dtype=dtype))
        self.a_log = nn.Parameter(torch.empty(H, dtype=torch.float32))
        self.dt_bias = nn.Parameter(torch.empty(H * D, dtype=torch.float32))
        self.out_norm = nn.Parameter(torch.empty(DV, dtype=torch.float32))
        self.out_weight = nn.Parameter(
            torch.empty(width, H * DV, dtype=dtype))

    def in_params(self):
        return [self.in_proj]

    @property
    def out_in(self) -> int:
        return self.H * self.DV

    def cache_shape(self):
        return ("multi", [("state", self.H, self.D, self.DV),
                          ("slots", (self.K - 1, self.C), None)])

    def forward(self, h: torch.Tensor, meta, cache, shared: dict,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        H, G, D, DV, C = self.H, self.G, self.D, self.DV, self.C
        state, conv_state = cache
        proj = gemm_policy.linear(h, self.in_proj)
        qkv = ops.short_conv_silu(proj[:, :C], self.conv_w, conv_state,
                                  meta.seq_rows)
        beta = proj[:, C:C + H]
        zdec = gemm_policy.linear(proj[:, C + H:C + H + self.ra], self.a2)
        zgate = gemm_policy.linear(proj[:, C + H + self.ra:], self.g2)
        return ops.gated_delta(
            qkv[:, :G * D], qkv[:, G * D:2 * G * D], qkv[:, 2 * G * D:],
            beta, zdec, zgate, self.a_log, self.dt_bias, self.out_norm,
            state, meta.seq_rows, H, G, self.eps, out=out)


class _ScanMixer(nn.Module):
    """Shared plumbing of the gated linear recurrences: one fused input
    projection, a per-sequence fp32 state heads x dim x vdim, one output
    projection."""

    def in_params(self):
        return [self.in_proj]

    def in_bias(self):
        return None

    @property
    def out_in(self) -> int:
        return self.H * self.DV

    def project(self, o: torch.Tensor) -> torch.Tensor:
        return gemm_policy.linear(o, self.out_weight)

    def forward(self, h: torch.Tensor, meta, cache, shared: dict,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self.forward_from_proj(gemm_policy.linear(h, self.in_proj),
                                      meta, cache, out)


class GatedLinearAttention(_ScanMixer):
    """Linear attention whose state rows decay per key channel:
    alpha = sigmoid(W_a2 W_a1 h + b)^(1/tau), S <- diag(alpha) S + k v^T,
    o = S^T (q dim^-1/2); o is RMS-normalised per head (weight shared by
    the heads) and multiplied by silu(W_g h)."""

    kind = "gla"

    def __init__(self, width: int, spec: MixerSpec, eps: float,
                 dtype: torch.dtype) -> None:
        super().__init__()
        self.spec, self.eps = spec, eps
        H, D, DV = spec.heads, spec.dim, spec.vdim or spec.dim
        self.H, self.D, self.DV, self.R = H, D, DV, spec.decay_rank
        # fused rows: q | k | v | output gate | decay rank
        self.in_proj = nn.Parameter(torch.empty(
            2 * H * D + 2 * H * DV + self.R, width, dtype=dtype))
        self.a2 = nn.Parameter(torch.empty(H * D, self.R, dtype=dtype))
        self.a_bias = nn.Parameter(torch.empty(H * D, dtype=torch.float32))
        self.out_norm = nn.Parameter(torch.empty(DV, dtype=torch.float32))
        self.out_weight = nn.Parameter(
            torch.empty(width, H * DV, dtype=dtype))

    def cache_shape(self):
        return ("state", self.H, self.D, self.DV)

    def forward_from_proj(self, proj, meta, cache, out=None):
        H, D, DV = self.H, self.D, self.DV
        a, b, c = H * D, 2 * H * D, 2 * H * D + H * DV
        z = gemm_policy.linear(proj[:, c + H * DV:], self.a2)
        return ops.linear_scan(
            "gla", proj[:, :a], proj[:, a:b], proj[:, b:c], z,
            proj[:, c:c + H * DV], cache, meta.seq_rows, H, H, self.eps,
            qscale=D ** -0.5, c0=1.0 / self.spec.tau, p0=self.a_bias,
            normw=self.out_norm, out=out)


class MatrixLSTM(_ScanMixer):
    """Matrix-memory LSTM: per head log gates i = cap(W_i h + b_i),
    f = logsigmoid(cap(W_f h + b_f)), cap(z) = c tanh(z / c); with the
    running maximum m' = max(f + m, i) (m starts at 0) the memory and its
    normaliser are S <- e^(f+m-m') S + e^(i-m') k v^T, n likewise with k;
    o = S^T q / (max(|n.q|, e^-m') + 1e-6), q scaled by dim^-1/2; o is
    divided by its per-head root mean square, scaled by a weight over all
    heads and by sigmoid(W_g h). Per sequence: S plus (n, m)."""

    kind = "mlstm"

    def __init__(self, width: int, spec: MixerSpec, eps: float,
                 dtype: torch.dtype) -> None:
        super().__init__()
        self.spec, self.eps = spec, eps
        H, D, DV = spec.heads, spec.dim, spec.vdim or spec.dim
        self.H, self.D, self.DV = H, D, DV
        # fused rows: q | k | v | output gate | input gate | forget gate
        self.in_proj = nn.Parameter(torch.empty(
            2 * H * D + 2 * H * DV + 2 * H, width, dtype=dtype))
        self.i_bias = nn.Parameter(torch.empty(H, dtype=torch.float32))
        self.f_bias = nn.Parameter(torch.empty(H, dtype=torch.float32))
        self.out_norm = nn.Parameter(torch.empty(H * DV,
                                                 dtype=torch.float32))
        self.out_weight = nn.Parameter(
            torch.empty(width, H * DV, dtype=dtype))

    def cache_shape(self):
        return ("multi", [("state", self.H, self.D, self.DV),
                          ("slots", (self.H, self.D + 1), torch.float32)])

    def forward_from_proj(self, proj, meta, cache, out=None):
        H, D, DV = self.H, self.D, self.DV
        a, b, c = H * D, 2 * H * D, 2 * H * D + H * DV
        e = c + H * DV
        state, aux = cache
        return ops.linear_scan(
            "mlstm", proj[:, :a], proj[:, a:b], proj[:, b:c],
            proj[:, e + H:e + 2 * H], proj[:, c:e], state, meta.seq_rows,
            H, H, self.eps, qscale=D ** -0.5, c0=self.spec.gate_cap,
            wr=proj[:, e:e + H], p0=self.i_bias, p1=self.f_bias,
            normw=self.out_norm, aux=aux, out=out)


class StateSpaceDuality(_ScanMixer):
    """State-space-duality mixer (scalar decay per head): the input
    projection gives z | x | B | C | dt; x, B, C pass a short causal
    convolution (with bias) and silu; dt = softplus(dt + dt_bias);
    S <- exp(-exp(A_log) dt) S + dt B x^T (state x vdim per head, B and C
    shared by groups of heads), y = S^T C + D x; y silu(z) is RMS-normalised
    in `norm_groups` equal parts and scaled. Per sequence: S and the
    convolution's last taps - 1 inputs."""

    kind = "ssd"

    def __init__(self, width: int, spec: MixerSpec, eps: float,
                 dtype: torch.dtype) -> None:
        super().__init__()
        self.spec, self.eps = spec, eps
        H, DV, N = spec.heads, spec.vdim or spec.dim, spec.state or spec.dim
        G = spec.groups or 1
        if H % G:
            raise ValueError("heads must be a multiple of groups")
        self.H, self.DV, self.N, self.G = H, DV, N, G
        self.D = N
        self.K = max(int(spec.conv), 1)
        inner = H * DV
        if inner % max(spec.norm_groups, 1):
            raise ValueError("norm_groups must divide heads * vdim")
        self.inner = inner
        self.C = inner + 2 * G * N        # convolved channels x | B | C
        self.in_proj = nn.Parameter(
            torch.empty(inner + self.C + H, width, dtype=dtype))
        self.conv_w = nn.Parameter(
            torch.empty(self.C, self.K, dtype=torch.float32))
        self.conv_b = nn.Parameter(torch.empty(self.C, dtype=torch.float32))
        self.dt_bias = nn.Parameter(torch.empty(H, dtype=torch.float32))
        self.a_log = nn.Parameter(torch.empty(H, dtype=torch.float32))
        self.d_skip = nn.Parameter(torch.empty(H, dtype=torch.float32))
        self.out_norm = nn.Parameter(torch.empty(inner, dtype=torch.float32))
        self.out_weight = nn.Parameter(
            torch.empty(width, inner, dtype=dtype))

    def cache_shape(self):
        return ("multi", [("state", self.H, self.N, self.DV),
                          ("slots", (self.K - 1, self.C), None)])

    def forward_from_proj(self, proj, meta, cache, out=None):
        H, G, N, inner, C = self.H, self.G, self.N, self.inner, self.C
        state, conv_state = cache
        xbc = ops.short_conv_silu(proj[:, inner:inner + C], self.conv_w,
                                  conv_state, meta.seq_rows,
                                  bias=self.conv_b)
        y32 = ops.linear_scan(
            "ssd", xbc[:, inner + G * N:], xbc[:, inner:inner + G * N],
            xbc[:, :inner], proj[:, inner + C:inner + C + H],
            proj[:, :inner], state, meta.seq_rows, H, G, self.eps,
            p0=self.dt_bias, p1=self.a_log, p2=self.d_skip)
        y = ops.add_rms_norm32(y32, [], self.out_norm, self.eps, proj.dtype,
                               max(self.spec.norm_groups, 1))
        if out is not None:
            out.copy_(y)
            return out
        return y


class MinGRU(_ScanMixer):
    """Minimal gated recurrent unit: an element-wise recurrence over
    `vdim` channels whose gate and candidate read the current token only,
    S <- (1 - z) S + z c with z = sigmoid(W_z h + b_z), u = W_x h + b_x,
    c = u + 1/2 for u >= 0 and sigmoid(u) below; the read-out is
    S silu(W_g h). Per sequence: S in fp32."""

    kind = "mingru"

    def __init__(self, width: int, spec: MixerSpec, eps: float,
                 dtype: torch.dtype) -> None:
        super().__init__()
        self.spec, self.eps = spec, eps
        C = spec.vdim or spec.dim
        self.H, self.D, self.DV, self.C = 1, 1, C, C
        # fused rows: gate | candidate | read-out gate
        self.in_proj = nn.Parameter(torch.empty(3 * C, width, dtype=dtype))
        self.z_bias = nn.Parameter(torch.empty(C, dtype=torch.float32))
        self.x_bias = nn.Parameter(torch.empty(C, dtype=torch.float32))
        self.out_weight = nn.Parameter(torch.empty(width, C, dtype=dtype))

    def cache_shape(self):
        return ("slots", (self.C,), torch.float32)

    def forward_from_proj(self, proj, meta, cache, out=None):
        C = self.C
        return ops.mingru_scan(proj[:, :C], proj[:, C:2 * C],
                               proj[:, 2 * C:3 * C], self.z_bias,
                               self.x_bias, cache, meta.seq_rows, out=out)


class MixerPair(nn.Module):
    """Two mixers fed the same input. `combine` "norm_mean": each half's
    projected output is RMS-normalised over the model width with its own
    weight and the result is their mean (fp32); "weighted": the result is
    left_scale * left + right_scale * right, which the caller's boundary
    kernel adds to the stream in fp32 (forward_parts). Both input
    projections are one GEMM."""

    kind = "pair"

    def __init__(self, width: int, spec: MixerSpec, eps: float,
                 dtype: torch.dtype, max_pos: int) -> None:
        super().__init__()
        self.spec, self.eps = spec, eps
        self.left = build_mixer(width, spec.left, eps, dtype, max_pos)
        self.right = build_mixer(width, spec.right, eps, dtype, max_pos)
        if spec.combine not in ("norm_mean", "weighted"):
            raise ValueError(f"unknown pair combine {spec.combine!r}")
        self.left_norm = self.right_norm = None
        if spec.combine == "norm_mean":
            self.left_norm = nn.Parameter(torch.empty(width,
                                                      dtype=torch.float32))
            self.right_norm = nn.Parameter(torch.empty(width,
                                                       dtype=torch.float32))
        self._fused = None

    def cache_shape(self):
        return ("multi", [self.left.cache_shape(),
                          self.right.cache_shape()])

    def _apply(self, fn, *a, **kw):
        self._fused = None
        return super()._apply(fn, *a, **kw)

    def fuse(self):
        """[left rows | right rows] of the input projections as one weight
        (the halves' parameters become views of it) and one bias (zeros
        where a half has none; None when neither has one)."""
        parts = list(self.left.in_params()) + list(self.right.in_params())
        w = torch.cat([p.data for p in parts], dim=0).contiguous()
        off = 0
        for p in parts:
            p.data = w[off:off + p.shape[0]]
            off += p.shape[0]
        n_left = sum(p.shape[0] for p in self.left.in_params())
        bias = None
        bl, br = self.left.in_bias(), self.right.in_bias()
        if bl is not None or br is not None:
            bias = torch.zeros(w.shape[0], dtype=w.dtype, device=w.device)
            if bl is not None:
                bias[:n_left] = bl.data
            if br is not None:
                bias[n_left:] = br.data
        self._fused = (w, bias, n_left)
        return self._fused

    def project(self, o: torch.Tensor) -> torch.Tensor:
        return o

    def forward_parts(self, h: torch.Tensor, meta, cache, shared: dict):
        """The halves' projected outputs (left, right)."""
        w, bias, n_left = self._fused or self.fuse()
        proj = (torch.addmm(bias, h, w.t()) if bias is not None
                else gemm_policy.linear(h, w))
        a = self.left.project(self.left.forward_from_proj(
            proj[:, :n_left], meta, cache[0], None, shared))
        b = self.right.project(self.right.forward_from_proj(
            proj[:, n_left:], meta, cache[1]))
        return a, b

    def forward(self, h: torch.Tensor, meta, cache, shared: dict,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        a, b = self.forward_parts(h, meta, cache, shared)
        if self.spec.combine == "weighted":
            return (a.float() * self.spec.left_scale
                    + b.float() * self.spec.right_scale)
        return ops.norm_sum32([a, b], [self.left_norm, self.right_norm],
                              0.5, self.eps)


def build_mixer(width: int, spec: MixerSpec, eps: float,
                dtype: torch.dtype, max_pos: int = 8192) -> nn.Module:
    if spec.kind == "attention":
        return TalkAttention(width, spec, dtype, eps, max_pos)
    if spec.kind == "gla":
        return GatedLinearAttention(width, spec, eps, dtype)
    if spec.kind == "mlstm":
        return MatrixLSTM(width, spec, eps, dtype)
    if spec.kind == "ssd":
        return StateSpaceDuality(width, spec, eps, dtype)
    if spec.kind == "mingru":
        return MinGRU(width, spec, eps, dtype)
    if spec.kind == "pair":
        return MixerPair(width, spec, eps, dtype, max_pos)
    if spec.kind == "latent_attention":
        return LatentAttention(width, spec, dtype, eps, max_pos)
    if spec.kind == "general_delta":
        return GeneralDelta(width, spec, eps, dtype)
    if spec.kind == "channel_delta":
        return ChannelDelta(width, spec, eps, dtype)
    raise ValueError(f"unknown mixer kind {spec.kind!r}")
