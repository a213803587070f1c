"""Op dispatch layer.

On a GPU (any tensor on `cuda`), every op REQUIRES the in-tree HIP extension
production_stack_amd._C and raises if it is missing -- there is no silent
eager fallback on MI355X. On CPU tensors the pure-PyTorch references run so
the engine and its tests work in GPU-less CI.
"""

from __future__ import annotations

import os

import torch

from production_stack_amd.ops import reference

try:
    from production_stack_amd import _C  # type: ignore[attr-defined]
except ImportError:  # pragma: no cover - exercised only when not built
    _C = None

HAVE_EXT = _C is not None


def _require_ext() -> None:
    if _C is None:
        raise RuntimeError(
            "production_stack_amd._C HIP extension is not built; run "
            "`PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace`. "
            "Refusing to fall back to eager PyTorch on GPU."
        )


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    if x.is_cuda:
        _require_ext()
        out = torch.empty_like(x)
        _C.rms_norm(out, x, w, eps)
        return out
    return reference.rms_norm(x, w, eps)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor, eps: float
) -> tuple[torch.Tensor, torch.Tensor]:
    """In-place on GPU: x <- normed(residual + x); residual <- residual + x."""
    if x.is_cuda:
        _require_ext()
        _C.fused_add_rms_norm(x, residual, w, eps)
        return x, residual
    normed, summed = reference.fused_add_rms_norm(x, residual, w, eps)
    return normed, summed


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    if x.is_cuda:
        _require_ext()
        d = x.shape[-1] // 2
        out = torch.empty(x.shape[:-1] + (d,), dtype=x.dtype, device=x.device)
        _C.silu_and_mul(out, x)
        return out
    return reference.silu_and_mul(x)


def rotary_embedding(
    positions: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    cos_sin: torch.Tensor,
    head_dim: int,
) -> tuple[torch.Tensor, torch.Tensor]:
    """In-place on GPU. positions int32, q/k bf16 [T, H*HD], cos_sin fp32."""
    if q.is_cuda:
        _require_ext()
        _C.rotary_embedding(positions, q, k, cos_sin, head_dim)
        return q, k
    return reference.rotary_embedding(positions, q, k, cos_sin, head_dim)


def fused_rope_cache(
    qkv: torch.Tensor,
    positions: torch.Tensor,
    cos_sin: torch.Tensor,
    slot_mapping: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    q_heads: int,
    head_dim: int,
) -> None:
    """Fused in-place RoPE on packed qkv + paged KV append (GPU only)."""
    _require_ext()
    _C.fused_rope_cache(
        qkv, positions, cos_sin, slot_mapping, k_cache, v_cache, q_heads,
        head_dim,
    )


def reshape_and_cache(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    if k_cache.is_cuda:
        _require_ext()
        _C.reshape_and_cache(
            k.view(k.shape[0], -1), v.view(v.shape[0], -1), k_cache, v_cache,
            slot_mapping,
        )
        return
    reference.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)


def paged_attn_decode(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    if q.is_cuda:
        _require_ext()
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        # variant 1 = low-register packed-q kernel (3 waves/SIMD): measured
        # +17-26% over variant 0 across batch/ctx (profiles/attn_bench).
        _C.paged_attn_decode(
            out, q, k_cache, v_cache, block_tables, seq_lens, scale, 0, 1,
            window
        )
        return out
    return reference.paged_attn_decode(
        q, k_cache, v_cache, block_tables, seq_lens, scale, window
    )


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
    if q.is_cuda:
        _require_ext()
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        _C.paged_attn_prefill(
            out, q, k_cache, v_cache, block_tables, token_seq, token_pos,
            scale, window
        )
        return out
    return reference.paged_attn_prefill(
        q, k_cache, v_cache, block_tables, token_seq, token_pos, scale,
        window
    )


# Default MFMA prefill variant: 5 = 8-wave 32x32 swapped-QK^T kernel
# (csrc/prefill_mfma32.hip); 3/4 = the 4-wave 16x16 kernel (64-row
# tiles). Overridable for A/B via PS_PREFILL_VARIANT.
PREFILL_VARIANT = int(os.environ.get("PS_PREFILL_VARIANT", "5"))


def prefill_tile_rows(num_q_heads: int, num_kv_heads: int) -> int:
    """Prefill tile row count for the active kernel. v5 splits its 8 waves
    into GQW head-columns x row-halves (GQW = largest pow2 divisor of the
    GQA ratio, <=4), so tiles carry 32*(8/GQW) rows (64..256)."""
    if PREFILL_VARIANT != 5:
        return 64
    gq = max(1, num_q_heads // max(1, num_kv_heads))
    gqw = 1
    while gqw < 4 and gq % (gqw * 2) == 0:
        gqw *= 2
    return 32 * (8 // gqw)


def paged_attn_prefill_mfma(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    tile_info: torch.Tensor,
    scale: float,
    window: int = 0,
    variant: int = None,
) -> torch.Tensor:
    """MFMA-tiled chunked prefill (GPU, head_dim 128 only). tile_info rows
    must be built with n_rows <= prefill_tile_rows() for the active
    variant."""
    _require_ext()
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    # v5's split-KV (up to 8 kv-splits) keeps CUs filled at small
    # serving launches, where it now beats v3 at the canonical shapes
    # (12-seq x 200-row continuation at hist 4600: 305 vs 263 TF; fresh
    # 900-row prefill: 400 vs 306) as well as at large ones — so v5 is
    # the default everywhere (PS_PREFILL_VARIANT=3 restores the 4-wave
    # kernel for A/B).
    v = PREFILL_VARIANT if variant is None else variant
    _C.paged_attn_prefill_mfma(
        out, q, k_cache, v_cache, block_tables, tile_info, scale, v, window
    )
    return out


def greedy_sample(logits: torch.Tensor) -> torch.Tensor:
    if logits.is_cuda:
        # fp32 rows (penalty-adjusted, or families that emit fp32 logits)
        # need no extension kernel
        if logits.dtype != torch.bfloat16:
            return logits.float().argmax(dim=-1)
        _require_ext()
        out = torch.empty(
            logits.shape[0], dtype=torch.long, device=logits.device
        )
        _C.greedy_sample(out, logits)
        return out
    return reference.greedy_sample(logits)


def kv_quant(x: torch.Tensor) -> tuple:
    """Row-wise int8 KV quantization (CacheGen-style serde)."""
    if x.is_cuda:
        _require_ext()
        hd = x.shape[-1]
        out = torch.empty(x.shape, dtype=torch.int8, device=x.device)
        scales = torch.empty(
            x.numel() // hd, dtype=torch.float32, device=x.device
        )
        _C.kv_quant(out, scales, x)
        return out, scales
    return reference.kv_quant(x)


def kv_dequant(
    q: torch.Tensor, scales: torch.Tensor, dtype=torch.bfloat16
) -> torch.Tensor:
    if q.is_cuda:
        _require_ext()
        out = torch.empty(q.shape, dtype=dtype, device=q.device)
        _C.kv_dequant(out, q, scales)
        return out
    return reference.kv_dequant(q, scales, dtype)


def skinny_gemm(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """out = x @ w.T for decode-shaped M<=128 (weight-stream-bound GEMMs
    where hipBLASLt tiles poorly — see csrc/skinny_gemm.hip). GPU only."""
    _require_ext()
    out = torch.empty(
        (x.shape[0], w.shape[0]), dtype=torch.bfloat16, device=x.device
    )
    _C.skinny_gemm(out, x, w)  # split-K partials + combine (no atomics)
    return out


def cachegen_encode(q: torch.Tensor) -> torch.Tensor:
    """Entropy-encode int8 KV (CPU adaptive range coder, per-channel
    contexts). Falls back to a pure-Python reference when the extension
    is unavailable (CPU CI)."""
    if _C is not None and hasattr(_C, "cachegen_encode"):
        return _C.cachegen_encode(q.contiguous().cpu())
    return reference.cachegen_encode(q)


def cachegen_decode(blob: torch.Tensor, hd: int) -> torch.Tensor:
    if _C is not None and hasattr(_C, "cachegen_decode"):
        return _C.cachegen_decode(blob.contiguous().cpu(), hd)
    return reference.cachegen_decode(blob, hd)


def gemm8p(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """out = x @ w.T via the 8-phase deep-pipelined MFMA GEMM
    (csrc/gemm8p.hip; 256x256 tiles + split-K for skinny M). GPU only."""
    _require_ext()
    out = torch.empty(
        (x.shape[0], w.shape[0]), dtype=torch.bfloat16, device=x.device
    )
    _C.gemm8p(out, x, w)
    return out


def lora_bgmv(
    out: torch.Tensor,
    x: torch.Tensor,
    A: torch.Tensor,
    B: torch.Tensor,
    scale: torch.Tensor,
    idx: torch.Tensor,
    col_off: int = 0,
) -> None:
    """out[t, col_off:+W] += scale[idx[t]] * B[idx[t]] @ (A[idx[t]] @ x[t]);
    idx[t] < 0 skips the row. hipGraph-safe (static shapes, no host sync)."""
    if out.is_cuda:
        _require_ext()
        _C.lora_bgmv(out, x, A, B, scale, idx, col_off)
        return
    reference.lora_bgmv(out, x, A, B, scale, idx, col_off)


def fp8_linear(
    x: torch.Tensor, w_q: torch.Tensor, w_scale: torch.Tensor
) -> torch.Tensor:
    """out = x @ (w_q * w_scale)^T with fp8 tensor cores.

    Weights are stored OCP fp8-e4m3 with a per-tensor scale; activations
    quantize dynamically per call (per-tensor amax / 448). On gfx950 this
    runs through hipBLASLt's fp8 MFMA path (torch._scaled_mm) at ~1.8x
    the bf16 GEMM rate for decode shapes. CPU fallback dequantizes.
    """
    if x.is_cuda:
        sx = (x.abs().amax().clamp(min=1e-6) / 448.0).to(torch.float32)
        xq = (x / sx).to(torch.float8_e4m3fn)
        if w_scale.dim() == 1:  # per-channel weight scales
            return fp8_linear_rowwise(
                xq, sx.expand(x.shape[0]), w_q, w_scale)
        return torch._scaled_mm(
            xq, w_q.t(), scale_a=sx, scale_b=w_scale,
            out_dtype=torch.bfloat16,
        )
    wf = w_q.float() * (
        w_scale.float()[:, None] if w_scale.dim() == 1
        else w_scale.float()
    )
    return torch.nn.functional.linear(x.float(), wf).to(x.dtype)


def fp8_quantize_weight(w: torch.Tensor):
    """Per-tensor weight quantization: returns (w_q fp8, scale f32)."""
    scale = (w.abs().amax().float().clamp(min=1e-6) / 448.0)
    w_q = (w.float() / scale).clamp(-448, 448).to(torch.float8_e4m3fn)
    return w_q, scale


def fp8_quantize_weight_rowwise(w: torch.Tensor):
    """Per-output-channel weight quantization: (w_q fp8 [N,K], scales
    [N] f32) — finer than per-tensor, same GEMM cost with rowwise-scaled
    fp8 matmul."""
    scales = (w.abs().amax(dim=1).float().clamp(min=1e-6) / 448.0)
    w_q = (w.float() / scales[:, None]).clamp(-448, 448).to(
        torch.float8_e4m3fn)
    return w_q, scales


def rms_norm_fp8(x, w, eps, residual=None):
    """Fused (add-)RMSNorm emitting fp8-e4m3 rows + per-row scales. When
    `residual` is given it is updated in place (residual += x) like
    fused_add_rms_norm. GPU only."""
    _require_ext()
    T, D = x.shape
    out_q = torch.empty((T, D), dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty(T, dtype=torch.float32, device=x.device)
    _C.rms_norm_fp8(out_q, scales, x,
                    residual if residual is not None else x, w, eps,
                    1 if residual is not None else 0)
    return out_q, scales


def silu_and_mul_fp8(x):
    _require_ext()
    T, D2 = x.shape
    out_q = torch.empty((T, D2 // 2), dtype=torch.float8_e4m3fn,
                        device=x.device)
    scales = torch.empty(T, dtype=torch.float32, device=x.device)
    _C.silu_and_mul_fp8(out_q, scales, x)
    return out_q, scales


_ROWWISE_SCALED_MM = None  # probed once: does _scaled_mm accept [M,1]x[1,N]?


def fp8_rowwise_supported(device="cuda") -> bool:
    """Whether this build's _scaled_mm takes rowwise scales. When it does
    not, the fused per-row act-quant path would need a slow fp32-out
    fallback, so callers keep the per-tensor fp8 pipeline instead."""
    global _ROWWISE_SCALED_MM
    if _ROWWISE_SCALED_MM is None:
        try:
            torch._scaled_mm(
                torch.zeros(16, 32, dtype=torch.float8_e4m3fn,
                            device=device),
                torch.zeros(32, 16, dtype=torch.float8_e4m3fn,
                            device=device),
                scale_a=torch.ones(16, 1, device=device),
                scale_b=torch.ones(1, 16, device=device),
                out_dtype=torch.bfloat16,
            )
            _ROWWISE_SCALED_MM = True
        except (RuntimeError, TypeError):
            _ROWWISE_SCALED_MM = False
    return _ROWWISE_SCALED_MM


def fp8_linear_rowwise(xq, sx, w_q, sw):
    """out[M,N] = (xq*sx[:,None]) @ (w_q*sw[None,:]).T in fp8 tensor
    cores with per-row activation + per-channel weight scales. Uses
    _scaled_mm's rowwise scaling when this build supports it, else a
    unit-scale fp8 GEMM with the outer-product scale applied after."""
    if fp8_rowwise_supported(xq.device):
        return torch._scaled_mm(
            xq, w_q.t(), scale_a=sx[:, None].contiguous(),
            scale_b=sw[None, :].contiguous(), out_dtype=torch.bfloat16,
        )
    one = torch.ones((), dtype=torch.float32, device=xq.device)
    out = torch._scaled_mm(xq, w_q.t(), scale_a=one, scale_b=one,
                           out_dtype=torch.float32)
    return (out * sx[:, None] * sw[None, :]).to(torch.bfloat16)


# ---------------------------------------------------------------------------
# fp32-residual stack ops (hybrid recurrent/attention models). On a GPU
# these run the kernels of `_mixops.so` (ops/native.py) for bf16 or float32
# activations; on CPU tensors the references run.
# ---------------------------------------------------------------------------
ACT_KINDS = {"silu": 0, "gelu_tanh": 1, "clamped_swish": 2, "sigmoid": 3,
             "relu2": 4}


def _mx():
    from production_stack_amd.ops import native

    return native.load()


def _mx_dtype(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return 0
    if dtype == torch.float32:
        return 1
    raise TypeError(f"mixer kernels take bfloat16 or float32, not {dtype}")


def _stream():
    import ctypes

    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    import ctypes

    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _rows(t: torch.Tensor, name: str) -> int:
    """Row stride (elements) of a 2-D view whose rows are contiguous."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name}: need a 2-D view with unit inner stride")
    return t.stride(0)


def embed_scale(tokens: torch.Tensor, embed: torch.Tensor,
                scale: float) -> torch.Tensor:
    """fp32 residual rows embed[token] * scale."""
    if not embed.is_cuda:
        return reference.embed_scale(tokens, embed, scale)
    T, W = tokens.shape[0], embed.shape[1]
    assert tokens.dtype == torch.long and tokens.is_contiguous()
    assert embed.is_contiguous()
    x = torch.empty((T, W), dtype=torch.float32, device=embed.device)
    _mx().mx_embed_scale(_p(x), _p(tokens), _p(embed),
                         _f(scale), T, W, _mx_dtype(embed.dtype), _stream())
    return x


def _f(v: float):
    import ctypes

    return ctypes.c_float(v)


def add_rms_norm32(x32: torch.Tensor, deltas, w32: torch.Tensor, eps: float,
                   out_dtype: torch.dtype, groups: int = 1,
                   out32: torch.Tensor = None) -> torch.Tensor:
    """out32 = x32 + sum(deltas) (fp32; up to two deltas of out_dtype;
    out32 defaults to x32, i.e. in place), returns rms_norm(out32) * w32
    rounded to out_dtype. groups > 1: every one of `groups` equal
    consecutive parts of a row has its own root mean square."""
    if not x32.is_cuda:
        return reference.add_rms_norm32(x32, deltas, w32, eps, out_dtype,
                                        groups, out32)
    T, W = x32.shape
    assert x32.dtype == torch.float32 and x32.is_contiguous()
    assert w32.dtype == torch.float32 and w32.numel() == W
    assert 1 <= groups <= 64 and W % groups == 0
    if out32 is None:
        out32 = x32
    assert out32.dtype == torch.float32 and out32.is_contiguous()
    assert out32.shape == x32.shape
    deltas = list(deltas)
    if len(deltas) > 2:
        raise ValueError("at most two deltas")
    for d in deltas:
        assert d.dtype == out_dtype and d.shape == (T, W)
    d0 = deltas[0] if deltas else None
    d1 = deltas[1] if len(deltas) > 1 else None
    h = torch.empty((T, W), dtype=out_dtype, device=x32.device)
    _mx().mx_add_group_norm32(
        _p(h), _p(out32), _p(x32), _p(d0),
        _rows(d0, "delta") if d0 is not None else 0,
        _p(d1), _rows(d1, "delta") if d1 is not None else 0, _p(w32),
        _f(eps), int(groups), T, W, _mx_dtype(out_dtype), _stream())
    return h


def _check_seq_rows(seq_rows: torch.Tensor) -> None:
    assert seq_rows.dtype == torch.int32 and seq_rows.dim() == 2
    assert seq_rows.shape[1] == 4 and seq_rows.is_contiguous()


def group_norm_shift(x32: torch.Tensor, w32: torch.Tensor, eps: float,
                     groups: int, out_dtype: torch.dtype,
                     shift: torch.Tensor, state: torch.Tensor,
                     token_seq: torch.Tensor,
                     seq_rows: torch.Tensor) -> torch.Tensor:
    """Grouped RMSNorm followed by the token shift h + (h_prev - h) * shift
    (see reference.group_norm_shift). x32 fp32 [T, W]; shift fp32 [W];
    state fp32 [slots, W] (the previous token's normed row per sequence),
    updated; token_seq int32 [T] gives every row's segment."""
    if not x32.is_cuda:
        return reference.group_norm_shift(x32, w32, eps, groups, out_dtype,
                                          shift, state, seq_rows)
    T, W = x32.shape
    assert x32.dtype == torch.float32 and x32.is_contiguous()
    assert w32.dtype == torch.float32 and w32.numel() == W
    assert shift.dtype == torch.float32 and shift.numel() == W
    assert state.dtype == torch.float32 and state.shape[1:] == (W,)
    assert state.is_contiguous() and 1 <= groups <= 64
    assert W % groups == 0
    assert token_seq.dtype == torch.int32 and token_seq.shape == (T,)
    _check_seq_rows(seq_rows)
    h = torch.empty((T, W), dtype=out_dtype, device=x32.device)
    _mx().mx_group_norm_shift(
        _p(h), _p(x32), _p(w32), _f(eps), int(groups), _p(shift), _p(state),
        _p(token_seq), _p(seq_rows), T, W, _mx_dtype(out_dtype), _stream())
    return h


def depth_mix(hist: torch.Tensor, n: int, weights: torch.Tensor,
              base: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    """hist fp32 [streams, T, W]: stores the newest stream hist[n-1] =
    base + delta (base fp32 [T, W], may be hist[n-1] itself; delta [T, W]
    of the serving dtype) and returns sum_{j<n} weights[j] * hist[j] as a
    new fp32 [T, W]."""
    if not hist.is_cuda:
        return reference.depth_mix(hist, n, weights, base, delta)
    _, T, W = hist.shape
    assert hist.dtype == torch.float32 and hist.is_contiguous()
    assert 1 <= n <= hist.shape[0]
    assert weights.dtype == torch.float32 and weights.numel() >= n
    assert base.dtype == torch.float32 and base.shape == (T, W)
    assert base.is_contiguous() and delta.shape == (T, W)
    out = torch.empty((T, W), dtype=torch.float32, device=hist.device)
    _mx().mx_depth_mix(
        _p(out), _p(hist), int(n), _p(weights), _p(base), _p(delta),
        _rows(delta, "delta"), T, W, _mx_dtype(delta.dtype), _stream())
    return out


def gated_act(gate: torch.Tensor, up: torch.Tensor, kind: str,
              limit: float = 0.0, out: torch.Tensor = None) -> torch.Tensor:
    """Gated-MLP inner activation on [T, F] views (row-strided allowed):
    silu | gelu_tanh | clamped_swish | sigmoid | relu2 (see
    reference.gated_act); out may be up itself. up None: the plain
    activation of `gate` (out may then be gate itself)."""
    T, F = gate.shape
    assert up is None or (up.shape == (T, F) and up.dtype == gate.dtype)
    if out is None:
        out = torch.empty((T, F), dtype=gate.dtype, device=gate.device)
    assert out.shape == (T, F) and out.dtype == gate.dtype
    if not gate.is_cuda:
        out.copy_(reference.gated_act(gate, up, kind, limit, gate.dtype))
        return out
    _mx().mx_gated_act(
        _p(out), _rows(out, "out"), _p(gate), _rows(gate, "gate"), _p(up),
        _rows(up, "up") if up is not None else 0, T, F, ACT_KINDS[kind],
        _f(limit),
        _mx_dtype(gate.dtype), _stream())
    return out


def kv_append(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
              v_cache: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """Append k [T, G*D] / v [T, G*DV] rows (row-strided views allowed) to
    paged caches [NB, G, BS, D] / [NB, G, BS, DV]."""
    NB, G, BS, D = k_cache.shape
    DV = v_cache.shape[3]
    T = k.shape[0]
    assert v_cache.shape[:3] == (NB, G, BS)
    assert k.shape == (T, G * D) and v.shape == (T, G * DV)
    assert slot_mapping.dtype == torch.long and slot_mapping.shape == (T,)
    if not k_cache.is_cuda:
        reference.kv_append(k.reshape(T, G, D), v.reshape(T, G, DV),
                            k_cache, v_cache, slot_mapping)
        return
    assert k.dtype == k_cache.dtype == v.dtype == v_cache.dtype
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    _mx().mx_kv_append(
        _p(k), _rows(k, "k"), _p(v), _rows(v, "v"), _p(k_cache),
        _p(v_cache), _p(slot_mapping), T, G, D, DV, BS,
        _mx_dtype(k.dtype), _stream())


def talk_attention(q: torch.Tensor, k_cache: torch.Tensor,
                   v_cache: torch.Tensor, block_tables: torch.Tensor,
                   token_seq: torch.Tensor, token_pos: torch.Tensor,
                   scale: float, heads: int, chunk: int = 0, window: int = 0,
                   sink: bool = False, talk: torch.Tensor = None,
                   out: torch.Tensor = None, variant: int = 0,
                   splits: int = 0, keep_first: int = 0,
                   softcap: float = 0.0, sink_vals: torch.Tensor = None,
                   vdim: int = 0, pool=None) -> torch.Tensor:
    """Paged attention of a ragged batch. q [T, H*D] (row-strided view
    allowed); token_seq/token_pos int32 [T] give each token's block-table
    row and position; talk: optional fp32 [H, H] score mix; chunk/window:
    visibility limits (0 = off), the first keep_first keys of a sequence
    stay visible behind the window; softcap > 0: scores become cap *
    tanh(score / cap); sink: a value-less key joins the softmax
    denominator with score 0, or sink_vals[h] (fp32 [H]) when given; vdim:
    the values are the first vdim entries of v_cache's rows (v_cache may be
    k_cache itself: keys that carry their values). pool = (kp_cache,
    vp_cache, P): with a window, every block of P positions that lies
    wholly before a query's window adds its pooled key and value (as
    pool_append stores them) to the same softmax.
    variant 0 picks the kernel for prompt portions (tiled thread-per-
    (head, query) where the shape fits), 3 for single tokens (split-key),
    both falling back to the plain one-workgroup-per-token kernel; 1 / 2 /
    4 force plain / tiled / split-key. bfloat16 batches without head mix
    and aligned chunks take the matrix-core kernel instead when the shape
    fits it (variants 0 and 3; 5 insists on it, 6 on its 128-row form).
    Returns [T, H*DV]."""
    NB, G, BS, D = k_cache.shape
    VR = v_cache.shape[3]
    DV = vdim or VR
    T = q.shape[0]
    H = heads
    assert q.shape == (T, H * D) and H % G == 0 and DV <= VR
    assert v_cache.shape[:3] == (NB, G, BS)
    assert token_seq.dtype == torch.int32 and token_pos.dtype == torch.int32
    assert token_seq.shape == (T,) and token_pos.shape == (T,)
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2
    if talk is not None:
        assert talk.dtype == torch.float32 and talk.shape == (H, H)
    if sink_vals is not None:
        assert sink and sink_vals.dtype == torch.float32
        assert sink_vals.shape == (H,)
    kp = vp = None
    P = PR = 0
    if pool is not None and window > 0:
        kp, vp, P = pool
        PR = (BS + P - 1) // P
        assert P >= 1 and chunk == 0 and keep_first == 0 and vdim == 0
        assert kp.shape == (NB, G, PR, D) and vp.shape == (NB, G, PR, DV)
        assert kp.dtype == k_cache.dtype and vp.dtype == v_cache.dtype
    else:
        pool = None
    if out is None:
        out = torch.empty((T, H * DV), dtype=q.dtype, device=q.device)
    assert out.shape == (T, H * DV) and out.dtype == q.dtype
    if not q.is_cuda:
        o = reference.talk_attention(
            q.reshape(T, H, D), k_cache, v_cache, block_tables, token_seq,
            token_pos, scale, chunk, window, sink, talk, keep_first,
            softcap, sink_vals, DV, pool)
        out.copy_(o.reshape(T, H * DV))
        return out
    assert q.dtype == k_cache.dtype == v_cache.dtype
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert block_tables.is_contiguous()
    if talk is not None:
        assert talk.is_contiguous()
    if pool is not None:
        assert kp.is_contiguous() and vp.is_contiguous()
    # single tokens: when the batch is too small to fill the chip with one
    # workgroup per token, each token's keys are shared out over several
    # workgroups whose partial softmax records are merged afterwards
    scratch = None
    if variant not in (3, 4, 5, 6):
        splits = 1
    elif splits <= 0:
        splits = (max(1, min(8, 512 // T))
                  if T < 256 and variant not in (5, 6) else 1)
    if splits > 1:
        scratch = torch.empty((T, splits, H, DV + 2),
                              dtype=torch.float32, device=q.device)
    # bf16 without head mix / aligned chunks: the matrix-core kernel, where
    # the shape fits it (variant 5 insists on it)
    if (variant in (0, 3, 5, 6) and q.dtype == torch.bfloat16
            and talk is None and chunk == 0):
        # 0: prompt portions, 1: single tokens, 2: 128-row workgroups
        mode = (2 if variant == 6 else
                int(variant == 3 or (variant == 5 and splits > 0)))
        rc = _mx().mx_mfma_attention(
            _p(out), _rows(out, "out"), _p(q), _rows(q, "q"), _p(k_cache),
            _p(v_cache), _p(block_tables), block_tables.shape[1],
            _p(token_seq), _p(token_pos), T, H, G, D, DV, BS, _f(scale),
            int(window), int(bool(sink)), int(keep_first), _f(softcap),
            _p(sink_vals), int(VR),
            int(v_cache.data_ptr() == k_cache.data_ptr()), int(splits),
            _p(scratch), mode, _p(kp), _p(vp), int(P), _stream())
        if rc == 0:
            return out
    if variant in (5, 6):
        raise RuntimeError(
            "talk_attention: shape or dtype outside the matrix-core kernel")
    rc = _mx().mx_talk_attention(
        _p(out), _rows(out, "out"), _p(q), _rows(q, "q"), _p(k_cache),
        _p(v_cache), _p(block_tables), block_tables.shape[1],
        _p(token_seq), _p(token_pos), _p(talk), T, H, G, D, DV, BS,
        _f(scale), int(chunk), int(window), int(bool(sink)),
        _mx_dtype(q.dtype), int(variant), int(splits), _p(scratch),
        int(keep_first), _f(softcap), _p(sink_vals), int(VR), _p(kp),
        _p(vp), int(P), _stream())
    if rc != 0:
        raise RuntimeError(
            f"talk_attention: heads x dim {H}x{D}/{DV} exceeds the kernel's "
            "LDS budget")
    return out


def attn_prep(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
              q_w, k_w, eps: float, vmix, v_first, k_cache: torch.Tensor,
              v_cache: torch.Tensor, slot_mapping: torch.Tensor,
              heads: int, cos_sin: torch.Tensor = None,
              positions: torch.Tensor = None, rot_dims: int = 0,
              norm_all: bool = False, half: bool = False) -> None:
    """Per-head query/key RMSNorm (weights q_w / k_w fp32 [D], None = no
    norm; q is rewritten in place), value blend (1 - vmix) v + vmix v_first
    when v_first [T, G*DV] is given (vmix a 0-dim fp32 tensor; v is
    rewritten in place), rotary turn of the first rot_dims entries of every
    query and key head (cos_sin fp32 [positions, rot_dims/2, 2] as
    rope_table builds it, positions int32 [T]; interleaved pairs; q is
    rewritten in place), and append of the keys and values to the paged
    caches [NB, G, BS, D|DV]. q/k/v are row-strided views. norm_all: one
    root mean square over the whole query (key) projection and weights
    q_w fp32 [H*D] / k_w fp32 [G*D]; half: the rotary pairs are (i, i +
    rot_dims/2) instead of (2i, 2i+1)."""
    NB, G, BS, D = k_cache.shape
    DV = v_cache.shape[3]
    T = q.shape[0]
    H = heads
    assert q.shape == (T, H * D) and k.shape == (T, G * D)
    assert v.shape == (T, G * DV) and v_cache.shape[:3] == (NB, G, BS)
    assert slot_mapping.dtype == torch.long and slot_mapping.shape == (T,)
    if v_first is not None:
        assert v_first.shape == v.shape and v_first.dtype == v.dtype
        assert vmix.dtype == torch.float32 and vmix.numel() == 1
    if cos_sin is not None:
        assert rot_dims % 2 == 0 and 0 < rot_dims <= D
        assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
        assert cos_sin.shape[1:] == (rot_dims // 2, 2)
        assert positions.dtype == torch.int32 and positions.shape == (T,)
    if not q.is_cuda:
        reference.attn_prep(q, k, v, q_w, k_w, eps, vmix, v_first, k_cache,
                            v_cache, slot_mapping, H, cos_sin, positions,
                            rot_dims, norm_all, half)
        return
    assert q.dtype == k.dtype == v.dtype == k_cache.dtype == v_cache.dtype
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    for w, n in ((q_w, H), (k_w, G)):
        if w is not None:
            assert w.dtype == torch.float32
            assert w.numel() == (n * D if norm_all else D)
    _mx().mx_attn_prep(
        _p(q), _rows(q, "q"), _p(k), _rows(k, "k"), _p(v), _rows(v, "v"),
        _p(q_w), _p(k_w), _f(eps), _p(vmix if v_first is not None else None),
        _p(v_first), _rows(v_first, "v_first") if v_first is not None else 0,
        _p(k_cache), _p(v_cache), _p(slot_mapping), T, H, G, D, DV, BS,
        _p(cos_sin), int(cos_sin.shape[0]) if cos_sin is not None else 0,
        int(rot_dims) if cos_sin is not None else 0, _p(positions),
        int(bool(norm_all)), int(bool(half)), _mx_dtype(q.dtype), _stream())


def rope_table(max_pos: int, dims: int, base: float,
               device=None, factor: float = 1.0,
               scaling=None) -> torch.Tensor:
    """fp32 [max_pos, dims/2, 2] (cos, sin) of position * base^(-2i/dims)
    / factor, correctly rounded (angles formed in float64 on the host);
    scaling = (factor, original, fast, slow) blends the frequencies and
    scales the magnitude (see reference.scaled_frequencies)."""
    return reference.rope_table(max_pos, dims, base, device, factor,
                                scaling)


def pool_append(k_cache: torch.Tensor, v_cache: torch.Tensor,
                kp_cache: torch.Tensor, vp_cache: torch.Tensor,
                block_tables: torch.Tensor, seq_rows: torch.Tensor,
                pool: int, num_tokens: int) -> None:
    """Stores the mean key and value of every block of `pool` consecutive
    positions that this step completed (see reference.pool_append):
    caches [NB, G, BS, D|DV] -> pooled caches [NB, G, ceil(BS/pool),
    D|DV]. Runs after the step's keys and values were appended;
    num_tokens is the step's row count (bounds a segment's blocks)."""
    NB, G, BS, D = k_cache.shape
    DV = v_cache.shape[3]
    PR = (BS + pool - 1) // pool
    assert pool >= 1 and kp_cache.shape == (NB, G, PR, D)
    assert vp_cache.shape == (NB, G, PR, DV)
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2
    assert block_tables.shape[0] == seq_rows.shape[0]
    if not k_cache.is_cuda:
        reference.pool_append(k_cache, v_cache, kp_cache, vp_cache,
                              block_tables, seq_rows, pool)
        return
    _check_seq_rows(seq_rows)
    assert k_cache.dtype == v_cache.dtype == kp_cache.dtype == vp_cache.dtype
    for t in (k_cache, v_cache, kp_cache, vp_cache, block_tables):
        assert t.is_contiguous()
    S = seq_rows.shape[0]
    # a segment of n rows completes at most n // pool + 1 blocks
    longest = num_tokens - (S - 1)
    _mx().mx_pool_append(
        _p(k_cache), _p(v_cache), _p(kp_cache), _p(vp_cache),
        _p(block_tables), block_tables.shape[1], _p(seq_rows), S,
        longest // pool + 1, G, D, DV, BS, int(pool),
        _mx_dtype(k_cache.dtype), _stream())


def add_layer_norm_conv32(x32: torch.Tensor, deltas, scales,
                          w32: torch.Tensor, b32: torch.Tensor, eps: float,
                          conv_w: torch.Tensor, state: torch.Tensor,
                          seq_rows: torch.Tensor,
                          out_dtype: torch.dtype) -> torch.Tensor:
    """Sublayer boundary with a layer norm and an input convolution (see
    reference.add_layer_norm_conv32): x32 fp32 [T, W] += sum scales[i] *
    deltas[i] in place (up to two deltas [T, W] of one dtype, row-strided
    views allowed), y = layernorm(x32) * w32 + b32, returns y + conv(y) in
    out_dtype, the causal convolution (conv_w fp32 [W, K]) running along
    the segments of seq_rows with state fp32 [slots, K-1, W] (a segment's
    previous K - 1 rows of y), which is updated. conv_w None: returns y."""
    T, W = x32.shape
    assert x32.dtype == torch.float32 and x32.is_contiguous()
    deltas, scales = list(deltas), [float(v) for v in scales]
    assert len(deltas) <= 2 and len(scales) == len(deltas)
    for d in deltas:
        assert d.shape == (T, W) and d.dtype == deltas[0].dtype
    for w in (w32, b32):
        assert w.dtype == torch.float32 and w.numel() == W
    K = 0
    if conv_w is not None:
        K = conv_w.shape[1]
        assert conv_w.dtype == torch.float32 and conv_w.shape == (W, K)
        assert K >= 1 and state.dtype == torch.float32
        assert state.shape[1:] == (K - 1, W)
    if not x32.is_cuda:
        return reference.add_layer_norm_conv32(
            x32, deltas, scales, w32, b32, eps, conv_w, state, seq_rows,
            out_dtype)
    h = torch.empty((T, W), dtype=out_dtype, device=x32.device)
    stats = None
    if conv_w is not None:
        _check_seq_rows(seq_rows)
        assert conv_w.is_contiguous() and state.is_contiguous()
        stats = torch.empty((T, 2), dtype=torch.float32, device=x32.device)
    d0 = deltas[0] if deltas else None
    d1 = deltas[1] if len(deltas) > 1 else None
    _mx().mx_add_layer_norm32(
        _p(h if conv_w is None else None), _p(x32), _p(d0),
        _rows(d0, "delta") if d0 is not None else 0,
        _f(scales[0] if deltas else 0.0), _p(d1),
        _rows(d1, "delta") if d1 is not None else 0,
        _f(scales[1] if d1 is not None else 0.0), _p(w32), _p(b32), _f(eps),
        _p(stats), T, W,
        _mx_dtype(d0.dtype) if d0 is not None else 0, _mx_dtype(out_dtype),
        _stream())
    if conv_w is not None:
        S = seq_rows.shape[0]
        rc = _mx().mx_norm_conv32(
            _p(h), _p(x32), _p(stats), _p(w32), _p(b32), _p(conv_w),
            _p(state), _p(seq_rows), S, W, K, T, _mx_dtype(out_dtype),
            _stream())
        if rc != 0:
            raise RuntimeError(
                f"add_layer_norm_conv32: {K} taps are not built (1-32)")
    return h


def mingru_scan(z: torch.Tensor, u: torch.Tensor, g: torch.Tensor,
                zb: torch.Tensor, ub: torch.Tensor, state: torch.Tensor,
                seq_rows: torch.Tensor,
                out: torch.Tensor = None) -> torch.Tensor:
    """Element-wise gated recurrence S <- (1 - a) S + a c over a ragged
    batch with read-out S * silu(g) (see reference.mingru_scan). z / u / g
    [T, C] row-strided views of one dtype; zb / ub fp32 [C]; state fp32
    [slots, C], updated in place. Returns [T, C] of the inputs' dtype."""
    T, C = z.shape
    assert u.shape == (T, C) and g.shape == (T, C)
    assert u.dtype == z.dtype and g.dtype == z.dtype
    assert state.dtype == torch.float32 and state.shape[1:] == (C,)
    for b in (zb, ub):
        assert b.dtype == torch.float32 and b.numel() == C
    if out is None:
        out = torch.empty((T, C), dtype=z.dtype, device=z.device)
    assert out.shape == (T, C) and out.dtype == z.dtype
    if not z.is_cuda:
        out.copy_(reference.mingru_scan(z, u, g, zb, ub, state, seq_rows,
                                        z.dtype))
        return out
    _check_seq_rows(seq_rows)
    assert state.is_contiguous()
    # long segments run as tiles whose composed maps meet in this scratch
    S = seq_rows.shape[0]
    need = _mx().mx_mingru_scratch(S, C, T)
    scratch = (torch.empty(need, dtype=torch.float32, device=z.device)
               if need > 0 else None)
    _mx().mx_mingru_scan(
        _p(out), _rows(out, "out"), _p(z), _rows(z, "z"), _p(u),
        _rows(u, "u"), _p(g), _rows(g, "g"), _p(zb), _p(ub), _p(state),
        _p(seq_rows), S, C, T, _p(scratch), _mx_dtype(z.dtype), _stream())
    return out


def latent_prep(q_lat: torch.Tensor, q: torch.Tensor, dkv: torch.Tensor,
                norm_w: torch.Tensor, eps: float, cos_sin: torch.Tensor,
                positions: torch.Tensor, cache: torch.Tensor,
                slot_mapping: torch.Tensor, heads: int, dim: int,
                rot_dim: int, rot_dims: int) -> torch.Tensor:
    """Inputs of latent attention (see reference.latent_prep): normalises
    the latent, turns the shared key part and the queries' rotated parts
    by their positions, appends [latent | key part] to the paged cache
    [NB, 1, BS, L+rot_dim] and returns the queries [T, H*(L+rot_dim)]."""
    H = heads
    T = q.shape[0]
    L = dkv.shape[1] - rot_dim
    assert q.shape == (T, H * (dim + rot_dim))
    assert q_lat.shape == (H, T, L) and q_lat.is_contiguous()
    assert cache.shape[1] == 1 and cache.shape[3] == L + rot_dim
    assert rot_dims % 2 == 0 and rot_dims <= rot_dim
    assert cos_sin.dtype == torch.float32
    assert cos_sin.shape[1:] == (rot_dims // 2, 2)
    assert positions.dtype == torch.int32 and positions.shape == (T,)
    assert slot_mapping.dtype == torch.long and slot_mapping.shape == (T,)
    if not q.is_cuda:
        return reference.latent_prep(
            q_lat, q, dkv, norm_w, eps, cos_sin, positions, cache,
            slot_mapping, H, dim, rot_dim, rot_dims, q.dtype)
    assert q.dtype == dkv.dtype == q_lat.dtype == cache.dtype
    assert norm_w.dtype == torch.float32 and norm_w.numel() == L
    assert cache.is_contiguous() and cos_sin.is_contiguous()
    out = torch.empty((T, H * (L + rot_dim)), dtype=q.dtype, device=q.device)
    _mx().mx_latent_prep(
        _p(out), _p(q_lat), _p(q), _rows(q, "q"), _p(dkv),
        _rows(dkv, "dkv"), _p(norm_w), _f(eps), _p(cos_sin),
        int(cos_sin.shape[0]), int(rot_dims), _p(positions), _p(cache),
        _p(slot_mapping), T, H, dim, rot_dim, L, cache.shape[2],
        _mx_dtype(q.dtype), _stream())
    return out


def short_conv_silu(x: torch.Tensor, w: torch.Tensor, state: torch.Tensor,
                    seq_rows: torch.Tensor, out: torch.Tensor = None,
                    bias: torch.Tensor = None) -> torch.Tensor:
    """Causal per-channel convolution over time + silu over a ragged batch
    (see reference.short_conv_silu). x [T, C] row-strided view; w fp32
    [C, K]; state [slots, K-1, C] of x's dtype, updated; bias: optional
    fp32 [C]."""
    T, C = x.shape
    K = w.shape[1]
    assert w.dtype == torch.float32 and w.shape == (C, K) and K >= 1
    assert state.shape[1:] == (K - 1, C) and state.dtype == x.dtype
    if out is None:
        out = torch.empty((T, C), dtype=x.dtype, device=x.device)
    assert out.shape == (T, C) and out.dtype == x.dtype
    if bias is not None:
        assert bias.dtype == torch.float32 and bias.shape == (C,)
    if not x.is_cuda:
        out.copy_(reference.short_conv_silu(x, w, state, seq_rows, x.dtype,
                                            bias))
        return out
    _check_seq_rows(seq_rows)
    assert w.is_contiguous() and state.is_contiguous()
    rc = _mx().mx_short_conv_silu(
        _p(out), _rows(out, "out"), _p(x), _rows(x, "x"), _p(w), _p(bias),
        _p(state), _p(seq_rows), seq_rows.shape[0], C, K, T,
        _mx_dtype(x.dtype), _stream())
    if rc != 0:
        raise RuntimeError(f"short_conv_silu: {K} taps are not built (1-8)")
    return out


def gated_delta(q, k, v, beta, zdec, zgate, a_log, dt_bias, normw, state,
                seq_rows, heads: int, kv_heads: int, eps: float,
                out: torch.Tensor = None) -> torch.Tensor:
    """Gated delta rule with per-(head, key channel) decay over a ragged
    batch (see reference.gated_delta). q/k [T, G*D], v [T, H*DV], beta
    [T, H], zdec [T, H*D], zgate [T, H*DV]: row-strided views of one
    dtype; a_log fp32 [H], dt_bias fp32 [H*D], normw fp32 [DV]; state fp32
    [slots, H, D, DV], updated in place. Returns [T, H*DV]."""
    T = q.shape[0]
    H, G = heads, kv_heads
    D = q.shape[1] // G
    DV = v.shape[1] // H
    assert H % G == 0 and q.shape == (T, G * D) and k.shape == (T, G * D)
    assert v.shape == (T, H * DV) and beta.shape == (T, H)
    assert zdec.shape == (T, H * D) and zgate.shape == (T, H * DV)
    assert state.dtype == torch.float32 and state.shape[1:] == (H, D, DV)
    for t in (k, v, beta, zdec, zgate):
        assert t.dtype == q.dtype
    assert a_log.dtype == torch.float32 and a_log.numel() == H
    assert dt_bias.dtype == torch.float32 and dt_bias.numel() == H * D
    assert normw.dtype == torch.float32 and normw.numel() == DV
    if out is None:
        out = torch.empty((T, H * DV), dtype=q.dtype, device=q.device)
    assert out.shape == (T, H * DV) and out.dtype == q.dtype
    if not q.is_cuda:
        y = reference.gated_delta(
            q.reshape(T, G, D), k.reshape(T, G, D), v.reshape(T, H, DV),
            beta, zdec.reshape(T, H, D), zgate.reshape(T, H, DV), a_log,
            dt_bias, normw, state, seq_rows, H, G, eps, q.dtype)
        out.copy_(y.reshape(T, H * DV))
        return out
    _check_seq_rows(seq_rows)
    assert state.is_contiguous()
    rc = _mx().mx_gated_delta(
        _p(out), _rows(out, "out"), _p(q), _rows(q, "q"), _p(k),
        _rows(k, "k"), _p(v), _rows(v, "v"), _p(beta), _rows(beta, "beta"),
        _p(zdec), _rows(zdec, "zdec"), _p(zgate), _rows(zgate, "zgate"),
        _p(a_log), _p(dt_bias), _p(normw), _p(state), _p(seq_rows),
        seq_rows.shape[0], H, G, D, DV, _f(eps), _f(D ** -0.5),
        _mx_dtype(q.dtype), _stream())
    if rc != 0:
        raise RuntimeError(
            f"gated_delta: state {D}x{DV} per head is not built "
            "(dims up to 256)")
    return out


def delta_rule(r, k, v, zw, za, g, w0, ab, normw, state, seq_rows,
               heads: int, eps: float, decay_scale: float,
               out: torch.Tensor = None) -> torch.Tensor:
    """Gated delta-rule recurrence over a ragged batch (see
    reference.delta_rule). r/k/v/zw/za/g: [T, H*D] row-strided views of one
    dtype; w0/ab/normw fp32 [H*D]; state fp32 [slots, H, D, D], updated in
    place; seq_rows int32 [S, 4] = (first row, rows, first position, state
    slot) per segment. Returns [T, H*D] (written into `out` when given)."""
    T, HD = r.shape
    H = heads
    D = HD // H
    assert state.dtype == torch.float32 and state.shape[1:] == (H, D, D)
    assert seq_rows.dtype == torch.int32 and seq_rows.shape[1] == 4
    for name, t in (("k", k), ("v", v), ("zw", zw), ("za", za), ("g", g)):
        assert t.shape == (T, HD) and t.dtype == r.dtype, name
    for t in (w0, ab, normw):
        assert t.dtype == torch.float32 and t.numel() == HD
    if out is None:
        out = torch.empty((T, HD), dtype=r.dtype, device=r.device)
    assert out.shape == (T, HD) and out.dtype == r.dtype
    if not r.is_cuda:
        sh = (T, H, D)
        y = reference.delta_rule(
            r.reshape(sh), k.reshape(sh), v.reshape(sh), zw.reshape(sh),
            za.reshape(sh), g.reshape(sh), w0, ab, normw, state, seq_rows,
            eps, decay_scale, r.dtype)
        out.copy_(y.reshape(T, HD))
        return out
    assert state.is_contiguous() and seq_rows.is_contiguous()
    rc = _mx().mx_delta_rule(
        _p(out), _rows(out, "out"), _p(r), _rows(r, "r"), _p(k),
        _rows(k, "k"), _p(v), _rows(v, "v"), _p(zw), _rows(zw, "zw"),
        _p(za), _rows(za, "za"), _p(g), _rows(g, "g"), _p(w0), _p(ab),
        _p(normw), _p(state), _p(seq_rows), seq_rows.shape[0], H, D,
        _f(eps), _f(decay_scale), _mx_dtype(r.dtype), _stream())
    if rc != 0:
        raise RuntimeError(f"delta_rule: head dim {D} above 256 is not built")
    return out


def norm_sum32(inputs, weights, scale: float, eps: float) -> torch.Tensor:
    """fp32 [T, W] = scale * sum_i rmsnorm(inputs[i]) * weights[i]: up to
    four branch outputs [T, W] of one dtype (row-strided views allowed),
    each divided by its own root mean square over the row and scaled by
    its fp32 weight [W]."""
    inputs, weights = list(inputs), list(weights)
    n = len(inputs)
    assert 1 <= n <= 4 and len(weights) == n
    T, W = inputs[0].shape
    for x, w in zip(inputs, weights):
        assert x.shape == (T, W) and x.dtype == inputs[0].dtype
        assert w.dtype == torch.float32 and w.numel() == W
    if not inputs[0].is_cuda:
        return reference.norm_sum32(inputs, weights, scale, eps)
    out = torch.empty((T, W), dtype=torch.float32, device=inputs[0].device)
    pad = [None] * (4 - n)
    xs, ws = inputs + pad, weights + pad
    _mx().mx_norm_sum32(
        _p(out), n, _p(xs[0]), _p(xs[1]), _p(xs[2]), _p(xs[3]),
        *[_rows(x, "input") if x is not None else 0 for x in xs],
        _p(ws[0]), _p(ws[1]), _p(ws[2]), _p(ws[3]), _f(scale), _f(eps), T, W,
        _mx_dtype(inputs[0].dtype), _stream())
    return out


def post_norm_add_norm32(x32: torch.Tensor, delta: torch.Tensor,
                         w_post: torch.Tensor, w_next: torch.Tensor,
                         eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """Sublayer boundary of a stack that normalises a sublayer's output
    before it joins the residual stream: x32 += rmsnorm(delta) * w_post
    (fp32 [T, W], in place; delta [T, W] fp32 or the serving dtype,
    row-strided view allowed), returns rmsnorm(x32) * w_next in out_dtype:
    the next sublayer's input. Weights fp32 [W]."""
    T, W = x32.shape
    assert x32.dtype == torch.float32 and x32.is_contiguous()
    assert delta.shape == (T, W)
    for w in (w_post, w_next):
        assert w.dtype == torch.float32 and w.numel() == W
    if not x32.is_cuda:
        return reference.post_norm_add_norm32(x32, delta, w_post, w_next,
                                              eps, out_dtype)
    h = torch.empty((T, W), dtype=out_dtype, device=x32.device)
    _mx().mx_post_norm_add_norm32(
        _p(h), _p(x32), _p(delta), _rows(delta, "delta"),
        _mx_dtype(delta.dtype), _p(w_post), _p(w_next), _f(eps), T, W,
        _mx_dtype(out_dtype), _stream())
    return h


SCAN_MODES = {"gla": 0, "ssd": 1, "mlstm": 2}


def linear_scan(mode: str, q, k, v, dec, gate, state, seq_rows, heads: int,
                groups: int, eps: float, qscale: float = 1.0,
                c0: float = 1.0, wr=None, p0=None, p1=None, p2=None,
                normw=None, aux=None, out=None) -> torch.Tensor:
    """Gated linear recurrences S <- diag(a) S + w k v^T, o = S^T q over a
    ragged batch (see reference.linear_scan for the three decay laws and
    read-outs: "gla" one decay per key channel, "ssd" one per head with a
    step size and a skip term, "mlstm" exponential gates with a running
    maximum and a normaliser). q/k [T, G*D], v/gate [T, H*DV], dec
    [T, H*D] (gla) or [T, H], wr [T, H] (mlstm): row-strided views of one
    dtype; p0/p1/p2/normw fp32; state fp32 [slots, H, D, DV] and aux fp32
    [slots, H, D+1] (mlstm) are updated in place. Returns [T, H*DV], fp32
    for "ssd" (a grouped norm follows), else the inputs' dtype."""
    T = q.shape[0]
    H, G = heads, groups
    D = q.shape[1] // G
    DV = v.shape[1] // H
    assert H % G == 0 and q.shape == (T, G * D) and k.shape == (T, G * D)
    assert v.shape == (T, H * DV) and gate.shape == (T, H * DV)
    assert state.dtype == torch.float32 and state.shape[1:] == (H, D, DV)
    dt = q.dtype
    for t in (k, v, dec, gate):
        assert t.dtype == dt
    if mode == "gla":
        assert dec.shape == (T, H * D) and G == H
        assert p0.numel() == H * D and normw.numel() == DV
    elif mode == "ssd":
        assert dec.shape == (T, H)
        assert p0.numel() == H and p1.numel() == H and p2.numel() == H
    elif mode == "mlstm":
        assert dec.shape == (T, H) and wr.shape == (T, H) and G == H
        assert wr.dtype == dt
        assert p0.numel() == H and p1.numel() == H
        assert normw.numel() == H * DV
        assert aux.dtype == torch.float32 and aux.shape[1:] == (H, D + 1)
        assert aux.shape[0] == state.shape[0]
    else:
        raise ValueError(f"unknown scan mode {mode!r}")
    for t in (p0, p1, p2, normw):
        assert t is None or t.dtype == torch.float32
    odt = torch.float32 if mode == "ssd" else dt
    if out is None:
        out = torch.empty((T, H * DV), dtype=odt, device=q.device)
    assert out.shape == (T, H * DV) and out.dtype == odt
    if not q.is_cuda:
        y = reference.linear_scan(
            mode, q.reshape(T, G, D), k.reshape(T, G, D),
            v.reshape(T, H, DV),
            dec.reshape(T, H, D) if mode == "gla" else dec, wr,
            gate.reshape(T, H, DV), p0, p1, p2, normw, state, aux, seq_rows,
            H, G, eps, qscale, c0, dt)
        out.copy_(y.reshape(T, H * DV))
        return out
    _check_seq_rows(seq_rows)
    assert state.is_contiguous() and (aux is None or aux.is_contiguous())
    # wide heads: a head's value columns are shared out over several
    # workgroups and the read-out norm runs as a second kernel over this
    # fp32 scratch
    raw = None
    if mode != "ssd" and _mx().mx_linear_scan_splits(
            SCAN_MODES[mode], seq_rows.shape[0], H, D, DV) > 1:
        raw = torch.empty(
            T * H * DV + seq_rows.shape[0] * H * (D + 1),
            dtype=torch.float32, device=q.device)
    rc = _mx().mx_linear_scan(
        SCAN_MODES[mode], _p(out), _rows(out, "out"), _p(q), _rows(q, "q"),
        _p(k), _rows(k, "k"), _p(v), _rows(v, "v"), _p(dec),
        _rows(dec, "dec"), _p(wr), _rows(wr, "wr") if wr is not None else 0,
        _p(gate), _rows(gate, "gate"), _p(p0), _p(p1), _p(p2), _p(normw),
        _p(state), _p(aux), _p(seq_rows), seq_rows.shape[0], H, G, D, DV,
        _f(eps), _f(qscale), _f(c0), T, _p(raw), _mx_dtype(dt), _stream())
    if rc != 0:
        raise RuntimeError(
            f"linear_scan: state {D}x{DV} per head is not built (key dims "
            "up to 256, value dims up to 1023)")
    return out


def moe_route(x: torch.Tensor, router_w: torch.Tensor, top: int,
              score: str = "softmax", renormalize: bool = True,
              correction: torch.Tensor = None, scale: float = 1.0,
              renorm_eps: float = 0.0):
    """Router of a routed feed-forward in one kernel (see
    reference.moe_route): fp32 logits of x [T, W] against router_w
    [n_out, W] (both of the serving dtype), softmax or sigmoid scores, the
    `top` best by score + correction (fp32 [n_out]), weights
    = chosen scores / (sum + renorm_eps) when renormalize, times scale.
    Returns (weights fp32 [T, top], indices int64 [T, top], dense fp32
    [T, n_out] with the weights at the chosen outputs and zeros
    elsewhere)."""
    T, W = x.shape
    n_out = router_w.shape[0]
    assert router_w.shape == (n_out, W) and router_w.dtype == x.dtype
    assert score in ("softmax", "sigmoid") and 1 <= top <= n_out
    if correction is not None:
        assert correction.dtype == torch.float32
        assert correction.shape == (n_out,)
    if not x.is_cuda:
        return reference.moe_route(x, router_w, top, score, renormalize,
                                   correction, scale, renorm_eps)
    assert router_w.is_contiguous()
    sel = torch.empty((T, top), dtype=torch.long, device=x.device)
    wts = torch.empty((T, top), dtype=torch.float32, device=x.device)
    dense = torch.empty((T, n_out), dtype=torch.float32, device=x.device)
    rc = _mx().mx_moe_route(
        _p(sel), _p(wts), _p(dense), _p(x), _rows(x, "x"), _p(router_w),
        _p(correction), T, W, n_out, int(top), int(score == "sigmoid"),
        int(bool(renormalize)), _f(renorm_eps), _f(scale),
        _mx_dtype(x.dtype), _stream())
    if rc != 0:
        raise RuntimeError(f"moe_route: {n_out} router outputs exceed 1024")
    return wts, sel, dense


def moe_combine(y: torch.Tensor, dense: torch.Tensor, x: torch.Tensor,
                experts: int, shared_y: torch.Tensor = None,
                shared_gate: torch.Tensor = None) -> torch.Tensor:
    """Weighted sum of the all-experts path in one kernel: y [E, T, W] is
    every expert's output for every row, dense fp32 [T, n_out] the routing
    weights (zero = not chosen; outputs from `experts` on are identity
    outputs that return the input x [T, W]); the shared expert's output
    shared_y [T, W] joins times sigmoid(shared_gate [T, 1]) (unscaled when
    shared_gate is None). Returns fp32 [T, W]."""
    E, T, W = y.shape
    n_out = dense.shape[1]
    assert E == experts and n_out >= E and dense.shape == (T, n_out)
    assert dense.dtype == torch.float32 and x.shape == (T, W)
    assert x.dtype == y.dtype
    if shared_y is not None:
        assert shared_y.shape == (T, W) and shared_y.dtype == y.dtype
        if shared_gate is not None:
            assert shared_gate.shape == (T, 1)
            assert shared_gate.dtype == y.dtype
    if not y.is_cuda:
        return reference.moe_combine(y, dense, x, experts, shared_y,
                                     shared_gate)
    assert y.is_contiguous() and dense.is_contiguous()
    out = torch.empty((T, W), dtype=torch.float32, device=y.device)
    _mx().mx_moe_combine(
        _p(out), _p(y), _p(dense), n_out, E, _p(x), _rows(x, "x"),
        _p(shared_y), _rows(shared_y, "shared_y") if shared_y is not None
        else 0, _p(shared_gate),
        _rows(shared_gate, "shared_gate") if shared_gate is not None else 0,
        T, W, _mx_dtype(y.dtype), _stream())
    return out
