// Gated linear recurrences without a removal term (prefill portions and
// single decode tokens in one launch):
//     S <- diag(a) S + w k v^T,   o = S^T q
// per head, S a D x DV fp32 matrix (rows = key channels, columns = value
// channels). Three decay laws / read-outs share the sweep:
//
//   GLA    a_i = sigmoid(dec_i + p0_i)^c0 per key channel, w = 1;
//          out = o / rms_DV(o) * normw[DV] * silu(gate)
//   SSD    dt = softplus(dec + p0[h]), a = exp(-exp(p1[h]) dt), w = dt, keys
//          and queries shared by groups of heads;
//          out = (o + p2[h] v) * silu(gate), stored as fp32 (a norm over
//          several heads follows)
//   MLSTM  i = cap(wr + p0[h]), f = logsigmoid(cap(dec + p1[h])),
//          cap(z) = c0 tanh(z / c0); running maximum m' = max(f + m, i),
//          a = exp(f + m - m'), w = exp(i - m'); the normaliser n <- a n + w k
//          is one more column of S (its "value" is 1), so n.q is that
//          column's read-out; o / (max(|n.q|, exp(-m')) + 1e-6), then
//          out = o / rms_DV(o) * normw[h][DV] * sigmoid(gate)
//
// q is scaled by qscale. Decays, gates, step sizes and maxima are formed in
// fp32 from the projections' outputs.
//
// Mapping (as the delta-rule kernels): one workgroup per (sequence segment,
// head). Column j of S lives in the registers of P adjacent lanes, lane p
// holding rows p, p+P, ... (D padded up to DKP). Tokens go through in tiles:
// the per-row vectors (k, q, and a for GLA) of a whole tile are prepared
// cooperatively into LDS (each lane's rows contiguous, segments padded
// against bank conflicts), per-token scalars (a, w, exp(-m)) beside them,
// then each thread walks the tile's tokens with broadcast LDS reads and no
// barrier. The running maximum is a sequential scan over the tile by one
// thread (a handful of scalar operations per token).
//
// Wide heads share their value columns out over several workgroups of four
// waves (columns never interact inside the
// recurrence; every part of a matrix-LSTM head carries the normaliser column
// itself). The read-out norm, which spans the head, then runs as a second
// kernel over an fp32 scratch, and the new normaliser and maximum wait in
// scratch until then: a part that starts late must still find the old ones.
#include "mix_common.h"

#define LS_GLA 0
#define LS_SSD 1
#define LS_MLSTM 2

PS_DEV float ls_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

PS_DEV float ls_log_sigmoid(float z) {
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

template <typename T, typename TO, int MODE, int DKP, int TILE, int P,
          int MAXT>
__global__ __launch_bounds__(MAXT) void linear_scan_kernel(
    TO* __restrict__ out, int ldo, const T* __restrict__ q, int ldq,
    const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const T* __restrict__ dec, int lddec, const T* __restrict__ wr, int ldwr,
    const T* __restrict__ gate, int ldg, const float* __restrict__ p0,
    const float* __restrict__ p1, const float* __restrict__ p2,
    const float* __restrict__ normw, float* __restrict__ state,
    float* __restrict__ aux, const int* __restrict__ seq_rows, int H, int G,
    int D, int DV, float eps, float qscale, float c0, int CS, int DVB,
    float* __restrict__ raw, float* __restrict__ naux) {
  extern __shared__ __align__(16) float lds[];
  constexpr int R = DKP / P;        // rows per lane
  constexpr int RP = P > 1 ? R + 4 : R;
  constexpr int TP = RP * P;        // words per token and array
  float* sk = lds;                  // [TILE][TP] key
  float* sq = sk + TILE * TP;       // query * qscale
  float* sg = sq + TILE * TP;       // per-row decay (GLA only)
  float* red = sg + (MODE == LS_GLA ? TILE * TP : 0);  // [16][TILE]
  float* sdec = red + 16 * TILE;    // [TILE] per-token decay
  float* swr = sdec + TILE;         // [TILE] per-token write scale
  float* sem = swr + TILE;          // [TILE] exp(-m)
  float* snq = sem + TILE;          // [TILE] n.q

  // a head's value columns may be shared out over CS workgroups of DVB
  // columns each (block cb owns columns cb * DVB ...); every block of a
  // matrix-LSTM head carries its own copy of the normaliser column
  const int cb = blockIdx.x % CS, sh = blockIdx.x / CS;
  const int seg = sh / H, hd = sh % H;
  const int t0 = seq_rows[4 * seg + 0], n = seq_rows[4 * seg + 1];
  const int pos0 = seq_rows[4 * seg + 2], slot = seq_rows[4 * seg + 3];
  const int jl = threadIdx.x / P, p = threadIdx.x % P;
  const int nloc = min(DVB, DV - cb * DVB);           // columns of this block
  const int j = cb * DVB + jl;
  const bool vcol = jl < nloc;                        // a value column
  const bool ncol = MODE == LS_MLSTM && jl == nloc;   // the normaliser
  const bool col = vcol || ncol;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int hk = (hd / (H / G)) * D;  // channel offset of the q/k group
  const int hz = hd * D;              // channel offset of per-row decays
  const int hv = hd * DV;             // channel offset in v / gate / out
  const float rate = MODE == LS_SSD ? expf(p1[hd]) : 0.f;
  const float skip = MODE == LS_SSD ? p2[hd] : 0.f;

  float* Sg = state + ((size_t)slot * H + hd) * (size_t)D * DV;
  float* Ng = MODE == LS_MLSTM ? aux + ((size_t)slot * H + hd) * (D + 1)
                               : nullptr;
  // Where the new normaliser and maximum go. With shared-out columns the
  // other workgroups of the head may still have to read the old ones, so
  // the new ones wait in scratch until the read-out kernel has started.
  float* Nw = (MODE == LS_MLSTM && naux != nullptr)
                  ? naux + ((size_t)seg * H + hd) * (D + 1)
                  : Ng;
  float S[R];  // S[r] = row p + P * r of column j
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = p + P * r;
    float s = 0.f;
    if (i < D && pos0 != 0) {
      if (vcol) s = Sg[(size_t)i * DV + j];
      if (ncol) s = Ng[i];
    }
    S[r] = s;
  }
  float m_run = 0.f;  // thread 0 carries the running maximum
  if (MODE == LS_MLSTM && threadIdx.x == 0 && pos0 != 0) m_run = Ng[D];

  for (int tb = 0; tb < n; tb += TILE) {
    const int nt = min(TILE, n - tb);
    __syncthreads();  // previous tile's LDS reads are done
    // this tile's value and gate entries of column j: issued together, up
    // front, so their latency hides behind the preparation
    float vreg[TILE], greg[TILE];
#pragma unroll
    for (int tt = 0; tt < TILE; ++tt) {
      const size_t row = (size_t)(t0 + tb + min(tt, nt - 1));
      vreg[tt] = vcol ? MxElem<T>::ld(v + row * ldv + hv + j) : 1.f;
      greg[tt] = vcol ? MxElem<T>::ld(gate + row * ldg + hv + j) : 0.f;
    }
    for (int idx = threadIdx.x; idx < nt * DKP; idx += blockDim.x) {
      const int tt = idx / DKP, i = idx % DKP;
      // row i is kept at (i % P) * RP + i / P: a lane's rows are contiguous
      const int at = tt * TP + (i % P) * RP + i / P;
      float kv = 0.f, qv = 0.f, gv = 0.f;
      if (i < D) {
        const size_t row = (size_t)(t0 + tb + tt);
        kv = MxElem<T>::ld(k + row * ldk + hk + i);
        qv = MxElem<T>::ld(q + row * ldq + hk + i) * qscale;
        if (MODE == LS_GLA) {
          const float z = MxElem<T>::ld(dec + row * lddec + hz + i);
          gv = expf(ls_log_sigmoid(z + p0[hz + i]) * c0);
        }
      }
      sk[at] = kv;
      sq[at] = qv;
      if (MODE == LS_GLA) sg[at] = gv;
    }
    if (threadIdx.x < nt) {
      const size_t row = (size_t)(t0 + tb + threadIdx.x);
      if (MODE == LS_SSD) {
        const float dt =
            ls_softplus(MxElem<T>::ld(dec + row * lddec + hd) + p0[hd]);
        sdec[threadIdx.x] = expf(-rate * dt);
        swr[threadIdx.x] = dt;
      } else if (MODE == LS_MLSTM) {
        // raw gates; thread 0 turns them into decay / write scale below
        const float zi = MxElem<T>::ld(wr + row * ldwr + hd) + p0[hd];
        const float zf = MxElem<T>::ld(dec + row * lddec + hd) + p1[hd];
        swr[threadIdx.x] = c0 * tanhf(zi / c0);
        sdec[threadIdx.x] = ls_log_sigmoid(c0 * tanhf(zf / c0));
      } else {
        swr[threadIdx.x] = 1.f;
      }
    }
    if (MODE == LS_MLSTM) {
      __syncthreads();
      if (threadIdx.x == 0) {
        for (int tt = 0; tt < nt; ++tt) {
          const float ig = swr[tt], fg = sdec[tt];
          const float mn = fmaxf(fg + m_run, ig);
          sdec[tt] = expf(fg + m_run - mn);
          swr[tt] = expf(ig - mn);
          sem[tt] = expf(-mn);
          m_run = mn;
        }
      }
    }
    __syncthreads();

    float o[TILE];
#pragma unroll
    for (int tt = 0; tt < TILE; ++tt) {
      o[tt] = 0.f;
      if (tt < nt) {
        const float4* pk = (const float4*)(sk + tt * TP + p * RP);
        const float4* pq = (const float4*)(sq + tt * TP + p * RP);
        const float4* pg = (const float4*)(sg + tt * TP + p * RP);
        const float u = swr[tt] * vreg[tt];
        const float a = MODE == LS_GLA ? 0.f : sdec[tt];
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < R / 4; ++i) {
          const float4 k4 = pk[i], q4 = pq[i];
          float gv[4] = {a, a, a, a};
          if (MODE == LS_GLA) {
            const float4 g4 = pg[i];
            gv[0] = g4.x;
            gv[1] = g4.y;
            gv[2] = g4.z;
            gv[3] = g4.w;
          }
          const float kv[4] = {k4.x, k4.y, k4.z, k4.w};
          const float qv[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float s = gv[e] * S[4 * i + e] + kv[e] * u;
            S[4 * i + e] = s;
            acc += s * qv[e];
          }
        }
#pragma unroll
        for (int off = 1; off < P; off <<= 1) acc += __shfl_xor(acc, off, 64);
        o[tt] = acc;
      }
    }

    if (MODE == LS_SSD) {
      if (vcol && p == 0) {
#pragma unroll
        for (int tt = 0; tt < TILE; ++tt) {
          if (tt < nt) {
            const size_t row = (size_t)(t0 + tb + tt);
            const float g = greg[tt];
            MxElem<TO>::st(out + row * ldo + hv + j,
                           (o[tt] + skip * vreg[tt]) * g * mx_sigmoid(g));
          }
        }
      }
      continue;
    }
    if (MODE == LS_MLSTM) {
      if (ncol && p == 0) {
#pragma unroll
        for (int tt = 0; tt < TILE; ++tt)
          if (tt < nt) snq[tt] = o[tt];
      }
      __syncthreads();
#pragma unroll
      for (int tt = 0; tt < TILE; ++tt)
        if (tt < nt) o[tt] /= fmaxf(fabsf(snq[tt]), sem[tt]) + 1e-6f;
    }
    if (raw != nullptr) {
      // the head's columns are spread over several workgroups: its norm is
      // taken by the read-out kernel
      if (vcol && p == 0) {
#pragma unroll
        for (int tt = 0; tt < TILE; ++tt)
          if (tt < nt)
            raw[(size_t)(t0 + tb + tt) * ((size_t)H * DV) + hv + j] = o[tt];
      }
      continue;
    }
    // per-token sum over the head's value columns of o^2
#pragma unroll
    for (int tt = 0; tt < TILE; ++tt) {
      const float s2 = mx_wave_sum((vcol && p == 0) ? o[tt] * o[tt] : 0.f);
      if (lane == 0) red[wave * TILE + tt] = s2;
    }
    __syncthreads();
    if (vcol && p == 0) {
#pragma unroll
      for (int tt = 0; tt < TILE; ++tt) {
        if (tt < nt) {
          float ss = 0.f;
          for (int w = 0; w < nw; ++w) ss += red[w * TILE + tt];
          const size_t row = (size_t)(t0 + tb + tt);
          const float inv = 1.0f / sqrtf(ss / (float)DV + eps);
          const float g = greg[tt];
          const float y =
              MODE == LS_GLA
                  ? o[tt] * inv * normw[j] * g * mx_sigmoid(g)
                  : o[tt] * inv * normw[hv + j] * mx_sigmoid(g);
          MxElem<TO>::st(out + row * ldo + hv + j, y);
        }
      }
    }
  }
  if (col) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = p + P * r;
      if (i < D) {
        if (vcol) Sg[(size_t)i * DV + j] = S[r];
        if (ncol && cb == 0) Nw[i] = S[r];
      }
    }
  }
  if (MODE == LS_MLSTM && threadIdx.x == 0 && cb == 0) Nw[D] = m_run;
}

// Read-out of heads whose columns were spread over several workgroups: one
// wave per (token, head): o / rms_DV(o) * weight * gate.
template <typename T, int MODE>
__global__ __launch_bounds__(256) void scan_readout_kernel(
    T* __restrict__ out, int ldo, const float* __restrict__ raw,
    const T* __restrict__ gate, int ldg, const float* __restrict__ normw,
    int T_, int H, int DV, float eps, const float* __restrict__ naux,
    float* __restrict__ aux, const int* __restrict__ seq_rows, int S_,
    int D) {
  const int w = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (w >= T_ * H) return;
  if (naux != nullptr && w < S_ * H) {
    // the matrix LSTM's new normaliser and maximum move into their slot
    const int slot = seq_rows[4 * (w / H) + 3];
    const float* src = naux + (size_t)w * (D + 1);
    float* dst = aux + ((size_t)slot * H + w % H) * (D + 1);
    for (int c = lane; c <= D; c += 64) dst[c] = src[c];
  }
  const int t = w / H, hd = w % H, hv = hd * DV;
  const float* r = raw + (size_t)t * ((size_t)H * DV) + hv;
  float ss = 0.f;
  for (int c = lane; c < DV; c += 64) ss += r[c] * r[c];
  ss = mx_wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)DV + eps);
  for (int c = lane; c < DV; c += 64) {
    const float g = MxElem<T>::ld(gate + (size_t)t * ldg + hv + c);
    const float y = MODE == LS_GLA
                        ? r[c] * inv * normw[c] * g * mx_sigmoid(g)
                        : r[c] * inv * normw[hv + c] * mx_sigmoid(g);
    MxElem<T>::st(out + (size_t)t * ldo + hv + c, y);
  }
}

#define LS_ARGS                                                              \
  void *out, int ldo, const void *q, int ldq, const void *k, int ldk,        \
      const void *v, int ldv, const void *dec, int lddec, const void *wr,    \
      int ldwr, const void *gate, int ldg, const void *p0, const void *p1,   \
      const void *p2, const void *normw, void *state, void *aux,             \
      const void *seq_rows, int S_, int H, int G, int D, int DV, float eps,  \
      float qscale, float c0, int T_, void *raw, void *stream
#define LS_PASS                                                              \
  out, ldo, q, ldq, k, ldk, v, ldv, dec, lddec, wr, ldwr, gate, ldg, p0, p1, \
      p2, normw, state, aux, seq_rows, S_, H, G, D, DV, eps, qscale, c0,     \
      T_, raw, stream

// Key width as the kernels pad it (0: not built).
static int ls_pad(int D) {
  const int pads[] = {16, 32, 48, 64, 96, 128, 192, 256};
  for (int p : pads)
    if (D <= p) return p;
  return 0;
}

// How many workgroups share a head's value columns. A wide head as one
// workgroup puts up to 16 waves on one CU's LDS (24 16-byte broadcast reads
// per token and wave) and, at 128 registers a lane, spills; its columns are
// shared out over up to 8 workgroups as long as every part keeps four waves.
// The rule does not look at the batch, so a sequence takes the same path
// whatever runs beside it.
static int ls_splits(int mode, int S_, int H, int D, int DV) {
  (void)S_;
  (void)H;
  const int dkp = ls_pad(D);
  if (dkp == 0) return 1;
  const int P0 = dkp >= 64 ? 4 : (dkp >= 32 ? 2 : 1);
  if ((DV + (mode == LS_MLSTM ? 1 : 0)) * P0 > 1024) return 1;
  int cs = 1;
  while (cs < 8 && DV % (cs * 2) == 0 && (DV / (cs * 2)) * P0 >= 256) cs *= 2;
  return cs;
}

// P lanes share a state column. WIDE: only the 1024-thread bound is built
// (fallback forms are reached with more than 256 columns only).
template <typename T, typename TO, int MODE, int DKP, int P, bool WIDE>
static int launch_linear_scan_p(LS_ARGS, int CS) {
  constexpr int TILE = DKP <= 128 ? 16 : 8;
  const int DVB = DV / CS;  // CS divides DV (ls_splits)
  const int cols = DVB + (MODE == LS_MLSTM ? 1 : 0);
  const int threads = ((cols * P + 63) / 64) * 64;
  if (threads > 1024) return 1;
  float* rawp = (CS > 1 && MODE != LS_SSD) ? (float*)raw : nullptr;
  // scratch layout: [T_][H * DV] read-outs, then [S_][H][D + 1]
  float* nauxp = (rawp != nullptr && MODE == LS_MLSTM)
                     ? rawp + (size_t)T_ * H * DV
                     : nullptr;
  const size_t lds =
      (size_t)((MODE == LS_GLA ? 3 : 2) * TILE * (DKP + (P > 1 ? 4 * P : 0)) +
               16 * TILE + 4 * TILE) *
      sizeof(float);
#define LS_LAUNCH(MAXT)                                                      \
  hipLaunchKernelGGL(                                                        \
      (linear_scan_kernel<T, TO, MODE, DKP, TILE, P, MAXT>),                 \
      dim3(S_ * H * CS), dim3(threads), lds, (hipStream_t)stream, (TO*)out,  \
      ldo, (const T*)q, ldq, (const T*)k, ldk, (const T*)v, ldv,             \
      (const T*)dec, lddec, (const T*)wr, ldwr, (const T*)gate, ldg,         \
      (const float*)p0, (const float*)p1, (const float*)p2,                  \
      (const float*)normw, (float*)state, (float*)aux, (const int*)seq_rows, \
      H, G, D, DV, eps, qscale, c0, CS, DVB, rawp, nauxp)
  // the launch bound follows the thread count, so small launches keep a
  // lane's rows and the tile's outputs out of scratch
  bool small = false;
  if constexpr (!WIDE) small = threads <= 256;
  if (small) {
    if constexpr (!WIDE) LS_LAUNCH(256);
  } else {
    LS_LAUNCH(1024);
  }
#undef LS_LAUNCH
  if constexpr (MODE != LS_SSD) {
    if (rawp != nullptr) {
      const long waves = (long)T_ * H;
      hipLaunchKernelGGL((scan_readout_kernel<T, MODE>),
                         dim3((unsigned)((waves + 3) / 4)), dim3(256), 0,
                         (hipStream_t)stream, (T*)out, ldo, rawp,
                         (const T*)gate, ldg, (const float*)normw, T_, H, DV,
                         eps, nauxp, (float*)aux, (const int*)seq_rows, S_,
                         D);
    }
  }
  return 0;
}

template <typename T, typename TO, int MODE, int DKP>
static int launch_linear_scan(LS_ARGS) {
  // lanes per column: enough to keep a lane's rows within 32 registers
  // where the column count allows it; heads with more value columns than
  // fit a workgroup that way take fewer lanes per column (more rows, and
  // scratch, per lane: correct, not fast)
  constexpr int P0 = DKP >= 64 ? 4 : (DKP >= 32 ? 2 : 1);
  const int cols = DV + (MODE == LS_MLSTM ? 1 : 0);
  if (cols * P0 <= 1024) {
    // without the scratch buffer the read-out norm cannot be split
    const int CS = (raw != nullptr || MODE == LS_SSD)
                       ? ls_splits(MODE, S_, H, D, DV)
                       : 1;
    return launch_linear_scan_p<T, TO, MODE, DKP, P0, false>(LS_PASS, CS);
  }
  if constexpr (P0 >= 4) {
    if (cols * 2 <= 1024)
      return launch_linear_scan_p<T, TO, MODE, DKP, 2, true>(LS_PASS, 1);
  }
  if constexpr (P0 >= 2) {
    if (cols <= 1024)
      return launch_linear_scan_p<T, TO, MODE, DKP, 1, true>(LS_PASS, 1);
  }
  return 1;
}

#define LS_CASE(PAD) \
  if (D <= PAD) return launch_linear_scan<T, TO, MODE, PAD>(LS_PASS);

template <typename T, typename TO, int MODE>
static int dispatch_linear_scan(LS_ARGS) {
  LS_CASE(16)
  LS_CASE(32)
  LS_CASE(48)
  LS_CASE(64)
  LS_CASE(96)
  LS_CASE(128)
  LS_CASE(192)
  LS_CASE(256)
  return 1;  // key dim above 256: not built
}

// The file is compiled once per (law, element type) pair (LS_ONLY = law * 2
// + dtype code) so the head-size instantiations build in parallel; unit 0
// also carries the entry point.
#define LS_UNIT(NAME) extern "C" int NAME(LS_ARGS)
LS_UNIT(mx_linear_scan_gla_bf16);
LS_UNIT(mx_linear_scan_gla_f32);
LS_UNIT(mx_linear_scan_ssd_bf16);
LS_UNIT(mx_linear_scan_ssd_f32);
LS_UNIT(mx_linear_scan_mlstm_bf16);
LS_UNIT(mx_linear_scan_mlstm_f32);

#if !defined(LS_ONLY) || LS_ONLY == 0
LS_UNIT(mx_linear_scan_gla_bf16) {
  return dispatch_linear_scan<mx_bf16, mx_bf16, LS_GLA>(LS_PASS);
}
#endif
#if !defined(LS_ONLY) || LS_ONLY == 1
LS_UNIT(mx_linear_scan_gla_f32) {
  return dispatch_linear_scan<float, float, LS_GLA>(LS_PASS);
}
#endif
#if !defined(LS_ONLY) || LS_ONLY == 2
LS_UNIT(mx_linear_scan_ssd_bf16) {
  return dispatch_linear_scan<mx_bf16, float, LS_SSD>(LS_PASS);
}
#endif
#if !defined(LS_ONLY) || LS_ONLY == 3
LS_UNIT(mx_linear_scan_ssd_f32) {
  return dispatch_linear_scan<float, float, LS_SSD>(LS_PASS);
}
#endif
#if !defined(LS_ONLY) || LS_ONLY == 4
LS_UNIT(mx_linear_scan_mlstm_bf16) {
  return dispatch_linear_scan<mx_bf16, mx_bf16, LS_MLSTM>(LS_PASS);
}
#endif
#if !defined(LS_ONLY) || LS_ONLY == 5
LS_UNIT(mx_linear_scan_mlstm_f32) {
  return dispatch_linear_scan<float, float, LS_MLSTM>(LS_PASS);
}
#endif

#if !defined(LS_ONLY) || LS_ONLY == 0
extern "C" int mx_linear_scan_splits(int mode, int S_, int H, int D,
                                     int DV) {
  return ls_splits(mode, S_, H, D, DV);
}

// raw: fp32 scratch of T_ * H * DV + S_ * H * (D + 1) entries, needed when
// mx_linear_scan_splits says a head's columns are shared out (ignored
// otherwise; without it the launch is not split).
extern "C" int mx_linear_scan(
    int mode, void* out, int ldo, const void* q, int ldq, const void* k,
    int ldk, const void* v, int ldv, const void* dec, int lddec,
    const void* wr, int ldwr, const void* gate, int ldg, const void* p0,
    const void* p1, const void* p2, const void* normw, void* state, void* aux,
    const void* seq_rows, int S_, int H, int G, int D, int DV, float eps,
    float qscale, float c0, int T_, void* raw, int dtype, void* stream) {
  if (S_ <= 0) return 0;
  if (G < 1 || H % G) return 2;
  const bool bf = dtype == MX_BF16;
  switch (mode) {
    case LS_GLA:
      return bf ? mx_linear_scan_gla_bf16(LS_PASS)
                : mx_linear_scan_gla_f32(LS_PASS);
    case LS_SSD:
      return bf ? mx_linear_scan_ssd_bf16(LS_PASS)
                : mx_linear_scan_ssd_f32(LS_PASS);
    case LS_MLSTM:
      if (aux == nullptr) return 2;
      return bf ? mx_linear_scan_mlstm_bf16(LS_PASS)
                : mx_linear_scan_mlstm_f32(LS_PASS);
  }
  return 2;
}
#endif
