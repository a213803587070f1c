// Paged attention with head-mixed ("talking") scores, aligned-chunk and
// trailing-window visibility (optionally keeping a sequence's first keys
// visible behind the window), capped scores and an optional denominator
// sink (score 0 or a learned per-head score). The values may be the leading
// entries of wider cache rows, so keys that carry their values (latent
// attention) need one cache. With a window, blocks of `pool` consecutive
// positions that lie wholly before a query's window can stay visible through
// one pooled key/value each (TaOpt::kp / vp): block b is seen by a query at
// position p when (b + 1) * pool <= p - window + 1, and lives in the page of
// its first position at row (first position mod BS) div pool of a pooled
// cache with ceil(BS / pool) rows per page. The kernels walk three key
// ranges in turn: kept first keys, pooled blocks, window.
//
// One launch covers a ragged batch: every token carries (its sequence's
// block-table row, its position); keys and values come from the paged
// cache, which already holds the token's own key. Because the score mix
//     s'_h = sum_g talk[h, g] * s_g
// couples all heads of one (query, key) pair before the softmax, a
// workgroup owns one query token with ALL its heads: per key tile it
// computes the raw scores of every head, mixes them, runs an online
// softmax per mixed head (the sink enters as an initial maximum of 0 with
// denominator 1 and no value) and accumulates P.V per head. Scores,
// weights and accumulators are fp32 in LDS.
#include "mix_common.h"

#define TA_KT 32

// Options beyond the basic shape. keep_first: keys [0, keep_first) stay
// visible to every later query; softcap > 0: score <- cap * tanh(score /
// cap), after the head mix; sink_vals: per-head sink scores (nullptr: 0);
// vr: elements per row of the value cache (>= DV).
struct TaOpt {
  int keep_first;
  float softcap;
  const float* sink_vals;
  int vr;
  const void* kp;  // pooled keys [NB, G, pr, D] (nullptr: none)
  const void* vp;  // pooled values [NB, G, pr, DV]
  int pool;        // positions per pooled block
  int pr;          // pooled rows per page
};

// Pooled blocks a query at position pos sees behind its window.
PS_DEV int ta_pool_count(int pos, int window, int pool) {
  const int past = pos - window + 1;  // positions before the window
  return (pool > 0 && window > 0 && past > 0) ? past / pool : 0;
}

// Row of key j in a paged cache with R rows per page, each row standing for
// P positions (the key/value cache: P = 1, R = BS).
PS_DEV int64_t ta_row(const int* __restrict__ table, int j, int G, int g,
                      int BS, int P, int R) {
  if (P == 1) return ((int64_t)table[j / BS] * G + g) * BS + (j % BS);
  const int pos = j * P;
  return ((int64_t)table[pos / BS] * G + g) * R + (pos % BS) / P;
}

PS_DEV float ta_cap(float sc, float cap) {
  return cap > 0.f ? cap * tanhf(sc / cap) : sc;
}

// Dynamic LDS a kernel may ask for: gfx950 has 160 KB per CU, but a launch
// above 64 KB needs the limit raised per kernel first. Falls back to 64 KB
// when the runtime refuses.
static size_t ta_lds_budget(const void* fn) {
  const int want = 160 * 1024;
  if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                          want) == hipSuccess)
    return (size_t)want;
  (void)hipGetLastError();
  return 64 * 1024;
}

template <typename T>
__global__ __launch_bounds__(256) void talk_attn_kernel(
    T* __restrict__ out, int ldout, const T* __restrict__ q, int ldq,
    const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ token_seq, const int* __restrict__ token_pos,
    const float* __restrict__ talk, int HT, int G, int D, int DV, int BS,
    float scale, int chunk, int window, int sink, TaOpt opt, int HB) {
  // Without a head mix the heads are independent: a workgroup then takes
  // the HB heads from blockIdx.y * HB on (HT heads in all), which bounds
  // the LDS need for wide heads. With a mix HB == HT.
  extern __shared__ float lds[];
  const int h0 = blockIdx.y * HB;
  const int H = min(HB, HT - h0);
  const int rep = HT / G;
  q += h0 * D;
  out += h0 * DV;
  if (opt.sink_vals) opt.sink_vals += h0;
  float* sq = lds;                 // [H*D]
  float* ss = sq + H * D;          // [H][KT] raw scores
  float* sp = ss + H * TA_KT;      // [H][KT] mixed scores -> weights
  float* sacc = sp + H * TA_KT;    // [H*DV]
  float* sm = sacc + H * DV;       // [H] running max
  float* sl = sm + H;              // [H] running denominator
  float* sal = sl + H;             // [H] rescale of this tile
  float* stk = sal + H;            // [H*H]

  const int t = blockIdx.x;
  const int pos = token_pos[t];
  const int* table = block_tables + (size_t)token_seq[t] * max_blocks;
  int lo = 0;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0) lo = max(lo, pos - window + 1);

  for (int c = threadIdx.x; c < H * D; c += blockDim.x)
    sq[c] = MxElem<T>::ld(q + (size_t)t * ldq + c);
  for (int c = threadIdx.x; c < H * DV; c += blockDim.x) sacc[c] = 0.f;
  if (talk != nullptr)
    for (int c = threadIdx.x; c < H * H; c += blockDim.x) stk[c] = talk[c];
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    sm[h] = sink ? (opt.sink_vals ? opt.sink_vals[h] : 0.f) : PS_NEG_INF;
    sl[h] = sink ? 1.f : 0.f;
  }
  __syncthreads();

  // key ranges: the kept first keys behind the window, the pooled blocks
  // behind it, then the window
  const int npool = opt.kp ? ta_pool_count(pos, window, opt.pool) : 0;
  for (int rg = 0; rg < 3; ++rg) {
  const int ra = rg == 2 ? lo : 0;
  const int rb = rg == 0 ? min(opt.keep_first, lo) - 1
                         : (rg == 1 ? npool - 1 : pos);
  const T* kcr = rg == 1 ? (const T*)opt.kp : kc;
  const T* vcr = rg == 1 ? (const T*)opt.vp : vc;
  const int cP = rg == 1 ? opt.pool : 1, cR = rg == 1 ? opt.pr : BS;
  const int cvr = rg == 1 ? DV : opt.vr;
  for (int j0 = ra; j0 <= rb; j0 += TA_KT) {
    const int nk = min(TA_KT, rb + 1 - j0);
    // raw scores of every (head, key) pair of the tile
    for (int it = threadIdx.x; it < H * nk; it += blockDim.x) {
      const int jj = it / H, h = it % H;
      const int j = j0 + jj;
      const T* kr =
          kcr + ta_row(table, j, G, (h0 + h) / rep, BS, cP, cR) * (int64_t)D;
      const float* qh = sq + h * D;
      float acc = 0.f;
      for (int d = 0; d < D; ++d) acc += qh[d] * MxElem<T>::ld(kr + d);
      ss[h * TA_KT + jj] = acc * scale;
    }
    __syncthreads();
    // mix across heads
    for (int it = threadIdx.x; it < H * nk; it += blockDim.x) {
      const int jj = it / H, h = it % H;
      float m;
      if (talk != nullptr) {
        m = 0.f;
        for (int g2 = 0; g2 < H; ++g2)
          m += stk[h * H + g2] * ss[g2 * TA_KT + jj];
      } else {
        m = ss[h * TA_KT + jj];
      }
      sp[h * TA_KT + jj] = ta_cap(m, opt.softcap);
    }
    __syncthreads();
    // online softmax bookkeeping: one thread per head
    for (int h = threadIdx.x; h < H; h += blockDim.x) {
      float mx = sm[h];
      for (int jj = 0; jj < nk; ++jj) mx = fmaxf(mx, sp[h * TA_KT + jj]);
      const float alpha = expf(sm[h] - mx);
      float l = sl[h] * alpha;
      for (int jj = 0; jj < nk; ++jj) {
        const float p = expf(sp[h * TA_KT + jj] - mx);
        sp[h * TA_KT + jj] = p;
        l += p;
      }
      sm[h] = mx;
      sl[h] = l;
      sal[h] = alpha;
    }
    __syncthreads();
    // P.V
    for (int it = threadIdx.x; it < H * DV; it += blockDim.x) {
      const int h = it / DV, d = it % DV;
      const int gk = (h0 + h) / rep;
      float acc = sacc[it] * sal[h];
      for (int jj = 0; jj < nk; ++jj) {
        const int j = j0 + jj;
        acc += sp[h * TA_KT + jj] *
               MxElem<T>::ld(vcr + ta_row(table, j, G, gk, BS, cP, cR) *
                                       (int64_t)cvr + d);
      }
      sacc[it] = acc;
    }
    __syncthreads();
  }
  }
  for (int it = threadIdx.x; it < H * DV; it += blockDim.x)
    MxElem<T>::st(out + (size_t)t * ldout + it, sacc[it] / sl[it / DV]);
}

// Stage nk keys x G kv heads of one cache (rows of Dw elements) into LDS as
// fp32 rows of PITCH floats, columns [Dw, DP) zeroed. Rows are read with
// 16-byte loads, several in flight per thread before any is consumed (the
// kernels run one wave per SIMD, so nothing else hides the latency).
template <typename T>
struct TaVec;
template <>
struct TaVec<float> {
  static constexpr int N = 4;
  static PS_DEV void put(float* dst, const float4& v) {
    *(float4*)dst = v;
  }
};
template <>
struct TaVec<mx_bf16> {
  static constexpr int N = 8;
  static PS_DEV void put(float* dst, const float4& v) {
    const unsigned int* u = (const unsigned int*)&v;
    float4 a, b;
    a.x = __uint_as_float(u[0] << 16);
    a.y = __uint_as_float(u[0] & 0xffff0000u);
    a.z = __uint_as_float(u[1] << 16);
    a.w = __uint_as_float(u[1] & 0xffff0000u);
    b.x = __uint_as_float(u[2] << 16);
    b.y = __uint_as_float(u[2] & 0xffff0000u);
    b.z = __uint_as_float(u[3] << 16);
    b.w = __uint_as_float(u[3] & 0xffff0000u);
    *(float4*)dst = a;
    *(float4*)(dst + 4) = b;
  }
};

template <typename T, int DP, int PITCH>
PS_DEV void ta_stage(float* __restrict__ sdst, const T* __restrict__ cache,
                     const int* __restrict__ table, int j0, int nk, int G,
                     int Dw, int BS, int RW, int P = 1, int R = 0) {
  if (R == 0) R = BS;
  // Dw elements of every cache row of RW elements are staged
  constexpr int VEC = TaVec<T>::N;
  constexpr int U = 8;
  const int tid = threadIdx.x, nt = blockDim.x;
  if (Dw % VEC == 0 && RW % VEC == 0) {
    const int vpr = Dw / VEC;
    const int total = nk * G * vpr;
    for (int base = 0; base < total; base += nt * U) {
      float4 buf[U];
      int off[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int idx = base + u * nt + tid;
        off[u] = -1;
        if (idx < total) {
          const int row = idx / vpr, c = idx - row * vpr;
          const int jj = row / G, g = row - jj * G;
          const int j = j0 + jj;
          const int64_t gb = ta_row(table, j, G, g, BS, P, R);
          buf[u] = *(const float4*)(cache + gb * RW + c * VEC);
          off[u] = row * PITCH + c * VEC;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (off[u] >= 0) TaVec<T>::put(sdst + off[u], buf[u]);
    }
    if (Dw < DP) {
      const int pad = DP - Dw;
      for (int e = tid; e < nk * G * pad; e += nt) {
        const int row = e / pad, d = Dw + e - row * pad;
        sdst[row * PITCH + d] = 0.f;
      }
    }
  } else {
    for (int e = tid; e < nk * G * DP; e += nt) {
      const int d = e % DP, row = e / DP;
      const int jj = row / G, g = row - jj * G;
      const int j = j0 + jj;
      const int64_t gb = ta_row(table, j, G, g, BS, P, R);
      sdst[row * PITCH + d] = d < Dw ? MxElem<T>::ld(cache + gb * RW + d) : 0.f;
    }
  }
}

// ---------------------------------------------------------------------------
// Tiled variant: one thread per (head, query) pair.
//
// A workgroup takes QT = 256 / H consecutive batch rows with all H heads;
// thread (h, i) keeps its query vector and its output accumulator in
// registers (DP floats each, head widths padded up to DP). Rows of the
// group that continue one sequence at consecutive positions form a run; a
// run shares every key/value tile, staged once into LDS as fp32 and read by
// the threads as wave-wide broadcasts (lanes of a wave hold few distinct
// heads). Per tile: raw scores -> LDS, head mix from LDS, one online-softmax
// rescale, P.V from the LDS value rows. Single decode tokens are runs of
// one row.
template <typename T, int DP>
__global__ __launch_bounds__(256) void talk_attn_tiled_kernel(
    T* __restrict__ out, int ldout, const T* __restrict__ q, int ldq,
    const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ token_seq, const int* __restrict__ token_pos,
    const float* __restrict__ talk, int T_total, int H, int G, int D, int DV,
    int BS, float scale, int chunk, int window, int sink, int QT, int KT,
    TaOpt opt) {
  extern __shared__ float lds[];
  const int NP = H * QT;
  float* sK = lds;                   // [KT][G][DP]
  float* sV = sK + KT * G * DP;      // [KT][G][DP]
  float* sS = sV + KT * G * DP;      // [KT][NP] raw scores
  float* sM = sS + KT * NP;          // [KT][NP] mixed scores
  float* sT = sM + KT * NP;          // [H*H]
  int* s_seq = (int*)(sT + H * H);   // [QT]
  int* s_pos = s_seq + QT;           // [QT]

  const int tid = threadIdx.x;
  const int row0 = blockIdx.x * QT;
  const int nrows = min(QT, T_total - row0);
  const int h = tid / QT, i = tid % QT;
  const bool valid = tid < NP && i < nrows;
  const int rep = H / G;
  const int gk = valid ? h / rep : 0;

  for (int c = tid; c < nrows; c += blockDim.x) {
    s_seq[c] = token_seq[row0 + c];
    s_pos[c] = token_pos[row0 + c];
  }
  if (talk != nullptr)
    for (int c = tid; c < H * H; c += blockDim.x) sT[c] = talk[c];

  float qv[DP], acc[DP];
#pragma unroll
  for (int d = 0; d < DP; ++d) {
    qv[d] = (valid && d < D)
                ? MxElem<T>::ld(q + (size_t)(row0 + i) * ldq + h * D + d)
                : 0.f;
    acc[d] = 0.f;
  }
  float m = sink ? ((opt.sink_vals && valid) ? opt.sink_vals[h] : 0.f)
                 : PS_NEG_INF;
  float l = sink ? 1.f : 0.f;
  __syncthreads();
  const int my_pos = valid ? s_pos[i] : 0;
  int my_lo = 0;
  if (chunk > 0) my_lo = (my_pos / chunk) * chunk;
  if (window > 0) my_lo = max(my_lo, my_pos - window + 1);
  const int my_pool = opt.kp ? ta_pool_count(my_pos, window, opt.pool) : 0;

  int rs = 0;
  while (rs < nrows) {
    int re = rs + 1;
    while (re < nrows && s_seq[re] == s_seq[rs] &&
           s_pos[re] == s_pos[re - 1] + 1)
      ++re;
    const bool mine = valid && i >= rs && i < re;
    const int* table = block_tables + (size_t)s_seq[rs] * max_blocks;
    int kmin = 0;
    if (chunk > 0) kmin = (s_pos[rs] / chunk) * chunk;
    if (window > 0) kmin = max(kmin, s_pos[rs] - window + 1);
    const int kmax = s_pos[re - 1];

    // kept first keys behind the run's earliest window, the pooled blocks
    // its last row sees, then the windows
    const int run_pool =
        opt.kp ? ta_pool_count(s_pos[re - 1], window, opt.pool) : 0;
    for (int rg = 0; rg < 3; ++rg) {
    const int ra = rg == 2 ? kmin : 0;
    const int rb = rg == 0 ? min(opt.keep_first, kmin) - 1
                           : (rg == 1 ? run_pool - 1 : kmax);
    for (int j0 = ra; j0 <= rb; j0 += KT) {
      const int nk = min(KT, rb + 1 - j0);
      __syncthreads();  // the previous tile is fully consumed
      if (rg == 1) {
        ta_stage<T, DP, DP>(sK, (const T*)opt.kp, table, j0, nk, G, D, BS, D,
                            opt.pool, opt.pr);
        ta_stage<T, DP, DP>(sV, (const T*)opt.vp, table, j0, nk, G, DV, BS,
                            DV, opt.pool, opt.pr);
      } else {
        ta_stage<T, DP, DP>(sK, kc, table, j0, nk, G, D, BS, D);
        ta_stage<T, DP, DP>(sV, vc, table, j0, nk, G, DV, BS, opt.vr);
      }
      __syncthreads();
      if (mine) {
        for (int jj = 0; jj < nk; ++jj) {
          const float4* kr = (const float4*)(sK + (jj * G + gk) * DP);
          float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
          for (int d4 = 0; d4 < DP / 4; ++d4) {
            const float4 kk = kr[d4];
            a0 += qv[4 * d4 + 0] * kk.x;
            a1 += qv[4 * d4 + 1] * kk.y;
            a2 += qv[4 * d4 + 2] * kk.z;
            a3 += qv[4 * d4 + 3] * kk.w;
          }
          sS[jj * NP + tid] = ((a0 + a1) + (a2 + a3)) * scale;
        }
      }
      __syncthreads();
      if (mine) {
        float mx = m;
        for (int jj = 0; jj < nk; ++jj) {
          float sc;
          if (talk != nullptr) {
            sc = 0.f;
            const float* tr = sT + h * H;
            const float* sr = sS + jj * NP + i;
            for (int g2 = 0; g2 < H; ++g2) sc += tr[g2] * sr[g2 * QT];
          } else {
            sc = sS[jj * NP + tid];
          }
          sc = ta_cap(sc, opt.softcap);
          const int j = j0 + jj;
          if (rg == 1 ? j >= my_pool
                      : (j > my_pos || (j < my_lo && j >= opt.keep_first)))
            sc = PS_NEG_INF;
          sM[jj * NP + tid] = sc;
          mx = fmaxf(mx, sc);
        }
        if (mx > PS_NEG_INF) {
          const float alpha = expf(m - mx);  // m = -inf gives 0
          if (alpha != 1.f) {
            l *= alpha;
#pragma unroll
            for (int d = 0; d < DP; ++d) acc[d] *= alpha;
          }
          m = mx;
          for (int jj = 0; jj < nk; ++jj) {
            const float sc = sM[jj * NP + tid];
            if (sc > PS_NEG_INF) {
              const float p = expf(sc - mx);
              l += p;
              const float4* vr = (const float4*)(sV + (jj * G + gk) * DP);
#pragma unroll
              for (int d4 = 0; d4 < DP / 4; ++d4) {
                const float4 vv = vr[d4];
                acc[4 * d4 + 0] += p * vv.x;
                acc[4 * d4 + 1] += p * vv.y;
                acc[4 * d4 + 2] += p * vv.z;
                acc[4 * d4 + 3] += p * vv.w;
              }
            }
          }
        }
      }
    }
    }
    rs = re;
  }
  if (valid) {
    const float inv = 1.0f / l;
    T* o = out + (size_t)(row0 + i) * ldout + h * DV;
#pragma unroll
    for (int d = 0; d < DP; ++d)
      if (d < DV) MxElem<T>::st(o + d, acc[d] * inv);
  }
}

template <typename T, int DP>
static int launch_tiled(void* out, int ldout, const void* q, int ldq,
                        const void* kc, const void* vc,
                        const void* block_tables, int max_blocks,
                        const void* token_seq, const void* token_pos,
                        const void* talk, int T_, int H, int G, int D, int DV,
                        int BS, float scale, int chunk, int window, int sink,
                        TaOpt opt, hipStream_t stream) {
  static const size_t budget =
      ta_lds_budget((const void*)talk_attn_tiled_kernel<T, DP>);
  const int QT = 256 / H, NP = H * QT;
  int KT = 32;
  size_t lds = 0;
  for (; KT >= 1; KT >>= 1) {
    lds = ((size_t)2 * KT * G * DP + (size_t)2 * KT * NP + (size_t)H * H +
           2 * QT) * sizeof(float);
    if (lds <= budget) break;
  }
  if (KT < 1) return 1;
  hipLaunchKernelGGL((talk_attn_tiled_kernel<T, DP>),
                     dim3((T_ + QT - 1) / QT), dim3(256), lds, stream,
                     (T*)out, ldout, (const T*)q, ldq, (const T*)kc,
                     (const T*)vc, (const int*)block_tables, max_blocks,
                     (const int*)token_seq, (const int*)token_pos,
                     (const float*)talk, T_, H, G, D, DV, BS, scale, chunk,
                     window, sink, QT, KT, opt);
  return 0;
}

// ---------------------------------------------------------------------------
// Split-key variant for single tokens (decode): one workgroup per token,
// thread (h, i) owns head h and key slice i of NS = 256 / H slices. Every
// tile stages NS * KPT keys (all kv heads, fp32, rows padded against bank
// conflicts) into LDS; thread (h, i) scores key c * NS + i of the tile for
// its head, the heads' raw scores meet in LDS for the mix, and each thread
// runs its own online softmax over its keys with the output accumulator in
// registers. The NS partial results of a head are merged at the end. The
// sink belongs to slice 0.
template <typename T, int DP>
__global__ __launch_bounds__(256) void talk_attn_split_kernel(
    T* __restrict__ out, int ldout, const T* __restrict__ q, int ldq,
    const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ token_seq, const int* __restrict__ token_pos,
    const float* __restrict__ talk, int H, int G, int D, int DV, int BS,
    float scale, int chunk, int window, int sink, int NS, int KPT, int KS,
    float* __restrict__ part, TaOpt opt) {
  extern __shared__ float lds[];
  constexpr int PITCH = DP + 4;
  const int TK = NS * KPT;           // keys per tile
  float* sK = lds;                   // [TK][G][PITCH]
  float* sV = sK + TK * G * PITCH;   // [TK][G][PITCH]
  float* sS = sV + TK * G * PITCH;   // [TK][H] raw scores
  float* sT = sS + TK * H;           // [H*H]
  float* sML = sT + H * H;           // [2][H*NS] partial max / denominator
  float* sQ = sML + 2 * H * NS;      // [H][PITCH] query rows (fp32)
  // the merge buffer [H][DP] reuses sK after the key loop

  const int tid = threadIdx.x;
  const int t = blockIdx.x / KS, ks = blockIdx.x % KS;
  const int h = tid / NS, i = tid % NS;
  const bool valid = tid < H * NS;
  const int rep = H / G;
  const int gk = valid ? h / rep : 0;
  const int* table = block_tables + (size_t)token_seq[t] * max_blocks;
  int lo = 0, pos = token_pos[t];
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0) lo = max(lo, pos - window + 1);
  // the kept first keys and the pooled blocks behind the window go to
  // share 0
  const int kept = ks == 0 ? min(opt.keep_first, lo) : 0;
  const int npool =
      (ks == 0 && opt.kp) ? ta_pool_count(pos, window, opt.pool) : 0;
  if (KS > 1) {
    // this workgroup's share of the visible keys, in whole tiles
    const int tiles = (pos + 1 - lo + TK - 1) / TK;
    const int per = (tiles + KS - 1) / KS;
    const int first = lo + ks * per * TK;
    pos = min(pos, first + per * TK - 1);
    lo = first;  // may pass pos: then this share is empty
  }

  if (talk != nullptr)
    for (int c = tid; c < H * H; c += blockDim.x) sT[c] = talk[c];
  // the query stays in LDS (each thread scores only KPT keys a tile), so
  // the registers hold just the output accumulator
  for (int c = tid; c < H * DP; c += blockDim.x) {
    const int hh = c / DP, d = c % DP;
    sQ[hh * PITCH + d] =
        d < D ? MxElem<T>::ld(q + (size_t)t * ldq + hh * D + d) : 0.f;
  }
  float acc[DP];
#pragma unroll
  for (int d = 0; d < DP; ++d) acc[d] = 0.f;
  const bool own_sink = sink && i == 0 && ks == 0;
  float m = own_sink ? ((opt.sink_vals && valid) ? opt.sink_vals[h] : 0.f)
                     : PS_NEG_INF;
  float l = own_sink ? 1.f : 0.f;

  for (int rg = 0; rg < 3; ++rg) {
  const int ra = rg == 2 ? lo : 0;
  const int rb = rg == 0 ? kept - 1 : (rg == 1 ? npool - 1 : pos);
  for (int j0 = ra; j0 <= rb; j0 += TK) {
    const int nk = min(TK, rb + 1 - j0);
    __syncthreads();
    if (rg == 1) {
      ta_stage<T, DP, PITCH>(sK, (const T*)opt.kp, table, j0, nk, G, D, BS, D,
                             opt.pool, opt.pr);
      ta_stage<T, DP, PITCH>(sV, (const T*)opt.vp, table, j0, nk, G, DV, BS,
                             DV, opt.pool, opt.pr);
    } else {
      ta_stage<T, DP, PITCH>(sK, kc, table, j0, nk, G, D, BS, D);
      ta_stage<T, DP, PITCH>(sV, vc, table, j0, nk, G, DV, BS, opt.vr);
    }
    __syncthreads();
    if (valid) {
      for (int c = 0; c < KPT; ++c) {
        const int jj = c * NS + i;
        if (jj < nk) {
          const float4* kr = (const float4*)(sK + (jj * G + gk) * PITCH);
          const float4* qr = (const float4*)(sQ + h * PITCH);
          float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
          for (int d4 = 0; d4 < DP / 4; ++d4) {
            const float4 kk = kr[d4], qq = qr[d4];
            a0 += qq.x * kk.x;
            a1 += qq.y * kk.y;
            a2 += qq.z * kk.z;
            a3 += qq.w * kk.w;
          }
          sS[jj * H + h] = ((a0 + a1) + (a2 + a3)) * scale;
        }
      }
    }
    __syncthreads();
    if (valid) {
      for (int c = 0; c < KPT; ++c) {
        const int jj = c * NS + i;
        if (jj < nk) {
          float sc;
          if (talk != nullptr) {
            sc = 0.f;
            const float* tr = sT + h * H;
            const float* sr = sS + jj * H;
            for (int g2 = 0; g2 < H; ++g2) sc += tr[g2] * sr[g2];
          } else {
            sc = sS[jj * H + h];
          }
          sc = ta_cap(sc, opt.softcap);
          const float mx = fmaxf(m, sc);
          const float alpha = expf(m - mx);  // m = -inf gives 0
          const float p = expf(sc - mx);
          l = l * alpha + p;
          m = mx;
          const float4* vr = (const float4*)(sV + (jj * G + gk) * PITCH);
#pragma unroll
          for (int d4 = 0; d4 < DP / 4; ++d4) {
            const float4 vv = vr[d4];
            acc[4 * d4 + 0] = acc[4 * d4 + 0] * alpha + p * vv.x;
            acc[4 * d4 + 1] = acc[4 * d4 + 1] * alpha + p * vv.y;
            acc[4 * d4 + 2] = acc[4 * d4 + 2] * alpha + p * vv.z;
            acc[4 * d4 + 3] = acc[4 * d4 + 3] * alpha + p * vv.w;
          }
        }
      }
    }
  }
  }
  // merge the NS slices of each head
  __syncthreads();
  float* sOut = sK;  // [H][DP]
  if (valid) {
    sML[tid] = m;
    sML[H * NS + tid] = l;
  }
  for (int c = tid; c < H * DP; c += blockDim.x) sOut[c] = 0.f;
  __syncthreads();
  float w = 0.f;
  float mh = PS_NEG_INF, lh = 0.f;
  if (valid) {
    for (int r = 0; r < NS; ++r) mh = fmaxf(mh, sML[h * NS + r]);
    for (int r = 0; r < NS; ++r) {
      const float mr = sML[h * NS + r];
      if (mr > PS_NEG_INF) lh += sML[H * NS + h * NS + r] * expf(mr - mh);
    }
    // one workgroup per token: normalise here; several: leave the sum
    // relative to mh for the combine kernel
    if (m > PS_NEG_INF) w = expf(m - mh) / (KS > 1 ? 1.f : lh);
  }
  for (int r = 0; r < NS; ++r) {
    if (valid && i == r && w != 0.f) {
#pragma unroll
      for (int d = 0; d < DP; ++d) sOut[h * DP + d] += acc[d] * w;
    }
    __syncthreads();
  }
  if (KS == 1) {
    for (int c = tid; c < H * DV; c += blockDim.x) {
      const int hh = c / DV, d = c % DV;
      MxElem<T>::st(out + (size_t)t * ldout + c, sOut[hh * DP + d]);
    }
  } else {
    // partial record per (token, share, head): max, denominator, DV sums
    float* rec = part + ((size_t)t * KS + ks) * H * (DV + 2);
    if (valid && i == 0) {
      rec[h * (DV + 2)] = mh;
      rec[h * (DV + 2) + 1] = lh;
    }
    for (int c = tid; c < H * DV; c += blockDim.x) {
      const int hh = c / DV, d = c % DV;
      rec[hh * (DV + 2) + 2 + d] = sOut[hh * DP + d];
    }
  }
}

// Merge the KS partial records of every (token, head).
template <typename T>
__global__ __launch_bounds__(256) void talk_attn_combine_kernel(
    T* __restrict__ out, int ldout, const float* __restrict__ part, int H,
    int DV, int KS) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < H * DV; c += blockDim.x) {
    const int h = c / DV, d = c % DV;
    const float* rec = part + (size_t)t * KS * H * (DV + 2) + h * (DV + 2);
    const size_t step = (size_t)H * (DV + 2);
    float mh = PS_NEG_INF;
    for (int s = 0; s < KS; ++s) mh = fmaxf(mh, rec[s * step]);
    float l = 0.f, a = 0.f;
    for (int s = 0; s < KS; ++s) {
      const float ms = rec[s * step];
      if (ms > PS_NEG_INF) {
        const float w = expf(ms - mh);
        l += rec[s * step + 1] * w;
        a += rec[s * step + 2 + d] * w;
      }
    }
    MxElem<T>::st(out + (size_t)t * ldout + c, a / l);
  }
}

template <typename T, int DP>
static int launch_split(void* out, int ldout, const void* q, int ldq,
                        const void* kc, const void* vc,
                        const void* block_tables, int max_blocks,
                        const void* token_seq, const void* token_pos,
                        const void* talk, int T_, int H, int G, int D, int DV,
                        int BS, float scale, int chunk, int window, int sink,
                        TaOpt opt, hipStream_t stream, int KS, float* part) {
  static const size_t budget =
      ta_lds_budget((const void*)talk_attn_split_kernel<T, DP>);
  if (KS < 1 || part == nullptr) KS = 1;
  int NS = 0, KPT = 0;
  size_t lds = 0;
  // most slices first (threads), then most keys per tile (fewer barriers)
  for (int ns = 256 / H; ns >= 1 && KPT == 0; ns >>= 1) {
    const size_t fixed =
        (size_t)H * H + 2 * H * ns + (size_t)H * (DP + 4);  // + query rows
    for (int k = 8; k >= 1; k >>= 1) {
      const size_t tk = (size_t)ns * k;
      size_t tile = 2 * tk * G * (DP + 4);
      if (tile < (size_t)H * DP) tile = (size_t)H * DP;  // merge buffer
      lds = (tile + tk * H + fixed) * sizeof(float);
      if (lds <= budget) {
        NS = ns;
        KPT = k;
        break;
      }
    }
  }
  if (KPT == 0) return 1;
  hipLaunchKernelGGL((talk_attn_split_kernel<T, DP>), dim3(T_ * KS),
                     dim3(256), lds, stream, (T*)out, ldout, (const T*)q, ldq,
                     (const T*)kc, (const T*)vc, (const int*)block_tables,
                     max_blocks, (const int*)token_seq,
                     (const int*)token_pos, (const float*)talk, H, G, D, DV,
                     BS, scale, chunk, window, sink, NS, KPT, KS, part, opt);
  if (KS > 1)
    hipLaunchKernelGGL((talk_attn_combine_kernel<T>), dim3(T_), dim3(256), 0,
                       stream, (T*)out, ldout, (const float*)part, H, DV, KS);
  return 0;
}

#define TA_BY_WIDTH(FN, rc, ...)                                               \
  MX_DISPATCH_DTYPE(dtype, {                                                 \
    if (dmax <= 32)                                                          \
      rc = FN<T, 32>(out, ldout, q, ldq, kc, vc, block_tables, max_blocks,   \
                     token_seq, token_pos, talk, T_, H, G, D, DV, BS, scale, \
                     chunk, window, sink, opt, (hipStream_t)stream,               \
                     ##__VA_ARGS__);                                         \
    else if (dmax <= 64)                                                     \
      rc = FN<T, 64>(out, ldout, q, ldq, kc, vc, block_tables, max_blocks,   \
                     token_seq, token_pos, talk, T_, H, G, D, DV, BS, scale, \
                     chunk, window, sink, opt, (hipStream_t)stream,               \
                     ##__VA_ARGS__);                                         \
    else                                                                     \
      rc = FN<T, 128>(out, ldout, q, ldq, kc, vc, block_tables, max_blocks,  \
                      token_seq, token_pos, talk, T_, H, G, D, DV, BS,       \
                      scale, chunk, window, sink, opt, (hipStream_t)stream,       \
                      ##__VA_ARGS__);                                        \
  })

// variant: 0 = pick for prompt portions (tiled where it fits), 3 = pick for
// single tokens (split-key where it fits), 1 = plain one-workgroup-per-token
// kernel, 2 = tiled only, 4 = split-key only
extern "C" int mx_talk_attention(void* out, int ldout, const void* q,
                                 int ldq, const void* kc, const void* vc,
                                 const void* block_tables, int max_blocks,
                                 const void* token_seq,
                                 const void* token_pos, const void* talk,
                                 int T_, int H, int G, int D, int DV, int BS,
                                 float scale, int chunk, int window,
                                 int sink, int dtype, int variant,
                                 int splits, void* scratch, int keep_first,
                                 float softcap, const void* sink_vals,
                                 int vrow, const void* kpool,
                                 const void* vpool, int pool, void* stream) {
  if (T_ <= 0) return 0;
  if (vrow < DV) return 3;
  const bool pooled = kpool != nullptr && pool > 0 && window > 0;
  const TaOpt opt = {keep_first > 0 ? keep_first : 0, softcap,
                     (const float*)sink_vals, vrow,
                     pooled ? kpool : nullptr, pooled ? vpool : nullptr,
                     pooled ? pool : 0, pooled ? (BS + pool - 1) / pool : 0};
  const int dmax = D > DV ? D : DV;
  if ((variant == 0 || variant == 2) && H <= 256 && dmax <= 128) {
    int rc = 1;
    TA_BY_WIDTH(launch_tiled, rc)
    if (rc == 0) return 0;
  }
  if ((variant == 3 || variant == 4) && H <= 256 && dmax <= 128) {
    int rc = 1;
    TA_BY_WIDTH(launch_split, rc, splits, (float*)scratch)
    if (rc == 0) return 0;
  }
  if (variant == 2 || variant == 4) return 2;
  // heads per workgroup: all of them with a head mix, otherwise as many as
  // fit 64 KB of LDS
  int HB = H;
  auto need = [&](int hb) {
    return (size_t)(hb * D + 2 * hb * TA_KT + hb * DV + 3 * hb +
                    (talk != nullptr ? H * H : 0)) * sizeof(float);
  };
  if (talk == nullptr)
    while (HB > 1 && need(HB) > 64 * 1024) HB = (HB + 1) / 2;
  const size_t lds = need(HB);
  if (lds > 64 * 1024) return 1;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((talk_attn_kernel<T>), dim3(T_, (H + HB - 1) / HB),
                       dim3(256), lds, (hipStream_t)stream, (T*)out, ldout,
                       (const T*)q, ldq, (const T*)kc, (const T*)vc,
                       (const int*)block_tables, max_blocks,
                       (const int*)token_seq, (const int*)token_pos,
                       (const float*)talk, H, G, D, DV, BS, scale, chunk,
                       window, sink, opt, HB);
  })
  return 0;
}
