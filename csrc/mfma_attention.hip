// Matrix-core paged attention for bf16 activations (gfx950, wave64).
//
// Covers what the fp32 vector kernels of talk_attention.hip cover except a
// head mix and aligned chunks: grouped-query or single-KV-head attention
// over the paged cache, trailing window with kept first keys, capped
// scores, denominator sink, values that are the leading entries of the key
// rows (latent attention: rows of several hundred entries), and pooled
// blocks behind the window (one mean key/value per block of `pool` positions
// that lies wholly before a query's window, read from a pooled cache that
// shares the pages of the key/value cache).
//
// A workgroup (4 waves) owns 32 rows = (tokens of consecutive batch rows) x
// (query heads of one KV head), so one staged key tile serves all of them.
// Both products run "swapped" on v_mfma_f32_32x32x16_bf16:
//     S^T[key, row] = K[key, :] . Q[row, :]^T
//     O^T[col, row] = V[:, col]^T . P[row, :]^T
// so every lane's accumulator entries belong to ONE row (lane & 31): the
// online softmax (running max, denominator, rescale) is lane-local plus one
// exchange with lane ^ 32, and P never leaves the registers. Two ways to
// share the work among the 4 waves:
//   column split (ROWS = 32): every wave computes the full S^T of the 32
//     rows and accumulates its own share of the value columns (column
//     blocks wave, wave + 4, ...): wide values (latent attention), and
//     single-token batches;
//   row split (ROWS = 128): the workgroup owns 128 rows, every wave 32 of
//     them with all value columns (at most 128): nothing is computed twice
//     and a staged key tile serves four times as many rows.
//
// Scores are fp32 sums of bf16 products; the softmax is fp32; the weights
// enter P.V as three bf16 terms (p = hi + mid + lo, each product exact,
// fp32 accumulation), which is a 32-bit weight times a bf16 value.
//
// Operand layouts of the 32x32x16 instruction: A lane l = A[l & 31]
// [8 (l >> 5) + i], B lane l = B[8 (l >> 5) + i][l & 31], D lane l reg r =
// D[(r & 3) + 8 (r >> 2) + 4 (l >> 5)][l & 31].
#include "mix_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 mf_bf16x8;
typedef __attribute__((ext_vector_type(16))) float mf_f32x16;

struct MfOpt {
  int keep_first;
  float softcap;
  const float* sink_vals;
  int vr;        // elements per row of the value cache
  int v_in_k;    // values are read from the key rows
  const unsigned short* kp;  // pooled keys [NB, G, pr, D] (nullptr: none)
  const unsigned short* vp;  // pooled values [NB, G, pr, DV]
  int pool;      // positions per pooled block
  int pr;        // pooled rows per page
};

// Pooled blocks a query at position pos sees behind its window.
PS_DEV int mf_pool_count(int pos, int window, int pool) {
  const int past = pos - window + 1;
  return (pool > 0 && window > 0 && past > 0) ? past / pool : 0;
}

// The softmax arithmetic of a tile is repeated by every wave that owns
// columns of the same rows, and a wave64 instruction takes four cycles, so
// the exponential and the cap use the hardware exponential (fp32, a few
// ulp) instead of the library's range-checked forms:
// tanh(x) = 1 - 2 / (exp(2x) + 1).
PS_DEV float mf_exp(float x) { return __expf(x); }

PS_DEV float mf_cap(float sc, float cap, float inv_cap2) {
  const float e = __expf(sc * inv_cap2);  // exp(2 sc / cap); inf is fine
  return cap * (1.0f - __fdividef(2.0f, e + 1.0f));
}

union MfPack {
  mf_bf16x8 v;
  unsigned short u[8];
  uint4 q;
};

// Stage the 32 cache rows whose element offsets are rowbase[0..31] (rows >=
// nk are zero-filled) into LDS rows of `pitch` elements, `width` elements
// each, zero-filled up to `wp` columns. The loads of a pass are all issued
// before any is stored, so their latencies overlap.
PS_DEV void mf_stage(unsigned short* __restrict__ dst, int pitch,
                     const unsigned short* __restrict__ cache,
                     const int64_t* __restrict__ rowbase, int nk, int width,
                     int wp, bool vec) {
  const int tid = threadIdx.x, nt = blockDim.x;
  if (vec) {
    constexpr int U = 5;
    const int cpr = wp / 8;
    const int total = 32 * cpr;
    for (int base = 0; base < total; base += nt * U) {
      uint4 val[U];
      int at[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int idx = base + u * nt + tid;
        at[u] = -1;
        val[u] = make_uint4(0, 0, 0, 0);
        if (idx < total) {
          const int row = idx / cpr, c = idx - row * cpr;
          at[u] = row * pitch + c * 8;
          if (row < nk && c * 8 < width)
            val[u] = *(const uint4*)(cache + rowbase[row] + c * 8);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (at[u] >= 0) *(uint4*)(dst + at[u]) = val[u];
    }
  } else {
    for (int idx = tid; idx < 32 * wp; idx += nt) {
      const int row = idx / wp, c = idx - row * wp;
      unsigned short val = 0;
      if (row < nk && c < width) val = cache[rowbase[row] + c];
      dst[row * pitch + c] = val;
    }
  }
}

// POOL: the instantiation with the pooled range; without it the kernel is
// the two-range form the families without pooled blocks have always run.
template <int CBW, int ROWS, bool POOL>
__global__ __launch_bounds__(256, 2) void mfma_attn_kernel(
    unsigned short* __restrict__ out, int ldout,
    const unsigned short* __restrict__ q, int ldq,
    const unsigned short* __restrict__ kc,
    const unsigned short* __restrict__ vc,
    const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ token_seq, const int* __restrict__ token_pos,
    int T_total, int H, int G, int D, int DV, int BS, float scale, int window,
    int sink, MfOpt opt, int KS, float* __restrict__ part, int tpb_max) {
  extern __shared__ __align__(16) unsigned short lds16[];
  __shared__ int s_seq[ROWS], s_pos[ROWS];
  __shared__ int64_t s_kbase[32], s_vbase[32];
  const int DP = (D + 15) & ~15, PK = DP + 8;
  const int DVP = (DV + 31) & ~31, PV = opt.v_in_k ? PK : DVP + 8;
  unsigned short* sQ = lds16;              // [ROWS][PK]
  unsigned short* sK = sQ + ROWS * PK;     // [32][PK]
  unsigned short* sV = opt.v_in_k ? sK : sK + 32 * PK;   // [32][PV]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int row = lane & 31, hi = lane >> 5;
  // this wave's row of the workgroup
  const int grow = (ROWS == 32 ? 0 : wave * 32) + row;
  const int rep = H / G;
  const int HPB = rep < 32 ? rep : 32;     // heads of a token in this group
  // tokens in this group; single tokens of different sequences share no
  // keys, so a batch of them runs one token per workgroup (tpb_max = 1)
  const int TPB = min(ROWS / HPB, tpb_max);
  const int hblocks = rep / HPB;
  const int g = blockIdx.y / hblocks, hb = blockIdx.y % hblocks;
  const int ks = blockIdx.z;
  const int tok0 = blockIdx.x * TPB;
  const int ntok = min(TPB, T_total - tok0);

  for (int c = tid; c < ntok; c += blockDim.x) {
    s_seq[c] = token_seq[tok0 + c];
    s_pos[c] = token_pos[tok0 + c];
  }
  // queries of the 32 rows, zero-padded
  const bool kvec = D % 8 == 0;
  const bool vvec = DV % 8 == 0 && opt.vr % 8 == 0;
  if (kvec && ldq % 8 == 0 && ((size_t)q & 15) == 0) {
    const int cpr = DP / 8;
    for (int idx = tid; idx < ROWS * cpr; idx += blockDim.x) {
      const int r = idx / cpr, c = idx - r * cpr;
      const int i = r / HPB, head = g * rep + hb * HPB + r % HPB;
      uint4 val = make_uint4(0, 0, 0, 0);
      if (i < ntok && c * 8 < D)
        val = *(const uint4*)(q + (size_t)(tok0 + i) * ldq + head * D + c * 8);
      *(uint4*)(sQ + r * PK + c * 8) = val;
    }
  } else {
    for (int idx = tid; idx < ROWS * DP; idx += blockDim.x) {
      const int r = idx / DP, d = idx - r * DP;
      const int i = r / HPB, head = g * rep + hb * HPB + r % HPB;
      unsigned short val = 0;
      if (i < ntok && d < D) val = q[(size_t)(tok0 + i) * ldq + head * D + d];
      sQ[r * PK + d] = val;
    }
  }
  __syncthreads();

  const int my_i = grow / HPB;
  const int my_head = g * rep + hb * HPB + grow % HPB;
  const bool valid = my_i < ntok;  // ntok <= TPB
  const int my_pos = valid ? s_pos[my_i] : 0;
  const int my_lo = window > 0 ? max(0, my_pos - window + 1) : 0;
  const int my_pool = POOL ? mf_pool_count(my_pos, window, opt.pool) : 0;
  const float inv_cap2 = opt.softcap > 0.f ? 2.0f / opt.softcap : 0.f;
  const bool own_sink = sink && ks == 0;
  float m = own_sink ? (opt.sink_vals ? opt.sink_vals[my_head] : 0.f)
                     : PS_NEG_INF;
  float l = own_sink ? 1.f : 0.f;
  mf_f32x16 acc[CBW];
#pragma unroll
  for (int c = 0; c < CBW; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;

  int tile_no = 0;
  int rs = 0;
  while (rs < ntok) {
    int re = rs + 1;
    while (re < ntok && s_seq[re] == s_seq[rs] &&
           s_pos[re] == s_pos[re - 1] + 1)
      ++re;
    const bool mine = valid && my_i >= rs && my_i < re;
    const int* table = block_tables + (size_t)s_seq[rs] * max_blocks;
    const int kmin = window > 0 ? max(0, s_pos[rs] - window + 1) : 0;
    const int kmax = s_pos[re - 1];
    // kept first keys behind the run's earliest window, the pooled blocks
    // its last row sees, then the windows
    const int run_pool =
        POOL ? mf_pool_count(s_pos[re - 1], window, opt.pool) : 0;
    constexpr int NR = POOL ? 3 : 2;
    for (int rg = 0; rg < NR; ++rg) {
      const bool pl = POOL && rg == 1;
      const int ra = rg == NR - 1 ? kmin : 0;
      const int rb = rg == 0 ? min(opt.keep_first, kmin) - 1
                             : (pl ? run_pool - 1 : kmax);
      for (int j0 = ra; j0 <= rb; j0 += 32, ++tile_no) {
        if (tile_no % KS != ks) continue;
        const int nk = min(32, rb + 1 - j0);
        __syncthreads();  // the previous tile is fully consumed
        if (tid < nk) {
          const int j = j0 + tid;
          if (pl) {
            const int p1 = j * opt.pool;
            const int64_t gb = ((int64_t)table[p1 / BS] * G + g) * opt.pr +
                               (p1 % BS) / opt.pool;
            s_kbase[tid] = gb * D;
            s_vbase[tid] = gb * DV;
          } else {
            const int64_t gb =
                ((int64_t)table[j / BS] * G + g) * BS + (j % BS);
            s_kbase[tid] = gb * D;
            s_vbase[tid] = gb * opt.vr;
          }
        }
        __syncthreads();
        mf_stage(sK, PK, pl ? opt.kp : kc, s_kbase, nk, D, DP, kvec);
        if (!opt.v_in_k)
          mf_stage(sV, PV, pl ? opt.vp : vc, s_vbase, nk, DV, DVP,
                   pl ? DV % 8 == 0 : vvec);
        __syncthreads();

        mf_f32x16 st;
#pragma unroll
        for (int r = 0; r < 16; ++r) st[r] = 0.f;
        const unsigned short* ka = sK + row * PK + 8 * hi;
        const unsigned short* qb = sQ + grow * PK + 8 * hi;
        for (int k0 = 0; k0 < DP; k0 += 16) {
          const mf_bf16x8 a = *(const mf_bf16x8*)(ka + k0);
          const mf_bf16x8 b = *(const mf_bf16x8*)(qb + k0);
          st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, st, 0, 0, 0);
        }
        // st[r] = score of key (r & 3) + 8 (r >> 2) + 4 hi for this row
        float p[16];
        float mx = PS_NEG_INF;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kk = (r & 3) + 8 * (r >> 2) + 4 * hi;
          const int j = j0 + kk;
          float sc = st[r] * scale;
          if (opt.softcap > 0.f) sc = mf_cap(sc, opt.softcap, inv_cap2);
          const bool vis =
              mine && kk < nk &&
              (pl ? j < my_pool
                  : (j <= my_pos && (j >= my_lo || j < opt.keep_first)));
          sc = vis ? sc : PS_NEG_INF;
          p[r] = sc;
          mx = fmaxf(mx, sc);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mnew = fmaxf(m, mx);
        float alpha = 1.f;
        if (mnew > PS_NEG_INF) {
          alpha = mf_exp(m - mnew);  // m = -inf gives 0
          float ps = 0.f;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            p[r] = p[r] > PS_NEG_INF ? mf_exp(p[r] - mnew) : 0.f;
            ps += p[r];
          }
          ps += __shfl_xor(ps, 32, 64);
          l = l * alpha + ps;
          m = mnew;
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) p[r] = 0.f;
        }
        if (alpha != 1.f) {
#pragma unroll
          for (int c = 0; c < CBW; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[c][r] *= alpha;
        }
        // O^T += V^T P^T, 16 keys a step; lane entry i of step s is key
        // 16 s + 8 (i >> 2) + 4 hi + (i & 3)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          MfPack b0, b1, b2;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            // p >= 0 cut into three bf16 terms of 8 mantissa bits each
            // (truncation; both remainders are exact)
            const float pv = p[8 * s + i];
            const unsigned int h0 = __float_as_uint(pv) & 0xffff0000u;
            const float r1 = pv - __uint_as_float(h0);
            const unsigned int h1 = __float_as_uint(r1) & 0xffff0000u;
            const float r2 = r1 - __uint_as_float(h1);
            b0.u[i] = (unsigned short)(h0 >> 16);
            b1.u[i] = (unsigned short)(h1 >> 16);
            b2.u[i] = (unsigned short)(__float_as_uint(r2) >> 16);
          }
#pragma unroll
          for (int c = 0; c < CBW; ++c) {
            const int cb = ROWS == 32 ? wave + 4 * c : c;
            if (cb * 32 < DV) {
              MfPack a;
              const unsigned short* vp = sV + cb * 32 + row;
#pragma unroll
              for (int i = 0; i < 8; ++i) {
                const int key = 16 * s + 8 * (i >> 2) + 4 * hi + (i & 3);
                a.u[i] = vp[key * PV];
              }
              acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  a.v, b0.v, acc[c], 0, 0, 0);
              acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  a.v, b1.v, acc[c], 0, 0, 0);
              acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  a.v, b2.v, acc[c], 0, 0, 0);
            }
          }
        }
      }
    }
    rs = re;
  }

  if (!valid) return;
  // acc[c][r] = O[row][column cb * 32 + (r & 3) + 8 (r >> 2) + 4 hi]
  if (KS == 1) {
    const float inv = 1.0f / l;
    unsigned short* o = out + (size_t)(tok0 + my_i) * ldout + my_head * DV;
#pragma unroll
    for (int c = 0; c < CBW; ++c) {
      const int cb = ROWS == 32 ? wave + 4 * c : c;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int col = cb * 32 + (r & 3) + 8 * (r >> 2) + 4 * hi;
        if (col < DV) o[col] = ps_f32_to_bf16(acc[c][r] * inv);
      }
    }
  } else {
    // partial record per (token, share, head): max, denominator, DV sums
    float* rec = part + (((size_t)(tok0 + my_i) * KS + ks) * H + my_head) *
                            (size_t)(DV + 2);
    if (hi == 0 && (wave == 0 || ROWS != 32)) {
      rec[0] = m;
      rec[1] = l;
    }
#pragma unroll
    for (int c = 0; c < CBW; ++c) {
      const int cb = ROWS == 32 ? wave + 4 * c : c;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int col = cb * 32 + (r & 3) + 8 * (r >> 2) + 4 * hi;
        if (col < DV) rec[2 + col] = acc[c][r];
      }
    }
  }
}

// Merge the KS partial records of every (token, head) (same record layout
// as the split-key vector kernel's).
__global__ __launch_bounds__(256) void mfma_attn_combine_kernel(
    unsigned short* __restrict__ out, int ldout,
    const float* __restrict__ part, int H, int DV, int KS) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* rec = part + ((size_t)t * KS * H + h) * (DV + 2);
  const size_t step = (size_t)H * (DV + 2);
  float mh = PS_NEG_INF;
  for (int s = 0; s < KS; ++s) mh = fmaxf(mh, rec[s * step]);
  float l = 0.f;
  for (int s = 0; s < KS; ++s) {
    const float ms = rec[s * step];
    if (ms > PS_NEG_INF) l += rec[s * step + 1] * expf(ms - mh);
  }
  const float inv = 1.0f / l;
  for (int d = threadIdx.x; d < DV; d += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < KS; ++s) {
      const float ms = rec[s * step];
      if (ms > PS_NEG_INF) a += rec[s * step + 2 + d] * expf(ms - mh);
    }
    out[(size_t)t * ldout + h * DV + d] = ps_f32_to_bf16(a * inv);
  }
}

static size_t mf_lds_budget(const void* fn) {
  // 160 KB per CU less the kernel's static arrays
  const int want = 160 * 1024 - 1024;
  if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                          want) == hipSuccess)
    return (size_t)want;
  (void)hipGetLastError();
  return 64 * 1024;
}

template <int CBW, int ROWS, bool POOL>
static int mf_launch_as(void* out, int ldout, const void* q, int ldq,
                     const void* kc, const void* vc, const void* block_tables,
                     int max_blocks, const void* token_seq,
                     const void* token_pos, int T_, int H, int G, int D,
                     int DV, int BS, float scale, int window, int sink,
                     MfOpt opt, int KS, float* part, int tpb_max,
                     hipStream_t stream) {
  static const size_t budget =
      mf_lds_budget((const void*)mfma_attn_kernel<CBW, ROWS, POOL>);
  const int DP = (D + 15) & ~15, PK = DP + 8;
  const int DVP = (DV + 31) & ~31;
  const size_t lds = ((size_t)(ROWS + 32) * PK +
                      (opt.v_in_k ? 0 : (size_t)32 * (DVP + 8))) * 2;
  if (lds > budget) return 1;
  const int rep = H / G;
  const int HPB = rep < 32 ? rep : 32;
  const int TPB = ROWS / HPB < tpb_max ? ROWS / HPB : tpb_max;
  dim3 grid((T_ + TPB - 1) / TPB, G * (rep / HPB), KS);
  hipLaunchKernelGGL((mfma_attn_kernel<CBW, ROWS, POOL>), grid, dim3(256), lds,
                     stream,
                     (unsigned short*)out, ldout, (const unsigned short*)q,
                     ldq, (const unsigned short*)kc,
                     (const unsigned short*)vc, (const int*)block_tables,
                     max_blocks, (const int*)token_seq, (const int*)token_pos,
                     T_, H, G, D, DV, BS, scale, window, sink, opt, KS, part,
                     tpb_max);
  if (KS > 1)
    hipLaunchKernelGGL(mfma_attn_combine_kernel, dim3(T_, H),
                       dim3(DV <= 64 ? 64 : (DV <= 128 ? 128 : 256)), 0,
                       stream, (unsigned short*)out, ldout,
                       (const float*)part, H, DV, KS);
  return 0;
}

template <int CBW, int ROWS>
static int mf_launch(void* out, int ldout, const void* q, int ldq,
                     const void* kc, const void* vc, const void* block_tables,
                     int max_blocks, const void* token_seq,
                     const void* token_pos, int T_, int H, int G, int D,
                     int DV, int BS, float scale, int window, int sink,
                     MfOpt opt, int KS, float* part, int tpb_max,
                     hipStream_t stream) {
  if (opt.kp != nullptr)
    return mf_launch_as<CBW, ROWS, true>(
        out, ldout, q, ldq, kc, vc, block_tables, max_blocks, token_seq,
        token_pos, T_, H, G, D, DV, BS, scale, window, sink, opt, KS, part,
        tpb_max, stream);
  return mf_launch_as<CBW, ROWS, false>(
      out, ldout, q, ldq, kc, vc, block_tables, max_blocks, token_seq,
      token_pos, T_, H, G, D, DV, BS, scale, window, sink, opt, KS, part,
      tpb_max, stream);
}

// Returns 0 when launched, 1 when the shape is outside this kernel (the
// caller then takes the vector kernels): heads per KV head must divide 32
// or be a multiple of 32, at most 512 value columns. mode 0: prompt
// portions (row split for large batches of narrow values, else column
// split), 1: single tokens of different sequences (one token per
// workgroup), 2: row split whatever the batch size.
extern "C" int mx_mfma_attention(
    void* out, int ldout, const void* q, int ldq, const void* kc,
    const void* vc, const void* block_tables, int max_blocks,
    const void* token_seq, const void* token_pos, int T_, int H, int G, int D,
    int DV, int BS, float scale, int window, int sink, int keep_first,
    float softcap, const void* sink_vals, int vrow, int v_in_k, int splits,
    void* scratch, int mode, const void* kpool, const void* vpool, int pool,
    void* stream) {
  if (T_ <= 0) return 0;
  if (G < 1 || H % G) return 1;
  const int rep = H / G;
  if (rep < 32 ? (32 % rep != 0) : (rep % 32 != 0)) return 1;
  if (DV > 512 || DV < 1 || D < 1 || vrow < DV) return 1;
  if (v_in_k && DV > D) return 1;
  const bool pooled = kpool != nullptr && pool > 0 && window > 0;
  if (pooled && v_in_k) return 1;
  const MfOpt opt = {keep_first > 0 ? keep_first : 0, softcap,
                     (const float*)sink_vals, vrow, v_in_k ? 1 : 0,
                     pooled ? (const unsigned short*)kpool : nullptr,
                     pooled ? (const unsigned short*)vpool : nullptr,
                     pooled ? pool : 0,
                     pooled ? (BS + pool - 1) / pool : 0};
  int KS = splits > 1 && scratch != nullptr ? splits : 1;
  const int cbw = ((DV + 31) / 32 + 3) / 4;
#define MF_GO(N)                                                             \
  return mf_launch<N, 32>(out, ldout, q, ldq, kc, vc, block_tables,          \
                          max_blocks, token_seq, token_pos, T_, H, G, D, DV, \
                          BS, scale, window, sink, opt, KS, (float*)scratch, \
                          mode == 1 ? 1 : 128, (hipStream_t)stream)
  // prompt portions with at most 128 value columns: row split (unless the
  // batch is too small to fill the chip with 128-row workgroups)
  if (DV <= 128 && rep <= 32 &&
      (mode == 2 || (mode == 0 && (long)T_ * H >= 128L * 512))) {
    const int rc = mf_launch<4, 128>(
        out, ldout, q, ldq, kc, vc, block_tables, max_blocks, token_seq,
        token_pos, T_, H, G, D, DV, BS, scale, window, sink, opt, KS,
        (float*)scratch, 128, (hipStream_t)stream);
    if (rc == 0) return 0;
  }
  switch (cbw) {
    case 1: MF_GO(1);
    case 2: MF_GO(2);
    case 3: MF_GO(3);
    default: MF_GO(4);
  }
#undef MF_GO
}
