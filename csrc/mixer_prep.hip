// Per-token preparation kernels of the attention and recurrent mixers:
//   attn_prep        per-head query/key RMSNorm, rotary turn of the heads'
//                    leading entries, value blend with another layer's
//                    values, paged K/V append;
//   latent_prep      latent RMSNorm, rotary turn of the shared key part and
//                    of the queries' rotary parts, paged append of
//                    [latent | key part], assembly of the latent-space
//                    queries;
//   pool_append      mean key/value of every block of positions a step
//                    completes, into the pooled caches;
//   short_conv_silu  causal per-channel convolution over time + silu with
//                    the last taps-1 inputs of every sequence as state.
// All arithmetic is fp32; the element type decides loads and the final
// rounding.
#include "mix_common.h"

// One wave per head: x / sqrt(mean(x^2) + eps) * w over D entries (the mean
// over the head, or with ALL over the whole query / key projection, whose
// weights then have H*D / G*D entries), then the first rot_dims entries turn
// by row `position` of the table cs [table_rows][rot_dims / 2][cos, sin].
// Interleaved pairs (2i, 2i+1): a lane reads its own entry and its pair
// partner's (a neighbouring lane's) before it stores, and the wave runs in
// step, so the query is rewritten in place. HALF pairs (i, i + rot_dims / 2):
// a lane owns both entries of a pair, reads them, turns them and stores
// them, so nothing it reads is another lane's to write.
template <typename T, bool HALF, bool ALL>
__global__ __launch_bounds__(256) void attn_prep_kernel(
    T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk,
    T* __restrict__ v, int ldv, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps, const float* __restrict__ vmix,
    const T* __restrict__ vfirst, int ldvf, T* __restrict__ kc,
    T* __restrict__ vc, const int64_t* __restrict__ slots, int H, int G,
    int D, int DV, int BS, const float* __restrict__ cs, int table_rows,
    int rot_dims, const int* __restrict__ positions) {
  __shared__ float red[17];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const float* csr = nullptr;
  if (cs != nullptr)
    csr = cs + (size_t)min(max(positions[t], 0), table_rows - 1) * rot_dims;
  const int64_t slot = slots[t];
  const int64_t blk = slot >= 0 ? slot / BS : 0;
  const int off = slot >= 0 ? (int)(slot % BS) : 0;
  // whole-projection norms: one sum of squares over all query entries and
  // one over all key entries
  float inv_q = 1.f, inv_k = 1.f;
  if (ALL && qw != nullptr) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < H * D; c += blockDim.x) {
      const float x = MxElem<T>::ld(q + (size_t)t * ldq + c);
      ss += x * x;
    }
    inv_q = 1.0f / sqrtf(mx_block_sum(ss, red) / (float)(H * D) + eps);
  }
  if (ALL && kw != nullptr) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < G * D; c += blockDim.x) {
      const float x = MxElem<T>::ld(k + (size_t)t * ldk + c);
      ss += x * x;
    }
    inv_k = 1.0f / sqrtf(mx_block_sum(ss, red) / (float)(G * D) + eps);
  }
  for (int hh = wave; hh < H + G; hh += nw) {
    const bool is_q = hh < H;
    const int g = hh - H;
    const T* src = is_q ? q + (size_t)t * ldq + hh * D
                        : k + (size_t)t * ldk + g * D;
    // weight row of this head
    const float* wgt = is_q ? qw : kw;
    if (ALL && wgt != nullptr) wgt += (is_q ? hh : g) * D;
    float inv = is_q ? inv_q : inv_k;
    if (!ALL && wgt != nullptr) {
      float ss = 0.f;
      for (int d = lane; d < D; d += 64) {
        const float x = MxElem<T>::ld(src + d);
        ss += x * x;
      }
      ss = mx_wave_sum(ss);
      inv = 1.0f / sqrtf(ss / (float)D + eps);
    }
    T* dst = nullptr;
    if (is_q) {
      if (wgt != nullptr || csr != nullptr) dst = q + (size_t)t * ldq + hh * D;
    } else if (slot >= 0) {
      dst = kc + ((blk * G + g) * BS + off) * (int64_t)D;
    }
    if (dst == nullptr) continue;
    if (!HALF) {
      for (int d = lane; d < D; d += 64) {
        float x = MxElem<T>::ld(src + d);
        if (wgt != nullptr) x *= inv * wgt[d];
        if (csr != nullptr && d < rot_dims) {
          float y = MxElem<T>::ld(src + (d ^ 1));
          if (wgt != nullptr) y *= inv * wgt[d ^ 1];
          const float* e = csr + (d & ~1);
          x = (d & 1) ? x * e[0] + y * e[1] : x * e[0] - y * e[1];
        }
        MxElem<T>::st(dst + d, x);
      }
    } else {
      const int hd = csr != nullptr ? rot_dims >> 1 : 0;
      for (int i = lane; i < hd; i += 64) {
        float x = MxElem<T>::ld(src + i);
        float y = MxElem<T>::ld(src + i + hd);
        if (wgt != nullptr) {
          x *= inv * wgt[i];
          y *= inv * wgt[i + hd];
        }
        const float c = csr[2 * i], sn = csr[2 * i + 1];
        MxElem<T>::st(dst + i, x * c - y * sn);
        MxElem<T>::st(dst + i + hd, y * c + x * sn);
      }
      for (int d = 2 * hd + lane; d < D; d += 64) {
        float x = MxElem<T>::ld(src + d);
        if (wgt != nullptr) x *= inv * wgt[d];
        MxElem<T>::st(dst + d, x);
      }
    }
  }
  const float lam = vfirst != nullptr ? vmix[0] : 0.f;
  for (int c = threadIdx.x; c < G * DV; c += blockDim.x) {
    float x = MxElem<T>::ld(v + (size_t)t * ldv + c);
    if (vfirst != nullptr) {
      x = (1.0f - lam) * x + lam * MxElem<T>::ld(vfirst + (size_t)t * ldvf + c);
      MxElem<T>::st(v + (size_t)t * ldv + c, x);
    }
    if (slot >= 0) {
      const int g = c / DV, d = c % DV;
      MxElem<T>::st(vc + ((blk * G + g) * BS + off) * (int64_t)DV + d, x);
    }
  }
}

// Pooled keys/values: workgroup (segment, i, column chunk) takes 256
// columns of the i-th block of `pool` positions whose last position this step
// appended (block b covers b*pool .. b*pool + pool - 1) and stores the fp32
// means of its cached keys and values, rounded to the cache type, in the
// pooled caches [NB, G, pr, D|DV]: in the page of the block's first position,
// at row (first position mod BS) div pool. A thread owns one column; its
// loads over the block's positions are independent and run eight at a time.
template <typename T>
__global__ __launch_bounds__(256) void pool_append_kernel(
    const T* __restrict__ kc, const T* __restrict__ vc, T* __restrict__ kp,
    T* __restrict__ vp, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ seq_rows, int G, int D, int DV, int BS, int pool,
    int pr) {
  const int* sr = seq_rows + 4 * blockIdx.x;
  const int n = sr[1], p0 = sr[2];
  const int b = p0 / pool + blockIdx.y;
  if (b >= (p0 + n) / pool) return;
  const int c = blockIdx.z * blockDim.x + threadIdx.x;
  if (c >= G * (D + DV)) return;
  const int* table = block_tables + (size_t)blockIdx.x * max_blocks;
  const int first = b * pool;
  const bool is_k = c < G * D;
  const int cc = is_k ? c : c - G * D;
  const int w = is_k ? D : DV;
  const int g = cc / w, d = cc - g * w;
  const T* cache = (is_k ? kc : vc) + d;
  float acc = 0.f;
  int j = first;
  for (; j + 8 <= first + pool; j += 8) {
    float x[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int jj = j + u;
      x[u] = MxElem<T>::ld(
          cache + (((int64_t)table[jj / BS] * G + g) * BS + (jj % BS)) * w);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += x[u];
  }
  for (; j < first + pool; ++j)
    acc += MxElem<T>::ld(
        cache + (((int64_t)table[j / BS] * G + g) * BS + (j % BS)) * w);
  const int64_t prow =
      ((int64_t)table[first / BS] * G + g) * pr + (first % BS) / pool;
  MxElem<T>::st((is_k ? kp : vp) + prow * w + d, acc / (float)pool);
}

// Turn the pair (u, w) by the table entry (cos, sin).
PS_DEV void mx_turn(float u, float w, const float* cs, float* ou, float* ow) {
  *ou = u * cs[0] - w * cs[1];
  *ow = w * cs[0] + u * cs[1];
}

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(
    T* __restrict__ qf, const T* __restrict__ qlat, const T* __restrict__ q,
    int ldq, const T* __restrict__ dkv, int lddkv,
    const float* __restrict__ normw, float eps,
    const float* __restrict__ cos_sin, int table_rows, int rot_dims,
    const int* __restrict__ positions, T* __restrict__ cache,
    const int64_t* __restrict__ slots, int T_, int H, int D, int R, int L,
    int BS) {
  __shared__ float red[17];
  const int t = blockIdx.x;
  const int pos = min(max(positions[t], 0), table_rows - 1);
  const float* cs = cos_sin + (size_t)pos * rot_dims;  // [rot_dims/2][2]
  const T* row = dkv + (size_t)t * lddkv;
  const int64_t slot = slots[t];
  T* crow = cache + (slot >= 0 ? slot : 0) * (int64_t)(L + R);
  float ss = 0.f;
  for (int c = threadIdx.x; c < L; c += blockDim.x) {
    const float x = MxElem<T>::ld(row + c);
    ss += x * x;
  }
  ss = mx_block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)L + eps);
  if (slot >= 0) {
    for (int c = threadIdx.x; c < L; c += blockDim.x)
      MxElem<T>::st(crow + c, MxElem<T>::ld(row + c) * inv * normw[c]);
    // shared key part: pairs below rot_dims turn, the rest passes
    for (int i = threadIdx.x; i < R / 2; i += blockDim.x) {
      float u = MxElem<T>::ld(row + L + 2 * i);
      float w = MxElem<T>::ld(row + L + 2 * i + 1);
      if (2 * i < rot_dims) mx_turn(u, w, cs + 2 * i, &u, &w);
      MxElem<T>::st(crow + L + 2 * i, u);
      MxElem<T>::st(crow + L + 2 * i + 1, w);
    }
    if ((R & 1) && threadIdx.x == 0)
      crow[L + R - 1] = row[L + R - 1];
  }
  // queries: per head [latent-space part | turned rotary part]
  const int QW = L + R;
  for (int c = threadIdx.x; c < H * L; c += blockDim.x) {
    const int h = c / L, l = c - h * L;
    qf[(size_t)t * H * QW + h * QW + l] = qlat[((size_t)h * T_ + t) * L + l];
  }
  for (int c = threadIdx.x; c < H * (R / 2); c += blockDim.x) {
    const int h = c / (R / 2), i = c - h * (R / 2);
    const T* src = q + (size_t)t * ldq + h * (D + R) + D;
    float u = MxElem<T>::ld(src + 2 * i);
    float w = MxElem<T>::ld(src + 2 * i + 1);
    if (2 * i < rot_dims) mx_turn(u, w, cs + 2 * i, &u, &w);
    T* dst = qf + (size_t)t * H * QW + h * QW + L;
    MxElem<T>::st(dst + 2 * i, u);
    MxElem<T>::st(dst + 2 * i + 1, w);
  }
  if (R & 1)
    for (int h = threadIdx.x; h < H; h += blockDim.x)
      qf[(size_t)t * H * QW + h * QW + QW - 1] =
          q[(size_t)t * ldq + h * (D + R) + D + R - 1];
}

// Thread = channel, workgroup = (channel tile, segment, chunk of CONV_CH
// tokens). A thread keeps the K-1 inputs before its current token in
// registers. Only chunk 0 of a segment reads the sequence's state, and it
// writes the new state (the segment's last K-1 inputs) afterwards, so no
// other workgroup races with it.
#define CONV_CH 64

template <typename T, int K>
__global__ __launch_bounds__(256) void short_conv_silu_kernel(
    T* __restrict__ y, int ldy, const T* __restrict__ x, int ldx,
    const float* __restrict__ w, const float* __restrict__ bias,
    T* __restrict__ state, const int* __restrict__ seq_rows, int C) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int* sr = seq_rows + 4 * blockIdx.y;
  const int t0 = sr[0], n = sr[1], p0 = sr[2], slot = sr[3];
  const int a = blockIdx.z * CONV_CH;
  if (c >= C || a >= n) return;
  const int b = min(n, a + CONV_CH);
  constexpr int P = K > 1 ? K - 1 : 1;
  float wk[K], win[P], old[P];
#pragma unroll
  for (int j = 0; j < K; ++j) wk[j] = w[(size_t)c * K + j];
  const float b0 = bias != nullptr ? bias[c] : 0.f;
  T* st = state + (size_t)slot * (K - 1) * C;
#pragma unroll
  for (int j = 0; j < K - 1; ++j) {
    const int r = a - (K - 1) + j;  // row of the segment, < 0: before it
    if (r >= 0)
      win[j] = MxElem<T>::ld(x + (size_t)(t0 + r) * ldx + c);
    else
      win[j] = p0 > 0 ? MxElem<T>::ld(st + (size_t)(K - 1 + r) * C + c) : 0.f;
    old[j] = win[j];
  }
  for (int t = a; t < b; ++t) {
    const float cur = MxElem<T>::ld(x + (size_t)(t0 + t) * ldx + c);
    float acc = b0 + wk[K - 1] * cur;
#pragma unroll
    for (int j = 0; j < K - 1; ++j) acc += wk[j] * win[j];
#pragma unroll
    for (int j = 0; j + 1 < K - 1; ++j) win[j] = win[j + 1];
    if (K > 1) win[K - 2] = cur;
    MxElem<T>::st(y + (size_t)(t0 + t) * ldy + c, acc * mx_sigmoid(acc));
  }
  if (a == 0) {
    // old[] holds the previous state (a == 0: rows -(K-1) .. -1)
#pragma unroll
    for (int j = 0; j < K - 1; ++j) {
      const int r = n - (K - 1) + j;
      float val;
      if (r >= 0) {
        val = MxElem<T>::ld(x + (size_t)(t0 + r) * ldx + c);
      } else {
        val = 0.f;
#pragma unroll
        for (int e = 0; e < K - 1; ++e)
          if (e == K - 1 + r) val = old[e];
      }
      MxElem<T>::st(st + (size_t)j * C + c, val);
    }
  }
}

extern "C" {

void mx_attn_prep(void* q, int ldq, const void* k, int ldk, void* v, int ldv,
                  const void* qw, const void* kw, float eps, const void* vmix,
                  const void* vfirst, int ldvf, void* kc, void* vc,
                  const void* slots, int T_, int H, int G, int D, int DV,
                  int BS, const void* cos_sin, int table_rows, int rot_dims,
                  const void* positions, int norm_all, int half, int dtype,
                  void* stream) {
  if (T_ <= 0) return;
#define AP_GO(HALF_, ALL_)                                                  \
  hipLaunchKernelGGL((attn_prep_kernel<T, HALF_, ALL_>), dim3(T_), dim3(256), \
                     0, (hipStream_t)stream, (T*)q, ldq, (const T*)k, ldk,   \
                     (T*)v, ldv, (const float*)qw, (const float*)kw, eps,    \
                     (const float*)vmix, (const T*)vfirst, ldvf, (T*)kc,     \
                     (T*)vc, (const int64_t*)slots, H, G, D, DV, BS,         \
                     (const float*)cos_sin, table_rows, rot_dims,            \
                     (const int*)positions)
  MX_DISPATCH_DTYPE(dtype, {
    if (half && norm_all) AP_GO(true, true);
    else if (half) AP_GO(true, false);
    else if (norm_all) AP_GO(false, true);
    else AP_GO(false, false);
  })
#undef AP_GO
}

void mx_pool_append(const void* kc, const void* vc, void* kp, void* vp,
                    const void* block_tables, int max_blocks,
                    const void* seq_rows, int S_, int blocks_per_seg, int G,
                    int D, int DV, int BS, int pool, int dtype,
                    void* stream) {
  if (S_ <= 0 || blocks_per_seg <= 0 || pool < 1) return;
  const int pr = (BS + pool - 1) / pool;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((pool_append_kernel<T>),
                       dim3(S_, blocks_per_seg, (G * (D + DV) + 255) / 256),
                       dim3(256), 0, (hipStream_t)stream, (const T*)kc,
                       (const T*)vc, (T*)kp, (T*)vp,
                       (const int*)block_tables, max_blocks,
                       (const int*)seq_rows, G, D, DV, BS, pool, pr);
  })
}

void mx_latent_prep(void* qf, const void* qlat, const void* q, int ldq,
                    const void* dkv, int lddkv, const void* normw, float eps,
                    const void* cos_sin, int table_rows, int rot_dims,
                    const void* positions, void* cache, const void* slots,
                    int T_, int H, int D, int R, int L, int BS, int dtype,
                    void* stream) {
  if (T_ <= 0) return;
  (void)BS;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((latent_prep_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (T*)qf, (const T*)qlat,
                       (const T*)q, ldq, (const T*)dkv, lddkv,
                       (const float*)normw, eps, (const float*)cos_sin,
                       table_rows, rot_dims, (const int*)positions,
                       (T*)cache, (const int64_t*)slots, T_, H, D, R, L, BS);
  })
}

#define CONV_CASE(KK)                                                        \
  case KK:                                                                   \
    hipLaunchKernelGGL((short_conv_silu_kernel<T, KK>), grid, dim3(256), 0,  \
                       (hipStream_t)stream, (T*)y, ldy, (const T*)x, ldx,    \
                       (const float*)w, (const float*)bias, (T*)state,       \
                       (const int*)seq_rows, C);                             \
    break;

int mx_short_conv_silu(void* y, int ldy, const void* x, int ldx,
                       const void* w, const void* bias, void* state,
                       const void* seq_rows,
                       int S_, int C, int K, int T_, int dtype,
                       void* stream) {
  if (S_ <= 0 || T_ <= 0) return 0;
  if (K < 1 || K > 8) return 1;
  // a segment has at most T_ - (S_ - 1) rows
  const int longest = T_ - (S_ - 1);
  dim3 grid((C + 255) / 256, S_, (longest + CONV_CH - 1) / CONV_CH);
  MX_DISPATCH_DTYPE(dtype, {
    switch (K) {
      CONV_CASE(1)
      CONV_CASE(2)
      CONV_CASE(3)
      CONV_CASE(4)
      CONV_CASE(5)
      CONV_CASE(6)
      CONV_CASE(7)
      CONV_CASE(8)
    }
  })
  return 0;
}

}  // extern "C"
