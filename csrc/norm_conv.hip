// Sublayer boundary of stacks with layer norms and input convolutions:
//   add_layer_norm32   x += s0 * d0 + s1 * d1 (fp32 stream, in place), then
//                      per row mean and 1 / sqrt(variance + eps), the
//                      variance being the mean squared deviation (two
//                      passes over the row); writes either the normed row
//                      (x - mean) * rstd * w + b or, for norm_conv32, the
//                      row's (mean, rstd);
//   norm_conv32        h = y + conv(y) with y the normed rows, formed on the
//                      fly from the stream and the rows' (mean, rstd):
//                      conv(y)_t = sum_j cw[:, j] * y_(t - K + 1 + j), a
//                      causal per-channel convolution along every segment of
//                      the ragged batch, the segment's previous K - 1 normed
//                      rows coming from (and its last K - 1 going to) fp32
//                      per-sequence state.
// Splitting at the row statistics keeps the stream's extra traffic to one
// re-read: neighbouring rows' normed values are recomputed from registers,
// never stored.
#include "mix_common.h"

// Four consecutive entries of a row as one load / store.
PS_DEV float4 nc_ld4(const float* p) { return *(const float4*)p; }
PS_DEV float4 nc_ld4(const mx_bf16* p) {
  const uint2 u = *(const uint2*)p;
  float4 r;
  r.x = __uint_as_float(u.x << 16);
  r.y = __uint_as_float(u.x & 0xffff0000u);
  r.z = __uint_as_float(u.y << 16);
  r.w = __uint_as_float(u.y & 0xffff0000u);
  return r;
}
PS_DEV void nc_st4(float* p, const float4& v) { *(float4*)p = v; }
PS_DEV void nc_st4(mx_bf16* p, const float4& v) {
  uint2 u;
  u.x = (unsigned int)ps_f32_to_bf16(v.x) |
        ((unsigned int)ps_f32_to_bf16(v.y) << 16);
  u.y = (unsigned int)ps_f32_to_bf16(v.z) |
        ((unsigned int)ps_f32_to_bf16(v.w) << 16);
  *(uint2*)p = u;
}

// TD: element type of the deltas, TO: of the normed output. One workgroup
// per row. VEC: the row is a multiple of four entries wide, at most 1024 *
// NC_Q entries, and all rows start 16-byte aligned: a thread then keeps its
// entries (four at a time) in registers between the passes.
#define NC_Q 8

template <typename TD, typename TO, bool VEC>
__global__ __launch_bounds__(256) void add_layer_norm32_kernel(
    TO* __restrict__ h, float* __restrict__ x, const TD* __restrict__ d0,
    int ld0, float s0, const TD* __restrict__ d1, int ld1, float s1,
    const float* __restrict__ w, const float* __restrict__ b, float eps,
    float* __restrict__ stats, int W) {
  __shared__ float red[17];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * W;
  if (VEC) {
    float4 v[NC_Q];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NC_Q; ++i) {
      const int c = (threadIdx.x + 256 * i) * 4;
      if (c < W) {
        v[i] = nc_ld4(xr + c);
        if (d0 != nullptr) {
          const float4 a = nc_ld4(d0 + (size_t)t * ld0 + c);
          v[i].x += s0 * a.x;
          v[i].y += s0 * a.y;
          v[i].z += s0 * a.z;
          v[i].w += s0 * a.w;
          if (d1 != nullptr) {
            const float4 e = nc_ld4(d1 + (size_t)t * ld1 + c);
            v[i].x += s1 * e.x;
            v[i].y += s1 * e.y;
            v[i].z += s1 * e.z;
            v[i].w += s1 * e.w;
          }
          nc_st4(xr + c, v[i]);
        }
        sum += (v[i].x + v[i].y) + (v[i].z + v[i].w);
      }
    }
    const float mean = mx_block_sum(sum, red) / (float)W;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < NC_Q; ++i) {
      const int c = (threadIdx.x + 256 * i) * 4;
      if (c < W) {
        const float e0 = v[i].x - mean, e1 = v[i].y - mean;
        const float e2 = v[i].z - mean, e3 = v[i].w - mean;
        sq += (e0 * e0 + e1 * e1) + (e2 * e2 + e3 * e3);
      }
    }
    const float rstd = 1.0f / sqrtf(mx_block_sum(sq, red) / (float)W + eps);
    if (stats != nullptr && threadIdx.x == 0) {
      stats[2 * t] = mean;
      stats[2 * t + 1] = rstd;
    }
    if (h != nullptr) {
#pragma unroll
      for (int i = 0; i < NC_Q; ++i) {
        const int c = (threadIdx.x + 256 * i) * 4;
        if (c < W) {
          const float4 ww = nc_ld4(w + c), bb = nc_ld4(b + c);
          float4 o;
          o.x = (v[i].x - mean) * rstd * ww.x + bb.x;
          o.y = (v[i].y - mean) * rstd * ww.y + bb.y;
          o.z = (v[i].z - mean) * rstd * ww.z + bb.z;
          o.w = (v[i].w - mean) * rstd * ww.w + bb.w;
          nc_st4(h + (size_t)t * W + c, o);
        }
      }
    }
    return;
  }
  float sum = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = xr[c];
    if (d0 != nullptr) {
      float d = s0 * MxElem<TD>::ld(d0 + (size_t)t * ld0 + c);
      if (d1 != nullptr) d += s1 * MxElem<TD>::ld(d1 + (size_t)t * ld1 + c);
      v += d;
      xr[c] = v;
    }
    sum += v;
  }
  const float mean = mx_block_sum(sum, red) / (float)W;
  // a thread re-reads only entries it wrote itself
  float sq = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float dv = xr[c] - mean;
    sq += dv * dv;
  }
  const float rstd = 1.0f / sqrtf(mx_block_sum(sq, red) / (float)W + eps);
  if (stats != nullptr && threadIdx.x == 0) {
    stats[2 * t] = mean;
    stats[2 * t + 1] = rstd;
  }
  if (h != nullptr)
    for (int c = threadIdx.x; c < W; c += blockDim.x)
      MxElem<TO>::st(h + (size_t)t * W + c,
                     (xr[c] - mean) * rstd * w[c] + b[c]);
}

// A workgroup takes 256 channels of up to NC_ROWS consecutive rows of one
// segment: grid (channel blocks, segments, row tiles). Only the tile at a
// segment's start reads the sequence's state, and it writes the new state
// (the segment's last K - 1 normed rows) afterwards, so no other workgroup
// races with it.
#define NC_ROWS 64

// KT: taps at compile time; 0: `taps` of them (up to NC_MAX_TAPS), with the
// window in arrays of that size.
#define NC_MAX_TAPS 32

template <typename TO, int KT>
__global__ __launch_bounds__(256) void norm_conv32_kernel(
    TO* __restrict__ h, const float* __restrict__ x,
    const float* __restrict__ stats, const float* __restrict__ w,
    const float* __restrict__ b, const float* __restrict__ cw,
    float* __restrict__ state, const int* __restrict__ seq_rows, int W,
    int taps) {
  constexpr int KA = KT > 0 ? KT : NC_MAX_TAPS;   // array sizes
  const int K = KT > 0 ? KT : taps;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int* sr = seq_rows + 4 * blockIdx.y;
  const int t0 = sr[0], n = sr[1], p0 = sr[2], slot = sr[3];
  const int a = blockIdx.z * NC_ROWS;
  if (c >= W || a >= n) return;
  const int e = min(n, a + NC_ROWS);
  constexpr int P = KA > 1 ? KA - 1 : 1;
  float wk[KA], win[P], old[P];
#pragma unroll
  for (int j = 0; j < K; ++j) wk[j] = cw[(size_t)c * K + j];
  const float wc = w[c], bc = b[c];
  float* st = state + (size_t)slot * (K - 1) * W;
#pragma unroll
  for (int j = 0; j < K - 1; ++j) {
    const int r = a - (K - 1) + j;  // row of the segment, < 0: before it
    if (r >= 0) {
      const int t = t0 + r;
      win[j] = (x[(size_t)t * W + c] - stats[2 * t]) * stats[2 * t + 1] * wc +
               bc;
    } else {
      win[j] = p0 > 0 ? st[(size_t)(K - 1 + r) * W + c] : 0.f;
    }
    old[j] = win[j];
  }
#pragma unroll 4
  for (int r = a; r < e; ++r) {
    const int t = t0 + r;
    const float cur =
        (x[(size_t)t * W + c] - stats[2 * t]) * stats[2 * t + 1] * wc + bc;
    float acc = cur + wk[K - 1] * cur;
#pragma unroll
    for (int j = 0; j < K - 1; ++j) acc += wk[j] * win[j];
#pragma unroll
    for (int j = 0; j + 1 < K - 1; ++j) win[j] = win[j + 1];
    if (K > 1) win[K - 2] = cur;
    MxElem<TO>::st(h + (size_t)t * W + c, acc);
  }
  if (a == 0) {
    // old[] holds the previous state (rows -(K-1) .. -1 of the segment)
#pragma unroll
    for (int j = 0; j < K - 1; ++j) {
      const int r = n - (K - 1) + j;
      float val;
      if (r >= 0) {
        const int t = t0 + r;
        val = (x[(size_t)t * W + c] - stats[2 * t]) * stats[2 * t + 1] * wc +
              bc;
      } else {
        val = 0.f;
#pragma unroll
        for (int i = 0; i < K - 1; ++i)
          if (i == K - 1 + r) val = old[i];
      }
      st[(size_t)j * W + c] = val;
    }
  }
}

extern "C" {

void mx_add_layer_norm32(void* h, void* x, const void* d0, int ld0, float s0,
                         const void* d1, int ld1, float s1, const void* w,
                         const void* b, float eps, void* stats, int T_, int W,
                         int delta_dtype, int out_dtype, void* stream) {
  if (T_ <= 0) return;
  // four entries per load: whole vectors per row, aligned row starts
  const bool vec =
      W % 4 == 0 && W <= 1024 * NC_Q && ld0 % 4 == 0 && ld1 % 4 == 0 &&
      (((size_t)h | (size_t)x | (size_t)d0 | (size_t)d1 | (size_t)w |
        (size_t)b) & 15) == 0;
#define ALN_GO(TD, TO)                                                       \
  if (vec)                                                                   \
    hipLaunchKernelGGL((add_layer_norm32_kernel<TD, TO, true>), dim3(T_),    \
                       dim3(256), 0, (hipStream_t)stream, (TO*)h, (float*)x, \
                       (const TD*)d0, ld0, s0, (const TD*)d1, ld1, s1,       \
                       (const float*)w, (const float*)b, eps, (float*)stats, \
                       W);                                                   \
  else                                                                       \
    hipLaunchKernelGGL((add_layer_norm32_kernel<TD, TO, false>), dim3(T_),   \
                       dim3(256), 0, (hipStream_t)stream, (TO*)h, (float*)x, \
                       (const TD*)d0, ld0, s0, (const TD*)d1, ld1, s1,       \
                       (const float*)w, (const float*)b, eps, (float*)stats, \
                       W)
  if (delta_dtype == MX_BF16) {
    if (out_dtype == MX_BF16) {
      ALN_GO(mx_bf16, mx_bf16);
    } else {
      ALN_GO(mx_bf16, float);
    }
  } else {
    if (out_dtype == MX_BF16) {
      ALN_GO(float, mx_bf16);
    } else {
      ALN_GO(float, float);
    }
  }
#undef ALN_GO
}

#define NC_CASE(KK)                                                          \
  case KK:                                                                   \
    hipLaunchKernelGGL((norm_conv32_kernel<T, KK>), grid, dim3(256), 0,      \
                       (hipStream_t)stream, (T*)h, (const float*)x,          \
                       (const float*)stats, (const float*)w,                 \
                       (const float*)b, (const float*)cw, (float*)state,     \
                       (const int*)seq_rows, W, K);                          \
    break;

int mx_norm_conv32(void* h, const void* x, const void* stats, const void* w,
                   const void* b, const void* cw, void* state,
                   const void* seq_rows, int S_, int W, int K, int T_,
                   int dtype, void* stream) {
  if (S_ <= 0 || T_ <= 0) return 0;
  if (K < 1 || K > NC_MAX_TAPS) return 1;
  // a segment has at most T_ - (S_ - 1) rows
  const int longest = T_ - (S_ - 1);
  dim3 grid((W + 255) / 256, S_, (longest + NC_ROWS - 1) / NC_ROWS);
  MX_DISPATCH_DTYPE(dtype, {
    switch (K) {
      NC_CASE(1)
      NC_CASE(2)
      NC_CASE(3)
      NC_CASE(4)
      NC_CASE(5)
      NC_CASE(6)
      NC_CASE(7)
      NC_CASE(8)
      default:
        hipLaunchKernelGGL((norm_conv32_kernel<T, 0>), grid, dim3(256), 0,
                           (hipStream_t)stream, (T*)h, (const float*)x,
                           (const float*)stats, (const float*)w,
                           (const float*)b, (const float*)cw, (float*)state,
                           (const int*)seq_rows, W, K);
    }
  })
  return 0;
}

}  // extern "C"
