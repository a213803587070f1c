// Router of a routed feed-forward, one kernel per layer and step:
//   logits = W_router x            (fp32 accumulation of the inputs' products)
//   scores = softmax(logits)  |  sigmoid(logits)
//   choice = the `top` largest of scores + correction (the correction only
//            moves the choice); sigmoid scores without a correction are
//            ranked by their logits (the fp32 sigmoid saturates and would
//            tie large scores)
//   weights = the chosen scores, divided by (their sum + renorm_eps) when
//            asked, times scale
// Outputs: the chosen outputs' indices and weights [T, top] (best first) and
// the dense weight matrix [T, n_out] (zero where an output was not chosen),
// which the all-experts path of small batches consumes directly.
//
// One workgroup per token: its waves share out the router outputs' dot
// products (16-byte loads where the rows allow it), then the first wave
// shares the outputs among its lanes for the softmax and the `top` rounds of
// arg-max.
#include "mix_common.h"

#define MR_MAX_OUT 1024

PS_DEV float mr_wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Partial dot product of two rows over this lane's share of W entries.
PS_DEV float mr_dot(const float* a, const float* b, int W, int lane,
                    bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int c = lane * 4; c < W; c += 256) {
      const float4 u = *(const float4*)(a + c), w = *(const float4*)(b + c);
      acc += u.x * w.x + u.y * w.y + u.z * w.z + u.w * w.w;
    }
  } else {
    for (int c = lane; c < W; c += 64) acc += a[c] * b[c];
  }
  return acc;
}

PS_DEV float mr_dot(const mx_bf16* a, const mx_bf16* b, int W, int lane,
                    bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int c = lane * 8; c < W; c += 512) {
      const uint4 u = *(const uint4*)(a + c), w = *(const uint4*)(b + c);
      const unsigned int uu[4] = {u.x, u.y, u.z, u.w};
      const unsigned int ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        acc += __uint_as_float(uu[k] << 16) * __uint_as_float(ww[k] << 16);
        acc += __uint_as_float(uu[k] & 0xffff0000u) *
               __uint_as_float(ww[k] & 0xffff0000u);
      }
    }
  } else {
    for (int c = lane; c < W; c += 64)
      acc += MxElem<mx_bf16>::ld(a + c) * MxElem<mx_bf16>::ld(b + c);
  }
  return acc;
}

template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(
    int64_t* __restrict__ sel, float* __restrict__ wts,
    float* __restrict__ dense, const T* __restrict__ x, int ldx,
    const T* __restrict__ rw, const float* __restrict__ corr, int T_, int W,
    int n_out, int top, int sigmoid_scores, int renorm, float renorm_eps,
    float scale, int vec) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nw = blockDim.x >> 6;
  const int t = blockIdx.x;
  float* score = lds;                   // scores
  float* pick = score + n_out;          // what the choice ranks
  int* chosen = (int*)(pick + n_out);   // [top]
  const T* xr = x + (size_t)t * ldx;
  for (int e = wave; e < n_out; e += nw) {
    const float acc =
        mx_wave_sum(mr_dot(xr, rw + (size_t)e * W, W, lane, vec != 0));
    if (lane == 0) score[e] = acc;
  }
  __syncthreads();
  if (wave != 0) return;  // the rest is one wave's work
  if (sigmoid_scores) {
    for (int e = lane; e < n_out; e += 64) {
      const float z = score[e];
      const float sg = mx_sigmoid(z);
      pick[e] = corr != nullptr ? sg + corr[e] : z;
      score[e] = sg;
    }
  } else {
    float m = -INFINITY;
    for (int e = lane; e < n_out; e += 64) m = fmaxf(m, score[e]);
    m = mr_wave_max(m);
    float s = 0.f;
    for (int e = lane; e < n_out; e += 64) s += expf(score[e] - m);
    s = mx_wave_sum(s);
    for (int e = lane; e < n_out; e += 64) {
      const float p = expf(score[e] - m) / s;
      score[e] = p;
      pick[e] = corr != nullptr ? p + corr[e] : p;
    }
  }
  __builtin_amdgcn_wave_barrier();
  // `top` rounds of arg-max; ties go to the lower index. The chosen indices
  // and scores wait in LDS (in order within a wave) until the sum is known.
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY;
    int bi = n_out;
    for (int e = lane; e < n_out; e += 64) {
      const float v = pick[e];
      if (v > bv) {
        bv = v;
        bi = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi >= n_out) bi = 0;  // only with non-finite scores
    total += score[bi];
    __builtin_amdgcn_wave_barrier();
    if (lane == 0) {
      chosen[j] = bi;
      pick[bi] = -INFINITY;  // taken
    }
    __builtin_amdgcn_wave_barrier();
  }
  const float f = (renorm ? 1.0f / (total + renorm_eps) : 1.0f) * scale;
  for (int j = lane; j < top; j += 64) {
    const int e = chosen[j];
    sel[(size_t)t * top + j] = e;
    wts[(size_t)t * top + j] = score[e] * f;
  }
  for (int e = lane; e < n_out; e += 64)
    dense[(size_t)t * n_out + e] = pick[e] == -INFINITY ? score[e] * f : 0.f;
}

// Weighted sum of the all-experts path: y [E][T][W] holds every expert's
// output for every row; out[t] = sum_e dense[t][e] y[e][t] (experts a row did
// not choose have weight 0 and are not read) + (sum of the identity outputs'
// weights) x[t] + sigmoid(sgate[t]) ys[t] (shared expert, optional; without
// sgate it joins unscaled). fp32 out.
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    float* __restrict__ out, const T* __restrict__ y,
    const float* __restrict__ dense, int n_out, int E,
    const T* __restrict__ x, int ldx, const T* __restrict__ ys, int ldys,
    const T* __restrict__ sgate, int ldsg, int T_, int W) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const float* dw = dense + (size_t)t * n_out;
  float acc = 0.f;
  for (int e = 0; e < E; ++e) {
    const float w = dw[e];
    if (w != 0.f) acc += w * MxElem<T>::ld(y + ((size_t)e * T_ + t) * W + c);
  }
  float wid = 0.f;
  for (int e = E; e < n_out; ++e) wid += dw[e];
  if (wid != 0.f) acc += wid * MxElem<T>::ld(x + (size_t)t * ldx + c);
  if (ys != nullptr)
    acc += (sgate != nullptr
                ? mx_sigmoid(MxElem<T>::ld(sgate + (size_t)t * ldsg))
                : 1.f) *
           MxElem<T>::ld(ys + (size_t)t * ldys + c);
  out[(size_t)t * W + c] = acc;
}

extern "C" void mx_moe_combine(void* out, const void* y, const void* dense,
                               int n_out, int E, const void* x, int ldx,
                               const void* ys, int ldys, const void* sgate,
                               int ldsg, int T_, int W, int dtype,
                               void* stream) {
  if (T_ <= 0 || W <= 0) return;
  dim3 grid((W + 255) / 256, T_);
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((moe_combine_kernel<T>), grid, dim3(256), 0,
                       (hipStream_t)stream, (float*)out, (const T*)y,
                       (const float*)dense, n_out, E, (const T*)x, ldx,
                       (const T*)ys, ldys, (const T*)sgate, ldsg, T_, W);
  })
}

extern "C" int mx_moe_route(void* sel, void* wts, void* dense, const void* x,
                            int ldx, const void* rw, const void* corr, int T_,
                            int W, int n_out, int top, int sigmoid_scores,
                            int renorm, float renorm_eps, float scale,
                            int dtype, void* stream) {
  if (T_ <= 0) return 0;
  if (n_out < 1 || n_out > MR_MAX_OUT || top < 1 || top > n_out) return 1;
  const size_t lds = (size_t)(2 * n_out + top) * sizeof(float);
  // 16-byte loads need whole vectors per row and aligned row starts
  const int per = dtype == MX_BF16 ? 8 : 4;
  const int vec = (W % per == 0 && ldx % per == 0 &&
                   (((size_t)x | (size_t)rw) & 15) == 0)
                      ? 1
                      : 0;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((moe_route_kernel<T>), dim3(T_), dim3(256), lds,
                       (hipStream_t)stream, (int64_t*)sel, (float*)wts,
                       (float*)dense, (const T*)x, ldx, (const T*)rw,
                       (const float*)corr, T_, W, n_out, top, sigmoid_scores,
                       renorm, renorm_eps, scale, vec);
  })
  return 0;
}
