// Router of a routed feed-forward, one kernel per layer and step:
//   logits = W_router x            (fp32 accumulation of the inputs' products)
//   scores = softmax(logits)  |  sigmoid(logits)
//   choice = the `top` largest of scores + correction (softmax; the
//            correction only moves the choice) or of the logits (sigmoid:
//            the fp32 sigmoid saturates and would tie large scores)
//   weights = the chosen scores, divided by (their sum + renorm_eps) when
//            asked, times scale
// Outputs: the chosen outputs' indices and weights [T, top] (best first) and
// the dense weight matrix [T, n_out] (zero where an output was not chosen),
// which the all-experts path of small batches consumes directly.
//
// One wave per token: the lanes share each dot product, then share the
// router outputs among them for the softmax and the `top` rounds of arg-max.
#include "mix_common.h"

#define MR_MAX_OUT 1024

PS_DEV float mr_wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(
    int64_t* __restrict__ sel, float* __restrict__ wts,
    float* __restrict__ dense, const T* __restrict__ x, int ldx,
    const T* __restrict__ rw, const float* __restrict__ corr, int T_, int W,
    int n_out, int top, int sigmoid_scores, int renorm, float renorm_eps,
    float scale) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * (blockDim.x >> 6) + wave;
  if (t >= T_) return;  // whole waves leave; no block-wide barrier below
  float* score = lds + (size_t)wave * (2 * n_out + top);  // scores
  float* pick = score + n_out;          // what the choice ranks
  int* chosen = (int*)(pick + n_out);   // [top]
  const T* xr = x + (size_t)t * ldx;
  for (int e = 0; e < n_out; ++e) {
    const T* wr = rw + (size_t)e * W;
    float acc = 0.f;
    for (int c = lane; c < W; c += 64)
      acc += MxElem<T>::ld(xr + c) * MxElem<T>::ld(wr + c);
    acc = mx_wave_sum(acc);
    if (lane == 0) score[e] = acc;
  }
  __builtin_amdgcn_wave_barrier();
  if (sigmoid_scores) {
    for (int e = lane; e < n_out; e += 64) {
      const float z = score[e];
      pick[e] = z;
      score[e] = mx_sigmoid(z);
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

extern "C" int mx_moe_route(void* sel, void* wts, void* dense, const void* x,
                            int ldx, const void* rw, const void* corr, int T_,
                            int W, int n_out, int top, int sigmoid_scores,
                            int renorm, float renorm_eps, float scale,
                            int dtype, void* stream) {
  if (T_ <= 0) return 0;
  if (n_out < 1 || n_out > MR_MAX_OUT || top < 1 || top > n_out) return 1;
  const int waves = 4;
  const size_t lds = (size_t)waves * (2 * n_out + top) * sizeof(float);
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((moe_route_kernel<T>), dim3((T_ + waves - 1) / waves),
                       dim3(64 * waves), lds, (hipStream_t)stream,
                       (int64_t*)sel, (float*)wts, (float*)dense,
                       (const T*)x, ldx, (const T*)rw, (const float*)corr, T_,
                       W, n_out, top, sigmoid_scores, renorm, renorm_eps,
                       scale);
  })
  return 0;
}
