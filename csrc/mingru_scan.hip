// Minimal gated recurrent unit: an element-wise recurrence over a ragged
// batch,
//   a = sigmoid(z + zb),  u' = u + ub,
//   c = u' + 1/2 (u' >= 0) | sigmoid(u') (u' < 0),
//   S <- (1 - a) S + a c,   out = S * silu(g),
// with S fp32 per sequence and channel. A thread owns one channel of one
// segment and walks its rows in order; the loads of a row do not depend on
// the recurrence, so the loop is unrolled and they run ahead of it. All
// arithmetic is fp32; the element type decides loads and the final
// rounding.
#include "mix_common.h"

template <typename T>
__global__ __launch_bounds__(64) void mingru_scan_kernel(
    T* __restrict__ out, int ldo, const T* __restrict__ z, int ldz,
    const T* __restrict__ u, int ldu, const T* __restrict__ g, int ldg,
    const float* __restrict__ zb, const float* __restrict__ ub,
    float* __restrict__ state, const int* __restrict__ seq_rows, int C) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int* sr = seq_rows + 4 * blockIdx.y;
  const int t0 = sr[0], n = sr[1], p0 = sr[2], slot = sr[3];
  const float bz = zb[c], bu = ub[c];
  float S = p0 > 0 ? state[(size_t)slot * C + c] : 0.f;
#pragma unroll 8
  for (int r = 0; r < n; ++r) {
    const size_t t = (size_t)(t0 + r);
    const float a = mx_sigmoid(MxElem<T>::ld(z + t * ldz + c) + bz);
    const float uu = MxElem<T>::ld(u + t * ldu + c) + bu;
    const float cand = uu >= 0.f ? uu + 0.5f : mx_sigmoid(uu);
    const float gg = MxElem<T>::ld(g + t * ldg + c);
    S = (1.0f - a) * S + a * cand;
    MxElem<T>::st(out + t * ldo + c, S * (gg * mx_sigmoid(gg)));
  }
  state[(size_t)slot * C + c] = S;
}

extern "C" void mx_mingru_scan(void* out, int ldo, const void* z, int ldz,
                               const void* u, int ldu, const void* g, int ldg,
                               const void* zb, const void* ub, void* state,
                               const void* seq_rows, int S_, int C, int T_,
                               int dtype, void* stream) {
  if (S_ <= 0 || T_ <= 0 || C <= 0) return;
  dim3 grid((C + 63) / 64, S_);
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((mingru_scan_kernel<T>), grid, dim3(64), 0,
                       (hipStream_t)stream, (T*)out, ldo, (const T*)z, ldz,
                       (const T*)u, ldu, (const T*)g, ldg, (const float*)zb,
                       (const float*)ub, (float*)state, (const int*)seq_rows,
                       C);
  })
}
