// fp32 residual-stream kernels: scaled embedding gather, fused
// (residual += deltas) + (grouped) RMSNorm, grouped RMSNorm + token shift,
// depth-weighted sum of residual streams, gated-MLP inner activations, paged
// KV append with independent key/value widths.
#include "mix_common.h"

template <typename T>
__global__ __launch_bounds__(256) void embed_scale_kernel(
    float* __restrict__ x, const int64_t* __restrict__ tokens,
    const T* __restrict__ embed, float scale, int W) {
  const int t = blockIdx.x;
  const T* row = embed + (size_t)tokens[t] * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    x[(size_t)t * W + c] = MxElem<T>::ld(row + c) * scale;
}

#define MX_MAX_GROUPS 64

// Per-group 1/rms of one fp32 row into sinv[groups] (LDS); the row is split
// into `groups` equal consecutive parts. Ends with a barrier.
PS_DEV void mx_group_inv(const float* __restrict__ xr, int W, int groups,
                         float eps, float* sinv, float* red) {
  const int gw = W / groups;
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
    for (int c = g * gw + threadIdx.x; c < (g + 1) * gw; c += blockDim.x)
      ss += xr[c] * xr[c];
    ss = mx_block_sum(ss, red);
    if (threadIdx.x == 0) sinv[g] = 1.0f / sqrtf(ss / (float)gw + eps);
  }
  __syncthreads();
}

// xo[t] = xi[t] + d0[t] + d1[t] (each optional; xo may be xi),
// h[t] = xo[t] / rms(part of xo[t]) * w, one rms per group of W / groups.
template <typename T>
__global__ __launch_bounds__(256) void add_group_norm32_kernel(
    T* __restrict__ h, float* xo, const float* xi, const T* __restrict__ d0,
    int ld0, const T* __restrict__ d1, int ld1, const float* __restrict__ w,
    float eps, int groups, int W) {
  __shared__ float red[17];
  __shared__ float sinv[MX_MAX_GROUPS];
  const int t = blockIdx.x;
  float* xr = xo + (size_t)t * W;
  const float* xs = xi + (size_t)t * W;
  if (d0 != nullptr || xo != xi) {
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      float v = xs[c];
      if (d0 != nullptr) {
        float d = MxElem<T>::ld(d0 + (size_t)t * ld0 + c);
        if (d1 != nullptr) d += MxElem<T>::ld(d1 + (size_t)t * ld1 + c);
        v += d;
      }
      xr[c] = v;
    }
    __syncthreads();  // the sums below read other threads' entries
  }
  mx_group_inv(xr, W, groups, eps, sinv, red);
  const int gw = W / groups;
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    MxElem<T>::st(h + (size_t)t * W + c, xr[c] * sinv[c / gw] * w[c]);
}

// Grouped RMSNorm + token shift. With hn(r) = x[r] / rms * w, row t gets
//   h[t] = hn(t) + (prev - hn(t)) * shift,
// prev = hn(t - 1) inside a segment, state[slot] for its first row (zeros at
// position 0). The workgroup of a segment's first row is the only one that
// reads state[slot], and it writes the segment's last hn there afterwards
// (same thread per channel), so no other workgroup races with it.
template <typename T>
__global__ __launch_bounds__(256) void group_norm_shift_kernel(
    T* __restrict__ h, const float* __restrict__ x,
    const float* __restrict__ w, float eps, int groups,
    const float* __restrict__ shift, float* __restrict__ state,
    const int* __restrict__ token_seq, const int* __restrict__ seq_rows,
    int W) {
  __shared__ float red[17];
  __shared__ float sinv[3][MX_MAX_GROUPS];
  const int t = blockIdx.x;
  const int* sr = seq_rows + 4 * token_seq[t];
  const int t0 = sr[0], n = sr[1], p0 = sr[2], slot = sr[3];
  const bool first = t == t0;
  const int last = t0 + n - 1;
  const float* xr = x + (size_t)t * W;
  const float* xp = x + (size_t)(first ? t : t - 1) * W;
  const float* xl = x + (size_t)last * W;
  mx_group_inv(xr, W, groups, eps, sinv[0], red);
  if (!first) mx_group_inv(xp, W, groups, eps, sinv[1], red);
  if (first && n > 1) mx_group_inv(xl, W, groups, eps, sinv[2], red);
  const int gw = W / groups;
  float* st = state + (size_t)slot * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const int g = c / gw;
    const float hn = xr[c] * sinv[0][g] * w[c];
    float prev;
    if (!first) {
      prev = xp[c] * sinv[1][g] * w[c];
    } else {
      prev = p0 > 0 ? st[c] : 0.f;
      st[c] = n > 1 ? xl[c] * sinv[2][g] * w[c] : hn;
    }
    MxElem<T>::st(h + (size_t)t * W + c, hn + (prev - hn) * shift[c]);
  }
}

// Newest stream = base + delta, stored at hist[n-1]; out = sum_j wts[j] *
// hist[j] over the n streams (fp32, ascending j).
template <typename T>
__global__ __launch_bounds__(256) void depth_mix_kernel(
    float* __restrict__ out, float* hist, int n,
    const float* __restrict__ wts, const float* base,
    const T* __restrict__ delta, int ldd, int T_, int W) {
  const size_t TS = (size_t)T_ * W;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < TS;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / W;
    const int c = (int)(idx - t * W);
    const float nw = base[idx] + MxElem<T>::ld(delta + t * ldd + c);
    float acc = 0.f;
    for (int j = 0; j < n - 1; ++j) acc += wts[j] * hist[j * TS + idx];
    acc += wts[n - 1] * nw;
    hist[(size_t)(n - 1) * TS + idx] = nw;
    out[idx] = acc;
  }
}

#define MX_ACT_SILU 0
#define MX_ACT_GELU_TANH 1
#define MX_ACT_CLAMPED_SWISH 2
#define MX_ACT_SIGMOID 3  // sigmoid(g) * u: an output gate
#define MX_ACT_RELU2 4    // relu(g)^2 * u
// up == nullptr: the plain activation (u = 1; the clamped form then has no
// second factor)

template <typename T, int KIND>
__global__ __launch_bounds__(256) void gated_act_kernel(
    T* out, int ldo, const T* __restrict__ gate, int ldg, const T* up,
    int ldu, int F, float limit) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= F) return;
  float g = MxElem<T>::ld(gate + (size_t)t * ldg + c);
  float u = up != nullptr ? MxElem<T>::ld(up + (size_t)t * ldu + c) : 1.f;
  float y;
  if (KIND == MX_ACT_RELU2) {
    const float r = fmaxf(g, 0.f);
    y = r * r * u;
  } else if (KIND == MX_ACT_SILU) {
    y = g * mx_sigmoid(g) * u;
  } else if (KIND == MX_ACT_GELU_TANH) {
    const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    y = 0.5f * g * (1.0f + tanhf(z)) * u;
  } else if (KIND == MX_ACT_SIGMOID) {
    y = mx_sigmoid(g) * u;
  } else {
    g = fminf(g, limit);
    u = up != nullptr ? fminf(fmaxf(u, -limit), limit) : 0.f;
    y = g * mx_sigmoid(1.702f * g) * (u + 1.0f);
  }
  MxElem<T>::st(out + (size_t)t * ldo + c, y);
}

// Eight bf16 entries per thread (16-byte loads and stores); the caller has
// checked widths, strides and pointers for alignment.
template <int KIND>
__global__ __launch_bounds__(256) void gated_act_bf16x8_kernel(
    unsigned short* out, int ldo, const unsigned short* __restrict__ gate,
    int ldg, const unsigned short* up, int ldu, int F, float limit) {
  const int t = blockIdx.y;
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c >= F) return;
  const uint4 gq = *(const uint4*)(gate + (size_t)t * ldg + c);
  // without `up` every factor is 1.0 (bf16 0x3f80)
  const uint4 uq = up != nullptr
                       ? *(const uint4*)(up + (size_t)t * ldu + c)
                       : make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u,
                                    0x3f803f80u);
  const unsigned int gw[4] = {gq.x, gq.y, gq.z, gq.w};
  const unsigned int uw[4] = {uq.x, uq.y, uq.z, uq.w};
  unsigned int ow[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float y[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      float g = __uint_as_float(e ? (gw[k] & 0xffff0000u) : (gw[k] << 16));
      float u = __uint_as_float(e ? (uw[k] & 0xffff0000u) : (uw[k] << 16));
      if (KIND == MX_ACT_RELU2) {
        const float r = fmaxf(g, 0.f);
        y[e] = r * r * u;
      } else if (KIND == MX_ACT_SILU) {
        y[e] = g * mx_sigmoid(g) * u;
      } else if (KIND == MX_ACT_GELU_TANH) {
        const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
        y[e] = 0.5f * g * (1.0f + tanhf(z)) * u;
      } else if (KIND == MX_ACT_SIGMOID) {
        y[e] = mx_sigmoid(g) * u;
      } else {
        g = fminf(g, limit);
        u = up != nullptr ? fminf(fmaxf(u, -limit), limit) : 0.f;
        y[e] = g * mx_sigmoid(1.702f * g) * (u + 1.0f);
      }
    }
    ow[k] = (unsigned int)ps_f32_to_bf16(y[0]) |
            ((unsigned int)ps_f32_to_bf16(y[1]) << 16);
  }
  *(uint4*)(out + (size_t)t * ldo + c) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

// k [T, G*D] (row stride ldk), v [T, G*DV] -> caches [NB, G, BS, D|DV]
template <typename T>
__global__ __launch_bounds__(256) void kv_append_kernel(
    const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    T* __restrict__ kc, T* __restrict__ vc,
    const int64_t* __restrict__ slots, int G, int D, int DV, int BS) {
  const int t = blockIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const int64_t blk = slot / BS;
  const int off = (int)(slot % BS);
  for (int c = threadIdx.x; c < G * D; c += blockDim.x) {
    const int g = c / D, d = c % D;
    kc[((blk * G + g) * BS + off) * (int64_t)D + d] = k[(size_t)t * ldk + c];
  }
  for (int c = threadIdx.x; c < G * DV; c += blockDim.x) {
    const int g = c / DV, d = c % DV;
    vc[((blk * G + g) * BS + off) * (int64_t)DV + d] = v[(size_t)t * ldv + c];
  }
}

// out[t] = scale * sum_i x_i[t] / rms(x_i[t]) * w_i  (fp32), up to four
// inputs of one element type: branch outputs that are normalised one by one
// before they are averaged.
template <typename T>
__global__ __launch_bounds__(256) void norm_sum32_kernel(
    float* __restrict__ out, int n, const T* __restrict__ x0,
    const T* __restrict__ x1, const T* __restrict__ x2,
    const T* __restrict__ x3, int ld0, int ld1, int ld2, int ld3,
    const float* __restrict__ w0, const float* __restrict__ w1,
    const float* __restrict__ w2, const float* __restrict__ w3, float scale,
    float eps, int W) {
  __shared__ float red[17];
  __shared__ float sinv[4];
  const int t = blockIdx.x;
  const T* xs[4] = {x0 + (size_t)t * ld0, x1 + (size_t)t * ld1,
                    x2 + (size_t)t * ld2, x3 + (size_t)t * ld3};
  const float* ws[4] = {w0, w1, w2, w3};
  for (int i = 0; i < n; ++i) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      const float v = MxElem<T>::ld(xs[i] + c);
      ss += v * v;
    }
    ss = mx_block_sum(ss, red);
    if (threadIdx.x == 0) sinv[i] = 1.0f / sqrtf(ss / (float)W + eps);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float acc = 0.f;
    for (int i = 0; i < n; ++i)
      acc += MxElem<T>::ld(xs[i] + c) * sinv[i] * ws[i][c];
    out[(size_t)t * W + c] = acc * scale;
  }
}

// Sublayer boundary of a stack that normalises a sublayer's output before it
// joins the stream: x[t] += d[t] / rms(d[t]) * wpost, then
// h[t] = x[t] / rms(x[t]) * wnext. TD is the element type of the sublayer
// output (fp32 for fp32 sums of experts), T of the next sublayer's input.
// Every thread revisits the entries it wrote itself.
template <typename TD, typename T>
__global__ __launch_bounds__(256) void post_norm_add_norm32_kernel(
    T* __restrict__ h, float* __restrict__ x, const TD* __restrict__ d,
    int ldd, const float* __restrict__ wpost, const float* __restrict__ wnext,
    float eps, int W) {
  __shared__ float red[17];
  const int t = blockIdx.x;
  const TD* dr = d + (size_t)t * ldd;
  float* xr = x + (size_t)t * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = MxElem<TD>::ld(dr + c);
    ss += v * v;
  }
  ss = mx_block_sum(ss, red);
  const float dinv = 1.0f / sqrtf(ss / (float)W + eps);
  float sx = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = xr[c] + MxElem<TD>::ld(dr + c) * dinv * wpost[c];
    xr[c] = v;
    sx += v * v;
  }
  sx = mx_block_sum(sx, red);
  const float xinv = 1.0f / sqrtf(sx / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    MxElem<T>::st(h + (size_t)t * W + c, xr[c] * xinv * wnext[c]);
}

extern "C" {

void mx_embed_scale(void* x, const void* tokens, const void* embed,
                    float scale, int T_, int W, int dtype, void* stream) {
  if (T_ <= 0) return;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((embed_scale_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (float*)x,
                       (const int64_t*)tokens, (const T*)embed, scale, W);
  })
}

void mx_add_group_norm32(void* h, void* xo, const void* xi, const void* d0,
                         int ld0, const void* d1, int ld1, const void* w,
                         float eps, int groups, int T_, int W, int dtype,
                         void* stream) {
  if (T_ <= 0) return;
  if (groups < 1 || groups > MX_MAX_GROUPS || W % groups) return;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((add_group_norm32_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (T*)h, (float*)xo,
                       (const float*)xi, (const T*)d0, ld0, (const T*)d1,
                       ld1, (const float*)w, eps, groups, W);
  })
}

void mx_add_rms_norm32(void* h, void* x, const void* d0, int ld0,
                       const void* d1, int ld1, const void* w, float eps,
                       int T_, int W, int dtype, void* stream) {
  mx_add_group_norm32(h, x, x, d0, ld0, d1, ld1, w, eps, 1, T_, W, dtype,
                      stream);
}

void mx_group_norm_shift(void* h, const void* x, const void* w, float eps,
                         int groups, const void* shift, void* state,
                         const void* token_seq, const void* seq_rows, int T_,
                         int W, int dtype, void* stream) {
  if (T_ <= 0) return;
  if (groups < 1 || groups > MX_MAX_GROUPS || W % groups) return;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((group_norm_shift_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (T*)h, (const float*)x,
                       (const float*)w, eps, groups, (const float*)shift,
                       (float*)state, (const int*)token_seq,
                       (const int*)seq_rows, W);
  })
}

void mx_depth_mix(void* out, void* hist, int n, const void* wts,
                  const void* base, const void* delta, int ldd, int T_, int W,
                  int dtype, void* stream) {
  if (T_ <= 0 || n < 1) return;
  const size_t total = (size_t)T_ * W;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((depth_mix_kernel<T>), dim3((unsigned)blocks),
                       dim3(256), 0, (hipStream_t)stream, (float*)out,
                       (float*)hist, n, (const float*)wts,
                       (const float*)base, (const T*)delta, ldd, T_, W);
  })
}

void mx_gated_act(void* out, int ldo, const void* gate, int ldg,
                  const void* up, int ldu, int T_, int F, int kind,
                  float limit, int dtype, void* stream) {
  if (T_ <= 0 || F <= 0) return;
  if (dtype == MX_BF16 && F % 8 == 0 && ldo % 8 == 0 && ldg % 8 == 0 &&
      ldu % 8 == 0 &&
      (((size_t)out | (size_t)gate | (size_t)up) & 15) == 0) {
    dim3 grid8((F / 8 + 255) / 256, T_);
    typedef unsigned short U;
    if (kind == MX_ACT_RELU2) {
      hipLaunchKernelGGL((gated_act_bf16x8_kernel<MX_ACT_RELU2>), grid8,
                         dim3(256), 0, (hipStream_t)stream, (U*)out, ldo,
                         (const U*)gate, ldg, (const U*)up, ldu, F, limit);
    } else if (kind == MX_ACT_SILU) {
      hipLaunchKernelGGL((gated_act_bf16x8_kernel<MX_ACT_SILU>), grid8,
                         dim3(256), 0, (hipStream_t)stream, (U*)out, ldo,
                         (const U*)gate, ldg, (const U*)up, ldu, F, limit);
    } else if (kind == MX_ACT_GELU_TANH) {
      hipLaunchKernelGGL((gated_act_bf16x8_kernel<MX_ACT_GELU_TANH>), grid8,
                         dim3(256), 0, (hipStream_t)stream, (U*)out, ldo,
                         (const U*)gate, ldg, (const U*)up, ldu, F, limit);
    } else if (kind == MX_ACT_SIGMOID) {
      hipLaunchKernelGGL((gated_act_bf16x8_kernel<MX_ACT_SIGMOID>), grid8,
                         dim3(256), 0, (hipStream_t)stream, (U*)out, ldo,
                         (const U*)gate, ldg, (const U*)up, ldu, F, limit);
    } else {
      hipLaunchKernelGGL((gated_act_bf16x8_kernel<MX_ACT_CLAMPED_SWISH>),
                         grid8, dim3(256), 0, (hipStream_t)stream, (U*)out,
                         ldo, (const U*)gate, ldg, (const U*)up, ldu, F,
                         limit);
    }
    return;
  }
  dim3 grid((F + 255) / 256, T_);
  MX_DISPATCH_DTYPE(dtype, {
    if (kind == MX_ACT_RELU2) {
      hipLaunchKernelGGL((gated_act_kernel<T, MX_ACT_RELU2>), grid, dim3(256),
                         0, (hipStream_t)stream, (T*)out, ldo,
                         (const T*)gate, ldg, (const T*)up, ldu, F, limit);
    } else if (kind == MX_ACT_SILU) {
      hipLaunchKernelGGL((gated_act_kernel<T, MX_ACT_SILU>), grid, dim3(256),
                         0, (hipStream_t)stream, (T*)out, ldo,
                         (const T*)gate, ldg, (const T*)up, ldu, F, limit);
    } else if (kind == MX_ACT_GELU_TANH) {
      hipLaunchKernelGGL((gated_act_kernel<T, MX_ACT_GELU_TANH>), grid,
                         dim3(256), 0, (hipStream_t)stream, (T*)out, ldo,
                         (const T*)gate, ldg, (const T*)up, ldu, F, limit);
    } else if (kind == MX_ACT_SIGMOID) {
      hipLaunchKernelGGL((gated_act_kernel<T, MX_ACT_SIGMOID>), grid,
                         dim3(256), 0, (hipStream_t)stream, (T*)out, ldo,
                         (const T*)gate, ldg, (const T*)up, ldu, F, limit);
    } else {
      hipLaunchKernelGGL((gated_act_kernel<T, MX_ACT_CLAMPED_SWISH>), grid,
                         dim3(256), 0, (hipStream_t)stream, (T*)out, ldo,
                         (const T*)gate, ldg, (const T*)up, ldu, F, limit);
    }
  })
}

void mx_kv_append(const void* k, int ldk, const void* v, int ldv, void* kc,
                  void* vc, const void* slots, int T_, int G, int D, int DV,
                  int BS, int dtype, void* stream) {
  if (T_ <= 0) return;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((kv_append_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (const T*)k, ldk, (const T*)v,
                       ldv, (T*)kc, (T*)vc, (const int64_t*)slots, G, D, DV,
                       BS);
  })
}

void mx_norm_sum32(void* out, int n, const void* x0, const void* x1,
                   const void* x2, const void* x3, int ld0, int ld1, int ld2,
                   int ld3, const void* w0, const void* w1, const void* w2,
                   const void* w3, float scale, float eps, int T_, int W,
                   int dtype, void* stream) {
  if (T_ <= 0 || n < 1 || n > 4) return;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((norm_sum32_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (float*)out, n, (const T*)x0,
                       (const T*)x1, (const T*)x2, (const T*)x3, ld0, ld1,
                       ld2, ld3, (const float*)w0, (const float*)w1,
                       (const float*)w2, (const float*)w3, scale, eps, W);
  })
}

void mx_post_norm_add_norm32(void* h, void* x, const void* d, int ldd,
                             int d_dtype, const void* wpost,
                             const void* wnext, float eps, int T_, int W,
                             int dtype, void* stream) {
  if (T_ <= 0) return;
  MX_DISPATCH_DTYPE(dtype, {
    if (d_dtype == MX_BF16) {
      hipLaunchKernelGGL((post_norm_add_norm32_kernel<mx_bf16, T>), dim3(T_),
                         dim3(256), 0, (hipStream_t)stream, (T*)h, (float*)x,
                         (const mx_bf16*)d, ldd, (const float*)wpost,
                         (const float*)wnext, eps, W);
    } else {
      hipLaunchKernelGGL((post_norm_add_norm32_kernel<float, T>), dim3(T_),
                         dim3(256), 0, (hipStream_t)stream, (T*)h, (float*)x,
                         (const float*)d, ldd, (const float*)wpost,
                         (const float*)wnext, eps, W);
    }
  })
}

}  // extern "C"
