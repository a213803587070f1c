// Minimal gated recurrent unit: an element-wise recurrence over a ragged
// batch,
//   a = sigmoid(z + zb),  u' = u + ub,
//   c = u' + 1/2 (u' >= 0) | sigmoid(u') (u' < 0),
//   S <- (1 - a) S + a c,   out = S * silu(g),
// with S fp32 per sequence and channel. All arithmetic is fp32; the element
// type decides loads and the final rounding.
//
// Short segments (single tokens, small portions): a thread owns one channel
// of one segment and walks its rows in order; the loads of a row do not
// depend on the recurrence, so the loop is unrolled and they run ahead.
//
// Long segments are cut into tiles of MG_TILE rows, because one step of the
// recurrence is the affine map S -> (1 - a) S + a c and maps compose:
//   pass 1  per (tile, channel) the tile's composed map (A, B) = (product of
//           the (1 - a), the tile's result from S = 0); the first tile of a
//           segment also copies the sequence's state aside;
//   pass 2  per (tile, channel) the state at the tile's start, by folding
//           the maps of the segment's earlier tiles over the saved state,
//           then the tile's rows in order with the read-out; the last tile
//           stores the new state.
// Pass 2 reads the saved copy, so the store of the new state races with
// nothing.
#include "mix_common.h"

#define MG_TILE 128

// Three sigmoids per element make these kernels arithmetic-bound with the
// library's range-checked exponential and IEEE division, so they use the
// hardware exponential and reciprocal (fp32, a few ulp).
PS_DEV float mg_sigmoid(float x) {
  return __fdividef(1.0f, 1.0f + __expf(-x));
}

PS_DEV void mg_gate(float zv, float uv, float bz, float bu, float* a,
                    float* cand) {
  *a = mg_sigmoid(zv + bz);
  const float uu = uv + bu;
  *cand = uu >= 0.f ? uu + 0.5f : mg_sigmoid(uu);
}

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
    float a, cand;
    mg_gate(MxElem<T>::ld(z + t * ldz + c), MxElem<T>::ld(u + t * ldu + c),
            bz, bu, &a, &cand);
    const float gg = MxElem<T>::ld(g + t * ldg + c);
    S = (1.0f - a) * S + a * cand;
    MxElem<T>::st(out + t * ldo + c, S * (gg * mg_sigmoid(gg)));
  }
  state[(size_t)slot * C + c] = S;
}

// grid (channel blocks, segments, tiles). maps [segments][tiles][2][C],
// init [segments][C].
template <typename T>
__global__ __launch_bounds__(64) void mingru_tile_map_kernel(
    const T* __restrict__ z, int ldz, const T* __restrict__ u, int ldu,
    const float* __restrict__ zb, const float* __restrict__ ub,
    const float* __restrict__ state, const int* __restrict__ seq_rows, int C,
    float* __restrict__ maps, float* __restrict__ init) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int* sr = seq_rows + 4 * blockIdx.y;
  const int t0 = sr[0], n = sr[1], p0 = sr[2], slot = sr[3];
  const int r0 = blockIdx.z * MG_TILE;
  if (r0 >= n) return;
  if (blockIdx.z == 0)
    init[(size_t)blockIdx.y * C + c] =
        p0 > 0 ? state[(size_t)slot * C + c] : 0.f;
  const int r1 = min(n, r0 + MG_TILE);
  const float bz = zb[c], bu = ub[c];
  float A = 1.f, B = 0.f;
#pragma unroll 8
  for (int r = r0; r < r1; ++r) {
    const size_t t = (size_t)(t0 + r);
    float a, cand;
    mg_gate(MxElem<T>::ld(z + t * ldz + c), MxElem<T>::ld(u + t * ldu + c),
            bz, bu, &a, &cand);
    A *= 1.0f - a;
    B = (1.0f - a) * B + a * cand;
  }
  float* m = maps + ((size_t)blockIdx.y * gridDim.z + blockIdx.z) * 2 * C;
  m[c] = A;
  m[C + c] = B;
}

template <typename T>
__global__ __launch_bounds__(64) void mingru_tile_scan_kernel(
    T* __restrict__ out, int ldo, const T* __restrict__ z, int ldz,
    const T* __restrict__ u, int ldu, const T* __restrict__ g, int ldg,
    const float* __restrict__ zb, const float* __restrict__ ub,
    float* __restrict__ state, const int* __restrict__ seq_rows, int C,
    const float* __restrict__ maps, const float* __restrict__ init) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int* sr = seq_rows + 4 * blockIdx.y;
  const int t0 = sr[0], n = sr[1], slot = sr[3];
  const int r0 = blockIdx.z * MG_TILE;
  if (r0 >= n) return;
  const int r1 = min(n, r0 + MG_TILE);
  float S = init[(size_t)blockIdx.y * C + c];
  const float* m = maps + (size_t)blockIdx.y * gridDim.z * 2 * C;
  for (int j = 0; j < (int)blockIdx.z; ++j)
    S = m[(size_t)j * 2 * C + c] * S + m[(size_t)j * 2 * C + C + c];
  const float bz = zb[c], bu = ub[c];
#pragma unroll 8
  for (int r = r0; r < r1; ++r) {
    const size_t t = (size_t)(t0 + r);
    float a, cand;
    mg_gate(MxElem<T>::ld(z + t * ldz + c), MxElem<T>::ld(u + t * ldu + c),
            bz, bu, &a, &cand);
    const float gg = MxElem<T>::ld(g + t * ldg + c);
    S = (1.0f - a) * S + a * cand;
    MxElem<T>::st(out + t * ldo + c, S * (gg * mg_sigmoid(gg)));
  }
  if (r1 == n) state[(size_t)slot * C + c] = S;
}

extern "C" {

// fp32 entries of scratch the tiled form needs (0: the plain kernel runs)
long mx_mingru_scratch(int S_, int C, int T_) {
  if (S_ <= 0 || T_ <= 0) return 0;
  const int longest = T_ - (S_ - 1);
  if (longest <= MG_TILE) return 0;
  const long tiles = (longest + MG_TILE - 1) / MG_TILE;
  return (long)S_ * tiles * 2 * C + (long)S_ * C;
}

void mx_mingru_scan(void* out, int ldo, const void* z, int ldz, const void* u,
                    int ldu, const void* g, int ldg, const void* zb,
                    const void* ub, void* state, const void* seq_rows, int S_,
                    int C, int T_, void* scratch, int dtype, void* stream) {
  if (S_ <= 0 || T_ <= 0 || C <= 0) return;
  const int longest = T_ - (S_ - 1);
  if (longest <= MG_TILE || scratch == nullptr) {
    dim3 grid((C + 63) / 64, S_);
    MX_DISPATCH_DTYPE(dtype, {
      hipLaunchKernelGGL((mingru_scan_kernel<T>), grid, dim3(64), 0,
                         (hipStream_t)stream, (T*)out, ldo, (const T*)z, ldz,
                         (const T*)u, ldu, (const T*)g, ldg,
                         (const float*)zb, (const float*)ub, (float*)state,
                         (const int*)seq_rows, C);
    })
    return;
  }
  const int tiles = (longest + MG_TILE - 1) / MG_TILE;
  float* maps = (float*)scratch;
  float* init = maps + (size_t)S_ * tiles * 2 * C;
  dim3 grid((C + 63) / 64, S_, tiles);
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((mingru_tile_map_kernel<T>), grid, dim3(64), 0,
                       (hipStream_t)stream, (const T*)z, ldz, (const T*)u,
                       ldu, (const float*)zb, (const float*)ub,
                       (const float*)state, (const int*)seq_rows, C, maps,
                       init);
    hipLaunchKernelGGL((mingru_tile_scan_kernel<T>), grid, dim3(64), 0,
                       (hipStream_t)stream, (T*)out, ldo, (const T*)z, ldz,
                       (const T*)u, ldu, (const T*)g, ldg, (const float*)zb,
                       (const float*)ub, (float*)state, (const int*)seq_rows,
                       C, (const float*)maps, (const float*)init);
  })
}

}  // extern "C"
