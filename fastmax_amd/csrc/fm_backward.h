// Small backward-side kernels: the per-token scalar c_i and the normalisation chain rule.
#pragma once
#include <type_traits>

#include "fm_common.h"

// c_i = (go_i . o_i) / den_i, one value per token.  A row is shared by d/4 threads, or, VEC, by
// d/8 threads for bf16 rows: 16 bytes per thread and tensor (VEC needs rows of o that start on a
// 16-byte boundary; otherwise o is read element by element, e.g. from the (d+1)-column layout).
template <class T, bool VEC>
__global__ __launch_bounds__(256) void bwd_prep_kernel(const T* __restrict__ go,
                                                       const T* __restrict__ o, int64_t ldo,
                                                       const float* __restrict__ den,
                                                       int64_t den_stride, float* __restrict__ cvec,
                                                       int64_t rows, int d) {
  constexpr int EPT = VEC ? (std::is_same<T, float>::value ? 4 : 8) : 4;
  const int tpr = d / EPT, rpp = 256 / tpr;
  const int sub = threadIdx.x % tpr;
  const int64_t row = (int64_t)blockIdx.x * rpp + threadIdx.x / tpr;
  float s = 0.f;
  if (row < rows) {
    const T* grow = go + row * d + sub * EPT;
    const T* orow = o + row * ldo + sub * EPT;
    if constexpr (VEC && !std::is_same<T, float>::value) {
      const uint4 a = *reinterpret_cast<const uint4*>(grow), b = *reinterpret_cast<const uint4*>(orow);
      s = (bf_lo(a.x) * bf_lo(b.x) + bf_hi(a.x) * bf_hi(b.x) + bf_lo(a.y) * bf_lo(b.y) + bf_hi(a.y) * bf_hi(b.y)) +
          (bf_lo(a.z) * bf_lo(b.z) + bf_hi(a.z) * bf_hi(b.z) + bf_lo(a.w) * bf_lo(b.w) + bf_hi(a.w) * bf_hi(b.w));
    } else {
      float a[4], b[4];
      load4(grow, a);
      if constexpr (VEC) {
        load4(orow, b);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) b[e] = to_f32(orow[e]);
      }
      s = a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
    }
  }
  for (int off = tpr >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (row < rows && sub == 0) cvec[row] = s / den[row * den_stride];
}

// ---------------------------------------------------------------------------------------
// Chain rule through x_hat = lim * x / max_n ||x_n||: the scaling by lim/M is already in dx;
// the max-norm row i* additionally gets  dx[i*] -= (sum dx_hat.x_hat) * x[i*] / M^2.
// One block per head; blockDim.x = d.  A row index outside [0, n) (only a caller-supplied
// qk_argmax can hold one) leaves the head untouched.
// ---------------------------------------------------------------------------------------
template <class T>
__global__ void norm_fix_kernel(T* __restrict__ dx, const T* __restrict__ x,
                                const float* __restrict__ scale, const int* __restrict__ arg,
                                const float* __restrict__ rpart, int nblk, int n, int d, float lim) {
  const int head = blockIdx.x, c = threadIdx.x;
  const int row = arg[head];
  if (row < 0 || row >= n) return;
  float r = 0.f;
  for (int b = 0; b < nblk; ++b) r += rpart[(int64_t)head * nblk + b];
  const float s = scale[head];
  const float fac = r * s * s / (lim * lim);
  const int64_t off = ((int64_t)head * n + row) * d + c;
  dx[off] = from_f32<T>(to_f32(dx[off]) - fac * to_f32(x[off]));
}

// ---------------------------------------------------------------------------------------
// Grouped key/value heads: out[g] = sum of the `ratio` per-query-head gradients of group g
// (fixed order, fp32 sum).  grid = (ceil(per_head / 1024), groups); per_head = n*d elements.
// ---------------------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(256) void group_sum_kernel(const T* __restrict__ part, T* __restrict__ out,
                                                        int64_t per_head, int ratio) {
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (idx >= per_head) return;
  const int64_t g = blockIdx.y;
  float a[4] = {0.f, 0.f, 0.f, 0.f};
  for (int r = 0; r < ratio; ++r) {
    float t[4];
    load4(part + (g * ratio + r) * per_head + idx, t);
#pragma unroll
    for (int e = 0; e < 4; ++e) a[e] += t[e];
  }
  store4(out + g * per_head + idx, a);
}
