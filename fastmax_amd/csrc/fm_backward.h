// Small backward-side kernels: the per-token scalar c_i and the normalisation chain rule.
#pragma once
#include <type_traits>

#include "fm_common.h"

// c_i = (go_i . o_i) / den_i, one value per token; grid = (row blocks, heads).  A row is shared by
// d/4 threads, or, VEC, by d/8 threads for bf16 rows: 16 bytes per thread and tensor (VEC needs rows
// of o and go that start on 16-byte boundaries; otherwise they are read element by element, e.g.
// from the (d+1)-column layout).
template <class T, bool VEC>
__global__ __launch_bounds__(256) void bwd_prep_kernel(Rows<const T> go, Rows<const T> o, RowScalars den,
                                                       float* __restrict__ cvec, int rows, int d) {
  constexpr int EPT = VEC ? (std::is_same<T, float>::value ? 4 : 8) : 4;
  // threads per row: the pieces of a row rounded up to a power of two (shuffle reduction)
  const int npc = d / EPT;
  int tpr = 1;
  while (tpr < npc) tpr *= 2;
  const int rpp = 256 / tpr;
  const int sub = threadIdx.x % tpr;
  const int head = blockIdx.y;
  const int row = blockIdx.x * rpp + threadIdx.x / tpr;
  float s = 0.f;
  if (row < rows && sub < npc) {
    const HeadRows<const T> gh = go.head(head), oh = o.head(head);
    const T* grow = gh.row(row) + sub * EPT;
    const T* orow = oh.row(row) + sub * EPT;
    if constexpr (VEC && !std::is_same<T, float>::value) {
      const uint4 a = *reinterpret_cast<const uint4*>(grow), b = *reinterpret_cast<const uint4*>(orow);
      s = (bf_lo(a.x) * bf_lo(b.x) + bf_hi(a.x) * bf_hi(b.x) + bf_lo(a.y) * bf_lo(b.y) + bf_hi(a.y) * bf_hi(b.y)) +
          (bf_lo(a.z) * bf_lo(b.z) + bf_hi(a.z) * bf_hi(b.z) + bf_lo(a.w) * bf_lo(b.w) + bf_hi(a.w) * bf_hi(b.w));
    } else {
      float a[4], b[4];
      if constexpr (VEC) {
        load4(grow, a);
        load4(orow, b);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[e] = to_f32(grow[e]);
          b[e] = to_f32(orow[e]);
        }
      }
      s = a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
    }
  }
  for (int off = tpr >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (row < rows && sub == 0) cvec[(int64_t)head * rows + row] = s / den.head(head)[(int64_t)row * den.stride];
}

// ---------------------------------------------------------------------------------------
// Chain rule through x_hat = lim * x / max_n ||x_n||: the scaling by lim/M is already in dx;
// the max-norm row i* additionally gets  dx[i*] -= (sum dx_hat.x_hat) * x[i*] / M^2.
// One launch serves both sides: blocks [0, heads of side a) fix dq, the rest dk; one block per head,
// blockDim.x = d.  A row index outside [0, n) (only a caller-supplied qk_argmax can hold one) leaves
// the head untouched.
// ---------------------------------------------------------------------------------------
template <class T>
struct NormFixSide {
  Rows<T> dx;
  Rows<const T> x;
  const float* scale;
  const int* arg;
  const float* rpart;
  int heads, nblk, n;
};

template <class T>
__global__ void norm_fix_kernel(NormFixSide<T> a, NormFixSide<T> b, int d, float lim) {
  const bool first = (int)blockIdx.x < a.heads;
  const NormFixSide<T>& sd = first ? a : b;
  const int head = first ? blockIdx.x : blockIdx.x - a.heads, c = threadIdx.x;
  const int row = sd.arg[head];
  if (row < 0 || row >= sd.n) return;
  // the block's threads share the partials (fixed order per thread and in the tree: the same sum every run)
  __shared__ float red[128];
  float r = 0.f;
  for (int bl = c; bl < sd.nblk; bl += blockDim.x) r += sd.rpart[(int64_t)head * sd.nblk + bl];
  red[c] = r;
  __syncthreads();
  r = 0.f;
  for (int t = 0; t < (int)blockDim.x; ++t) r += red[t];
  const float s = sd.scale[head];
  const float fac = r * s * s / (lim * lim);
  const HeadRows<T> dh = sd.dx.head(head);
  const HeadRows<const T> xh = sd.x.head(head);
  T* dst = dh.row(row) + c;
  *dst = from_f32<T>(to_f32(*dst) - fac * to_f32(xh.row(row)[c]));
}

// ---------------------------------------------------------------------------------------
// Grouped key/value heads: out[g] = sum of the `ratio` per-query-head gradients of group g
// (fixed order, fp32 sum).  part holds n x d contiguous elements per query head;
// grid = (ceil(n * d / 1024), groups).
// ---------------------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(256) void group_sum_kernel(const T* __restrict__ part, Rows<T> out, int n, int d,
                                                        int ratio) {
  const int64_t per_head = (int64_t)n * d;
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
  const HeadRows<T> oh = out.head((int)g);
  store4(oh.row((int)(idx / d)) + idx % d, a);
}
