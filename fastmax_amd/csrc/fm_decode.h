// Recurrent form of Fastmax attention: the fp32 moment state of a head is carried between
// calls (the role a key/value cache plays for softmax attention, reference model.py:828-852).
//   state_accumulate_kernel  state (+)= sum of the partial states an unmasked build wrote
//   decode_update_kernel     one new token per head: state += phi(k) (x) [v,1], and the partial
//                            products phi(q) . state of a slice of the state rows
//   decode_finish_kernel     adds the slices and divides by the denominator
// Everything is HBM-bound: a step reads and writes each state once (592 KB per head at
// d = 64, p = 2).
#pragma once
#include "fm_common.h"

// state[head] = (accumulate ? state[head] : 0) + sum_{part < nparts} slots[head][part]
// (state[head] starts at state + head * state_stride floats; it may be a further slot of `slots`)
// grid = (ceil(state_floats / 1024), heads), 256 threads, one float4 each.
__global__ __launch_bounds__(256) void state_accumulate_kernel(float* __restrict__ state, int64_t state_stride,
                                                               const float* __restrict__ slots,
                                                               int nslots, int nparts, int64_t ss,
                                                               int accumulate) {
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (idx >= ss) return;
  const int head = blockIdx.y;
  float4* dst = reinterpret_cast<float4*>(state + (int64_t)head * state_stride + idx);
  float4 a = accumulate ? *dst : make_float4(0.f, 0.f, 0.f, 0.f);
  for (int part = 0; part < nparts; ++part) {
    const float4 t = *reinterpret_cast<const float4*>(slots + ((int64_t)head * nslots + part) * ss + idx);
    a.x += t.x; a.y += t.y; a.z += t.z; a.w += t.w;
  }
  *dst = a;
}

// grid = (rsplit, key/value heads).  Block (split, head) owns state rows [rows*split/rsplit,
// rows*(split+1)/rsplit) of that key/value head's state; a thread owns one 16-byte piece of a row
// per sweep.  The state takes in (k, v) during the sweep for the group's first query head; the
// other `ratio - 1` query heads of the group (fastmax_cuda_forward.cu:38) sweep the updated rows
// again (each thread re-reads what it wrote itself).
template <int D, class T>
__global__ __launch_bounds__(256) void decode_update_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const float* __restrict__ qscale, const float* __restrict__ kscale, float kdefault,
    float* __restrict__ state, float* __restrict__ part, int p2, float a0, float a1, float a2, int ratio) {
  using G = Geo<D>;
  constexpr int LD = G::LD, VPR = LD / 4, RPI = 256 / VPR, H2 = G::H2;
  __shared__ float ql[D], kl[D];
  __shared__ __attribute__((aligned(16))) float vl[LD];
  __shared__ float4 red[RPI][VPR];
  const int tid = threadIdx.x, split = blockIdx.x, rsplit = gridDim.x, head = blockIdx.y;
  if (tid < D) {
    kl[tid] = to_f32(k[(int64_t)head * D + tid]) * (kscale ? kscale[head] : kdefault);
    vl[tid] = to_f32(v[(int64_t)head * D + tid]);
  } else if (tid < LD) {
    vl[tid] = tid == D ? 1.0f : 0.f;  // the extra column counts the token; the padding stays put
  }
  const int rows = G::rows(p2), rows2 = G::rows2(p2);
  const int r_lo = (int)((int64_t)rows * split / rsplit), r_hi = (int)((int64_t)rows * (split + 1) / rsplit);
  const int c4 = tid % VPR, rr = tid / VPR;
  for (int j = 0; j < ratio; ++j) {
    const int qh = head * ratio + j;
    __syncthreads();   // (ql and red of the previous query head are no longer read)
    if (tid < D) ql[tid] = to_f32(q[(int64_t)qh * D + tid]) * (qscale ? qscale[qh] : 1.0f);
    __syncthreads();
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (rr < RPI) {
      const float4 vx = *reinterpret_cast<const float4*>(vl + 4 * c4);
      float* sh = state + (int64_t)head * G::state_floats(p2);
      // four rows per sweep: their loads are issued together (the kernel is bound by HBM latency x
      // bytes in flight, and the compiler cannot move a load above the store of the row before)
      constexpr int UB = 4;
      for (int row0 = r_lo + rr; row0 < r_hi; row0 += UB * RPI) {
        float4 s4[UB];
#pragma unroll
        for (int u = 0; u < UB; ++u) {
          const int row = row0 + u * RPI;
          s4[u] = row < r_hi ? *reinterpret_cast<const float4*>(sh + (int64_t)row * LD + 4 * c4)
                             : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < UB; ++u) {
          const int row = row0 + u * RPI;
          if (row >= r_hi) break;
          float fk, fq;
          if (row < rows2) {
            const int s = row / D, a = row % D, b = (a + s) & (D - 1);
            fk = kl[a] * kl[b];
            fq = ((s == 0 || s == H2) ? a2 : 2.0f * a2) * ql[a] * ql[b];
          } else if (row < rows2 + D) {
            fk = kl[row - rows2];
            fq = a1 * ql[row - rows2];
          } else {
            fk = 1.0f;
            fq = a0;
          }
          float4 t = s4[u];
          if (j == 0) {
            t.x += fk * vx.x; t.y += fk * vx.y; t.z += fk * vx.z; t.w += fk * vx.w;
            *reinterpret_cast<float4*>(sh + (int64_t)row * LD + 4 * c4) = t;
          }
          acc.x += fq * t.x; acc.y += fq * t.y; acc.z += fq * t.z; acc.w += fq * t.w;
        }
      }
      red[rr][c4] = acc;
    }
    __syncthreads();
    if (tid < VPR) {
      float4 t = red[0][tid];
      for (int r = 1; r < RPI; ++r) {
        const float4 u = red[r][tid];
        t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
      }
      *reinterpret_cast<float4*>(part + ((int64_t)qh * rsplit + split) * LD + 4 * tid) = t;
    }
  }
}

// grid = heads, LD threads: column c of the numerator (c < D) or the denominator (c == D)
template <int D, class T>
__global__ void decode_finish_kernel(const float* __restrict__ part, int rsplit, T* __restrict__ o,
                                     int64_t ldo, float* __restrict__ den, int64_t den_stride) {
  constexpr int LD = Geo<D>::LD;
  __shared__ float dsh;
  const int head = blockIdx.x, c = threadIdx.x;
  float s = 0.f;
  for (int sp = 0; sp < rsplit; ++sp) s += part[((int64_t)head * rsplit + sp) * LD + c];
  if (c == D) dsh = s;
  __syncthreads();
  if (c < D) o[(int64_t)head * ldo + c] = from_f32<T>(s / dsh);
  if (c == D && den) den[(int64_t)head * den_stride] = s;
}
