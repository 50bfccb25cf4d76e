// Caller-side helper of a GPT block: the fused query/key/value projection is split into
// contiguous (B, heads, T, hs) tensors and the rotary embedding is applied to q and k on the
// way, in one pass (reference: model.py:474-497 views qkv as (B, T, groups, q_per_kv + 2, hs),
// permutes and splits it; model.py:812-825 apply_rope on the first rope_n channels; the
// attention then wants contiguous q, k, v, model.py:572-574).  HBM-bound: every element is read
// once and written once.
//   out = x * cos + rot(x) * sin,  rot(x) = (-x2, x1) with x1, x2 the halves of x[:rope_n]
// The gradient kernel is the adjoint: dx = dy * cos + rotT(dy * sin), rotT(z) = (z2, -z1).
// With q == nullptr the rotation (or its adjoint) is applied IN PLACE to the q and k rows of the
// packed tensor and nothing is copied (a thread reads and writes both halves of its channels, so in
// place is safe).  With q != nullptr and k == nullptr, q is a second packed tensor
// (b, t, groups, q_per_kv + 1, hs) that receives the rotated q and k rows (v is not touched).  Either
// way the attention kernels then read q, k, v as strided views of the packed tensors.
#pragma once
#include "fm_common.h"

struct RopeShape {
  int b, t, groups, qpk, hs, rn;  // rn = rotary channels (even, a multiple of 8, <= hs)
};

// One thread = one unit of a (b, t, slot) row: a rotary unit covers channels [4u, 4u+4) and their
// partners [4u + rn/2, ...); a copy unit covers four channels at or beyond rn.  slot < qpk: query
// head g*qpk + slot; slot == qpk: key head g; slot == qpk + 1: value head g (no rotation).
template <class T, bool GRAD>
__global__ __launch_bounds__(256) void qkv_rope_kernel(RopeShape s, T* __restrict__ qkv,
                                                       const float* __restrict__ cosv,
                                                       const float* __restrict__ sinv, T* __restrict__ q,
                                                       T* __restrict__ k, T* __restrict__ v) {
  const int upr = s.hs / 4;  // units per row (upper bound: all copy units)
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)s.b * s.t * s.groups * (s.qpk + 2) * upr;
  if (idx >= total) return;
  const int u = (int)(idx % upr);
  int64_t r = idx / upr;
  const int slot = (int)(r % (s.qpk + 2));
  r /= (s.qpk + 2);
  const int g = (int)(r % s.groups);
  r /= s.groups;
  const int t = (int)(r % s.t);
  const int b = (int)(r / s.t);
  T* src = qkv + ((((int64_t)b * s.t + t) * s.groups + g) * (s.qpk + 2) + slot) * s.hs;
  T* dst;
  const bool inplace = q == nullptr, packed = k == nullptr;   // (packed: no split, no copy units)
  if (inplace) dst = src;
  else if (packed) dst = q + ((((int64_t)b * s.t + t) * s.groups + g) * (s.qpk + 1) + (slot <= s.qpk ? slot : 0)) * s.hs;
  else if (slot < s.qpk) dst = q + (((int64_t)b * s.groups * s.qpk + g * s.qpk + slot) * s.t + t) * s.hs;
  else if (slot == s.qpk) dst = k + (((int64_t)b * s.groups + g) * s.t + t) * s.hs;
  else dst = v + (((int64_t)b * s.groups + g) * s.t + t) * s.hs;
  // forward reads the packed row and writes the split tensor; the gradient goes the other way
  T* from = GRAD ? dst : src;
  T* to = GRAD ? src : dst;
  const int rn = slot <= s.qpk ? s.rn : 0;
  const int nrot = rn / 8;  // rotary units
  if (u < nrot) {
    const int c = 4 * u, h = rn / 2;
    float x1[4], x2[4], y1[4], y2[4];
    load4(from + c, x1);
    load4(from + c + h, x2);
    const float4 c1 = *reinterpret_cast<const float4*>(cosv + (int64_t)t * rn + c);
    const float4 s1 = *reinterpret_cast<const float4*>(sinv + (int64_t)t * rn + c);
    const float4 c2 = *reinterpret_cast<const float4*>(cosv + (int64_t)t * rn + c + h);
    const float4 s2 = *reinterpret_cast<const float4*>(sinv + (int64_t)t * rn + c + h);
    const float cc1[4] = {c1.x, c1.y, c1.z, c1.w}, ss1[4] = {s1.x, s1.y, s1.z, s1.w};
    const float cc2[4] = {c2.x, c2.y, c2.z, c2.w}, ss2[4] = {s2.x, s2.y, s2.z, s2.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (GRAD) {  // dx1 = dy1 c1 + dy2 s2,  dx2 = dy2 c2 - dy1 s1
        y1[e] = x1[e] * cc1[e] + x2[e] * ss2[e];
        y2[e] = x2[e] * cc2[e] - x1[e] * ss1[e];
      } else {     // y1 = x1 c1 - x2 s1,  y2 = x2 c2 + x1 s2
        y1[e] = x1[e] * cc1[e] - x2[e] * ss1[e];
        y2[e] = x2[e] * cc2[e] + x1[e] * ss2[e];
      }
    }
    store4(to + c, y1);
    store4(to + c + h, y2);
  } else if (!packed || (!inplace && slot <= s.qpk)) {
    const int c = rn + 4 * (u - nrot);
    if (c < s.hs) {
      float x[4];
      load4(from + c, x);
      store4(to + c, x);
    }
  }
}

// Wider variant for hs % 16 == 0 and rn % 16 == 0 (the usual head sizes): a unit is 16 channels --
// a rotary unit covers [8u, 8u+8) and their partners [8u + rn/2, ...), a copy unit 16 contiguous
// channels at or beyond rn -- so every thread of a row has work and every access is 16 bytes
// (bf16) or two of them (fp32).
__device__ __forceinline__ void load8(const float* p, float (&o)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float (&o)[8]) {
  const uint4 u = *reinterpret_cast<const uint4*>(p);
  o[0] = bf_lo(u.x); o[1] = bf_hi(u.x); o[2] = bf_lo(u.y); o[3] = bf_hi(u.y);
  o[4] = bf_lo(u.z); o[5] = bf_hi(u.z); o[6] = bf_lo(u.w); o[7] = bf_hi(u.w);
}
__device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16_t* p, const float (&v)[8]) {
  *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7]));
}

template <class T, bool GRAD>
__global__ __launch_bounds__(256) void qkv_rope16_kernel(RopeShape s, T* __restrict__ qkv,
                                                         const float* __restrict__ cosv,
                                                         const float* __restrict__ sinv, T* __restrict__ q,
                                                         T* __restrict__ k, T* __restrict__ v) {
  const int upr = s.hs / 16;  // units per row
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)s.b * s.t * s.groups * (s.qpk + 2) * upr;
  if (idx >= total) return;
  const int u = (int)(idx % upr);
  int64_t r = idx / upr;
  const int slot = (int)(r % (s.qpk + 2));
  r /= (s.qpk + 2);
  const int g = (int)(r % s.groups);
  r /= s.groups;
  const int t = (int)(r % s.t);
  const int b = (int)(r / s.t);
  T* src = qkv + ((((int64_t)b * s.t + t) * s.groups + g) * (s.qpk + 2) + slot) * s.hs;
  T* dst;
  const bool inplace = q == nullptr, packed = k == nullptr;   // (packed: no split, no copy units)
  if (inplace) dst = src;
  else if (packed) dst = q + ((((int64_t)b * s.t + t) * s.groups + g) * (s.qpk + 1) + (slot <= s.qpk ? slot : 0)) * s.hs;
  else if (slot < s.qpk) dst = q + (((int64_t)b * s.groups * s.qpk + g * s.qpk + slot) * s.t + t) * s.hs;
  else if (slot == s.qpk) dst = k + (((int64_t)b * s.groups + g) * s.t + t) * s.hs;
  else dst = v + (((int64_t)b * s.groups + g) * s.t + t) * s.hs;
  T* from = GRAD ? dst : src;
  T* to = GRAD ? src : dst;
  const int rn = slot <= s.qpk ? s.rn : 0;
  const int nrot = rn / 16;  // rotary units
  if (u < nrot) {
    const int c = 8 * u, h = rn / 2;
    float x1[8], x2[8], c1[8], s1[8], c2[8], s2[8], y1[8], y2[8];
    load8(from + c, x1);
    load8(from + c + h, x2);
    load8(cosv + (int64_t)t * rn + c, c1);
    load8(sinv + (int64_t)t * rn + c, s1);
    load8(cosv + (int64_t)t * rn + c + h, c2);
    load8(sinv + (int64_t)t * rn + c + h, s2);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (GRAD) {  // dx1 = dy1 c1 + dy2 s2,  dx2 = dy2 c2 - dy1 s1
        y1[e] = x1[e] * c1[e] + x2[e] * s2[e];
        y2[e] = x2[e] * c2[e] - x1[e] * s1[e];
      } else {     // y1 = x1 c1 - x2 s1,  y2 = x2 c2 + x1 s2
        y1[e] = x1[e] * c1[e] - x2[e] * s1[e];
        y2[e] = x2[e] * c2[e] + x1[e] * s2[e];
      }
    }
    store8(to + c, y1);
    store8(to + c + h, y2);
  } else if (!packed || (!inplace && slot <= s.qpk)) {
    const int c = rn + 16 * (u - nrot);
    float x[8], y[8];
    load8(from + c, x);
    load8(from + c + 8, y);
    store8(to + c, x);
    store8(to + c + 8, y);
  }
}
