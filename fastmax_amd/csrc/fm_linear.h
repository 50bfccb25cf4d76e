// Causal p = 1 (f(s) = a0 + a1 s) at head dimension 64 as ONE sequential scan per head.
//
// With p = 1 the moment state of a head is only 64 x 64 floats (+ two 64-vectors): it fits the
// accumulator registers of a single wavefront.  So a wave owns a head, walks its tokens in tiles
// of 32, and keeps the running state in registers from the first token to the last: no state
// snapshot ever goes to memory, every input element is read once per layout it is used in, and
// there is no LDS staging and no barrier (LDS only carries two tiny vectors across lanes).
// Per tile and kernel: 192 v_mfma_f32_32x32x2f32 =
//   32 (score tile, contraction over channels) + 32 (intra-tile product with the masked
//   weights, which sit in accumulator registers and are fed back as the A operand)
//   + 64 (own rows x running state, the state's accumulator registers being the B operand)
//   + 64 (state update).
// bf16 inputs take the same path with eight of those instructions at a time as one
// v_mfma_f32_32x32x16_bf16 (24 per tile; kPackedMma below) and half the memory traffic.
//
// Operand layouts (lane l: i = l % 32, hh = l / 32; trow(t, hh) = row of accumulator register t):
//   channel-major X^ch[c][t] = X[tile row trow(t, hh)][chan(c, i)], c = 0, 1: the lane's two channels
//   token-major   X^tok[e]   = X[tile row i][channel of e], 32 of the row's 64 channels per lane half
// A state tile (rc, cc) holds State[chan(rc, m)][chan(cc, n')] at accumulator (row m, column n'),
// and the token-major element tok_of(t, rc) is the channel chan(rc, trow(t, hh)) of the state row
// that register t of the lane holds in tile row-class rc: a token-major operand and the state's
// registers contract against each other with no data movement.  (The k index of an MFMA and the
// order of output rows / columns may be permuted freely as long as both operands, respectively
// the final store, agree.)  Two channel maps, chosen so that every load is one full instruction:
//   fp32: chan(c, i) = 32 c + i (4-byte loads, a half-wave reads 128 contiguous bytes; 32-bit
//         destinations keep the loop-carried operand registers free of pairing constraints);
//         token-major loads are 16 bytes at channel 32 rc + 8 g + 4 hh -> elements rc*16 + 4 g + u
//   bf16: chan(c, i) = 2 i + c (one 4-byte load gives both); token-major loads are 16 bytes =
//         8 channels at 16 g + 8 hh -> elements 8 g + e
//
// Every tile is a full 32-row tile (the sequence has at least 32 tokens): when the length is
// not a multiple of 32, the last tile of a scan is moved back so that it ends at the sequence's
// end (a forward scan's last tile is rows [n-32, n); a reverse scan runs its tiles down from the
// end and its last one is rows [0, 32)).  The rows it shares with the tile before it are already
// in the state and already written; they are masked out of the weights and the stores (and a
// scan's last tile never joins the state).  So all loads are unclamped, with one per-lane offset
// and immediates, and the hot loop has a single straight path.
//
// Order of work in a loop iteration (tile m): fold tile m-1 into the state (its channel-major
// operands are still in registers) -> load tile m's channel-major operands into those registers
// -> score tile and own rows x state with the token-major operands -> load tile m+1's
// token-major operands into those registers -> weights -> intra-tile product -> store.  Every
// load is thus issued right after the last use of the registers it replaces and at least a
// third of an iteration before its first use, and only the token-major loads are still in flight
// at the loop's back edge (where the compiler waits for whatever is outstanding).  The state
// update of the last tile is never needed.  Per-row and per-head factors are applied to the
// accumulators, not to the operands: the weights are kept divided by a1' (resp. by 1/den_i) so
// that the state product and the intra-tile product share one accumulator (hence a1 != 0).
#pragma once
#include "fm_common.h"

namespace lin {

constexpr int D = 64;

// The next tile's loads are issued at fixed points of the current tile's work, far ahead of
// their use; without a fence the scheduler sinks them to the end of the loop body (shorter live
// ranges), where their latency is fully exposed.  Nothing may be moved across FM_PIN().
#define FM_PIN() __builtin_amdgcn_sched_barrier(0)

// Channel maps (see above).
template <class T>
struct Map;
template <>
struct Map<float> {
  static constexpr bool PAIR = false;
  static constexpr bool CLOSED_R = true;
  __device__ static constexpr int chan(int c, int i) { return 32 * c + i; }
  __device__ static constexpr int tok_of(int t, int rc) { return rc * 16 + t; }
};
template <>
struct Map<bf16_t> {
  static constexpr bool PAIR = true;
  static constexpr bool CLOSED_R = false;   // (see linear_dq_kernel)
  __device__ static constexpr int chan(int c, int i) { return 2 * i + c; }
  __device__ static constexpr int tok_of(int t, int rc) { return (t >> 2) * 8 + 2 * (t & 3) + rc; }
};

// Tile operands are addressed as (uniform pointer to the tile's first row) + (per-lane element
// offset, the same for every tile) so that the loads take a scalar base and an immediate.
template <class T>
struct Lane {
  int l, i, hh;
  int tok;   // token-major: row i, first channel of the lane half
  int ch;    // channel-major: row 4 hh, channel chan(0, i)
  __device__ __forceinline__ Lane() {
    l = threadIdx.x; i = l & 31; hh = l >> 5;
    tok = i * D + (Map<T>::PAIR ? 8 : 4) * hh;
    ch = 4 * hh * D + Map<T>::chan(0, i);
  }
};

__device__ __forceinline__ void load_tok(const float* hp, int base, const Lane<float>& L, float (&x)[32]) {
  const float* tp = hp + (int64_t)base * D;
#pragma unroll
  for (int rc = 0; rc < 2; ++rc)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 a = *reinterpret_cast<const float4*>(tp + (L.tok + 32 * rc + 8 * g));
      float* y = &x[rc * 16 + 4 * g];
      y[0] = a.x; y[1] = a.y; y[2] = a.z; y[3] = a.w;
    }
}
__device__ __forceinline__ void load_tok(const bf16_t* hp, int base, const Lane<bf16_t>& L, float (&x)[32]) {
  const bf16_t* tp = hp + (int64_t)base * D;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const uint4 u = *reinterpret_cast<const uint4*>(tp + (L.tok + 16 * g));
    float* y = &x[8 * g];
    y[0] = bf_lo(u.x); y[1] = bf_hi(u.x); y[2] = bf_lo(u.y); y[3] = bf_hi(u.y);
    y[4] = bf_lo(u.z); y[5] = bf_hi(u.z); y[6] = bf_lo(u.w); y[7] = bf_hi(u.w);
  }
}
__device__ __forceinline__ void load_ch(const float* hp, int base, const Lane<float>& L, float (&x)[2][16]) {
  const float* tp = hp + (int64_t)base * D;
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    x[0][t] = tp[L.ch + (8 * (t >> 2) + (t & 3)) * D];
    x[1][t] = tp[L.ch + (8 * (t >> 2) + (t & 3)) * D + 32];
  }
}
__device__ __forceinline__ void load_ch(const bf16_t* hp, int base, const Lane<bf16_t>& L, float (&x)[2][16]) {
  const bf16_t* tp = hp + (int64_t)base * D;
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    const uint32_t u = *reinterpret_cast<const uint32_t*>(tp + (L.ch + (8 * (t >> 2) + (t & 3)) * D));
    x[0][t] = bf_lo(u);
    x[1][t] = bf_hi(u);
  }
}

// A channel-major operand whose conversion is put off until ready(): with bf16 tensors the 16
// loaded dwords stay as they are (half the registers of the 32 floats, and nothing consumes them
// while they travel); with fp32 tensors the loads are the floats.
template <class T>
struct ChOperand;
template <>
struct ChOperand<float> {
  float x[2][16] = {};
  __device__ __forceinline__ void load(const float* hp, int base, const Lane<float>& L) { load_ch(hp, base, L, x); }
  __device__ __forceinline__ void ready() {}
};
template <>
struct ChOperand<bf16_t> {
  float x[2][16] = {};
  uint32_t raw[16] = {};
  __device__ __forceinline__ void load(const bf16_t* hp, int base, const Lane<bf16_t>& L) {
    const bf16_t* tp = hp + (int64_t)base * D;
#pragma unroll
    for (int t = 0; t < 16; ++t)
      raw[t] = *reinterpret_cast<const uint32_t*>(tp + (L.ch + (8 * (t >> 2) + (t & 3)) * D));
  }
  __device__ __forceinline__ void ready() {
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      x[0][t] = bf_lo(raw[t]);
      x[1][t] = bf_hi(raw[t]);
    }
  }
};

// x[c][t] -> row trow(t, hh) of the tile, columns chan(c, i), for the tile rows in [lo, hi)
// (ALIGNED, bf16 only: the row pitch keeps the lane's channel pair 4-byte aligned)
template <bool ALIGNED>
__device__ __forceinline__ void store_row(float* rp, const Lane<float>& L, float a, float b) {
  rp[L.i] = a;
  rp[32 + L.i] = b;
}
template <bool ALIGNED>
__device__ __forceinline__ void store_row(bf16_t* rp, const Lane<bf16_t>& L, float a, float b) {
  if constexpr (ALIGNED) {
    *reinterpret_cast<uint32_t*>(rp + 2 * L.i) = pack_bf2(a, b);
  } else {
    rp[2 * L.i] = from_f32<bf16_t>(a);
    rp[2 * L.i + 1] = from_f32<bf16_t>(b);
  }
}
template <bool ALIGNED, class T>
__device__ __forceinline__ void store_tile(T* hp, int ld, int base, int lo, int hi, const Lane<T>& L,
                                           const float (&x)[2][16]) {
  T* tp = hp + (int64_t)base * ld;
  if (lo == 0 && hi == 32) {
#pragma unroll
    for (int t = 0; t < 16; ++t) store_row<ALIGNED>(tp + trow(t, L.hh) * ld, L, x[0][t], x[1][t]);
  } else {
#pragma unroll
    for (int t = 0; t < 16; ++t)
      if (trow(t, L.hh) >= lo && trow(t, L.hh) < hi) store_row<ALIGNED>(tp + trow(t, L.hh) * ld, L, x[0][t], x[1][t]);
  }
}

__device__ __forceinline__ float half_swap_add(float x) { return x + __shfl_xor(x, 32, 64); }
__device__ __forceinline__ float rcp(float x) { return __builtin_amdgcn_rcpf(x); }  // 1 ulp

// A 64-vector over channels, held as (chan(0, i), chan(1, i)) by the lanes of either half, goes
// through LDS to be dotted with a token-major operand: returns the lane half's part of x . vec.
template <class T>
__device__ __forceinline__ void vec_put(float* lds64, const Lane<T>& L, float v0, float v1) {
  if (L.l < 32) {
    lds64[Map<T>::chan(0, L.i)] = v0;
    lds64[Map<T>::chan(1, L.i)] = v1;
  }
}
template <class T>
__device__ __forceinline__ float vec_dot(const float* lds64, const Lane<T>& L, const float (&x)[32]) {
  float s = 0.f;
  if constexpr (Map<T>::PAIR) {
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      const float4 u = *reinterpret_cast<const float4*>(&lds64[16 * (g >> 1) + 8 * L.hh + 4 * (g & 1)]);
      s += x[4 * g] * u.x + x[4 * g + 1] * u.y + x[4 * g + 2] * u.z + x[4 * g + 3] * u.w;
    }
  } else {
#pragma unroll
    for (int g = 0; g < 8; ++g) {   // g = rc * 4 + (group of four rows)
      const float4 u = *reinterpret_cast<const float4*>(&lds64[32 * (g >> 2) + 8 * (g & 3) + 4 * L.hh]);
      s += x[4 * g] * u.x + x[4 * g + 1] * u.y + x[4 * g + 2] * u.z + x[4 * g + 3] * u.w;
    }
  }
  return s;
}

// ---- the matrix phases of a tile (all kernels of this file share them) ----------------------

// Score tile P (rows = rows of `a`, columns = rows of `b`, contraction over the 64 channels) and
// own rows x running state, O[own row][chan(cc, n)] = sum_ch own[ch] State[ch][chan(cc, n)] (the
// state's accumulator registers are the B operand).  The three accumulation chains are
// independent and issued interleaved.
// With bf16 tensors the contractions run on v_mfma_f32_32x32x16_bf16: eight of the per-lane operand values
// that the fp32 path feeds to eight v_mfma_f32_32x32x2f32 make one instruction (the k index of a contraction
// may be permuted freely as long as both operands agree, so any eight pairs will do).  Operands that come
// from the tensors are bf16 values already (the conversion back is exact); weights and the running state,
// which live in fp32 accumulator registers, are rounded to bf16 on their way into an operand, as everywhere
// on the bf16 paths.
template <class T>
constexpr bool kPackedMma = false;
template <>
constexpr bool kPackedMma<bf16_t> = true;

__device__ __forceinline__ bf8v pk8(float a, float b, float c, float d, float e, float f, float g, float h) {
  return __builtin_bit_cast(bf8v, fm_u4{pack_bf2(a, b), pack_bf2(c, d), pack_bf2(e, f), pack_bf2(g, h)});
}
__device__ __forceinline__ bf8v pk8(const float* x) { return pk8(x[0], x[1], x[2], x[3], x[4], x[5], x[6], x[7]); }
// registers 8 F .. 8 F + 7 of an accumulator tile
template <int F>
__device__ __forceinline__ bf8v pk8(const f16v& a) {
  return pk8(a[8 * F], a[8 * F + 1], a[8 * F + 2], a[8 * F + 3], a[8 * F + 4], a[8 * F + 5], a[8 * F + 6], a[8 * F + 7]);
}
// the own-row elements that meet registers 8 F .. 8 F + 7 of a state tile of row class rc
template <class T, int F, int RC>
__device__ __forceinline__ bf8v pk8_own(const float (&own)[32]) {
  return pk8(own[Map<T>::tok_of(8 * F, RC)], own[Map<T>::tok_of(8 * F + 1, RC)], own[Map<T>::tok_of(8 * F + 2, RC)],
             own[Map<T>::tok_of(8 * F + 3, RC)], own[Map<T>::tok_of(8 * F + 4, RC)], own[Map<T>::tok_of(8 * F + 5, RC)],
             own[Map<T>::tok_of(8 * F + 6, RC)], own[Map<T>::tok_of(8 * F + 7, RC)]);
}

// own rows x state, O[own row][chan(cc, n)] (+)= sum_ch own[ch] State[ch][chan(cc, n)]: the state's accumulator
// registers are the B operand
template <class T>
__device__ __forceinline__ void own_times_state(const float (&own)[32], const f16v (&S)[2][2], f16v (&O)[2]) {
  if constexpr (kPackedMma<T>) {
    const bf8v a00 = pk8_own<T, 0, 0>(own), a10 = pk8_own<T, 1, 0>(own), a01 = pk8_own<T, 0, 1>(own), a11 = pk8_own<T, 1, 1>(own);
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      O[cc] = FM_MFMA_BF16(a00, pk8<0>(S[0][cc]), O[cc]);
      O[cc] = FM_MFMA_BF16(a10, pk8<1>(S[0][cc]), O[cc]);
      O[cc] = FM_MFMA_BF16(a01, pk8<0>(S[1][cc]), O[cc]);
      O[cc] = FM_MFMA_BF16(a11, pk8<1>(S[1][cc]), O[cc]);
    }
  } else {
#pragma unroll
    for (int t = 0; t < 16; ++t)
#pragma unroll
      for (int rc = 0; rc < 2; ++rc) {
        O[0] = FM_MFMA(own[Map<T>::tok_of(t, rc)], S[rc][0][t], O[0]);
        O[1] = FM_MFMA(own[Map<T>::tok_of(t, rc)], S[rc][1][t], O[1]);
      }
  }
}

// Score tile P (rows = rows of `a`, columns = rows of `b`, contraction over the 64 channels) and
// own rows x running state.  The three accumulation chains are independent and issued interleaved.
template <class T>
__device__ __forceinline__ void score_and_state(const float (&a)[32], const float (&b)[32],
                                                const float (&own)[32], const f16v (&S)[2][2], f16v& P,
                                                f16v (&O)[2]) {
#pragma unroll
  for (int t = 0; t < 16; ++t) P[t] = 0.f, O[0][t] = 0.f, O[1][t] = 0.f;
  if constexpr (kPackedMma<T>) {
#pragma unroll
    for (int m = 0; m < 4; ++m) P = FM_MFMA_BF16(pk8(a + 8 * m), pk8(b + 8 * m), P);
    own_times_state<T>(own, S, O);
  } else {
#pragma unroll
    for (int t = 0; t < 16; ++t)
#pragma unroll
      for (int rc = 0; rc < 2; ++rc) {
        P = FM_MFMA(a[2 * t + rc], b[2 * t + rc], P);
        O[0] = FM_MFMA(own[Map<T>::tok_of(t, rc)], S[rc][0][t], O[0]);
        O[1] = FM_MFMA(own[Map<T>::tok_of(t, rc)], S[rc][1][t], O[1]);
      }
  }
}

// State[chan(rc, m)][chan(cc, n)] += sum over the tile's rows of ua[row][chan(rc, m)] * ub[row][chan(cc, n)]
template <class T>
__device__ __forceinline__ void state_update(f16v (&S)[2][2], const float (&ua)[2][16], const float (&ub)[2][16]) {
  if constexpr (kPackedMma<T>) {
#pragma unroll
    for (int f = 0; f < 2; ++f) {
      const bf8v a0 = pk8(ua[0] + 8 * f), a1 = pk8(ua[1] + 8 * f), b0 = pk8(ub[0] + 8 * f), b1 = pk8(ub[1] + 8 * f);
      S[0][0] = FM_MFMA_BF16(a0, b0, S[0][0]);
      S[0][1] = FM_MFMA_BF16(a0, b1, S[0][1]);
      S[1][0] = FM_MFMA_BF16(a1, b0, S[1][0]);
      S[1][1] = FM_MFMA_BF16(a1, b1, S[1][1]);
    }
  } else {
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      S[0][0] = FM_MFMA(ua[0][t], ub[0][t], S[0][0]);
      S[0][1] = FM_MFMA(ua[0][t], ub[1][t], S[0][1]);
      S[1][0] = FM_MFMA(ua[1][t], ub[0][t], S[1][0]);
      S[1][1] = FM_MFMA(ua[1][t], ub[1][t], S[1][1]);
    }
  }
}

// O[own row][chan(cc, n)] += sum over streamed rows of W[streamed][own] * ub[streamed][chan(cc, n)];
// the weights are fed from their accumulator registers as the A operand
template <class T>
__device__ __forceinline__ void weight_product(const f16v& W, const float (&ub)[2][16], f16v (&O)[2]) {
  if constexpr (kPackedMma<T>) {
    const bf8v w0 = pk8<0>(W), w1 = pk8<1>(W);
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      O[cc] = FM_MFMA_BF16(w0, pk8(ub[cc]), O[cc]);
      O[cc] = FM_MFMA_BF16(w1, pk8(ub[cc] + 8), O[cc]);
    }
  } else {
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      O[0] = FM_MFMA(W[t], ub[0][t], O[0]);
      O[1] = FM_MFMA(W[t], ub[1][t], O[1]);
    }
  }
}

// x[t] = v[trow(t, hh)] for a value v held per lane (lane i of either half = tile row i)
template <class T>
__device__ __forceinline__ void rows_from_lanes(float v, float* lds32, const Lane<T>& L, float (&x)[16]) {
  if (L.l < 32) lds32[L.l] = v;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const float4 u = *reinterpret_cast<const float4*>(&lds32[8 * g + 4 * L.hh]);
    x[4 * g] = u.x; x[4 * g + 1] = u.y; x[4 * g + 2] = u.z; x[4 * g + 3] = u.w;
  }
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
  return x;
}

__device__ __forceinline__ void zero_state(f16v (&S)[2][2]) {
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int t = 0; t < 16; ++t) S[a][b][t] = 0.f;
}

// per-lane sums over the tile's rows of a channel-major operand: s[c] = sum_rows x[row][chan(c, i)]
__device__ __forceinline__ void column_sums(const float (&x)[2][16], float (&s)[2]) {
  float a = 0.f, b = 0.f;
#pragma unroll
  for (int t = 0; t < 16; ++t) a += x[0][t], b += x[1][t];
  s[0] = half_swap_add(a);
  s[1] = half_swap_add(b);
}

// Tiles of a forward scan: tile tt covers rows [fbase, fbase + 32), fbase = min(32 tt, n - 32);
// its first 32 tt - fbase rows were already part of tile tt - 1.
__device__ __forceinline__ int fbase(int tt, int n) { return 32 * tt < n - 32 ? 32 * tt : n - 32; }
// Tiles of a reverse scan: tile tt covers rows [rbase, rbase + 32), rbase = max(n - 32 (tt + 1), 0);
// only its first n - 32 tt - rbase rows are new.
__device__ __forceinline__ int rbase(int tt, int n) { return n - 32 * (tt + 1) > 0 ? n - 32 * (tt + 1) : 0; }

// ---------------------------------------------------------------------------------------
// Forward: o_i = [a0 sum_{j<=i} v_j + a1' sum_{j<=i} (q_i.k_j) v_j] / [a0 (i+1) + a1' q_i . sum_{j<=i} k_j]
// with a1' = a1 * qscale * kscale (the normaliser folded into the coefficient; the state is built
// from the raw keys).  State: S1[a][c] = sum k_j[a] v_j[c], s1[a] = sum k_j[a], s0[c] = sum v_j[c].
// The weights are kept as f(s)/a1' = a0/a1' + q_i.k_j, so one accumulator takes q_i S1 and the
// intra-tile product.  grid = heads, block = one wave; n >= 32, a1 != 0.
// ---------------------------------------------------------------------------------------
template <class T, bool ALIGNED>
__global__ __launch_bounds__(64) void linear_fwd_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                        const T* __restrict__ v,
                                                        const float* __restrict__ qscale,
                                                        const float* __restrict__ kscale, T* __restrict__ o,
                                                        int64_t ldo, float* __restrict__ den,
                                                        int64_t den_stride, int n, float a0, float a1) {
  __shared__ __attribute__((aligned(16))) float s1l[D];
  __shared__ __attribute__((aligned(16))) float denl[32];
  const Lane<T> L;
  const int head = blockIdx.x;
  const T* qh = q + (int64_t)head * n * D;
  const T* kh = k + (int64_t)head * n * D;
  const T* vh = v + (int64_t)head * n * D;
  T* oh = o + (int64_t)head * n * ldo;
  float* dh = den + (int64_t)head * n * den_stride;
  const float a1s = a1 * qscale[head] * kscale[head];
  const float a0r = a0 / a1s;

  f16v S1[2][2];
  zero_state(S1);
  float s0[2] = {0.f, 0.f}, s1[2] = {0.f, 0.f};
  float qt[32], kt[32];
  ChOperand<T> kc, vc;   // (tile "-1" is empty)
  load_tok(kh, 0, L, kt);
  load_tok(qh, 0, L, qt);

  const int ntiles = (n + 31) >> 5;
  for (int tt = 0; tt < ntiles; ++tt) {
    const int base = fbase(tt, n), skip = 32 * tt - base;
    // (after the last tile the "next" one is this one again, unused: one straight path)
    const int nb = tt + 1 < ntiles ? fbase(tt + 1, n) : base;

    // the previous tile joins the state
    kc.ready();
    state_update<T>(S1, kc.x, vc.x);
    {
      float ks[2], vs[2];
      column_sums(kc.x, ks);
      column_sums(vc.x, vs);
      s1[0] += ks[0]; s1[1] += ks[1];
      s0[0] += vs[0]; s0[1] += vs[1];
      vec_put<T>(s1l, L, s1[0], s1[1]);
    }
    FM_PIN();
    kc.load(kh, base, L);
    vc.load(vh, base, L);
    FM_PIN();

    // transposed score tile (rows = keys of the tile, columns = queries); own rows x state
    f16v P, O[2];
    score_and_state<T>(kt, qt, qt, S1, P, O);
    // q_i . s1 (the lane's 32 channels, then the other half's)
    const float qs = half_swap_add(vec_dot<T>(s1l, L, qt));
    FM_PIN();
    load_tok(kh, nb, L, kt);
    load_tok(qh, nb, L, qt);
    FM_PIN();

    // weights f(s)/a1' of the visible keys and their sum
    float dsum = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int r = trow(t, L.hh);
      const float w = (r <= L.i && r >= skip) ? a0r + P[t] : 0.f;
      P[t] = w;
      dsum += w;
    }
    // query base + i sees the 32 tt keys of the state and the tile's visible ones
    const float den_i = a1s * (half_swap_add(dsum) + qs) + a0 * (float)(32 * tt);

    // intra-tile part: weights x values
    vc.ready();
    weight_product<T>(P, vc.x, O);

    // denominators move from "lane = token" to the row order of the output registers
    if (L.l < 32 && L.l >= skip) dh[(int64_t)(base + L.l) * den_stride] = den_i;
    float inv[16], x[2][16];
    rows_from_lanes(rcp(den_i), denl, L, inv);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) x[c][t] = (a1s * O[c][t] + a0 * s0[c]) * inv[t];
    store_tile<ALIGNED, T>(oh, (int)ldo, base, skip, 32, L, x);
  }
}

// ---------------------------------------------------------------------------------------
// Backward.  g_i = go_i / den_i, c_i = g_i . o_i (cvec), a1' as above.  Gradients with respect to
// the raw inputs (the normaliser's factor folded in).
//
// dq_i = a1' [ sum_{j<=i} (g_i.v_j - c_i) k_j ]:  forward scan, state T[c][a] = sum v_j[c] k_j[a],
//        s1[a] = sum k_j[a];  dq_i = a1' [ g_i T - c_i s1 + intra-tile part ].  The weights are kept
// multiplied by den_i, go_i.v_j - c_i den_i, so that one accumulator takes go_i T and the
// intra-tile product; 1/den_i scales its rows at the end.
// When NORM, rpart[head] = sum_i dq_hat_i . q_hat_i for the normalisation chain rule (the same
// number serves k: sum_j dk_hat_j . k_hat_j = sum_ij W_ij s_ij as well).  With f linear it has
// a closed form that needs no q: a1 sum_j s_ij = den_i - a0 (i+1) and a1 sum_j s_ij g_i.v_j =
// c_i den_i - a0 g_i . V_i, V_i = sum_{j<=i} v_j, give  sum_ij W_ij s_ij = a0 sum_i [c_i (i+1) - g_i . V_i].
// That rests on o_i = num_i / den_i holding to working precision, so it is used for fp32 only;
// with bf16 tensors (o rounded to 8 bits) the partial is formed directly as sum_i dq_i . q_i.
// PREP: c_i is not read from cvec but formed from the forward output (rows of pitch D) and
// written to cvec for the dk kernel, which saves the separate pass over grad and o.
// ---------------------------------------------------------------------------------------
template <class T, bool NORM, bool PREP>
__global__ __launch_bounds__(64) void linear_dq_kernel(const T* __restrict__ go, const float* __restrict__ den,
                                                       int64_t den_stride, float* __restrict__ cvec,
                                                       const T* __restrict__ o, const T* __restrict__ q,
                                                       const T* __restrict__ k,
                                                       const T* __restrict__ v,
                                                       const float* __restrict__ qscale,
                                                       const float* __restrict__ kscale, T* __restrict__ dq,
                                                       float* __restrict__ rpart, int n, float a0, float a1) {
  __shared__ __attribute__((aligned(16))) float cl[32];
  __shared__ __attribute__((aligned(16))) float dl[32];
  __shared__ __attribute__((aligned(16))) float s0l[D];
  const Lane<T> L;
  const int head = blockIdx.x;
  const T* gh = go + (int64_t)head * n * D;
  const T* kh = k + (int64_t)head * n * D;
  const T* vh = v + (int64_t)head * n * D;
  const float* dh = den + (int64_t)head * n * den_stride;
  float* ch = cvec + (int64_t)head * n;
  const T* fh = PREP ? o + (int64_t)head * n * D : nullptr;   // forward output, rows of pitch D
  T* oh = dq + (int64_t)head * n * D;
  const float a1s = a1 * qscale[head] * kscale[head];
  constexpr bool CLOSED = NORM && Map<T>::CLOSED_R, DIRECT = NORM && !Map<T>::CLOSED_R;
  const T* qh = q + (int64_t)head * n * D;

  f16v S[2][2];
  zero_state(S);
  float s1[2] = {0.f, 0.f}, s0[2] = {0.f, 0.f}, rs = 0.f;
  float gt[32], vt[32], vc[2][16] = {}, kc[2][16] = {};   // (tile "-1" is empty)
  float qc[2][16], ot[32];
  load_tok(vh, 0, L, vt);
  load_tok(gh, 0, L, gt);
  if (PREP) load_tok(fh, 0, L, ot);
  float den_l = dh[(int64_t)L.i * den_stride], c_l = PREP ? 0.f : ch[L.i];

  const int ntiles = (n + 31) >> 5;
  for (int tt = 0; tt < ntiles; ++tt) {
    const int base = fbase(tt, n), skip = 32 * tt - base;
    const int nb = tt + 1 < ntiles ? fbase(tt + 1, n) : base;   // next tile (see linear_fwd_kernel)
    const float den_cur = den_l, inv_l = rcp(den_l);
    float c_cur = c_l;
    if (PREP) {   // c_i = (go_i . o_i) / den_i, formed here and left behind for the dk kernel
      float d = 0.f;
#pragma unroll
      for (int e = 0; e < 32; ++e) d += gt[e] * ot[e];
      c_cur = half_swap_add(d) * inv_l;
      if (L.l < 32 && L.i >= skip) ch[base + L.i] = c_cur;
    }

    // the previous tile joins the state
    state_update<T>(S, vc, kc);
    {
      float ks[2];
      column_sums(kc, ks);
      s1[0] += ks[0]; s1[1] += ks[1];
      if (CLOSED) {
        float vs[2];
        column_sums(vc, vs);
        s0[0] += vs[0]; s0[1] += vs[1];
        vec_put<T>(s0l, L, s0[0], s0[1]);
      }
    }
    FM_PIN();
    load_ch(vh, base, L, vc);
    load_ch(kh, base, L, kc);
    if (DIRECT) load_ch(qh, base, L, qc);
    FM_PIN();

    // rows = keys, columns = queries: go_i . v_j; own rows (go) x state
    f16v W, O[2];
    score_and_state<T>(vt, gt, gt, S, W, O);
    float gv = 0.f;
    if (CLOSED) gv = half_swap_add(vec_dot<T>(s0l, L, gt));   // go_i . (sum of the state's v_j)
    FM_PIN();
    load_tok(vh, nb, L, vt);
    load_tok(gh, nb, L, gt);
    if (PREP) load_tok(fh, nb, L, ot);
    den_l = dh[(int64_t)(nb + L.i) * den_stride];
    if (!PREP) c_l = ch[nb + L.i];
    FM_PIN();
    {
      const float cd = c_cur * den_cur;
      float psum = 0.f;
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const int r = trow(t, L.hh);
        const bool vis = r <= L.i && r >= skip;
        psum += vis ? W[t] : 0.f;
        W[t] = vis ? W[t] - cd : 0.f;
      }
      if (CLOSED) {
        const float ri = c_cur * (float)(base + L.i + 1) - inv_l * (half_swap_add(psum) + gv);
        rs += (L.l < 32 && L.i >= skip) ? ri : 0.f;
      }
    }
    float cT[16], inv[16];
    rows_from_lanes(c_cur, cl, L, cT);
    rows_from_lanes(inv_l, dl, L, inv);

    weight_product<T>(W, kc, O);

    float x[2][16];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) x[c][t] = a1s * (inv[t] * O[c][t] - cT[t] * s1[c]);
    store_tile<true, T>(oh, D, base, skip, 32, L, x);
    if (DIRECT) {
#pragma unroll
      for (int t = 0; t < 16; ++t)
        rs += trow(t, L.hh) >= skip ? x[0][t] * qc[0][t] + x[1][t] * qc[1][t] : 0.f;
    }
  }
  if (NORM) {
    rs = wave_sum(rs);
    if (L.l == 0) rpart[head] = CLOSED ? a0 * rs : rs;
  }
}

// ---------------------------------------------------------------------------------------
// dv_j = sum_{i>=j} f(s_ij) g_i:  reverse scan, state R[a][c] = sum q_i[a] g_i[c], r0[c] = sum g_i[c];
//        dv_j = a0 r0 + a1' [ k_j R + intra-tile part with the weights f(s)/a1' ].  Rows of a
// moved-back tile that are already in the state enter with g = 0.
// ---------------------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(64) void linear_dv_kernel(const T* __restrict__ go, const float* __restrict__ den,
                                                       int64_t den_stride, const T* __restrict__ q,
                                                       const T* __restrict__ k,
                                                       const float* __restrict__ qscale,
                                                       const float* __restrict__ kscale, T* __restrict__ dv,
                                                       int n, float a0, float a1) {
  __shared__ __attribute__((aligned(16))) float dl[32];
  const Lane<T> L;
  const int head = blockIdx.x;
  const T* gh = go + (int64_t)head * n * D;
  const T* qh = q + (int64_t)head * n * D;
  const T* kh = k + (int64_t)head * n * D;
  const float* dh = den + (int64_t)head * n * den_stride;
  T* oh = dv + (int64_t)head * n * D;
  const float a1s = a1 * qscale[head] * kscale[head];
  const float a0r = a0 / a1s;

  f16v S[2][2];
  zero_state(S);
  float r0[2] = {0.f, 0.f};

  const int ntiles = (n + 31) >> 5;
  float qt[32], kt[32], qc[2][16] = {}, gc[2][16] = {};   // (tile "-1" is empty)
  load_tok(qh, n - 32, L, qt);
  load_tok(kh, n - 32, L, kt);
  float den_l = dh[(int64_t)(n - 32 + L.i) * den_stride];

  for (int tt = 0; tt < ntiles; ++tt) {
    const int base = rbase(tt, n), hi = n - 32 * tt - base;      // tile rows [0, hi) are new
    const int nb = tt + 1 < ntiles ? rbase(tt + 1, n) : base;    // next tile (see linear_fwd_kernel)
    const float inv_l = L.i < hi ? rcp(den_l) : 0.f;

    // the previous tile (its g rows already divided by den) joins the state
    state_update<T>(S, qc, gc);
    {
      float gs[2];
      column_sums(gc, gs);
      r0[0] += gs[0]; r0[1] += gs[1];
    }
    FM_PIN();
    load_ch(qh, base, L, qc);
    load_ch(gh, base, L, gc);
    FM_PIN();

    // rows = queries, columns = keys; own rows (k) x state
    f16v P, O[2];
    score_and_state<T>(qt, kt, kt, S, P, O);
    FM_PIN();
    load_tok(qh, nb, L, qt);
    load_tok(kh, nb, L, kt);
    den_l = dh[(int64_t)(nb + L.i) * den_stride];
    FM_PIN();
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int r = trow(t, L.hh);
      P[t] = (r >= L.i && r < hi) ? a0r + P[t] : 0.f;
    }
    float inv[16];
    rows_from_lanes(inv_l, dl, L, inv);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) gc[c][t] *= inv[t];

    weight_product<T>(P, gc, O);

    float x[2][16];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) x[c][t] = a1s * O[c][t] + a0 * r0[c];
    store_tile<true, T>(oh, D, base, 0, hi, L, x);
  }
}

// ---------------------------------------------------------------------------------------
// dk_j = a1' [ sum_{i>=j} (g_i.v_j - c_i) q_i ]:  reverse scan, state Rt[c][a] = sum g_i[c] q_i[a],
//        r1[a] = sum c_i q_i[a];  dk_j = a1' [ v_j Rt - r1 + intra-tile part ].
// ---------------------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(64) void linear_dk_kernel(const T* __restrict__ go, const float* __restrict__ den,
                                                       int64_t den_stride, const float* __restrict__ cvec,
                                                       const T* __restrict__ q, const T* __restrict__ v,
                                                       const float* __restrict__ qscale,
                                                       const float* __restrict__ kscale, T* __restrict__ dk,
                                                       int n, float a1) {
  __shared__ __attribute__((aligned(16))) float dl[32];
  __shared__ __attribute__((aligned(16))) float cl[32];
  const Lane<T> L;
  const int head = blockIdx.x;
  const T* gh = go + (int64_t)head * n * D;
  const T* qh = q + (int64_t)head * n * D;
  const T* vh = v + (int64_t)head * n * D;
  const float* dh = den + (int64_t)head * n * den_stride;
  const float* ch = cvec + (int64_t)head * n;
  T* oh = dk + (int64_t)head * n * D;
  const float a1s = a1 * qscale[head] * kscale[head];

  f16v S[2][2];
  zero_state(S);
  float r1[2] = {0.f, 0.f}, r1next[2] = {0.f, 0.f};

  const int ntiles = (n + 31) >> 5;
  float gt[32], vt[32], gc[2][16] = {}, qc[2][16] = {};   // (tile "-1" is empty)
  load_tok(gh, n - 32, L, gt);
  load_tok(vh, n - 32, L, vt);
  float den_l = dh[(int64_t)(n - 32 + L.i) * den_stride], c_l = ch[n - 32 + L.i];

  for (int tt = 0; tt < ntiles; ++tt) {
    const int base = rbase(tt, n), hi = n - 32 * tt - base;      // tile rows [0, hi) are new
    const int nb = tt + 1 < ntiles ? rbase(tt + 1, n) : base;    // next tile (see linear_fwd_kernel)
    const bool fresh = L.i < hi;
    const float inv_l = fresh ? rcp(den_l) : 0.f;
    const float c_cur = fresh ? c_l : 0.f;
    float inv[16], cT[16];
    rows_from_lanes(inv_l, dl, L, inv);
    rows_from_lanes(c_cur, cl, L, cT);

    // the previous tile (its g rows already divided by den) joins the state
    state_update<T>(S, gc, qc);
    r1[0] += r1next[0];
    r1[1] += r1next[1];
    FM_PIN();
    load_ch(gh, base, L, gc);
    load_ch(qh, base, L, qc);
    FM_PIN();

    // rows = queries, columns = keys: go_i . v_j; own rows (v) x state
    f16v W, O[2];
    score_and_state<T>(gt, vt, vt, S, W, O);
    FM_PIN();
    load_tok(gh, nb, L, gt);
    load_tok(vh, nb, L, vt);
    den_l = dh[(int64_t)(nb + L.i) * den_stride];
    c_l = ch[nb + L.i];
    FM_PIN();
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int r = trow(t, L.hh);
      W[t] = (r >= L.i && r < hi) ? W[t] * inv[t] - cT[t] : 0.f;
    }
    {
      float ca = 0.f, cb = 0.f;
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        gc[0][t] *= inv[t];
        gc[1][t] *= inv[t];
        ca += cT[t] * qc[0][t];
        cb += cT[t] * qc[1][t];
      }
      r1next[0] = half_swap_add(ca);
      r1next[1] = half_swap_add(cb);
    }

    weight_product<T>(W, qc, O);

    float x[2][16];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) x[c][t] = a1s * (O[c][t] - r1[c]);
    store_tile<true, T>(oh, D, base, 0, hi, L, x);
  }
}

// =======================================================================================
// Unmasked p = 1 at head dimension 64: every row sees the state of the whole sequence, so after
// the state is built (the chunked build kernel: token-split partial states, summed) each output
// is one pass over the rows: out[row] = f(own[row] x State).  A wave loads the 64 x 64 state once
// into the registers that serve as the B operand (see the layouts above) and walks ROWS_PER_WAVE
// rows in tiles of 32, 64 matrix instructions per tile.  State layout in memory: rows of LD = 68
// floats, row a < 64 = [State[a][0..63], vec1[a], pad], row 64 = [vec0[0..63], count, pad]
// (the moment state of the chunked kernels for p = 1), built from the SCALED x of its first
// factor:  S  = sum k^_j (x) [v_j, 1]      (k^ = kscale k;  vec1 = sum k^, vec0 = sum v)
//          R  = sum q^_i (x) [g_i, c_i]    (q^ = qscale q;  vec1 = sum c_i q^_i, vec0 = sum g_i)
//   FWD: own = q, S:    o_i  = (a0 vec0 + a1 qs q_i S) / den_i,  den_i = a0 n + a1 qs q_i . vec1
//   DV:  own = k, R:    dv_j = a0 vec0 + a1 ks k_j R
//   DQ:  own = grad, S^T: dq_i = a1 qs (go_i S^T / den_i - c_i vec1)
//   DK:  own = v, R^T:  dk_j = a1 ks (v_j R^T - vec1)
// (qs, ks: the per-head normaliser factors; gradients are with respect to the raw inputs).
// DQ with NORM also leaves the normalisation partial of its rows in rpart[head * gridDim.x + block]
// (closed form a0 sum_i [c_i n - g_i . vec0] for fp32, sum_i dq_i . q_i for bf16; see linear_dq_kernel).
// grid = (ceil(n / ROWS_PER_WAVE), heads), block = one wave; n >= 32.
// =======================================================================================
constexpr int ROWS_PER_WAVE = 256;
constexpr int SLD = 68;   // row pitch of the state in memory
enum { ROWPASS_FWD = 0, ROWPASS_DV = 1, ROWPASS_DQ = 2, ROWPASS_DK = 3 };

template <class T>
__device__ __forceinline__ void state_only(const float (&own)[32], const f16v (&S)[2][2], f16v (&O)[2]) {
#pragma unroll
  for (int t = 0; t < 16; ++t) O[0][t] = 0.f, O[1][t] = 0.f;
  own_times_state<T>(own, S, O);
}

template <class T, int MODE, bool NORM, bool ALIGNED>
__global__ __launch_bounds__(64, 2) void linear_rowpass_kernel(const T* __restrict__ own, const float* __restrict__ state,
                                                            int64_t state_stride, const float* __restrict__ xscale,
                                                            const float* __restrict__ den_in, int64_t den_stride,
                                                            const float* __restrict__ cvec, const T* __restrict__ xraw,
                                                            T* __restrict__ out, int64_t ldo, float* __restrict__ den_out,
                                                            float* __restrict__ rpart, int n, float a0, float a1) {
  __shared__ __attribute__((aligned(16))) float vl[D];
  __shared__ __attribute__((aligned(16))) float al[32];
  __shared__ __attribute__((aligned(16))) float bl[32];
  constexpr bool FWD = MODE == ROWPASS_FWD, DQ = MODE == ROWPASS_DQ, DK = MODE == ROWPASS_DK;
  constexpr bool TRANSPOSED = DQ || DK;
  constexpr bool CLOSED = DQ && NORM && Map<T>::CLOSED_R, DIRECT = DQ && NORM && !Map<T>::CLOSED_R;
  const Lane<T> L;
  const int head = blockIdx.y, r0 = blockIdx.x * ROWS_PER_WAVE;
  const int r1 = r0 + ROWS_PER_WAVE < n ? r0 + ROWS_PER_WAVE : n;
  const T* xh = own + (int64_t)head * n * D;
  const float* st = state + (int64_t)head * state_stride;
  T* oh = out + (int64_t)head * n * ldo;
  const float fac = a1 * xscale[head];

  // the state as B operand: register t of tile (rc, cc) = M[chan(rc, trow)][chan(cc, i)], M = State or its transpose
  f16v S[2][2];
#pragma unroll
  for (int rc = 0; rc < 2; ++rc)
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const int row = Map<T>::chan(rc, trow(t, L.hh)), col = Map<T>::chan(cc, L.i);
        S[rc][cc][t] = TRANSPOSED ? st[col * SLD + row] : st[row * SLD + col];
      }
  // the vector that enters per output column (vec0 for FWD / DV, vec1 for DQ / DK)
  float vcol[2];
#pragma unroll
  for (int cc = 0; cc < 2; ++cc) {
    const int col = Map<T>::chan(cc, L.i);
    vcol[cc] = TRANSPOSED ? st[col * SLD + D] : st[D * SLD + col];
  }
  // the vector that is dotted with the own rows: vec1 for the denominators, vec0 for the closed-form partial
  if (FWD) vec_put<T>(vl, L, st[Map<T>::chan(0, L.i) * SLD + D], st[Map<T>::chan(1, L.i) * SLD + D]);
  if (CLOSED) vec_put<T>(vl, L, st[D * SLD + Map<T>::chan(0, L.i)], st[D * SLD + Map<T>::chan(1, L.i)]);
  const float* dh = den_in ? den_in + (int64_t)head * n * den_stride : nullptr;
  const float* ch = cvec ? cvec + (int64_t)head * n : nullptr;
  float* dout = den_out ? den_out + (int64_t)head * n * den_stride : nullptr;
  const T* qh = DIRECT ? xraw + (int64_t)head * n * D : nullptr;

  // tiles of this wave's rows: tile tt covers [base, base + 32), base = min(r0 + 32 tt, n - 32); only a
  // sequence's very last tile can be moved back, its first `skip` rows belong to the tile before
  const int ntiles = (r1 - r0 + 31) >> 5;
  auto tile_base = [&](int tt) { return r0 + 32 * tt < n - 32 ? r0 + 32 * tt : n - 32; };
  float xt[32], qc[2][16];
  load_tok(xh, tile_base(0), L, xt);
  float den_l = DQ ? dh[(int64_t)(tile_base(0) + L.i) * den_stride] : 0.f;
  float c_l = DQ ? ch[tile_base(0) + L.i] : 0.f;
  float rs = 0.f;
  for (int tt = 0; tt < ntiles; ++tt) {
    const int base = tile_base(tt), skip = r0 + 32 * tt - base;
    const int nb = tt + 1 < ntiles ? tile_base(tt + 1) : base;
    if (DIRECT) load_ch(qh, base, L, qc);
    f16v O[2];
    state_only<T>(xt, S, O);
    float dot = 0.f;
    if (FWD || CLOSED) dot = half_swap_add(vec_dot<T>(vl, L, xt));
    const float den_cur = den_l, c_cur = c_l;
    FM_PIN();
    load_tok(xh, nb, L, xt);
    if (DQ) {
      den_l = dh[(int64_t)(nb + L.i) * den_stride];
      c_l = ch[nb + L.i];
    }
    FM_PIN();

    float x[2][16];
    if (FWD) {
      const float den_i = a0 * (float)n + fac * dot;
      if (L.l < 32 && L.i >= skip) dout[(int64_t)(base + L.i) * den_stride] = den_i;
      float inv[16];
      rows_from_lanes(rcp(den_i), al, L, inv);
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 16; ++t) x[c][t] = (fac * O[c][t] + a0 * vcol[c]) * inv[t];
    } else if (DQ) {
      const float inv_l = rcp(den_cur);
      float inv[16], cT[16];
      rows_from_lanes(inv_l, al, L, inv);
      rows_from_lanes(c_cur, bl, L, cT);
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 16; ++t) x[c][t] = fac * (inv[t] * O[c][t] - cT[t] * vcol[c]);
      if (CLOSED) rs += (L.l < 32 && L.i >= skip) ? c_cur * (float)n - inv_l * dot : 0.f;
      if (DIRECT) {
#pragma unroll
        for (int t = 0; t < 16; ++t)
          rs += trow(t, L.hh) >= skip ? x[0][t] * qc[0][t] + x[1][t] * qc[1][t] : 0.f;
      }
    } else if (DK) {
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 16; ++t) x[c][t] = fac * (O[c][t] - vcol[c]);
    } else {
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 16; ++t) x[c][t] = fac * O[c][t] + a0 * vcol[c];
    }
    store_tile<ALIGNED, T>(oh, (int)ldo, base, skip, 32, L, x);
  }
  if (DQ && NORM) {
    rs = wave_sum(rs);
    if (L.l == 0) rpart[(int64_t)head * gridDim.x + blockIdx.x] = CLOSED ? a0 * rs : rs;
  }
}

#undef FM_PIN

}  // namespace lin
