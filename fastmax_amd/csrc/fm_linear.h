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
// bf16 inputs take the same path (fp32 matrix instruction, half the memory traffic).
//
// Operand layouts (lane l: i = l % 32, hh = l / 32; trow(t, hh) = row of accumulator register t):
//   token-major   X^tok[g*8 + e]  = X[tile row i][16 g + 8 hh + e]      (8 contiguous channels x 4)
//   channel-major X^ch[c][t]      = X[tile row trow(t, hh)][2 i + c]    (2 contiguous channels x 16)
// A state tile (rc, cc) holds State[2 m + rc][2 n' + cc] at accumulator (row m, column n'), so
// register t of a lane holds state row 2 trow(t, hh) + rc = 16 (t/4) + 8 hh + 2 (t%4) + rc, which
// is exactly the channel of token-major element (t/4)*8 + 2 (t%4) + rc: a token-major operand and
// the state's registers contract against each other with no data movement.  (The k index of an
// MFMA and the order of output rows / columns may be permuted freely as long as both operands,
// respectively the final store, agree.)
//
// Rows past the end of the sequence are read from the last valid row (clamped) and kept out of
// the results by the masks / zeroed factors named at each use.
#pragma once
#include "fm_common.h"

namespace lin {

constexpr int D = 64;

// The next tile's loads are issued at fixed points of the current tile's work, far ahead of
// their use; without a fence the scheduler sinks them to the end of the loop body (shorter live
// ranges), where their latency is fully exposed.  Nothing may be moved across FM_PIN().
#define FM_PIN() __builtin_amdgcn_sched_barrier(0)

template <class T>
__device__ __forceinline__ void ld8(const T* p, float* x);
template <>
__device__ __forceinline__ void ld8<float>(const float* p, float* x) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
  x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
}
template <>
__device__ __forceinline__ void ld8<bf16_t>(const bf16_t* p, float* x) {
  const uint4 u = *reinterpret_cast<const uint4*>(p);
  x[0] = bf_lo(u.x); x[1] = bf_hi(u.x); x[2] = bf_lo(u.y); x[3] = bf_hi(u.y);
  x[4] = bf_lo(u.z); x[5] = bf_hi(u.z); x[6] = bf_lo(u.w); x[7] = bf_hi(u.w);
}
__device__ __forceinline__ void ld2(const float* p, float& a, float& b) {
  const float2 t = *reinterpret_cast<const float2*>(p);
  a = t.x; b = t.y;
}
__device__ __forceinline__ void ld2(const bf16_t* p, float& a, float& b) {
  const uint32_t u = *reinterpret_cast<const uint32_t*>(p);
  a = bf_lo(u); b = bf_hi(u);
}
// (aligned: the pair may be written as one 8- or 4-byte store)
template <bool ALIGNED>
__device__ __forceinline__ void st2(float* p, float a, float b) {
  if constexpr (ALIGNED) {
    *reinterpret_cast<float2*>(p) = make_float2(a, b);
  } else {
    p[0] = a; p[1] = b;
  }
}
template <bool ALIGNED>
__device__ __forceinline__ void st2(bf16_t* p, float a, float b) {
  if constexpr (ALIGNED) {
    *reinterpret_cast<uint32_t*>(p) = pack_bf2(a, b);
  } else {
    p[0] = from_f32<bf16_t>(a); p[1] = from_f32<bf16_t>(b);
  }
}

// Tile operands are addressed as (uniform pointer to the tile's first row) + (per-lane element
// offset, constant from tile to tile) so that the loads take a scalar base and an immediate.
// token-major operand of the tile starting at row `base` of one head (hp)
template <class T>
__device__ __forceinline__ void load_tok(const T* hp, int base, int n, int i, int hh, float (&x)[32]) {
  const T* tp = hp + (int64_t)base * D;
  const int last = n - 1 - base;                       // last valid row of the tile
  const int off = (i < last ? i : last) * D + 8 * hh;  // (rows past the end read the last valid row)
#pragma unroll
  for (int g = 0; g < 4; ++g) ld8<T>(tp + (off + 16 * g), &x[8 * g]);
}

// channel-major operand; roff[t] = element offset of the lane's pair in row trow(t, hh) of a tile
// (row_offsets: rows past the tile's last valid row read that row).  The offsets live in
// registers and are only recomputed for a ragged last tile, so the hot loop has one load path.
__device__ __forceinline__ void row_offsets(int last, int i, int hh, int (&roff)[16]) {
#pragma unroll
  for (int t = 0; t < 16; ++t) roff[t] = (trow(t, hh) < last ? trow(t, hh) : last) * D + 2 * i;
}
template <class T>
__device__ __forceinline__ void load_ch(const T* hp, int base, const int (&roff)[16], float (&x)[2][16]) {
  const T* tp = hp + (int64_t)base * D;
#pragma unroll
  for (int t = 0; t < 16; ++t) ld2(tp + roff[t], x[0][t], x[1][t]);
}

// one value per tile row, lane i of either half holding row i (clamped like the operands)
__device__ __forceinline__ float load_lane(const float* hp, int64_t stride, int base, int n, int i) {
  const int last = n - 1 - base;
  return hp[(int64_t)(base + (i < last ? i : last)) * stride];
}

__device__ __forceinline__ float half_swap_add(float x) { return x + __shfl_xor(x, 32, 64); }
__device__ __forceinline__ float rcp(float x) { return __builtin_amdgcn_rcpf(x); }  // 1 ulp

// token-major element that contracts against register t of state tile row-class rc
__device__ __forceinline__ constexpr int tok_of(int t, int rc) { return (t >> 2) * 8 + 2 * (t & 3) + rc; }

// ---- the matrix phases of a tile (all kernels of this file share them) ----------------------

// Score tile P (rows = rows of `a`, columns = rows of `b`, contraction over the 64 channels) and
// own rows x running state, O[own row][2n+cc] = sum_ch own[ch] State[ch][2n+cc] (the state's
// accumulator registers are the B operand).  The three accumulation chains are independent and
// issued interleaved.
__device__ __forceinline__ void score_and_state(const float (&a)[32], const float (&b)[32],
                                                const float (&own)[32], const f16v (&S)[2][2], f16v& P,
                                                f16v (&O)[2]) {
#pragma unroll
  for (int t = 0; t < 16; ++t) P[t] = 0.f, O[0][t] = 0.f, O[1][t] = 0.f;
#pragma unroll
  for (int t = 0; t < 16; ++t)
#pragma unroll
    for (int rc = 0; rc < 2; ++rc) {
      P = FM_MFMA(a[2 * t + rc], b[2 * t + rc], P);
      O[0] = FM_MFMA(own[tok_of(t, rc)], S[rc][0][t], O[0]);
      O[1] = FM_MFMA(own[tok_of(t, rc)], S[rc][1][t], O[1]);
    }
}

// State[2m+rc][2n+cc] += sum over the tile's rows of ua[row][2m+rc] * ub[row][2n+cc]
__device__ __forceinline__ void state_update(f16v (&S)[2][2], const float (&ua)[2][16], const float (&ub)[2][16]) {
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    S[0][0] = FM_MFMA(ua[0][t], ub[0][t], S[0][0]);
    S[0][1] = FM_MFMA(ua[0][t], ub[1][t], S[0][1]);
    S[1][0] = FM_MFMA(ua[1][t], ub[0][t], S[1][0]);
    S[1][1] = FM_MFMA(ua[1][t], ub[1][t], S[1][1]);
  }
}

// O[own row][2n+cc] += sum over streamed rows of W[streamed][own] * ub[streamed][2n+cc]; the
// weights are fed from their accumulator registers as the A operand
__device__ __forceinline__ void weight_product(const f16v& W, const float (&ub)[2][16], f16v (&O)[2]) {
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    O[0] = FM_MFMA(W[t], ub[0][t], O[0]);
    O[1] = FM_MFMA(W[t], ub[1][t], O[1]);
  }
}

// x[t] = v[trow(t, hh)] for a value v held per lane (lane i of either half = tile row i)
__device__ __forceinline__ void rows_from_lanes(float v, float* lds32, int l, int hh, float (&x)[16]) {
  if (l < 32) lds32[l] = v;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const float4 u = *reinterpret_cast<const float4*>(&lds32[8 * g + 4 * hh]);
    x[4 * g] = u.x; x[4 * g + 1] = u.y; x[4 * g + 2] = u.z; x[4 * g + 3] = u.w;
  }
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
  return x;
}

// x[c][t] -> row trow(t, hh) of the tile, columns 2i + c (rows past the end are skipped)
template <bool ALIGNED, class T>
__device__ __forceinline__ void store_tile(T* hp, int ld, int base, int n, int i, int hh, const float (&x)[2][16]) {
  T* tp = hp + (int64_t)base * ld;
  if (base + 32 <= n) {
#pragma unroll
    for (int t = 0; t < 16; ++t) st2<ALIGNED>(tp + (trow(t, hh) * ld + 2 * i), x[0][t], x[1][t]);
  } else {
#pragma unroll
    for (int t = 0; t < 16; ++t)
      if (base + trow(t, hh) < n) st2<ALIGNED>(tp + (trow(t, hh) * ld + 2 * i), x[0][t], x[1][t]);
  }
}

// sum over the tile's valid rows of x . y (both in the output layout)
__device__ __forceinline__ float tile_dot(const float (&x)[2][16], const float (&y)[2][16], int base, int n, int hh) {
  float s = 0.f;
  if (base + 32 <= n) {
#pragma unroll
    for (int t = 0; t < 16; ++t) s += x[0][t] * y[0][t] + x[1][t] * y[1][t];
  } else {
#pragma unroll
    for (int t = 0; t < 16; ++t)
      if (base + trow(t, hh) < n) s += x[0][t] * y[0][t] + x[1][t] * y[1][t];
  }
  return s;
}

__device__ __forceinline__ void zero_state(f16v (&S)[2][2]) {
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int t = 0; t < 16; ++t) S[a][b][t] = 0.f;
}

// ---------------------------------------------------------------------------------------
// Forward: o_i = [a0 sum_{j<=i} v_j + a1' sum_{j<=i} (q_i.k_j) v_j] / [a0 (i+1) + a1' q_i . sum_{j<=i} k_j]
// with a1' = a1 * qscale * kscale (the normaliser folded into the coefficient, which is applied
// to the query rows as they are loaded; the state is built from the raw keys).
// State: S1[a][c] = sum k_j[a] v_j[c], s1[a] = sum k_j[a], s0[c] = sum v_j[c].
// grid = heads, block = one wave.
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
  const int head = blockIdx.x, l = threadIdx.x, i = l & 31, hh = l >> 5;
  const T* qh = q + (int64_t)head * n * D;
  const T* kh = k + (int64_t)head * n * D;
  const T* vh = v + (int64_t)head * n * D;
  T* oh = o + (int64_t)head * n * ldo;
  float* dh = den + (int64_t)head * n * den_stride;
  const float a1s = a1 * qscale[head] * kscale[head];

  f16v S1[2][2];
  zero_state(S1);
  float s0[2] = {0.f, 0.f}, s1[2] = {0.f, 0.f};
  if (l < 32) *reinterpret_cast<float2*>(&s1l[2 * l]) = make_float2(0.f, 0.f);

  float qt[32], kt[32], kc[2][16], vc[2][16];
  int roff[16];
  row_offsets(n - 1, i, hh, roff);
  load_tok<T>(kh, 0, n, i, hh, kt);
  load_tok<T>(qh, 0, n, i, hh, qt);
  load_ch<T>(kh, 0, roff, kc);
  load_ch<T>(vh, 0, roff, vc);

  const int ntiles = (n + 31) >> 5;
  for (int tile = 0; tile < ntiles; ++tile) {
    const int base = tile << 5;
    // the next tile is fetched while this one is worked on (after the last tile: this one again,
    // unused, so that the loop has a single straight path); a ragged next tile needs new offsets
    const int nb = tile + 1 < ntiles ? base + 32 : base;
    if (n - 1 - nb < 31) row_offsets(n - 1 - nb, i, hh, roff);
#pragma unroll
    for (int e = 0; e < 32; ++e) qt[e] *= a1s;

    // transposed score tile (rows = keys of the tile, columns = queries); own rows x state
    f16v P, O[2];
    score_and_state(kt, qt, qt, S1, P, O);
    FM_PIN();
    load_tok<T>(kh, nb, n, i, hh, kt);
    FM_PIN();

    // weights f(s) of the visible keys (key <= query; a key past the end is only ever "visible"
    // to queries past the end) and their sum
    float dsum = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const float w = trow(t, hh) <= i ? a0 + P[t] : 0.f;
      P[t] = w;
      dsum += w;
    }
    dsum = half_swap_add(dsum);
    // a1' q_i . s1 (the lane's 32 channels, then the other half's)
    float qs = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 u0 = *reinterpret_cast<const float4*>(&s1l[16 * g + 8 * hh]);
      const float4 u1 = *reinterpret_cast<const float4*>(&s1l[16 * g + 8 * hh + 4]);
      qs += qt[8 * g] * u0.x + qt[8 * g + 1] * u0.y + qt[8 * g + 2] * u0.z + qt[8 * g + 3] * u0.w +
            qt[8 * g + 4] * u1.x + qt[8 * g + 5] * u1.y + qt[8 * g + 6] * u1.z + qt[8 * g + 7] * u1.w;
    }
    const float den_i = dsum + a0 * (float)base + half_swap_add(qs);   // query base + i
    FM_PIN();
    load_tok<T>(qh, nb, n, i, hh, qt);
    FM_PIN();

    // state update (rows past the end only reach a state nobody reads: this is the last tile)
    const float s0a[2] = {a0 * s0[0], a0 * s0[1]};   // order-0 term of this tile's rows
    state_update(S1, kc, vc);
    {
      float ks[2] = {0.f, 0.f}, vs[2] = {0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 16; ++t) ks[c] += kc[c][t], vs[c] += vc[c][t];
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        s1[c] += half_swap_add(ks[c]);
        s0[c] += half_swap_add(vs[c]);
      }
      if (l < 32) *reinterpret_cast<float2*>(&s1l[2 * l]) = make_float2(s1[0], s1[1]);
    }
    FM_PIN();
    load_ch<T>(kh, nb, roff, kc);
    FM_PIN();

    // intra-tile part: weights x values
    weight_product(P, vc, O);
    FM_PIN();
    load_ch<T>(vh, nb, roff, vc);
    FM_PIN();

    // denominators move from "lane = token" to the row order of the output registers
    if (l < 32 && base + l < n) dh[(int64_t)(base + l) * den_stride] = den_i;
    float inv[16];
    rows_from_lanes(rcp(den_i), denl, l, hh, inv);
    float x[2][16];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) x[c][t] = (O[c][t] + s0a[c]) * inv[t];
    store_tile<ALIGNED, T>(oh, (int)ldo, base, n, i, hh, x);
  }
}

// ---------------------------------------------------------------------------------------
// Backward.  g_i = go_i / den_i, c_i = g_i . o_i (cvec), a1' as above.  Gradients with respect to
// the raw inputs (the normaliser's factor folded in), plus, when NORM, rpart[head] =
// sum_rows dx_hat . x_hat for the normalisation chain rule.
//
// dq_i = a1' [ sum_{j<=i} (g_i.v_j - c_i) k_j ]:  forward scan, state T[c][a] = sum v_j[c] k_j[a],
//        s1[a] = sum k_j[a];  dq_i = a1' [ g_i T - c_i s1 + intra-tile part ].
// ---------------------------------------------------------------------------------------
template <class T, bool NORM>
__global__ __launch_bounds__(64) void linear_dq_kernel(const T* __restrict__ go, const float* __restrict__ den,
                                                       int64_t den_stride, const float* __restrict__ cvec,
                                                       const T* __restrict__ q, const T* __restrict__ k,
                                                       const T* __restrict__ v,
                                                       const float* __restrict__ qscale,
                                                       const float* __restrict__ kscale, T* __restrict__ dq,
                                                       float* __restrict__ rpart, int n, float a1) {
  __shared__ __attribute__((aligned(16))) float cl[32];
  const int head = blockIdx.x, l = threadIdx.x, i = l & 31, hh = l >> 5;
  const T* gh = go + (int64_t)head * n * D;
  const T* qh = q + (int64_t)head * n * D;
  const T* kh = k + (int64_t)head * n * D;
  const T* vh = v + (int64_t)head * n * D;
  const float* dh = den + (int64_t)head * n * den_stride;
  const float* ch = cvec + (int64_t)head * n;
  T* oh = dq + (int64_t)head * n * D;
  const float a1s = a1 * qscale[head] * kscale[head];

  f16v S[2][2];
  zero_state(S);
  float s1[2] = {0.f, 0.f}, rs = 0.f;

  float gt[32], vt[32], vc[2][16], kc[2][16], qc[2][16];
  int roff[16];
  row_offsets(n - 1, i, hh, roff);
  load_tok<T>(vh, 0, n, i, hh, vt);
  load_tok<T>(gh, 0, n, i, hh, gt);
  float den_l = load_lane(dh, den_stride, 0, n, i), c_l = load_lane(ch, 1, 0, n, i);
  load_ch<T>(vh, 0, roff, vc);
  load_ch<T>(kh, 0, roff, kc);

  const int ntiles = (n + 31) >> 5;
  for (int tile = 0; tile < ntiles; ++tile) {
    const int base = tile << 5;
    if (NORM) load_ch<T>(qh, base, roff, qc);   // only for the normalisation partial at the end
    const int nb = tile + 1 < ntiles ? base + 32 : base;   // next tile (see linear_fwd_kernel)
    if (n - 1 - nb < 31) row_offsets(n - 1 - nb, i, hh, roff);
    {
      const float inv = rcp(den_l);
#pragma unroll
      for (int e = 0; e < 32; ++e) gt[e] *= inv;
    }
    const float c_cur = c_l;
    // rows = keys, columns = queries: g_i . v_j; own rows x state
    f16v W, O[2];
    score_and_state(vt, gt, gt, S, W, O);
    FM_PIN();
    load_tok<T>(vh, nb, n, i, hh, vt);
    load_tok<T>(gh, nb, n, i, hh, gt);
    den_l = load_lane(dh, den_stride, nb, n, i);
    c_l = load_lane(ch, 1, nb, n, i);
    FM_PIN();
#pragma unroll
    for (int t = 0; t < 16; ++t) W[t] = trow(t, hh) <= i ? W[t] - c_cur : 0.f;
    float cT[16];
    rows_from_lanes(c_cur, cl, l, hh, cT);

    const float s1old[2] = {s1[0], s1[1]};
    state_update(S, vc, kc);
    {
      float ks[2] = {0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 16; ++t) ks[c] += kc[c][t];
      s1[0] += half_swap_add(ks[0]);
      s1[1] += half_swap_add(ks[1]);
    }
    FM_PIN();
    load_ch<T>(vh, nb, roff, vc);
    FM_PIN();

    weight_product(W, kc, O);
    FM_PIN();
    load_ch<T>(kh, nb, roff, kc);
    FM_PIN();

    float x[2][16];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) x[c][t] = a1s * (O[c][t] - cT[t] * s1old[c]);
    store_tile<true, T>(oh, D, base, n, i, hh, x);
    if (NORM) rs += tile_dot(x, qc, base, n, hh);
  }
  if (NORM) {
    rs = wave_sum(rs);
    if (l == 0) rpart[head] = rs;
  }
}

// ---------------------------------------------------------------------------------------
// dv_j = sum_{i>=j} f(s_ij) g_i:  reverse scan, state R[a][c] = sum q_i[a] g_i[c], r0[c] = sum g_i[c];
//        dv_j = a0 r0 + a1' k_j R + intra-tile part.  Rows past the end enter with g = 0.
// ---------------------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(64) void linear_dv_kernel(const T* __restrict__ go, const float* __restrict__ den,
                                                       int64_t den_stride, const T* __restrict__ q,
                                                       const T* __restrict__ k,
                                                       const float* __restrict__ qscale,
                                                       const float* __restrict__ kscale, T* __restrict__ dv,
                                                       int n, float a0, float a1) {
  __shared__ __attribute__((aligned(16))) float dl[32];
  const int head = blockIdx.x, l = threadIdx.x, i = l & 31, hh = l >> 5;
  const T* gh = go + (int64_t)head * n * D;
  const T* qh = q + (int64_t)head * n * D;
  const T* kh = k + (int64_t)head * n * D;
  const float* dh = den + (int64_t)head * n * den_stride;
  T* oh = dv + (int64_t)head * n * D;
  const float a1s = a1 * qscale[head] * kscale[head];

  f16v S[2][2];
  zero_state(S);
  float r0[2] = {0.f, 0.f};

  const int ntiles = (n + 31) >> 5;
  const int b0 = (ntiles - 1) << 5;
  float qt[32], kt[32], qc[2][16], gc[2][16];
  int roff[16];
  row_offsets(n - 1 - b0, i, hh, roff);   // the last tile may be ragged; it is the first one here
  load_tok<T>(qh, b0, n, i, hh, qt);
  load_tok<T>(kh, b0, n, i, hh, kt);
  float den_l = load_lane(dh, den_stride, b0, n, i);
  load_ch<T>(qh, b0, roff, qc);
  load_ch<T>(gh, b0, roff, gc);
  if (ntiles > 1) row_offsets(31, i, hh, roff);   // every other tile is full

  for (int tile = ntiles - 1; tile >= 0; --tile) {
    const int base = tile << 5;
    const int nb = tile > 0 ? base - 32 : base;   // next tile (see linear_fwd_kernel)
#pragma unroll
    for (int e = 0; e < 32; ++e) kt[e] *= a1s;
    const float inv_l = base + i < n ? rcp(den_l) : 0.f;
    // rows = queries, columns = keys; own rows x state
    f16v P, O[2];
    score_and_state(qt, kt, kt, S, P, O);
    FM_PIN();
    load_tok<T>(qh, nb, n, i, hh, qt);
    load_tok<T>(kh, nb, n, i, hh, kt);
    den_l = load_lane(dh, den_stride, nb, n, i);
    FM_PIN();
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int r = trow(t, hh);
      P[t] = (r >= i && base + r < n) ? a0 + P[t] : 0.f;
    }
    float inv[16];
    rows_from_lanes(inv_l, dl, l, hh, inv);
    const float r0a[2] = {a0 * r0[0], a0 * r0[1]};
    {
      float gs[2] = {0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 16; ++t) {
          gc[c][t] *= inv[t];
          gs[c] += gc[c][t];
        }
      state_update(S, qc, gc);
      r0[0] += half_swap_add(gs[0]);
      r0[1] += half_swap_add(gs[1]);
    }
    FM_PIN();
    load_ch<T>(qh, nb, roff, qc);
    FM_PIN();

    weight_product(P, gc, O);
    FM_PIN();
    load_ch<T>(gh, nb, roff, gc);
    FM_PIN();

    float x[2][16];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) x[c][t] = O[c][t] + r0a[c];
    store_tile<true, T>(oh, D, base, n, i, hh, x);
  }
}

// ---------------------------------------------------------------------------------------
// dk_j = a1' [ sum_{i>=j} (g_i.v_j - c_i) q_i ]:  reverse scan, state Rt[c][a] = sum g_i[c] q_i[a],
//        r1[a] = sum c_i q_i[a];  dk_j = a1' [ v_j Rt - r1 + intra-tile part ].
// (No normalisation partial here: sum_j dk_hat_j . k_hat_j = sum_ij W_ij s_ij = sum_i dq_hat_i . q_hat_i,
// the dq kernel's.)
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
  const int head = blockIdx.x, l = threadIdx.x, i = l & 31, hh = l >> 5;
  const T* gh = go + (int64_t)head * n * D;
  const T* qh = q + (int64_t)head * n * D;
  const T* vh = v + (int64_t)head * n * D;
  const float* dh = den + (int64_t)head * n * den_stride;
  const float* ch = cvec + (int64_t)head * n;
  T* oh = dk + (int64_t)head * n * D;
  const float a1s = a1 * qscale[head] * kscale[head];

  f16v S[2][2];
  zero_state(S);
  float r1[2] = {0.f, 0.f};

  const int ntiles = (n + 31) >> 5;
  const int b0 = (ntiles - 1) << 5;
  float gt[32], vt[32], gc[2][16], qc[2][16];
  int roff[16];
  row_offsets(n - 1 - b0, i, hh, roff);   // the last tile may be ragged; it is the first one here
  load_tok<T>(gh, b0, n, i, hh, gt);
  load_tok<T>(vh, b0, n, i, hh, vt);
  float den_l = load_lane(dh, den_stride, b0, n, i), c_l = load_lane(ch, 1, b0, n, i);
  load_ch<T>(gh, b0, roff, gc);
  load_ch<T>(qh, b0, roff, qc);
  if (ntiles > 1) row_offsets(31, i, hh, roff);   // every other tile is full

  for (int tile = ntiles - 1; tile >= 0; --tile) {
    const int base = tile << 5;
    const int nb = tile > 0 ? base - 32 : base;   // next tile (see linear_fwd_kernel)
    const bool inside = base + i < n;
    const float inv_l = inside ? rcp(den_l) : 0.f;
    const float c_cur = inside ? c_l : 0.f;
#pragma unroll
    for (int e = 0; e < 32; ++e) gt[e] *= inv_l;

    // rows = queries, columns = keys: g_i . v_j; own rows x state
    f16v W, O[2];
    score_and_state(gt, vt, vt, S, W, O);
    FM_PIN();
    load_tok<T>(gh, nb, n, i, hh, gt);
    load_tok<T>(vh, nb, n, i, hh, vt);
    den_l = load_lane(dh, den_stride, nb, n, i);
    c_l = load_lane(ch, 1, nb, n, i);
    FM_PIN();
    float inv[16], cT[16];
    rows_from_lanes(inv_l, dl, l, hh, inv);
    rows_from_lanes(c_cur, cl, l, hh, cT);
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int r = trow(t, hh);
      W[t] = (r >= i && base + r < n) ? W[t] - cT[t] : 0.f;
    }

    const float r1old[2] = {r1[0], r1[1]};
    {
      float cs[2] = {0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < 16; ++t) {
          gc[c][t] *= inv[t];
          cs[c] += cT[t] * qc[c][t];
        }
      state_update(S, gc, qc);
      r1[0] += half_swap_add(cs[0]);
      r1[1] += half_swap_add(cs[1]);
    }
    FM_PIN();
    load_ch<T>(gh, nb, roff, gc);
    FM_PIN();

    weight_product(W, qc, O);
    FM_PIN();
    load_ch<T>(qh, nb, roff, qc);
    FM_PIN();

    float x[2][16];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int t = 0; t < 16; ++t) x[c][t] = a1s * (O[c][t] - r1old[c]);
    store_tile<true, T>(oh, D, base, n, i, hh, x);
  }
}

#undef FM_PIN

}  // namespace lin
