// Per-head row-norm statistics and the moment-state build (used by both passes; the kernels
// that consume the states are in fm_apply.h and fm_grad.h).
#pragma once
#include <type_traits>

#include "fm_common.h"

// ---------------------------------------------------------------------------------------
// Per-head normaliser: scale[h] = lim / max_i ||x_i||_2 and the row that attains the max
// (first one on ties).  Replaces calc_norms / find_max of the reference
// (fastmax_cuda_forward.cu:223-253) with the PyTorch path's definition (example.py:105-108).
// One block of NT threads per head; a row is shared by d/4 (fp32) or d/8 (bf16) threads, 16 bytes each (any d that is
// a whole number of such pieces).  (NT = 1024 when there are too few
// heads to fill the chip with 256-thread blocks: four times the loads in flight per head.)
// ---------------------------------------------------------------------------------------
// a thread's piece of a row: 16 bytes = 4 fp32 or 8 bf16 elements
template <class T>
struct RowPiece;
template <>
struct RowPiece<float> {
  static constexpr int N = 4;
  __device__ __forceinline__ static float sumsq(const uint4& r) {
    const float x = __uint_as_float(r.x), y = __uint_as_float(r.y), z = __uint_as_float(r.z), w = __uint_as_float(r.w);
    return x * x + y * y + z * z + w * w;
  }
};
template <>
struct RowPiece<bf16_t> {
  static constexpr int N = 8;
  __device__ __forceinline__ static float sumsq(const uint4& t) {
    const float a0 = bf_lo(t.x), a1 = bf_hi(t.x), a2 = bf_lo(t.y), a3 = bf_hi(t.y);
    const float a4 = bf_lo(t.z), a5 = bf_hi(t.z), a6 = bf_lo(t.w), a7 = bf_hi(t.w);
    return (a0 * a0 + a1 * a1 + a2 * a2 + a3 * a3) + (a4 * a4 + a5 * a5 + a6 * a6 + a7 * a7);
  }
};

// One launch serves two tensors (q and k): blocks 0 .. nh1-1 take the heads of x1 (n1 rows each),
// the blocks after them the heads of x2 (n2 rows each); results go to index blockIdx.x.
template <class T, int NT>
__global__ __launch_bounds__(NT) void rowstat_kernel(Rows<const T> x1, int n1, int nh1, Rows<const T> x2, int n2,
                                                     int d, float lim, float* __restrict__ scale_out,
                                                     int* __restrict__ arg_out) {
  __shared__ float sbest[NT];
  __shared__ int sarg[NT];
  constexpr int EPT = RowPiece<T>::N;
  const int tid = threadIdx.x;
  // threads per row: the pieces of a row rounded up to a power of two (the lanes past the row's
  // end add zero), so that a row's threads reduce with shuffles
  const int npc = d / EPT;
  int tpr = 1;
  while (tpr < npc) tpr *= 2;
  const int rpp = NT / tpr;
  const int sub = tid % tpr, rowi = tid / tpr;
  const bool second = (int)blockIdx.x >= nh1;
  const int n = second ? n2 : n1;
  // rows 0 .. n-1 of the tensor itself (lo is not used)
  const HeadRows<const T> xh = second ? x2.head(blockIdx.x - nh1) : x1.head(blockIdx.x);
  const T* base = xh.base;
  const unsigned pitch = xh.pitch;
  // A NaN row norm wins over every number (the maximum of the reference's path propagates NaN,
  // example.py:105-108), so the head's scale becomes NaN and the reported row is always a row
  // of the tensor: first NaN row if there is one, else first row of maximal norm.
  auto better = [](float ss, int idx, float best, int bi) {
    const bool ssnan = ss != ss, bnan = best != best;
    if (ssnan) return !bnan || idx < bi;
    return !bnan && (ss > best || (ss == best && idx < bi));
  };
  float best = -1.f;
  int bi = 0;
  // U row groups per trip, loaded before any of them is reduced (rows past the end are clamped to the
  // last row: a duplicate cannot change the maximum or its first index).  With few heads a block walks
  // its head alone and only what it has in flight hides the memory latency: 16 loads per thread there.
  constexpr int U = NT >= 1024 ? 16 : 8;
  for (int i0 = 0; i0 < n; i0 += U * rpp) {
    uint4 raw[U];
    int idx[U];
    // (unconditional loads of clamped addresses, nothing computed from them yet: a load under a condition, or
    // one whose value is used at once, gets a wait of its own and the trip becomes one memory round trip per group)
    const unsigned piece = (unsigned)((sub < npc ? sub : npc - 1) * EPT);
    const unsigned keep = sub < npc ? 0xffffffffu : 0u;   // (the lanes past the row's end: their piece, a duplicate, becomes zeros)
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * rpp + rowi;
      idx[u] = i < n ? i : n - 1;
      raw[u] = *reinterpret_cast<const uint4*>(base + ((unsigned)idx[u] * pitch + piece));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (tpr != npc) {   // (block-uniform: only head dimensions whose pieces are not a power of two have such lanes)
        raw[u].x &= keep; raw[u].y &= keep; raw[u].z &= keep; raw[u].w &= keep;
      }
      float ss = RowPiece<T>::sumsq(raw[u]);
      for (int off = tpr >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      if (better(ss, idx[u], best, bi)) {
        best = ss;
        bi = idx[u];
      }
    }
  }
  sbest[tid] = best;
  sarg[tid] = bi;
  __syncthreads();
  for (int off = NT / 2; off > 0; off >>= 1) {
    if (tid < off) {
      const float ob = sbest[tid + off];
      const int oi = sarg[tid + off];
      if (better(ob, oi, sbest[tid], sarg[tid])) {
        sbest[tid] = ob;
        sarg[tid] = oi;
      }
    }
    __syncthreads();
  }
  if (tid == 0) {
    scale_out[blockIdx.x] = lim / sqrtf(sbest[0]);
    arg_out[blockIdx.x] = min(max(sarg[0], 0), n - 1);
  }
}

__global__ void fill_scale_kernel(float* scale, int* arg, int count, float value) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) {
    scale[i] = value;
    arg[i] = 0;
  }
}

// x <- x * scale[head]; the reference's in-place apply_norm (fastmax_cuda_forward.cu:255-269)
template <class T>
__global__ void scale_rows_kernel(T* x, const float* __restrict__ scale, int64_t per_head) {
  const int64_t i4 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i4 < per_head) {
    T* p = x + (int64_t)blockIdx.y * per_head + i4;
    float v[4];
    load4(p, v);
    const float s = scale[blockIdx.y];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] *= s;
    store4(p, v);
  }
}

// ---------------------------------------------------------------------------------------
// Moment-state build.
//
//   state[row(f)][c] = sum_j feat_f(x_j) * y_j[c]     c < D
//   state[row(f)][D] = sum_j feat_f(x_j) * e_j        the "extra" column
//
// over a token range, with x_j = X_j * xscale[head], y_j = Y_j / yden_j (when given) and
// e_j = ew_j or 1.  The forward pass uses (X,Y,e) = (k, v, 1); the backward pass also builds
// the mirror-image suffix state with (q, grad_out/den, c).  A block is four waves; each wave
// owns RTW row tiles (32 features x D columns) as MFMA accumulators for the whole walk, the
// features being generated on the fly as products of two LDS reads of the staged X tile.
// gridDim.x feature splits cover all row tiles of a head, gridDim.y = heads.
//
// masked != 0: the walk is a scan over `chunk`-token chunks and a snapshot of the running
//   state is written before each chunk is added (slot c = everything strictly before chunk
//   c, or strictly after it when reverse != 0).  The first chunk in scan order needs no
//   state (it is all zero) and the last one is never added.
// masked == 0: gridDim.z blocks each sum zlen tokens and write slot blockIdx.z; consumers
//   add the slots.
// ---------------------------------------------------------------------------------------
template <int D, class T, int RTW, bool BF>
__global__ __launch_bounds__(256, 2) void build_kernel(
    Rows<const T> X, Rows<const T> Y, const float* __restrict__ xscale, RowScalars yden,
    RowScalars ew, float* __restrict__ state, int n, int chunk, int nslots, int masked, int reverse,
    int p2, int zlen) {
  using G = Geo<D>;
  // tokens per pipeline step (= per barrier).  The p = 2 kernels at D = 64 take 64 tokens, staged as two halves of 32:
  // the step's fixed costs (barrier, staging round trip, step bookkeeping) are paid half as often
  // (bf16 build 7 % faster than with 32-token steps, fp32 1 %); the D = 32 kernels, with five row
  // tiles of accumulators per wave, have no registers for it, and the p = 1 kernels (RTW == 1) keep
  // the smaller tiles for their occupancy.  chunk is a multiple of TS.
  constexpr int TS = (D == 64 && RTW > 1) ? 64 : 32;
  constexpr int TP = TS + 4;    // pitch of the transposed tiles: 16-byte aligned rows, and the
                                // 8 lanes of a 128-bit LDS access phase fall in distinct banks
  constexpr int LD = G::LD;
  // RTW == 1 is the p = 1 configuration: a head has only D/32 row tiles, so for D = 64 the four
  // waves split the 2 x 2 (row tile, column tile) grid instead of leaving two waves without work
  constexpr bool CSPLIT = RTW == 1 && G::CB == 2;
  constexpr int CB = CSPLIT ? 1 : G::CB;  // column tiles per wave
  // X and Y tiles are staged TRANSPOSED ([channel][token]) so that the four tokens a lane feeds
  // into four consecutive MFMAs come from one 128-bit LDS read.  Row D of the X tile is 1 for
  // real tokens and 0 for padding: order-1 features are x[a] * 1.
  __shared__ __attribute__((aligned(16))) float Kt[2][(D + 1) * TP];
  // BF: the value tile is kept as bf16 (pitch TPB 16-bit elements: 8-byte aligned rows, the 16
  // lanes of a 64-bit access phase in distinct banks) and every four fp32 MFMAs become one
  // bf16 MFMA on features rounded after the fp32 product
  constexpr int TPB = TS + 4;
  __shared__ __attribute__((aligned(16))) float Vt[BF ? 1 : 2][BF ? 4 : D * TP];
  __shared__ __attribute__((aligned(16))) uint16_t Vtb[BF ? 2 : 1][BF ? D * TPB : 4];
  __shared__ __attribute__((aligned(16))) float El[2][TS];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  // logical block = (feature split g fastest, then head, then token split z)
  const int lid = xcd_logical_id(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z),
                                 gridDim.x * gridDim.y * gridDim.z);
  const int g = lid % gridDim.x, head = (lid / gridDim.x) % gridDim.y, zsplit = lid / (gridDim.x * gridDim.y);
  const int rows2 = G::rows2(p2);
  const int rt2 = p2 ? G::NS * G::AB : 0, rt_total = rt2 + G::AB;
  // slot pitch: causal bf16 scans write packed states only, which are about half the fp32 size
  const int64_t SS = (BF && masked) ? PackedGeo<D>::slot_floats(p2) : G::state_floats(p2);

  // per owned row tile: LDS offsets of the lane's own channel row and of its rotated partner
  int ownoff[RTW], rotoff[RTW], rowbase[RTW];
  int nx = 0;  // row tiles this wave really owns (wave-uniform)
#pragma unroll
  for (int x = 0; x < RTW; ++x) {
    const int rt = CSPLIT ? g * 2 + (w & 1) : (g * 4 + w) * RTW + x;
    ownoff[x] = rotoff[x] = 4 * hh;
    rowbase[x] = 0;
    if (rt < rt_total) {
      nx = x + 1;
      if (rt < rt2) {
        const int s = rt / G::AB, ab = rt % G::AB;
        ownoff[x] = (ab * 32 + i) * TP + 4 * hh;
        rotoff[x] = ((ab * 32 + i + s) % D) * TP + 4 * hh;
        rowbase[x] = s * D + ab * 32;
      } else {
        const int ab = rt - rt2;
        ownoff[x] = (ab * 32 + i) * TP + 4 * hh;
        rotoff[x] = D * TP + 4 * hh;
        rowbase[x] = rows2 + ab * 32;
      }
    }
  }
  // fp32, D = 64, p = 2: the feature list ends inside the last block of a head and leaves one wave
  // of it without a row tile.  That wave forms the state's extra column for the whole head instead:
  // the extra column of row (s, a) is sum_t e_t x_a x_(a+s) = G[a][(a+s) % D] with the Gram matrix
  // G = sum_t e_t x_t x_t^T (three 32 x 32 tiles by symmetry, 12 matrix instructions per 8 tokens),
  // and that of the order-1 row a is K1[a] = sum_t e_t x_a.  The other waves then spend no VALU
  // work on the extra column (it was four FMAs per row tile and four tokens).
  constexpr bool GT = D == 64 && RTW == 3 && !BF;
  const bool gwave = GT && nx == 0;   // (RTW == 3 is the p = 2 configuration)
  const int cbase = CSPLIT ? w >> 1 : 0;  // first column tile of this wave
  int voff[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) voff[cb] = ((cbase + cb) * 32 + i) * (BF ? TPB : TP) + 4 * hh;

  f16v acc[RTW][CB];
  float dacc[RTW];
#pragma unroll
  for (int x = 0; x < RTW; ++x) {
    dacc[x] = 0.f;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[x][cb][r] = 0.f;
  }
  float s0 = 0.f;  // order-0 sums: threads 0..D-1 of split 0 own a value column, thread D the extra one

  const HeadRows<const T> Xh = X.head(head), Yh = Y.head(head);
  const float* ydh = yden.head(head);
  const float* ewh = ew.head(head);
  const int64_t yden_stride = yden.stride;
  const float xs = xscale[head];
  // positions below lo have no row (query-side tensors behind a key prefix): they read as zero, and
  // a reverse scan stops at the chunk that holds position lo (the chunks below add nothing)
  const int lo = Xh.lo;

  // a step is staged in halves of 32 tokens (one half when TS == 32), so that only one half's
  // rows are in registers at a time
  constexpr int NH = TS / 32;
  std::conditional_t<BF, RawTileBf<D, 32>, RowTile<D, T, 32, true>> kx, vy;
  float ereg = 0.f;

  auto load = [&](int t0, int tend) {
    kx.load(Xh, t0, tend, tid);
    vy.load(Yh, t0, tend, tid, ydh, yden_stride);
    if (tid < 32) {
      const int tok = t0 + tid;
      ereg = (tok < tend && tok >= lo) ? (ewh ? ewh[tok] : 1.0f) : 0.f;
    }
  };
  auto store = [&](int buf, int h, int t0, int tend) {
    kx.store_t(Kt[buf] + 32 * h, TP, xs, tid);
    if constexpr (BF) vy.store_t_bf(Vtb[buf] + 32 * h, TPB, 1.0f, tid, ydh == nullptr);
    else vy.store_t(Vt[buf] + 32 * h, TP, 1.0f, tid);
    if (tid < 32) {
      El[buf][32 * h + tid] = ereg;
      Kt[buf][D * TP + 32 * h + tid] = (t0 + tid < tend && t0 + tid >= lo) ? 1.0f : 0.f;
    }
  };
  // operands of one group of 8 tokens (lane half hh takes tokens 8*grp + 4*hh + u, u = 0..3,
  // as the k index of MFMA u)
  struct GroupOps {
    float4 own[RTW], rot[RTW], vv[BF ? 1 : CB], e4;
    uint2 vb[BF ? CB : 1];
  };
  auto fetch = [&](const float* kb, int buf, const float* eb, int grp, GroupOps& g4) __attribute__((always_inline)) {
    const int go8 = 8 * grp;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
      if constexpr (BF) g4.vb[cb] = *reinterpret_cast<const uint2*>(Vtb[buf] + voff[cb] + go8);
      else g4.vv[cb] = *reinterpret_cast<const float4*>(Vt[buf] + voff[cb] + go8);
    }
    g4.e4 = *reinterpret_cast<const float4*>(eb + go8 + 4 * hh);
#pragma unroll
    for (int x = 0; x < RTW; ++x) {
      g4.own[x] = *reinterpret_cast<const float4*>(kb + ownoff[x] + go8);
      g4.rot[x] = *reinterpret_cast<const float4*>(kb + rotoff[x] + go8);
    }
  };
  auto compute = [&](int buf, int h) __attribute__((always_inline)) {
    const float* kb = Kt[buf];
    const float* eb = El[buf];
    GroupOps cur, nxt;
    // BF: the packed operands of an even group wait for the odd group that follows, and the two
    // go into one k = 16 MFMA
    uint2 ap_even[RTW], vb_even[BF ? CB : 1];
    fetch(kb, buf, eb, 4 * h, cur);
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const int grp = 4 * h + gq;
      if (gq + 1 < 4) fetch(kb, buf, eb, grp + 1, nxt);
      // tiles past the end of the feature list (x >= nx) run on dummy operands and are never stored
#pragma unroll
      for (int x = 0; x < RTW; ++x) {
        const float a0 = cur.own[x].x * cur.rot[x].x, a1 = cur.own[x].y * cur.rot[x].y;
        const float a2 = cur.own[x].z * cur.rot[x].z, a3 = cur.own[x].w * cur.rot[x].w;
        if constexpr (BF) {
          const uint2 ap = pack_bf4u(a0, a1, a2, a3);
          // the extra column sums the features as rounded for the matrix instruction (two 2-term
          // bf16 dot products instead of four fp32 FMAs), so it is consistent with the value columns
          dacc[x] = fm_dot2_bf16(ap.x, pack_bf2(cur.e4.x, cur.e4.y), dacc[x]);
          dacc[x] = fm_dot2_bf16(ap.y, pack_bf2(cur.e4.z, cur.e4.w), dacc[x]);
          if ((gq & 1) == 0) {
            ap_even[x] = ap;
          } else {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
              acc[x][cb] = FM_MFMA_BF16(as_bf8(ap_even[x], ap), as_bf8(vb_even[cb], cur.vb[cb]), acc[x][cb]);
          }
        } else {
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) {
            acc[x][cb] = FM_MFMA(a0, cur.vv[cb].x, acc[x][cb]);
            acc[x][cb] = FM_MFMA(a1, cur.vv[cb].y, acc[x][cb]);
            acc[x][cb] = FM_MFMA(a2, cur.vv[cb].z, acc[x][cb]);
            acc[x][cb] = FM_MFMA(a3, cur.vv[cb].w, acc[x][cb]);
          }
        }
        if constexpr (!BF && !GT) {
          dacc[x] += a0 * cur.e4.x + a1 * cur.e4.y + a2 * cur.e4.z + a3 * cur.e4.w;
        }
      }
      if constexpr (BF) {
        if ((gq & 1) == 0) {
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) vb_even[cb] = cur.vb[cb];
        }
      }
      if (gq + 1 < 4) cur = nxt;
    }
  };
  // the Gram wave's share of a half step: G tiles (0,0), (0,1), (1,1) in acc[0][0], acc[0][1],
  // acc[1][0] (rows = channel a, columns = channel b), K1 of channel blocks 0, 1 in dacc[0], dacc[1]
  auto compute_gram = [&](int buf, int h) __attribute__((always_inline)) {
    if constexpr (GT) {
      const float* kb = Kt[buf];
      const float* eb = El[buf];
      const int r0 = i * TP + 4 * hh, r1 = (32 + i) * TP + 4 * hh;
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const int go8 = 8 * (4 * h + gq);
        const float4 x0 = *reinterpret_cast<const float4*>(kb + r0 + go8);
        const float4 x1 = *reinterpret_cast<const float4*>(kb + r1 + go8);
        const float4 e4 = *reinterpret_cast<const float4*>(eb + go8 + 4 * hh);
        const float4 y0 = make_float4(x0.x * e4.x, x0.y * e4.y, x0.z * e4.z, x0.w * e4.w);
        const float4 y1 = make_float4(x1.x * e4.x, x1.y * e4.y, x1.z * e4.z, x1.w * e4.w);
        acc[0][0] = FM_MFMA(x0.x, y0.x, acc[0][0]);
        acc[0][1] = FM_MFMA(x0.x, y1.x, acc[0][1]);
        acc[1][0] = FM_MFMA(x1.x, y1.x, acc[1][0]);
        acc[0][0] = FM_MFMA(x0.y, y0.y, acc[0][0]);
        acc[0][1] = FM_MFMA(x0.y, y1.y, acc[0][1]);
        acc[1][0] = FM_MFMA(x1.y, y1.y, acc[1][0]);
        acc[0][0] = FM_MFMA(x0.z, y0.z, acc[0][0]);
        acc[0][1] = FM_MFMA(x0.z, y1.z, acc[0][1]);
        acc[1][0] = FM_MFMA(x1.z, y1.z, acc[1][0]);
        acc[0][0] = FM_MFMA(x0.w, y0.w, acc[0][0]);
        acc[0][1] = FM_MFMA(x0.w, y1.w, acc[0][1]);
        acc[1][0] = FM_MFMA(x1.w, y1.w, acc[1][0]);
        dacc[0] += (y0.x + y0.y) + (y0.z + y0.w);
        dacc[1] += (y1.x + y1.y) + (y1.z + y1.w);
      }
    }
  };
  // order-0 sums of the staged step
  auto sum0 = [&](int buf) __attribute__((always_inline)) {
    const float* eb = El[buf];
    if (g == 0 && tid <= D) {
      if (BF && tid < D) {
        const uint16_t* src = Vtb[buf] + tid * TPB;
#pragma unroll
        for (int j = 0; j < TS; j += 4) {
          const uint2 u = *reinterpret_cast<const uint2*>(src + j);
          s0 += (bf_lo(u.x) + bf_hi(u.x)) + (bf_lo(u.y) + bf_hi(u.y));
        }
      } else {
        const float* src = tid < D ? Vt[buf] + tid * TP : eb;
#pragma unroll
        for (int j = 0; j < TS; j += 4) {
          const float4 t4 = *reinterpret_cast<const float4*>(src + j);
          s0 += (t4.x + t4.y) + (t4.z + t4.w);
        }
      }
    }
  };
  // lane part of a snapshot address: row 4*hh (+ 8j + e per register), column i (+ 32*cb)
  const unsigned lane_off = (unsigned)(4 * hh * LD + cbase * 32 + i);
  auto snapshot = [&](int slot, auto gtag) __attribute__((always_inline)) {
    constexpr bool GW = decltype(gtag)::value;   // the Gram wave's own copy of the scan (see below)
    float* st = state + ((int64_t)head * nslots + slot) * SS;  // uniform: scalar base + 32-bit lane offsets
#pragma unroll
    for (int x = 0; x < RTW; ++x) {
      if (x < nx) {
        float* sx = st + (unsigned)(rowbase[x] * LD);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned oj = lane_off + (unsigned)(8 * j * LD);
#pragma unroll
          for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) sx[oj + (unsigned)(e * LD + cb * 32)] = acc[x][cb][4 * j + e];
        }
        if constexpr (!GT) {
          const float ds = dacc[x] + __shfl_xor(dacc[x], 32, 64);
          if (hh == 0 && cbase == 0) sx[(unsigned)(i * LD + D)] = ds;
        }
      }
    }
    if constexpr (GW) {
      {
        // the extra column of the whole head from the Gram tiles: element (a, b) belongs to row
        // (s, a) with s = (b - a) mod D when s <= D/2, else to row (D - s, b); a diagonal tile holds
        // every pair twice (the copies with s > D/2 are dropped), and s = D/2 lists every pair from
        // both sides (rows (D/2, a) and (D/2, b))
        // (the lane's coordinates pass through an empty volatile statement: the 64 store offsets are
        // then formed here, not once before the scan loop, where they would occupy 64 registers)
        int li = i, lh = hh;
        asm volatile("" : "+v"(li), "+v"(lh));
        auto put = [&](const f16v& gacc, int ra, int cb) __attribute__((always_inline)) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int a = ra * 32 + trow(r, lh), b = cb * 32 + li, sft = (b - a) & (D - 1);
            if (sft <= G::H2) {
              st[(unsigned)((sft * D + a) * LD + D)] = gacc[r];
              if (sft == G::H2) st[(unsigned)((sft * D + b) * LD + D)] = gacc[r];
            } else if (ra != cb) {
              st[(unsigned)(((D - sft) * D + b) * LD + D)] = gacc[r];
            }
            if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0);   // (a few stores at a time: register pressure)
          }
        };
        put(acc[0][0], 0, 0);
        put(acc[0][1], 0, 1);
        put(acc[1][0], 1, 1);
        const float k0 = dacc[0] + __shfl_xor(dacc[0], 32, 64), k1 = dacc[1] + __shfl_xor(dacc[1], 32, 64);
        if (lh == 0) {
          st[(unsigned)((rows2 + li) * LD + D)] = k0;
          st[(unsigned)((rows2 + 32 + li) * LD + D)] = k1;
        }
      }
    }
    if (g == 0 && tid <= D) st[(unsigned)((rows2 + D) * LD + tid)] = s0;
  };

  // BF, masked: the snapshot goes out in the packed bf16 form (PackedGeo) with the fp32 order-0 row.
  auto snapshot_packed = [&](int slot) __attribute__((always_inline)) {
    using PG = PackedGeo<D>;
    char* sb = reinterpret_cast<char*>(state + ((int64_t)head * nslots + slot) * SS);  // uniform
    uint16_t* fsec = reinterpret_cast<uint16_t*>(sb);
#pragma unroll
    for (int x = 0; x < RTW; ++x) {
      if (x < nx) {
        const int slab = rowbase[x] / D, arow = rowbase[x] % D;
        const bool dbl = rowbase[x] < rows2 && slab != 0 && slab != G::H2;  // pair weight 2
        const float ds = dacc[x] + __shfl_xor(dacc[x], 32, 64);
        {
          const float wgt = dbl ? 2.0f : 1.0f;
          // accumulator registers 4j..4j+3 are rows 8j + 4hh .. + 3 of the tile: half hh of the
          // 16-byte word of row octet (arow / 8) + j
          uint16_t* fx = fsec + (unsigned)(slab * PG::FSL + (arow >> 3) * PG::NCF * 8);
          const unsigned lo = (unsigned)((cbase * 32 + i) * 8 + 4 * hh);
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
              const f16v& a = acc[x][cb];
              *reinterpret_cast<uint2*>(fx + lo + (unsigned)((j * PG::NCF + cb * 32) * 8)) =
                  make_uint2(pack_bf2(a[4 * j] * wgt, a[4 * j + 1] * wgt), pack_bf2(a[4 * j + 2] * wgt, a[4 * j + 3] * wgt));
            }
          if (hh == 0 && cbase == 0) {   // the extra column, split into hi + lo parts: columns D..D+3 = (hi, hi, lo, lo)
            const float ew = ds * wgt, ehi = bf_lo(pack_bf2(ew, 0.f));
            const uint16_t h16 = (uint16_t)pack_bf2(ehi, 0.f), l16 = (uint16_t)pack_bf2(ew - ehi, 0.f);
            uint16_t* ex = fx + (unsigned)(((i >> 3) * PG::NCF + D) * 8 + (i & 7));
            ex[0] = h16; ex[8] = h16; ex[16] = l16; ex[24] = l16;
          }
        }
      }
    }
    if (g == 0 && tid <= D) reinterpret_cast<float*>(sb + PG::z_off(p2))[tid] = s0;
  };
  auto emit = [&](int slot, auto gtag) __attribute__((always_inline)) {
    if constexpr (BF) {
      if (masked) {
        snapshot_packed(slot);
        return;
      }
    }
    snapshot(slot, gtag);
  };

  // The walk is one software pipeline over all 32-token steps: the loads of step p+1 are issued
  // before the MFMAs of step p and consumed after them; a snapshot is stored right after that,
  // so its stores drain under the next step's MFMAs.
  //   masked, forward : chunks 0 .. nc-2 in order; after chunk c the state goes to slot c+1
  //   masked, reverse : chunks nc-1 .. 1;          after chunk c the state goes to slot c-1
  //   unmasked        : tokens [z*zlen, (z+1)*zlen) ; at the end the state goes to slot z
  const int spc = chunk / TS;  // steps per full chunk
  int nsteps, first_len = 0, tbase = 0, tend = n;
  if (masked) {
    const int nc = (n + chunk - 1) / chunk;
    if (reverse) {
      first_len = (n - (nc - 1) * chunk + TS - 1) / TS;  // the last chunk may be short
      const int cl = lo / chunk;   // (<= nc - 1)
      nsteps = nc > 1 ? first_len + (nc - 1 - (cl > 1 ? cl : 1)) * spc : 0;
    } else {
      nsteps = (nc - 1) * spc;
    }
  } else {
    tbase = zsplit * zlen;
    tend = tbase + zlen < n ? tbase + zlen : n;
    nsteps = tend > tbase ? (tend - tbase + TS - 1) / TS : 0;
  }
  // token base of step p and the slot to write after it (-1: none)
  auto step_tok = [&](int p) {
    if (!masked) return tbase + p * TS;
    if (!reverse) return p * TS;
    const int nc = (n + chunk - 1) / chunk;
    if (p < first_len) return (nc - 1) * chunk + p * TS;
    const int q = p - first_len;
    return (nc - 2 - q / spc) * chunk + (q % spc) * TS;
  };
  auto step_slot = [&](int p) {
    if (!masked) return p + 1 == nsteps ? zsplit : -1;
    if (!reverse) return (p + 1) % spc == 0 ? (p + 1) / spc : -1;
    const int nc = (n + chunk - 1) / chunk;
    if (p < first_len) return p + 1 == first_len ? nc - 2 : -1;
    const int q = p - first_len;
    return (q + 1) % spc == 0 ? nc - 3 - q / spc : -1;
  };

  if constexpr (BF) {
    // bf16: the tiles are requested two steps before they are staged (two sets of registers that
    // take turns; the requests are unconditional, the last ones repeat the last step and are not
    // used), so that a step's global latency and the drain of a snapshot's stores -- which the
    // same in-order counter makes later loads wait for -- are spread over two steps of work.
    using Tile = RawTileBf<D, 32>;
    Tile kxa[NH], vya[NH], kxb[NH], vyb[NH];
    float era[NH], erb[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) era[h] = erb[h] = 0.f;
    auto load_into = [&](Tile (&k_)[NH], Tile (&v_)[NH], float (&e_)[NH], int t0) __attribute__((always_inline)) {
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        k_[h].load(Xh, t0 + 32 * h, tend, tid);
        v_[h].load(Yh, t0 + 32 * h, tend, tid, ydh, yden_stride);
        if (tid < 32) {
          const int tok = t0 + 32 * h + tid;
          e_[h] = (tok < tend && tok >= lo) ? (ewh ? ewh[tok] : 1.0f) : 0.f;
        }
      }
    };
    auto store_from = [&](const Tile (&k_)[NH], const Tile (&v_)[NH], const float (&e_)[NH], int buf, int t0) __attribute__((always_inline)) {
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        k_[h].store_t(Kt[buf] + 32 * h, TP, xs, tid);
        v_[h].store_t_bf(Vtb[buf] + 32 * h, TPB, 1.0f, tid, ydh == nullptr);
        if (tid < 32) {
          const int tok = t0 + 32 * h + tid;
          El[buf][32 * h + tid] = e_[h];
          Kt[buf][D * TP + 32 * h + tid] = (tok < tend && tok >= lo) ? 1.0f : 0.f;
        }
      }
    };
    // AHEAD = steps between a tile's request and its staging: two 32-token steps or one 64-token step
    // (the same time; with one step a single set of registers does)
    constexpr int AHEAD = NH == 1 ? 2 : 1;
    auto step = [&](int p, Tile (&lk)[NH], Tile (&lv)[NH], float (&le)[NH], const Tile (&sk)[NH],
                    const Tile (&sv)[NH], const float (&se)[NH]) __attribute__((always_inline)) {
      __builtin_amdgcn_sched_barrier(0);
      const int pl = p + AHEAD < nsteps ? p + AHEAD : nsteps - 1;
      load_into(lk, lv, le, step_tok(pl));
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        compute(p & 1, h);
        __builtin_amdgcn_sched_barrier(0);   // (keeps the halves apart: register pressure)
      }
      sum0(p & 1);
      if (p + 1 < nsteps) store_from(sk, sv, se, (p + 1) & 1, step_tok(p + 1));
      const int slot = step_slot(p);
      if (slot >= 0) emit(slot, std::false_type{});
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
    };
    if (nsteps > 0) {
      load_into(kxa, vya, era, step_tok(0));
      store_from(kxa, vya, era, 0, step_tok(0));
      if constexpr (AHEAD == 2) load_into(kxb, vyb, erb, step_tok(nsteps > 1 ? 1 : 0));
    }
    __syncthreads();
    if constexpr (AHEAD == 2) {
      for (int p = 0; p < nsteps; p += 2) {
        step(p, kxa, vya, era, kxb, vyb, erb);
        if (p + 1 < nsteps) step(p + 1, kxb, vyb, erb, kxa, vya, era);
      }
    } else {
      // (the set is requested at the start of a step and staged at its end)
      for (int p = 0; p < nsteps; ++p) step(p, kxa, vya, era, kxa, vya, era);
    }
  }
  // The scan itself, in two copies where a head has a Gram wave (GW: that wave's copy; the copies
  // differ in the compute and snapshot calls only, and as separate loops they do not add their
  // register needs).  Every wave of the block stages tiles and meets the barriers alike.
  auto tail = [&](auto gtag) __attribute__((always_inline)) {
    if (!masked && nsteps == 0) emit(zsplit, gtag);  // an empty token split still owns its slot
    if (masked && reverse && nsteps > 0) {
      // chunks below the one that holds position lo see the same suffix state
      for (int slot = lo / chunk - 2; slot >= 0; --slot) emit(slot, gtag);
    }
  };
  auto scan = [&](auto gtag) __attribute__((always_inline)) {
    constexpr bool GW = decltype(gtag)::value;
    if (nsteps > 0) {
  #pragma unroll
      for (int h = 0; h < NH; ++h) {
        load(step_tok(0) + 32 * h, tend);
        store(0, h, step_tok(0) + 32 * h, tend);
      }
    }
    __syncthreads();
    for (int p = 0; p < nsteps; ++p) {
      const bool more = p + 1 < nsteps;
      const int tnext = step_tok(more ? p + 1 : p);
  #pragma unroll 1
      for (int h = 0; h < NH; ++h) {
        if (more) load(tnext + 32 * h, tend);
        if constexpr (GW) compute_gram(p & 1, h);
        else compute(p & 1, h);
        if (h == NH - 1) sum0(p & 1);
        if (more) store((p + 1) & 1, h, tnext + 32 * h, tend);
        if constexpr (NH > 1) __builtin_amdgcn_sched_barrier(0);   // (keeps the halves apart: register pressure)
      }
      // after the staged tile has been consumed: waiting for loads while stores are pending
      // would wait for the stores too (one in-order counter covers both)
      const int slot = step_slot(p);
      if (slot >= 0) emit(slot, gtag);
      __syncthreads();
    }
    tail(gtag);
  };
  if constexpr (BF) {
    tail(std::false_type{});
  } else if constexpr (GT) {
    if (gwave) scan(std::true_type{});
    else scan(std::false_type{});
  } else {
    scan(std::false_type{});
  }
}

// ---------------------------------------------------------------------------------------
// Packs one slab of an fp32 state held in LDS (Sl: the D rows of a shift, or the order-1 rows
// followed by the order-0 row) into the packed bf16 form (PackedGeo) at sb.  256 threads.
// ---------------------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void pack_slab_from_lds(const float* Sl, char* sb, int slab, bool ord1, int p2, int tid) {
  using G = Geo<D>;
  using PG = PackedGeo<D>;
  constexpr int LD = G::LD;
  uint16_t* fsec = reinterpret_cast<uint16_t*>(sb) + slab * PG::FSL;
  const float wgt = (!ord1 && slab != 0 && slab != G::H2) ? 2.0f : 1.0f;
  for (int idx = tid; idx < (D / 4) * (D + 1); idx += 256) {
    const int tg = idx / (D + 1), col = idx % (D + 1);
    const float* f = Sl + 4 * tg * LD + col;
    const float f0 = f[0] * wgt, f1 = f[LD] * wgt, f2 = f[2 * LD] * wgt, f3 = f[3 * LD] * wgt;
    // rows 4 tg .. 4 tg + 3: half tg % 2 of the 16-byte word of row octet tg / 2 (a column further is
    // two 8-byte pieces further)
    uint2* dst = reinterpret_cast<uint2*>(fsec + ((tg >> 1) * PG::NCF + col) * 8 + (tg & 1) * 4);
    if (col < D) {
      *dst = make_uint2(pack_bf2(f0, f1), pack_bf2(f2, f3));
    } else {   // the extra column, split into hi + lo parts: columns D..D+3 = (hi, hi, lo, lo)
      const float h0 = bf_lo(pack_bf2(f0, 0.f)), h1 = bf_lo(pack_bf2(f1, 0.f));
      const float h2 = bf_lo(pack_bf2(f2, 0.f)), h3 = bf_lo(pack_bf2(f3, 0.f));
      const uint2 hi = make_uint2(pack_bf2(h0, h1), pack_bf2(h2, h3));
      const uint2 lo = make_uint2(pack_bf2(f0 - h0, f1 - h1), pack_bf2(f2 - h2, f3 - h3));
      dst[0] = hi; dst[2] = hi; dst[4] = lo; dst[6] = lo;
    }
  }
  if (ord1 && tid <= D) reinterpret_cast<float*>(sb + PG::z_off(p2))[tid] = Sl[D * LD + tid];
}

// ---------------------------------------------------------------------------------------
// bf16 inputs, unmasked: sums the nparts fp32 partial states of a head (slots 0..nparts-1)
// and writes the packed bf16 form (PackedGeo) into the head's last slot, nslots-1.
// grid = (slabs, heads), 256 threads.
// ---------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void state_pack_kernel(float* __restrict__ state, int nslots, int nparts, int p2) {
  using G = Geo<D>;
  using PG = PackedGeo<D>;
  constexpr int LD = G::LD;
  __shared__ __attribute__((aligned(16))) float Sl[(D + 1) * LD];
  const int slab = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int64_t SS = G::state_floats(p2);
  const bool ord1 = slab == PG::nslab(p2) - 1;  // the order-1 rows, followed by the order-0 row
  const float* src = state + (int64_t)head * nslots * SS + (int64_t)slab * D * LD;
  const int nf = (ord1 ? D + 1 : D) * LD;
  for (int idx = tid * 4; idx < nf; idx += 1024) {
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int part = 0; part < nparts; ++part) {
      const float4 t = *reinterpret_cast<const float4*>(src + part * SS + idx);
      a.x += t.x; a.y += t.y; a.z += t.z; a.w += t.w;
    }
    *reinterpret_cast<float4*>(Sl + idx) = a;
  }
  __syncthreads();
  char* sb = reinterpret_cast<char*>(state + ((int64_t)head * nslots + nslots - 1) * SS);
  pack_slab_from_lds<D>(Sl, sb, slab, ord1, p2, tid);
}

// ---------------------------------------------------------------------------------------
// Causal states from per-chunk partial states (a head's chunks built side by side, for cases
// with too few heads for one sequential walk per head to fill the chip).  part holds, per head,
// nslots fp32 partial states (slot c = the state of chunk c alone).
//   forward: slot c of the result = sum of the partial states of chunks < c
//   reverse: slot c of the result = sum of the partial states of chunks > c
// state_prefix_kernel works in place on fp32 slots (grid = (ceil(ss / 1024), heads), one
// float4 per thread); state_pack_slots_kernel then writes every slot in the packed bf16 form
// into `state` (grid = (slabs, heads, slots)).
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void state_prefix_kernel(float* __restrict__ state, int nslots, int64_t ss, int reverse) {
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (idx >= ss) return;
  float* base = state + (int64_t)blockIdx.y * nslots * ss + idx;
  float4 run = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int step = 0; step < nslots; ++step) {
    const int c = reverse ? nslots - 1 - step : step;
    float4* p = reinterpret_cast<float4*>(base + c * ss);
    const float4 t = *p;
    *p = run;
    run.x += t.x; run.y += t.y; run.z += t.z; run.w += t.w;
  }
}

template <int D>
__global__ __launch_bounds__(256) void state_pack_slots_kernel(const float* __restrict__ src_states, float* __restrict__ state,
                                                               int nslots, int p2) {
  using G = Geo<D>;
  using PG = PackedGeo<D>;
  constexpr int LD = G::LD;
  __shared__ __attribute__((aligned(16))) float Sl[(D + 1) * LD];
  const int slab = blockIdx.x, head = blockIdx.y, c = blockIdx.z, tid = threadIdx.x;
  const int64_t SS = G::state_floats(p2), PS = PG::slot_floats(p2);
  const bool ord1 = slab == PG::nslab(p2) - 1;  // the order-1 rows, followed by the order-0 row
  const float* src = src_states + ((int64_t)head * nslots + c) * SS + (int64_t)slab * D * LD;
  const int nf = (ord1 ? D + 1 : D) * LD;
  for (int idx = tid * 4; idx < nf; idx += 1024)
    *reinterpret_cast<float4*>(Sl + idx) = *reinterpret_cast<const float4*>(src + idx);
  __syncthreads();
  pack_slab_from_lds<D>(Sl, reinterpret_cast<char*>(state + ((int64_t)head * nslots + c) * PS), slab, ord1, p2, tid);
}
