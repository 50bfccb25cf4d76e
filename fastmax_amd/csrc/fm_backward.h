// Backward-side kernels.
//
// With g_i = go_i/den_i, c_i = g_i.o_i and W_ij = f'(s_ij)(g_i.v_j - c_i):
//   dqh_i = sum_j W_ij kh_j      dkh_j = sum_i W_ij qh_i      dv_j = sum_i f(s_ij) g_i
// In moment form the inter-chunk part of dqh needs the prefix state S = sum phi(kh) (x) [v,1]
// contracted over its D+1 columns with [g_i, -c_i]; dkh needs the suffix state
// R = sum phi(qh) (x) [g,c] contracted with [v_j, -1]; dv is phi(kh_j) . R.  Both column
// contractions produce, per token, the symmetric matrix T[a][b] whose product with the
// token's own vector is the order-2 gradient.  The kernels hold tokens in lanes
// (transposed tiles), so that product is a register FMA per accumulator element.
#pragma once
#include "fm_common.h"

// c_i = (go_i . o_i) / den_i, one value per token.  d/4 threads share a row.
template <class T>
__global__ __launch_bounds__(256) void bwd_prep_kernel(const T* __restrict__ go,
                                                       const T* __restrict__ o, int64_t ldo,
                                                       const float* __restrict__ den,
                                                       int64_t den_stride, float* __restrict__ cvec,
                                                       int64_t rows, int d) {
  const int tpr = d >> 2, rpp = 256 / tpr;
  const int sub = threadIdx.x % tpr;
  const int64_t row = (int64_t)blockIdx.x * rpp + threadIdx.x / tpr;
  float s = 0.f;
  if (row < rows) {
    float a[4], b[4];
    load4(go + row * d + sub * 4, a);
    const T* orow = o + row * ldo + sub * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) b[e] = to_f32(orow[e]);
    s = a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
  }
  for (int off = tpr >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (row < rows && sub == 0) cvec[row] = s / den[row * den_stride];
}

// One column-contraction tile:  Tt[r] = sum_col slab[arow][col] * gext[col]  for the 32 state
// rows arow = (ab*32 + lane%32 + ro) mod D of the slab in LDS, tokens in lanes.
template <int D>
__device__ __forceinline__ f16v contract_cols(const float* sl, int arow, int hh,
                                              const float (&Gr)[D / 2], float gx) {
  constexpr int LD = D + 4, H2 = D / 2;
  f16v t;
#pragma unroll
  for (int r = 0; r < 16; ++r) t[r] = 0.f;
  const float* ar = sl + arow * LD + hh * H2;
#pragma unroll
  for (int k = 0; k < H2; ++k) t = FM_MFMA(ar[k], Gr[k], t);
  t = FM_MFMA(sl[arow * LD + D], gx, t);
  return t;
}

// ---------------------------------------------------------------------------------------
// dq kernel (MODE 0) and the dk half of the dk/dv kernel share this body:
//   out_i[a] = a1 (S1[a][:] . gext_i) + 2 a2 sum_b x_i[b] (S2[a,b][:] . gext_i)
// with x = qh, gext = [g, -c] (dq) or x = kh, gext = [v, -1] (dk).  The state holds each
// unordered pair {a, a+s} once; SYM selects how the second member of the pair is credited:
//   SYM = false  a second column contraction over the rotated rows (twice the MFMA work)
//   SYM = true   an LDS float add of T * x[a] into channel (a+s) of a per-token accumulator
// ---------------------------------------------------------------------------------------
template <int D, bool SYM>
__device__ __forceinline__ void grad_from_slab(const float* sl, bool ord2, int s, int i, int hh,
                                               const float (&Gr)[D / 2], float gx,
                                               const float* xl_row,  // LDS row of this token's x
                                               float* mir_row,       // LDS accumulator row (SYM)
                                               f16v (&out)[D / 32]) {
  constexpr int AB = D / 32, H2 = D / 2;
  if (!ord2) {
#pragma unroll
    for (int ab = 0; ab < AB; ++ab) {
      const f16v t = contract_cols<D>(sl, ab * 32 + i, hh, Gr, gx);
#pragma unroll
      for (int r = 0; r < 16; ++r) out[ab][r] += t[r];
    }
    return;
  }
  const bool twice = s > 0 && s < H2;
#pragma unroll
  for (int ab = 0; ab < AB; ++ab) {
    const f16v t = contract_cols<D>(sl, ab * 32 + i, hh, Gr, gx);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int a = ab * 32 + trow(r, hh);
      int rc = a + s;
      rc -= (rc >= D) ? D : 0;
      out[ab][r] += t[r] * xl_row[rc];
      if (SYM) {
        if (twice) atomicAdd(&mir_row[rc], t[r] * xl_row[a]);
      }
    }
  }
  if (!SYM && twice) {
#pragma unroll
    for (int ab = 0; ab < AB; ++ab) {
      int arow = ab * 32 + i - s;
      arow += (arow < 0) ? D : 0;
      const f16v t = contract_cols<D>(sl, arow, hh, Gr, gx);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        int rc = ab * 32 + trow(r, hh) - s;
        rc += (rc < 0) ? D : 0;
        out[ab][r] += t[r] * xl_row[rc];
      }
    }
  }
}

// Write a (128 tokens x D) gradient tile held as transposed accumulators through LDS to
// global memory, scaled by `scale`, and return sum(grad * xhat) over the block (the scalar
// the normalisation backward needs).  stage is >= 128*LD floats of LDS nobody else reads.
template <int D, class T>
__device__ __forceinline__ float write_grad_tile(const f16v (&g)[D / 32], float* stage,
                                                 const float* mir,  // nullable LDS [128][LD]
                                                 const float* xl,   // nullable LDS [128][LD]
                                                 T* out_head, int tok0, int n, float scale, int w,
                                                 int i, int hh, int tid) {
  constexpr int LD = D + 4, AB = D / 32, VPR = D / 4;
  const int qrow = w * 32 + i;
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) stage[qrow * LD + ab * 32 + trow(r, hh)] = g[ab][r];
  __syncthreads();
  float rs = 0.f;
  for (int idx = tid; idx < 128 * VPR; idx += 256) {
    const int row = idx / VPR, c4 = idx % VPR;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float x = stage[row * LD + c4 * 4 + e];
      if (mir) x += mir[row * LD + c4 * 4 + e];
      if (xl) rs += x * xl[row * LD + c4 * 4 + e];
      v[e] = x * scale;
    }
    if (tok0 + row < n) store4(out_head + (int64_t)(tok0 + row) * D + c4 * 4, v);
  }
  return rs;
}

// ---------------------------------------------------------------------------------------
// dq:  one block = 128 query tokens of one head, one wave = 32 of them, tokens in lanes.
// Streams the prefix state S (slot = chunk) and, when causal, the key tiles of the block's
// own chunk up to its own position.  rpart[head*gridDim.x + block] = sum dqh . qh.
// ---------------------------------------------------------------------------------------
template <int D, class T, bool SYM>
__global__ __launch_bounds__(256) void bwd_dq_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
    const T* __restrict__ GO, const float* __restrict__ den, int64_t den_stride,
    const float* __restrict__ cvec, const float* __restrict__ qscale,
    const float* __restrict__ kscale, const float* __restrict__ state, int nslots,
    T* __restrict__ DQ, float* __restrict__ rpart, int n, int chunk, int masked, int p2, float a1,
    float a2) {
  using G = Geo<D>;
  constexpr int LD = G::LD, AB = G::AB, H2 = G::H2, NS = G::NS, SLABF = G::SLABF;
  __shared__ __attribute__((aligned(16))) float Ql[128 * LD];
  __shared__ __attribute__((aligned(16))) float Sl[2 * SLABF];
  __shared__ float Ml[SYM ? 128 * LD : 1];
  __shared__ float red[4];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  const int head = blockIdx.y, tok0 = blockIdx.x * 128;
  const int c = tok0 / chunk;
  const int rows2 = G::rows2(p2);
  const int64_t SS = G::state_floats(p2);
  const T* Qh = Q + (int64_t)head * n * D;
  const T* Kh = K + (int64_t)head * n * D;
  const T* Vh = V + (int64_t)head * n * D;
  const T* Gh = GO + (int64_t)head * n * D;
  const float qs = qscale[head], ks = kscale[head];
  const int qrow = w * 32 + i, tok = tok0 + qrow;

  {
    RowTile<D, T, 128> t;
    t.load(Qh, tok0, n, tid);
    t.store(Ql, LD, qs, tid);
    t.load(Gh, tok0, n, tid, den + (int64_t)head * n * den_stride, den_stride);
    t.store(Sl, LD, 1.0f, tid);
    if (SYM)
      for (int idx = tid; idx < 128 * LD; idx += 256) Ml[idx] = 0.f;
  }
  __syncthreads();
  float Qr[H2], Gr[H2];
#pragma unroll
  for (int t = 0; t < H2; ++t) {
    Qr[t] = Ql[qrow * LD + t + hh * H2];
    Gr[t] = Sl[qrow * LD + t + hh * H2];
  }
  const float ci = tok < n ? cvec[(int64_t)head * n + tok] : 0.f;
  const float gx = hh == 0 ? -ci : 0.f;
  __syncthreads();

  const int n_state = (masked && c == 0) ? 0 : (p2 ? NS : 0) + 1;
  int n_key = 0, kt0 = 0;
  if (masked) {
    kt0 = (c * chunk) >> 5;
    const int last = tok0 + 127 < n ? tok0 + 127 : n - 1;
    n_key = (last >> 5) - kt0 + 1;
  }
  const int n_stage = n_state + n_key;
  const float* sbase = state + ((int64_t)head * nslots + (masked ? c : 0)) * SS;
  const int nsum = masked ? 1 : nslots;

  StateSlab<D * LD> slab;
  RowTile<D, T, 32> kt_k, kt_v;
  auto stage_load = [&](int st) {
    if (st < n_state) {
      const bool ord2 = p2 && st < NS;
      slab.load(sbase + (ord2 ? st * D * LD : rows2 * LD), SS, nsum, D * LD, tid);
    } else {
      const int kt = kt0 + (st - n_state);
      kt_k.load(Kh, kt * 32, n, tid);
      kt_v.load(Vh, kt * 32, n, tid);
    }
  };
  auto stage_store = [&](int st) {
    float* dst = Sl + (st & 1) * SLABF;
    if (st < n_state) {
      const float cf = (p2 && st < NS) ? 2.0f * a2 : a1;
      slab.store(dst, D * LD, D * LD, cf, cf, tid);
    } else {
      kt_k.store(dst, LD, ks, tid);
      kt_v.store(dst + 32 * LD, LD, 1.0f, tid);
    }
  };

  f16v dq[AB];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[ab][r] = 0.f;

  if (n_stage > 0) {
    stage_load(0);
    stage_store(0);
  }
  __syncthreads();
  const int qt_mine = (tok0 >> 5) + w;
  const float twoa2 = 2.0f * a2;
  for (int st = 0; st < n_stage; ++st) {
    const bool more = st + 1 < n_stage;
    if (more) stage_load(st + 1);
    const float* sl = Sl + (st & 1) * SLABF;
    if (st < n_state) {
      grad_from_slab<D, SYM>(sl, p2 && st < NS, st, i, hh, Gr, gx, Ql + qrow * LD,
                             SYM ? Ml + qrow * LD : nullptr, dq);
    } else {
      const int kt = kt0 + (st - n_state);
      if (kt <= qt_mine) {
        const float* kl = sl;
        const float* vl = sl + 32 * LD;
        f16v sc, gv;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = gv[r] = 0.f;
#pragma unroll
        for (int t = 0; t < H2; ++t) {
          sc = FM_MFMA(kl[i * LD + t + hh * H2], Qr[t], sc);
          gv = FM_MFMA(vl[i * LD + t + hh * H2], Gr[t], gv);
        }
        const bool diag = kt == qt_mine;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float wv = (a1 + twoa2 * sc[r]) * (gv[r] - ci);
          if (diag && trow(r, hh) > i) wv = 0.f;
          sc[r] = wv;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float* krow = kl + trow(r, hh) * LD;
#pragma unroll
          for (int ab = 0; ab < AB; ++ab) dq[ab] = FM_MFMA(krow[ab * 32 + i], sc[r], dq[ab]);
        }
      }
    }
    if (more) stage_store(st + 1);
    __syncthreads();
  }

  float rs = write_grad_tile<D, T>(dq, Sl, SYM ? Ml : nullptr, Ql, DQ + (int64_t)head * n * D, tok0,
                                   n, qs, w, i, hh, tid);
  rs = block_sum_256(rs, red, tid);
  if (tid == 0) rpart[(int64_t)head * gridDim.x + blockIdx.x] = rs;
}

// ---------------------------------------------------------------------------------------
// dk and dv:  one block = 128 key tokens of one head, tokens in lanes.  Streams the suffix
// state R (slot = chunk) once for both gradients and, when causal, the query tiles of the
// block's own chunk from its own position to the chunk end.
// ---------------------------------------------------------------------------------------
template <int D, class T, bool SYM>
__global__ __launch_bounds__(256, 2) void bwd_dkdv_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
    const T* __restrict__ GO, const float* __restrict__ den, int64_t den_stride,
    const float* __restrict__ cvec, const float* __restrict__ qscale,
    const float* __restrict__ kscale, const float* __restrict__ state, int nslots,
    T* __restrict__ DK, T* __restrict__ DV, float* __restrict__ rpart, int n, int chunk,
    int masked, int p2, float a0, float a1, float a2) {
  using G = Geo<D>;
  constexpr int LD = G::LD, AB = G::AB, CB = G::CB, H2 = G::H2, NS = G::NS, SLABF = G::SLABF;
  __shared__ __attribute__((aligned(16))) float Kl[128 * LD];
  __shared__ __attribute__((aligned(16))) float Sl[2 * SLABF];
  __shared__ float Cl[2][32];
  __shared__ float Ml[SYM ? 128 * LD : 1];
  __shared__ float red[4];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  const int head = blockIdx.y, tok0 = blockIdx.x * 128;
  const int c = tok0 / chunk;
  const int nc = (n + chunk - 1) / chunk;
  const int rows2 = G::rows2(p2);
  const int64_t SS = G::state_floats(p2);
  const T* Qh = Q + (int64_t)head * n * D;
  const T* Kh = K + (int64_t)head * n * D;
  const T* Vh = V + (int64_t)head * n * D;
  const T* Gh = GO + (int64_t)head * n * D;
  const float* denh = den + (int64_t)head * n * den_stride;
  const float* ch = cvec + (int64_t)head * n;
  const float qs = qscale[head], ks = kscale[head];
  const int krow = w * 32 + i;

  {
    RowTile<D, T, 128> t;
    t.load(Kh, tok0, n, tid);
    t.store(Kl, LD, ks, tid);
    if (tid < 128) Kl[tid * LD + D] = 1.0f;
    t.load(Vh, tok0, n, tid);
    t.store(Sl, LD, 1.0f, tid);
    if (SYM)
      for (int idx = tid; idx < 128 * LD; idx += 256) Ml[idx] = 0.f;
  }
  __syncthreads();
  float Kr[H2], Vr[H2];
#pragma unroll
  for (int t = 0; t < H2; ++t) {
    Kr[t] = Kl[krow * LD + t + hh * H2];
    Vr[t] = Sl[krow * LD + t + hh * H2];
  }
  const float vx = hh == 0 ? -1.0f : 0.f;
  __syncthreads();

  const int n_state = (masked && c == nc - 1) ? 0 : (p2 ? NS : 0) + 1;
  int n_qt = 0, qt0 = 0;
  if (masked) {
    qt0 = tok0 >> 5;  // first query tile that can see this block's keys
    int cend = (c + 1) * chunk < n ? (c + 1) * chunk : n;
    n_qt = ((cend - 1) >> 5) - qt0 + 1;
  }
  const int n_stage = n_state + n_qt;
  const float* sbase = state + ((int64_t)head * nslots + (masked ? c : 0)) * SS;
  const int nsum = masked ? 1 : nslots;

  StateSlab<(D + 1) * LD> slab;
  RowTile<D, T, 32> qt_q, qt_g;
  float creg = 0.f;
  auto stage_load = [&](int st) {
    if (st < n_state) {
      const bool ord2 = p2 && st < NS;
      slab.load(sbase + (ord2 ? st * D * LD : rows2 * LD), SS, nsum, ord2 ? D * LD : (D + 1) * LD,
                tid);
    } else {
      const int qt = qt0 + (st - n_state);
      qt_q.load(Qh, qt * 32, n, tid);
      qt_g.load(Gh, qt * 32, n, tid, denh, den_stride);
      if (tid < 32) creg = (qt * 32 + tid < n) ? ch[qt * 32 + tid] : 0.f;
    }
  };
  auto stage_store = [&](int st) {
    float* dst = Sl + (st & 1) * SLABF;
    if (st < n_state) {
      if (p2 && st < NS) {
        slab.store(dst, D * LD, D * LD, 2.0f * a2, 2.0f * a2, tid);
      } else {
        slab.store(dst, (D + 1) * LD, D * LD, a1, a0, tid);
      }
    } else {
      qt_q.store(dst, LD, qs, tid);
      qt_g.store(dst + 32 * LD, LD, 1.0f, tid);
      if (tid < 32) Cl[st & 1][tid] = creg;
    }
  };

  f16v dk[AB], dv[CB];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) dk[ab][r] = 0.f;
#pragma unroll
  for (int cb = 0; cb < CB; ++cb)
#pragma unroll
    for (int r = 0; r < 16; ++r) dv[cb][r] = 0.f;

  if (n_stage > 0) {
    stage_load(0);
    stage_store(0);
  }
  __syncthreads();
  const int kt_mine = (tok0 >> 5) + w;
  const float twoa2 = 2.0f * a2;
  for (int st = 0; st < n_stage; ++st) {
    const bool more = st + 1 < n_stage;
    if (more) stage_load(st + 1);
    const float* sl = Sl + (st & 1) * SLABF;
    if (st < n_state) {
      const bool ord2 = p2 && st < NS;
      grad_from_slab<D, SYM>(sl, ord2, st, i, hh, Vr, vx, Kl + krow * LD,
                             SYM ? Ml + krow * LD : nullptr, dk);
      // dv^T (cols x tokens) += R^T (cols x features) . phi(k)^T; the slab carries 2*a2, so
      // the two weight-1 shifts take half of it
      const float half = (ord2 && (st == 0 || st == H2)) ? 0.5f : 1.0f;
      const int rbase = hh * H2 + st;
      const float* kr = Kl + krow * LD;
#pragma unroll
      for (int t = 0; t < H2; ++t) {
        int rc = rbase + t;
        rc -= (rc >= D) ? D : 0;
        rc = ord2 ? rc : D;
        const float b = Kr[t] * kr[rc] * half;
        const float* srow = sl + (t + hh * H2) * LD;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) dv[cb] = FM_MFMA(srow[cb * 32 + i], b, dv[cb]);
      }
      if (!ord2) {
        const float* s0 = sl + D * LD;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
          for (int r = 0; r < 16; ++r) dv[cb][r] += s0[cb * 32 + trow(r, hh)];
      }
    } else {
      const int qt = qt0 + (st - n_state);
      if (qt >= kt_mine) {
        const float* ql = sl;
        const float* gl = sl + 32 * LD;
        const float* cl = Cl[st & 1];
        f16v sc, gv;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = gv[r] = 0.f;
#pragma unroll
        for (int t = 0; t < H2; ++t) {
          sc = FM_MFMA(ql[i * LD + t + hh * H2], Kr[t], sc);
          gv = FM_MFMA(gl[i * LD + t + hh * H2], Vr[t], gv);
        }
        const bool diag = qt == kt_mine;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float s = sc[r];
          float f = a0 + s * (a1 + a2 * s);
          float wv = (a1 + twoa2 * s) * (gv[r] - cl[trow(r, hh)]);
          if (diag && trow(r, hh) < i) {
            f = 0.f;
            wv = 0.f;
          }
          sc[r] = f;
          gv[r] = wv;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float* qrow = ql + trow(r, hh) * LD;
          const float* grow = gl + trow(r, hh) * LD;
#pragma unroll
          for (int ab = 0; ab < AB; ++ab) dk[ab] = FM_MFMA(qrow[ab * 32 + i], gv[r], dk[ab]);
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) dv[cb] = FM_MFMA(grow[cb * 32 + i], sc[r], dv[cb]);
        }
      }
    }
    if (more) stage_store(st + 1);
    __syncthreads();
  }

  float rs = write_grad_tile<D, T>(dk, Sl, SYM ? Ml : nullptr, Kl, DK + (int64_t)head * n * D, tok0,
                                   n, ks, w, i, hh, tid);
  __syncthreads();
  write_grad_tile<D, T>(dv, Sl, nullptr, nullptr, DV + (int64_t)head * n * D, tok0, n, 1.0f, w, i,
                        hh, tid);
  rs = block_sum_256(rs, red, tid);
  if (tid == 0) rpart[(int64_t)head * gridDim.x + blockIdx.x] = rs;
}

// ---------------------------------------------------------------------------------------
// Chain rule through x_hat = lim * x / max_n ||x_n||: the scaling by lim/M is already in dx;
// the max-norm row i* additionally gets  dx[i*] -= (sum dx_hat.x_hat) * x[i*] / M^2.
// One block per head; blockDim.x = d.
// ---------------------------------------------------------------------------------------
template <class T>
__global__ void norm_fix_kernel(T* __restrict__ dx, const T* __restrict__ x,
                                const float* __restrict__ scale, const int* __restrict__ arg,
                                const float* __restrict__ rpart, int nblk, int n, int d, float lim) {
  const int head = blockIdx.x, c = threadIdx.x;
  float r = 0.f;
  for (int b = 0; b < nblk; ++b) r += rpart[(int64_t)head * nblk + b];
  const float s = scale[head];
  const float fac = r * s * s / (lim * lim);
  const int64_t off = ((int64_t)head * n + arg[head]) * d + c;
  dx[off] = from_f32<T>(to_f32(dx[off]) - fac * to_f32(x[off]));
}
