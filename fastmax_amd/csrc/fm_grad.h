// Column-contraction kernel: gradients with respect to the normalised q (MODE 0) or k (MODE 1).
//
// With g_i = go_i/den_i, c_i = g_i.o_i and W_ij = f'(s_ij)(g_i.v_j - c_i):
//   dqh_i = sum_j W_ij kh_j = a1 S1 [g_i,-c_i] + 2 a2 sum_b qh_i[b] (S2[.,b,:] [g_i,-c_i])   (+ intra-chunk)
//   dkh_j = sum_i W_ij qh_i = a1 R1 [v_j,-1]  + 2 a2 sum_b kh_j[b] (R2[.,b,:] [v_j,-1])     (+ intra-chunk)
// where S = sum phi(kh) (x) [v,1] over the keys before the chunk and R = sum phi(qh) (x) [g,c] over
// the queries after it.  Both are the same computation with the roles of the operands swapped.
#pragma once
#include "fm_apply.h"
#include "fm_common.h"

// ---------------------------------------------------------------------------------------
// One block = 128 own tokens of one head, one wave = 32 of them.  Per shift slab s of the state
// the kernel contracts the token's extended value vector y_ext = [y, yx] (A operand straight
// from registers, one extra MFMA for the extra column) with 32 state rows at a time (B operand,
// 128-bit LDS reads along the columns).  The result tile T (tokens x channels a) holds entry
// (a, a+s) of every token's symmetric matrix; the state stores each unordered pair once, so
// both members are credited from the same T:
//     out[tok][a]         += T[tok][a] * x[tok][(a+s)%D]        (one LDS read, lanes = channels)
//     out[tok][(a+s)%D]   += T[tok][a] * x[tok][a]              (0 < s < D/2 only)
// The second credit moves along the channel ring, which is the lane dimension here: the two
// 32-channel blocks are merged by a lane select and rotated by s with one ds_bpermute.
// Causal intra-chunk part: for every streamed 32-token tile the transposed score and g.v tiles
// are formed (streamed x own), W is built in registers and fed back as the A operand of
// out += W^T-as-rows . A1.
//
//   MODE 0 (dq): X = q, Y = grad_out/den, yx = -c_i, state S, streamed A1 = k, A2 = v over tiles
//                at or before the own tile, W = f'(s)(g.v - c_own)
//   MODE 1 (dk): X = k, Y = v, yx = -1, state R, streamed A1 = q, A2 = grad_out/den over tiles
//                at or after the own tile, W = f'(s)(g.v - c_streamed)
// rpart[head*gridDim.x + block] = sum over the block of out . x_hat (normalisation backward).
// ---------------------------------------------------------------------------------------
template <int D, class T, int MODE>
__global__ __launch_bounds__(256, 2) void grad_kernel(
    Rows<const T> X, Rows<const T> Y, RowScalars yden, RowScalars cvec, Rows<const T> A1,
    Rows<const T> A2, RowScalars a2den,
    const float* __restrict__ xscale, const float* __restrict__ a1scale,
    const float* __restrict__ state, int nslots, Rows<T> OUT, float* __restrict__ rpart,
    int n, int chunk, int masked, int p2, float a1, float a2, int xdiv, int adiv) {
  using G = Geo<D>;
  constexpr bool DQ = MODE == 0;
  constexpr int LD = G::LD, AB = G::AB, H2 = G::H2, NS = G::NS, SLABF = G::SLABF;
  __shared__ __attribute__((aligned(16))) float Xl[128 * LD];
  __shared__ __attribute__((aligned(16))) float Sl[2 * SLABF];
  __shared__ float Cl[2][32];
  __shared__ float red[4];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  // logical block = (128-token block fastest, then head): neighbours in a chunk share their state
  const int lid = xcd_logical_id(blockIdx.x + gridDim.x * blockIdx.y, gridDim.x * gridDim.y);
  // (own positions start at X.lo: the grid covers the 128-token blocks from that one on)
  const int head = lid / gridDim.x, bidx = lid % gridDim.x, tblk = (X.lo >> 7) + bidx, tok0 = tblk * 128;
  const int c = tok0 / chunk;
  const int nc = (n + chunk - 1) / chunk;
  const int rows2 = G::rows2(p2);
  const int64_t SS = G::state_floats(p2);
  // grouped key/value heads: the own rows belong to head hx = head / xdiv, the streamed rows
  // and the state to head ha = head / adiv (one of the divisors is 1; c_i, the output and the
  // normalisation partial are per query head = head)
  const int hx = head / xdiv, ha = head / adiv;
  const HeadRows<const T> Xh = X.head(hx), Yh = Y.head(hx), A1h = A1.head(ha), A2h = A2.head(ha);
  const float* ydh = yden.head(hx);
  const float* a2dh = a2den.head(ha);
  const int64_t yden_stride = yden.stride, a2den_stride = a2den.stride;
  // c belongs to the query side: own tokens for dq, streamed tokens for dk (cvec.stride == 1)
  const float* ch = cvec.head(head);
  const int xlo = Xh.lo, alo = A1h.lo;
  const float xs = xscale[hx], a1s = a1scale[ha];
  const int xrow = w * 32 + i, tok = tok0 + xrow;

  const bool no_state = masked && (DQ ? c == 0 : c == nc - 1);
  const int n_state = no_state ? 0 : (p2 ? NS : 0) + 1;
  int n_tile = 0, tile0 = 0;
  if (masked) {
    if (DQ) {
      tile0 = (c * chunk) >> 5;
      const int last = tok0 + 127 < n ? tok0 + 127 : n - 1;
      n_tile = (last >> 5) - tile0 + 1;
    } else {
      tile0 = tok0 >> 5;
      const int cend = (c + 1) * chunk < n ? (c + 1) * chunk : n;
      n_tile = ((cend - 1) >> 5) - tile0 + 1;
    }
  }
  // this block's chunk snapshot (masked) or the head's summed state (last slot)
  const float* sbase = state + ((int64_t)ha * nslots + (masked ? c : nslots - 1)) * SS;

  StateSlab<D * LD> slab;
  RowTile<D, T, 32> t1, t2;
  float creg = 0.f;
  auto slab_load = [&](int st) {
    slab.load(sbase + ((p2 && st < NS) ? st * D * LD : rows2 * LD), D * LD, tid);
  };
  auto slab_store = [&](int st) {
    const float cf = (p2 && st < NS) ? 2.0f * a2 : a1;
    slab.store(Sl + (st & 1) * SLABF, D * LD, D * LD, cf, cf, tid);
  };
  auto tiles_load = [&](int kk) {
    const int r0 = (tile0 + kk) * 32;
    t1.load(A1h, r0, n, tid);
    t2.load(A2h, r0, n, tid, a2dh, a2den_stride);
    if (!DQ && tid < 32) creg = (r0 + tid < n && r0 + tid >= alo) ? ch[r0 + tid] : 0.f;
  };
  auto tiles_store = [&](int buf) {
    t1.store(Sl + buf * SLABF, LD, a1s, tid);
    t2.store(Sl + buf * SLABF + 32 * LD, LD, 1.0f, tid);
    if (!DQ && tid < 32) Cl[buf][tid] = creg;
  };

  // out[ab][r]: token w*32 + trow(r,hh), channel ab*32 + i
  f16v out[AB];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) out[ab][r] = 0.f;

  // Everything the block needs first is requested before anything is waited for (one memory
  // latency instead of three in a row): the first slab, the first streamed tile, c of the own
  // token, the own rows.
  if (n_tile > 0) tiles_load(0);
  if (n_state > 0) slab_load(0);
  const float c_ld = DQ ? ch[max(tok < n ? tok : n - 1, xlo)] : 0.f;
  {
    RowTile<D, T, 128> t, u;
    t.load(Xh, tok0, n, tid);
    u.load(Yh, tok0, n, tid, ydh, yden_stride);
    t.store(Xl, LD, xs, tid);
    u.store(Sl, LD, 1.0f, tid);
  }
  __syncthreads();
  // own token of this lane = row xrow: its half of y (A operand of the state contraction, B of g.v)
  float Yr[H2];
#pragma unroll
  for (int t = 0; t < H2; t += 4) {
    const float4 y4 = *reinterpret_cast<const float4*>(Sl + xrow * LD + hh * H2 + t);
    Yr[t] = y4.x; Yr[t + 1] = y4.y; Yr[t + 2] = y4.z; Yr[t + 3] = y4.w;
  }
  const float c_own = (DQ && tok < n && tok >= xlo) ? c_ld : 0.f;
  const float yx = hh == 0 ? (DQ ? -c_own : -1.0f) : 0.f;
  __syncthreads();
  if (n_state > 0) {
    slab_store(0);
  } else if (n_tile > 0) {
    tiles_store(0);
  }
  __syncthreads();

  // B operands of one 32-row tile of a slab: the row's D value columns and its extra column
  struct BOps {
    float4 b4[H2 / 4];
    float bx;
  };
  auto fetch = [&](const float* sl, int ab, BOps& o) {
    const float* ar = sl + (ab * 32 + i) * LD;
#pragma unroll
    for (int k = 0; k < H2 / 4; ++k) o.b4[k] = *reinterpret_cast<const float4*>(ar + hh * H2 + 4 * k);
    o.bx = ar[D];
  };
  auto chain = [&](const BOps& o) {
    f16v t;
#pragma unroll
    for (int r = 0; r < 16; ++r) t[r] = 0.f;
#pragma unroll
    for (int k = 0; k < H2 / 4; ++k) {
      t = FM_MFMA(Yr[4 * k], o.b4[k].x, t);
      t = FM_MFMA(Yr[4 * k + 1], o.b4[k].y, t);
      t = FM_MFMA(Yr[4 * k + 2], o.b4[k].z, t);
      t = FM_MFMA(Yr[4 * k + 3], o.b4[k].w, t);
    }
    return FM_MFMA(yx, o.bx, t);
  };
  // x rows of the 16 tokens this lane holds results for: row w*32 + trow(r,hh), r = 4j+e
  const float* xtok = Xl + (w * 32 + 4 * hh) * LD;
  auto xat = [&](int r, int col) { return xtok[((r >> 2) * 8 + (r & 3)) * LD + col]; };
  // x of the lane's own channels for the 16 token rows of its accumulator registers (the factor
  // of the mirrored credit and of the normalisation partial), read once
  float xown[AB][16];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) xown[ab][r] = xat(r, ab * 32 + i);

  for (int st = 0; st < n_state; ++st) {
    slab_load(st + 1 < n_state ? st + 1 : st);
    const float* sl = Sl + (st & 1) * SLABF;
    BOps ops[AB];
#pragma unroll
    for (int ab = 0; ab < AB; ++ab) fetch(sl, ab, ops[ab]);
    f16v tt[AB];
#pragma unroll
    for (int ab = 0; ab < AB; ++ab) tt[ab] = chain(ops[ab]);
    if (p2 && st < NS) {
      const int s = st;
#pragma unroll
      for (int ab = 0; ab < AB; ++ab) {
        const int rc = (ab * 32 + i + s) & (D - 1);
#pragma unroll
        for (int r = 0; r < 16; ++r) out[ab][r] += tt[ab][r] * xat(r, rc);
      }
      if (s > 0 && s < H2) {
        // credit the other member of each pair: channel (a+s)%D gets T[a]*x[a]
#pragma unroll
        for (int ab = 0; ab < AB; ++ab)
#pragma unroll
          for (int r = 0; r < 16; ++r) tt[ab][r] *= xown[ab][r];
        const bool keep = i < 32 - s;                    // source lanes that stay in their block
        const int src = (((i - s) & 31) + 32 * hh) << 2;  // byte index of the source lane
#pragma unroll
        for (int ab = 0; ab < AB; ++ab)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            // lanes i >= s of block ab take U[ab][i-s]; lanes i < s take U[ab-1][i-s+32]
            const float v = keep ? tt[ab][r] : tt[(ab + 1) % AB][r];
            out[ab][r] += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src, __builtin_bit_cast(int, v)));
          }
      }
    } else {
#pragma unroll
      for (int ab = 0; ab < AB; ++ab)
#pragma unroll
        for (int r = 0; r < 16; ++r) out[ab][r] += tt[ab][r];
    }
    if (st + 1 < n_state) slab_store(st + 1);
    else if (n_tile > 0) tiles_store((st + 1) & 1);
    __syncthreads();
  }

  if (n_tile > 0) {
    float Xr[H2];
#pragma unroll
    for (int t = 0; t < H2; t += 4) {
      const float4 x4 = *reinterpret_cast<const float4*>(Xl + xrow * LD + hh * H2 + t);
      Xr[t] = x4.x; Xr[t + 1] = x4.y; Xr[t + 2] = x4.z; Xr[t + 3] = x4.w;
    }
    const int mine = (tok0 >> 5) + w;
    const float twoa2 = 2.0f * a2;
    for (int kk = 0; kk < n_tile; ++kk) {
      const int buf = (n_state + kk) & 1;
      tiles_load(kk + 1 < n_tile ? kk + 1 : kk);
      const int tl = tile0 + kk;
      if (DQ ? tl <= mine : tl >= mine) {
        const float* l1 = Sl + buf * SLABF;
        const float* l2 = l1 + 32 * LD;
        // rows = streamed tokens trow(r,hh), lanes = own tokens
        f16v sc, gv;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = gv[r] = 0.f;
#pragma unroll
        for (int t = 0; t < H2; t += 4) {
          const float4 p4 = *reinterpret_cast<const float4*>(l1 + i * LD + hh * H2 + t);
          const float4 v4 = *reinterpret_cast<const float4*>(l2 + i * LD + hh * H2 + t);
          sc = FM_MFMA(p4.x, Xr[t], sc);
          gv = FM_MFMA(v4.x, Yr[t], gv);
          sc = FM_MFMA(p4.y, Xr[t + 1], sc);
          gv = FM_MFMA(v4.y, Yr[t + 1], gv);
          sc = FM_MFMA(p4.z, Xr[t + 2], sc);
          gv = FM_MFMA(v4.z, Yr[t + 2], gv);
          sc = FM_MFMA(p4.w, Xr[t + 3], sc);
          gv = FM_MFMA(v4.w, Yr[t + 3], gv);
        }
        float pa[16][AB];
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
          for (int ab = 0; ab < AB; ++ab) pa[r][ab] = l1[trow(r, hh) * LD + ab * 32 + i];
        const bool diag = tl == mine;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float cc = DQ ? c_own : Cl[buf][trow(r, hh)];
          float wv = (a1 + twoa2 * sc[r]) * (gv[r] - cc);
          if (diag && (DQ ? trow(r, hh) > i : trow(r, hh) < i)) wv = 0.f;
          sc[r] = wv;
        }
        // out (own x channels) += W (own x streamed) . A1 (streamed x channels)
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
          for (int ab = 0; ab < AB; ++ab) out[ab] = FM_MFMA(sc[r], pa[r][ab], out[ab]);
      }
      if (kk + 1 < n_tile) tiles_store(buf ^ 1);
      __syncthreads();
    }
  }

  // rows of out are tokens, lanes are channels: store directly, scaled by the normaliser
  float rs = 0.f;
  const HeadRows<T> Oh = OUT.head(head);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int tk = tok0 + w * 32 + trow(r, hh);
#pragma unroll
    for (int ab = 0; ab < AB; ++ab) {
      const float g = out[ab][r];
      rs += g * xown[ab][r];
      if (tk < n && tk >= xlo) Oh.base[(unsigned)tk * Oh.pitch + (unsigned)(ab * 32 + i)] = from_f32<T>(g * xs);
    }
  }
  rs = block_sum_256(rs, red, tid);
  if (tid == 0) rpart[(int64_t)head * gridDim.x + bidx] = rs;
}

// ---------------------------------------------------------------------------------------
// bf16 variant of grad_kernel (bf16 inputs and outputs): every contraction runs on
// v_mfma_f32_32x32x16_bf16 with fp32 accumulation.  The state arrives in the packed bf16 form
// (PackedGeo): a feature-packed slab ([row / 4][column][row % 4], rows carrying their pair weights,
// extra column split into hi + lo parts) is copied to LDS as it is and read through the
// transposing LDS load, which hands every lane = row four consecutive columns per 64-bit piece;
// the two slabs of pair weight 1 are doubled after their contraction, a2 multiplies the
// accumulated order-2 credits and a1 the order-1 tile.  The token's extended value vector is
// packed once, so a 32-row tile costs D/8 + 1 MFMAs; the credits are the fp32 register/LDS work
// of the fp32 kernel.  Streamed tiles are staged as bf16, the first one in both orientations
// (rows for the scores, transposed for the product with W).
// ---------------------------------------------------------------------------------------
template <int D, int MODE>
__global__ __launch_bounds__(256, 2) void grad_kernel_bf(
    Rows<const bf16_t> X, Rows<const bf16_t> Y, RowScalars yden, RowScalars cvec, Rows<const bf16_t> A1,
    Rows<const bf16_t> A2, RowScalars a2den,
    const float* __restrict__ xscale, const float* __restrict__ a1scale,
    const float* state, int nslots, Rows<bf16_t> OUT, float* __restrict__ rpart,
    int n, int chunk, int masked, int p2, float a1, float a2, int xdiv, int adiv) {
  using G = Geo<D>;
  using T = bf16_t;
  constexpr bool DQ = MODE == 0;
  constexpr int LD = G::LD, AB = G::AB, H2 = G::H2, NS = G::NS;
  constexpr int LB = D + 4;   // bf16 row pitch (elements)
  constexpr int TPB = 36;     // pitch of the transposed 32-token tile
  constexpr int SLB0 = D * LB, SLB1 = 2 * 32 * LB + D * TPB;
  constexpr int SLB = ((SLB0 > SLB1 ? SLB0 : SLB1) + 7) / 8 * 8;
  __shared__ __attribute__((aligned(16))) float Xl[128 * LD];
  __shared__ __attribute__((aligned(16))) uint16_t Sb[2][SLB];
  __shared__ float Cl[2][32];
  __shared__ float red[4];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  const int lid = xcd_logical_id(blockIdx.x + gridDim.x * blockIdx.y, gridDim.x * gridDim.y);
  // (own positions start at X.lo: the grid covers the 128-token blocks from that one on)
  const int head = lid / gridDim.x, bidx = lid % gridDim.x, tblk = (X.lo >> 7) + bidx, tok0 = tblk * 128;
  const int c = tok0 / chunk;
  const int nc = (n + chunk - 1) / chunk;
  const int rows2 = G::rows2(p2);
  const int64_t SS = masked ? PackedGeo<D>::slot_floats(p2) : G::state_floats(p2);   // slot pitch
  // grouped key/value heads: the own rows belong to head hx = head / xdiv, the streamed rows
  // and the state to head ha = head / adiv (one of the divisors is 1; c_i, the output and the
  // normalisation partial are per query head = head)
  const int hx = head / xdiv, ha = head / adiv;
  const HeadRows<const T> Xh = X.head(hx), Yh = Y.head(hx), A1h = A1.head(ha), A2h = A2.head(ha);
  const float* ydh = yden.head(hx);
  const float* a2dh = a2den.head(ha);
  const int64_t yden_stride = yden.stride, a2den_stride = a2den.stride;
  // c belongs to the query side: own tokens for dq, streamed tokens for dk (cvec.stride == 1)
  const float* ch = cvec.head(head);
  const int xlo = Xh.lo, alo = A1h.lo;
  const float xs = xscale[hx], a1s = a1scale[ha];
  const int xrow = w * 32 + i, tok = tok0 + xrow;

  const bool no_state = masked && (DQ ? c == 0 : c == nc - 1);
  const int n_state = no_state ? 0 : (p2 ? NS : 0) + 1;
  int n_tile = 0, tile0 = 0;
  if (masked) {
    if (DQ) {
      tile0 = (c * chunk) >> 5;
      const int last = tok0 + 127 < n ? tok0 + 127 : n - 1;
      n_tile = (last >> 5) - tile0 + 1;
    } else {
      tile0 = tok0 >> 5;
      const int cend = (c + 1) * chunk < n ? (c + 1) * chunk : n;
      n_tile = ((cend - 1) >> 5) - tile0 + 1;
    }
  }
  // packed state of this block's chunk (masked) or the head's summed state (last slot)
  using PG = PackedGeo<D>;
  constexpr int NCF = PG::NCF;
  static_assert(PG::FSL <= SLB, "a feature-packed slab must fit a stage buffer");
  const char* sbase = reinterpret_cast<const char*>(state + ((int64_t)ha * nslots + (masked ? c : nslots - 1)) * SS);
  const uint16_t* fsec = reinterpret_cast<const uint16_t*>(sbase);

  // a C slab is copied as it is: 16-byte pieces global -> registers -> LDS
  // (no branches: threads past the end wrap round and copy an early piece a second time, so that
  // every load is issued up front and stays in flight under the MFMAs)
  constexpr int NPC = PG::FSL / 8, NVS = (NPC + 255) / 256;
  static_assert(NVS <= 3, "three named pieces per thread (an indexed array would live in scratch)");
  uint4 sv0, sv1, sv2;
  RowTile<D, T, 32> t1, t2;
  float creg = 0.f;
  auto slab_load = [&](int st) {
    const uint4* src = reinterpret_cast<const uint4*>(fsec + st * PG::FSL);
    sv0 = src[tid % NPC];
    if constexpr (NVS > 1) sv1 = src[(tid + 256) % NPC];
    if constexpr (NVS > 2) sv2 = src[(tid + 512) % NPC];
  };
  auto slab_store = [&](int st) {
    uint4* dst = reinterpret_cast<uint4*>(Sb[st & 1]);
    dst[tid % NPC] = sv0;
    if constexpr (NVS > 1) dst[(tid + 256) % NPC] = sv1;
    if constexpr (NVS > 2) dst[(tid + 512) % NPC] = sv2;
  };
  auto tiles_load = [&](int kk) {
    const int r0 = (tile0 + kk) * 32;
    t1.load(A1h, r0, n, tid);
    t2.load(A2h, r0, n, tid, a2dh, a2den_stride);
    if (!DQ && tid < 32) creg = (r0 + tid < n && r0 + tid >= alo) ? ch[r0 + tid] : 0.f;
  };
  auto tiles_store = [&](int buf) {
    t1.store_bf(Sb[buf], LB, a1s, tid);
    t2.store_bf(Sb[buf] + 32 * LB, LB, 1.0f, tid);
    t1.store_t_bf(Sb[buf] + 2 * 32 * LB, TPB, a1s, tid);
    if (!DQ && tid < 32) Cl[buf][tid] = creg;
  };

  f16v out[AB];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) out[ab][r] = 0.f;

  // Everything the block needs first is requested before anything is waited for (one memory
  // latency instead of three in a row): the first slab, the first streamed tile, c of the own
  // token, the own rows.
  if (n_tile > 0) tiles_load(0);
  if (n_state > 0) slab_load(0);
  const float c_ld = DQ ? ch[max(tok < n ? tok : n - 1, xlo)] : 0.f;
  {
    RowTile<D, T, 128> t, u;
    t.load(Xh, tok0, n, tid);
    u.load(Yh, tok0, n, tid, ydh, yden_stride);
    t.store(Xl, LD, xs, tid);
    // the own y rows only pass through LDS to reach their lanes: [128][LB] bf16 fits one stage pair
    static_assert(128 * LB <= 2 * SLB, "own-row staging must fit the stage buffers");
    u.store_bf(&Sb[0][0], LB, 1.0f, tid);
  }
  __syncthreads();
  // own token of this lane = row xrow: its half of y, packed (A operand of the state
  // contraction, B operand of g.v)
  uint2 Yp[H2 / 4];
#pragma unroll
  for (int g4 = 0; g4 < H2 / 4; ++g4)
    Yp[g4] = *reinterpret_cast<const uint2*>(&Sb[0][0] + xrow * LB + hh * H2 + 4 * g4);
  const float c_own = (DQ && tok < n && tok >= xlo) ? c_ld : 0.f;
  const float yx = hh == 0 ? (DQ ? -c_own : -1.0f) : 0.f, yxhi = bf_lo(pack_bf2(yx, 0.f));
  // pairs with (e_hi, e_hi, e_lo, e_lo); the upper four k slots of that MFMA are empty
  const bf8v yxp = as_bf8(pack_bf4u(yxhi, yx - yxhi, yxhi, yx - yxhi), make_uint2(0u, 0u));
  __syncthreads();
  if (n_state > 0) {
    slab_store(0);
  } else if (n_tile > 0) {
    tiles_store(0);
  }
  __syncthreads();

  // The slab is feature-packed, [row / 4][column][row % 4]; the B operand of the contraction over
  // columns wants, per lane = row, four consecutive columns per 64-bit piece: the transposing LDS
  // read delivers exactly that when, in every group of 16 lanes (16 consecutive rows), lane J
  // addresses the word of row group J % 4 and column J / 4 of the piece.
  const int trj = l & 15;
  const int troff = (((i >> 4) * 4 + (trj & 3)) * NCF + (trj >> 2)) * 4;   // + (ab * 8 * NCF + column) * 4
  auto chain = [&](const uint16_t* sl, int ab) {
    const uint16_t* ar = sl + ab * 8 * NCF * 4 + troff;
    uint2 b[H2 / 4 + 1];
#pragma unroll
    for (int g4 = 0; g4 < H2 / 4; ++g4) b[g4] = lds_read_tr16(ar + (hh * H2 + 4 * g4) * 4);
    b[H2 / 4] = lds_read_tr16(ar + D * 4);  // extra column as (hi, hi, lo, lo)
    f16v t;
#pragma unroll
    for (int r = 0; r < 16; ++r) t[r] = 0.f;
#pragma unroll
    for (int m = 0; m < H2 / 8; ++m) t = FM_MFMA_BF16(as_bf8(Yp[2 * m], Yp[2 * m + 1]), as_bf8(b[2 * m], b[2 * m + 1]), t);
    return FM_MFMA_BF16(yxp, as_bf8(b[H2 / 4], make_uint2(0u, 0u)), t);
  };
  const float* xtok = Xl + (w * 32 + 4 * hh) * LD;
  auto xat = [&](int r, int col) { return xtok[((r >> 2) * 8 + (r & 3)) * LD + col]; };
  // x of the lane's own channels for the 16 token rows of its accumulator registers (the factor
  // of the mirrored credit and of the normalisation partial), read once
  float xown[AB][16];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) xown[ab][r] = xat(r, ab * 32 + i);

  auto slab_step = [&](int st) {
    const uint16_t* sl = Sb[st & 1];
    f16v tt[AB];
#pragma unroll
    for (int ab = 0; ab < AB; ++ab) tt[ab] = chain(sl, ab);
    if (p2 && st < NS) {
      const int s = st;
      // the order-2 slabs carry their pair weights (2, except shifts 0 and D/2): bring those two up
      // to the others, the common factor goes into the final scale
      if (s == 0 || s == H2) {
#pragma unroll
        for (int ab = 0; ab < AB; ++ab)
#pragma unroll
          for (int r = 0; r < 16; ++r) tt[ab][r] *= 2.0f;
      }
#pragma unroll
      for (int ab = 0; ab < AB; ++ab) {
        const int rc = (ab * 32 + i + s) & (D - 1);
#pragma unroll
        for (int r = 0; r < 16; ++r) out[ab][r] += tt[ab][r] * xat(r, rc);
      }
      if (s > 0 && s < H2) {
#pragma unroll
        for (int ab = 0; ab < AB; ++ab)
#pragma unroll
          for (int r = 0; r < 16; ++r) tt[ab][r] *= xown[ab][r];
        const bool keep = i < 32 - s;
        const int src = (((i - s) & 31) + 32 * hh) << 2;
#pragma unroll
        for (int ab = 0; ab < AB; ++ab)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float v = keep ? tt[ab][r] : tt[(ab + 1) % AB][r];
            out[ab][r] += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src, __builtin_bit_cast(int, v)));
          }
      }
      if (st == NS - 1) {  // f'(s) contributes 2*a2 to the order-2 sum, the pair weight 2 is already in
#pragma unroll
        for (int ab = 0; ab < AB; ++ab)
#pragma unroll
          for (int r = 0; r < 16; ++r) out[ab][r] *= a2;
      }
    } else {
#pragma unroll
      for (int ab = 0; ab < AB; ++ab)
#pragma unroll
        for (int r = 0; r < 16; ++r) out[ab][r] += a1 * tt[ab][r];
    }
  };
  // the last slab is peeled off so that load and store of the next slab are unconditional in
  // the loop (a load whose only use sits in a branch is moved there and waited for at once)
  for (int st = 0; st + 1 < n_state; ++st) {
    slab_load(st + 1);
    slab_step(st);
    slab_store(st + 1);
    __syncthreads();
  }
  if (n_state > 0) {
    slab_step(n_state - 1);
    if (n_tile > 0) tiles_store(n_state & 1);
    __syncthreads();
  }

  if (n_tile > 0) {
    uint2 Xp[H2 / 4];
#pragma unroll
    for (int g4 = 0; g4 < H2 / 4; ++g4) {
      const float4 x4 = *reinterpret_cast<const float4*>(Xl + xrow * LD + hh * H2 + 4 * g4);
      Xp[g4] = pack_bf4u(x4.x, x4.y, x4.z, x4.w);
    }
    const int mine = (tok0 >> 5) + w;
    const float twoa2 = 2.0f * a2;
    for (int kk = 0; kk < n_tile; ++kk) {
      const int buf = (n_state + kk) & 1;
      tiles_load(kk + 1 < n_tile ? kk + 1 : kk);
      const int tl = tile0 + kk;
      if (DQ ? tl <= mine : tl >= mine) {
        const uint16_t* l1 = Sb[buf];
        const uint16_t* l2 = l1 + 32 * LB;
        const uint16_t* l1t = l1 + 2 * 32 * LB;
        f16v sc, gv;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = gv[r] = 0.f;
#pragma unroll
        for (int m = 0; m < H2 / 8; ++m) {
          const uint16_t* r1 = l1 + i * LB + hh * H2 + 8 * m;
          const uint16_t* r2 = l2 + i * LB + hh * H2 + 8 * m;
          sc = FM_MFMA_BF16(as_bf8(*reinterpret_cast<const uint2*>(r1), *reinterpret_cast<const uint2*>(r1 + 4)),
                            as_bf8(Xp[2 * m], Xp[2 * m + 1]), sc);
          gv = FM_MFMA_BF16(as_bf8(*reinterpret_cast<const uint2*>(r2), *reinterpret_cast<const uint2*>(r2 + 4)),
                            as_bf8(Yp[2 * m], Yp[2 * m + 1]), gv);
        }
        const bool diag = tl == mine;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float cc = DQ ? c_own : Cl[buf][trow(r, hh)];
          float wv = (a1 + twoa2 * sc[r]) * (gv[r] - cc);
          if (diag && (DQ ? trow(r, hh) > i : trow(r, hh) < i)) wv = 0.f;
          sc[r] = wv;
        }
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          // accumulator rows 8m..8m+7 of this lane half = tokens 16m + 4hh + {0..3} and + 8
          const bf8v wp = as_bf8(pack_bf4u(sc[8 * m], sc[8 * m + 1], sc[8 * m + 2], sc[8 * m + 3]),
                                 pack_bf4u(sc[8 * m + 4], sc[8 * m + 5], sc[8 * m + 6], sc[8 * m + 7]));
#pragma unroll
          for (int ab = 0; ab < AB; ++ab) {
            const uint16_t* trw = l1t + (ab * 32 + i) * TPB + 16 * m + 4 * hh;
            out[ab] = FM_MFMA_BF16(wp, as_bf8(*reinterpret_cast<const uint2*>(trw), *reinterpret_cast<const uint2*>(trw + 8)),
                                   out[ab]);
          }
        }
      }
      if (kk + 1 < n_tile) tiles_store(buf ^ 1);
      __syncthreads();
    }
  }

  float rs = 0.f;
  const HeadRows<T> Oh = OUT.head(head);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int tk = tok0 + w * 32 + trow(r, hh);
#pragma unroll
    for (int ab = 0; ab < AB; ++ab) {
      const float g = out[ab][r];
      rs += g * xown[ab][r];
      if (tk < n && tk >= xlo) Oh.base[(unsigned)tk * Oh.pitch + (unsigned)(ab * 32 + i)] = from_f32<T>(g * xs);
    }
  }
  rs = block_sum_256(rs, red, tid);
  if (tid == 0) rpart[(int64_t)head * gridDim.x + bidx] = rs;
}
