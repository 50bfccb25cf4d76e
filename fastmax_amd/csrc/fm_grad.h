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
// Shared by the fp32 and the bf16 kernel.  A result tile T of slab s has rows = channels and lanes
// = own tokens: lane (i, hh) holds, for its token, channel 32 ab + 8 (r / 4) + 4 hh + r % 4 of tile ab
// in accumulator register r, i.e. the lane halves own alternating groups of four channels, and
// own index 16 ab + r counts a half's channels.  xo[own index] is x of that channel, xp[own index]
// x of the channel four above it (round the ring), out / outx the sums owed to those channels.
//
// credit_tile: both credits of tile ABI of shift S (compile-time; S == NS: the order-1 slab, added
// with coefficient a1).  With S = 8 sg + tau and u = r % 4 + tau: u <= 3 and u >= 8 keep the partner
// in the lane's own half (group + sg, or + sg + 1), 4 <= u <= 7 puts it four above own index
// 4 (group + sg) + u - 4 -- for both halves alike.  WEIGHTED: the rows carry their pair weights
// (1 for shifts 0 and D/2, 2 otherwise), so those two tiles are doubled.
// ---------------------------------------------------------------------------------------
template <int D, int S, int ABI, bool WEIGHTED>
__device__ __forceinline__ void credit_tile(const f16v& t, f16v (&out)[D / 32], f16v (&outx)[D / 32],
                                            const float (&xo)[D / 2], const float (&xp)[D / 2], float a1) {
  constexpr int H2 = D / 2, NS = D / 2 + 1, NG = D / 8;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int e = r & 3, grp = 4 * ABI + (r >> 2), own = 16 * ABI + r;
    const float v = (WEIGHTED && (S == 0 || S == H2)) ? t[r] + t[r] : t[r];
    if constexpr (S == NS) {           // the order-1 slab
      out[ABI][r] += a1 * t[r];
    } else if constexpr (S == 0) {     // the diagonal: one member
      out[ABI][r] += v * xo[own];
    } else {
      constexpr int TAU = S % 8, SG = S / 8;
      const int u = e + TAU;
      const int g2 = (grp + SG + (u >= 8 ? 1 : 0)) % NG;
      const int idx = 4 * g2 + (u & 3);
      if (u <= 3 || u >= 8) {
        out[ABI][r] += v * xo[idx];
        if constexpr (S != H2) out[idx >> 4][idx & 15] += v * xo[own];   // (s = D/2 lists every pair from both sides)
      } else {
        out[ABI][r] += v * xp[idx];
        outx[idx >> 4][idx & 15] += v * xo[own];
      }
    }
  }
}

// out += what the token's other lane collected for this lane's channels: the lane of half 1 holds
// those of the same own index, the lane of half 0 those of the own index four higher (round the ring).
template <int D>
__device__ __forceinline__ void exchange_halves(f16v (&out)[D / 32], const f16v (&outx)[D / 32], int hh) {
  constexpr int H2 = D / 2;
#pragma unroll
  for (int ab = 0; ab < D / 32; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int idx = 16 * ab + r, below = (idx + H2 - 4) % H2;
      out[ab][r] += swap_halves(outx[below >> 4][below & 15], outx[ab][r], hh);
    }
}

// ---------------------------------------------------------------------------------------
// One block = 128 own tokens of one head, one wave = 32 of them, one lane pair (i, hh = 0/1) per
// token.  Per shift slab s of the state the kernel contracts 32 state rows at a time (A operand,
// 128-bit LDS reads along the columns) with the token's extended value vector y_ext = [y, yx]
// (B operand straight from registers, one extra MFMA for the extra column).  The result tile T
// (channels a x tokens) holds entry (a, a+s) of every token's symmetric matrix; rows = channels,
// lanes = tokens, so a lane holds, for ITS token, the channels 32 ab + 8 j + 4 hh + e (j, e = 0..3)
// of tile ab in its 16 accumulator registers: the lane halves own alternating groups of four
// channels.  The state stores each unordered pair once, so both members are credited from the
// same T, and with the token's whole x row in registers both credits are register FMAs with
// compile-time register numbers (the shift loop is fully unrolled):
//     out[a]         += T[a] * x[(a+s)%D]
//     out[(a+s)%D]   += T[a] * x[a]                 (0 < s < D/2 only)
// Whether channel a+s lies in the lane's own half depends only on (a mod 4) + (s mod 8), not on hh;
// when it does not, it is one of "the four channels just above an own group", for both halves:
// those x values sit in a second register bank (xp), and what is owed to them is collected in a
// second accumulator bank (outx) that the two lanes of a token exchange once at the end.
// Slabs go global -> LDS directly (no staging registers), two slabs ahead into four buffers, one
// barrier per two slabs; the coefficients multiply the accumulated sums (2 a2 after the order-2
// slabs, a1 on the order-1 tile).  Two tiles are contracted at a time, their matrix instructions
// taking turns (back-to-back instructions on one accumulator wait for each other).
// Causal intra-chunk part: for every streamed 32-token tile the transposed score and g.v tiles
// are formed (streamed x own), W is built in registers and fed back as the B operand of
// out (channels x own) += A1^T (channels x streamed) . W (streamed x own).
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
    const float* state, int nslots, Rows<T> OUT, float* __restrict__ rpart,
    int n, int chunk, int masked, int p2, float a1, float a2, int xdiv, int adiv) {
  static_assert(std::is_same<T, float>::value, "fp32 rows (bf16 rows run grad_kernel_bf)");
  using G = Geo<D>;
  constexpr bool DQ = MODE == 0;
  constexpr int LD = G::LD, AB = G::AB, H2 = G::H2, NS = G::NS;
  constexpr int NG = D / 8;                          // groups of eight channels
  constexpr int SLF = D * LD;                        // floats of a slab (D rows)
  constexpr int NPC = SLF / 4;                       // 16-byte pieces of a slab
  constexpr int NPCR = (NPC + 63) / 64 * 64;
  constexpr int NVS = (NPC + 255) / 256;             // transfers per wave and slab
  constexpr int TILEF = 2 * 32 * LD;                 // both 32-token tiles of a streamed step
  constexpr int SLB = NPCR * 4 > TILEF ? NPCR * 4 : TILEF;
  // four slab buffers as four arrays (the compiler tracks outstanding global -> LDS transfers per
  // LDS object) and a dump for transfers nobody needs; the streamed tiles of the intra-chunk part
  // go through Sb2 and Sb3, which the last step of the state part leaves alone
  __shared__ __attribute__((aligned(16))) float Sb0[SLB];
  __shared__ __attribute__((aligned(16))) float Sb1[SLB];
  __shared__ __attribute__((aligned(16))) float Sb2[SLB];
  __shared__ __attribute__((aligned(16))) float Sb3[SLB];
  __shared__ __attribute__((aligned(16))) float Sjunk[256];
  __shared__ float Cl[2][32];
  __shared__ float red[4];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  // logical block = (128-token block fastest, then head): neighbours in a chunk share their state
  const int lid = xcd_logical_id(blockIdx.x + gridDim.x * blockIdx.y, gridDim.x * gridDim.y);
  // (own positions start at X.lo: the grid covers the 128-token blocks from that one on)
  const int head = lid / gridDim.x, bidx = lid % gridDim.x, tblk = (X.lo >> 7) + bidx, tok0 = tblk * 128;
  const int c = tok0 / chunk;
  const int nc = (n + chunk - 1) / chunk;
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
  const int tok = tok0 + w * 32 + i;   // the lane's own token
  const bool live = tok < n && tok >= xlo;
  const int tokc = max(tok < n ? tok : n - 1, xlo);

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
  // this block's chunk snapshot (masked) or the head's summed state (last slot); the order-2 slabs
  // and the order-1 slab are consecutive runs of D rows
  const float* sbase = state + ((int64_t)ha * nslots + (masked ? c : nslots - 1)) * SS;

  // Transfers of slab st into `buf` (wave-uniform).  No branches: pieces past the slab's end wrap
  // round at the source, and a wave transfer that lies wholly past the end, or a slab past the
  // last one, is sent to Sjunk.
  auto slab_dma = [&](int st, float* buf) __attribute__((always_inline)) {
    const bool on = st < n_state;
    const float* src = sbase + (on ? st : 0) * SLF;
#pragma unroll
    for (int r = 0; r < NVS; ++r) {
      const int first = r * 256 + w * 64;
      float* dst = (on && first < NPCR) ? buf + first * 4 : Sjunk;
      __builtin_amdgcn_global_load_lds(src + ((first + l) % NPC) * 4,
                                       (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    }
  };
  RowTile<D, T, 32> t1, t2;
  float creg = 0.f;
  auto tiles_load = [&](int kk) __attribute__((always_inline)) {
    const int r0 = (tile0 + kk) * 32;
    t1.load(A1h, r0, n, tid);
    t2.load(A2h, r0, n, tid, a2dh, a2den_stride);
    if (!DQ && tid < 32) creg = (r0 + tid < n && r0 + tid >= alo) ? ch[r0 + tid] : 0.f;
  };
  auto tiles_store = [&](int kk) __attribute__((always_inline)) {
    float* tb = (kk & 1) ? Sb3 : Sb2;
    t1.store(tb, LD, a1s, tid);
    t2.store(tb + 32 * LD, LD, 1.0f, tid);
    if (!DQ && tid < 32) Cl[kk & 1][tid] = creg;
  };

  // Everything the block needs first is requested before anything is waited for: the first two
  // slabs, the first streamed tile, the own rows, c of the own token.
  if (n_state > 0) {
    slab_dma(0, Sb0);
    slab_dma(1, Sb1);
  }
  if (n_tile > 0) tiles_load(0);
  const float c_ld = DQ ? ch[tokc] : 0.f;
  // the lane's own token: x of its own channels (xo[4g + e] = channel 8g + 4hh + e) and of the four
  // channels just above each own group (xp[4g + e] = channel 8g + 4hh + 4 + e, round the ring),
  // scaled; its half of y (channels hh H2 ..), the B operand of the state contraction and of g.v
  float xo[H2], xp[H2], Yr[H2];
  {
    const float4* xr = reinterpret_cast<const float4*>(Xh.row(tokc));
    const float4* yr = reinterpret_cast<const float4*>(Yh.row(tokc) + hh * H2);
    float4 xa[NG], xb[NG], ya[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      xa[g] = xr[2 * g + hh];
      xb[g] = xr[(2 * g + hh + 1) % (2 * NG)];
      ya[g] = yr[g];
    }
    const float ysc = live ? (ydh ? 1.0f / ydh[(unsigned)tokc * (unsigned)yden_stride] : 1.0f) : 0.f;
    const float xsc = live ? xs : 0.f;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      xo[4 * g] = xa[g].x * xsc; xo[4 * g + 1] = xa[g].y * xsc; xo[4 * g + 2] = xa[g].z * xsc; xo[4 * g + 3] = xa[g].w * xsc;
      xp[4 * g] = xb[g].x * xsc; xp[4 * g + 1] = xb[g].y * xsc; xp[4 * g + 2] = xb[g].z * xsc; xp[4 * g + 3] = xb[g].w * xsc;
      Yr[4 * g] = ya[g].x * ysc; Yr[4 * g + 1] = ya[g].y * ysc; Yr[4 * g + 2] = ya[g].z * ysc; Yr[4 * g + 3] = ya[g].w * ysc;
    }
  }
  const float c_own = (DQ && live) ? c_ld : 0.f;
  const float yx = hh == 0 ? (DQ ? -c_own : (live ? -1.0f : 0.f)) : 0.f;

  // out[ab][r]: channel 32 ab + 8 (r / 4) + 4 hh + r % 4 of the lane's token, i.e. own index
  // 16 ab + r; outx[.]: what the lane collects for the channel four above that one
  f16v out[AB], outx[AB];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) out[ab][r] = outx[ab][r] = 0.f;

  // Two 32-row tiles at a time (tile ab0 of slab sl0 and tile ab1 of slab sl1), their matrix
  // instructions interleaved: consecutive instructions on the same accumulator wait for each other's
  // result, two accumulators that take turns do not.  A operands: a row's D value columns (this lane
  // half's part) in 128-bit LDS reads, one read ahead of their use, and its extra column.
  auto tile_pair = [&](const float* sl0, int ab0, const float* sl1, int ab1, f16v& t0, f16v& t1) __attribute__((always_inline)) {
    constexpr int NK = H2 / 4;
    const float* r0 = sl0 + (ab0 * 32 + i) * LD;
    const float* r1 = sl1 + (ab1 * 32 + i) * LD;
#pragma unroll
    for (int r = 0; r < 16; ++r) t0[r] = t1[r] = 0.f;
    float4 c0 = *reinterpret_cast<const float4*>(r0 + hh * H2), c1 = *reinterpret_cast<const float4*>(r1 + hh * H2);
    const float x0 = r0[D], x1 = r1[D];
#pragma unroll
    for (int k = 0; k < NK; ++k) {
      float4 n0 = c0, n1 = c1;
      if (k + 1 < NK) {
        n0 = *reinterpret_cast<const float4*>(r0 + hh * H2 + 4 * (k + 1));
        n1 = *reinterpret_cast<const float4*>(r1 + hh * H2 + 4 * (k + 1));
      }
      t0 = FM_MFMA(c0.x, Yr[4 * k], t0);
      t1 = FM_MFMA(c1.x, Yr[4 * k], t1);
      t0 = FM_MFMA(c0.y, Yr[4 * k + 1], t0);
      t1 = FM_MFMA(c1.y, Yr[4 * k + 1], t1);
      t0 = FM_MFMA(c0.z, Yr[4 * k + 2], t0);
      t1 = FM_MFMA(c1.z, Yr[4 * k + 2], t1);
      t0 = FM_MFMA(c0.w, Yr[4 * k + 3], t0);
      t1 = FM_MFMA(c1.w, Yr[4 * k + 3], t1);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // the two reads ahead ...
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);   // ... then this step's eight matrix instructions
      c0 = n0;
      c1 = n1;
    }
    t0 = FM_MFMA(x0, yx, t0);
    t1 = FM_MFMA(x1, yx, t1);
  };
  auto credit = [&](const f16v& t, auto stag, auto abtag) __attribute__((always_inline)) {
    credit_tile<D, decltype(stag)::value, decltype(abtag)::value, false>(t, out, outx, xo, xp, a1);
  };

  // The credits are pure arithmetic, which instruction selection may order freely between the
  // matrix instructions' results and the end of the kernel (it was seen to postpone them all, keeping
  // every tile in scratch memory): an empty volatile statement that takes the accumulators in and out
  // keeps each unit's credits in that unit.
  auto pin_accumulators = [&]() __attribute__((always_inline)) {
    if constexpr (AB == 2) asm volatile("" : "+v"(out[0]), "+v"(out[1]), "+v"(outx[0]), "+v"(outx[1]));
    else asm volatile("" : "+v"(out[0]), "+v"(outx[0]));
  };

  if (n_state > 0) {
    FM_WAIT_VM(0);
    __syncthreads();
  }
  if (n_state > 1) {
    // p = 2.  Slabs 0 .. NS (slab NS is the order-1 slab); slabs 2k, 2k+1 sit in buffers (Sb0, Sb1) for
    // even k and (Sb2, Sb3) for odd k.
    static_assert(NS % 2 == 1 && ((NS + 1) / 2) % 2 == 1, "whole steps of two slabs, the last one in Sb0 and Sb1");
    f16v t0, t1;
    static_for<(NS + 1) / 2>([&](auto ktag) __attribute__((always_inline)) {
      constexpr int K = decltype(ktag)::value;
      float* cur0 = (K & 1) ? Sb2 : Sb0;
      float* cur1 = (K & 1) ? Sb3 : Sb1;
      float* nxt0 = (K & 1) ? Sb0 : Sb2;
      float* nxt1 = (K & 1) ? Sb1 : Sb3;
      __builtin_amdgcn_sched_barrier(0);
      // (every wave is past the buffers of the step before: it has passed the barrier)
      slab_dma(2 * K + 2, nxt0);
      slab_dma(2 * K + 3, nxt1);
      // the 2 AB tile units of the step, two at a time: units v and v + 1 (unit v = tile v % AB of
      // slab 2K + v / AB)
      static_for<AB>([&](auto vtag) __attribute__((always_inline)) {
        constexpr int V0 = 2 * decltype(vtag)::value, V1 = V0 + 1;
        constexpr int S0 = 2 * K + V0 / AB, S1 = 2 * K + V1 / AB;
        tile_pair((V0 / AB) ? cur1 : cur0, V0 % AB, (V1 / AB) ? cur1 : cur0, V1 % AB, t0, t1);
        __builtin_amdgcn_sched_barrier(0);
        auto scale_if_order2_done = [&](auto stag, auto abtag) __attribute__((always_inline)) {
          if constexpr (decltype(stag)::value == NS && decltype(abtag)::value == 0) {
            // order 2 is complete: f'(s) contributes 2 a2
#pragma unroll
            for (int ab = 0; ab < AB; ++ab)
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                out[ab][r] *= 2.0f * a2;
                outx[ab][r] *= 2.0f * a2;
              }
          }
        };
        scale_if_order2_done(std::integral_constant<int, S0>{}, std::integral_constant<int, V0 % AB>{});
        credit(t0, std::integral_constant<int, S0>{}, std::integral_constant<int, V0 % AB>{});
        scale_if_order2_done(std::integral_constant<int, S1>{}, std::integral_constant<int, V1 % AB>{});
        credit(t1, std::integral_constant<int, S1>{}, std::integral_constant<int, V1 % AB>{});
        pin_accumulators();
        __builtin_amdgcn_sched_barrier(0);   // (keeps the units apart: register pressure)
      });
      if constexpr (2 * K + 2 <= NS) {
        FM_WAIT_VM(0);
        __builtin_amdgcn_s_barrier();
      } else {
        // the last step: the first streamed tile can be staged (Sb2 was last read a step ago)
        if (n_tile > 0) tiles_store(0);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    exchange_halves<D>(out, outx, hh);
  } else {
    if (n_state == 1) {
      // p = 1: the order-1 slab is the only one
      f16v t0, t1;
      tile_pair(Sb0, 0, Sb0, AB - 1, t0, t1);
      credit(t0, std::integral_constant<int, NS>{}, std::integral_constant<int, 0>{});
      if constexpr (AB == 2) credit(t1, std::integral_constant<int, NS>{}, std::integral_constant<int, 1>{});
    }
    if (n_tile > 0) tiles_store(0);
  }
  if (n_tile > 0) __syncthreads();   // the first streamed tile is staged

  if (n_tile > 0) {
    const int mine = (tok0 >> 5) + w;
    const float twoa2 = 2.0f * a2;
    for (int kk = 0; kk < n_tile; ++kk) {
      tiles_load(kk + 1 < n_tile ? kk + 1 : kk);
      const int tl = tile0 + kk;
      if (DQ ? tl <= mine : tl >= mine) {
        const float* l1 = (kk & 1) ? Sb3 : Sb2;
        const float* l2 = l1 + 32 * LD;
        // scores and g.v: rows = streamed tokens trow(r,hh), lanes = own tokens (the scores pair the
        // channels in the order of xo)
        f16v sc, gv;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = gv[r] = 0.f;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          const float4 p4 = *reinterpret_cast<const float4*>(l1 + i * LD + 8 * g + 4 * hh);
          const float4 v4 = *reinterpret_cast<const float4*>(l2 + i * LD + hh * H2 + 4 * g);
          sc = FM_MFMA(p4.x, xo[4 * g], sc);
          gv = FM_MFMA(v4.x, Yr[4 * g], gv);
          sc = FM_MFMA(p4.y, xo[4 * g + 1], sc);
          gv = FM_MFMA(v4.y, Yr[4 * g + 1], gv);
          sc = FM_MFMA(p4.z, xo[4 * g + 2], sc);
          gv = FM_MFMA(v4.z, Yr[4 * g + 2], gv);
          sc = FM_MFMA(p4.w, xo[4 * g + 3], sc);
          gv = FM_MFMA(v4.w, Yr[4 * g + 3], gv);
        }
        float pa[16][AB];
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
          for (int ab = 0; ab < AB; ++ab) pa[r][ab] = l1[trow(r, hh) * LD + ab * 32 + i];
        const bool diag = tl == mine;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float cc = DQ ? c_own : Cl[kk & 1][trow(r, hh)];
          float wv = (a1 + twoa2 * sc[r]) * (gv[r] - cc);
          if (diag && (DQ ? trow(r, hh) > i : trow(r, hh) < i)) wv = 0.f;
          sc[r] = wv;
        }
        // out (channels x own) += A1^T (channels x streamed) . W (streamed x own)
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
          for (int ab = 0; ab < AB; ++ab) out[ab] = FM_MFMA(pa[r][ab], sc[r], out[ab]);
      }
      if (kk + 1 < n_tile) tiles_store(kk + 1);
      __syncthreads();
    }
  }

  // the lane holds groups of four consecutive channels of its token: 16-byte stores, scaled by the
  // normaliser
  float rs = 0.f;
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) rs += out[ab][r] * xo[16 * ab + r];
  if (live) {
    T* orow = OUT.head(head).row(tok) + 4 * hh;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const f16v& o = out[g >> 2];
      const int r0 = 4 * (g & 3);
      *reinterpret_cast<float4*>(orow + 8 * g) = make_float4(o[r0] * xs, o[r0 + 1] * xs, o[r0 + 2] * xs, o[r0 + 3] * xs);
    }
  }
  rs = block_sum_256(rs, red, tid);
  if (tid == 0) rpart[(int64_t)head * gridDim.x + bidx] = rs;
}

// ---------------------------------------------------------------------------------------
// bf16 variant of grad_kernel (bf16 inputs and outputs): the same decomposition -- result tiles with
// rows = channels and lanes = own tokens, the lane halves owning alternating groups of four
// channels, both credits of a pair as register FMAs (credit_tile), one exchange between the two
// lanes of a token at the end -- with every contraction on v_mfma_f32_32x32x16_bf16 and fp32
// accumulation.
//
// The state arrives in the packed bf16 form (PackedGeo): a slab goes global -> LDS directly, two
// slabs ahead, into four buffers, one barrier per two slabs.  The state rows are the A operand,
// read through the transposing LDS load (four consecutive columns of a row per 64-bit piece, 16
// consecutive rows per 16 lanes).  The token's extended value vector [y, yx] is the B operand,
// packed once; a 32-row tile costs D/16 + 1 MFMAs.  The matrix instructions of one tile run while
// the credits of the tile before are formed and the operands of the next are read.  The two slabs
// of pair weight 1 are doubled, a2 multiplies the accumulated order-2 credits and a1 the order-1
// tile.  Streamed tiles of the intra-chunk part have buffers of their own (staged as bf16 in both
// orientations: rows for the scores, transposed for the product with W).
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
  using PG = PackedGeo<D>;
  constexpr bool DQ = MODE == 0;
  constexpr int AB = G::AB, H2 = G::H2, NS = G::NS, NG = D / 8;
  constexpr int LB = D + 4;   // bf16 row pitch (elements)
  constexpr int TPB = 36;     // pitch of the transposed 32-token tile
  constexpr int NCF = PG::NCF, FSL = PG::FSL;
  constexpr int NPC = FSL / 8;                       // 16-byte pieces of a slab
  constexpr int NPCR = (NPC + 63) / 64 * 64;
  constexpr int NVS = (NPC + 255) / 256;             // transfers per wave and slab
  constexpr int SLB = NPCR * 8;
  constexpr int TILE = (2 * 32 * LB + D * TPB + 7) / 8 * 8;
  // four slab buffers as four arrays (the compiler tracks outstanding global -> LDS transfers per
  // LDS object), a dump for transfers nobody needs, two buffers for the streamed tiles
  __shared__ __attribute__((aligned(16))) uint16_t Sb0[SLB];
  __shared__ __attribute__((aligned(16))) uint16_t Sb1[SLB];
  __shared__ __attribute__((aligned(16))) uint16_t Sb2[SLB];
  __shared__ __attribute__((aligned(16))) uint16_t Sb3[SLB];
  __shared__ __attribute__((aligned(16))) uint16_t Sjunk[512];
  __shared__ __attribute__((aligned(16))) uint16_t Tl[2][TILE];
  __shared__ float Cl[2][32];
  __shared__ float red[4];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  const int lid = xcd_logical_id(blockIdx.x + gridDim.x * blockIdx.y, gridDim.x * gridDim.y);
  // (own positions start at X.lo: the grid covers the 128-token blocks from that one on)
  const int head = lid / gridDim.x, bidx = lid % gridDim.x, tblk = (X.lo >> 7) + bidx, tok0 = tblk * 128;
  const int c = tok0 / chunk;
  const int nc = (n + chunk - 1) / chunk;
  const int64_t SS = masked ? PG::slot_floats(p2) : G::state_floats(p2);   // slot pitch
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
  const int tok = tok0 + w * 32 + i;   // the lane's own token
  const bool live = tok < n && tok >= xlo;
  const int tokc = max(tok < n ? tok : n - 1, xlo);

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
  const char* sbase = reinterpret_cast<const char*>(state + ((int64_t)ha * nslots + (masked ? c : nslots - 1)) * SS);
  const uint16_t* fsec = reinterpret_cast<const uint16_t*>(sbase);

  // Transfers of slab st into `buf` (wave-uniform).  No branches: pieces past the slab's end wrap
  // round at the source, and a wave transfer that lies wholly past the end, or a slab past the
  // last one, is sent to Sjunk.
  auto slab_dma = [&](int st, uint16_t* buf) __attribute__((always_inline)) {
    const bool on = st < n_state;
    const uint16_t* src = fsec + (on ? st : 0) * FSL;
#pragma unroll
    for (int r = 0; r < NVS; ++r) {
      const int first = r * 256 + w * 64;
      uint16_t* dst = (on && first < NPCR) ? buf + first * 8 : Sjunk;
      __builtin_amdgcn_global_load_lds(src + ((first + l) % NPC) * 8,
                                       (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    }
  };
  RowTile<D, T, 32> t1, t2;
  float creg = 0.f;
  auto tiles_load = [&](int kk) __attribute__((always_inline)) {
    const int r0 = (tile0 + kk) * 32;
    t1.load(A1h, r0, n, tid);
    t2.load(A2h, r0, n, tid, a2dh, a2den_stride);
    if (!DQ && tid < 32) creg = (r0 + tid < n && r0 + tid >= alo) ? ch[r0 + tid] : 0.f;
  };
  auto tiles_store = [&](int buf) __attribute__((always_inline)) {
    t1.store_bf(Tl[buf], LB, a1s, tid);
    t2.store_bf(Tl[buf] + 32 * LB, LB, 1.0f, tid);
    t1.store_t_bf(Tl[buf] + 2 * 32 * LB, TPB, a1s, tid);
    if (!DQ && tid < 32) Cl[buf][tid] = creg;
  };

  // Everything the block needs first is requested before anything is waited for: the first two
  // slabs, the first streamed tile, the own rows, c of the own token.
  if (n_state > 0) {
    slab_dma(0, Sb0);
    slab_dma(1, Sb1);
  }
  if (n_tile > 0) tiles_load(0);
  const float c_ld = DQ ? ch[tokc] : 0.f;
  // the lane's own token: x of its own channels (xo[4g + e] = channel 8g + 4hh + e) and of the four
  // channels just above each own group (xp[4g + e] = channel 8g + 4hh + 4 + e, round the ring),
  // scaled; its half of y (channels hh H2 ..) packed, the B operand of the state contraction and of g.v
  float xo[H2], xp[H2];
  uint2 Yp[H2 / 4];
  {
    const uint4* xr = reinterpret_cast<const uint4*>(Xh.row(tokc));
    const uint4* yr = reinterpret_cast<const uint4*>(Yh.row(tokc) + hh * H2);
    uint4 xa[NG], ya[H2 / 8];
#pragma unroll
    for (int g = 0; g < NG; ++g) xa[g] = xr[g];   // piece g = channels 8g .. 8g+7
#pragma unroll
    for (int u = 0; u < H2 / 8; ++u) ya[u] = yr[u];
    const float ydiv = ydh ? ydh[(unsigned)tokc * (unsigned)yden_stride] : 1.0f;
    const float xsc = live ? xs : 0.f;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const uint4 nx = xa[(g + 1) % NG];
      // own four: the lower or the upper half of piece g; the four above: its upper half, or the
      // lower half of the next piece
      const uint2 own = hh ? make_uint2(xa[g].z, xa[g].w) : make_uint2(xa[g].x, xa[g].y);
      const uint2 abv = hh ? make_uint2(nx.x, nx.y) : make_uint2(xa[g].z, xa[g].w);
      xo[4 * g] = bf_lo(own.x) * xsc; xo[4 * g + 1] = bf_hi(own.x) * xsc;
      xo[4 * g + 2] = bf_lo(own.y) * xsc; xo[4 * g + 3] = bf_hi(own.y) * xsc;
      xp[4 * g] = bf_lo(abv.x) * xsc; xp[4 * g + 1] = bf_hi(abv.x) * xsc;
      xp[4 * g + 2] = bf_lo(abv.y) * xsc; xp[4 * g + 3] = bf_hi(abv.y) * xsc;
    }
    auto unpack8 = [](const uint4& t, float* o, float sc) {
      o[0] = bf_lo(t.x) * sc; o[1] = bf_hi(t.x) * sc; o[2] = bf_lo(t.y) * sc; o[3] = bf_hi(t.y) * sc;
      o[4] = bf_lo(t.z) * sc; o[5] = bf_hi(t.z) * sc; o[6] = bf_lo(t.w) * sc; o[7] = bf_hi(t.w) * sc;
    };
#pragma unroll
    for (int u = 0; u < H2 / 8; ++u) {
      uint4 t = ya[u];
      if (ydh) {   // y = grad_out / den, rounded once
        float f[8];
        unpack8(t, f, 1.0f / ydiv);
        t = make_uint4(pack_bf2(f[0], f[1]), pack_bf2(f[2], f[3]), pack_bf2(f[4], f[5]), pack_bf2(f[6], f[7]));
      }
      if (!live) t = make_uint4(0u, 0u, 0u, 0u);
      Yp[2 * u] = make_uint2(t.x, t.y);
      Yp[2 * u + 1] = make_uint2(t.z, t.w);
    }
  }
  const float c_own = (DQ && live) ? c_ld : 0.f;
  const float yx = hh == 0 ? (DQ ? -c_own : (live ? -1.0f : 0.f)) : 0.f, yxhi = bf_lo(pack_bf2(yx, 0.f));
  // pairs with the state's extra column stored as (e_hi, e_hi, e_lo, e_lo); the upper four k slots
  // of that MFMA are empty
  const bf8v yxp = as_bf8(pack_bf4u(yxhi, yx - yxhi, yxhi, yx - yxhi), make_uint2(0u, 0u));
  if (n_tile > 0) tiles_store(0);

  // out[ab][r]: channel 32 ab + 8 (r / 4) + 4 hh + r % 4 of the lane's token, i.e. own index
  // 16 ab + r; outx[.]: what the lane collects for the channel four above that one
  f16v out[AB], outx[AB];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) out[ab][r] = outx[ab][r] = 0.f;

  // A operand of tile ab: tile row m = lane i is state row 32 ab + i.  The slab is feature-packed,
  // [row / 8][column][row % 8]; the transposing read hands every lane = row four consecutive columns
  // per 64-bit piece when, in every group of 16 lanes (16 consecutive rows), lane J addresses the
  // 8-byte half (J % 4) % 2 of the word of row octet (J % 4) / 2 and column J / 4 of the piece.
  const int trj = l & 15;
  const int troff = (((i >> 4) * 2 + ((trj & 3) >> 1)) * NCF + (trj >> 2)) * 8 + (trj & 1) * 4;
  int tro[AB];
#pragma unroll
  for (int ab = 0; ab < AB; ++ab) tro[ab] = troff + ab * 4 * NCF * 8;
  constexpr int NB = H2 / 4 + 1;
  struct BOps {
    uint2 b[NB];
  };
  auto fetch = [&](const uint16_t* sl, int ab, BOps& o) __attribute__((always_inline)) {
    const uint16_t* ar = sl + tro[ab];
#pragma unroll
    for (int g4 = 0; g4 < H2 / 4; ++g4) o.b[g4] = lds_read_tr16(ar + (hh * H2 + 4 * g4) * 8);
    o.b[H2 / 4] = lds_read_tr16(ar + D * 8);  // extra column as (hi, hi, lo, lo)
  };
  auto chain = [&](const BOps& o) __attribute__((always_inline)) {
    f16v t;
#pragma unroll
    for (int r = 0; r < 16; ++r) t[r] = 0.f;
#pragma unroll
    for (int m = 0; m < H2 / 8; ++m)
      t = FM_MFMA_BF16(as_bf8(o.b[2 * m], o.b[2 * m + 1]), as_bf8(Yp[2 * m], Yp[2 * m + 1]), t);
    return FM_MFMA_BF16(as_bf8(o.b[H2 / 4], make_uint2(0u, 0u)), yxp, t);
  };
  auto credit = [&](const f16v& t, auto stag, auto abtag) __attribute__((always_inline)) {
    credit_tile<D, decltype(stag)::value, decltype(abtag)::value, true>(t, out, outx, xo, xp, a1);
  };
  // (an empty volatile statement that takes the accumulators in and out keeps each unit's credits in
  // that unit: see grad_kernel)
  auto pin_accumulators = [&]() __attribute__((always_inline)) {
    if constexpr (AB == 2) asm volatile("" : "+v"(out[0]), "+v"(out[1]), "+v"(outx[0]), "+v"(outx[1]));
    else asm volatile("" : "+v"(out[0]), "+v"(outx[0]));
  };

  if (n_state > 0) {
    FM_WAIT_VM(0);
    __syncthreads();
  }
  if (n_state > 1) {
    // p = 2.  Tile units u = slab * AB + ab over slabs 0 .. NS (slab NS is the order-1 slab).  Slabs
    // 2k, 2k+1 sit in buffers (Sb0, Sb1) for even k and (Sb2, Sb3) for odd k.  Per unit: read the
    // operands of the next unit, run this unit's matrix instructions, form the credits of the unit
    // before (whose results are complete by now).
    static_assert(NS % 2 == 1, "the order-2 slabs and the order-1 slab make whole steps of two");
    constexpr int NU = (NS + 1) * AB;
    BOps bc, bn;
    f16v tp, tn;
    fetch(Sb0, 0, bc);
    static_for<(NS + 1) / 2>([&](auto ktag) __attribute__((always_inline)) {
      constexpr int K = decltype(ktag)::value;
      uint16_t* cur0 = (K & 1) ? Sb2 : Sb0;
      uint16_t* cur1 = (K & 1) ? Sb3 : Sb1;
      uint16_t* nxt0 = (K & 1) ? Sb0 : Sb2;
      uint16_t* nxt1 = (K & 1) ? Sb1 : Sb3;
      __builtin_amdgcn_sched_barrier(0);
      // (every wave is past the buffers of the step before: it has passed the barrier)
      slab_dma(2 * K + 2, nxt0);
      slab_dma(2 * K + 3, nxt1);
      static_for<2 * AB>([&](auto vtag) __attribute__((always_inline)) {
        constexpr int V = decltype(vtag)::value, U = 2 * K * AB + V;
        // operands of the next unit of this step (the first unit of the next step is read after the barrier)
        if constexpr (V + 1 < 2 * AB) fetch(((V + 1) / AB) ? cur1 : cur0, (V + 1) % AB, bn);
        tn = chain(bc);
        if constexpr (U > 0) {
          constexpr int PS = (U - 1) / AB, PAB = (U - 1) % AB;
          if constexpr (PS == NS && PAB == 0) {
            // order 2 is complete: its coefficient (the pair weight 2 of f' is in the stored rows)
#pragma unroll
            for (int ab = 0; ab < AB; ++ab)
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                out[ab][r] *= a2;
                outx[ab][r] *= a2;
              }
          }
          credit(tp, std::integral_constant<int, PS>{}, std::integral_constant<int, PAB>{});
          pin_accumulators();
        }
        tp = tn;
        if constexpr (V + 1 < 2 * AB) bc = bn;
      });
      if constexpr (2 * K + 2 <= NS) {
        FM_WAIT_VM(0);
        __builtin_amdgcn_s_barrier();
        fetch(nxt0, 0, bc);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (AB == 1) {   // the order-1 slab is a single unit: order 2 ends with the unit before
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        out[0][r] *= a2;
        outx[0][r] *= a2;
      }
    }
    credit(tp, std::integral_constant<int, (NU - 1) / AB>{}, std::integral_constant<int, (NU - 1) % AB>{});
    exchange_halves<D>(out, outx, hh);
  } else if (n_state == 1) {
    // p = 1: the order-1 slab is the only one
    static_for<AB>([&](auto abtag) __attribute__((always_inline)) {
      BOps b1;
      fetch(Sb0, decltype(abtag)::value, b1);
      const f16v t = chain(b1);
      credit(t, std::integral_constant<int, NS>{}, abtag);
    });
  }
  if (n_tile > 0) __syncthreads();   // the first streamed tile is staged

  if (n_tile > 0) {
    uint2 Xp[H2 / 4];
#pragma unroll
    for (int g4 = 0; g4 < H2 / 4; ++g4) Xp[g4] = pack_bf4u(xo[4 * g4], xo[4 * g4 + 1], xo[4 * g4 + 2], xo[4 * g4 + 3]);
    const int mine = (tok0 >> 5) + w;
    const float twoa2 = 2.0f * a2;
    for (int kk = 0; kk < n_tile; ++kk) {
      const int buf = kk & 1;
      tiles_load(kk + 1 < n_tile ? kk + 1 : kk);
      const int tl = tile0 + kk;
      if (DQ ? tl <= mine : tl >= mine) {
        const uint16_t* l1 = Tl[buf];
        const uint16_t* l2 = l1 + 32 * LB;
        const uint16_t* l1t = l1 + 2 * 32 * LB;
        // scores and g.v: rows = streamed tokens trow(r,hh), lanes = own tokens
        f16v sc, gv;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = gv[r] = 0.f;
#pragma unroll
        for (int m = 0; m < H2 / 8; ++m) {
          // (the scores pair the channels in the order of xo: groups 2m and 2m+1 of this lane half)
          const uint16_t* r1 = l1 + i * LB + 16 * m + 4 * hh;
          const uint16_t* r2 = l2 + i * LB + hh * H2 + 8 * m;
          sc = FM_MFMA_BF16(as_bf8(*reinterpret_cast<const uint2*>(r1), *reinterpret_cast<const uint2*>(r1 + 8)),
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
        // out (channels x own) += A1^T (channels x streamed) . W (streamed x own)
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          // accumulator rows 8m..8m+7 of this lane half = streamed tokens 16m + 4hh + {0..3} and + 8
          const bf8v wp = as_bf8(pack_bf4u(sc[8 * m], sc[8 * m + 1], sc[8 * m + 2], sc[8 * m + 3]),
                                 pack_bf4u(sc[8 * m + 4], sc[8 * m + 5], sc[8 * m + 6], sc[8 * m + 7]));
#pragma unroll
          for (int ab = 0; ab < AB; ++ab) {
            const uint16_t* trw = l1t + (ab * 32 + i) * TPB + 16 * m + 4 * hh;
            out[ab] = FM_MFMA_BF16(as_bf8(*reinterpret_cast<const uint2*>(trw), *reinterpret_cast<const uint2*>(trw + 8)),
                                   wp, out[ab]);
          }
        }
      }
      if (kk + 1 < n_tile) tiles_store(buf ^ 1);
      __syncthreads();
    }
  }

  // the lane holds groups of four consecutive channels of its token: 8-byte stores, scaled by the
  // normaliser
  float rs = 0.f;
#pragma unroll
  for (int ab = 0; ab < AB; ++ab)
#pragma unroll
    for (int r = 0; r < 16; ++r) rs += out[ab][r] * xo[16 * ab + r];
  if (live) {
    bf16_t* orow = OUT.head(head).row(tok) + 4 * hh;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const f16v& o = out[g >> 2];
      const int r0 = 4 * (g & 3);
      *reinterpret_cast<uint2*>(orow + 8 * g) = make_uint2(pack_bf2(o[r0] * xs, o[r0 + 1] * xs), pack_bf2(o[r0 + 2] * xs, o[r0 + 3] * xs));
    }
  }
  rs = block_sum_256(rs, red, tid);
  if (tid == 0) rpart[(int64_t)head * gridDim.x + bidx] = rs;
}
