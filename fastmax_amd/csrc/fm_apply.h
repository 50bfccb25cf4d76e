// Row-apply kernel: contracts generated features of the block's own tokens with a moment state.
//   MODE 0  forward:  [num_i, den_i] = phi(qh_i) . S (+ causal intra-chunk tile), o = num/den
//   MODE 1  dv:       dv_j = phi(kh_j) . R (+ causal intra-chunk tile  sum_{i>=j} f(s_ij) g_i)
#pragma once
#include <type_traits>

#include "fm_common.h"

// interleave hint for the instruction scheduler: n x (1 MFMA, 1 LDS read, 1 VALU)
#define FM_SCHED_MFMA_DS_VALU(n)                            \
  _Pragma("unroll") for (int q_ = 0; q_ < (n); ++q_) {      \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      \
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      \
    __builtin_amdgcn_sched_group_barrier(0x002, 1, 0);      \
  }

// ---------------------------------------------------------------------------------------
// One block = 128 tokens of one head, one wave = 32 of them.  Lane (i = l%32, hh = l/32) keeps
// its own half of x_i in registers (channels t + hh*D/2) and a window of the rotated
// partners x_i[(a+s)%D] (reloaded from LDS every fourth shift and read at a compile-time position
// in between), so an order-2 feature costs one multiply of two registers.  The state streams
// through a double-buffered LDS slab (one shift = D rows at a time, global -> LDS directly, one slab
// ahead); the coefficients a2*w_s / a1 / a0 ride on the features; the slab's rows are the B operands
// (two column tiles per feature) and, in the forward pass, its extra column gives the denominator.
// For causal attention 32-token tiles of the block's own chunk follow through the same
// buffers: scores are formed transposed (streamed tokens x own tokens) so that the polynomial
// of the score tile, still in accumulator registers, is directly the A operand of the product
// with the streamed value rows.
//
// A wave cannot overlap its own VALU/LDS work with its own MFMAs, so the kernel is built for
// two resident blocks per CU and keeps the non-MFMA instruction count low: operands of eight
// MFMA k-steps are fetched one batch ahead of their use.
//
//   X   own rows (q forward, k for dv), scaled by xscale[head]
//   A1  streamed rows the scores are taken with (k forward, q for dv), scaled by a1scale[head]
//   A2  streamed value rows (v forward; grad_out for dv, divided by a2den per row)
// ---------------------------------------------------------------------------------------
template <int D, class T, int MODE>
__global__ __launch_bounds__(256, 2) void apply_kernel(
    Rows<const T> X, Rows<const T> A1, Rows<const T> A2,
    const float* __restrict__ xscale, const float* __restrict__ a1scale,
    RowScalars a2den, const float* __restrict__ state,
    int nslots, Rows<T> OUT, RowScalarsOut den, int n,
    int chunk, int masked, int p2, float a0, float a1, float a2, int xdiv,
    int adiv) {
  using G = Geo<D>;
  constexpr bool FWD = MODE == 0;
  constexpr int LD = G::LD, CB = G::CB, H2 = G::H2, NS = G::NS;
  constexpr int KB = 8;  // k-steps per operand batch
  // A slab (the D rows of one shift, or the order-1 rows) travels global -> LDS without passing through
  // registers (global_load_lds_dwordx4: lane l of a wave delivers its 16 bytes at a wave-uniform LDS
  // base + 16 l), one slab ahead of its use, into the buffer the slab before was read from.  Two
  // separate arrays: the compiler's bookkeeping of outstanding transfers is per LDS object.
  constexpr int SLF = D * LD;                        // floats of a slab
  constexpr int NPC = SLF / 4;                       // 16-byte pieces of a slab
  constexpr int NPCR = (NPC + 63) / 64 * 64;
  constexpr int NVS = (NPC + 255) / 256;             // transfers per wave and slab
  constexpr int TILEF = 2 * 32 * LD;                 // both 32-token tiles of a streamed step
  constexpr int SLB = NPCR * 4 > TILEF ? NPCR * 4 : TILEF;
  __shared__ __attribute__((aligned(16))) float Xl[128 * LD];
  __shared__ __attribute__((aligned(16))) float Sl0[SLB];
  __shared__ __attribute__((aligned(16))) float Sl1[SLB];
  __shared__ __attribute__((aligned(16))) float Sjunk[256];   // where transfers nobody needs end up
  __shared__ float denl[128];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  // logical block = (128-token block fastest, then head): neighbours in a chunk share their state
  const int lid = xcd_logical_id(blockIdx.x + gridDim.x * blockIdx.y, gridDim.x * gridDim.y);
  // (own positions start at X.lo: the grid covers the 128-token blocks from that one on)
  const int head = lid / gridDim.x, tblk = (X.lo >> 7) + lid % gridDim.x, tok0 = tblk * 128;
  const int c = tok0 / chunk;
  const int nc = (n + chunk - 1) / chunk;
  const int rows2 = G::rows2(p2);
  const int64_t SS = G::state_floats(p2);
  // grouped key/value heads: the own rows belong to head hx = head / xdiv, the streamed rows
  // and the state to head ha = head / adiv (one of the divisors is 1)
  const int hx = head / xdiv, ha = head / adiv;
  const HeadRows<const T> Xh = X.head(hx), A1h = A1.head(ha), A2h = A2.head(ha);
  const float* a2dh = a2den.head(ha);
  const int64_t a2den_stride = a2den.stride;
  const float xs = xscale[hx], a1s = a1scale[ha];

  // (the own rows are requested here and staged after the first slab and streamed tile have been
  // requested too: one memory latency at the start of a block instead of two in a row)
  RowTile<D, T, 128> xt;
  xt.load(Xh, tok0, n, tid);

  // the state is all zero for the first chunk in scan order
  const bool no_state = masked && (FWD ? c == 0 : c == nc - 1);
  const int n_state = no_state ? 0 : (p2 ? NS : 0) + 1;
  // streamed tiles: forward = key tiles from the chunk start to this block's last tile;
  // dv = query tiles from this block's first tile to the chunk end
  int n_tile = 0, tile0 = 0;
  if (masked) {
    if (FWD) {
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

  // Transfers of slab st into `buf` (wave-uniform; the order-2 slabs and the order-1 slab are
  // consecutive runs of D rows).  No branches: pieces past the slab's end wrap round at the source, and
  // a wave transfer that lies wholly past the end, or a slab past the last one, is sent to Sjunk.
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
  auto tiles_load = [&](int kk) {
    t1.load(A1h, (tile0 + kk) * 32, n, tid);
    t2.load(A2h, (tile0 + kk) * 32, n, tid, a2dh, a2den_stride);
  };
  auto tiles_store = [&](int buf) {
    float* tb = buf ? Sl1 : Sl0;
    t1.store(tb, LD, a1s, tid);
    t2.store(tb + 32 * LD, LD, 1.0f, tid);
  };

  if (n_tile > 0) tiles_load(0);
  if (n_state > 0) slab_dma(0, Sl0);
  // the order-0 row of the state: value columns i and 32 + i, and the extra column
  // (requested together and whatever n_state says -- a slot that is not used is still memory of the state
  // array -- and masked afterwards: a load under a condition gets a wait of its own, for it and for every
  // transfer requested before it, one memory round trip per value)
  float z0[CB], zd = 0.f;
  {
    float zraw[CB + 1];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) zraw[cb] = sbase[(rows2 + D) * LD + cb * 32 + i];
    zraw[CB] = sbase[(rows2 + D) * LD + D];
    const unsigned keep = n_state > 0 ? 0xffffffffu : 0u;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) z0[cb] = a0 * __uint_as_float(__float_as_uint(zraw[cb]) & keep);
    if (FWD) zd = a0 * __uint_as_float(__float_as_uint(zraw[CB]) & (hh == 0 ? keep : 0u));
  }
  xt.store(Xl, LD, xs, tid);
  if (n_state == 0 && n_tile > 0) tiles_store(0);
  FM_WAIT_VM(0);
  __syncthreads();

  const int xrow = w * 32 + i;
  float Xr[H2];
#pragma unroll
  for (int t = 0; t < H2; t += 4) {
    const float4 q4 = *reinterpret_cast<const float4*>(Xl + xrow * LD + hh * H2 + t);
    Xr[t] = q4.x; Xr[t + 1] = q4.y; Xr[t + 2] = q4.z; Xr[t + 3] = q4.w;
  }

  f16v acc[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[cb][r] = 0.f;
  float dn = 0.f;

  // rotated partners: after window_load(s0, cf) (s0 % 4 == 0), Wn[x] = cf * x_i[(hh*H2 + s0 + x) % D].
  // The state is stored raw and each unordered pair once: cf carries a2 and the pair weight (2 for the
  // shifts 0 < s < D/2; the window of shifts 0..3 takes 2 a2 as well and the sums are halved after shift 0).
  float Wn[H2 + 4];
  auto window_load = [&](int s0, float cf) {
#pragma unroll
    for (int j = 0; j < H2 / 4 + 1; ++j) {
      const int c0 = (hh * H2 + s0 + 4 * j) & (D - 1);
      const float4 q4 = *reinterpret_cast<const float4*>(Xl + xrow * LD + c0);
      Wn[4 * j] = q4.x * cf; Wn[4 * j + 1] = q4.y * cf; Wn[4 * j + 2] = q4.z * cf; Wn[4 * j + 3] = q4.w * cf;
    }
  };

  // operands of KB k-steps of a slab: rows a = t + hh*H2, value columns i and 32+i, extra column
  struct Batch {
    float b[KB][CB], dd[KB];
  };
  auto batch_fetch = [&](const float* sl, int t0, Batch& bt) {
    const float* base = sl + (hh * H2 + t0) * LD;
#pragma unroll
    for (int e = 0; e < KB; ++e) {
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) bt.b[e][cb] = base[e * LD + cb * 32 + i];
      if (FWD) bt.dd[e] = base[e * LD + D];
    }
  };
  // one slab; ORD2 = false is the order-1 sweep (feature = x[a] itself).  WO = position of the
  // window: Wn[WO + x] is the partner of channel x for the current shift
  auto slab_compute = [&](const float* sl, auto tag, auto wo) __attribute__((always_inline)) {
    constexpr bool ORD2 = decltype(tag)::value;
    constexpr int WO = decltype(wo)::value;
    Batch cur, nxt;
    batch_fetch(sl, 0, cur);
#pragma unroll
    for (int t0 = 0; t0 < H2; t0 += KB) {
      if (t0 + KB < H2) batch_fetch(sl, t0 + KB, nxt);
#pragma unroll
      for (int e = 0; e < KB; ++e) {
        const float a = ORD2 ? Xr[t0 + e] * Wn[WO + t0 + e] : Xr[t0 + e] * a1;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[cb] = FM_MFMA(a, cur.b[e][cb], acc[cb]);
        if (FWD) dn += a * cur.dd[e];
      }
      FM_SCHED_MFMA_DS_VALU(KB * CB)
      // (an empty volatile statement that takes the denominator sum in and out keeps its FMAs in their
      // batch; without it the scheduler collects them behind the slab's matrix instructions with every
      // feature still alive, and the unrolled shifts spill)
      if (FWD) asm volatile("" : "+v"(dn));
      if (t0 + KB < H2) cur = nxt;
    }
  };
  // one pipeline step: start the transfer of slab st+1 into the other buffer (every wave is past it: it
  // has passed the barrier), work on slab st, wait for the wave's own transfers, barrier (which covers
  // the other waves').  After the last slab the first streamed tile is staged instead.  PAR = st % 2.
  auto slab_iter = [&](int st, auto par, auto tag, auto wo) __attribute__((always_inline)) {
    constexpr bool ORD2 = decltype(tag)::value;
    constexpr int PAR = decltype(par)::value;
    __builtin_amdgcn_sched_barrier(0);   // (keeps the unrolled steps from being interleaved: register pressure)
    slab_dma(st + 1, PAR ? Sl0 : Sl1);
    slab_compute(PAR ? Sl1 : Sl0, tag, wo);
    if (!ORD2) {
      // order 0
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[cb][r] += z0[cb];
      if (FWD) dn += zd;
    }
    if (st + 1 >= n_state && n_tile > 0) tiles_store(PAR ^ 1);
    FM_WAIT_VM(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;

  if (n_state > 1) {
    // p = 2: shifts 0 .. NS-1, then the order-1 slab.  The window of rotated partners is loaded
    // every fourth shift and read at a compile-time position in between (no register moves).
    static_assert((NS - 1) % 4 == 0, "shifts come in groups of four plus the last one");
    for (int st = 0; st < NS - 1; st += 4) {
      window_load(st, 2.0f * a2);
      slab_iter(st, P0{}, std::true_type{}, std::integral_constant<int, 0>{});
      if (st == 0) {   // shift 0 lists every pair once
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[cb][r] *= 0.5f;
        dn *= 0.5f;
      }
      slab_iter(st + 1, P1{}, std::true_type{}, std::integral_constant<int, 1>{});
      slab_iter(st + 2, P0{}, std::true_type{}, std::integral_constant<int, 2>{});
      slab_iter(st + 3, P1{}, std::true_type{}, std::integral_constant<int, 3>{});
    }
    window_load(NS - 1, a2);   // shift D/2 lists every pair once, too
    slab_iter(NS - 1, P0{}, std::true_type{}, std::integral_constant<int, 0>{});
    slab_iter(NS, P1{}, std::false_type{}, std::integral_constant<int, 0>{});
  } else if (n_state == 1) {
    slab_iter(0, P0{}, std::false_type{}, std::integral_constant<int, 0>{});
  }

  const int mine = (tok0 >> 5) + w;
  for (int kk = 0; kk < n_tile; ++kk) {
    const int buf = (n_state + kk) & 1;
    tiles_load(kk + 1 < n_tile ? kk + 1 : kk);
    const int tl = tile0 + kk;
    if (FWD ? tl <= mine : tl >= mine) {
      const float* l1 = buf ? Sl1 : Sl0;
      const float* l2 = l1 + 32 * LD;
      // scores, transposed: rows = streamed tokens trow(r,hh), lanes = own tokens
      f16v sc;
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
      for (int t = 0; t < H2; t += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(l1 + i * LD + hh * H2 + t);
        sc = FM_MFMA(k4.x, Xr[t], sc);
        sc = FM_MFMA(k4.y, Xr[t + 1], sc);
        sc = FM_MFMA(k4.z, Xr[t + 2], sc);
        sc = FM_MFMA(k4.w, Xr[t + 3], sc);
      }
      float vv[16][CB];
#pragma unroll
      for (int r = 0; r < 16; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) vv[r][cb] = l2[trow(r, hh) * LD + cb * 32 + i];
      const bool diag = tl == mine;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float s = sc[r];
        float f = a0 + s * (a1 + a2 * s);
        // causal: a key may not lie after the query
        if (diag && (FWD ? trow(r, hh) > i : trow(r, hh) < i)) f = 0.f;
        sc[r] = f;
        if (FWD) dn += f;
      }
#pragma unroll
      for (int r = 0; r < 16; ++r)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[cb] = FM_MFMA(sc[r], vv[r][cb], acc[cb]);
    }
    if (kk + 1 < n_tile) tiles_store(buf ^ 1);
    __syncthreads();
  }

  if (FWD) {
    const float dtot = dn + __shfl_xor(dn, 32, 64);
    const int tok = tok0 + xrow;
    if (hh == 0) {
      denl[xrow] = dtot;
      if (tok < n && tok >= Xh.lo) den.head(head)[(int64_t)tok * den.stride] = dtot;
    }
    __syncthreads();
  }
  const HeadRows<T> Oh = OUT.head(head);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = w * 32 + trow(r, hh);
    const int tk = tok0 + row;
    if (tk < n && tk >= Xh.lo) {
      const float inv = FWD ? 1.0f / denl[row] : 1.0f;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) Oh.base[(unsigned)tk * Oh.pitch + (unsigned)(cb * 32 + i)] = from_f32<T>(acc[cb][r] * inv);
    }
  }
}

// ---------------------------------------------------------------------------------------
// bf16 variant of apply_kernel (bf16 inputs and outputs): same decomposition, but every
// contraction runs on v_mfma_f32_32x32x16_bf16 with fp32 accumulation.  Features are formed in
// fp32 from the fp32-scaled inputs and rounded when packed.  The state arrives in the packed
// bf16 form (PackedGeo): a feature-packed slab is copied to LDS as it is and the four features
// of a lane's k-slots are one 64-bit LDS read; the order-2 slabs carry their pair weights, a2
// multiplies their accumulated sum, a1 the order-1 features and a0 the fp32 order-0 row.  The
// forward denominator comes from a third accumulator tile whose B operand is the state's extra
// column broadcast to every
// lane, which leaves den[row] in every lane that holds that row of the output.
// Lane half hh owns features/channels 32*hh + t as in the fp32 kernel; MFMA g of a sweep takes
// t = 4g..4g+3 from both halves.
// Pipeline of the state part: slabs go global -> LDS directly (no staging registers), two slabs
// ahead, into four buffers; a step is two slabs and one barrier; the window of rotated partner
// channels is read at compile-time positions (four unrolled shifts per window load); within a
// slab all B operands are requested first, the features are formed while they travel, and the
// matrix instructions then run back to back.  Streamed tiles of the intra-chunk part are
// fetched two tiles ahead.
// ---------------------------------------------------------------------------------------
template <int D, int MODE>
__global__ __launch_bounds__(256, 2) void apply_kernel_bf(
    Rows<const bf16_t> X, Rows<const bf16_t> A1, Rows<const bf16_t> A2,
    const float* __restrict__ xscale, const float* __restrict__ a1scale,
    RowScalars a2den, const float* state,
    int nslots, Rows<bf16_t> OUT, RowScalarsOut den,
    int n, int chunk, int masked, int p2, float a0, float a1, float a2, int xdiv,
    int adiv) {
  using G = Geo<D>;
  using T = bf16_t;
  constexpr bool FWD = MODE == 0;
  constexpr int LD = G::LD, CB = G::CB, H2 = G::H2, NS = G::NS;
  using PG = PackedGeo<D>;
  constexpr int LB = D + 4;            // pitch of bf16 rows (16-bit elements): 8-byte aligned, and the
                                       // 16 lanes of a 64-bit access phase fall in distinct banks
  constexpr int TPB = 36;              // pitch of the transposed 32-token value tile
  constexpr int NCF = PG::NCF, FSL = PG::FSL;
  constexpr int SLB1 = 32 * LB + D * TPB;  // both 32-token tiles
  // A slab travels global -> LDS without passing through registers (global_load_lds_dwordx4: lane
  // l of a wave delivers its 16 bytes at a wave-uniform LDS base + 16 l), two slabs ahead of its
  // use, into one of four buffers (four separate arrays: the compiler's bookkeeping of outstanding
  // transfers is per LDS object).  A buffer is a whole number of 64-piece wave transfers.
  constexpr int NPC = FSL / 8;                       // 16-byte pieces of a slab
  constexpr int NPCR = (NPC + 63) / 64 * 64;
  constexpr int NVS = (NPC + 255) / 256;             // transfers per wave and slab
  constexpr int SLB = (NPCR * 8 > SLB1 ? NPCR * 8 : (SLB1 + 7) / 8 * 8);
  __shared__ __attribute__((aligned(16))) float Xl[128 * LD];
  __shared__ __attribute__((aligned(16))) uint16_t Sb0[SLB];
  __shared__ __attribute__((aligned(16))) uint16_t Sb1[SLB];
  __shared__ __attribute__((aligned(16))) uint16_t Sb2[SLB];
  __shared__ __attribute__((aligned(16))) uint16_t Sb3[SLB];
  __shared__ __attribute__((aligned(16))) uint16_t Sjunk[512];   // where transfers nobody needs end up

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  const int lid = xcd_logical_id(blockIdx.x + gridDim.x * blockIdx.y, gridDim.x * gridDim.y);
  // (own positions start at X.lo: the grid covers the 128-token blocks from that one on)
  const int head = lid / gridDim.x, tblk = (X.lo >> 7) + lid % gridDim.x, tok0 = tblk * 128;
  const int c = tok0 / chunk;
  const int nc = (n + chunk - 1) / chunk;
  const int rows2 = G::rows2(p2);
  const int64_t SS = masked ? PackedGeo<D>::slot_floats(p2) : G::state_floats(p2);   // slot pitch
  // grouped key/value heads: the own rows belong to head hx = head / xdiv, the streamed rows
  // and the state to head ha = head / adiv (one of the divisors is 1)
  const int hx = head / xdiv, ha = head / adiv;
  const HeadRows<const T> Xh = X.head(hx), A1h = A1.head(ha), A2h = A2.head(ha);
  const float* a2dh = a2den.head(ha);
  const int64_t a2den_stride = a2den.stride;
  const float xs = xscale[hx], a1s = a1scale[ha];

  // (the own rows are requested here and staged after the first slabs and streamed tiles have been
  // requested too: one memory latency at the start of a block instead of two in a row)
  RowTile<D, T, 128> xt;
  xt.load(Xh, tok0, n, tid);

  const bool no_state = masked && (FWD ? c == 0 : c == nc - 1);
  const int n_state = no_state ? 0 : (p2 ? NS : 0) + 1;
  int n_tile = 0, tile0 = 0;
  if (masked) {
    if (FWD) {
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
  const float* zsec = reinterpret_cast<const float*>(sbase + PG::z_off(p2));

  // Transfers of slab st into `buf` (wave-uniform).  No branches: pieces past the slab's end wrap
  // round at the source, and a wave transfer that lies wholly past the end, or a slab past the
  // last one, is sent to Sjunk.
  auto slab_dma = [&](int st, uint16_t* buf) __attribute__((always_inline)) {
    const bool live = st < n_state;
    const uint16_t* src = fsec + (live ? st : 0) * FSL;
#pragma unroll
    for (int r = 0; r < NVS; ++r) {
      const int first = r * 256 + w * 64;
      uint16_t* dst = (live && first < NPCR) ? buf + first * 8 : Sjunk;
      __builtin_amdgcn_global_load_lds(src + ((first + l) % NPC) * 8,
                                       (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    }
  };
  // streamed tiles travel through registers (they are scaled, and one of them transposed, on the
  // way), two tiles ahead of their use: two sets of registers that take turns
  RowTile<D, T, 32> t1a, t2a, t1b, t2b;
  auto tiles_load = [&](int kk, auto& u1, auto& u2) __attribute__((always_inline)) {
    u1.load(A1h, (tile0 + kk) * 32, n, tid);
    u2.load(A2h, (tile0 + kk) * 32, n, tid, a2dh, a2den_stride);
  };
  auto tiles_store = [&](int buf, auto& u1, auto& u2) __attribute__((always_inline)) {
    uint16_t* tb = buf ? Sb1 : Sb0;
    u1.store_bf(tb, LB, a1s, tid);
    u2.store_t_bf(tb + 32 * LB, TPB, 1.0f, tid);
  };

  if (n_tile > 0) {
    tiles_load(0, t1a, t2a);
    tiles_load(n_tile > 1 ? 1 : 0, t1b, t2b);
  }
  if (n_state > 0) {
    slab_dma(0, Sb0);
    slab_dma(1, Sb1);
  }
  xt.store(Xl, LD, xs, tid);
  if (n_state == 0 && n_tile > 0) tiles_store(0, t1a, t2a);
  __syncthreads();

  const int xrow = w * 32 + i;
  float Xr[H2];
#pragma unroll
  for (int t = 0; t < H2; t += 4) {
    const float4 q4 = *reinterpret_cast<const float4*>(Xl + xrow * LD + hh * H2 + t);
    Xr[t] = q4.x; Xr[t + 1] = q4.y; Xr[t + 2] = q4.z; Xr[t + 3] = q4.w;
  }

  f16v acc[CB], accd;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    accd[r] = 0.f;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) acc[cb][r] = 0.f;
  }

  float Wn[H2 + 4];
  auto window_load = [&](int s0) {
#pragma unroll
    for (int j = 0; j < H2 / 4 + 1; ++j) {
      const int c0 = (hh * H2 + s0 + 4 * j) & (D - 1);
      const float4 q4 = *reinterpret_cast<const float4*>(Xl + xrow * LD + c0);
      Wn[4 * j] = q4.x; Wn[4 * j + 1] = q4.y; Wn[4 * j + 2] = q4.z; Wn[4 * j + 3] = q4.w;
    }
  };

  // one slab: B operands are 64-bit reads of [feature group][column][4 features]; two feature
  // groups (8 features per lane half) make one k = 16 MFMA.  Operands are fetched one step ahead
  // of the MFMAs that use them.
  auto slab_compute = [&](const uint16_t* sl, auto tag, auto wo) __attribute__((always_inline)) {
    constexpr bool ORD2 = decltype(tag)::value;
    constexpr int WO = decltype(wo)::value;   // Wn[WO + t] is the partner of channel t for this shift
    constexpr int NB = FWD ? CB + 1 : CB;
    constexpr int NM = H2 / 8;  // MFMA steps per column tile
    // the eight features of MFMA step m of lane half hh are row octet hh H2/8 + m: one 16-byte word
    // per column
    const uint16_t* brow = sl + (hh * (H2 / 8) * NCF + i) * 8;
    const uint16_t* erow = sl + (hh * (H2 / 8) * NCF + D) * 8;
    auto fetch = [&](int m, fm_u4 (&b)[NB]) {
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) b[cb] = *reinterpret_cast<const fm_u4*>(brow + (m * NCF + cb * 32) * 8);
      if (FWD) b[NB - 1] = *reinterpret_cast<const fm_u4*>(erow + m * NCF * 8);
    };
    auto feat = [&](int g4) {
      const int t = 4 * g4;
      return ORD2 ? pack_bf4u(Xr[t] * Wn[WO + t], Xr[t + 1] * Wn[WO + t + 1], Xr[t + 2] * Wn[WO + t + 2],
                              Xr[t + 3] * Wn[WO + t + 3])
                  : pack_bf4u(Xr[t] * a1, Xr[t + 1] * a1, Xr[t + 2] * a1, Xr[t + 3] * a1);
    };
    // all B operands of the slab are requested first, the features are formed while they are on
    // their way, then the matrix instructions run back to back
    fm_u4 b[NM][NB];
    uint2 a[NM][2];
#pragma unroll
    for (int m = 0; m < NM; ++m) fetch(m, b[m]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      a[m][0] = feat(2 * m);
      a[m][1] = feat(2 * m + 1);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      const bf8v ap = as_bf8(a[m][0], a[m][1]);
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) acc[cb] = FM_MFMA_BF16(ap, __builtin_bit_cast(bf8v, b[m][cb]), acc[cb]);
      if (FWD) accd = FM_MFMA_BF16(ap, __builtin_bit_cast(bf8v, b[m][NB - 1]), accd);
    }
  };

  // the order-2 slabs carry their pair weights; a2 is applied to their sum, a1 to the order-1
  // features and a0 to the order-0 row
  float zc[CB], zd = 0.f;
  {   // (requested together and whatever n_state says, masked afterwards: a load under a condition gets a wait
      // of its own -- for it and for every transfer requested before it)
    float zraw[CB + 1];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) zraw[cb] = zsec[cb * 32 + i];
    zraw[CB] = zsec[D];
    const unsigned keep = n_state > 0 ? 0xffffffffu : 0u;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) zc[cb] = a0 * __uint_as_float(__float_as_uint(zraw[cb]) & keep);
    if (FWD) zd = a0 * __uint_as_float(__float_as_uint(zraw[CB]) & keep);
  }

  // One pipeline step = two slabs and one barrier: start the transfers of slabs st+2, st+3 into the
  // buffers the previous step read from (every wave is past them: it has passed the barrier),
  // work on slabs st and st+1, wait for the wave's own transfers, barrier (which covers the other
  // waves').  After the last slab the first streamed tile is staged instead.
  auto order0 = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) acc[cb][r] += zc[cb];
      if (FWD) accd[r] += zd;
    }
  };
  auto step_begin = [&](int st, uint16_t* ahead0, uint16_t* ahead1) __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);   // (keeps the unrolled steps apart: register pressure)
    slab_dma(st + 2, ahead0);
    slab_dma(st + 3, ahead1);
  };
  auto step_end = [&](bool last) __attribute__((always_inline)) {
    if (!last) {
      FM_WAIT_VM(0);
      __builtin_amdgcn_s_barrier();
    } else {
      if (n_tile > 0) tiles_store(n_state & 1, t1a, t2a);
      __syncthreads();
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using W0 = std::integral_constant<int, 0>;
  if (n_state > 1) {
    // p = 2: shifts 0 .. NS-1, then the order-1 slab.  The window of rotated partners is loaded
    // every fourth shift and read at a compile-time position in between (no register moves).
    static_assert((NS - 1) % 4 == 0, "shifts come in groups of four plus the last one");
    for (int st = 0; st < NS - 1; st += 4) {
      window_load(st);
      step_begin(st, Sb2, Sb3);
      slab_compute(Sb0, std::true_type{}, W0{});
      __builtin_amdgcn_sched_barrier(0);
      slab_compute(Sb1, std::true_type{}, std::integral_constant<int, 1>{});
      step_end(false);
      step_begin(st + 2, Sb0, Sb1);
      slab_compute(Sb2, std::true_type{}, std::integral_constant<int, 2>{});
      __builtin_amdgcn_sched_barrier(0);
      slab_compute(Sb3, std::true_type{}, std::integral_constant<int, 3>{});
      step_end(false);
    }
    window_load(NS - 1);
    step_begin(NS - 1, Sb2, Sb3);   // (nothing left to bring in: these go to Sjunk)
    slab_compute(Sb0, std::true_type{}, W0{});
    // the order-2 slabs carry their pair weights; a2 multiplies their sum
#pragma unroll
    for (int r = 0; r < 16; ++r) {
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) acc[cb][r] *= a2;
      if (FWD) accd[r] *= a2;
    }
    slab_compute(Sb1, std::false_type{}, W0{});
    order0();
    step_end(true);
  } else if (n_state == 1) {
    slab_compute(Sb0, std::false_type{}, W0{});
    order0();
    step_end(true);
  }

  if (n_tile > 0) {
    uint2 Xp[H2 / 4];
#pragma unroll
    for (int g4 = 0; g4 < H2 / 4; ++g4) Xp[g4] = pack_bf4u(Xr[4 * g4], Xr[4 * g4 + 1], Xr[4 * g4 + 2], Xr[4 * g4 + 3]);
    const bf8v ones = as_bf8(make_uint2(0x3f803f80u, 0x3f803f80u), make_uint2(0x3f803f80u, 0x3f803f80u));
    const int mine = (tok0 >> 5) + w;
    // tile kk is in LDS, tile kk+1 in the registers `nx`; the registers `ld` that carried tile kk are
    // free and take tile kk+2
    auto tile_iter = [&](int kk, auto& ld1, auto& ld2, auto& nx1, auto& nx2) __attribute__((always_inline)) {
      const int buf = (n_state + kk) & 1;
      tiles_load(kk + 2 < n_tile ? kk + 2 : n_tile - 1, ld1, ld2);
      const int tl = tile0 + kk;
      if (FWD ? tl <= mine : tl >= mine) {
        const uint16_t* l1 = buf ? Sb1 : Sb0;
        const uint16_t* l2 = l1 + 32 * LB;
        // every LDS operand of the tile is requested first; the scores accumulate in two
        // independent chains
        uint2 ka[H2 / 8][2], vb[2][CB][2];
#pragma unroll
        for (int m = 0; m < H2 / 8; ++m) {
          ka[m][0] = *reinterpret_cast<const uint2*>(l1 + i * LB + hh * H2 + 8 * m);
          ka[m][1] = *reinterpret_cast<const uint2*>(l1 + i * LB + hh * H2 + 8 * m + 4);
        }
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) {
            const uint16_t* vrow = l2 + (cb * 32 + i) * TPB + 16 * m + 4 * hh;
            vb[m][cb][0] = *reinterpret_cast<const uint2*>(vrow);
            vb[m][cb][1] = *reinterpret_cast<const uint2*>(vrow + 8);
          }
        f16v sc, sc1;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = sc1[r] = 0.f;
        static_assert((H2 / 8) % 2 == 0, "score steps come in pairs");
#pragma unroll
        for (int m = 0; m < H2 / 8; m += 2) {
          sc = FM_MFMA_BF16(as_bf8(ka[m][0], ka[m][1]), as_bf8(Xp[2 * m], Xp[2 * m + 1]), sc);
          sc1 = FM_MFMA_BF16(as_bf8(ka[m + 1][0], ka[m + 1][1]), as_bf8(Xp[2 * m + 2], Xp[2 * m + 3]), sc1);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] += sc1[r];
        const bool diag = tl == mine;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float s = sc[r];
          float f = a0 + s * (a1 + a2 * s);
          if (diag && (FWD ? trow(r, hh) > i : trow(r, hh) < i)) f = 0.f;
          sc[r] = f;
        }
        // accumulator rows 8m..8m+7 of this lane half (tokens 16m + 4hh + {0..3} and + 8) are the
        // eight k slots of one MFMA; the transposed value tile supplies the same tokens
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          const bf8v pp = as_bf8(pack_bf4u(sc[8 * m], sc[8 * m + 1], sc[8 * m + 2], sc[8 * m + 3]),
                                 pack_bf4u(sc[8 * m + 4], sc[8 * m + 5], sc[8 * m + 6], sc[8 * m + 7]));
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) acc[cb] = FM_MFMA_BF16(pp, as_bf8(vb[m][cb][0], vb[m][cb][1]), acc[cb]);
          if (FWD) accd = FM_MFMA_BF16(pp, ones, accd);
        }
      }
      if (kk + 1 < n_tile) tiles_store(buf ^ 1, nx1, nx2);
      __syncthreads();
    };
    for (int kk = 0; kk < n_tile; kk += 2) {
      tile_iter(kk, t1a, t2a, t1b, t2b);
      if (kk + 1 < n_tile) tile_iter(kk + 1, t1b, t2b, t1a, t2a);
    }
  }

  const HeadRows<T> Oh = OUT.head(head);
  float* denh = FWD ? den.head(head) : nullptr;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int tk = tok0 + w * 32 + trow(r, hh);
    if (tk < n && tk >= Xh.lo) {
      const float inv = FWD ? 1.0f / accd[r] : 1.0f;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) Oh.base[(unsigned)tk * Oh.pitch + (unsigned)(cb * 32 + i)] = from_f32<T>(acc[cb][r] * inv);
      if (FWD && i == 0) denh[(int64_t)tk * den.stride] = accd[r];
    }
  }
}
