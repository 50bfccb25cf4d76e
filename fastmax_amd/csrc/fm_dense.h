// Dense-tile form of Fastmax attention: every (query, key) score tile is formed and the polynomial
// applied to it, with no moment states at all.
//
// The moment form costs about 2.1 d^3 flop per token and pass whatever the sequence length (p = 2, each
// unordered channel pair once), the dense form 2 n d per token under the causal mask.  Below n ~ d^2
// (and for every head dimension the moment kernels are not built for) the dense form is the cheaper
// one, it needs no workspace, and all of its work is plain matrix tiles.  It is the chunked scan of the
// other kernels with a single chunk: the intra-chunk masked score tile is all there is.
//
//   forward   o_i  = sum_j f(s_ij) v_j / sum_j f(s_ij)                 s_ij = qh_i . kh_j
//   dq        dqh_i = sum_j W_ij kh_j      W_ij = f'(s_ij) (g_i . v_j - c_i),  g = grad_out / den,  c_i = g_i . o_i
//   dk, dv    dkh_j = sum_i W_ij qh_i      dv_j = sum_i f(s_ij) g_i
// (reference: example.py:199-212 is this dense form; fastmax_cuda_forward.cu:102-197 and
// fastmax_cuda_backward.cu:26-882 are the token loops it replaces).
//
// One block = 4 or 8 waves; a wave owns RT tiles of 32 "own" rows (queries in forward / dq, keys in dk/dv)
// whose operands stay in registers, and walks the "streamed" rows (keys, resp. queries) in stages of
// BN rows that all the block's waves share through LDS (double buffered, one barrier per stage).  Score tiles
// are formed with the streamed rows as the A operand (rows of the tile) and the own rows as the B
// operand (columns = lanes), so that f(score), still in the accumulator registers, is directly the A
// operand of the second contraction (rows = own... of the transposed tile), whose B operand is the
// streamed tile stored transposed.  Head dimensions are handled as DP = d rounded up to a multiple of
// 32: channels past d are zero on load and skipped on store.
#pragma once
#include <type_traits>

#include "fm_common.h"

namespace dense {

// Matrix-instruction policy.  A "fragment" is the 16 bytes one lane feeds into one step of a
// contraction: 8 bf16 (one v_mfma_f32_32x32x16_bf16, lane half hh supplies k = 8 hh .. 8 hh + 7 of the
// step's 16) or 4 floats (four v_mfma_f32_32x32x2f32, lane half hh supplies k = 4 hh + u to instruction u
// of the step's 8).  Both operands of a contraction use the same mapping, so any such assignment of k
// indices is valid.
template <class T>
struct Mma;

template <>
struct Mma<bf16_t> {
  using Elt = uint16_t;
  using Frag = fm_u4;
  static constexpr int EPL = 8;    // elements per lane and fragment
  static constexpr int KF = 16;    // contraction length of a fragment step
  static constexpr int PAD = 8;    // row padding of LDS tiles (elements): 16 bytes, conflict-free 128-bit rows
  static __device__ __forceinline__ Frag zero() { return Frag{0u, 0u, 0u, 0u}; }
  static __device__ __forceinline__ f16v mma(const Frag& a, const Frag& b, const f16v& c) {
    return FM_MFMA_BF16(__builtin_bit_cast(bf8v, a), __builtin_bit_cast(bf8v, b), c);
  }
  // Fragment f of an accumulator tile used as an operand whose k index is the tile's row: registers
  // 8 f .. 8 f + 7 of lane half hh are rows 16 f + 8 (e / 4) + 4 hh + e % 4.
  template <int F>
  static __device__ __forceinline__ Frag from_acc(const f16v& a) {
    return Frag{pack_bf2(a[8 * F], a[8 * F + 1]), pack_bf2(a[8 * F + 2], a[8 * F + 3]),
                pack_bf2(a[8 * F + 4], a[8 * F + 5]), pack_bf2(a[8 * F + 6], a[8 * F + 7])};
  }
  // where row x of a transposed tile is stored, so that the eight rows of such a fragment are
  // contiguous: one 128-bit read at 16 f + 8 hh
  static __device__ __forceinline__ int tpos(int x) {
    return (x & ~15) | (((x >> 2) & 1) << 3) | (((x >> 3) & 1) << 2) | (x & 3);
  }
  // acc + the sum of the fragment's elements, as rounded
  static __device__ __forceinline__ float fsum(const Frag& w, float acc) {
    acc = fm_dot2_bf16(w.x, 0x3f803f80u, acc);
    acc = fm_dot2_bf16(w.y, 0x3f803f80u, acc);
    acc = fm_dot2_bf16(w.z, 0x3f803f80u, acc);
    return fm_dot2_bf16(w.w, 0x3f803f80u, acc);
  }
  static __device__ __forceinline__ void unpack(const uint4& r, float (&o)[8]) {
    o[0] = bf_lo(r.x); o[1] = bf_hi(r.x); o[2] = bf_lo(r.y); o[3] = bf_hi(r.y);
    o[4] = bf_lo(r.z); o[5] = bf_hi(r.z); o[6] = bf_lo(r.w); o[7] = bf_hi(r.w);
  }
  static __device__ __forceinline__ uint4 pack(const float (&o)[8]) {
    return make_uint4(pack_bf2(o[0], o[1]), pack_bf2(o[2], o[3]), pack_bf2(o[4], o[5]), pack_bf2(o[6], o[7]));
  }
  static __device__ __forceinline__ Elt elt(const uint4& r, int e) {
    const uint32_t w = e < 2 ? r.x : e < 4 ? r.y : e < 6 ? r.z : r.w;
    return (Elt)((e & 1) ? (w >> 16) : w);
  }
  static __device__ __forceinline__ Elt to_elt(float v) { return (Elt)pack_bf2(v, 0.f); }
};

template <>
struct Mma<float> {
  using Elt = float;
  using Frag = float4;
  static constexpr int EPL = 4;
  static constexpr int KF = 8;
  static constexpr int PAD = 4;
  static __device__ __forceinline__ Frag zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
  static __device__ __forceinline__ f16v mma(const Frag& a, const Frag& b, f16v c) {
    c = FM_MFMA(a.x, b.x, c);
    c = FM_MFMA(a.y, b.y, c);
    c = FM_MFMA(a.z, b.z, c);
    return FM_MFMA(a.w, b.w, c);
  }
  // registers 4 f .. 4 f + 3 of lane half hh are rows 8 f + 4 hh + u
  template <int F>
  static __device__ __forceinline__ Frag from_acc(const f16v& a) {
    return make_float4(a[4 * F], a[4 * F + 1], a[4 * F + 2], a[4 * F + 3]);
  }
  static __device__ __forceinline__ int tpos(int x) { return x; }
  static __device__ __forceinline__ float fsum(const Frag& w, float acc) { return acc + ((w.x + w.y) + (w.z + w.w)); }
  static __device__ __forceinline__ void unpack(const uint4& r, float (&o)[4]) {
    o[0] = __uint_as_float(r.x); o[1] = __uint_as_float(r.y); o[2] = __uint_as_float(r.z); o[3] = __uint_as_float(r.w);
  }
  static __device__ __forceinline__ uint4 pack(const float (&o)[4]) {
    return make_uint4(__float_as_uint(o[0]), __float_as_uint(o[1]), __float_as_uint(o[2]), __float_as_uint(o[3]));
  }
  static __device__ __forceinline__ Elt elt(const uint4& r, int e) {
    return __uint_as_float(e == 0 ? r.x : e == 1 ? r.y : e == 2 ? r.z : r.w);
  }
  static __device__ __forceinline__ Elt to_elt(float v) { return v; }
};

// The per-element mask tests of a score tile sit in blocks that only the diagonal and the ragged last tiles
// enter (a wave-uniform condition).  Left alone the compiler turns such a block into selects that every tile
// executes -- 16 compares and 32 selects per tile, half as many instructions again as the tile's arithmetic;
// a statement it may not speculate keeps the block a branch.
#define FM_KEEP_BRANCH() asm volatile("" ::: "memory")

// an all-zero accumulator tile (the C operand of a contraction's first step)
constexpr f16v kZero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

// sum over the NW waves of a block; red is NW floats of LDS; the result is valid in every thread
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red, int tid) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  __syncthreads();
  if ((tid & 63) == 0) red[tid >> 6] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) t += red[w];
  return t;
}

__device__ __forceinline__ float to_f32_elt(float v) { return v; }
__device__ __forceinline__ float to_f32_elt(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

template <class T>
__device__ __forceinline__ typename Mma<T>::Frag lds_frag(const typename Mma<T>::Elt* p) {
  return *reinterpret_cast<const typename Mma<T>::Frag*>(p);
}

// R rows x DP channels of one head on their way global -> registers -> LDS, by the NT threads of a block.
// Consecutive threads take consecutive rows (16 bytes of a row each), which makes both the row-major
// and the transposed LDS writes conflict-free.  Rows outside [lo, pend) and channels past d are zero.
template <int DP, class T, int R, int NT>
struct TileRegs {
  using M = Mma<T>;
  using Elt = typename M::Elt;
  static constexpr int EPP = 16 / (int)sizeof(T);   // elements per 16-byte piece
  static constexpr int PPR = DP / EPP;
  static constexpr int TOTAL = R * PPR;
  static constexpr int NV = (TOTAL + NT - 1) / NT;
  uint4 raw[NV];
  float rf[NV];   // row divisor of scaled tiles: rowdiv[row] (of the nearest row that exists: the others' elements are zero)

  __device__ __forceinline__ void load(const HeadRows<const T>& hr, int pos0, int pend, int d, int tid,
                                       const float* rowdiv = nullptr, int64_t rdstride = 0) {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * NT;
      const bool in = idx < TOTAL;
      const int row = in ? idx % R : 0, pc = in ? idx / R : 0;
      const int pos = pos0 + row;
      const bool live = in && pos >= hr.lo && pos < pend && pc * EPP < d;
      const int ps = max(pos < pend ? pos : pend - 1, hr.lo);
      const uint4 t = *reinterpret_cast<const uint4*>(hr.base + ((unsigned)ps * hr.pitch + (unsigned)(live ? pc * EPP : 0)));
      raw[u] = live ? t : make_uint4(0u, 0u, 0u, 0u);
      // (the divisor as loaded: anything computed from it here would make this a wait for every load above it)
      rf[u] = 1.0f;
      if (rowdiv) rf[u] = rowdiv[(unsigned)ps * (unsigned)rdstride];
    }
  }
  // as loaded: row-major [R][pr] and / or transposed [DP][pt] (row x at column tpos(x))
  __device__ __forceinline__ void store(Elt* rm, int pr, Elt* tr, int pt, int tid) const {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * NT;
      if (idx < TOTAL) {
        const int row = idx % R, pc = idx / R;
        if (rm) *reinterpret_cast<uint4*>(rm + row * pr + pc * EPP) = raw[u];
        if (tr) {
          Elt* t0 = tr + pc * EPP * pt + M::tpos(row);
#pragma unroll
          for (int e = 0; e < EPP; ++e) t0[e * pt] = M::elt(raw[u], e);
        }
      }
    }
  }
  // over the row divisor and times a constant each: srm for the row-major copy, str for the transposed one
  __device__ __forceinline__ void store_scaled(Elt* rm, int pr, float srm, Elt* tr, int pt, float str, int tid) const {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * NT;
      if (idx < TOTAL) {
        const int row = idx % R, pc = idx / R;
        float x[EPP], y[EPP];
        M::unpack(raw[u], x);
        const float inv = 1.0f / rf[u], f1 = inv * srm, f2 = inv * str;
#pragma unroll
        for (int e = 0; e < EPP; ++e) {
          y[e] = x[e] * f2;
          x[e] *= f1;
        }
        if (rm) *reinterpret_cast<uint4*>(rm + row * pr + pc * EPP) = M::pack(x);
        if (tr) {
          const uint4 yt = M::pack(y);
          Elt* t0 = tr + pc * EPP * pt + M::tpos(row);
#pragma unroll
          for (int e = 0; e < EPP; ++e) t0[e * pt] = M::elt(yt, e);
        }
      }
    }
  }
};

// The fragments of one own row (position pos of the head), times `scale`: fragment m holds channels
// KF m + EPL hh .. + EPL - 1.  A row outside [lo, pend) gives zeros, and so do channels past d.
template <int DP, class T>
__device__ __forceinline__ void load_own_frags(const HeadRows<const T>& hr, int pos, int pend, int d, int hh, float scale,
                                               typename Mma<T>::Frag (&f)[DP / Mma<T>::KF]) {
  using M = Mma<T>;
  const bool live = pos >= hr.lo && pos < pend;
  const int ps = max(pos < pend ? pos : pend - 1, hr.lo);
  const T* row = hr.base + (unsigned)ps * hr.pitch;
#pragma unroll
  for (int m = 0; m < DP / M::KF; ++m) {
    const int ch = M::KF * m + M::EPL * hh;
    const bool ok = live && ch < d;
    const uint4 t = *reinterpret_cast<const uint4*>(row + (ok ? ch : 0));
    float x[M::EPL];
    M::unpack(t, x);
#pragma unroll
    for (int e = 0; e < M::EPL; ++e) x[e] = ok ? x[e] * scale : 0.f;
    f[m] = __builtin_bit_cast(typename M::Frag, M::pack(x));
  }
}

// The own-row fragments of g = grad_out / den for position pos, and c = grad_out . out / den of that row (the lane
// half's channels summed with the other half's): what a separate pass over grad_out and out would leave in memory.
template <int DP, class T>
__device__ __forceinline__ float load_g_frags_and_c(const HeadRows<const T>& gr, const HeadRows<const T>& orow, int pos,
                                                    int pend, int d, int hh, float rden,
                                                    typename Mma<T>::Frag (&f)[DP / Mma<T>::KF]) {
  using M = Mma<T>;
  const bool live = pos >= gr.lo && pos < pend;
  const int ps = max(pos < pend ? pos : pend - 1, gr.lo);
  const T* grow = gr.base + (unsigned)ps * gr.pitch;
  const T* orw = orow.base + (unsigned)ps * orow.pitch;
  float dot = 0.f;
#pragma unroll
  for (int m = 0; m < DP / M::KF; ++m) {
    const int ch = M::KF * m + M::EPL * hh;
    const bool ok = live && ch < d;
    const uint4 tg = *reinterpret_cast<const uint4*>(grow + (ok ? ch : 0));
    const uint4 to = *reinterpret_cast<const uint4*>(orw + (ok ? ch : 0));
    float x[M::EPL], y[M::EPL];
    M::unpack(tg, x);
    M::unpack(to, y);
#pragma unroll
    for (int e = 0; e < M::EPL; ++e) {
      dot += ok ? x[e] * y[e] : 0.f;
      x[e] = ok ? x[e] * rden : 0.f;
    }
    f[m] = __builtin_bit_cast(typename M::Frag, M::pack(x));
  }
  return (dot + __shfl_xor(dot, 32, 64)) * rden;
}

// LDS layout shared by the three kernels: NA row-major and NT transposed streamed tiles per buffer, two
// buffers, then `tail` floats.
template <int DP, class T, int BN>
struct Lds {
  using M = Mma<T>;
  static constexpr int PR = DP + M::PAD;   // pitch of row-major tiles (elements)
  static constexpr int PT = BN + M::PAD;   // pitch of transposed tiles
  static constexpr int RM = BN * PR;       // elements of a row-major tile
  static constexpr int TR = DP * PT;       // elements of a transposed tile
  static constexpr size_t bytes(int na, int nt, int tail_floats) {
    return (size_t)2 * (na * RM + nt * TR) * sizeof(typename M::Elt) + (size_t)tail_floats * sizeof(float);
  }
};

template <int DP, class T>
struct Shape {
  static constexpr bool BF = std::is_same<T, bf16_t>::value;
  static constexpr int BN = BF ? 64 : 32;           // streamed rows per stage
  static constexpr int BN_KV = BN;                  // (the dk / dv kernel's; 128 at bf16 d = 64 measured 5 % slower)
  // Own 32-row tiles per wave.  Matrix instructions and everything else a SIMD issues (VALU, LDS reads)
  // take turns rather than overlap on this chip, and with one own tile every matrix instruction needs a
  // 16-byte LDS operand read of its own -- the CU's whole LDS bandwidth; two own tiles share each
  // streamed operand and halve that, at the price of the registers of a second set of accumulators,
  // which for the backward kernels means one resident block per CU.
  // Waves per block.  Staging a stage of streamed rows costs a block the same whatever its size, so the
  // backward kernels, whose stages are the costliest (four staged tiles, one of them rescaled), run eight
  // waves on it where the registers allow two waves per SIMD.
  static constexpr int NW_FWD = (BF && DP == 64) ? 8 : 4;
  static constexpr int NW_DQ = (BF && DP == 64) ? 8 : 4;
  static constexpr int NW_KV = (BF && DP == 64) ? 8 : 4;
  static constexpr int RT_FWD = 1;
  static constexpr int RT_DQ = 1;
  static constexpr int RT_KV = 1;
  // resident blocks per CU each kernel is built for (fp32 operand fragments take twice the registers)
  static constexpr int OCC_FWD = (BF && DP == 64) ? 2 : (BF && DP <= 32) ? 3 : (DP <= 32) ? 2 : 1;
  static constexpr int OCC_DQ = (BF && DP == 64) ? 2 : (DP <= 32) ? 2 : 1;   // (8-wave blocks: one is two waves per SIMD)
  static constexpr int OCC_KV = (BF && DP == 64) ? 1 : (DP <= 32) ? 2 : 1;
};

// ---------------------------------------------------------------------------------------
// p = 1 in linear time on top of the dense tiles ("linear mode").  With f(s) = a0 + a1 s everything a query
// needs from the keys before its chunk is one small state
//     S = sum_j [k_j; 1] (x) [v_j, 1]        (DP + 1) x (DP + 1) floats
// (sum k (x) v, sum k, sum v, the count; reference: example.py:167-193), and the backward pass needs the
// mirror image R = sum_i [q_i; 1] (x) [g_i, c_i] over the queries after a key's chunk.  The sequence is cut
// into chunks of `lchunk` positions; dense_state_kernel forms the state of every chunk alone, a scan over
// the chunks (lin_scan_kernel; unmasked: their plain sum) turns them into what each chunk needs, and
// the three dense kernels start from that state and walk only their own chunk's score tiles.  Cost per
// token: ~lchunk d (tiles) + ~4 d^2 (state), whatever the sequence length, for every head dimension.
// The states are sums over the rows as stored; the normaliser scales ride on the kernels' register-side
// operands and epilogues, as in the tile part, except where a whole block can carry them (below).
//
// A state slot in memory: nblk blocks of DP rows x LD floats -- the DP x DP part sum X (x) Y, times a
// constant the consumer wants folded in (a1; on the query side a1 times the head's query scale), as [x][y]
// ("natural") and / or [y][x] ("transposed"), whichever layouts the consumers read rows of -- then the
// vectors as they are: sum_t e_t X_t, sum_t Y_t, and sum_t e_t.
// ---------------------------------------------------------------------------------------
template <int DP>
struct LinState {
  static constexpr int LD = DP + 4;            // row pitch of a block: rows stay 16-byte aligned
  static constexpr int BLOCK = DP * LD;
  __host__ __device__ static constexpr int64_t floats(int nblk) {
    return ((int64_t)nblk * BLOCK + 2 * DP + 4 + 63) / 64 * 64;
  }
};

// slots of fp32 states, in place: mode 0: slot c = sum of the slots before c; 1: of the slots after c;
// 2: slot 0 = the sum of all.  One launch serves two arrays of states (the key side's and the query side's of a
// backward pass; heads_b = 0: one): grid = (ceil(max slot floats / 1024), heads_a + heads_b), one float4 per thread.
__global__ __launch_bounds__(256) void lin_scan_kernel(float* __restrict__ sa, int64_t ssa, int heads_a, int mode_a,
                                                       float* __restrict__ sb, int64_t ssb, int mode_b, int nslots) {
  const bool first = (int)blockIdx.y < heads_a;
  const int64_t ss = first ? ssa : ssb;
  const int mode = first ? mode_a : mode_b, head = first ? blockIdx.y : blockIdx.y - heads_a;
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (idx >= ss) return;
  float* base = (first ? sa : sb) + (int64_t)head * nslots * ss + idx;
  float4 run = make_float4(0.f, 0.f, 0.f, 0.f);
  // eight slots at a time: their loads are all requested before the first store (a load that had to stay behind
  // a store that may alias it would make the walk one memory round trip per slot)
  for (int s0 = 0; s0 < nslots; s0 += 8) {
    float4 t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int step = s0 + u < nslots ? s0 + u : nslots - 1;
      const int c = mode == 1 ? nslots - 1 - step : step;
      t[u] = *reinterpret_cast<const float4*>(base + c * ss);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (s0 + u < nslots) {
        const int c = mode == 1 ? nslots - 1 - (s0 + u) : s0 + u;
        if (mode != 2) *reinterpret_cast<float4*>(base + c * ss) = run;
        run.x += t[u].x; run.y += t[u].y; run.z += t[u].z; run.w += t[u].w;
      }
    }
  }
  if (mode == 2) *reinterpret_cast<float4*>(base) = run;
}

__device__ __forceinline__ void lin_store4(float* p, const float4& v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void lin_store4(uint16_t* p, const float4& v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf2(v.x, v.y), pack_bf2(v.z, v.w));
}

// One block of a state on its way into LDS as a matrix operand: DP rows of DP elements, pitch DP + PAD.
// Up to eight 16-byte loads per thread are in flight before the first is used.
template <int DP, class T, int NT>
__device__ __forceinline__ void lin_stage_block(const float* __restrict__ g, typename Mma<T>::Elt* l, int tid) {
  using M = Mma<T>;
  constexpr int PS = DP + M::PAD, LD = LinState<DP>::LD, V4 = DP / 4, TOTAL = DP * V4, NV = (TOTAL + NT - 1) / NT;
  constexpr int B = NV < 8 ? NV : 8;
  static_assert(TOTAL % NT == 0, "every thread moves the same number of pieces");
  static_for<(NV + B - 1) / B>([&](auto btag) {
    constexpr int U0 = decltype(btag)::value * B, N = NV - U0 < B ? NV - U0 : B;
    float4 t[N];
#pragma unroll
    for (int u = 0; u < N; ++u) {
      const int idx = tid + (U0 + u) * NT;
      t[u] = *reinterpret_cast<const float4*>(g + (idx / V4) * LD + (idx % V4) * 4);
    }
#pragma unroll
    for (int u = 0; u < N; ++u) {
      const int idx = tid + (U0 + u) * NT;
      lin_store4(l + (idx / V4) * PS + (idx % V4) * 4, t[u]);
    }
  });
}

// t + (own rows x DP, fragments af) . B, where brow is the LDS row that holds output column i's DP
// contraction elements, already offset by the lane half's EPL hh
template <int DP, class T>
__device__ __forceinline__ f16v lin_own_times(const typename Mma<T>::Frag (&af)[DP / Mma<T>::KF],
                                              const typename Mma<T>::Elt* brow, f16v t) {
  using M = Mma<T>;
#pragma unroll
  for (int m0 = 0; m0 < DP / M::KF; m0 += 2) {   // (two operand reads in flight, not all of them: register pressure)
    const typename M::Frag b0 = lds_frag<T>(brow + M::KF * m0), b1 = lds_frag<T>(brow + M::KF * (m0 + 1));
    t = M::mma(af[m0], b0, t);
    t = M::mma(af[m0 + 1], b1, t);
    __builtin_amdgcn_sched_barrier(0);
  }
  return t;
}

// The state of every chunk alone.  With X_t, Y_t the rows at position t of chunk c (Y_t divided by ydiv_t when
// given), e_t = ew_t (1 when not given) and bs = cscale hscale[head] (hscale: 1 when not given):
//   block nat_blk [x][y] = block trn_blk [y][x] = bs sum_t X_t[x] Y_t[y]          (a block index < 0: not written)
//   vectors: [x] = sum_t e_t X_t[x],   [DP + y] = sum_t Y_t[y],   [2 DP] = sum_t e_t
// One launch serves two sets of tensors (the key side and the query side of a backward pass; b.heads = 0: one):
// grid = (a.heads + b.heads, chunks), 256 threads; the (DP / 32)^2 tiles of the x-by-y block are dealt to the four
// waves, and the wave that has column block 0 (row block 0) of a block row (column) also sums that row block's X e
// (column block's Y) from the operand fragments it reads anyway.
template <class T>
struct StateSide {
  Rows<const T> X, Y;
  RowScalars ydiv, ew;
  const float* hscale;
  float cscale;
  float* state;
  int nblk, nat_blk, trn_blk, npos, heads;
};

template <int DP, class T>
__global__ __launch_bounds__(256) void dense_state_kernel(StateSide<T> sa, StateSide<T> sb, int d, int lchunk) {
  using M = Mma<T>;
  using Elt = typename M::Elt;
  using Frag = typename M::Frag;
  using LS = LinState<DP>;
  constexpr int KF = M::KF, EPL = M::EPL, CB = DP / 32, NTL = CB * CB, TPW = (NTL + 3) / 4;
  constexpr int BN = Shape<DP, T>::BN, PT = BN + M::PAD;
  static_assert(256 % BN == 0, "a thread stages the same row of every stage");
  __shared__ __attribute__((aligned(16))) Elt Xt[DP * PT];
  __shared__ __attribute__((aligned(16))) Elt Yt[DP * PT];
  __shared__ __attribute__((aligned(16))) float El[BN];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  const bool first = (int)blockIdx.x < sa.heads;
  const StateSide<T>& sd = first ? sa : sb;
  const int head = first ? blockIdx.x : blockIdx.x - sa.heads, c = blockIdx.y, nch = gridDim.y;
  const HeadRows<const T> Xh = sd.X.head(head), Yh = sd.Y.head(head);
  const RowScalars ydiv = sd.ydiv, ew = sd.ew;
  const float* ydh = ydiv.head(head);
  const float* ewh = ew.head(head);
  const int nblk = sd.nblk, nat_blk = sd.nat_blk, trn_blk = sd.trn_blk, npos = sd.npos;
  const float* hscale = sd.hscale;
  const float cscale = sd.cscale;
  float* state = sd.state;
  const int lo = Xh.lo;
  const int t0 = c * lchunk, t1 = (t0 + lchunk < npos ? t0 + lchunk : npos);

  f16v acc[TPW];
  float xs[TPW], ys[TPW];   // this lane's part of sum e X[rb 32 + i] / sum Y[cb 32 + i] where tile t is the one that sums
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    xs[t] = ys[t] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
  }
  float esum = 0.f;   // threads < BN: sum of e over the positions tb + tid of every stage

  TileRegs<DP, T, BN, 256> xt, yt;
  float ev = 1.0f, em = 0.f;   // e of the position this thread stages, as loaded, and whether the position exists
  auto stage_load = [&](int tb) {
    xt.load(Xh, tb, t1, d, tid);
    yt.load(Yh, tb, t1, d, tid, ydh, ydiv.stride);
    // (every thread, clamped, not predicated, nothing computed from it yet: a wait here would wait for the rows too)
    const int pos = tb + tid % BN;
    if (ewh) ev = ewh[(int64_t)max(pos < t1 ? pos : t1 - 1, lo) * ew.stride];
    em = (pos >= lo && pos < t1) ? 1.0f : 0.f;
  };
  if (t0 < t1) stage_load(t0);
  for (int tb = t0; tb < t1; tb += BN) {
    __syncthreads();   // the previous stage has been read
    xt.store(nullptr, 0, Xt, PT, tid);
    if (ydh) yt.store_scaled(nullptr, 0, 1.0f, Yt, PT, 1.0f, tid);
    else yt.store(nullptr, 0, Yt, PT, tid);
    if (tid < BN) {
      const float e = ev * em;
      esum += e;
      El[M::tpos(tid)] = e;   // (same column order as the transposed tiles)
    }
    __syncthreads();
    if (tb + BN < t1) stage_load(tb + BN);   // (the next stage's rows arrive under this stage's tiles)
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const int tile = w + 4 * t;
      if (tile < NTL) {
        const int rb = tile / CB, cb = (tile % CB + rb) % CB;   // (skewed: every wave gets its share of the summing tiles)
#pragma unroll
        for (int f = 0; f < BN / KF; ++f) {
          const Frag a = lds_frag<T>(Xt + (rb * 32 + i) * PT + KF * f + EPL * hh);
          const Frag b = lds_frag<T>(Yt + (cb * 32 + i) * PT + KF * f + EPL * hh);
          acc[t] = M::mma(a, b, acc[t]);
          if (cb == 0) {
            float x[EPL];
            M::unpack(__builtin_bit_cast(uint4, a), x);
#pragma unroll
            for (int e4 = 0; e4 < EPL; e4 += 4) {
              const float4 ev = *reinterpret_cast<const float4*>(El + KF * f + EPL * hh + e4);
              xs[t] += x[e4] * ev.x + x[e4 + 1] * ev.y + x[e4 + 2] * ev.z + x[e4 + 3] * ev.w;
            }
          }
          if (rb == 0) {
            float y[EPL];
            M::unpack(__builtin_bit_cast(uint4, b), y);
#pragma unroll
            for (int e4 = 0; e4 < EPL; ++e4) ys[t] += y[e4];
          }
        }
      }
    }
  }
  float* st = state + ((int64_t)head * nch + c) * LS::floats(nblk);
  float* vec = st + (int64_t)nblk * LS::BLOCK;
  const float bs = cscale * (hscale ? hscale[head] : 1.0f);
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    const int tile = w + 4 * t;
    if (tile < NTL) {
      const int rb = tile / CB, cb = (tile % CB + rb) % CB;
      if (nat_blk >= 0) {
        float* nb = st + (int64_t)nat_blk * LS::BLOCK;
#pragma unroll
        for (int r = 0; r < 16; ++r) nb[(rb * 32 + trow(r, hh)) * LS::LD + cb * 32 + i] = bs * acc[t][r];
      }
      if (trn_blk >= 0) {   // registers 4 j .. 4 j + 3 are four consecutive x
        float* tb = st + (int64_t)trn_blk * LS::BLOCK + (cb * 32 + i) * LS::LD + rb * 32 + 4 * hh;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          *reinterpret_cast<float4*>(tb + 8 * j) =
              make_float4(bs * acc[t][4 * j], bs * acc[t][4 * j + 1], bs * acc[t][4 * j + 2], bs * acc[t][4 * j + 3]);
      }
      const float xsum = xs[t] + __shfl_xor(xs[t], 32, 64), ysum = ys[t] + __shfl_xor(ys[t], 32, 64);
      if (cb == 0 && hh == 0) vec[rb * 32 + i] = xsum;
      if (rb == 0 && hh == 0) vec[DP + cb * 32 + i] = ysum;
    }
  }
  if (w == 0) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) esum += __shfl_xor(esum, off, 64);
    if (tid == 0) vec[2 * DP] = esum;
  }
}

// ---------------------------------------------------------------------------------------
// Forward.  grid = (heads, query blocks of 128 RT positions from the one that holds position Q.lo).
// npos: positions of the queries end here (nk under the mask: query i sits at position i + nk - nq).
// ---------------------------------------------------------------------------------------
template <int DP, class T, int RT, int BN, int NW>
__global__ __launch_bounds__(64 * NW, (Shape<DP, T>::OCC_FWD)) void dense_fwd_kernel(
    Rows<const T> Q, Rows<const T> K, Rows<const T> V, const float* __restrict__ qscale,
    const float* __restrict__ kscale, Rows<T> O, RowScalarsOut den, int npos, int nk, int d, int masked, float a0,
    float a1, float a2, int ratio, const float* __restrict__ lstate, int lchunk, int lslots) {
  using M = Mma<T>;
  using Elt = typename M::Elt;
  using Frag = typename M::Frag;
  using L = Lds<DP, T, BN>;
  constexpr int KF = M::KF, EPL = M::EPL, NF = DP / KF, CB = DP / 32, NFA = 32 / KF, NT = 64 * NW, BM = 32 * RT * NW;
  constexpr int HC = (Shape<DP, T>::BF && NF % 4 == 0) ? 4 : 2;   // operand fragments read ahead at a time
  static_assert(NF % HC == 0, "whole groups of fragments");
  constexpr int PR = L::PR, PT = L::PT;
  static_assert(L::bytes(1, 1, 0) >= (size_t)DP * (DP + M::PAD) * sizeof(Elt) + 2 * DP * sizeof(float), "a state fits the stage buffers");
  extern __shared__ __attribute__((aligned(16))) unsigned char dense_smem[];
  Elt* Kl = reinterpret_cast<Elt*>(dense_smem);   // [2][BN][PR]
  Elt* Vt = Kl + 2 * L::RM;                       // [2][DP][PT]
  float* denl = reinterpret_cast<float*>(Vt + 2 * L::TR);   // [BM]

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  // grid = (heads, row blocks): blocks are dispatched head-fastest, so under the mask the row blocks with
  // the most keys to walk start first for every head, and (workgroups go round-robin to the 8 XCDs) the
  // blocks of a head meet in one XCD's L2 whenever the head count is a multiple of 8
  const int nb = gridDim.y, bx = blockIdx.y;
  const int head = blockIdx.x, hkv = head / ratio;
  const int tok0 = (Q.lo / BM + (masked ? nb - 1 - bx : bx)) * BM;
  const HeadRows<const T> Qh = Q.head(head), Kh = K.head(hkv), Vh = V.head(hkv);
  const float kq = qscale[head] * kscale[hkv];

  Frag qf[RT][NF];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) load_own_frags<DP, T>(Qh, tok0 + (w * RT + rt) * 32 + i, npos, d, hh, kq, qf[rt]);

  const int kend = masked ? (tok0 + BM < nk ? tok0 + BM : nk) : nk;
  const int nst = (kend + BN - 1) / BN;
  // linear mode: the keys before the block's chunk (unmasked: all keys) come as a state
  const int lc = (lstate && masked) ? tok0 / lchunk : 0;
  const int st0 = lstate ? (masked ? lc * (lchunk / BN) : nst) : 0;
  TileRegs<DP, T, BN, NT> kt, vt;
  auto stage_load = [&](int st) {
    kt.load(Kh, st * BN, nk, d, tid);
    vt.load(Vh, st * BN, nk, d, tid);
  };
  auto stage_store = [&](int buf) {
    kt.store(Kl + buf * L::RM, PR, nullptr, 0, tid);
    vt.store(nullptr, 0, Vt + buf * L::TR, PT, tid);
  };

  f16v acc[RT][CB];
  float dn[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    dn[rt] = 0.f;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][cb][r] = 0.f;
  }

  if (st0 < nst) stage_load(st0);   // (requested before the state is: one memory latency, not two)
  if (lstate && (!masked || lc > 0)) {
    // o += a1 qh . S1 + a0 sum v,  den += a1 qh . sum k + a0 count   (S1 = sum k (x) v of the keys in the state)
    constexpr int PS = DP + M::PAD;
    Elt* St = reinterpret_cast<Elt*>(dense_smem);             // a1 S1 as [value channel][key channel]
    float* sk = reinterpret_cast<float*>(St + DP * PS);       // sum k
    float* sv = sk + DP;                                      // sum v
    const float* sp = lstate + ((int64_t)hkv * lslots + lc) * LinState<DP>::floats(1);   // (one block: transposed)
    lin_stage_block<DP, T, NT>(sp, St, tid);
    for (int idx = tid; idx < 2 * DP; idx += NT) sk[idx] = sp[LinState<DP>::BLOCK + idx];
    __syncthreads();
    const int before = masked ? lc * lchunk : nk;
    const float cnt = (float)(before < nk ? before : nk);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const float z = a0 * sv[cb * 32 + i];
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rt][cb][r] = z;
        acc[rt][cb] = lin_own_times<DP, T>(qf[rt], St + (cb * 32 + i) * PS + EPL * hh, acc[rt][cb]);
      }
      float dd = 0.f;
#pragma unroll
      for (int m = 0; m < NF; ++m) {
        float x[EPL];
        M::unpack(__builtin_bit_cast(uint4, qf[rt][m]), x);
#pragma unroll
        for (int e = 0; e < EPL; ++e) dd += x[e] * sk[KF * m + EPL * hh + e];
      }
      dn[rt] = a1 * dd + (hh == 0 ? a0 * cnt : 0.f);
    }
    __syncthreads();
  }

  // One 32-key tile against the wave's own tiles, as straight-line code.  rel = key tile base - first
  // position of own tile 0 (a multiple of 32; masked only): own tile rt has the key tile on its diagonal
  // when rel == 32 rt and wholly after its queries when rel > 32 rt (its weights are then zeroed; this
  // happens once per wave, and one code path keeps the accumulators in place).  tail: (unmasked) the tile
  // holds keys past the end.  Only those tiles pay for per-element tests.
  auto tile = [&](int t32, int kb, int rel, bool tail, const Elt* kl, const Elt* vl) __attribute__((always_inline)) {
    // (the value fragments are requested first: they arrive under the score tile's work)
    Frag vb[NFA][CB];
#pragma unroll
    for (int f = 0; f < NFA; ++f)
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) vb[f][cb] = lds_frag<T>(vl + (cb * 32 + i) * PT + t32 * 32 + KF * f + EPL * hh);
    // scores, transposed: rows = keys trow(r, hh), lanes = own queries
    f16v sc[RT];
#pragma unroll
    for (int m0 = 0; m0 < NF; m0 += HC) {   // (HC operand fragments are read ahead of the instructions that use them)
      Frag ka[HC];
#pragma unroll
      for (int m = 0; m < HC; ++m) ka[m] = lds_frag<T>(kl + (t32 * 32 + i) * PR + KF * (m0 + m) + EPL * hh);
#pragma unroll
      for (int m = 0; m < HC; ++m)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) sc[rt] = M::mma(ka[m], qf[rt][m0 + m], m0 + m == 0 ? kZero16 : sc[rt]);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float s = sc[rt][r];
        sc[rt][r] = a0 + s * (a1 + a2 * s);
      }
      if (masked && rel >= 32 * rt) {   // (wave-uniform) a key may not lie after the query
        FM_KEEP_BRANCH();
        const int lim = rel > 32 * rt ? -1 : i;
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (trow(r, hh) > lim) sc[rt][r] = 0.f;
      }
      if (tail) {   // (wave-uniform) keys past the end
        FM_KEEP_BRANCH();
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (kb + trow(r, hh) >= nk) sc[rt][r] = 0.f;
      }
    }
    // own rows x channels += f(scores) (own x keys) . V (keys x channels)
    static_for<NFA>([&](auto ftag) {
      constexpr int F = decltype(ftag)::value;
      Frag wa[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        wa[rt] = M::template from_acc<F>(sc[rt]);
        dn[rt] = M::fsum(wa[rt], dn[rt]);
      }
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt][cb] = M::mma(wa[rt], vb[F][cb], acc[rt][cb]);
    });
  };

  if (st0 < nst) stage_store(0);
  __syncthreads();
  const int q00 = tok0 + w * RT * 32;   // first position of the wave's own tile 0
  for (int st = st0; st < nst; ++st) {
    const int buf = (st - st0) & 1;
    if (st + 1 < nst) stage_load(st + 1);
    const Elt* kl = Kl + buf * L::RM;
    const Elt* vl = Vt + buf * L::TR;
#pragma unroll 1
    for (int t32 = 0; t32 < BN / 32; ++t32) {
      __builtin_amdgcn_sched_barrier(0);   // (tiles are not interleaved: register pressure)
      const int kb = st * BN + t32 * 32;
      if (kb >= kend) continue;
      if (masked && kb > q00 + 32 * (RT - 1)) continue;   // after every own query
      tile(t32, kb, kb - q00, !masked && kb + 32 > nk, kl, vl);
    }
    if (st + 1 < nst) stage_store(buf ^ 1);
    __syncthreads();
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float tot = dn[rt] + __shfl_xor(dn[rt], 32, 64);
    if (hh == 0) denl[(w * RT + rt) * 32 + i] = tot;
  }
  __syncthreads();
  const HeadRows<T> Oh = O.head(head);
  float* denh = den.head(head);
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = (w * RT + rt) * 32 + trow(r, hh), pos = tok0 + row;
      if (pos < npos && pos >= Qh.lo) {
        const float dsum = denl[row], inv = 1.0f / dsum;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
          if (cb * 32 + i < d) Oh.base[(unsigned)pos * Oh.pitch + (unsigned)(cb * 32 + i)] = from_f32<T>(acc[rt][cb][r] * inv);
        if (i == 0) denh[(int64_t)pos * den.stride] = dsum;
      }
    }
}

// ---------------------------------------------------------------------------------------
// dq.  Same walk as the forward pass; the own rows carry q (times 2 a2, so that the score accumulator,
// started at a1, is f'(s)) and g = grad_out / den.  rpart[head * gridDim.y + block] receives the block's
// sum of dqh . qh for the normalisation chain rule (when rpart is given).  cprep given: c is not read from cvec
// but formed from OUTF, the forward output, and written to cprep (the same array) for the kernel that runs after
// this one.
// ---------------------------------------------------------------------------------------
template <int DP, class T, int RT, int BN, int NW>
__global__ __launch_bounds__(64 * NW, (Shape<DP, T>::OCC_DQ)) void dense_dq_kernel(
    Rows<const T> Q, Rows<const T> GO, RowScalars den, RowScalars cvec, Rows<const T> K, Rows<const T> V,
    const float* __restrict__ qscale, const float* __restrict__ kscale, Rows<T> DQ, float* __restrict__ rpart,
    int npos, int nk, int d, int masked, int p2, float a1, float a2, int ratio, const float* __restrict__ lstate,
    int lchunk, int lslots, Rows<const T> OUTF, RowScalarsOut cprep) {
  using M = Mma<T>;
  using Elt = typename M::Elt;
  using Frag = typename M::Frag;
  using L = Lds<DP, T, BN>;
  constexpr int KF = M::KF, EPL = M::EPL, NF = DP / KF, CB = DP / 32, NFA = 32 / KF, NT = 64 * NW, BM = 32 * RT * NW;
  constexpr int HC = (Shape<DP, T>::BF && NF % 4 == 0) ? 4 : 2;   // operand fragments read ahead at a time
  static_assert(NF % HC == 0, "whole groups of fragments");
  constexpr int PR = L::PR, PT = L::PT;
  static_assert(L::bytes(2, 1, 0) >= (size_t)DP * (DP + M::PAD) * sizeof(Elt) + DP * sizeof(float), "a state fits the stage buffers");
  extern __shared__ __attribute__((aligned(16))) unsigned char dense_smem[];
  Elt* Kl = reinterpret_cast<Elt*>(dense_smem);   // [2][BN][PR]
  Elt* Vl = Kl + 2 * L::RM;                       // [2][BN][PR]
  Elt* Kt = Vl + 2 * L::RM;                       // [2][DP][PT]
  float* red = reinterpret_cast<float*>(Kt + 2 * L::TR);   // [NW]

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  const int nb = gridDim.y, bx = blockIdx.y;   // (heads, row blocks), as in the forward kernel
  const int head = blockIdx.x, hkv = head / ratio;
  const int tok0 = (Q.lo / BM + (masked ? nb - 1 - bx : bx)) * BM;
  const HeadRows<const T> Qh = Q.head(head), Gh = GO.head(head), Kh = K.head(hkv), Vh = V.head(hkv);
  const float* denh = den.head(head);
  const float* ch = cvec.head(head);
  float* cw = cprep.head(head);
  const float kq = qscale[head] * kscale[hkv];

  Frag qf[RT][NF], gf[RT][NF];
  float cown[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int pos = tok0 + (w * RT + rt) * 32 + i;
    const bool live = pos >= Qh.lo && pos < npos;
    const int ps = max(pos < npos ? pos : npos - 1, Qh.lo);
    // (clamped loads whose values are used whatever `live` says: the compiler moves a load that only one side of a
    // select uses under that condition, where it gets a wait of its own -- for every load issued before it)
    const float dnv = denh[(int64_t)ps * den.stride], lm = live ? 1.0f : 0.f;
    const float rden = lm / dnv;
    if (p2) load_own_frags<DP, T>(Qh, pos, npos, d, hh, kq * 2.0f * a2, qf[rt]);
    if (cw) {   // (block-uniform)
      // c_i = grad_out_i . out_i / den_i is formed here from rows the block reads anyway (plus those of out) and left
      // in cvec for the dk / dv kernel: no separate pass over grad_out and out
      cown[rt] = load_g_frags_and_c<DP, T>(Gh, OUTF.head(head), pos, npos, d, hh, rden, gf[rt]);
      if (live && hh == 0) cw[(int64_t)pos * cprep.stride] = cown[rt];
    } else {
      cown[rt] = lm * ch[(int64_t)ps * cvec.stride];
      load_own_frags<DP, T>(Gh, pos, npos, d, hh, rden, gf[rt]);
    }
  }

  const int kend = masked ? (tok0 + BM < nk ? tok0 + BM : nk) : nk;
  const int nst = (kend + BN - 1) / BN;
  const int lc = (lstate && masked) ? tok0 / lchunk : 0;   // (linear mode, as in the forward kernel)
  const int st0 = lstate ? (masked ? lc * (lchunk / BN) : nst) : 0;
  TileRegs<DP, T, BN, NT> kt, vt;
  auto stage_load = [&](int st) {
    kt.load(Kh, st * BN, nk, d, tid);
    vt.load(Vh, st * BN, nk, d, tid);
  };
  auto stage_store = [&](int buf) {
    kt.store(Kl + buf * L::RM, PR, Kt + buf * L::TR, PT, tid);
    vt.store(Vl + buf * L::RM, PR, nullptr, 0, tid);
  };

  f16v acc[RT][CB];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][cb][r] = 0.f;

  if (st0 < nst) stage_load(st0);   // (requested before the state is: one memory latency, not two)
  if (lstate && (!masked || lc > 0)) {
    // sum_j a1 (g . v_j - c) k_j over the keys in the state = a1 (g . S1^T - c sum k)
    constexpr int PS = DP + M::PAD;
    Elt* Sn = reinterpret_cast<Elt*>(dense_smem);             // a1 S1 as [key channel][value channel]
    float* sk = reinterpret_cast<float*>(Sn + DP * PS);       // sum k
    const float* sp = lstate + ((int64_t)hkv * lslots + lc) * LinState<DP>::floats(1);   // (one block: natural)
    lin_stage_block<DP, T, NT>(sp, Sn, tid);
    for (int idx = tid; idx < DP; idx += NT) sk[idx] = sp[LinState<DP>::BLOCK + idx];
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float crow[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int pos = tok0 + (w * RT + rt) * 32 + trow(r, hh);
        const float cvv = ch[(int64_t)max(pos < npos ? pos : npos - 1, Qh.lo) * cvec.stride];   // (clamped, not predicated)
        crow[r] = -a1 * cvv * ((pos >= Qh.lo && pos < npos) ? 1.0f : 0.f);
      }
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const float z = sk[cb * 32 + i];
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rt][cb][r] = crow[r] * z;
        acc[rt][cb] = lin_own_times<DP, T>(gf[rt], Sn + (cb * 32 + i) * PS + EPL * hh, acc[rt][cb]);
      }
    }
    __syncthreads();
  }

  // (rel as in the forward kernel: own tile rt has the key tile on its diagonal when rel == 32 rt and
  // wholly after its queries when rel > 32 rt)
  auto tile = [&](int t32, int rel, const Elt* kl, const Elt* vl, const Elt* ktl) __attribute__((always_inline)) {
    // transposed tiles (rows = keys, lanes = own queries): f'(s) and g . v - c
    f16v sc[RT], pt[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sc[rt][r] = a1;
        pt[rt][r] = -cown[rt];
      }
#pragma unroll
    for (int m0 = 0; m0 < NF; m0 += HC) {
      Frag va[HC], ka[HC];
#pragma unroll
      for (int m = 0; m < HC; ++m) {
        va[m] = lds_frag<T>(vl + (t32 * 32 + i) * PR + KF * (m0 + m) + EPL * hh);
        if (p2) ka[m] = lds_frag<T>(kl + (t32 * 32 + i) * PR + KF * (m0 + m) + EPL * hh);
      }
#pragma unroll
      for (int m = 0; m < HC; ++m)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          pt[rt] = M::mma(va[m], gf[rt][m0 + m], pt[rt]);
          if (p2) sc[rt] = M::mma(ka[m], qf[rt][m0 + m], sc[rt]);
        }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) pt[rt][r] = sc[rt][r] * pt[rt][r];
      if (masked && rel >= 32 * rt) {   // (wave-uniform) a key may not lie after the query
        FM_KEEP_BRANCH();
        const int lim = rel > 32 * rt ? -1 : i;
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (trow(r, hh) > lim) pt[rt][r] = 0.f;
      }
    }
    // own rows x channels += W (own x keys) . K (keys x channels)
    static_for<NFA>([&](auto ftag) {
      constexpr int F = decltype(ftag)::value;
      Frag kb_[CB], wa[RT];
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) kb_[cb] = lds_frag<T>(ktl + (cb * 32 + i) * PT + t32 * 32 + KF * F + EPL * hh);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) wa[rt] = M::template from_acc<F>(pt[rt]);
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt][cb] = M::mma(wa[rt], kb_[cb], acc[rt][cb]);
    });
  };

  if (st0 < nst) stage_store(0);
  __syncthreads();
  const int q00 = tok0 + w * RT * 32;
  for (int st = st0; st < nst; ++st) {
    const int buf = (st - st0) & 1;
    if (st + 1 < nst) stage_load(st + 1);
    const Elt* kl = Kl + buf * L::RM;
    const Elt* vl = Vl + buf * L::RM;
    const Elt* ktl = Kt + buf * L::TR;
#pragma unroll 1
    for (int t32 = 0; t32 < BN / 32; ++t32) {
      __builtin_amdgcn_sched_barrier(0);   // (tiles are not interleaved: register pressure)
      const int kb = st * BN + t32 * 32;
      if (kb >= kend) continue;
      if (masked && kb > q00 + 32 * (RT - 1)) continue;   // after every own query
      tile(t32, kb - q00, kl, vl, ktl);
    }
    if (st + 1 < nst) stage_store(buf ^ 1);
    __syncthreads();
  }

  // dq = qs ks acc (the keys went in unscaled); sum of dqh . qh = qs ks sum acc . q
  const HeadRows<T> Dh = DQ.head(head);
  float rs = 0.f;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    // (the q elements are all requested before the first store: a load that had to stay behind a store that
    // may alias it would cost one memory round trip per element)
    float qv[CB][16];
    if (rpart) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int pos = tok0 + (w * RT + rt) * 32 + trow(r, hh);
        const int ps = max(pos < npos ? pos : npos - 1, Qh.lo);   // (clamped, not predicated: predicated loads get a wait each)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
          qv[cb][r] = to_f32(Qh.base[(unsigned)ps * Qh.pitch + (unsigned)(cb * 32 + i < d ? cb * 32 + i : 0)]);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int pos = tok0 + (w * RT + rt) * 32 + trow(r, hh);
      if (pos < npos && pos >= Qh.lo) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
          const int c = cb * 32 + i;
          if (c < d) {
            const float v = acc[rt][cb][r] * kq;
            Dh.base[(unsigned)pos * Dh.pitch + (unsigned)c] = from_f32<T>(v);
            if (rpart) rs += v * qv[cb][r];
          }
        }
      }
    }
  }
  if (rpart) {
    rs = block_sum<NW>(rs, red, tid);
    if (tid == 0) rpart[(int64_t)head * nb + bx] = rs;
  }
}

// ---------------------------------------------------------------------------------------
// dk and dv.  grid = (key/value heads, key blocks of 128 RT positions); the own rows are keys, the
// streamed rows the queries at or after them (all of them when unmasked) of every query head of the
// group in turn.  Score tiles have rows = queries, lanes = own keys.  The streamed g rows go to LDS
// twice: times qs / den row-major (so that W comes out times qs, the factor of qh in dkh = sum W qh) and
// times 1 / den transposed (the B operand of dv).  rpart[kvhead * gridDim.y + block] = sum dkh . kh.
// ---------------------------------------------------------------------------------------
template <int DP, class T, int RT, int BN, int NW>
__global__ __launch_bounds__(64 * NW, (Shape<DP, T>::OCC_KV)) void dense_dkdv_kernel(
    Rows<const T> K, Rows<const T> V, Rows<const T> Q, Rows<const T> GO, RowScalars den, RowScalars cvec,
    const float* __restrict__ qscale, const float* __restrict__ kscale, Rows<T> DK, Rows<T> DV,
    float* __restrict__ rpart, int npos, int nk, int d, int masked, float a0, float a1, float a2, int ratio,
    const float* __restrict__ lstate, int lchunk, int lslots) {
  using M = Mma<T>;
  using Elt = typename M::Elt;
  using Frag = typename M::Frag;
  using L = Lds<DP, T, BN>;
  constexpr int KF = M::KF, EPL = M::EPL, NF = DP / KF, CB = DP / 32, NFA = 32 / KF, NT = 64 * NW, BM = 32 * RT * NW;
  constexpr int HC = (Shape<DP, T>::BF && NF % 4 == 0) ? 4 : 2;   // operand fragments read ahead at a time
  static_assert(NF % HC == 0, "whole groups of fragments");
  constexpr int PR = L::PR, PT = L::PT;
  static_assert(L::bytes(2, 2, 0) >= (size_t)2 * DP * (DP + M::PAD) * sizeof(Elt) + 2 * DP * sizeof(float), "a state fits the stage buffers");
  extern __shared__ __attribute__((aligned(16))) unsigned char dense_smem[];
  Elt* Ql = reinterpret_cast<Elt*>(dense_smem);   // [2][BN][PR]
  Elt* Gl = Ql + 2 * L::RM;                       // [2][BN][PR]
  Elt* Qt = Gl + 2 * L::RM;                       // [2][DP][PT]
  Elt* Gt = Qt + 2 * L::TR;                       // [2][DP][PT]
  float* Cl = reinterpret_cast<float*>(Gt + 2 * L::TR);   // [2][BN]: -qs c of the streamed queries
  float* red = Cl + 2 * BN;                       // [NW]

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, i = l & 31, hh = l >> 5;
  const int nb = gridDim.y, bx = blockIdx.y;   // (key/value heads, key blocks)
  const int hkv = blockIdx.x;
  const int tok0 = bx * BM;   // (under the mask the first key blocks see the most queries: already first)
  const HeadRows<const T> Kh = K.head(hkv), Vh = V.head(hkv);
  const float ks = kscale[hkv];

  Frag kf[RT][NF], vf[RT][NF];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int pos = tok0 + (w * RT + rt) * 32 + i;
    load_own_frags<DP, T>(Kh, pos, nk, d, hh, ks, kf[rt]);
    load_own_frags<DP, T>(Vh, pos, nk, d, hh, 1.0f, vf[rt]);
  }
  f16v dk[RT][CB], dv[RT][CB];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int r = 0; r < 16; ++r) dk[rt][cb][r] = dv[rt][cb][r] = 0.f;

  float dvc[CB], dkc[CB];   // (linear mode) what every own row's dv / dk gets on top, per channel cb * 32 + i
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) dvc[cb] = dkc[cb] = 0.f;
  TileRegs<DP, T, BN, NT> qt, gt;
  float creg = 0.f, cmask = 0.f;
  for (int hq = 0; hq < ratio; ++hq) {
    const int head = hkv * ratio + hq;
    const HeadRows<const T> Qh = Q.head(head), Gh = GO.head(head);
    const float* denh = den.head(head);
    const float* ch = cvec.head(head);
    const float qs = qscale[head];
    // f and f' of s = qs sr, where sr = q . kh is what the score tile holds
    const float c2 = a2 * qs * qs, c1 = a1 * qs, b2 = 2.0f * a2 * qs;
    const int lo = Qh.lo;
    // linear mode: the queries after the block's chunk (unmasked: all queries) come as a state
    const int lc = (lstate && masked) ? tok0 / lchunk : 0;
    const int qend = (lstate && masked && (lc + 1) * lchunk < npos) ? (lc + 1) * lchunk : npos;
    const int nst = (qend + BN - 1) / BN;
    const int st0 = lstate && !masked ? nst : masked ? (tok0 > lo ? tok0 : lo) / BN : 0;
    auto stage_load = [&](int st) {
      qt.load(Qh, st * BN, npos, d, tid);
      gt.load(Gh, st * BN, npos, d, tid, denh, den.stride);
      {   // (every thread, clamped, not predicated: a predicated load gets a wait that would also wait for the tiles' loads)
        const int pos = st * BN + tid % BN;
        creg = ch[(int64_t)max(pos < npos ? pos : npos - 1, lo) * cvec.stride];   // (as loaded: nothing here may wait for it)
        cmask = (pos >= lo && pos < npos) ? 1.0f : 0.f;
      }
    };
    auto stage_store = [&](int buf) {
      qt.store(Ql + buf * L::RM, PR, Qt + buf * L::TR, PT, tid);
      gt.store_scaled(Gl + buf * L::RM, PR, qs, Gt + buf * L::TR, PT, 1.0f, tid);
      if (tid < BN) Cl[buf * BN + tid] = -creg * qs * cmask;   // (-qs c: the tile's start value)
    };
    // (requested before the state is -- one memory latency, not two -- where the registers are there: with fp32
    // fragments of 96 or 128 channels the state's own loads would be left with one register set and a wait each)
    constexpr bool EARLY = Shape<DP, T>::BF || DP <= 64;
    if (EARLY && st0 < nst) stage_load(st0);
    if (lstate && (!masked || lc + 1 < lslots)) {
      // dv += a0 sum g + a1 qs kh . R1,  dk += a1 qs (v . R1^T - sum c q)   (R1 = sum q (x) g of the queries in the state);
      // the two sums, the same for every own row, wait in dvc / dkc for the epilogue
      constexpr int PS = DP + M::PAD;
      Elt* Rn = reinterpret_cast<Elt*>(dense_smem);             // a1 qs R1 as [query channel][value channel]
      Elt* Rt = Rn + DP * PS;                                   // and as [value channel][query channel]
      float* rq = reinterpret_cast<float*>(Rt + DP * PS);       // sum c q
      float* rg = rq + DP;                                      // sum g
      const float aq = a1 * qs;
      const float* sp = lstate + ((int64_t)head * lslots + lc) * LinState<DP>::floats(2);   // (two blocks: natural, transposed)
      lin_stage_block<DP, T, NT>(sp, Rn, tid);
      lin_stage_block<DP, T, NT>(sp + LinState<DP>::BLOCK, Rt, tid);
      for (int idx = tid; idx < 2 * DP; idx += NT) rq[idx] = sp[2 * LinState<DP>::BLOCK + idx];
      __syncthreads();
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        dvc[cb] += a0 * rg[cb * 32 + i];
        dkc[cb] -= aq * rq[cb * 32 + i];
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
          dv[rt][cb] = lin_own_times<DP, T>(kf[rt], Rt + (cb * 32 + i) * PS + EPL * hh, dv[rt][cb]);
          dk[rt][cb] = lin_own_times<DP, T>(vf[rt], Rn + (cb * 32 + i) * PS + EPL * hh, dk[rt][cb]);
        }
      __syncthreads();
    }
    if (!EARLY && st0 < nst) stage_load(st0);
    if (st0 < nst) stage_store(0);
    __syncthreads();
    // One 32-query tile against the wave's own key tiles, as straight-line code.  rel = query tile base -
    // first position of own tile 0 (masked only): own tile rt has the query tile on its diagonal when
    // rel == 32 rt and wholly before its keys when rel < 32 rt (its weights are then zeroed).
    auto tile = [&](int t32, int rel, const Elt* ql, const Elt* gl, const Elt* qtl, const Elt* gtl, const float* cl)
                    __attribute__((always_inline)) {
      // tiles with rows = queries trow(r, hh), lanes = own keys: sr and qs (g . v - c)
      f16v sc[RT], pt[RT];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4 c4 = *reinterpret_cast<const float4*>(cl + t32 * 32 + 8 * j + 4 * hh);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          pt[rt][4 * j] = c4.x; pt[rt][4 * j + 1] = c4.y; pt[rt][4 * j + 2] = c4.z; pt[rt][4 * j + 3] = c4.w;
        }
      }
#pragma unroll
      for (int m0 = 0; m0 < NF; m0 += HC) {
        Frag qa[HC], ga[HC];
#pragma unroll
        for (int m = 0; m < HC; ++m) {
          qa[m] = lds_frag<T>(ql + (t32 * 32 + i) * PR + KF * (m0 + m) + EPL * hh);
          ga[m] = lds_frag<T>(gl + (t32 * 32 + i) * PR + KF * (m0 + m) + EPL * hh);
        }
#pragma unroll
        for (int m = 0; m < HC; ++m)
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            sc[rt] = M::mma(qa[m], kf[rt][m0 + m], m0 + m == 0 ? kZero16 : sc[rt]);
            pt[rt] = M::mma(ga[m], vf[rt][m0 + m], pt[rt]);
          }
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float s = sc[rt][r];
          sc[rt][r] = a0 + s * (c1 + c2 * s);
          pt[rt][r] = (a1 + b2 * s) * pt[rt][r];
        }
        if (masked && rel <= 32 * rt) {   // (wave-uniform) a query may not lie before the key
          FM_KEEP_BRANCH();
          const int lim = rel < 32 * rt ? 32 : i;
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (trow(r, hh) < lim) sc[rt][r] = pt[rt][r] = 0.f;
        }
      }
      // own keys x channels: dv += f^T (keys x queries) . g,   dk += W^T . q
      static_for<NFA>([&](auto ftag) {
        constexpr int F = decltype(ftag)::value;
        Frag bg[CB], bq[CB], fa[RT], wa[RT];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
          bg[cb] = lds_frag<T>(gtl + (cb * 32 + i) * PT + t32 * 32 + KF * F + EPL * hh);
          bq[cb] = lds_frag<T>(qtl + (cb * 32 + i) * PT + t32 * 32 + KF * F + EPL * hh);
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          fa[rt] = M::template from_acc<F>(sc[rt]);
          wa[rt] = M::template from_acc<F>(pt[rt]);
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            dv[rt][cb] = M::mma(fa[rt], bg[cb], dv[rt][cb]);
            dk[rt][cb] = M::mma(wa[rt], bq[cb], dk[rt][cb]);
          }
      });
    };
    const int k00 = tok0 + w * RT * 32;   // first position of the wave's own tile 0
    for (int st = st0; st < nst; ++st) {
      const int buf = (st - st0) & 1;
      if (st + 1 < nst) stage_load(st + 1);
      const Elt* ql = Ql + buf * L::RM;
      const Elt* gl = Gl + buf * L::RM;
      const Elt* qtl = Qt + buf * L::TR;
      const Elt* gtl = Gt + buf * L::TR;
      const float* cl = Cl + buf * BN;
#pragma unroll 1
      for (int t32 = 0; t32 < BN / 32; ++t32) {
        __builtin_amdgcn_sched_barrier(0);   // (tiles are not interleaved: register pressure)
        const int qb = st * BN + t32 * 32;
        if (qb >= npos || (masked && qb < k00)) continue;
        tile(t32, qb - k00, ql, gl, qtl, gtl, cl);
      }
      if (st + 1 < nst) stage_store(buf ^ 1);
      __syncthreads();
    }
  }

  // dk = ks dkh (dkh = the accumulated sum); sum of dkh . kh = ks sum acc . k
  const HeadRows<T> DKh = DK.head(hkv), DVh = DV.head(hkv);
  float rs = 0.f;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float kv[CB][16];   // (requested before the first store, as in the dq kernel)
    if (rpart) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int pos = tok0 + (w * RT + rt) * 32 + trow(r, hh);
        const int ps = pos < nk ? pos : nk - 1;   // (clamped, not predicated: predicated loads get a wait each)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
          kv[cb][r] = to_f32(Kh.base[(unsigned)ps * Kh.pitch + (unsigned)(cb * 32 + i < d ? cb * 32 + i : 0)]);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int pos = tok0 + (w * RT + rt) * 32 + trow(r, hh);
      if (pos < nk) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
          const int c = cb * 32 + i;
          if (c < d) {
            const float v = (dk[rt][cb][r] + dkc[cb]) * ks;
            DKh.base[(unsigned)pos * DKh.pitch + (unsigned)c] = from_f32<T>(v);
            DVh.base[(unsigned)pos * DVh.pitch + (unsigned)c] = from_f32<T>(dv[rt][cb][r] + dvc[cb]);
            if (rpart) rs += v * kv[cb][r];
          }
        }
      }
    }
  }
  if (rpart) {
    rs = block_sum<NW>(rs, red, tid);
    if (tid == 0) rpart[(int64_t)hkv * nb + bx] = rs;
  }
}

}  // namespace dense
