// Shared device helpers for the gfx950 Fastmax kernels.
//
// Everything here is written for 64-wide wavefronts and the fp32 matrix instruction
// v_mfma_f32_32x32x2f32.  Operand layouts of that instruction (lane l of the wave):
//   A (32 x 2):  row  l%32, k = l/32         -> one float per lane
//   B (2 x 32):  k = l/32,  col l%32         -> one float per lane
//   D (32 x 32): col  l%32, rows trow(r,l/32) for the 16 accumulator registers r
// Because the reduction index k of an MFMA can be any permutation as long as A and B agree,
// an accumulator register can be fed straight back as the A or B operand of the next
// contraction (k=0/1 then stand for rows trow(r,0)/trow(r,1)); the kernels use that to chain
// score tiles into value/gradient tiles without going through memory.
#pragma once
#include <type_traits>
#include <utility>
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float f16v __attribute__((ext_vector_type(16)));

#define FM_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32((a), (b), (c), 0, 0, 0)

// bf16 matrix instructions (fp32 accumulate).  Operands are built in the k = 8 layout,
//   A (32 x 8): row l%32, k = 4*(l/32) + {0,1,2,3}  -> four bf16 per lane
//   B (8 x 32): col l%32, k = 4*(l/32) + {0,1,2,3}
//   D (32 x 32): as for the fp32 instruction
// where one operand pair replaces four fp32 MFMAs whose k indices were 2*u + l/32, u = 0..3.
typedef __bf16 bf2v __attribute__((ext_vector_type(2)));
// v_mfma_f32_32x32x16_bf16: eight bf16 per lane, k = 8*(l/32) + {0..7}; issues at the rate of
// the k = 8 form (measured ~35 cycles), i.e. twice its throughput.  Because the k index of A and
// B may be permuted together, two k = 8 operand pairs (each the four k-slots of a lane) are
// simply concatenated: slots 0..3 from the first pair, 4..7 from the second.
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
typedef uint32_t fm_u4 __attribute__((ext_vector_type(4)));   // the same 16 bytes as four dwords
#define FM_MFMA_BF16(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16((a), (b), (c), 0, 0, 0)
// wait until at most n vector-memory operations of this wave are outstanding (they complete in
// order), leaving the other counters alone: s_waitcnt simm16 = vmcnt[3:0] | expcnt << 4 |
// lgkmcnt << 8 | vmcnt[5:4] << 14
#define FM_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

__device__ __forceinline__ uint32_t pack_bf2(float lo, float hi) {
  const bf2v p = {(__bf16)lo, (__bf16)hi};  // round to nearest even (v_cvt_pk_bf16_f32)
  return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ bf8v as_bf8(uint2 lo, uint2 hi) {
  const uint4 u = make_uint4(lo.x, lo.y, hi.x, hi.y);
  return __builtin_bit_cast(bf8v, u);
}
// acc + a.lo * b.lo + a.hi * b.hi of two bf16 pairs (v_dot2c_f32_bf16)
typedef __bf16 fm_bf2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float fm_dot2_bf16(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(fm_bf2, a), __builtin_bit_cast(fm_bf2, b), acc, false);
}
__device__ __forceinline__ uint2 pack_bf4u(float a, float b, float c, float d) {
  return make_uint2(pack_bf2(a, b), pack_bf2(c, d));
}
__device__ __forceinline__ float bf_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// The value lane l ^ 32 holds (hh = l / 32): v_permlane32_swap exchanges lanes 32..63 of its first
// operand with lanes 0..31 of its second, so with the same value in both, the first result carries
// the lower half's values in the upper lanes and the second the upper half's in the lower lanes.
// (A ds_bpermute with the address (l ^ 32) * 4 does the same, but a loop of them over the elements of
// a register vector was seen compiled into ONE permute whose result went to every element.)
__device__ __forceinline__ float other_half(float v, int hh) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, hh ? r[0] : r[1]);
}

// For a lane of the lower half: the value `from_upper` holds in lane l + 32; for a lane of the upper
// half: the value `from_lower` holds in lane l - 32 (one v_permlane32_swap serves both directions).
__device__ __forceinline__ float swap_halves(float from_upper, float from_lower, int hh) {
  const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, from_upper),
                                                  __builtin_bit_cast(unsigned, from_lower), false, false);
  return __builtin_bit_cast(float, hh ? r[0] : r[1]);
}

// row of a 32x32 accumulator tile held by register r in lane half hh
__device__ __forceinline__ int trow(int r, int hh) { return 8 * (r >> 2) + 4 * hh + (r & 3); }

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2) in linear block-id
// order.  This permutation makes a run of consecutive LOGICAL ids land on one XCD, in order,
// so that blocks that read the same data (feature splits of a head, the two halves of a chunk)
// share an L2.  The ragged tail (total not a multiple of 8) keeps its place.
__device__ __forceinline__ int xcd_logical_id(int linear, int total) {
  constexpr int NX = 8;
  const int per = total / NX;
  if (linear >= per * NX) return linear;
  return (linear % NX) * per + linear / NX;
}

struct bf16_t {
  uint16_t x;
};

// f(integral_constant<int, 0>), ..., f(integral_constant<int, N-1>): a loop whose index is a
// compile-time constant in every iteration
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v.x) << 16); }

template <class T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) {
  uint32_t u = __float_as_uint(v);
  bf16_t o;
  if ((u & 0x7fffffffu) > 0x7f800000u) {  // NaN stays NaN
    o.x = (uint16_t)((u >> 16) | 0x40);
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
    o.x = (uint16_t)(u >> 16);
  }
  return o;
}

// Transposing 64-bit LDS read of 16-bit elements (gfx950): in every group of 16 lanes, lane L
// receives, for k = 0..3, element L % 4 of the 8-byte word whose address lane 4 k + L / 4 of the
// group supplied.  So if the 16 lanes address a 4 x 4 arrangement of words, word (r, k) by lane
// 4 k + r, lane L gets one element of each word of its row L / 4: a 4 x 4 transpose of 16-bit
// elements between "four lanes x one word" and "one lane x four words".
typedef short fm_v4s __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint2 lds_read_tr16(const uint16_t* p) {
  const fm_v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) fm_v4s*)(const_cast<uint16_t*>(p)));
  return __builtin_bit_cast(uint2, r);
}

// four consecutive elements <-> four floats
__device__ __forceinline__ void load4(const float* p, float (&o)[4]) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float (&o)[4]) {
  const uint2 t = *reinterpret_cast<const uint2*>(p);
  o[0] = __uint_as_float(t.x << 16);
  o[1] = __uint_as_float(t.x & 0xffff0000u);
  o[2] = __uint_as_float(t.y << 16);
  o[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float (&v)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const float (&v)[4]) {
  uint2 t;
  t.x = (uint32_t)from_f32<bf16_t>(v[0]).x | ((uint32_t)from_f32<bf16_t>(v[1]).x << 16);
  t.y = (uint32_t)from_f32<bf16_t>(v[2]).x | ((uint32_t)from_f32<bf16_t>(v[3]).x << 16);
  *reinterpret_cast<uint2*>(p) = t;
}

// Rows of one tensor the way a kernel addresses them.  The tensor is (batch, group, head within the
// group, token, channel) with unit channel stride: head h of the tensor, counted over all batch
// elements, starts at
//     p + (h / (ng nh)) sb + ((h / nh) % ng) sg + (h % nh) sh
// and consecutive tokens are `pitch` elements apart.  A contiguous (heads, tokens, D) tensor has
// ng = nh = 1 and sb = tokens * D.  Token positions below `lo` have no row (a key prefix: query-side
// tensors start at position nk - nq); the host moves p back by lo * pitch, so position t >= lo is
// at head(h) + t * pitch like everywhere else, and loads clamp their position to [lo, n).  h0 is
// added to the head index a kernel derives from its block index (head batches).
// (the rows of one head span less than 4 GiB -- the host checks it -- so a row's offset from the
// head's base fits 32 bits: uniform 64-bit base + 32-bit lane offset is the cheapest address form)
template <class T>
struct HeadRows {
  T* base;
  unsigned pitch;
  int lo;
  __device__ __forceinline__ T* row(int tok) const { return base + (unsigned)tok * pitch; }
};
template <class T>
struct Rows {
  T* p;
  int64_t sb, sg, sh, pitch;
  int ng, nh, h0, lo;
  __device__ __forceinline__ HeadRows<T> head(int h) const {
    h += h0;
    if (ng == 1 && nh == 1) return HeadRows<T>{p + (int64_t)h * sb, (unsigned)pitch, lo};   // one level (no divisions)
    const int gb = h / nh, j = h - gb * nh, b = gb / ng, g = gb - b * ng;
    return HeadRows<T>{p + ((int64_t)b * sb + (int64_t)g * sg + (int64_t)j * sh), (unsigned)pitch, lo};
  }
};
// One float per (head, token): den, c.  Head h starts at p + h * hs, tokens are `stride` apart;
// like Rows, p is moved back by lo * stride when positions start at lo.
template <class F>
struct RowScalarsT {
  F* p;
  int64_t hs, stride;
  __device__ __forceinline__ F* head(int h) const { return p ? p + (int64_t)h * hs : nullptr; }
};
using RowScalars = RowScalarsT<const float>;
using RowScalarsOut = RowScalarsT<float>;

// Geometry of the symmetric moment state for head dimension D.
//
// The order-2 feature of a vector x is stored once per unordered channel pair, indexed by
// (shift s, channel a) -> x[a] * x[(a+s) mod D], s = 0..D/2.  Shifts 1..D/2-1 carry every
// pair {a, a+s} exactly once (weight 2 in a full contraction); s = 0 is the diagonal and
// s = D/2 lists each pair twice (weight 1 each).  Rows of a state, each LD = D+4 floats
// (D value columns, the "extra" column that carries the denominator moments, 3 of padding):
//   [0, NS*D)            order 2, row s*D + a        (absent when p == 1)
//   [.., +D)             order 1, row a
//   last row             order 0
template <int D>
struct Geo {
  static constexpr int NS = D / 2 + 1;
  static constexpr int AB = D / 32;  // 32-row blocks per shift
  static constexpr int CB = D / 32;  // 32-column blocks of the value dimension
  static constexpr int LD = D + 4;   // row pitch of states and of every LDS tile: column D is the
                                     // extra column, D+1..D+3 pad the row to 16 bytes so that
                                     // row-strided accesses can be 128-bit and bank-conflict-free
  static constexpr int H2 = D / 2;   // channels handled by each lane half per MFMA sweep
  __host__ __device__ static constexpr int rows2(int p2) { return p2 ? NS * D : 0; }
  __host__ __device__ static constexpr int rows(int p2) { return rows2(p2) + D + 1; }
  __host__ __device__ static constexpr int64_t state_floats(int p2) {
    return ((int64_t)rows(p2) * LD + 63) / 64 * 64;
  }
  // floats of one LDS stage buffer: a state slab of D(+1) rows or a pair of 32-row tiles
  static constexpr int SLAB = ((D + 1) * LD > 2 * 32 * LD ? (D + 1) * LD : 2 * 32 * LD) + 3;
  static constexpr int SLABF = (SLAB + 3) / 4 * 4;
};

// Packed bf16 form of a state, used when the inputs are bf16 (it occupies the front of the same
// state_floats slot as the fp32 form).  A "slab" is the D feature rows of one shift s (order 2;
// rows carry their pair weight: x2 for 0 < s < D/2) or the D order-1 rows (slab NS, or slab 0
// when p == 1), stored feature-packed,
//   [a/8][column 0..D+3][a%8]
// i.e. 16-byte words of eight consecutive rows, which is the B operand of the bf16 matrix
// instruction for a contraction over features (apply kernels: one 128-bit LDS read per operand);
// for a contraction over columns (grad kernels) the two 8-byte halves of the words are read through
// the transposing LDS load (lds_read_tr16).  Consumers stage a slab with plain 16-byte copies.
// Columns D..D+3 hold the extra (denominator) column split into hi + lo bf16 parts as
// (hi, hi, lo, lo), because in the grad kernels that term nearly cancels the value columns' sum.
// The slabs are followed by the order-0 row as D+1 floats.
template <int D>
struct PackedGeo {
  using G = Geo<D>;
  static constexpr int NCF = D + 4;
  static constexpr int FSL = (D / 8) * NCF * 8;  // bf16 elements of a slab (a multiple of 128)
  __host__ __device__ static constexpr int nslab(int p2) { return (p2 ? G::NS : 0) + 1; }
  __host__ __device__ static constexpr int64_t z_off(int p2) { return ((int64_t)nslab(p2) * FSL * 2 + 255) / 256 * 256; }
  __host__ __device__ static constexpr int64_t bytes(int p2) { return z_off(p2) + (D + 1) * 4; }
  // floats between the packed states of consecutive slots (causal scans only: an unmasked state
  // sits in the last of the fp32 slots its partial sums were built in)
  __host__ __device__ static constexpr int64_t slot_floats(int p2) { return (bytes(p2) + 255) / 256 * 64; }
  static_assert(bytes(1) <= G::state_floats(1) * 4 && bytes(0) <= G::state_floats(0) * 4,
                "the packed form must fit the fp32 state slot");
};

// A tile of ROWS token rows x D channels staged global -> registers -> LDS by 256 threads.
// ROWFAST = false: consecutive threads take consecutive 16-byte pieces of a row (coalesced
// global reads, conflict-free row-major LDS writes).  ROWFAST = true: consecutive threads
// take consecutive rows, which makes the TRANSPOSED LDS write (store_t) conflict-free.
template <int D, class T, int ROWS, bool ROWFAST = false>
struct RowTile {
  static constexpr int VPR = D / 4;
  static constexpr int TOTAL = ROWS * VPR;
  static constexpr int NV = (TOTAL + 255) / 256;
  // The pieces stay as loaded (and the divisors unread) until a store converts, masks and scales
  // them: nothing in load() consumes what it fetches, and it has no branch, so the loads of a
  // tile can stay in flight under whatever work separates load() from the store.
  using Raw = typename std::conditional<std::is_same<T, float>::value, float4, uint2>::type;
  Raw raw[NV];
  float rdiv[NV];  // per-row divisors fetched by load(), applied by the stores
  uint32_t keep[NV];   // all ones for a row inside the range, zero for one outside: the stores AND it in
  __device__ __forceinline__ static int row_of(int idx) { return ROWFAST ? idx % ROWS : idx / VPR; }
  __device__ __forceinline__ static int c4_of(int idx) { return ROWFAST ? idx / ROWS : idx % VPR; }
  // whether piece idx exists (compile-time true when the pieces fill the block's sweeps)
  __device__ __forceinline__ static bool has(int idx) { return TOTAL % 256 == 0 || idx < TOTAL; }
  __device__ __forceinline__ static void unpack(const float4& r, uint32_t k, float (&o)[4]) {
    o[0] = __uint_as_float(__float_as_uint(r.x) & k);
    o[1] = __uint_as_float(__float_as_uint(r.y) & k);
    o[2] = __uint_as_float(__float_as_uint(r.z) & k);
    o[3] = __uint_as_float(__float_as_uint(r.w) & k);
  }
  __device__ __forceinline__ static void unpack(const uint2& r, uint32_t k, float (&o)[4]) {
    const uint32_t x = r.x & k, y = r.y & k;
    o[0] = __uint_as_float(x << 16);
    o[1] = __uint_as_float(x & 0xffff0000u);
    o[2] = __uint_as_float(y << 16);
    o[3] = __uint_as_float(y & 0xffff0000u);
  }
  // piece u converted, times `scale` over the row's divisor; zero for a row outside the range.  The mask
  // goes on as bits, on the piece and on the factor (whose divisor is that of the nearest row inside): as
  // a choice between the value and zero it would become a branch around the use of the fetched registers,
  // and a loop that reuses them would then have to wait for every older memory operation first.
  __device__ __forceinline__ void piece(int u, float scale, float (&o)[4]) const {
    const float sc = __uint_as_float(__float_as_uint(scale / rdiv[u]) & keep[u]);
    unpack(raw[u], keep[u], o);
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] *= sc;
  }

  // rows tok0.. of one head; rows outside [lo, n) read as zero (they are fetched from the nearest
  // row inside, a valid address, and zeroed by the store).
  // rowdiv, when given, makes the stores divide every row by rowdiv[tok * rowdiv_stride].
  __device__ __forceinline__ void load(const HeadRows<const T>& hr, int tok0, int n, int tid,
                                       const float* rowdiv = nullptr, int64_t rowdiv_stride = 0) {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * 256;
      const bool in = idx < TOTAL;
      const int row = in ? row_of(idx) : 0, c4 = in ? c4_of(idx) : 0;
      const int tok = tok0 + row;
      keep[u] = (in && tok < n && tok >= hr.lo) ? 0xffffffffu : 0u;
      const int tk = max(tok < n ? tok : n - 1, hr.lo);
      raw[u] = *reinterpret_cast<const Raw*>(hr.base + ((unsigned)tk * hr.pitch + (unsigned)(c4 * 4)));
      rdiv[u] = 1.0f;
      if (rowdiv) rdiv[u] = rowdiv[(unsigned)tk * (unsigned)rowdiv_stride];
    }
  }
  // dst is [ROWS][ld] floats in LDS, 16-byte aligned, ld a multiple of 4
  __device__ __forceinline__ void store(float* dst, int ld, float scale, int tid) const {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * 256;
      const int row = row_of(idx), c4 = c4_of(idx);
      if (has(idx)) {
        float x[4];
        piece(u, scale, x);
        *reinterpret_cast<float4*>(dst + row * ld + c4 * 4) = make_float4(x[0], x[1], x[2], x[3]);
      }
    }
  }
  // same with scalar stores, for an odd pitch
  __device__ __forceinline__ void store_s(float* dst, int ld, float scale, int tid) const {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * 256;
      const int row = row_of(idx), c4 = c4_of(idx);
      if (has(idx)) {
        float x[4];
        piece(u, scale, x);
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[row * ld + c4 * 4 + e] = x[e];
      }
    }
  }
  // transposed and rounded to bf16: dst is [D][ld] 16-bit elements in LDS
  __device__ __forceinline__ void store_t_bf(uint16_t* dst, int ld, float scale, int tid) const {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * 256;
      const int row = row_of(idx), c4 = c4_of(idx);
      if (has(idx)) {
        float x[4];
        piece(u, scale, x);
        const uint32_t p01 = pack_bf2(x[0], x[1]), p23 = pack_bf2(x[2], x[3]);
        dst[(c4 * 4 + 0) * ld + row] = (uint16_t)p01;
        dst[(c4 * 4 + 1) * ld + row] = (uint16_t)(p01 >> 16);
        dst[(c4 * 4 + 2) * ld + row] = (uint16_t)p23;
        dst[(c4 * 4 + 3) * ld + row] = (uint16_t)(p23 >> 16);
      }
    }
  }
  // row-major, rounded to bf16: dst is [ROWS][ld] 16-bit elements in LDS, 8-byte aligned rows
  __device__ __forceinline__ void store_bf(uint16_t* dst, int ld, float scale, int tid) const {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * 256;
      const int row = row_of(idx), c4 = c4_of(idx);
      if (has(idx)) {
        float x[4];
        piece(u, scale, x);
        *reinterpret_cast<uint2*>(dst + row * ld + c4 * 4) = make_uint2(pack_bf2(x[0], x[1]), pack_bf2(x[2], x[3]));
      }
    }
  }
  // transposed: dst is [D][ld] floats in LDS, token rows become columns
  __device__ __forceinline__ void store_t(float* dst, int ld, float scale, int tid) const {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + u * 256;
      const int row = row_of(idx), c4 = c4_of(idx);
      if (has(idx)) {
        float x[4];
        piece(u, scale, x);
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[(c4 * 4 + e) * ld + row] = x[e];
      }
    }
  }
};

// bf16 variant of RowTile<D, bf16_t, ROWS, true> that keeps the rows as loaded (two registers
// per 4-element piece) until they are stored, so that a 64-row tile costs no more registers
// than a converted 32-row one.  Only the transposed stores exist.
template <int D, int ROWS>
struct RawTileBf {
  static_assert(256 % ROWS == 0 && (ROWS * D / 4) % 256 == 0, "every thread owns whole pieces of one row");
  static constexpr int RG = 256 / ROWS;          // 4-channel groups covered per sweep of the block
  static constexpr int NV = (D / 4) / RG;        // pieces per thread: row tid % ROWS, groups tid / ROWS + u * RG
  uint2 raw[NV];
  float rdiv;

  __device__ __forceinline__ void load(const HeadRows<const bf16_t>& hr, int tok0, int n, int tid,
                                       const float* rowdiv = nullptr, int64_t rowdiv_stride = 0) {
    const int tok = tok0 + tid % ROWS;
    const bool live = tok < n && tok >= hr.lo;
    const bf16_t* src = hr.base + ((unsigned)(live ? tok : hr.lo) * hr.pitch + (unsigned)((tid / ROWS) * 4));
    rdiv = (live && rowdiv) ? rowdiv[(unsigned)tok * (unsigned)rowdiv_stride] : 1.0f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const uint2 t = *reinterpret_cast<const uint2*>(src + u * RG * 4);
      raw[u] = live ? t : make_uint2(0u, 0u);
    }
  }
  // transposed, converted to fp32 and scaled: dst is [D][ld] floats in LDS
  __device__ __forceinline__ void store_t(float* dst, int ld, float scale, int tid) const {
    const float sc = scale / rdiv;
    float* d0 = dst + (tid / ROWS) * 4 * ld + tid % ROWS;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      d0[(u * RG * 4 + 0) * ld] = bf_lo(raw[u].x) * sc;
      d0[(u * RG * 4 + 1) * ld] = bf_hi(raw[u].x) * sc;
      d0[(u * RG * 4 + 2) * ld] = bf_lo(raw[u].y) * sc;
      d0[(u * RG * 4 + 3) * ld] = bf_hi(raw[u].y) * sc;
    }
  }
  // transposed bf16: dst is [D][ld] 16-bit elements in LDS.  exact: the rows go out as loaded
  // (no scale, no divisor); otherwise they are scaled in fp32 and rounded again.
  __device__ __forceinline__ void store_t_bf(uint16_t* dst, int ld, float scale, int tid, bool exact) const {
    const float sc = scale / rdiv;
    uint16_t* d0 = dst + (tid / ROWS) * 4 * ld + tid % ROWS;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      uint32_t p01 = raw[u].x, p23 = raw[u].y;
      if (!exact) {
        p01 = pack_bf2(bf_lo(raw[u].x) * sc, bf_hi(raw[u].x) * sc);
        p23 = pack_bf2(bf_lo(raw[u].y) * sc, bf_hi(raw[u].y) * sc);
      }
      d0[(u * RG * 4 + 0) * ld] = (uint16_t)p01;
      d0[(u * RG * 4 + 1) * ld] = (uint16_t)(p01 >> 16);
      d0[(u * RG * 4 + 2) * ld] = (uint16_t)p23;
      d0[(u * RG * 4 + 3) * ld] = (uint16_t)(p23 >> 16);
    }
  }
};

// sum over the 256 threads of a block; red is 4 floats of LDS; result valid in every thread
__device__ __forceinline__ float block_sum_256(float v, float* red, int tid) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  __syncthreads();
  if ((tid & 63) == 0) red[tid >> 6] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}
