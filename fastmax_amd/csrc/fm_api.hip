// C ABI of the gfx950 Fastmax library: argument checking, workspace carving, head batching
// and kernel launches.  No torch, no allocation; the only state kept between calls is the
// per-device address of the built-in scratch array (fastmax_forward_noalloc) and the opt-in
// per-thread kernel timer.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <vector>

#include "fastmax_amd.h"
#include "fm_apply.h"
#include "fm_backward.h"
#include "fm_decode.h"
#include "fm_dense.h"
#include "fm_forward.h"
#include "fm_grad.h"
#include "fm_linear.h"
#include "fm_rope.h"

// Scratch memory of fastmax_forward_noalloc: lives in every device's copy of the code object from
// the moment the library is loaded there until the process ends.  In host code the name is only a
// handle for hipGetSymbolAddress; kernels and copies get the per-device address it returns.
static __device__ __align__(256) unsigned char scratch[FASTMAX_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Optional per-thread kernel timing (fastmax_profile_begin/end): every launch is bracketed by
// two HIP events on the caller's stream; nothing is synchronised until fastmax_profile_end.
struct Profiler {
  bool on = false;
  std::vector<hipEvent_t> ev;   // start/stop pairs
  std::vector<int> cls;
  size_t used = 0;
};
thread_local Profiler g_prof;

struct ScopedKernel {
  hipStream_t st;
  bool on;
  ScopedKernel(int kclass, hipStream_t stream) : st(stream), on(g_prof.on) {
    if (!on) return;
    if (g_prof.used + 2 > g_prof.ev.size()) {
      hipEvent_t a, b;
      if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) {
        on = false;
        return;
      }
      g_prof.ev.push_back(a);
      g_prof.ev.push_back(b);
    }
    g_prof.cls.push_back(kclass);
    (void)hipEventRecord(g_prof.ev[g_prof.used], st);
  }
  ~ScopedKernel() {
    if (!on) return;
    (void)hipEventRecord(g_prof.ev[g_prof.used + 1], st);
    g_prof.used += 2;
  }
};

// Tokens between causal state snapshots (a multiple of the 128-token block of the consumers).
// Longer chunks mean fewer snapshots to write and read but more intra-chunk score tiles (at 384 tokens
// they are more than a quarter of a consumer's matrix instructions).  Measured at the headline shapes,
// p = 2: fp32 d = 64 is fastest at 256 (384: +2.4 %, 128: +0.8 %), fp32 d = 32 at 128, bf16 d = 64 at 384
// (256: +2 %: its build kernel pays more per snapshot).
constexpr int kChunkP1 = 128;  // p = 1: a state is only d+1 rows, a snapshot per block is cheapest
inline int chunk_for(int d, int p2, int dtype) {
  if (!p2) return kChunkP1;
  if (dtype == FASTMAX_BF16) return 384;
  return d == 64 ? 256 : 128;
}
constexpr size_t kWorkspaceBudget = 16ull << 30;   // what fastmax_workspace_bytes aims for

struct Plan {
  int d, p2, masked, bh;
  int nq, nk;          // query rows, key rows per head
  int n;               // positions the scans and state slots are laid out over: nk under the causal
                       // mask (queries sit at positions off .. nk-1), max(nq, nk) otherwise
  int off;             // causal: position of the first query, nk - nq (the key prefix); else 0
  int nblk_q, nblk_k;  // 128-token blocks launched by the kernels whose own rows are query-side /
                       // key-side tensors
  int bhkv, ratio;     // key/value heads; query heads per key/value head
  int rtw, gsplit;     // build kernel: row tiles per wave, feature splits per head
  int nslots, zlen;    // state slots per head; tokens per slot when unmasked
  int nparts;          // token splits the unmasked build sums separately (1 when masked); bf16
                       // inputs add one slot that receives their sum in packed form
  int chunk;           // tokens between causal state snapshots
  bool plain;          // every tensor is a plain contiguous (heads, tokens, d) array
  bool scan;           // causal p = 1 as one scan per head (fm_linear.h): no states in memory
  bool rowpass;        // unmasked p = 1: states from the build kernel, one pass over the rows per output
  bool dense;          // dense score tiles, no moment states (fm_dense.h): short sequences, and every head
                       // dimension other than 32 and 64
  bool lin;            // dense kernels in linear mode (p = 1, long sequences): chunk states of (dp + 1) rows in
                       // the workspace, lslots of them per head, one per lchunk positions
  int lchunk, lslots, ldp;
  bool split;          // causal p = 1 with few heads: the chunks of a head are built side by side as partial
                       // states and a prefix pass over the chunks makes the causal states of them
  size_t scratch_bytes;   // per head: where the fp32 partial states of a split build go when the
                          // states themselves are packed bf16 (last part of per_head_bytes; a forward
                          // pass that keeps its states has it behind the states in the caller's buffer)
  int pass;
  int64_t state_floats;
  size_t fixed_bytes;     // scale/argmax/cvec/rpart
  size_t per_head_bytes;  // states of one head
};

int64_t state_floats_for(int d, int p2) {
  return d == 64 ? Geo<64>::state_floats(p2) : Geo<32>::state_floats(p2);
}
// floats per state slot of a pass: causal bf16 passes keep packed states only
int64_t slot_floats_for(int d, int p2, bool packed) {
  if (!packed) return state_floats_for(d, p2);
  return d == 64 ? PackedGeo<64>::slot_floats(p2) : PackedGeo<32>::slot_floats(p2);
}

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

int64_t lin_state_floats(int dp, int nblk) {
  return dp == 32 ? dense::LinState<32>::floats(nblk) : dp == 64 ? dense::LinState<64>::floats(nblk)
       : dp == 96 ? dense::LinState<96>::floats(nblk) : dense::LinState<128>::floats(nblk);
}

// Causal p = 1 at d = 64 runs as one sequential scan per head (fm_linear.h: one wave per head, the
// state never leaves its registers) once there are enough heads: with fp32 tensors (fp32 matrix
// instruction, matrix-bound) from about half of the chip's 1024 SIMDs filled, below which the chunked
// kernels, which split a head over many blocks, win; with bf16 tensors (bf16 matrix instruction: a
// scan then costs 0.24 us per position up to 256 heads and is memory-bound beyond) from 208 heads, below
// which the dense kernels' linear mode wins (1.2 ns per position and head).
#ifndef FM_LINEAR_MIN_HEADS
#define FM_LINEAR_MIN_HEADS 512
#endif
#ifndef FM_LINEAR_MIN_HEADS_BF16
#define FM_LINEAR_MIN_HEADS_BF16 208
#endif
int linear_min_heads(const fastmax_desc* ds) {
  return ds->dtype == FASTMAX_BF16 ? FM_LINEAR_MIN_HEADS_BF16 : FM_LINEAR_MIN_HEADS;
}
bool use_linear_scan(const fastmax_desc* ds, const Plan& pl);

// Dense score tiles cost 2 n d flop per token under the mask (4 n d without it), the moment form about
// 2.1 d^3 (p = 2) whatever n is: below these key counts the dense kernels are the faster ones (measured,
// forward + backward, 96 and 768 heads; with few heads the sequential state build of the moment form
// fills the chip badly and the dense kernels stay ahead for longer).  A causal sequence of a single chunk
// has no states to build either way and stays with the moment kernels' own intra-chunk tiles.  Head
// dimensions without moment kernels always take the dense ones (p = 1 at d = 32 / 64: see below).
bool use_dense(const fastmax_desc* ds, bool plain = true) {
  if (ds->d != 32 && ds->d != 64) return true;
  // FASTMAX_PATH = moments | dense overrides the choice where both kernel families exist
  if (const char* e = getenv("FASTMAX_PATH")) {
    if (!strcmp(e, "moments")) return false;
    if (!strcmp(e, "dense")) return true;
  }
  const bool bf = ds->dtype == FASTMAX_BF16;
  if (ds->p != 2) {
    // p = 1: the moment states are tiny and the moment kernels win -- except for bf16 inputs under the mask
    // past 1024 keys with too few heads for the one-scan-per-head kernels (linear_min_heads; or no such kernels:
    // d = 32, grouped heads, a key prefix, a1 = 0, strided tensors): there the dense kernels' linear mode (chunk states plus the
    // own chunk's tiles, all of it parallel over heads and chunks) beats the chunked moment kernels at every
    // head count measured (16 .. 768 heads: 1.0 - 1.4x)
    if (!(bf && ds->mask && ds->nk > 1024)) return false;
    const bool scan = plain && ds->d == 64 && ds->bh == ds->bhkv && ds->nq == ds->nk && ds->a1 != 0.f && ds->bh >= linear_min_heads(ds);
    return !scan;
  }
  const bool few = ds->bh <= 128;   // (few heads: the moment form's sequential state build fills the chip badly)
  int limit;
  if (ds->d == 64) {
    if (ds->mask) limit = bf ? (few ? 5632 : 4096) : (few ? 3584 : 3072);
    else limit = bf ? (few ? 2048 : 1536) : 1024;
  } else {
    if (ds->mask) limit = bf ? (few ? 3072 : 2048) : (few ? 1536 : 1024);
    else limit = bf ? (few ? 1024 : 768) : 512;
  }
  if (ds->mask && ds->nk <= chunk_for(ds->d, 1, ds->dtype)) return false;
  return ds->nk <= limit;
}

Plan make_plan(const fastmax_desc* ds, int pass, bool plain = true, bool allow_dense = true) {
  Plan pl;
  pl.pass = pass;
  pl.dense = allow_dense && use_dense(ds, plain);
  pl.d = ds->d;
  pl.p2 = ds->p == 2;
  pl.masked = ds->mask != 0;
  pl.plain = plain;
  pl.nq = ds->nq;
  pl.nk = ds->nk;
  pl.n = pl.masked ? ds->nk : (ds->nq > ds->nk ? ds->nq : ds->nk);
  pl.off = pl.masked ? ds->nk - ds->nq : 0;
  pl.nblk_k = (ds->nk + 127) / 128;
  pl.nblk_q = pl.masked ? pl.nblk_k - pl.off / 128 : (ds->nq + 127) / 128;
  pl.bh = ds->bh;
  pl.bhkv = ds->bhkv;
  pl.ratio = ds->bh / ds->bhkv;
  if (pl.dense) {
    // no states: the workspace holds the per-head scalars only (and c_i, normalisation partials)
    pl.rtw = pl.gsplit = pl.nslots = pl.nparts = 1;
    pl.zlen = pl.chunk = 0;
    pl.scan = pl.rowpass = pl.split = false;
    pl.scratch_bytes = pl.per_head_bytes = 0;
    pl.state_floats = 0;
    size_t fx = align256((size_t)2 * pl.bh * sizeof(float)) + align256((size_t)2 * pl.bh * sizeof(int));
    if (pass == FASTMAX_PASS_BACKWARD) {
      fx += align256((size_t)pl.bh * pl.nq * sizeof(float));
      fx += align256((size_t)pl.bh * (pl.nblk_q + pl.nblk_k) * sizeof(float));
    }
    // p = 1 is linear in the keys: past these lengths the tiles of a 256-position chunk plus one state of
    // everything outside it cost less than the tiles of the whole sequence
    pl.lchunk = 256;
    pl.lslots = (pl.n + pl.lchunk - 1) / pl.lchunk;
    pl.ldp = (pl.d + 31) / 32 * 32;
    pl.lin = !pl.p2 && pl.n > (pl.masked ? 1024 : 512);
    if (pl.lin) {
      // key-side states (one layout of the d x d block per pass), query-side states (both layouts)
      fx += align256((size_t)pl.bhkv * pl.lslots * lin_state_floats(pl.ldp, 1) * sizeof(float));
      if (pass == FASTMAX_PASS_BACKWARD) fx += align256((size_t)pl.bh * pl.lslots * lin_state_floats(pl.ldp, 2) * sizeof(float));
    }
    pl.fixed_bytes = fx;
    return pl;
  }
  const int rt_total = (pl.p2 ? (pl.d / 2 + 1) * (pl.d / 32) : 0) + pl.d / 32;
  // (p = 1, d = 64: the four waves of a block share its two row tiles, one column tile each)
  auto splits = [&](int rtw) { return !pl.p2 && pl.d == 64 ? 1 : (rt_total + 4 * rtw - 1) / (4 * rtw); };
  if (!pl.p2) {
    pl.rtw = 1;
  } else if (pl.d == 64) {
    // 3 row tiles per wave, 6 blocks per head (4 tiles per wave would save a block per head
    // but does not fit the register file: measured 1.6x slower)
    pl.rtw = 3;
  } else {
    pl.rtw = 5;
  }
  pl.gsplit = splits(pl.rtw);
  // p = 1: a state is only (d+1) rows, so a snapshot per 128-token block is cheaper than a longer
  // intra-chunk part
  pl.chunk = chunk_for(pl.d, pl.p2, ds->dtype);
  if (pl.masked) {
    pl.nslots = (pl.n + pl.chunk - 1) / pl.chunk;
    pl.nparts = 1;
    pl.zlen = 0;
  } else {
    // enough token splits to put ~1024 blocks in flight, at least 256 tokens each
    int z = (1024 + pl.gsplit * pl.bh - 1) / (pl.gsplit * pl.bh);
    const int zmax = (pl.n + 255) / 256;
    if (z > zmax) z = zmax;
    if (z < 1) z = 1;
    int zlen = ((pl.n + z - 1) / z + 31) / 32 * 32;
    pl.zlen = zlen;
    pl.nparts = (pl.n + zlen - 1) / zlen;
    // consumers read one state per head, the last slot: the sum of the partial states (for bf16
    // inputs in packed form), or the only partial state itself
    pl.nslots = pl.nparts + ((ds->dtype == FASTMAX_BF16 || pl.nparts > 1) ? 1 : 0);
  }
  pl.state_floats = slot_floats_for(pl.d, pl.p2, pl.masked && ds->dtype == FASTMAX_BF16);
  size_t fixed = align256((size_t)2 * pl.bh * sizeof(float)) + align256((size_t)2 * pl.bh * sizeof(int));
  if (pass == FASTMAX_PASS_BACKWARD) {
    fixed += align256((size_t)pl.bh * pl.nq * sizeof(float));                        // c_i
    fixed += align256((size_t)pl.bh * (pl.nblk_q + pl.nblk_k) * sizeof(float));      // norm partials for q, k
  }
  pl.fixed_bytes = fixed;
  pl.per_head_bytes = (size_t)pl.nslots * pl.state_floats * sizeof(float) *
                      (pass == FASTMAX_PASS_BACKWARD ? 2 : 1);
  // grouped key/value heads, backward: dk and dv are formed per query head and then added up
  if (pass == FASTMAX_PASS_BACKWARD && pl.ratio > 1)
    pl.per_head_bytes += 2 * (size_t)pl.nk * pl.d * (ds->dtype == FASTMAX_BF16 ? 2 : 4);
  pl.scan = use_linear_scan(ds, pl);
  if (pl.scan) pl.per_head_bytes = 0;
  // One sequential walk per head leaves most of the chip idle when there are few heads; a p = 1 state
  // is small (d + 1 rows), so the chunks are built side by side and a cheap pass adds them up.
  pl.split = pl.masked && !pl.p2 && !pl.scan && pl.nslots >= 3 && (int64_t)pl.bh * pl.gsplit < 1024;
  pl.scratch_bytes = (pl.split && ds->dtype == FASTMAX_BF16)
                         ? (size_t)pl.nslots * state_floats_for(pl.d, pl.p2) * sizeof(float) : 0;
  pl.per_head_bytes += pl.scratch_bytes;
  pl.rowpass = !pl.p2 && !pl.masked && pl.d == 64 && pl.ratio == 1 && pl.n >= 32 && pl.plain && pl.nq == pl.nk;
  return pl;
}

bool use_linear_scan(const fastmax_desc* ds, const Plan& pl) {
  // (its kernels keep the weights divided by a1, and every tile is a full 32 rows)
  return !pl.p2 && pl.masked && pl.d == 64 && pl.ratio == 1 && pl.n >= 32 && ds->a1 != 0.f &&
         pl.bh >= linear_min_heads(ds) && pl.plain && pl.nq == pl.nk;
}

// Heads per launch that fit the workspace.  When several batches are needed the batch is
// rounded down so that the build grid (gsplit blocks per head, two resident blocks per CU)
// is a whole number of rounds over the 256 CUs; a ragged last round would idle most of the chip.
// (with_saved: the prefix states live in the caller's saved-state buffer, not in the workspace)
size_t batch_bytes_per_head(const Plan& pl, bool with_saved) {
  if (pl.scan) return 0;
  if (!with_saved) return pl.per_head_bytes;
  return pl.per_head_bytes - (size_t)pl.nslots * pl.state_floats * sizeof(float) -
         (pl.pass == FASTMAX_PASS_FORWARD ? pl.scratch_bytes : 0);
}

int heads_per_batch(const Plan& pl, size_t ws_bytes, bool with_saved = false) {
  const size_t per_head = batch_bytes_per_head(pl, with_saved);
  if (per_head == 0) return pl.bh;
  size_t hb = (ws_bytes - pl.fixed_bytes) / per_head;
  if (hb >= (size_t)pl.bh) return pl.bh;
  int g = pl.gsplit, m = 512;
  while (g % 2 == 0 && m > 1) {
    g /= 2;
    m /= 2;
  }
  if (hb >= (size_t)m) hb = hb / m * m;
  hb = hb / pl.ratio * pl.ratio;  // whole key/value groups
  if (hb < (size_t)pl.ratio) hb = pl.ratio;  // (check_ws made sure one group fits)
  return (int)hb;
}

int check_desc(const fastmax_desc* ds) {
  if (!ds) return fail(FASTMAX_E_NULL, "desc is NULL");
  if (ds->dtype != FASTMAX_F32 && ds->dtype != FASTMAX_BF16)
    return fail(FASTMAX_E_DTYPE, "dtype %d is neither FASTMAX_F32 nor FASTMAX_BF16", ds->dtype);
  {
    // rows are read in 16-byte pieces; the dense kernels hold a head dimension of up to 128 in registers
    const int step = ds->dtype == FASTMAX_BF16 ? 8 : 4;
    if (ds->d < step || ds->d > 128 || ds->d % step)
      return fail(FASTMAX_E_SHAPE, "d = %d; the head dimension must be a multiple of %d (16 bytes of %s) in [%d, 128]",
                  ds->d, step, ds->dtype == FASTMAX_BF16 ? "bf16" : "fp32", step);
  }
  if (ds->bh < 1 || ds->bh > 65535) return fail(FASTMAX_E_SHAPE, "bh = %d outside [1, 65535]", ds->bh);
  if (ds->bhkv < 1 || ds->bh % ds->bhkv != 0)
    return fail(FASTMAX_E_SHAPE, "bhkv = %d does not divide bh = %d", ds->bhkv, ds->bh);
  if (ds->nq < 1) return fail(FASTMAX_E_SHAPE, "nq = %d < 1", ds->nq);
  if (ds->nk < 1) return fail(FASTMAX_E_SHAPE, "nk = %d < 1", ds->nk);
  if (ds->mask && ds->nk < ds->nq)
    return fail(FASTMAX_E_SHAPE, "nk = %d < nq = %d under the causal mask (the keys are a prefix plus one per query)", ds->nk, ds->nq);
  if ((int64_t)(ds->nq > ds->nk ? ds->nq : ds->nk) * ds->d * ds->bh >= (int64_t)1 << 40)
    return fail(FASTMAX_E_SHAPE, "tensor too large");
  if (ds->p != 1 && ds->p != 2) return fail(FASTMAX_E_PARAM, "p must be 1 or 2, got: %d", ds->p);
  if (ds->normalize) {
    if (!(ds->lim > 0.f)) return fail(FASTMAX_E_PARAM, "lim = %g must be positive when normalize is set", (double)ds->lim);
  } else if (ds->temperature == 0.f || ds->temperature != ds->temperature) {
    return fail(FASTMAX_E_PARAM, "temperature = %g", (double)ds->temperature);
  }
  return FASTMAX_OK;
}

int check_ws(const Plan& pl, void* ws, size_t ws_bytes, bool with_saved = false) {
  if (!ws) return fail(FASTMAX_E_WORKSPACE, "workspace is NULL");
  if (((uintptr_t)ws) & 255) return fail(FASTMAX_E_WORKSPACE, "workspace is not 256-byte aligned");
  const size_t need = pl.fixed_bytes + pl.ratio * batch_bytes_per_head(pl, with_saved);
  if (ws_bytes < need)
    return fail(FASTMAX_E_WORKSPACE, "workspace of %zu bytes is below the minimum of %zu", ws_bytes, need);
  return FASTMAX_OK;
}

size_t saved_bytes_for(const Plan& pl) {
  if (pl.scan || pl.dense) return 256;   // nothing to keep; a token size, so that 0 still means "bad descriptor"
  // (a split build of packed states sums fp32 partial states: room for them behind the states)
  return (size_t)pl.bhkv * (pl.nslots * pl.state_floats * sizeof(float) + pl.scratch_bytes);
}

int check_saved(const Plan& pl, const void* saved, size_t saved_bytes) {
  if (!saved) return FASTMAX_OK;
  if (((uintptr_t)saved) & 255) return fail(FASTMAX_E_WORKSPACE, "saved-state buffer is not 256-byte aligned");
  if (saved_bytes < saved_bytes_for(pl))
    return fail(FASTMAX_E_WORKSPACE, "saved-state buffer of %zu bytes is below the %zu needed", saved_bytes,
                saved_bytes_for(pl));
  return FASTMAX_OK;
}

int launch_status(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(FASTMAX_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return FASTMAX_OK;
}

#define FM_TRY(expr)            \
  do {                          \
    const int rc_ = (expr);     \
    if (rc_ != FASTMAX_OK) return rc_; \
  } while (0)

// Strides of one tensor (elements): head h sits at (h / (ng nh)) sb + ((h / nh) % ng) sg + (h % nh) sh
struct Str {
  int64_t sb, sg, sh, pitch;
  int ng, nh;
};
// a plain (heads, rows, pitch) array
Str plain_str(int64_t rows, int64_t pitch) { return Str{rows * pitch, 0, 0, pitch, 1, 1}; }
// levels with uniform strides are merged (a contiguous tensor ends up as one level)
Str make_str(const fastmax_strides& f, int groups, int heads_per_group) {
  Str t{f.batch, f.group, heads_per_group > 1 ? f.head : 0, f.token, groups, heads_per_group};
  if (t.nh > 1 && t.sg == t.nh * t.sh) {
    t.ng *= t.nh;
    t.sg = t.sh;
    t.nh = 1;
    t.sh = 0;
  }
  if (t.nh == 1 && t.sb == t.ng * t.sg) {
    t.sb = t.sg;
    t.ng = 1;
    t.sg = 0;
  }
  return t;
}
struct Layout {
  Str q, k, v, o, go, dq, dk, dv;
};
Layout plain_layout(const fastmax_desc* ds, int64_t ldo) {
  const Str tq = plain_str(ds->nq, ds->d), tk = plain_str(ds->nk, ds->d);
  return Layout{tq, tk, tk, plain_str(ds->nq, ldo), tq, tq, tk, tk};
}
bool is_plain(const Str& t, int64_t rows, int64_t pitch) { return t.ng == 1 && t.nh == 1 && t.pitch == pitch && t.sb == rows * pitch; }
bool is_plain(const Layout& L, const fastmax_desc* ds, bool backward) {
  const int d = ds->d;
  bool ok = is_plain(L.q, ds->nq, d) && is_plain(L.k, ds->nk, d) && is_plain(L.v, ds->nk, d) &&
            L.o.ng == 1 && L.o.nh == 1 && L.o.sb == ds->nq * L.o.pitch;
  if (backward)
    ok = ok && is_plain(L.go, ds->nq, d) && is_plain(L.dq, ds->nq, d) && is_plain(L.dk, ds->nk, d) &&
         is_plain(L.dv, ds->nk, d);
  return ok;
}

// first head of a batch h0, first position lo (the pointer is moved back by lo rows, so that
// position t >= lo is row t - lo of the tensor)
template <class T>
Rows<T> mk_rows(T* p, const Str& t, int h0 = 0, int lo = 0) {
  return Rows<T>{p - (int64_t)lo * t.pitch, t.sb, t.sg, t.sh, t.pitch, t.ng, t.nh, h0, lo};
}
template <class F>
RowScalarsT<F> mk_scalars(F* p, int64_t rows, int64_t stride, int h0 = 0, int lo = 0) {
  if (!p) return RowScalarsT<F>{nullptr, 0, 0};
  return RowScalarsT<F>{p + ((int64_t)h0 * rows - lo) * stride, rows * stride, stride};
}
const RowScalars kNoScalars{nullptr, 0, 0};

// the kernels read and write whole 16-byte pieces of rows
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool aligned16(const Str& t, size_t es) {
  return (t.sb * es) % 16 == 0 && (t.sg * es) % 16 == 0 && (t.sh * es) % 16 == 0 && (t.pitch * es) % 16 == 0;
}

// scale[0..bh) for q, scale[bh..2bh) for k
template <class T>
int compute_scales(const fastmax_desc* ds, const Layout& L, const T* q, const T* k, float* scale, int* arg,
                   hipStream_t stream) {
  const int bh = ds->bh, bhkv = ds->bhkv;
  ScopedKernel sk(FASTMAX_K_ROWSTAT, stream);
  if (ds->normalize) {
    const Rows<const T> qr = mk_rows(q, L.q), kr = mk_rows(k, L.k);
    // (q and k in one launch; with few heads a block is 1024 threads so that the chip still fills)
    if (bh + bhkv >= 1024)
      rowstat_kernel<T, 256><<<bh + bhkv, 256, 0, stream>>>(qr, ds->nq, bh, kr, ds->nk, ds->d, ds->lim, scale, arg);
    else
      rowstat_kernel<T, 1024><<<bh + bhkv, 1024, 0, stream>>>(qr, ds->nq, bh, kr, ds->nk, ds->d, ds->lim, scale, arg);
  } else {
    fill_scale_kernel<<<(bh + 255) / 256, 256, 0, stream>>>(scale, arg, bh, 1.0f);
    fill_scale_kernel<<<(bhkv + 255) / 256, 256, 0, stream>>>(scale + bh, arg + bh, bhkv, 1.0f / ds->temperature);
  }
  return launch_status("scale kernels");
}

// bf16 inputs run the contractions on the bf16 matrix instruction (fp32 accumulate)
template <class T>
constexpr bool kBf16Mfma = false;
template <>
constexpr bool kBf16Mfma<bf16_t> = true;

// State of (X, Y, extra) over n positions of `heads` heads (X.h0 is the first of them).
template <int D, class T>
int launch_build(const Plan& pl, int heads, int n, const Rows<const T>& X, const Rows<const T>& Y,
                 const float* xscale, const RowScalars& yden, const RowScalars& ew, float* state, int reverse,
                 hipStream_t stream, bool finish = true, float* scratch = nullptr) {
  if (pl.masked && pl.nslots < 2) return FASTMAX_OK;  // a single chunk never needs a state
  ScopedKernel sk(FASTMAX_K_BUILD, stream);
  if (pl.split) {
    // every chunk as a token split of its own (the unmasked form of the kernel: fp32 partial states,
    // slot c = chunk c), then the sums over the chunks before (after, for a reverse scan) each chunk
    float* part = kBf16Mfma<T> ? scratch : state;
    const dim3 sgrid(pl.gsplit, heads, pl.nslots);
    build_kernel<D, T, 1, kBf16Mfma<T>><<<sgrid, 256, 0, stream>>>(X, Y, xscale, yden, ew, part, n, pl.chunk, pl.nslots,
                                                                   0, 0, pl.p2, pl.chunk);
    const int64_t ss = state_floats_for(pl.d, pl.p2);
    state_prefix_kernel<<<dim3((unsigned)((ss / 4 + 255) / 256), heads), 256, 0, stream>>>(part, pl.nslots, ss, reverse);
    if constexpr (kBf16Mfma<T>)
      state_pack_slots_kernel<D><<<dim3(PackedGeo<D>::nslab(pl.p2), heads, pl.nslots), 256, 0, stream>>>(part, state,
                                                                                                      pl.nslots, pl.p2);
    return launch_status("build_kernel (chunks side by side)");
  }
  const dim3 grid(pl.gsplit, heads, pl.nparts);
#define FM_BUILD(RTW)                                                                            \
  build_kernel<D, T, RTW, kBf16Mfma<T>><<<grid, 256, 0, stream>>>(X, Y, xscale, yden, ew, state, \
                                                    n, pl.chunk, pl.nslots, pl.masked, reverse, \
                                                    pl.p2, pl.zlen)
  if (pl.rtw == 1) {
    FM_BUILD(1);
  } else if constexpr (D == 64) {
    FM_BUILD(3);
  } else {
    FM_BUILD(5);
  }
#undef FM_BUILD
  // unmasked: the partial states of a head are summed into its last slot (finish = false leaves
  // that to the caller)
  if (!pl.masked && finish) {
    if constexpr (kBf16Mfma<T>) {
      state_pack_kernel<D><<<dim3(PackedGeo<D>::nslab(pl.p2), heads), 256, 0, stream>>>(state, pl.nslots, pl.nparts, pl.p2);
    } else if (pl.nparts > 1) {
      const int64_t ss = pl.state_floats;
      state_accumulate_kernel<<<dim3((unsigned)((ss / 4 + 255) / 256), heads), 256, 0, stream>>>(
          state + (int64_t)pl.nparts * ss, (int64_t)pl.nslots * ss, state, pl.nslots, pl.nparts, ss, 0);
    }
  }
  return launch_status("build_kernel");
}

// Unmasked p = 1 row passes read the head's state in fp32: the partial states of the token splits are
// summed into slot nparts (with a single split, slot 0 is the state).  Returns that slot.
inline int finish_state_fp32(const Plan& pl, int heads, float* state, hipStream_t stream) {
  if (pl.nparts == 1) return 0;
  const int64_t ss = pl.state_floats;
  state_accumulate_kernel<<<dim3((unsigned)((ss / 4 + 255) / 256), heads), 256, 0, stream>>>(
      state + (int64_t)pl.nparts * ss, (int64_t)pl.nslots * ss, state, pl.nslots, pl.nparts, ss, 0);
  return pl.nparts;
}

// Unmasked p = 1 with bf16 tensors has two consumers of a kept state: the chunked kernels read the packed
// form in the head's last slot, the row passes the fp32 sum.  A forward pass that keeps its states leaves
// both (the sum in slot 0, over the first partial state), so that a backward pass may take either family
// whatever the forward pass took.  `state` holds the fp32 partial states of `heads` heads.
template <int D>
inline void finish_state_both(const Plan& pl, int heads, float* state, hipStream_t stream) {
  const int64_t ss = pl.state_floats;
  state_pack_kernel<D><<<dim3(PackedGeo<D>::nslab(pl.p2), heads), 256, 0, stream>>>(state, pl.nslots, pl.nparts, pl.p2);
  if (pl.nparts > 1)
    state_accumulate_kernel<<<dim3((unsigned)((ss / 4 + 255) / 256), heads), 256, 0, stream>>>(
        state, (int64_t)pl.nslots * ss, state, pl.nslots, pl.nparts, ss, 0);
}

template <int D, class T>
int forward_impl(const fastmax_desc* ds, const Plan& pl, const Layout& L, const T* q, const T* k, const T* v, T* o,
                 float* den, int64_t den_stride, float* scale_out, int32_t* arg_out,
                 char* ws, size_t ws_bytes, float* saved, hipStream_t stream) {
  const int bh = pl.bh, nq = pl.nq, nk = pl.nk;
  const int64_t ldo = L.o.pitch;
  // per-head factors and arg-max rows: straight into the caller's arrays when it wants them
  float* scale = scale_out ? scale_out : reinterpret_cast<float*>(ws);
  int* arg = arg_out ? arg_out : reinterpret_cast<int*>(ws + align256((size_t)2 * bh * sizeof(float)));
  // the prefix states go to the workspace (one head batch at a time) or, when the caller keeps
  // them for the backward pass, straight into its buffer (all heads)
  const int hb = heads_per_batch(pl, ws_bytes, saved != nullptr);
  const int64_t head_floats = (int64_t)pl.nslots * pl.state_floats;

  FM_TRY(compute_scales<T>(ds, L, q, k, scale, arg, stream));

  if constexpr (D == 64) {
    if (pl.scan) {   // (plain tensors, nq == nk)
      const int n = nq;
      ScopedKernel sk(FASTMAX_K_FWD_APPLY, stream);
      // (pairs of output columns go out as one store when the row pitch keeps them aligned)
      if (ldo % 2 == 0)
        lin::linear_fwd_kernel<T, true><<<bh, 64, 0, stream>>>(q, k, v, scale, scale + bh, o, ldo, den, den_stride, n,
                                                                ds->a0, ds->a1);
      else
        lin::linear_fwd_kernel<T, false><<<bh, 64, 0, stream>>>(q, k, v, scale, scale + bh, o, ldo, den, den_stride, n,
                                                                 ds->a0, ds->a1);
      return launch_status("linear_fwd_kernel");
    }
  }

  const int ratio = pl.ratio;
  // positions the consumers' own rows run over (the queries sit at off .. nk-1 under the mask)
  const int nown = pl.masked ? nk : nq;
  for (int h0 = 0; h0 < bh; h0 += hb) {
    const int heads = bh - h0 < hb ? bh - h0 : hb;
    const int kv0 = h0 / ratio;                          // first key/value head of the batch
    float* state = saved ? saved + kv0 * head_floats : reinterpret_cast<float*>(ws + pl.fixed_bytes);
    if constexpr (D == 64) {
      if (pl.rowpass) {   // (plain tensors, nq == nk)
        const int n = nq;
        const int64_t off = (int64_t)h0 * n * D, koff = (int64_t)kv0 * n * D;
        FM_TRY((launch_build<D, T>(pl, heads, n, mk_rows(k, L.k, kv0), mk_rows(v, L.v, kv0), scale + bh + kv0, kNoScalars,
                                   kNoScalars, state, 0, stream, false)));
        (void)koff;
        int slot = 0;
        if (saved && kBf16Mfma<T>) finish_state_both<D>(pl, heads, state, stream);
        else slot = finish_state_fp32(pl, heads, state, stream);
        ScopedKernel sk(FASTMAX_K_FWD_APPLY, stream);
        const dim3 rgrid((n + lin::ROWS_PER_WAVE - 1) / lin::ROWS_PER_WAVE, heads);
#define FM_ROWFWD(AL)                                                                                          \
  lin::linear_rowpass_kernel<T, lin::ROWPASS_FWD, false, AL><<<rgrid, 64, 0, stream>>>(                          \
      q + off, state + (int64_t)slot * pl.state_floats, head_floats, scale + h0, nullptr, den_stride, nullptr, \
      nullptr, o + (int64_t)h0 * n * ldo, ldo, den + (int64_t)h0 * n * den_stride, nullptr, n, ds->a0, ds->a1)
        if (ldo % 2 == 0) FM_ROWFWD(true); else FM_ROWFWD(false);
#undef FM_ROWFWD
        FM_TRY(launch_status("linear_rowpass_kernel (forward)"));
        continue;
      }
    }
    const Rows<const T> kr = mk_rows(k, L.k, kv0), vr = mk_rows(v, L.v, kv0);
    // (scratch of a split build: behind the batch's states in the workspace, or behind all states in
    // the caller's buffer)
    float* scratch = saved ? reinterpret_cast<float*>(reinterpret_cast<char*>(saved + (int64_t)pl.bhkv * head_floats) +
                                                      (size_t)kv0 * pl.scratch_bytes)
                           : reinterpret_cast<float*>(ws + pl.fixed_bytes + (size_t)hb * (pl.per_head_bytes - pl.scratch_bytes));
    FM_TRY((launch_build<D, T>(pl, heads / ratio, nk, kr, vr, scale + bh + kv0, kNoScalars, kNoScalars, state, 0,
                               stream, true, scratch)));
    if constexpr (D == 64 && kBf16Mfma<T>) {
      // (kept states of unmasked p = 1: also the fp32 sum a row-pass backward would read)
      if (saved && !pl.masked && !pl.p2 && pl.nparts > 1) {
        const int64_t ss = pl.state_floats;
        state_accumulate_kernel<<<dim3((unsigned)((ss / 4 + 255) / 256), heads / ratio), 256, 0, stream>>>(
            state, (int64_t)pl.nslots * ss, state, pl.nslots, pl.nparts, ss, 0);
      }
    }
    {
      ScopedKernel sk(FASTMAX_K_FWD_APPLY, stream);
      const dim3 agrid(pl.nblk_q, heads);
      const Rows<const T> qr = mk_rows(q, L.q, h0, pl.off);
      const Rows<T> orow = mk_rows(o, L.o, h0, pl.off);
      const RowScalarsOut dn = mk_scalars(den, nq, den_stride, h0, pl.off);
      if constexpr (kBf16Mfma<T>) {
        apply_kernel_bf<D, 0><<<agrid, 256, 0, stream>>>(
            qr, kr, vr, scale + h0, scale + bh + kv0, kNoScalars, state, pl.nslots, orow, dn, nown, pl.chunk,
            pl.masked, pl.p2, ds->a0, ds->a1, pl.p2 ? ds->a2 : 0.f, 1, ratio);
      } else {
        apply_kernel<D, T, 0><<<agrid, 256, 0, stream>>>(
            qr, kr, vr, scale + h0, scale + bh + kv0, kNoScalars, state, pl.nslots, orow, dn, nown, pl.chunk,
            pl.masked, pl.p2, ds->a0, ds->a1, pl.p2 ? ds->a2 : 0.f, 1, ratio);
      }
    }
    FM_TRY(launch_status("fwd_apply_kernel"));
  }
  return FASTMAX_OK;
}

// c_i = go_i . o_i / den_i for every query row: 16-byte accesses when the rows of o allow it
template <class T>
int launch_bwd_prep(const Plan& pl, const Layout& L, const T* go, const T* o, const float* den, int64_t den_stride,
                    float* cvec, hipStream_t stream) {
  ScopedKernel sk(FASTMAX_K_BWD_PREP, stream);
  const bool vec = aligned16(L.o, sizeof(T)) && aligned16(o) && aligned16(L.go, sizeof(T)) && aligned16(go);
  const Rows<const T> gr = mk_rows(go, L.go), orow = mk_rows(o, L.o);
  const RowScalars dn = mk_scalars(den, pl.nq, den_stride);
  auto pow2 = [](int x) { int t = 1; while (t < x) t *= 2; return t; };
  if (vec) {
    const int rpp = 256 / pow2(pl.d * (int)sizeof(T) / 16);
    bwd_prep_kernel<T, true><<<dim3((pl.nq + rpp - 1) / rpp, pl.bh), 256, 0, stream>>>(gr, orow, dn, cvec, pl.nq, pl.d);
  } else {
    const int rpp = 256 / pow2(pl.d / 4);
    bwd_prep_kernel<T, false><<<dim3((pl.nq + rpp - 1) / rpp, pl.bh), 256, 0, stream>>>(gr, orow, dn, cvec, pl.nq, pl.d);
  }
  return launch_status("bwd_prep_kernel");
}

template <int D, class T>
int backward_impl(const fastmax_desc* ds, const Plan& pl, const Layout& L, const T* q, const T* k, const T* v,
                  const T* o, const float* den, int64_t den_stride, const T* go, T* dq,
                  T* dk, T* dv, const float* scale_in, const int32_t* arg_in, char* ws,
                  size_t ws_bytes, const float* saved, hipStream_t stream) {
  const int bh = pl.bh, nq = pl.nq, nk = pl.nk;
  const int64_t ldo = L.o.pitch;
  char* p = ws;
  const bool given = scale_in && arg_in;  // the forward pass's values: read in place
  const float* scale = given ? scale_in : reinterpret_cast<float*>(p);
  float* scale_ws = reinterpret_cast<float*>(p);
  p += align256((size_t)2 * bh * sizeof(float));
  const int* arg = given ? arg_in : reinterpret_cast<int*>(p);
  int* arg_ws = reinterpret_cast<int*>(p);
  p += align256((size_t)2 * bh * sizeof(int));
  float* cvec = reinterpret_cast<float*>(p);
  p += align256((size_t)bh * nq * sizeof(float));
  float* rpart = reinterpret_cast<float*>(p);           // q: bh x nblk_q, then k: bh x nblk_k
  float* rpart_k = rpart + (int64_t)bh * pl.nblk_q;
  float* state = reinterpret_cast<float*>(ws + pl.fixed_bytes);
  const int hb = heads_per_batch(pl, ws_bytes, saved != nullptr);

  if (!given) FM_TRY(compute_scales<T>(ds, L, q, k, scale_ws, arg_ws, stream));
  if constexpr (D == 64) {
    if (pl.scan) {   // (plain tensors, nq == nk)
      const int n = nq;
      const float* qs = scale;
      const float* ks = scale + bh;
      // one normalisation partial per head, shared by q and k:
      // sum_i dq_hat_i . q_hat_i = sum_ij W_ij s_ij = sum_j dk_hat_j . k_hat_j
      float* rq = rpart;
      // the dq kernel forms c_i itself when the forward output has plain rows; otherwise the
      // separate pass does
      const bool prep_in_dq = ldo == D;
      if (!prep_in_dq) {
        FM_TRY((launch_bwd_prep<T>(pl, L, go, o, den, den_stride, cvec, stream)));
      }
      {
        ScopedKernel sk(FASTMAX_K_BWD_DQ, stream);
#define FM_DQ(NORM, PREP)                                                                                   \
  lin::linear_dq_kernel<T, NORM, PREP><<<bh, 64, 0, stream>>>(go, den, den_stride, cvec, o, q, k, v, qs, ks, dq, rq, \
                                                              n, ds->a0, ds->a1)
        if (ds->normalize) {
          if (prep_in_dq) FM_DQ(true, true); else FM_DQ(true, false);
        } else {
          if (prep_in_dq) FM_DQ(false, true); else FM_DQ(false, false);
        }
#undef FM_DQ
      }
      FM_TRY(launch_status("linear_dq_kernel"));
      {
        ScopedKernel sk(FASTMAX_K_BWD_DK, stream);
        lin::linear_dk_kernel<T><<<bh, 64, 0, stream>>>(go, den, den_stride, cvec, q, v, qs, ks, dk, n, ds->a1);
      }
      FM_TRY(launch_status("linear_dk_kernel"));
      {
        ScopedKernel sk(FASTMAX_K_BWD_DV, stream);
        lin::linear_dv_kernel<T><<<bh, 64, 0, stream>>>(go, den, den_stride, q, k, qs, ks, dv, n, ds->a0, ds->a1);
      }
      FM_TRY(launch_status("linear_dv_kernel"));
      if (ds->normalize) {
        ScopedKernel sk(FASTMAX_K_NORM_FIX, stream);
        norm_fix_kernel<T><<<2 * bh, D, 0, stream>>>(NormFixSide<T>{mk_rows(dq, L.dq), mk_rows(q, L.q), qs, arg, rq, bh, 1, n},
                                                     NormFixSide<T>{mk_rows(dk, L.dk), mk_rows(k, L.k), ks, arg + bh, rq, bh, 1, n},
                                                     D, ds->lim);
        FM_TRY(launch_status("norm_fix_kernel"));
      }
      return FASTMAX_OK;
    }
  }
  {
    FM_TRY((launch_bwd_prep<T>(pl, L, go, o, den, den_stride, cvec, stream)));
  }
  const float a2 = pl.p2 ? ds->a2 : 0.f;
  const int ratio = pl.ratio, bhkv = pl.bhkv;
  const int64_t state_bytes = (int64_t)pl.nslots * pl.state_floats * sizeof(float);
  // positions the own rows of the query-side / key-side kernels run over, and where the query-side
  // rows start (the queries sit at positions off .. nk-1 under the mask)
  const int nown_q = pl.masked ? nk : nq, nown_k = nk, off = pl.off;
  for (int h0 = 0; h0 < bh; h0 += hb) {
    const int heads = bh - h0 < hb ? bh - h0 : hb;
    const int kv0 = h0 / ratio;                // first key/value head of the batch
    // prefix states: the ones the forward pass saved, or rebuilt into the workspace
    const float* stS = saved ? saved + (int64_t)kv0 * pl.nslots * pl.state_floats : state;
    float* stR = saved ? state : state + (int64_t)hb * pl.nslots * pl.state_floats;
    if constexpr (D == 64) {
      if (pl.rowpass) {   // (plain tensors, nq == nk)
        const int n = nq;
        const int64_t toff = (int64_t)h0 * n * D, koff = (int64_t)kv0 * n * D;
        const float* denh = den + (int64_t)h0 * n * den_stride;
        const float* ch = cvec + (int64_t)h0 * n;
        // states of the whole sequence in fp32 (S as the forward pass left it when it was kept), then one
        // pass over the rows per gradient
        const int64_t ss = pl.state_floats, hf = (int64_t)pl.nslots * ss;
        // (kept bf16 states carry their fp32 sum in slot 0, the packed form in the last slot)
        int slot = (pl.nparts > 1 && !(saved && kBf16Mfma<T>)) ? pl.nparts : 0;
        if (!saved) {
          FM_TRY((launch_build<D, T>(pl, heads, n, mk_rows(k, L.k, kv0), mk_rows(v, L.v, kv0), scale + bh + kv0,
                                     kNoScalars, kNoScalars, state, 0, stream, false)));
          slot = finish_state_fp32(pl, heads, state, stream);
        }
        FM_TRY((launch_build<D, T>(pl, heads, n, mk_rows(q, L.q, h0), mk_rows(go, L.go, h0), scale + h0,
                                   mk_scalars(den, n, den_stride, h0), mk_scalars<const float>(cvec, n, 1, h0), stR, 1,
                                   stream, false)));
        const int slot_r = finish_state_fp32(pl, heads, stR, stream);
        const int nrb = (n + lin::ROWS_PER_WAVE - 1) / lin::ROWS_PER_WAVE;
        const dim3 rgrid(nrb, heads);
        {
          ScopedKernel sk(FASTMAX_K_BWD_DQ, stream);
          if (ds->normalize)
            lin::linear_rowpass_kernel<T, lin::ROWPASS_DQ, true, true><<<rgrid, 64, 0, stream>>>(
                go + toff, stS + slot * ss, hf, scale + h0, denh, den_stride, ch, q + toff, dq + toff, D, nullptr,
                rpart + (int64_t)h0 * nrb, n, ds->a0, ds->a1);
          else
            lin::linear_rowpass_kernel<T, lin::ROWPASS_DQ, false, true><<<rgrid, 64, 0, stream>>>(
                go + toff, stS + slot * ss, hf, scale + h0, denh, den_stride, ch, q + toff, dq + toff, D, nullptr,
                nullptr, n, ds->a0, ds->a1);
        }
        FM_TRY(launch_status("linear_rowpass_kernel (dq)"));
        {
          ScopedKernel sk(FASTMAX_K_BWD_DK, stream);
          lin::linear_rowpass_kernel<T, lin::ROWPASS_DK, false, true><<<rgrid, 64, 0, stream>>>(
              v + koff, stR + slot_r * ss, hf, scale + bh + kv0, nullptr, 0, nullptr, nullptr, dk + toff, D, nullptr,
              nullptr, n, ds->a0, ds->a1);
        }
        FM_TRY(launch_status("linear_rowpass_kernel (dk)"));
        {
          ScopedKernel sk(FASTMAX_K_BWD_DV, stream);
          lin::linear_rowpass_kernel<T, lin::ROWPASS_DV, false, true><<<rgrid, 64, 0, stream>>>(
              k + koff, stR + slot_r * ss, hf, scale + bh + kv0, nullptr, 0, nullptr, nullptr, dv + toff, D, nullptr,
              nullptr, n, ds->a0, ds->a1);
        }
        FM_TRY(launch_status("linear_rowpass_kernel (dv)"));
        continue;
      }
    }
    const Rows<const T> kr = mk_rows(k, L.k, kv0), vr = mk_rows(v, L.v, kv0);
    const Rows<const T> qr = mk_rows(q, L.q, h0, off), gr = mk_rows(go, L.go, h0, off);
    const RowScalars dn = mk_scalars(den, nq, den_stride, h0, off);
    const RowScalars cv = mk_scalars<const float>(cvec, nq, 1, h0, off);
    // grouped key/value heads: dk and dv per query head (plain arrays in the workspace), added up
    // over each group afterwards
    Rows<T> dk_q = mk_rows(dk, L.dk, kv0), dv_q = mk_rows(dv, L.dv, kv0);
    T* dk_tmp = nullptr;
    T* dv_tmp = nullptr;
    if (ratio > 1) {
      char* tmp = reinterpret_cast<char*>(state) + (saved ? 1 : 2) * hb * state_bytes;
      dk_tmp = reinterpret_cast<T*>(tmp);
      dv_tmp = dk_tmp + (int64_t)hb * nk * D;
      dk_q = mk_rows(dk_tmp, plain_str(nk, D));
      dv_q = mk_rows(dv_tmp, plain_str(nk, D));
    }
    // prefix state of (kh, v, 1) per key/value head and suffix state of (qh, go/den, c) per query head
    // (scratch of a split build: behind everything else of the batch in the workspace)
    float* scratch = reinterpret_cast<float*>(ws + pl.fixed_bytes + (size_t)hb * (batch_bytes_per_head(pl, saved != nullptr) - pl.scratch_bytes));
    if (!saved)
      FM_TRY((launch_build<D, T>(pl, heads / ratio, nk, kr, vr, scale + bh + kv0, kNoScalars, kNoScalars, state, 0,
                                 stream, true, scratch)));
    FM_TRY((launch_build<D, T>(pl, heads, nown_q, qr, gr, scale + h0, dn, cv, stR, 1, stream, true, scratch)));
    {
      ScopedKernel sk(FASTMAX_K_BWD_DQ, stream);
      const dim3 grid(pl.nblk_q, heads);
      const Rows<T> dqr = mk_rows(dq, L.dq, h0, off);
      if constexpr (kBf16Mfma<T>) {
        grad_kernel_bf<D, 0><<<grid, 256, 0, stream>>>(
            qr, gr, dn, cv, kr, vr, kNoScalars, scale + h0, scale + bh + kv0, stS, pl.nslots, dqr,
            rpart + (int64_t)h0 * pl.nblk_q, nown_q, pl.chunk, pl.masked, pl.p2, ds->a1, a2, 1, ratio);
      } else {
        grad_kernel<D, T, 0><<<grid, 256, 0, stream>>>(
            qr, gr, dn, cv, kr, vr, kNoScalars, scale + h0, scale + bh + kv0, stS, pl.nslots, dqr,
            rpart + (int64_t)h0 * pl.nblk_q, nown_q, pl.chunk, pl.masked, pl.p2, ds->a1, a2, 1, ratio);
      }
    }
    FM_TRY(launch_status("grad_kernel (dq)"));
    const dim3 kgrid(pl.nblk_k, heads);
    {
      ScopedKernel sk(FASTMAX_K_BWD_DK, stream);
      if constexpr (kBf16Mfma<T>) {
        grad_kernel_bf<D, 1><<<kgrid, 256, 0, stream>>>(
            kr, vr, kNoScalars, cv, qr, gr, dn, scale + bh + kv0, scale + h0, stR, pl.nslots, dk_q,
            rpart_k + (int64_t)h0 * pl.nblk_k, nown_k, pl.chunk, pl.masked, pl.p2, ds->a1, a2, ratio, 1);
      } else {
        grad_kernel<D, T, 1><<<kgrid, 256, 0, stream>>>(
            kr, vr, kNoScalars, cv, qr, gr, dn, scale + bh + kv0, scale + h0, stR, pl.nslots, dk_q,
            rpart_k + (int64_t)h0 * pl.nblk_k, nown_k, pl.chunk, pl.masked, pl.p2, ds->a1, a2, ratio, 1);
      }
    }
    FM_TRY(launch_status("grad_kernel (dk)"));
    {
      ScopedKernel sk(FASTMAX_K_BWD_DV, stream);
      if constexpr (kBf16Mfma<T>) {
        apply_kernel_bf<D, 1><<<kgrid, 256, 0, stream>>>(
            kr, qr, gr, scale + bh + kv0, scale + h0, dn, stR, pl.nslots, dv_q, RowScalarsOut{nullptr, 0, 0}, nown_k,
            pl.chunk, pl.masked, pl.p2, ds->a0, ds->a1, a2, ratio, 1);
      } else {
        apply_kernel<D, T, 1><<<kgrid, 256, 0, stream>>>(
            kr, qr, gr, scale + bh + kv0, scale + h0, dn, stR, pl.nslots, dv_q, RowScalarsOut{nullptr, 0, 0}, nown_k,
            pl.chunk, pl.masked, pl.p2, ds->a0, ds->a1, a2, ratio, 1);
      }
    }
    FM_TRY(launch_status("apply_kernel (dv)"));
    if (ratio > 1) {
      const int64_t per_head = (int64_t)nk * D;
      const dim3 sgrid((unsigned)((per_head / 4 + 255) / 256), heads / ratio);
      group_sum_kernel<T><<<sgrid, 256, 0, stream>>>(dk_tmp, mk_rows(dk, L.dk, kv0), nk, D, ratio);
      group_sum_kernel<T><<<sgrid, 256, 0, stream>>>(dv_tmp, mk_rows(dv, L.dv, kv0), nk, D, ratio);
      FM_TRY(launch_status("group_sum_kernel"));
    }
  }
  if (ds->normalize && pl.rowpass) {
    // one partial per row block of the dq pass; sum_j dk_hat_j . k_hat_j is the same number
    const int nrb = (nq + lin::ROWS_PER_WAVE - 1) / lin::ROWS_PER_WAVE;
    ScopedKernel sk(FASTMAX_K_NORM_FIX, stream);
    norm_fix_kernel<T><<<2 * bh, D, 0, stream>>>(
        NormFixSide<T>{mk_rows(dq, L.dq), mk_rows(q, L.q), scale, arg, rpart, bh, nrb, nq},
        NormFixSide<T>{mk_rows(dk, L.dk), mk_rows(k, L.k), scale + bh, arg + bh, rpart, bh, nrb, nk}, D, ds->lim);
    FM_TRY(launch_status("norm_fix_kernel"));
  } else if (ds->normalize) {
    ScopedKernel sk(FASTMAX_K_NORM_FIX, stream);
    norm_fix_kernel<T><<<bh + bhkv, D, 0, stream>>>(
        NormFixSide<T>{mk_rows(dq, L.dq), mk_rows(q, L.q), scale, arg, rpart, bh, pl.nblk_q, nq},
        NormFixSide<T>{mk_rows(dk, L.dk), mk_rows(k, L.k), scale + bh, arg + bh, rpart_k, bhkv, pl.nblk_k * ratio, nk}, D,
        ds->lim);
    FM_TRY(launch_status("norm_fix_kernel"));
  }
  return FASTMAX_OK;
}

// ---- dense score-tile path (fm_dense.h) ---------------------------------------------------------
// Blocks that need more than the 64 KB of LDS a kernel gets by default ask for it by attribute.
int allow_lds(const void* kernel, size_t bytes) {
  if (bytes <= (size_t)64 * 1024) return FASTMAX_OK;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) return fail(FASTMAX_E_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS): %s", bytes, hipGetErrorString(e));
  return FASTMAX_OK;
}

// The states of the dense kernels' linear mode.  Key side: cscale sum k (x) v and the sums of k, of v of every chunk
// of keys alone, then (masked) of the chunks before each / (unmasked) of all, in slot 0; the forward kernel reads rows
// of the transposed block, dq of the natural one.  Query side (backward; qstate == nullptr: none): qs a1 sum q (x) g,
// sum c q, sum g (g = grad_out / den) of every chunk of queries alone, then of the chunks after each / of all, in both
// layouts.  One state launch and one scan launch serve both sides.
template <int DP, class T>
int dense_lin_states(const fastmax_desc* ds, const Plan& pl, const Layout& L, const T* q, const T* k, const T* v,
                     const T* go, const float* den, int64_t den_stride, const float* cvec, const float* scale,
                     bool transposed, float* kstate, float* qstate, hipStream_t stream) {
  const int npos = pl.masked ? pl.nk : pl.nq;
  const RowScalars none{nullptr, 0, 0};
  dense::StateSide<T> ks{mk_rows(k, L.k), mk_rows(v, L.v), none, none, nullptr, ds->a1, kstate, 1,
                         transposed ? -1 : 0, transposed ? 0 : -1, pl.nk, pl.bhkv};
  dense::StateSide<T> qs = ks;
  qs.heads = 0;
  const int64_t sfk = dense::LinState<DP>::floats(1), sfq = dense::LinState<DP>::floats(2);
  if (qstate)
    qs = dense::StateSide<T>{mk_rows(q, L.q, 0, pl.off), mk_rows(go, L.go, 0, pl.off), mk_scalars(den, pl.nq, den_stride, 0, pl.off),
                             mk_scalars<const float>(cvec, pl.nq, 1, 0, pl.off), scale, ds->a1, qstate, 2, 0, 1, npos, pl.bh};
  ScopedKernel sk(FASTMAX_K_BUILD, stream);
  dense::dense_state_kernel<DP, T><<<dim3(ks.heads + qs.heads, pl.lslots), 256, 0, stream>>>(ks, qs, ds->d, pl.lchunk);
  const int64_t sfmax = qstate ? sfq : sfk;
  dense::lin_scan_kernel<<<dim3((unsigned)((sfmax / 4 + 255) / 256), ks.heads + qs.heads), 256, 0, stream>>>(
      kstate, sfk, ks.heads, pl.masked ? 0 : 2, qstate, sfq, pl.masked ? 1 : 2, pl.lslots);
  return launch_status("dense_state_kernel");
}

template <int DP, class T>
int dense_forward_dp(const fastmax_desc* ds, const Plan& pl, const Layout& L, const T* q, const T* k, const T* v, T* o,
                     float* den, int64_t den_stride, const float* scale, float* kstate, hipStream_t stream) {
  using S = dense::Shape<DP, T>;
  constexpr int RT = S::RT_FWD, BN = S::BN, NW = S::NW_FWD, BM = 32 * RT * NW;
  static_assert(256 % BM == 0 && 256 % BN == 0, "blocks and stages do not straddle the chunks of the linear mode");
  const size_t smem = dense::Lds<DP, T, BN>::bytes(1, 1, BM);
  auto kern = dense::dense_fwd_kernel<DP, T, RT, BN, NW>;
  FM_TRY(allow_lds(reinterpret_cast<const void*>(kern), smem));
  const int npos = pl.masked ? pl.nk : pl.nq;
  const int nb = (npos + BM - 1) / BM - pl.off / BM;
  if (pl.lin)
    FM_TRY((dense_lin_states<DP, T>(ds, pl, L, q, k, v, nullptr, nullptr, 0, nullptr, scale, true, kstate, nullptr, stream)));
  ScopedKernel sk(FASTMAX_K_FWD_APPLY, stream);
  kern<<<dim3(pl.bh, nb), 64 * NW, smem, stream>>>(mk_rows(q, L.q, 0, pl.off), mk_rows(k, L.k), mk_rows(v, L.v), scale,
                                               scale + pl.bh, mk_rows(o, L.o, 0, pl.off),
                                               mk_scalars(den, pl.nq, den_stride, 0, pl.off), npos, pl.nk, ds->d,
                                               pl.masked, ds->a0, ds->a1, pl.p2 ? ds->a2 : 0.f, pl.ratio,
                                               pl.lin ? kstate : nullptr, pl.lchunk, pl.lslots);
  return launch_status("dense_fwd_kernel");
}

template <class T>
int dense_forward(const fastmax_desc* ds, const Plan& pl, const Layout& L, const T* q, const T* k, const T* v, T* o,
                  float* den, int64_t den_stride, float* scale_out, int32_t* arg_out, char* ws, hipStream_t stream) {
  float* scale = scale_out ? scale_out : reinterpret_cast<float*>(ws);
  int* arg = arg_out ? arg_out : reinterpret_cast<int*>(ws + align256((size_t)2 * pl.bh * sizeof(float)));
  FM_TRY(compute_scales<T>(ds, L, q, k, scale, arg, stream));
  float* kstate = reinterpret_cast<float*>(ws + align256((size_t)2 * pl.bh * sizeof(float)) + align256((size_t)2 * pl.bh * sizeof(int)));
#define FM_DENSE_FWD(DP) return dense_forward_dp<DP, T>(ds, pl, L, q, k, v, o, den, den_stride, scale, kstate, stream)
  if (ds->d <= 32) FM_DENSE_FWD(32);
  if (ds->d <= 64) FM_DENSE_FWD(64);
  if (ds->d <= 96) FM_DENSE_FWD(96);
  FM_DENSE_FWD(128);
#undef FM_DENSE_FWD
}

template <int DP, class T>
int dense_backward_dp(const fastmax_desc* ds, const Plan& pl, const Layout& L, const T* q, const T* k, const T* v,
                      const T* o, const float* den, int64_t den_stride, const T* go, T* dq, T* dk, T* dv,
                      const float* scale, float* cvec_w, float* rpart, float* kstate, float* qstate, int* nbq_out,
                      int* nbk_out, hipStream_t stream) {
  // c_i = grad_out_i . out_i / den_i: the dq kernel forms it from rows it holds anyway and leaves it in cvec for the
  // dk / dv kernel -- except in the linear mode, whose query-side states need it before any of them runs
  const bool prep_in_dq = !pl.lin;
  if (!prep_in_dq) FM_TRY((launch_bwd_prep<T>(pl, L, go, o, den, den_stride, cvec_w, stream)));
  const float* cvec = cvec_w;
  using S = dense::Shape<DP, T>;
  constexpr int BN = S::BN;
  const int npos = pl.masked ? pl.nk : pl.nq;
  const float a2 = pl.p2 ? ds->a2 : 0.f;
  float* rq = ds->normalize ? rpart : nullptr;
  const RowScalars dn = mk_scalars(den, pl.nq, den_stride, 0, pl.off);
  const RowScalars cv = mk_scalars<const float>(cvec, pl.nq, 1, 0, pl.off);
  const Rows<const T> qr = mk_rows(q, L.q, 0, pl.off), gr = mk_rows(go, L.go, 0, pl.off);
  const Rows<const T> kr = mk_rows(k, L.k), vr = mk_rows(v, L.v);
  if (pl.lin)
    FM_TRY((dense_lin_states<DP, T>(ds, pl, L, q, k, v, go, den, den_stride, cvec, scale, false, kstate, qstate, stream)));
  const float* ksl = pl.lin ? kstate : nullptr;
  const float* qsl = pl.lin ? qstate : nullptr;
  {
    constexpr int RT = S::RT_DQ, NW = S::NW_DQ, BM = 32 * RT * NW;
    static_assert(256 % BM == 0, "blocks do not straddle the chunks of the linear mode");
    const size_t smem = dense::Lds<DP, T, BN>::bytes(2, 1, NW);
    auto kern = dense::dense_dq_kernel<DP, T, RT, BN, NW>;
    FM_TRY(allow_lds(reinterpret_cast<const void*>(kern), smem));
    const int nb = (npos + BM - 1) / BM - pl.off / BM;
    *nbq_out = nb;
    ScopedKernel sk(FASTMAX_K_BWD_DQ, stream);
    kern<<<dim3(pl.bh, nb), 64 * NW, smem, stream>>>(qr, gr, dn, cv, kr, vr, scale, scale + pl.bh, mk_rows(dq, L.dq, 0, pl.off), rq,
                                                 npos, pl.nk, ds->d, pl.masked, pl.p2 && a2 != 0.f, ds->a1, a2, pl.ratio,
                                                 ksl, pl.lchunk, pl.lslots, mk_rows(o, L.o, 0, pl.off),
                                                 prep_in_dq ? mk_scalars<float>(cvec_w, pl.nq, 1, 0, pl.off) : RowScalarsOut{nullptr, 0, 0});
    FM_TRY(launch_status("dense_dq_kernel"));
  }
  {
    constexpr int RT = S::RT_KV, NW = S::NW_KV, BM = 32 * RT * NW, BNK = S::BN_KV;
    static_assert(256 % BM == 0 && 256 % BNK == 0, "blocks and stages do not straddle the chunks of the linear mode");
    const size_t smem = dense::Lds<DP, T, BNK>::bytes(2, 2, 2 * BNK + NW);
    auto kern = dense::dense_dkdv_kernel<DP, T, RT, BNK, NW>;
    FM_TRY(allow_lds(reinterpret_cast<const void*>(kern), smem));
    const int nb = (pl.nk + BM - 1) / BM;
    *nbk_out = nb;
    float* rk = ds->normalize ? rpart + (int64_t)pl.bh * (*nbq_out) : nullptr;
    ScopedKernel sk(FASTMAX_K_BWD_DK, stream);
    kern<<<dim3(pl.bhkv, nb), 64 * NW, smem, stream>>>(kr, vr, qr, gr, dn, cv, scale, scale + pl.bh, mk_rows(dk, L.dk),
                                                   mk_rows(dv, L.dv), rk, npos, pl.nk, ds->d, pl.masked, ds->a0, ds->a1,
                                                   a2, pl.ratio, qsl, pl.lchunk, pl.lslots);
    FM_TRY(launch_status("dense_dkdv_kernel"));
  }
  return FASTMAX_OK;
}

template <class T>
int dense_backward(const fastmax_desc* ds, const Plan& pl, const Layout& L, const T* q, const T* k, const T* v,
                   const T* o, const float* den, int64_t den_stride, const T* go, T* dq, T* dk, T* dv,
                   const float* scale_in, const int32_t* arg_in, char* ws, hipStream_t stream) {
  const int bh = pl.bh;
  char* p = ws;
  const bool given = scale_in && arg_in;
  const float* scale = given ? scale_in : reinterpret_cast<float*>(p);
  float* scale_ws = reinterpret_cast<float*>(p);
  p += align256((size_t)2 * bh * sizeof(float));
  const int* arg = given ? arg_in : reinterpret_cast<int*>(p);
  int* arg_ws = reinterpret_cast<int*>(p);
  p += align256((size_t)2 * bh * sizeof(int));
  float* cvec = reinterpret_cast<float*>(p);
  p += align256((size_t)bh * pl.nq * sizeof(float));
  float* rpart = reinterpret_cast<float*>(p);
  p += align256((size_t)bh * (pl.nblk_q + pl.nblk_k) * sizeof(float));
  float* kstate = reinterpret_cast<float*>(p);
  float* qstate = kstate;
  if (pl.lin) qstate = reinterpret_cast<float*>(p + align256((size_t)pl.bhkv * pl.lslots * lin_state_floats(pl.ldp, 1) * sizeof(float)));
  if (!given) FM_TRY(compute_scales<T>(ds, L, q, k, scale_ws, arg_ws, stream));
  int nbq = 0, nbk = 0;
#define FM_DENSE_BWD(DP)                                                                                              \
  FM_TRY((dense_backward_dp<DP, T>(ds, pl, L, q, k, v, o, den, den_stride, go, dq, dk, dv, scale, cvec, rpart, kstate, \
                                   qstate, &nbq, &nbk, stream)))
  if (ds->d <= 32) FM_DENSE_BWD(32);
  else if (ds->d <= 64) FM_DENSE_BWD(64);
  else if (ds->d <= 96) FM_DENSE_BWD(96);
  else FM_DENSE_BWD(128);
#undef FM_DENSE_BWD
  if (ds->normalize) {
    ScopedKernel sk(FASTMAX_K_NORM_FIX, stream);
    norm_fix_kernel<T><<<bh + pl.bhkv, ds->d, 0, stream>>>(
        NormFixSide<T>{mk_rows(dq, L.dq), mk_rows(q, L.q), scale, arg, rpart, bh, nbq, pl.nq},
        NormFixSide<T>{mk_rows(dk, L.dk), mk_rows(k, L.k), scale + bh, arg + bh, rpart + (int64_t)bh * nbq, pl.bhkv, nbk, pl.nk},
        ds->d, ds->lim);
    FM_TRY(launch_status("norm_fix_kernel"));
  }
  return FASTMAX_OK;
}

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

int scratch_on_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(FASTMAX_E_NO_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(FASTMAX_E_NO_DEVICE, "device index %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(FASTMAX_E_NO_DEVICE, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return FASTMAX_OK;
}

constexpr int kDecodeSplits = 8;  // blocks per head in a decode step (row slices of the state)

size_t decode_ws_bytes(const fastmax_desc* ds) {
  return align256((size_t)ds->bh * kDecodeSplits * (ds->d + 4) * sizeof(float));
}

// one state per key/value head: the descriptor handed in has bh = bhkv = the key/value heads
template <int D, class T>
int state_update_impl(const fastmax_desc* ds, const Plan& pl, const T* k, const T* v, const float* kscale,
                      float* state, int accumulate, char* ws, size_t ws_bytes, hipStream_t stream) {
  const int bh = pl.bh, n = pl.nk;
  float* scale = reinterpret_cast<float*>(ws);
  int* arg = reinterpret_cast<int*>(ws + align256((size_t)2 * bh * sizeof(float)));
  float* slots = reinterpret_cast<float*>(ws + pl.fixed_bytes);
  const int hb = heads_per_batch(pl, ws_bytes);
  if (!kscale) {
    fill_scale_kernel<<<(bh + 255) / 256, 256, 0, stream>>>(scale + bh, arg + bh, bh, 1.0f / ds->temperature);
    kscale = scale + bh;
  }
  const int64_t ss = pl.state_floats;
  const Str t = plain_str(n, D);
  for (int h0 = 0; h0 < bh; h0 += hb) {
    const int heads = bh - h0 < hb ? bh - h0 : hb;
    FM_TRY((launch_build<D, T>(pl, heads, n, mk_rows(k, t, h0), mk_rows(v, t, h0), kscale + h0, kNoScalars, kNoScalars,
                               slots, 0, stream, false)));
    state_accumulate_kernel<<<dim3((unsigned)((ss / 4 + 255) / 256), heads), 256, 0, stream>>>(
        state + (int64_t)h0 * ss, ss, slots, pl.nslots, pl.nparts, ss, accumulate);
  }
  return launch_status("state_accumulate_kernel");
}

template <int D, class T>
int decode_impl(const fastmax_desc* ds, const T* q, const T* k, const T* v, const float* qscale,
                const float* kscale, float* state, T* o, int64_t ldo, float* den, int64_t den_stride,
                float* part, hipStream_t stream) {
  const int p2 = ds->p == 2;
  decode_update_kernel<D, T><<<dim3(kDecodeSplits, ds->bhkv), 256, 0, stream>>>(
      q, k, v, qscale, kscale, 1.0f / ds->temperature, state, part, p2, ds->a0, ds->a1, p2 ? ds->a2 : 0.f,
      ds->bh / ds->bhkv);
  decode_finish_kernel<D, T><<<ds->bh, D + 4, 0, stream>>>(part, kDecodeSplits, o, ldo, den, den_stride);
  return launch_status("decode kernels");
}

// The kernels address a row by a 32-bit byte offset from its head's first position.
int check_spans(const fastmax_desc* ds, const Layout& L, int64_t den_stride, bool backward) {
  const int64_t es = ds->dtype == FASTMAX_BF16 ? 2 : 4, lim = (int64_t)1 << 32;
  const int64_t nq = ds->mask ? ds->nk : ds->nq, nk = ds->nk;   // positions (queries sit behind the prefix)
  bool ok = nq * L.q.pitch * es < lim && nk * L.k.pitch * es < lim && nk * L.v.pitch * es < lim &&
            nq * L.o.pitch * es < lim && nq * den_stride * 4 < lim;
  if (backward)
    ok = ok && nq * L.go.pitch * es < lim && nq * L.dq.pitch * es < lim && nk * L.dk.pitch * es < lim &&
         nk * L.dv.pitch * es < lim;
  if (!ok) return fail(FASTMAX_E_SHAPE, "the rows of one head span 4 GiB or more (tokens x token stride)");
  return FASTMAX_OK;
}

// checks a caller's layout and turns it into the kernels' strides (layout == NULL: plain arrays)
int resolve_layout(const fastmax_desc* ds, const fastmax_layout* lay, int64_t ldo, bool backward, Layout* out) {
  if (!lay) {
    *out = plain_layout(ds, ldo);
    return FASTMAX_OK;
  }
  const int ratio = ds->bh / ds->bhkv;
  if (lay->groups < 1 || ds->bhkv % lay->groups != 0)
    return fail(FASTMAX_E_SHAPE, "layout.groups = %d does not divide bhkv = %d", lay->groups, ds->bhkv);
  const size_t es = ds->dtype == FASTMAX_BF16 ? 2 : 4;
  auto one = [&](const fastmax_strides& f, bool kv, bool is_o, const char* name, Str* t) {
    if (f.token < ds->d) return fail(FASTMAX_E_PARAM, "layout.%s.token = %lld < d = %d", name, (long long)f.token, ds->d);
    if (f.batch < 0 || f.group < 0 || f.head < 0) return fail(FASTMAX_E_PARAM, "layout.%s has a negative stride", name);
    *t = make_str(f, lay->groups, kv ? 1 : ratio);
    if (!is_o && !aligned16(*t, es))
      return fail(FASTMAX_E_PARAM, "layout.%s: every stride must be a multiple of 16 bytes", name);
    return (int)FASTMAX_OK;
  };
  // (the rows of one head must span less than 4 GiB: the kernels address them with 32-bit offsets)
  FM_TRY(one(lay->q, false, false, "q", &out->q));
  FM_TRY(one(lay->k, true, false, "k", &out->k));
  FM_TRY(one(lay->v, true, false, "v", &out->v));
  FM_TRY(one(lay->o, false, true, "o", &out->o));
  if (backward) {
    FM_TRY(one(lay->go, false, false, "go", &out->go));
    FM_TRY(one(lay->dq, false, false, "dq", &out->dq));
    FM_TRY(one(lay->dk, true, false, "dk", &out->dk));
    FM_TRY(one(lay->dv, true, false, "dv", &out->dv));
  } else {
    out->go = out->dq = out->q;
    out->dk = out->dv = out->k;
  }
  return FASTMAX_OK;
}

}  // namespace

extern "C" {

const char* fastmax_version(void) { return "0.1"; }

const char* fastmax_last_error(void) { return g_err; }

int fastmax_profile_begin(void) {
  g_err[0] = 0;
  g_prof.on = true;
  g_prof.used = 0;
  g_prof.cls.clear();
  return FASTMAX_OK;
}

int fastmax_profile_end(fastmax_kernel_times* out) {
  g_err[0] = 0;
  g_prof.on = false;
  if (!out) return fail(FASTMAX_E_NULL, "out is NULL");
  memset(out, 0, sizeof(*out));
  for (size_t e = 0; e + 1 < g_prof.used; e += 2) {
    float ms = 0.f;
    if (hipEventSynchronize(g_prof.ev[e + 1]) != hipSuccess ||
        hipEventElapsedTime(&ms, g_prof.ev[e], g_prof.ev[e + 1]) != hipSuccess)
      return fail(FASTMAX_E_LAUNCH, "event timing failed: %s", hipGetErrorString(hipGetLastError()));
    const int c = g_prof.cls[e / 2];
    out->ms[c] += ms;
    out->launches[c] += 1;
  }
  g_prof.used = 0;
  g_prof.cls.clear();
  return FASTMAX_OK;
}

int fastmax_check_desc(const fastmax_desc* desc) {
  g_err[0] = 0;
  return check_desc(desc);
}

int fastmax_uses_dense_tiles(const fastmax_desc* desc) {
  g_err[0] = 0;
  FM_TRY(check_desc(desc));
  return use_dense(desc) ? 1 : 0;
}

// (a layout only matters through "plain or not": plain tensors may take the register-resident
// p = 1 paths, which need no state memory)
static bool layout_is_plain(const fastmax_desc* desc, const fastmax_layout* layout, bool backward) {
  if (!layout) return true;
  Layout L;
  if (resolve_layout(desc, layout, desc->d, backward, &L) != FASTMAX_OK) return false;
  return is_plain(L, desc, backward) && L.o.pitch == desc->d;
}

size_t fastmax_workspace_min_bytes_strided(const fastmax_desc* desc, const fastmax_layout* layout, int pass) {
  g_err[0] = 0;
  if (check_desc(desc) != FASTMAX_OK) return 0;
  if (pass != FASTMAX_PASS_FORWARD && pass != FASTMAX_PASS_BACKWARD) {
    fail(FASTMAX_E_PARAM, "pass = %d", pass);
    return 0;
  }
  const Plan pl = make_plan(desc, pass, layout_is_plain(desc, layout, pass == FASTMAX_PASS_BACKWARD));
  return pl.fixed_bytes + pl.ratio * pl.per_head_bytes;  // one whole key/value group
}

size_t fastmax_workspace_bytes_strided(const fastmax_desc* desc, const fastmax_layout* layout, int pass) {
  const size_t mn = fastmax_workspace_min_bytes_strided(desc, layout, pass);
  if (!mn) return 0;
  const Plan pl = make_plan(desc, pass, layout_is_plain(desc, layout, pass == FASTMAX_PASS_BACKWARD));
  if (!pl.per_head_bytes) return mn;
  size_t heads = (kWorkspaceBudget - (pl.fixed_bytes < kWorkspaceBudget ? pl.fixed_bytes : 0)) / pl.per_head_bytes;
  if (heads < (size_t)pl.ratio) heads = pl.ratio;
  if (heads > (size_t)pl.bh) heads = pl.bh;
  return pl.fixed_bytes + heads * pl.per_head_bytes;
}

size_t fastmax_saved_state_bytes_strided(const fastmax_desc* desc, const fastmax_layout* layout) {
  g_err[0] = 0;
  if (check_desc(desc) != FASTMAX_OK) return 0;
  return saved_bytes_for(make_plan(desc, FASTMAX_PASS_FORWARD, layout_is_plain(desc, layout, false)));
}

size_t fastmax_workspace_min_bytes(const fastmax_desc* desc, int pass) {
  return fastmax_workspace_min_bytes_strided(desc, nullptr, pass);
}
size_t fastmax_workspace_bytes(const fastmax_desc* desc, int pass) {
  return fastmax_workspace_bytes_strided(desc, nullptr, pass);
}
size_t fastmax_saved_state_bytes(const fastmax_desc* desc) { return fastmax_saved_state_bytes_strided(desc, nullptr); }

static int forward_entry(const fastmax_desc* desc, const fastmax_layout* layout, const void* q, const void* k,
                         const void* v, void* o, int64_t ldo, float* den, int64_t den_stride, float* qk_scale,
                         int32_t* qk_argmax, void* workspace, size_t workspace_bytes, void* saved_states,
                         size_t saved_bytes, fastmax_stream_t stream) {
  g_err[0] = 0;
  FM_TRY(check_desc(desc));
  if (!q || !k || !v || !o || !den) return fail(FASTMAX_E_NULL, "q, k, v, o and den must be non-NULL");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v)) return fail(FASTMAX_E_PARAM, "q, k and v must be 16-byte aligned");
  if (ldo < desc->d) return fail(FASTMAX_E_PARAM, "ldo = %lld < d = %d", (long long)ldo, desc->d);
  if (den_stride < 1) return fail(FASTMAX_E_PARAM, "den_stride = %lld < 1", (long long)den_stride);
  Layout L;
  FM_TRY(resolve_layout(desc, layout, ldo, false, &L));
  FM_TRY(check_spans(desc, L, den_stride, false));
  const Plan pl = make_plan(desc, FASTMAX_PASS_FORWARD, is_plain(L, desc, false));
  FM_TRY(check_ws(pl, workspace, workspace_bytes, saved_states != nullptr));
  FM_TRY(check_saved(pl, saved_states, saved_bytes));
  char* ws = static_cast<char*>(workspace);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (pl.dense) {
    if (desc->dtype == FASTMAX_F32)
      return dense_forward<float>(desc, pl, L, (const float*)q, (const float*)k, (const float*)v, (float*)o, den,
                                  den_stride, qk_scale, qk_argmax, ws, st);
    return dense_forward<bf16_t>(desc, pl, L, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, (bf16_t*)o, den,
                                 den_stride, qk_scale, qk_argmax, ws, st);
  }
#define FM_FWD(DD, TT)                                                                             \
  return forward_impl<DD, TT>(desc, pl, L, (const TT*)q, (const TT*)k, (const TT*)v, (TT*)o, den, \
                              den_stride, qk_scale, qk_argmax, ws, workspace_bytes, (float*)saved_states, st)
  if (desc->dtype == FASTMAX_F32) {
    if (desc->d == 64) FM_FWD(64, float);
    FM_FWD(32, float);
  }
  if (desc->d == 64) FM_FWD(64, bf16_t);
  FM_FWD(32, bf16_t);
#undef FM_FWD
}

int fastmax_forward_saving(const fastmax_desc* desc, const void* q, const void* k, const void* v, void* o,
                           int64_t ldo, float* den, int64_t den_stride, float* qk_scale,
                           int32_t* qk_argmax, void* workspace, size_t workspace_bytes,
                           void* saved_states, size_t saved_bytes, fastmax_stream_t stream) {
  return forward_entry(desc, nullptr, q, k, v, o, ldo, den, den_stride, qk_scale, qk_argmax, workspace,
                       workspace_bytes, saved_states, saved_bytes, stream);
}

int fastmax_forward_strided(const fastmax_desc* desc, const fastmax_layout* layout, const void* q, const void* k,
                            const void* v, void* o, float* den, int64_t den_stride, float* qk_scale,
                            int32_t* qk_argmax, void* workspace, size_t workspace_bytes, void* saved_states,
                            size_t saved_bytes, fastmax_stream_t stream) {
  if (!layout) {
    g_err[0] = 0;
    return fail(FASTMAX_E_NULL, "layout is NULL");
  }
  return forward_entry(desc, layout, q, k, v, o, layout->o.token, den, den_stride, qk_scale, qk_argmax, workspace,
                       workspace_bytes, saved_states, saved_bytes, stream);
}

int fastmax_forward(const fastmax_desc* desc, const void* q, const void* k, const void* v, void* o,
                    int64_t ldo, float* den, int64_t den_stride, float* qk_scale,
                    int32_t* qk_argmax, void* workspace, size_t workspace_bytes,
                    fastmax_stream_t stream) {
  return fastmax_forward_saving(desc, q, k, v, o, ldo, den, den_stride, qk_scale, qk_argmax, workspace,
                                workspace_bytes, nullptr, 0, stream);
}

size_t fastmax_noalloc_scratch_bytes(void) {
  // (also the warm-up a graph-capturing caller needs: the per-device address is resolved here)
  void* p = nullptr;
  (void)scratch_on_current_device(&p);
  g_err[0] = 0;
  return FASTMAX_NOALLOC_SCRATCH_BYTES;
}

int fastmax_forward_noalloc(const fastmax_desc* desc, const void* q, const void* k, const void* v, void* o,
                            int64_t ldo, float* den, int64_t den_stride, float* qk_scale,
                            int32_t* qk_argmax, fastmax_stream_t stream) {
  g_err[0] = 0;
  FM_TRY(check_desc(desc));
  const Plan pl = make_plan(desc, FASTMAX_PASS_FORWARD);
  const size_t need = pl.fixed_bytes + pl.ratio * batch_bytes_per_head(pl, false);
  if (need > (size_t)FASTMAX_NOALLOC_SCRATCH_BYTES)
    return fail(FASTMAX_E_WORKSPACE,
                "this problem needs %zu bytes of scratch memory; the allocation-free entry point holds %zu "
                "(use fastmax_forward with a workspace of the caller's)", need, (size_t)FASTMAX_NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  FM_TRY(scratch_on_current_device(&ws));
  // nothing in the forward pass reads scratch memory it has not written in the same call, so the
  // previous call's contents need no clearing
  return fastmax_forward_saving(desc, q, k, v, o, ldo, den, den_stride, qk_scale, qk_argmax, ws,
                                FASTMAX_NOALLOC_SCRATCH_BYTES, nullptr, 0, stream);
}

static int backward_entry(const fastmax_desc* desc, const fastmax_layout* layout, const void* q, const void* k,
                          const void* v, const void* o, int64_t ldo, const float* den, int64_t den_stride,
                          const void* go, void* dq, void* dk, void* dv, const float* qk_scale,
                          const int32_t* qk_argmax, void* workspace, size_t workspace_bytes,
                          const void* saved_states, size_t saved_bytes, fastmax_stream_t stream) {
  g_err[0] = 0;
  FM_TRY(check_desc(desc));
  if (!q || !k || !v || !o || !den || !go || !dq || !dk || !dv)
    return fail(FASTMAX_E_NULL, "q, k, v, o, den, go, dq, dk and dv must be non-NULL");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(go) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv))
    return fail(FASTMAX_E_PARAM, "q, k, v, go, dq, dk and dv must be 16-byte aligned");
  if (ldo < desc->d) return fail(FASTMAX_E_PARAM, "ldo = %lld < d = %d", (long long)ldo, desc->d);
  if (den_stride < 1) return fail(FASTMAX_E_PARAM, "den_stride = %lld < 1", (long long)den_stride);
  Layout L;
  FM_TRY(resolve_layout(desc, layout, ldo, true, &L));
  FM_TRY(check_spans(desc, L, den_stride, true));
  const Plan pl = make_plan(desc, FASTMAX_PASS_BACKWARD, is_plain(L, desc, true));
  if (saved_states) {
    // The kept states are only usable when the forward pass that wrote them (planned on q, k, v, o alone) wrote
    // kept states at all: the register-resident scan and the dense kernels keep nothing (a 256-byte token),
    // and this pass, which also looks at grad_output and the gradients, may plan differently.  Then it
    // rebuilds its states.  (The row passes and the chunked kernels of unmasked p = 1 read the same buffer.)
    const Plan plf = make_plan(desc, FASTMAX_PASS_FORWARD, is_plain(L, desc, false));
    if (plf.scan != pl.scan || plf.dense != pl.dense) {
      saved_states = nullptr;
      saved_bytes = 0;
    }
  }
  FM_TRY(check_ws(pl, workspace, workspace_bytes, saved_states != nullptr));
  FM_TRY(check_saved(pl, saved_states, saved_bytes));
  char* ws = static_cast<char*>(workspace);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (pl.dense) {
    if (desc->dtype == FASTMAX_F32)
      return dense_backward<float>(desc, pl, L, (const float*)q, (const float*)k, (const float*)v, (const float*)o,
                                   den, den_stride, (const float*)go, (float*)dq, (float*)dk, (float*)dv, qk_scale,
                                   qk_argmax, ws, st);
    return dense_backward<bf16_t>(desc, pl, L, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)o,
                                  den, den_stride, (const bf16_t*)go, (bf16_t*)dq, (bf16_t*)dk, (bf16_t*)dv, qk_scale,
                                  qk_argmax, ws, st);
  }
#define FM_BWD(DD, TT)                                                                              \
  return backward_impl<DD, TT>(desc, pl, L, (const TT*)q, (const TT*)k, (const TT*)v, (const TT*)o, \
                               den, den_stride, (const TT*)go, (TT*)dq, (TT*)dk, (TT*)dv, qk_scale,  \
                               qk_argmax, ws, workspace_bytes, (const float*)saved_states, st)
  if (desc->dtype == FASTMAX_F32) {
    if (desc->d == 64) FM_BWD(64, float);
    FM_BWD(32, float);
  }
  if (desc->d == 64) FM_BWD(64, bf16_t);
  FM_BWD(32, bf16_t);
#undef FM_BWD
}

int fastmax_backward_saved(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                           const void* o, int64_t ldo, const float* den, int64_t den_stride,
                           const void* go, void* dq, void* dk, void* dv, const float* qk_scale,
                           const int32_t* qk_argmax, void* workspace, size_t workspace_bytes,
                           const void* saved_states, size_t saved_bytes, fastmax_stream_t stream) {
  return backward_entry(desc, nullptr, q, k, v, o, ldo, den, den_stride, go, dq, dk, dv, qk_scale, qk_argmax,
                        workspace, workspace_bytes, saved_states, saved_bytes, stream);
}

int fastmax_backward_strided(const fastmax_desc* desc, const fastmax_layout* layout, const void* q, const void* k,
                             const void* v, const void* o, const float* den, int64_t den_stride, const void* go,
                             void* dq, void* dk, void* dv, const float* qk_scale, const int32_t* qk_argmax,
                             void* workspace, size_t workspace_bytes, const void* saved_states, size_t saved_bytes,
                             fastmax_stream_t stream) {
  if (!layout) {
    g_err[0] = 0;
    return fail(FASTMAX_E_NULL, "layout is NULL");
  }
  return backward_entry(desc, layout, q, k, v, o, layout->o.token, den, den_stride, go, dq, dk, dv, qk_scale,
                        qk_argmax, workspace, workspace_bytes, saved_states, saved_bytes, stream);
}

int fastmax_backward(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                     const void* o, int64_t ldo, const float* den, int64_t den_stride,
                     const void* go, void* dq, void* dk, void* dv, const float* qk_scale,
                     const int32_t* qk_argmax, void* workspace, size_t workspace_bytes,
                     fastmax_stream_t stream) {
  return fastmax_backward_saved(desc, q, k, v, o, ldo, den, den_stride, go, dq, dk, dv, qk_scale, qk_argmax,
                                workspace, workspace_bytes, nullptr, 0, stream);
}

int fastmax_normalize_inplace(const fastmax_desc* desc, void* q, void* k, void* workspace,
                              size_t workspace_bytes, fastmax_stream_t stream) {
  g_err[0] = 0;
  FM_TRY(check_desc(desc));
  if (!q || !k) return fail(FASTMAX_E_NULL, "q and k must be non-NULL");
  if (!workspace || (((uintptr_t)workspace) & 255) || workspace_bytes < (size_t)16 * desc->bh + 512)
    return fail(FASTMAX_E_WORKSPACE, "workspace must be 256-byte aligned and hold 16*bh+512 bytes");
  if (!desc->normalize) return FASTMAX_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int bh = desc->bh;
  float* scale = static_cast<float*>(workspace);
  int* arg = reinterpret_cast<int*>(static_cast<char*>(workspace) + align256((size_t)2 * bh * sizeof(float)));
  const int64_t per_head = (int64_t)desc->nq * desc->d, per_head_k = (int64_t)desc->nk * desc->d;
  const dim3 grid((unsigned)((per_head / 4 + 255) / 256), bh);
  const dim3 kgrid((unsigned)((per_head_k / 4 + 255) / 256), desc->bhkv);
  const Layout L = plain_layout(desc, desc->d);
  if (desc->dtype == FASTMAX_F32) {
    FM_TRY(compute_scales<float>(desc, L, (const float*)q, (const float*)k, scale, arg, st));
    scale_rows_kernel<float><<<grid, 256, 0, st>>>((float*)q, scale, per_head);
    scale_rows_kernel<float><<<kgrid, 256, 0, st>>>((float*)k, scale + bh, per_head_k);
  } else {
    FM_TRY(compute_scales<bf16_t>(desc, L, (const bf16_t*)q, (const bf16_t*)k, scale, arg, st));
    scale_rows_kernel<bf16_t><<<grid, 256, 0, st>>>((bf16_t*)q, scale, per_head);
    scale_rows_kernel<bf16_t><<<kgrid, 256, 0, st>>>((bf16_t*)k, scale + bh, per_head_k);
  }
  return launch_status("scale_rows_kernel");
}

// The recurrent form keeps a moment state per head: it exists for the head dimensions the moment
// kernels are built for.
static int check_recurrent(const fastmax_desc* desc) {
  FM_TRY(check_desc(desc));
  if (desc->d != 32 && desc->d != 64)
    return fail(FASTMAX_E_SHAPE, "d = %d: the recurrent entry points keep moment states, which exist for d = 32 and 64", desc->d);
  return FASTMAX_OK;
}

size_t fastmax_state_bytes(const fastmax_desc* desc) {
  g_err[0] = 0;
  if (check_recurrent(desc) != FASTMAX_OK) return 0;
  return (size_t)state_floats_for(desc->d, desc->p == 2) * sizeof(float);
}

size_t fastmax_decode_workspace_bytes(const fastmax_desc* desc) {
  g_err[0] = 0;
  if (check_recurrent(desc) != FASTMAX_OK) return 0;
  return decode_ws_bytes(desc);
}

int fastmax_state_update(const fastmax_desc* desc, const void* k, const void* v, const float* k_scale,
                         void* state, int accumulate, void* workspace, size_t workspace_bytes,
                         fastmax_stream_t stream) {
  g_err[0] = 0;
  FM_TRY(check_recurrent(desc));
  if (!k || !v || !state) return fail(FASTMAX_E_NULL, "k, v and state must be non-NULL");
  if (desc->normalize && !k_scale)
    return fail(FASTMAX_E_NULL, "normalize is set: k_scale (the factor a forward pass reported) is required");
  // one state per key/value head: the build runs over the bhkv heads of k, v
  fastmax_desc d2 = *desc;
  d2.mask = 0;
  d2.bh = d2.bhkv;
  d2.nq = d2.nk;
  const Plan pl = make_plan(&d2, FASTMAX_PASS_FORWARD, true, false);   // (the moment state itself is wanted)
  FM_TRY(check_ws(pl, workspace, workspace_bytes));
  char* ws = static_cast<char*>(workspace);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
#define FM_UPD(DD, TT)                                                                            \
  return state_update_impl<DD, TT>(&d2, pl, (const TT*)k, (const TT*)v, k_scale, (float*)state, \
                                   accumulate, ws, workspace_bytes, st)
  if (desc->dtype == FASTMAX_F32) {
    if (desc->d == 64) FM_UPD(64, float);
    FM_UPD(32, float);
  }
  if (desc->d == 64) FM_UPD(64, bf16_t);
  FM_UPD(32, bf16_t);
#undef FM_UPD
}

int fastmax_decode_step(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                        const float* q_scale, const float* k_scale, void* state, void* o, int64_t ldo,
                        float* den, int64_t den_stride, void* workspace, size_t workspace_bytes,
                        fastmax_stream_t stream) {
  g_err[0] = 0;
  FM_TRY(check_recurrent(desc));
  if (!q || !k || !v || !state || !o) return fail(FASTMAX_E_NULL, "q, k, v, state and o must be non-NULL");
  if (desc->nq != 1 || desc->nk != 1) return fail(FASTMAX_E_SHAPE, "a decode step takes one token per head (nq = nk = 1), got nq = %d", desc->nq);
  if (desc->normalize && (!q_scale || !k_scale))
    return fail(FASTMAX_E_NULL, "normalize is set: q_scale and k_scale (the factors a forward pass reported) are required");
  if (ldo < desc->d) return fail(FASTMAX_E_PARAM, "ldo = %lld < d = %d", (long long)ldo, desc->d);
  if (den && den_stride < 1) return fail(FASTMAX_E_PARAM, "den_stride = %lld < 1", (long long)den_stride);
  if (!workspace || (((uintptr_t)workspace) & 255) || workspace_bytes < decode_ws_bytes(desc))
    return fail(FASTMAX_E_WORKSPACE, "workspace must be 256-byte aligned and hold %zu bytes", decode_ws_bytes(desc));
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
#define FM_DEC(DD, TT)                                                                              \
  return decode_impl<DD, TT>(desc, (const TT*)q, (const TT*)k, (const TT*)v, q_scale, k_scale,     \
                             (float*)state, (TT*)o, ldo, den, den_stride, (float*)workspace, st)
  if (desc->dtype == FASTMAX_F32) {
    if (desc->d == 64) FM_DEC(64, float);
    FM_DEC(32, float);
  }
  if (desc->d == 64) FM_DEC(64, bf16_t);
  FM_DEC(32, bf16_t);
#undef FM_DEC
}

int fastmax_qkv_rope(const fastmax_rope_desc* desc, int grad, void* qkv, const float* cos, const float* sin,
                     void* q, void* k, void* v, fastmax_stream_t stream) {
  g_err[0] = 0;
  if (!desc) return fail(FASTMAX_E_NULL, "desc is NULL");
  if (!qkv) return fail(FASTMAX_E_NULL, "qkv must be non-NULL");
  if ((k || v) && (!q || !k || !v))
    return fail(FASTMAX_E_NULL, "q, k and v must be all non-NULL (split), q alone (rotated q, k rows packed), or all NULL (in place)");
  if (desc->dtype != FASTMAX_F32 && desc->dtype != FASTMAX_BF16)
    return fail(FASTMAX_E_DTYPE, "dtype %d is neither FASTMAX_F32 nor FASTMAX_BF16", desc->dtype);
  if (desc->b < 1 || desc->t < 1 || desc->groups < 1 || desc->q_per_kv < 1 || desc->hs < 4 || desc->hs % 4)
    return fail(FASTMAX_E_SHAPE, "b, t, groups, q_per_kv must be positive and hs a positive multiple of 4");
  if (desc->rope_n < 0 || desc->rope_n > desc->hs || desc->rope_n % 8)
    return fail(FASTMAX_E_SHAPE, "rope_n = %d must be a multiple of 8 in [0, hs]", desc->rope_n);
  if (desc->rope_n > 0 && (!cos || !sin)) return fail(FASTMAX_E_NULL, "cos and sin must be non-NULL when rope_n > 0");
  const RopeShape sh{desc->b, desc->t, desc->groups, desc->q_per_kv, desc->hs, desc->rope_n};
  const bool wide = sh.hs % 16 == 0 && sh.rn % 16 == 0;   // 16-channel units, 16-byte accesses
  const int64_t total = (int64_t)sh.b * sh.t * sh.groups * (sh.qpk + 2) * (wide ? sh.hs / 16 : sh.hs / 4);
  if (total >= ((int64_t)1 << 39)) return fail(FASTMAX_E_SHAPE, "tensor too large");
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
#define FM_ROPE(KERNEL, T, G) KERNEL<T, G><<<blocks, 256, 0, st>>>(sh, (T*)qkv, cos, sin, (T*)q, (T*)k, (T*)v)
  if (desc->dtype == FASTMAX_F32) {
    if (wide) { if (grad) FM_ROPE(qkv_rope16_kernel, float, true); else FM_ROPE(qkv_rope16_kernel, float, false); }
    else { if (grad) FM_ROPE(qkv_rope_kernel, float, true); else FM_ROPE(qkv_rope_kernel, float, false); }
  } else {
    if (wide) { if (grad) FM_ROPE(qkv_rope16_kernel, bf16_t, true); else FM_ROPE(qkv_rope16_kernel, bf16_t, false); }
    else { if (grad) FM_ROPE(qkv_rope_kernel, bf16_t, true); else FM_ROPE(qkv_rope_kernel, bf16_t, false); }
  }
#undef FM_ROPE
  return launch_status("qkv_rope_kernel");
}

}  // extern "C"
