/*
 * fastmax_amd.h -- C ABI of the MI355X (gfx950) Fastmax attention library.
 *
 * Fastmax attention replaces the softmax by a row-normalised polynomial score
 *     o_i = sum_j f(q_i.k_j) v_j / sum_j f(q_i.k_j),   f(s) = a0 + a1 s + a2 s^2  (p=2)
 * (j <= i when mask != 0).  This header is the whole drop-in boundary for that path:
 * plain pointers and sizes, no torch types.  Every entry point is asynchronous on the
 * given stream, allocates nothing on the device, keeps no state between calls (the built-in
 * scratch array of fastmax_forward_noalloc and the opt-in kernel timer at the end of this
 * header aside) and returns 0 or a negative FASTMAX_E_* code (text via fastmax_last_error()).
 *
 * Layout contract (reference: fastmax_cuda_forward.cu:331-336): q, k, v, grad_output and
 * the gradients are (bh, n, d) row-major with d contiguous; a (b,h,n,d) tensor is the
 * same memory.  The output may carry a row pitch ldo >= d so that the reference's
 * (bh, n, d+1) "o with the denominator in column d" (fastmax_cuda_forward.cu:353,
 * example.py:47) is written in place: pass ldo = d+1, den = o + d, den_stride = d+1.
 * q, k, v, grad_output and the gradients must be 16-byte aligned.  The *_strided entry points
 * take the same tensors with explicit batch / group / head / token strides (fastmax_layout), e.g.
 * views into a fused (b, t, groups*(q_per_kv+2)*hs) projection and a token-major (b, t, h*hs)
 * output, which is how the reference's GPT block holds them before its permute / .contiguous()
 * copies (model.py:474-499, 572-574, 603).
 *
 * Key prefix (fastmax_cuda_forward.cu:109-150): with mask != 0 and nk > nq, query i sits at
 * key position i + (nk - nq), i.e. the first nk - nq keys are visible to every query.  With
 * mask == 0 any nq, nk are allowed (every query sees every key).
 */
#ifndef FASTMAX_AMD_H
#define FASTMAX_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* fastmax_stream_t; /* == hipStream_t */

enum {
  FASTMAX_OK = 0,
  FASTMAX_E_NULL = -1,        /* a required pointer is NULL                         */
  FASTMAX_E_SHAPE = -2,       /* unsupported bh / n / d, bhkv not dividing bh, nk < nq under mask */
  FASTMAX_E_DTYPE = -3,       /* dtype not FASTMAX_F32 / FASTMAX_BF16               */
  FASTMAX_E_PARAM = -4,       /* p not in {1,2}, bad lim / temperature / pitch      */
  FASTMAX_E_WORKSPACE = -5,   /* workspace NULL, misaligned or too small            */
  FASTMAX_E_LAUNCH = -6,      /* the HIP runtime refused a launch                   */
  FASTMAX_E_NO_DEVICE = -7    /* no gfx950 device is current                        */
};

enum { FASTMAX_F32 = 0, FASTMAX_BF16 = 1 };
enum { FASTMAX_PASS_FORWARD = 0, FASTMAX_PASS_BACKWARD = 1 };

/* Problem descriptor.  Mirrors the scalar arguments of the reference's
 * forwardpass(q,k,v,drop_noise,mask,dropout,normalize,temperature,a0,a1,a2,lim,p)
 * (fastmax_cuda.cpp:17, fastmax_cuda_forward.cu:297-314) plus the sizes its launcher reads
 * from the tensors (fastmax_cuda_forward.cu:331-336). */
typedef struct fastmax_desc {
  int32_t bh;          /* query heads  (b*h)                                             */
  int32_t bhkv;        /* key/value heads; divides bh: query head i reads key/value head
                          i / (bh / bhkv)  (fastmax_cuda_forward.cu:38); k, v, dk, dv are
                          then (bhkv, n, d)                                              */
  int32_t nq;          /* query tokens                                                   */
  int32_t nk;          /* key tokens; mask != 0: nk >= nq, the first nk - nq keys are a
                          prefix every query sees (fastmax_cuda_forward.cu:109-150)      */
  int32_t d;           /* head dimension, read at run time like the reference's launcher does
                          (fastmax_cuda_forward.cu:331-338): any whole number of 16-byte
                          pieces of a row (a multiple of 4 for fp32, of 8 for bf16) up to
                          128.  d = 32 and 64 have both kernel families (moment states,
                          linear in n; dense score tiles for short sequences); every other
                          d runs on the dense score tiles, whose cost grows with nq * nk   */
  int32_t dtype;       /* FASTMAX_F32 or FASTMAX_BF16 (bf16 in/out, fp32 accumulation)    */
  int32_t mask;        /* 0: every key visible, 1: causal (j <= i)                       */
  int32_t normalize;   /* 1: x <- lim * x / max_n ||x_n||_2 per head for q and k,
                          differentiated through (example.py:101-108)                    */
  int32_t p;           /* polynomial order, 1 or 2                                       */
  float lim;           /* see normalize                                                  */
  float temperature;   /* used only when normalize == 0: k <- k / temperature
                          (fastmax_cuda_forward.cu:212-221,366; gradk / temperature at
                          example.py:80)                                                 */
  float a0, a1, a2;    /* score coefficients                                             */
} fastmax_desc;

/* Library version, "major.minor". */
const char* fastmax_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char* fastmax_last_error(void);

/* Checks a descriptor without touching the device.  Replaces the shape reads and the
 * implicit assumptions of fastmax_cuda_forward.cu:331-345 (d == 64). */
int fastmax_check_desc(const fastmax_desc* desc);

/* Which kernel family a descriptor runs on: 1 = dense score tiles (no states, no state memory, work
 * ~ nq * nk * d), 0 = moment states (work ~ n * d^3 for p = 2), negative = bad descriptor.  d = 32 and
 * 64 have both and the library picks the faster one by sequence length; the environment variable
 * FASTMAX_PATH = moments | dense overrides that choice (read at every call).  No counterpart in the
 * reference, whose kernels are the moment form only (fastmax_cuda_forward.cu:25-197). */
int fastmax_uses_dense_tiles(const fastmax_desc* desc);

/* Bytes of device workspace that let a pass run all heads in as few batches as a 16 GiB
 * budget allows (the passes accept anything >= fastmax_workspace_min_bytes and then loop
 * over smaller head batches).  Replaces the torch::zeros scratch tensors of
 * fastmax_cuda_forward.cu:353-357 and fastmax_cuda_backward.cu:957-959.  0 on error. */
size_t fastmax_workspace_bytes(const fastmax_desc* desc, int pass);
size_t fastmax_workspace_min_bytes(const fastmax_desc* desc, int pass);

/* Forward pass.  Replaces forward_cuda (fastmax_cuda_forward.cu:297-411).
 *   q           (bh, n, d)             input, never modified
 *   k, v        (bhkv, n, d)           inputs, never modified
 *   o           (bh, n, ldo >= d)      out: attention output, columns [0,d)
 *   den         den[(h*n+i)*den_stride] out: row denominators sum_j f(s_ij); may alias
 *                                      column d of o (see layout contract)
 *   qk_scale    2*bh floats or NULL    out: per-head factors applied to q (bh values) then k
 *                                      (bhkv values, from index bh);
 *                                      (lim / max row norm, 1/temperature, or 1)
 *   qk_argmax   2*bh int32 or NULL     out: row index of the max-norm row per head
 *   workspace   256-byte aligned device memory of workspace_bytes bytes               */
int fastmax_forward(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                    void* o, int64_t ldo, float* den, int64_t den_stride,
                    float* qk_scale, int32_t* qk_argmax,
                    void* workspace, size_t workspace_bytes, fastmax_stream_t stream);

/* Backward pass.  Replaces backward_cuda (fastmax_cuda_backward.cu:900-1006) and adds the
 * chain rule through the normalisation that autograd applies to the reference's PyTorch
 * path (example.py:101-108).
 *   q, k, v, o, den  as given to / produced by fastmax_forward (q, k un-normalised)
 *   go               (bh, n, d) upstream gradient, never modified (the reference divides it
 *                    in place, fastmax_cuda_backward.cu:874-882,970)
 *   dq               (bh, n, d) out;  dk, dv  (bhkv, n, d) out
 *   qk_scale, qk_argmax  values written by fastmax_forward, or NULL to recompute them   */
int fastmax_backward(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                     const void* o, int64_t ldo, const float* den, int64_t den_stride,
                     const void* go, void* dq, void* dk, void* dv,
                     const float* qk_scale, const int32_t* qk_argmax,
                     void* workspace, size_t workspace_bytes, fastmax_stream_t stream);

/* Strided tensors.  A tensor is addressed as (batch b, key/value group g, query head j within
 * the group, token t, channel c) at  b*batch + g*group + j*head + t*token + c  elements from its
 * pointer; key/value tensors (k, v, dk, dv) have no j.  Head index h of the plain entry points is
 * (b*groups + g)*q_per_kv + j for query-side tensors, b*groups + g for key/value tensors, with
 * q_per_kv = bh / bhkv; groups must divide bhkv.  Every stride must keep rows 16-byte aligned
 * (o: any token stride >= d).  No counterpart in the reference's kernels, which require the
 * contiguous (b, h, n, d) copies its callers make (model.py:572-574); this replaces those copies
 * and the transpose of the result (model.py:603).
 * Causal p = 1 at d = 64 with many heads runs as a register-resident scan only for plain
 * contiguous tensors with nq == nk; strided or prefixed calls of that shape use the chunked
 * kernels, so their workspace sizes come from the *_strided queries below (layout == NULL there
 * means contiguous).  den stays (bh, nq) with den_stride between tokens. */
typedef struct fastmax_strides {
  int64_t batch, group, head, token;
} fastmax_strides;
typedef struct fastmax_layout {
  int32_t groups;       /* key/value heads per batch element                              */
  int32_t reserved;     /* 0                                                              */
  fastmax_strides q, k, v, o, go, dq, dk, dv;
} fastmax_layout;
size_t fastmax_workspace_bytes_strided(const fastmax_desc* desc, const fastmax_layout* layout, int pass);
size_t fastmax_workspace_min_bytes_strided(const fastmax_desc* desc, const fastmax_layout* layout, int pass);
size_t fastmax_saved_state_bytes_strided(const fastmax_desc* desc, const fastmax_layout* layout);
/* As fastmax_forward_saving / fastmax_backward_saved (saved_states may be NULL); layout->o.token
 * takes the place of ldo.  The forward pass reads layout->q, k, v, o; the backward pass reads
 * all eight members. */
int fastmax_forward_strided(const fastmax_desc* desc, const fastmax_layout* layout, const void* q,
                            const void* k, const void* v, void* o, float* den, int64_t den_stride,
                            float* qk_scale, int32_t* qk_argmax, void* workspace, size_t workspace_bytes,
                            void* saved_states, size_t saved_bytes, fastmax_stream_t stream);
int fastmax_backward_strided(const fastmax_desc* desc, const fastmax_layout* layout, const void* q,
                             const void* k, const void* v, const void* o, const float* den,
                             int64_t den_stride, const void* go, void* dq, void* dk, void* dv,
                             const float* qk_scale, const int32_t* qk_argmax, void* workspace,
                             size_t workspace_bytes, const void* saved_states, size_t saved_bytes,
                             fastmax_stream_t stream);

/* Keeping the prefix states for the backward pass (no counterpart in the reference, whose
 * backward re-walks the sequence, fastmax_cuda_backward.cu:26-882).  The backward pass needs
 * the same prefix states S of (k, v) the forward pass built; fastmax_backward rebuilds them
 * (one of its three state builds).  A caller with memory to spare passes a buffer of
 * fastmax_saved_state_bytes(desc) bytes (256-byte aligned; bhkv * slots * state bytes, 24 GB
 * at bh = 1024, n = 10000, d = 64, p = 2) to fastmax_forward_saving, keeps it untouched, and
 * hands it to fastmax_backward_saved, which then skips that build.  With saved_states == NULL
 * the two calls are fastmax_forward / fastmax_backward.  When a buffer is given the workspace
 * need not hold the prefix states: 16*bh + 512 bytes suffice for fastmax_forward_saving, and
 * fastmax_backward_saved needs one state per head less.  (The size query is the contract: for
 * causal p = 1 with few heads and bf16 tensors the buffer also holds, behind the states, the
 * fp32 per-chunk partial states the forward pass adds up.)  Kernels that keep nothing answer the
 * size query with a token 256 bytes: the buffer is then left untouched and the two calls need the
 * workspace of fastmax_forward / fastmax_backward.  Those are the one register-resident scan per
 * head of causal p = 1 at d = 64 with at least 512 heads (bf16: 208; workspace: per-head and per-token scalars
 * only) and the dense score tiles (fastmax_uses_dense_tiles; their workspace holds scalars -- and for
 * p = 1 past 1024 causal / 512 unmasked positions the chunk states of their linear mode, which both
 * passes rebuild). */
size_t fastmax_saved_state_bytes(const fastmax_desc* desc);
int fastmax_forward_saving(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                           void* o, int64_t ldo, float* den, int64_t den_stride,
                           float* qk_scale, int32_t* qk_argmax,
                           void* workspace, size_t workspace_bytes,
                           void* saved_states, size_t saved_bytes, fastmax_stream_t stream);
int fastmax_backward_saved(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                           const void* o, int64_t ldo, const float* den, int64_t den_stride,
                           const void* go, void* dq, void* dk, void* dv,
                           const float* qk_scale, const int32_t* qk_argmax,
                           void* workspace, size_t workspace_bytes,
                           const void* saved_states, size_t saved_bytes, fastmax_stream_t stream);

/* Forward pass for callers that cannot allocate device memory or carry a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose launcher allocates five tensors per call,
 * fastmax_cuda_forward.cu:347-358).  Same arguments and results as fastmax_forward (bit for bit),
 * minus the workspace: the head statistics and moment states go to a scratch array of
 * FASTMAX_NOALLOC_SCRATCH_BYTES that is part of the library's device image (every GPU the library
 * runs on holds it until the process ends; its address is looked up on the first call per device).
 * The call allocates and frees nothing.  Problems whose smallest workspace
 * (fastmax_workspace_min_bytes(desc, FASTMAX_PASS_FORWARD)) exceeds the array are refused with
 * FASTMAX_E_WORKSPACE.  All calls on one GPU share the array: calls that overlap in time on
 * one GPU (different streams, or threads) race and must be serialised by the caller.
 * The address lookup of the first call on a device is a host-side runtime query behind a mutex: a
 * caller that captures a HIP graph makes it happen before the capture begins, either with one
 * uncaptured call or with fastmax_noalloc_scratch_bytes(), which also resolves the address on the
 * current device (and still returns the size when no device is current). */
#define FASTMAX_NOALLOC_SCRATCH_BYTES (64u << 20)
size_t fastmax_noalloc_scratch_bytes(void);
int fastmax_forward_noalloc(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                            void* o, int64_t ldo, float* den, int64_t den_stride,
                            float* qk_scale, int32_t* qk_argmax, fastmax_stream_t stream);

/* In-place q <- lim*q/max||q_n||, k likewise: the side effect the reference's forward has
 * on its inputs (calc_norms/find_max/apply_norm, fastmax_cuda_forward.cu:223-269,368-382,
 * with the PyTorch path's definition of the norm, example.py:105-108).  Only the legacy
 * forwardpass binding uses it.  workspace: >= 16*bh + 512 bytes, 256-byte aligned. */
int fastmax_normalize_inplace(const fastmax_desc* desc, void* q, void* k,
                              void* workspace, size_t workspace_bytes, fastmax_stream_t stream);

/* Recurrent form: the moment state S = sum_j phi(k_j) (x) [v_j, 1] of a head is kept by the
 * caller between calls and plays the part of the key/value cache (reference model.py:828-852,
 * which caches k and v because its attention is recomputed from them).  The reference has
 * no such kernel; the arithmetic is the running state of its causal loop
 * (fastmax_cuda_forward.cu:102-197).  A state is fastmax_state_bytes(desc) bytes of fp32 per
 * key/value head (bhkv of them), heads contiguous; its layout is private to the library.  The normalisation by the
 * maximum row norm is not causal, so with normalize != 0 the caller passes the per-head
 * factors (bh floats each, device memory) that a forward pass over the prompt reported in
 * qk_scale (q factors first, then k factors); with normalize == 0 they may be NULL (q: 1,
 * k: 1/temperature).  mask is ignored by these calls.
 *
 * fastmax_state_update: state (+)= the sum over desc->nk tokens of k, v (bhkv, nk, d); with
 *   accumulate == 0 the state is overwritten.  workspace: as fastmax_forward for the same
 *   descriptor with mask = 0.
 * fastmax_decode_step: one new token per head (desc->nq = desc->nk = 1; q is (bh, 1, d), k and v
 *   are (bhkv, 1, d)): the state of a key/value head takes in (k, v), then every query head of its
 *   group gets o = phi(q).S / den -- the causal output row of that token
 *   (fastmax_cuda_forward.cu:38).
 *   den may be NULL.  workspace: fastmax_decode_workspace_bytes(desc), 256-byte aligned. */
size_t fastmax_state_bytes(const fastmax_desc* desc);
size_t fastmax_decode_workspace_bytes(const fastmax_desc* desc);
int fastmax_state_update(const fastmax_desc* desc, const void* k, const void* v, const float* k_scale,
                         void* state, int accumulate, void* workspace, size_t workspace_bytes,
                         fastmax_stream_t stream);
int fastmax_decode_step(const fastmax_desc* desc, const void* q, const void* k, const void* v,
                        const float* q_scale, const float* k_scale, void* state, void* o, int64_t ldo,
                        float* den, int64_t den_stride, void* workspace, size_t workspace_bytes,
                        fastmax_stream_t stream);

/* Caller-side helper of a GPT block (no kernel of the reference does this; it replaces the
 * chain of PyTorch ops at model.py:474-497 -- view the fused projection as
 * (b, t, groups, q_per_kv + 2, hs), permute, split -- then model.py:812-825 apply_rope on the
 * first rope_n channels of q and k, then the .contiguous() calls at model.py:572-574).
 *   grad == 0: qkv (b, t, groups*(q_per_kv+2)*hs) in;  q (b, groups*q_per_kv, t, hs),
 *              k, v (b, groups, t, hs) out, q and k rotated:
 *              y = x*cos + (-x2, x1)*sin on channels [0, rope_n), x1/x2 = its halves
 *   grad != 0: the adjoint: q, k, v hold the gradients of the three outputs (in), qkv receives
 *              the gradient of the projection (out)
 * cos, sin: (t, rope_n) fp32, rope_n a multiple of 8 (0: no rotation, they may be NULL).
 * No split, for callers that hand strided views to the *_strided attention entry points:
 *   q == k == v == NULL: the rotation (grad == 0) or its adjoint (grad != 0) is applied in place to
 *              the q and k rows of qkv (e.g. to the gradient of the projection after the backward pass
 *              has written dq, dk, dv into it);
 *   k == v == NULL, q != NULL: q is (b, t, groups, q_per_kv + 1, hs) and receives the rotated q and k rows
 *              of qkv (grad == 0; v is read by the attention from qkv itself). */
typedef struct fastmax_rope_desc {
  int32_t b, t, groups, q_per_kv, hs, rope_n;
  int32_t dtype;       /* FASTMAX_F32 or FASTMAX_BF16 */
} fastmax_rope_desc;
int fastmax_qkv_rope(const fastmax_rope_desc* desc, int grad, void* qkv, const float* cos, const float* sin,
                     void* q, void* k, void* v, fastmax_stream_t stream);

/* Kernel timing aid (no counterpart in the reference, which only wall-clocks whole calls,
 * test_fastmax.py:351-356).  Between begin and end every kernel the calling thread launches
 * through this library is bracketed by two HIP events on the caller's stream; end waits for
 * them and adds up milliseconds and launch counts per kernel class.  Events are created on
 * first use and kept by the thread. */
enum {
  FASTMAX_K_ROWSTAT = 0,   /* per-head max row norm (or the constant fill)               */
  FASTMAX_K_BUILD = 1,     /* moment-state build (prefix and suffix states)              */
  FASTMAX_K_FWD_APPLY = 2, /* forward apply + divide                                     */
  FASTMAX_K_BWD_PREP = 3,  /* c_i = go_i.o_i/den_i                                       */
  FASTMAX_K_BWD_DQ = 4,    /* dq                                                         */
  FASTMAX_K_BWD_DK = 5,    /* dk                                                         */
  FASTMAX_K_BWD_DV = 6,    /* dv                                                         */
  FASTMAX_K_NORM_FIX = 7,  /* normalisation chain rule on the max-norm rows              */
  FASTMAX_NUM_KERNELS = 8
};
typedef struct fastmax_kernel_times {
  float ms[FASTMAX_NUM_KERNELS];
  int32_t launches[FASTMAX_NUM_KERNELS];
} fastmax_kernel_times;
int fastmax_profile_begin(void);
int fastmax_profile_end(fastmax_kernel_times* out);

#ifdef __cplusplus
}
#endif
#endif /* FASTMAX_AMD_H */
