/* C ABI of libua_hip.so -- Universal Attention forward/backward on AMD Instinct MI355X (gfx950).
 *
 * These entry points are what a binding for the reference's hot path would call in place of its
 * Triton launchers.  Each declaration cites the reference interface it replaces
 * (paths relative to the reference repository root).
 *
 * Conventions
 *  - All pointers are DEVICE pointers unless stated; the caller owns every buffer.
 *  - No entry point allocates or frees device memory; scratch comes from `ws` (size from
 *    ua_workspace_bytes).  Work is enqueued on `stream` and the call returns without synchronising
 *    (ua_autotune is the exception: it times candidates and synchronises).
 *  - Return value: 0 on success, a negative UA_E* code otherwise; ua_last_error() then describes it.
 *    Nothing throws, nothing aborts.
 *  - z indices: Zk = b*h (batch x kv head), Zq = b*h*r (r query groups per kv head, kv-major).
 */
#ifndef UA_H_
#define UA_H_
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* ua_stream_t; /* == hipStream_t */

enum { UA_F32 = 0, UA_BF16 = 1 };
enum {
  UA_OK = 0,
  UA_EINVAL = -1,    /* bad shape / dtype / null pointer / unsupported size */
  UA_EWORKSPACE = -2,/* workspace too small or misaligned */
  UA_ELAUNCH = -3    /* HIP reported an error while enqueuing */
};
enum {
  UA_OP_FWD = 0,       /* ua_fwd        */
  UA_OP_BWD = 1,       /* ua_bwd        */
  UA_OP_FUSED_FWD = 2, /* ua_fused_fwd  */
  UA_OP_FUSED_BWD = 3, /* ua_fused_bwd  */
  UA_OP_BWD_SCRATCH = 4,       /* ua_workspace_bytes only: ua_bwd's workspace when it is given the forward state */
  UA_OP_FUSED_BWD_SCRATCH = 5  /* ua_workspace_bytes only: likewise for ua_fused_bwd */
};
enum {
  UA_FLAG_SKIP_MASKED = 1, /* ua_bwd: the upstream gradient is zero for (query, chunk) pairs in which the
                              query precedes the whole chunk (true when it comes from ua_merge_bwd).  Without the
                              flag ua_bwd finds this out by itself for chunks that are multiples of 64 (one pass
                              over g_out and g_denom that it makes anyway); the flag saves that check and, for the
                              other chunk sizes, the sweep over those pairs. */
  UA_FLAG_RECOMPUTE = 4,   /* bf16 (all ops and ua_workspace_bytes): by default the kernels of the fused operator pass the
                              decay bias and the score / decay gradients of every tile to one another through the
                              workspace (2 bytes per causal (key, query) pair and tensor: about Lp*Lp bytes per kv head for
                              the bias, per query head and per kv head for the gradients; the chunked backward with a
                              chunk that is a multiple of 64 does the same for the gradients).  With this flag every
                              kernel recomputes what it needs instead: slower, workspace O(L*L/16). */
  UA_FLAG_SHARE_GROUPS = 8, /* bf16 fused ops with r > 1 (and ua_workspace_bytes): the key side of the backward sweeps the r
                              query groups of a kv head inside one workgroup, sharing the key-key part of every step.
                              Without the flag it does so only when there are enough kv heads to fill the device and
                              otherwise divides the groups into parts with a sweep each (more workspace: the key-side
                              partial sums are then kept per part).  Same results up to summation order. */
  UA_FLAG_GATES_F32 = 16,  /* bf16 ops: static_src, static_dest and the gradients dsrc, ddest are float32 tensors (the
                              reference allocates dstatic_src in static_src.dtype and accepts float32 gates next to
                              bf16 q, k, v: universal_attention_kernel.py:825-829).  float32 ops: always so. */
  UA_FLAG_PRUNE = 2        /* fused ops: skip (key, query) pairs whose softmax weight is provably below 2^-48 because
                              of the accumulated decay (no counterpart in the reference, which visits every pair).
                              The bound uses the largest key and query norms of the head; results change by less
                              than float32 rounding.  ua_fused_bwd with the forward state follows what the forward recorded. */
};

/* Problem description.  kc, vc: [b,h,L,d] seen as [b,h,n,c,d]; xq: [b,h,r,L,d]; gates: [b,h,L].
 * Head dim d: 1..128 everywhere (zero-padded to 64 or 128 inside); 129..256 (padded to 256, as the reference's
 * second-generation kernel pads to a power of two up to 256, universal_attention_kernel_opt.py:441-456) for the bf16
 * fused operator without UA_FLAG_RECOMPUTE. */
typedef struct ua_desc {
  int32_t b, h, r, L, d;
  int32_t chunk; /* keys per chunk c (L % c == 0; a multiple of 64, or 16 or a multiple of 32 up to 256); ignored by fused ops */
  int32_t dtype; /* UA_F32 or UA_BF16, the dtype of every tensor except where noted */
  int32_t flags;
} ua_desc;

/* A row-major tensor whose last (feature) dimension has stride 1; all strides in ELEMENTS.
 * Row index `row` in [0,L) is addressed as (row / inner_len)*stride_outer + (row % inner_len)*stride_inner,
 * which covers both [.., L, d] (inner_len = L) and chunked [.., n, c, d] views. */
typedef struct ua_rows {
  const void* ptr;
  int64_t stride_b, stride_h, stride_r, stride_outer, stride_inner;
  int32_t inner_len;
} ua_rows;

/* The per-chunk partial output tensor out[b,h,r,L,d,n]: element (zq, t, dd, i) lives at
 * ptr + zq*stride_z + t*stride_t + dd*stride_d + i*stride_i (elements). */
typedef struct ua_chunked {
  void* ptr;
  int64_t stride_z, stride_t, stride_d, stride_i;
} ua_chunked;

int ua_version(void);
/* Hash of the sources this library was compiled from (csrc/ and this header), as computed by the build script; a host
 * binding can compare it with the sources it sees to refuse a stale binary.  No counterpart in the reference. */
const char* ua_source_hash(void);
/* Thread-local description of the last failure on this thread ("" if none). */
const char* ua_last_error(void);

/* Bytes of scratch `ws` the given op needs (0 and an error string if the shape is unsupported).
 * A forward op leaves its state (packed inputs, log-gates, bias tiles or carries, normalisers) in its workspace.  A
 * backward op either receives that buffer as `fwd_state` -- its own `ws` then needs UA_OP_(FUSED_)BWD_SCRATCH bytes -- or
 * rebuilds the state inside a `ws` of UA_OP_(FUSED_)BWD bytes (= forward state + scratch).  What a caller keeps alive
 * between forward and backward is therefore the forward state at most, and nothing with fwd_state = NULL. */
size_t ua_workspace_bytes(const ua_desc* desc, int op);

/* Chunked forward: replaces _universal_attention_fwd
 * (Universal_Attention/triton/universal_attention_kernel.py:192-239) and the torch operator
 * UniversalAttention.forward (universal_attention_autograd.py:9-38).
 * static_src, static_dest: contiguous [b,h,L].  denom: contiguous [b,h,r,L,n] in desc->dtype.
 * lse2_out: NULL, or [b*h*r][L/chunk][Lp] float (Lp = L rounded up to 128) that receives the per-chunk normalisers in
 * float32 (log2 units; `denom` in bf16 is too coarse for the backward): the one part of the forward state that is
 * expensive to rebuild, 1/(d+1) of the size of `out`.  Hand it to ua_bwd as lse2_in.  The workspace holds a copy
 * either way, so it is a complete fwd_state for ua_bwd with or without lse2_in. */
int ua_fwd(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
           const void* static_dest, const ua_chunked* out, void* denom, float* lse2_out, void* ws, size_t ws_bytes,
           ua_stream_t stream);

/* Chunked backward: replaces _universal_attention_bwd (universal_attention_kernel.py:793-862) and
 * UniversalAttention.backward (universal_attention_autograd.py:47-99).
 * out: the forward's result; g_out: same indexing; g_denom: contiguous float32 [b,h,r,L,n].
 * Gradients are written contiguous: dkc, dvc [b,h,L,d]; dxq [b,h,r,L,d]; dsrc, ddest [b,h,L].
 * fwd_state: NULL, or the workspace ua_fwd ran on for the same inputs and flags, contents intact (skips the recompute;
 * the backward rewrites parts of it with the same values).
 * delta: NULL, or what ua_merge_bwd left when it produced exactly these (g_out, g_denom) from `out`
 * ([b*h*r][L/chunk][Lp] float, Lp = L rounded up to 128, zero beyond L): the backward then skips its own pass over
 * out and g_out (8.6 GB at b=1 h=32 L=8192 d=128).  Needs UA_FLAG_SKIP_MASKED and a chunk that is a multiple of 64.
 * lse2_in: NULL, or what ua_fwd wrote to lse2_out: without fwd_state the backward then repacks the inputs and
 * rebuilds the decay carries but does not run the forward kernel again for the normalisers. */
int ua_bwd(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
           const void* static_dest, const ua_chunked* out, const ua_chunked* g_out, const float* g_denom, void* dkc,
           void* dvc, void* dxq, void* dsrc, void* ddest, const float* delta, const float* lse2_in, void* fwd_state, void* ws,
           size_t ws_bytes, ua_stream_t stream);

/* Fused forward: the chunked operator followed by SMVecMatMul (universal_attention_autograd.py:278-283)
 * without materialising the per-chunk tensor; same role as the reference's second-generation
 * _attention.forward (Universal_Attention/triton/universal_attention_kernel_opt.py:436-502).
 * O: contiguous [b,h,r,L,d]; lse: contiguous float32 [b,h,r,L] (natural log). */
int ua_fused_fwd(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
                 const void* static_dest, void* O, float* lse, void* ws, size_t ws_bytes, ua_stream_t stream);

/* The fused forward for callers that cannot allocate or supply device scratch (code under HIP graph capture, serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as ua_fused_fwd
 * minus the workspace: the scratch is a device array inside the library, UA_NOALLOC_SCRATCH_BYTES per GPU, held from
 * the library's load until the process ends.  Problems whose ua_workspace_bytes(desc, UA_OP_FUSED_FWD) exceeds it are
 * refused with UA_EWORKSPACE.  Calls no hipMalloc / hipFree.  All calls on one GPU share the array: two calls that
 * overlap on one GPU (different streams or threads) race, and the forward state a later ua_fused_bwd could reuse is not
 * kept (call ua_fused_bwd with fwd_state = NULL).  The first call on a device looks up the array's address and sets
 * kernel attributes: make it outside any stream capture; every later call only enqueues kernels. */
#define UA_NOALLOC_SCRATCH_BYTES (64u << 20)
size_t ua_noalloc_scratch_bytes(void);
int ua_fused_fwd_noalloc(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
                         const void* static_dest, void* O, float* lse, ua_stream_t stream);

/* Fused backward: replaces SMVecMatMul.backward + UniversalAttention.backward
 * (universal_attention_autograd.py:291-297, :47-99) / _attention.backward (universal_attention_kernel_opt.py:504-581).
 * O, lse: as produced by ua_fused_fwd; dO contiguous [b,h,r,L,d].  fwd_state: as for ua_bwd (the workspace of
 * ua_fused_fwd, or NULL). */
int ua_fused_bwd(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
                 const void* static_dest, const void* O, const float* lse, const void* dO, void* dkc, void* dvc,
                 void* dxq, void* dsrc, void* ddest, void* fwd_state, void* ws, size_t ws_bytes, ua_stream_t stream);

/* Chunk merge: replaces SMVecMatMul.forward / .backward (universal_attention_autograd.py:278-297).
 * rows = number of (b,h,r,t) rows, n chunks, d features.  mat element (row, dd, i) at
 * row_off(row) + dd*stride_d + i*stride_i with row_off = (row / L)*stride_z + (row % L)*stride_t.
 * vec: contiguous [rows, n] in `dtype`; result contiguous [rows, d]. */
int ua_merge_fwd(int dtype, int64_t rows, int32_t L, int32_t d, int32_t n, const ua_chunked* mat, const void* vec,
                 void* result, ua_stream_t stream);
/* g: contiguous [rows, d]; d_mat indexed like mat; d_vec contiguous [rows, n] in `dtype`.  Slices whose weight is exactly
 * zero (chunks no key of which a query sees: normaliser -1e12) are not read, by either kernel.
 * delta: NULL, or [rows / L][n][Lp] float (Lp = L rounded up to 128; the caller zeroes it beyond L) that receives
 * sum_dd mat d_mat - d_vec per (row, chunk), for ua_bwd. */
int ua_merge_bwd(int dtype, int64_t rows, int32_t L, int32_t d, int32_t n, const ua_chunked* mat, const void* vec,
                 const void* g, const ua_chunked* d_mat, void* d_vec, float* delta, ua_stream_t stream);

/* Stand-alone decay bias ("affinity scores"): replaces _affinity_fwd / _affinity_bwd and the AffinityScores wrapper
 * (Universal_Attention/triton/affinity_kernel_opt.py:100-127, :130-423, :425-450).  desc: b, h, L, d, dtype (r, chunk and
 * flags are ignored).  k: [b,h,L,d] rows; src, dest: contiguous [b,h,L]; aff / daff: contiguous [b,h,L,L] in the
 * dtype, aff[b,h,t,s] = bias of key s towards query t in natural-log units (0 on the diagonal, -1e12 where s > t).
 * dk contiguous [b,h,L,d]; dsrc, ddest contiguous [b,h,L].  Workspace: ua_affinity_workspace_bytes(desc, backward).
 * bf16 with L a multiple of 8: daff must be 16-byte aligned (UA_EINVAL otherwise). */
size_t ua_affinity_workspace_bytes(const ua_desc* desc, int backward);
int ua_affinity_fwd(const ua_desc* desc, const ua_rows* k, const void* src, const void* dest, void* aff, void* ws,
                    size_t ws_bytes, ua_stream_t stream);
int ua_affinity_bwd(const ua_desc* desc, const ua_rows* k, const void* src, const void* dest, const void* daff, void* dk,
                    void* dsrc, void* ddest, void* ws, size_t ws_bytes, ua_stream_t stream);

/* On-device autotune table: replaces the @triton.autotune wrappers
 * (universal_attention_kernel.py:10-25, universal_attention_kernel_opt.py:8-36,115-118,309-312, affinity_kernel_opt.py:6-27).
 * The table is process-wide and thread-safe, keyed by (kernel slot, dtype, padded head dim, r, log2 bucket of L, log2
 * bucket of b*h).  Every launch of a slot's kernel consults it: an entry set by ua_tune_set / ua_autotune wins, then the
 * built-in entries shipped for the reference's benchmark shapes, then a size heuristic.
 * Kernel slots (the `slot` argument of ua_tune_get / set / variants): */
enum {
  UA_TUNE_FWD_RECOMPUTE = 2, /* == UA_OP_FUSED_FWD.  Forward without bias tiles (fp32, UA_FLAG_RECOMPUTE): bf16 0 = 8 waves
                                two LDS stages, 1 = 8 waves one stage, 2 = 12 waves, 3 = 16 waves, 4 = 4 waves; fp32: one */
  UA_TUNE_CARRY = 16,        /* bias pre-pass of the bf16 operator: 0 = 8 waves x 16 keys per workgroup, 1 = 4 waves,
                                2 = 4 waves, two key groups of complementary length per workgroup */
  UA_TUNE_FWD_TILES = 17,    /* bf16 forward over bias tiles: 0 = one 32-query block per wave (256-query workgroups, two
                                LDS stages), 1 = 16 queries per wave (128-query workgroups, one stage, two per CU),
                                2 = 16 queries per wave, 64-query workgroups (r = 1 only) */
  UA_TUNE_BWD_PARTS = 18,    /* key side of the bf16 backward with r > 1: variant i divides the query groups of a kv
                                head into the i-th smallest divisor of r parts with a sweep each (0 = one shared sweep).
                                Changes ua_workspace_bytes: set it before sizing the workspace. */
  UA_TUNE_BWD_QUERIES = 19,  /* query side of the bf16 backward over gradient tiles: 0 = steps of 32 keys, two workgroups
                                per CU; 1 = steps of 64 keys, one workgroup per CU */
  UA_TUNE_BWD_KEYS = 20,     /* key side of the bf16 backward over bias tiles, r = 1, head dim 65..128: 0 = 16 keys per
                                wave on 16x16 tiles, two waves per SIMD; 1 = 32 keys per wave on 32x32 tiles, one wave per
                                SIMD, the step laid out by hand */
  UA_TUNE_CHUNKED_PAIR = 21, /* chunked operator, chunk a multiple of 64 (ua_fwd, ua_bwd): work items (query blocks of the
                                forward, key groups of the backward's key side) per workgroup: 0 = two of complementary
                                length once the launch gives every CU several single ones, 1 = one, 2 = two */
  UA_TUNE_AFF_PAIR = 22      /* stand-alone bias (ua_affinity_fwd, ua_affinity_bwd): key groups per workgroup, as above.
                                ua_autotune does not time these two slots: time the op itself under each variant
                                (ua_tune_set), as the Python layer's autotune_chunked / autotune_affinity do */
};
/* ua_autotune(desc, op, ...) with op = UA_OP_FUSED_FWD or UA_OP_FUSED_BWD times every variant of every kernel slot on
 * that op's path for desc (hipEvents on `stream`, synchronises) and records the fastest of each.  `ws` must hold what
 * the op itself left there for desc, state and scratch in ONE buffer of ua_workspace_bytes(desc, UA_OP_FUSED_BWD) bytes:
 * call ua_fused_fwd on it, and for the backward also ua_fused_bwd with fwd_state = ws and its scratch at
 * ws + ua_workspace_bytes(desc, UA_OP_FUSED_FWD); the tuning runs re-launch the kernels on that state.  UA_OP_FUSED_BWD
 * clobbers the scratch part (the forward state stays valid).  Returns 0 or a negative error. */
int ua_autotune(const ua_desc* desc, int op, void* ws, size_t ws_bytes, ua_stream_t stream);
/* Table access for persistence: entry of (slot, desc) set by ua_tune_set / ua_autotune, -1 if none. */
int ua_tune_get(const ua_desc* desc, int slot);
int ua_tune_set(const ua_desc* desc, int slot, int variant);   /* variant -1 removes the entry */
/* What a launch of the slot's kernel would use for desc right now (entry, else built-in, else heuristic). */
int ua_tune_choice(const ua_desc* desc, int slot);
/* Number of variants a slot has for this description (>= 1), or a negative error. */
int ua_tune_variants(const ua_desc* desc, int slot);

/* Per-kernel timing, no counterpart in the reference (its harness times whole calls with CUDA events,
 * Universal_Attention/triton/_debug.py:413-446).  While enabled every kernel group the ops enqueue is bracketed
 * by hipEvents on the launch stream.  ua_prof_collect synchronises the device, writes "name:count:total_ms;..."
 * into buf (NUL terminated, truncated to cap) and clears the records; returns the untruncated length. */
void ua_prof_enable(int on);
int ua_prof_collect(char* buf, size_t cap);

#ifdef __cplusplus
}
#endif
#endif /* UA_H_ */
