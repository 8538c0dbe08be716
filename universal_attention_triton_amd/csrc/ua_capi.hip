// C ABI of libua_hip.so: validation, workspace layout, kernel sequencing, autotune table.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/ua.h"
#include "ua_internal.hpp"
#include "ua_merge.hpp"
#include "ua_pack.hpp"
#include "ua_bwd.hpp"   // k_bwd_finish only (k_bwd_keys is instantiated in ua_inst_bwd.hip)

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct Layout {
  int D, Lp, nT, nch, Zk, Zq;
  size_t esz;
  // forward state
  size_t Kp, KT, Vp, VT, Qp, QT, lsrc, ldest, C, lse2, knorm2, qnorm2, reach, minkey, Bt, fwd_end;
  // backward scratch
  size_t dOp, dOT, delta, dQacc, dKdacc, Dsuf, dKrow, dVrow, dsrc_raw, masked_nz, dS_st, dG_st, total;
  bool tiles;       // bf16 merged operator: bias, dS and dG tiles are exchanged through the workspace
  bool grad_tiles;  // ... dS and dG tiles (also the chunked operator with a chunk that is a multiple of 64)
  int key_parts;    // key side of the backward: sweeps per kv head, each over r / key_parts query groups (see make_layout)
};

// head dims are zero-padded to 64, 128 or 256 (as the reference's second-generation kernel pads to a power of two up to
// 256, Universal_Attention/triton/universal_attention_kernel_opt.py:441-456)
int padded_dim(int d) { return d <= 64 ? 64 : (d <= 128 ? 128 : 256); }

int check_desc(const ua_desc* d, bool chunked) {
  if (!d) return fail(UA_EINVAL, "null descriptor");
  if (d->dtype != UA_F32 && d->dtype != UA_BF16) return fail(UA_EINVAL, "dtype %d: only UA_F32 and UA_BF16 are supported", d->dtype);
  if (d->b < 1 || d->h < 1 || d->r < 1 || d->L < 1 || d->d < 1) return fail(UA_EINVAL, "b,h,r,L,d must be positive (got %d,%d,%d,%d,%d)", d->b, d->h, d->r, d->L, d->d);
  // A (key, query) product contracts over the whole head dim inside one workgroup, whose LDS stages and accumulators
  // are laid out for at most 256 features (the reference's second-generation kernel stops there too,
  // universal_attention_kernel_opt.py:441-456; the self-test of its first one runs d = 512,
  // Universal_Attention/triton/universal_attention_kernel.py:1189, which this library refuses)
  if (d->d > 256) return fail(UA_EINVAL, "head dim %d > 256 is not supported (LDS stages and accumulators are laid out for at most 256 features)", d->d);
  if (d->d > 128 && (chunked || d->dtype != UA_BF16 || (d->flags & UA_FLAG_RECOMPUTE)))
    return fail(UA_EINVAL, "head dim %d > 128: only the bf16 fused operator without UA_FLAG_RECOMPUTE (float32 tiles of 256 features "
                           "do not fit the LDS stages; the chunked operator has no 256-feature instantiation)", d->d);
  // one grid row (y) per head; callers with more heads split the batch or the kv heads, which are independent
  // (the Python operators do that by themselves)
  if ((long)d->b * d->h * d->r > 65535)
    return fail(UA_EINVAL, "b*h*r = %ld exceeds the grid limit 65535: split the call along b or h (heads are independent)", (long)d->b * d->h * d->r);
  if (chunked) {
    const int c = d->chunk;
    if (c < 1 || d->L % c != 0) return fail(UA_EINVAL, "chunk %d must divide L = %d", c, d->L);
    // multiples of 64 of any size run on the query-/key-stationary kernels, which take the chunk as a run-time bound;
    // 16 and the other multiples of 32 on the key-chunk-stationary ones, whose LDS holds a whole chunk
    if (!(c % 64 == 0 || ((c == 16 || c % 32 == 0) && c <= 256)))
      return fail(UA_EINVAL, "chunk %d unsupported: need a multiple of 64, or 16 or a multiple of 32 up to 256", c);
    if ((long)d->b * d->h * d->r * (d->L / c) > 65535)
      return fail(UA_EINVAL, "b*h*r*(L/chunk) exceeds the grid limit 65535: split the call along b or h (heads are independent)");
  }
  return UA_OK;
}

// ---- autotune table ------------------------------------------------------------------------
// key: kernel slot, dtype, padded head dim, r, log2 bucket of L, log2 bucket of b*h
using TuneKey = std::tuple<int, int, int, int, int, int>;
std::mutex g_tune_mu;
std::map<TuneKey, int> g_tune;

int l_bucket(int L) { int b = 0; while ((128 << b) < L) ++b; return b; }
int z_bucket(long z) { int b = 0; while ((1L << b) < z) ++b; return b; }
TuneKey tune_key(const ua_desc& d, int slot) {
  return TuneKey(slot, d.dtype, padded_dim(d.d), d.r, l_bucket(d.L), z_bucket((long)d.b * d.h));
}
bool known_slot(int slot) {
  return slot == UA_TUNE_FWD_RECOMPUTE || slot == UA_TUNE_CARRY || slot == UA_TUNE_FWD_TILES || slot == UA_TUNE_BWD_PARTS ||
         slot == UA_TUNE_BWD_QUERIES || slot == UA_TUNE_BWD_KEYS || slot == UA_TUNE_CHUNKED_PAIR || slot == UA_TUNE_AFF_PAIR;
}
int n_divisors(int r) { int n = 0; for (int p = 1; p <= r; ++p) n += r % p == 0; return n; }
int nth_divisor(int r, int i) { for (int p = 1; p <= r; ++p) if (r % p == 0 && i-- == 0) return p; return 1; }
int divisor_index(int r, int p) { int i = 0; for (int q = 1; q < p; ++q) i += r % q == 0; return i; }
int n_variants(const ua_desc& d, int slot) {
  const bool bf = d.dtype == UA_BF16;
  switch (slot) {
    case UA_TUNE_FWD_RECOMPUTE: return ua::fwd_fused_variants(d.dtype, padded_dim(d.d));
    case UA_TUNE_CARRY: return bf ? 3 : 1;
    case UA_TUNE_FWD_TILES: return bf ? (d.d > 128 ? 1 : (d.r % 2 == 0 ? 2 : 3)) : 1;     // above 128: 16 queries per wave only
    case UA_TUNE_BWD_PARTS: return bf ? n_divisors(d.r) : 1;
    case UA_TUNE_BWD_QUERIES: return bf && d.d <= 128 ? 2 : 1;
    case UA_TUNE_BWD_KEYS: return bf && padded_dim(d.d) == 128 && d.r == 1 ? 2 : 1;
    case UA_TUNE_CHUNKED_PAIR: return 3;     // by launch size / one / two work items per workgroup (ua::paired_items)
    case UA_TUNE_AFF_PAIR: return 3;
  }
  return 1;
}
// Entries shipped with the library: measured with ua_autotune on one MI355X for the shapes the reference's benchmark
// recipes name (bf16; b, h, r, L, d).  {slot, D, r, L bucket, b*h bucket, variant}
struct BuiltIn { int slot, D, r, lb, zb, variant; };
const BuiltIn kBuiltIn[] = {
#include "ua_tune_defaults.inc"
};
// size heuristics for everything else
int heuristic_variant(const ua_desc& d, int slot) {
  const long Zk = (long)d.b * d.h, Zq = Zk * d.r;
  const int Lp = (int)align_up((size_t)d.L, 128);
  switch (slot) {
    case UA_TUNE_CARRY: {    // 4-wave workgroups won at every tuned shape; two key groups each when the single ones make
      const long n4 = Zk * (Lp / 64);      // one to four rounds of the 1024 resident workgroups
      return (n4 >= 1024 && n4 < 4096) ? 2 : 1;
    }
    case UA_TUNE_FWD_TILES:  // 256-query workgroups need about four per CU to balance; small launches run 64-query pieces
      if (Zq * (Lp / 256) >= 1024) return 0;
      return (d.r % 2 == 0 || Zq * (Lp / 128) >= 1536) ? 1 : 2;
    case UA_TUNE_BWD_PARTS: {
      // Grouped queries: the key-stationary kernel sweeps the r query groups of a kv head in one workgroup, sharing the
      // key-key part of every step (a step of a further group costs about 0.7 of a full one).  Its longest workgroup then
      // runs Lp/32 * r steps, and with few kv heads the launch waits for it.  The groups can instead be divided into p
      // parts with a sweep each (p times the workgroups, a longest one p times shorter, the key-key part repeated per
      // part).  p = the divisor of r with the smallest estimate max(longest workgroup, 1.1 x average load of the 256 CUs).
      int best_p = 1;
      const double blocks = Lp / 32, wgs = (double)Zk * (Lp / 128);
      double best = 0;
      for (int p = 1; p <= d.r; ++p) {
        if (d.r % p) continue;
        const double w = 1.0 + 0.7 * (d.r / p - 1);                 // cost of one query block for the groups of a part
        const double longest = blocks * w, average = 1.1 * wgs * p * (blocks / 2) * w / 256.0;
        const double cost = longest > average ? longest : average;
        if (p == 1 || cost < best) { best = cost; best_p = p; }
      }
      return divisor_index(d.r, best_p);
    }
  }
  return 0;
}
int tune_entry(const ua_desc& d, int slot) {
  std::lock_guard<std::mutex> g(g_tune_mu);
  auto it = g_tune.find(tune_key(d, slot));
  return it == g_tune.end() ? -1 : it->second;
}
int tuned_variant(const ua_desc& d, int slot) {
  const int n = n_variants(d, slot);
  int v = tune_entry(d, slot);
  if (v >= 0 && v < n) return v;
  const TuneKey k = tune_key(d, slot);
  if (d.dtype == UA_BF16)
    for (const BuiltIn& e : kBuiltIn)
      if (e.slot == slot && e.D == std::get<2>(k) && e.r == d.r && e.lb == std::get<4>(k) && e.zb == std::get<5>(k) && e.variant < n)
        return e.variant;
  v = heuristic_variant(d, slot);
  return v < n ? v : 0;
}

Layout make_layout(const ua_desc& d, bool chunked, int force_parts = 0) {
  Layout l{};
  l.D = padded_dim(d.d);
  l.Lp = (int)align_up((size_t)d.L, 128);
  l.nT = l.Lp / 16;     // carries are kept per 16-query tile
  l.nch = chunked ? d.L / d.chunk : 1;
  l.Zk = d.b * d.h;
  l.Zq = l.Zk * d.r;
  l.esz = d.dtype == UA_BF16 ? 2 : 4;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const size_t kbytes = (size_t)l.Zk * l.Lp * l.D * l.esz, qbytes = (size_t)l.Zq * l.Lp * l.D * l.esz;
  l.Kp = take(kbytes); l.KT = take(kbytes); l.Vp = take(kbytes); l.VT = take(kbytes);
  l.Qp = take(qbytes);
  l.lsrc = take((size_t)l.Zk * l.Lp * 4); l.ldest = take((size_t)l.Zk * l.Lp * 4);
  const size_t carries = (size_t)l.Zk * l.nT * l.Lp * 4;     // one float per (16-query tile, key)
  l.lse2 = take((size_t)l.Zq * l.nch * l.Lp * 4);
  // pruning state of the fused mode: largest squared row norm of every 32-row block of K and Q, reach of every key
  // tile, first key tile reaching every query block
  l.knorm2 = take((size_t)l.Zk * (l.nT / 2) * 4); l.qnorm2 = take((size_t)l.Zq * (l.nT / 2) * 4); l.reach = take((size_t)l.Zk * l.nT * 4); l.minkey = take((size_t)l.Zk * (l.nT / 2) * 4);
  // bf16 fused operator: the kernels exchange tiles through the workspace instead of recomputing them (fp16 bias of every
  // (16 keys, 32 queries) tile here; score and decay gradients in the backward part), 1 KB per tile
  l.tiles = !chunked && d.dtype == UA_BF16 && !(d.flags & UA_FLAG_RECOMPUTE);
  const size_t sq = (size_t)ua::tri_tiles(l.Lp / 32) * 1024;     // the causal triangle of 1 KB tiles, per head
  l.Bt = l.tiles ? take((size_t)l.Zk * sq) : 0;
  l.C = l.tiles ? 0 : take(carries);      // the bias tiles replace the forward carries
  // transposed queries (and upstream gradient below): read by the key-stationary backward only, which takes its
  // transposed operands out of the natural tiles when it exchanges tiles
  // (so does the chunked backward with a chunk that is a multiple of 64)
  l.grad_tiles = l.tiles || (chunked && d.chunk % 64 == 0 && d.dtype == UA_BF16 && !(d.flags & UA_FLAG_RECOMPUTE));
  l.QT = l.grad_tiles ? 0 : take(qbytes);
  l.fwd_end = off;
  const size_t gbytes = (size_t)l.Zq * l.nch * l.Lp * l.D * l.esz;
  l.dOp = take(gbytes); l.dOT = l.grad_tiles ? 0 : take(gbytes);
  l.delta = take((size_t)l.Zq * l.nch * l.Lp * 4);
  // the key-chunk-stationary backward (chunk not a multiple of 64) adds up dQ through atomics; the other paths keep
  // suffix carries instead
  const bool atomics = chunked && d.chunk % 64 != 0;
  l.dQacc = atomics ? take((size_t)l.Zq * l.Lp * l.D * 4) : 0;
  l.dKdacc = take((size_t)(atomics ? l.Zk : l.Zq) * l.Lp * l.D * 4);   // one slice per query group without atomics
  l.Dsuf = (atomics || l.tiles) ? 0 : take(carries);     // ... and the gradient tiles the suffix carries
  l.masked_nz = take(256);
  // score and decay gradients of every (32 keys, 16 queries) tile (grad_tiles)
  // Grouped queries: the key side sweeps the query groups of a kv head in key_parts parts (UA_TUNE_BWD_PARTS; the key-side
  // sums are then kept per (kv head, part)).  UA_FLAG_SHARE_GROUPS forces one shared sweep.
  l.key_parts = 1;
  if (l.tiles && d.r > 1 && !(d.flags & UA_FLAG_SHARE_GROUPS)) l.key_parts = nth_divisor(d.r, tuned_variant(d, UA_TUNE_BWD_PARTS));
  if (force_parts > 0) l.key_parts = force_parts;
  const size_t Zs = (size_t)l.Zk * l.key_parts;
  const size_t sg = (size_t)ua::grp_tiles(l.Lp / 32) * 1024;    // grouped by the consuming workgroup, per head
  l.dS_st = l.grad_tiles ? take((size_t)l.Zq * sg) : 0;
  l.dG_st = l.grad_tiles ? take(Zs * sg) : 0;
  l.dKrow = take(Zs * l.Lp * l.D * 4);
  l.dVrow = take(Zs * l.Lp * l.D * 4);
  l.dsrc_raw = take(Zs * l.Lp * 4);
  l.total = off;
  return l;
}

ua::RowsView rows_view(const ua_rows& r, int H, int R) {
  ua::RowsView v;
  v.p = r.ptr; v.sb = r.stride_b; v.sh = r.stride_h; v.sr = r.stride_r; v.sn = 0;
  v.so = r.stride_outer; v.si = r.stride_inner; v.sc = 1; v.inner = r.inner_len > 0 ? r.inner_len : 1;
  v.H = H; v.R = R; v.N = 1;
  return v;
}
// contiguous [Z][L] (gates, lse) or [Z][L][d]
ua::RowsView contiguous_view(const void* p, long z_stride, long row_stride) {
  ua::RowsView v;
  v.p = p; v.sb = z_stride; v.sh = 0; v.sr = 0; v.sn = 0; v.so = 0; v.si = row_stride; v.sc = 1;
  v.inner = 1 << 30; v.H = 1; v.R = 1; v.N = 1;
  return v;
}
// chunked tensor (zq, t, dd, i) seen as rows of z = zq*nch + i
ua::RowsView chunked_view(const ua_chunked& c, int nch) {
  ua::RowsView v;
  v.p = c.ptr; v.sb = c.stride_z; v.sh = 0; v.sr = 0; v.sn = c.stride_i; v.so = 0; v.si = c.stride_t; v.sc = c.stride_d;
  v.inner = 1 << 30; v.H = 1; v.R = 1; v.N = nch;
  return v;
}
ua::RowsView null_view() { ua::RowsView v{}; v.inner = 1; v.H = v.R = v.N = 1; return v; }

// tr_mode: column order of the transposed copy inside each group of 32 positions
enum { TR_PERM16 = 0, TR_PERM32 = 1, TR_NATURAL = 2 };
// rows of the view start 16-byte aligned and the feature stride is 1: 16-byte loads are allowed
bool vector_ok(const ua::RowsView& v, size_t esz, int d) {
  const long V = 16 / (long)esz;
  auto al = [&](long stride) { return stride % V == 0; };
  return v.sc == 1 && d % V == 0 && (uintptr_t)v.p % 16 == 0 && al(v.sb) && al(v.sh) && al(v.sr) && al(v.sn) && al(v.so) && al(v.si);
}
template <class T>
hipError_t pack_t(int D, const ua::RowsView& x, void* nat, void* tr, int d, int L, int Lp, int Z, int tr_mode, float* norm2,
                  hipStream_t s, const int* masked_nz, int c) {
  const int tiled = tr_mode != TR_PERM16;      // the fused kernels read tiled working tensors, the chunked ones row-major
  const int vec = vector_ok(x, sizeof(T), d) ? 1 : 0;
  if (D == 256) {
    if constexpr (sizeof(T) == 2) hipLaunchKernelGGL((ua::k_pack<T, 256>), dim3(Lp / 32, Z), dim3(256), 0, s, x, (T*)nat, (T*)tr, d, L, Lp, tr_mode, tiled, vec, norm2, masked_nz, c);
    else return hipErrorInvalidValue;
  } else if (D == 64) hipLaunchKernelGGL((ua::k_pack<T, 64>), dim3(Lp / 32, Z), dim3(256), 0, s, x, (T*)nat, (T*)tr, d, L, Lp, tr_mode, tiled, vec, norm2, masked_nz, c);
  else hipLaunchKernelGGL((ua::k_pack<T, 128>), dim3(Lp / 32, Z), dim3(256), 0, s, x, (T*)nat, (T*)tr, d, L, Lp, tr_mode, tiled, vec, norm2, masked_nz, c);
  return hipGetLastError();
}
// norm2 (optional): [Z][Lp/32] receives the largest squared row norm of every block of 32 rows
// masked_nz, c (optional, chunked upstream gradient): see k_pack
hipError_t pack(int dtype, int D, const ua::RowsView& x, void* nat, void* tr, int d, int L, int Lp, int Z, int tr_mode, hipStream_t s,
                float* norm2 = nullptr, const int* masked_nz = nullptr, int c = 0) {
  return dtype == UA_BF16 ? pack_t<ua::bf16>(D, x, nat, tr, d, L, Lp, Z, tr_mode, norm2, s, masked_nz, c)
                          : pack_t<float>(D, x, nat, tr, d, L, Lp, Z, tr_mode, norm2, s, masked_nz, c);
}

// ---- optional per-kernel timing (hipEvents on the launch stream) ---------------------------
struct ProfRec { const char* name; hipEvent_t e0, e1; };
std::mutex g_prof_mu;
bool g_prof_on = false;
std::vector<ProfRec> g_prof;
struct ProfScope {
  hipEvent_t e1 = nullptr; hipStream_t s;
  ProfScope(const char* name, hipStream_t stream) : s(stream) {
    if (!g_prof_on) return;
    ProfRec r{name, nullptr, nullptr};
    if (hipEventCreate(&r.e0) != hipSuccess || hipEventCreate(&r.e1) != hipSuccess) return;
    (void)hipEventRecord(r.e0, s);
    e1 = r.e1;
    std::lock_guard<std::mutex> g(g_prof_mu);
    g_prof.push_back(r);
  }
  ~ProfScope() { if (e1) (void)hipEventRecord(e1, s); }
};
#define UA_PROF(name, s) ProfScope prof_scope_(name, s)

#define UA_HIP(expr)                                                                         \
  do {                                                                                       \
    hipError_t e_ = (expr);                                                                  \
    if (e_ != hipSuccess) return fail(UA_ELAUNCH, "%s: %s", #expr, hipGetErrorString(e_));   \
  } while (0)

// Workspace conventions of the entry points.  Forward ops: `ws` holds the forward state (l.fwd_end bytes).  Backward ops:
// `fwd_state` is null or the buffer the forward op ran on; `ws` then holds the backward scratch alone (l.total - l.fwd_end
// bytes), else state and scratch together (l.total).  Bases: a forward-state field lives at wf + l.field, a backward
// field at wb + l.field (wb is the scratch pointer minus l.fwd_end when the state is a separate buffer).
int check_common(const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* src, const void* dest, void* ws,
                 size_t ws_bytes, size_t need) {
  if (!kc || !vc || !xq || !kc->ptr || !vc->ptr || !xq->ptr || !src || !dest) return fail(UA_EINVAL, "null input tensor");
  if (!ws) return fail(UA_EWORKSPACE, "null workspace");
  if ((uintptr_t)ws % 256 != 0) return fail(UA_EWORKSPACE, "workspace must be 256-byte aligned");
  if (ws_bytes < need) return fail(UA_EWORKSPACE, "workspace has %zu bytes, %zu needed", ws_bytes, need);
  return UA_OK;
}
int bwd_bases(const Layout& l, void* fwd_state, void* ws, char** wf, char** wb) {
  if (fwd_state) {
    if ((uintptr_t)fwd_state % 256 != 0) return fail(UA_EWORKSPACE, "forward state must be 256-byte aligned");
    *wf = (char*)fwd_state;
    *wb = (char*)ws - l.fwd_end;
  } else {
    *wf = *wb = (char*)ws;
  }
  return UA_OK;
}

hipError_t zero_fill(void* p, size_t bytes, hipStream_t s) {   // bytes is a multiple of 16
  const size_t n16 = bytes / 16;
  const unsigned grid = (unsigned)((n16 + 255) / 256 < 4096 ? (n16 + 255) / 256 : 4096);
  hipLaunchKernelGGL(ua::k_zero, dim3(grid), dim3(256), 0, s, (float4*)p, n16);
  return hipGetLastError();
}

// the gates (static_src, static_dest) and their gradients are float32: always with float32 tensors, with bf16 tensors
// when the caller says so (the reference keeps dstatic_src in static_src.dtype whatever the dtype of q, k, v)
bool gates_f32(const ua_desc& d) { return d.dtype == UA_F32 || (d.flags & UA_FLAG_GATES_F32); }

// packs K, V and Q in both orientations and the log-gates
// chunk sizes the query-stationary kernels handle (the others go through the key-chunk-stationary ones)
bool fast_chunk(const ua_desc& d) { return d.chunk % 64 == 0; }

// rowmajor: working tensors for the key-chunk-stationary (32x32 tile) kernels; otherwise the tiled layout
int pack_inputs(const ua_desc& d, const Layout& l, bool rowmajor, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq,
                const void* src, const void* dest, char* wf, hipStream_t s) {
  const bool chunked = rowmajor;
  UA_PROF("pack_inputs", s);
  const ua::RowsView K = rows_view(*kc, d.h, 1), V = rows_view(*vc, d.h, 1), Q = rows_view(*xq, d.h, d.r);
  // the chunked kernels work on 32x32 tiles, the fused ones on 16x16 tiles (and read V^T in natural order)
  const int mode = chunked ? TR_PERM16 : TR_PERM32;
  const bool prune = !chunked && (d.flags & UA_FLAG_PRUNE);
  UA_HIP(pack(d.dtype, l.D, K, wf + l.Kp, wf + l.KT, d.d, d.L, l.Lp, l.Zk, mode, s, prune ? (float*)(wf + l.knorm2) : nullptr));
  UA_HIP(pack(d.dtype, l.D, V, wf + l.Vp, wf + l.VT, d.d, d.L, l.Lp, l.Zk, chunked ? TR_PERM16 : TR_NATURAL, s));
  UA_HIP(pack(d.dtype, l.D, Q, wf + l.Qp, l.grad_tiles ? nullptr : wf + l.QT, d.d, d.L, l.Lp, l.Zq, mode, s,
              prune ? (float*)(wf + l.qnorm2) : nullptr));
  const dim3 grid((l.Lp + 255) / 256, l.Zk);
  if (!gates_f32(d))
    hipLaunchKernelGGL((ua::k_gates<ua::bf16>), grid, dim3(256), 0, s, (const ua::bf16*)src, (const ua::bf16*)dest,
                       (float*)(wf + l.lsrc), (float*)(wf + l.ldest), d.L, l.Lp);
  else
    hipLaunchKernelGGL((ua::k_gates<float>), grid, dim3(256), 0, s, (const float*)src, (const float*)dest,
                       (float*)(wf + l.lsrc), (float*)(wf + l.ldest), d.L, l.Lp);
  UA_HIP(hipGetLastError());
  return UA_OK;
}

int launch_carry_for(const ua_desc& d, const Layout& l, char* wf, int variant, hipStream_t s) {
  UA_HIP(ua::launch_carry(d.dtype, l.D, wf + l.Kp, (const float*)(wf + l.lsrc), (const float*)(wf + l.ldest),
                          (float*)(wf + l.C), l.Lp, l.Zk, 1, (d.flags & UA_FLAG_PRUNE) ? (const float*)(wf + l.knorm2) : nullptr,
                          (const float*)(wf + l.qnorm2), d.r, (int*)(wf + l.reach), (int*)(wf + l.minkey), s,
                          l.tiles ? wf + l.Bt : nullptr, variant));
  return UA_OK;
}
int launch_fwd_for(const ua_desc& d, const Layout& l, char* wf, void* O, float* lse, int variant, hipStream_t s) {
  UA_HIP(ua::launch_fwd_fused(d.dtype, l.D, variant, wf + l.Qp, wf + l.Kp, wf + l.VT, (const float*)(wf + l.lsrc),
                              (const float*)(wf + l.ldest), (const float*)(wf + l.C), O, lse, (float*)(wf + l.lse2),
                              (const int*)(wf + l.reach), (const int*)(wf + l.minkey), d.r, d.L, l.Lp, d.d, l.Zq, s,
                              l.tiles ? wf + l.Bt : nullptr));
  return UA_OK;
}
int run_fused_fwd_kernels(const ua_desc& d, const Layout& l, char* wf, void* O, float* lse, hipStream_t s) {
  {
    UA_PROF("k_carry", s);
    if (int e = launch_carry_for(d, l, wf, l.tiles ? tuned_variant(d, UA_TUNE_CARRY) : 0, s)) return e;
  }
  UA_PROF("k_fwd_fused", s);
  return launch_fwd_for(d, l, wf, O, lse, tuned_variant(d, l.tiles ? UA_TUNE_FWD_TILES : UA_TUNE_FWD_RECOMPUTE), s);
}

template <class T, class TG>
hipError_t finish_t(const Layout& l, const ua_desc& d, char* wf, char* wb, bool chunked, const void* src, const void* dest, void* dk,
                    void* dv, void* dq, void* dsrc, void* ddest, hipStream_t s) {
  const int Z = l.Zq > l.Zk ? l.Zq : l.Zk;
  hipLaunchKernelGGL((ua::k_bwd_finish<T, TG>), dim3((d.L + 3) / 4, Z), dim3(256), 0, s, (const float*)(wb + l.dKrow),
                     (const float*)(wb + l.dVrow), (const float*)(wb + l.dKdacc), chunked ? (const float*)(wb + l.dQacc) : nullptr,
                     (const float*)(wb + l.dsrc_raw), (const T*)(wf + l.Kp), (const TG*)src, (const TG*)dest, (T*)dk, (T*)dv,
                     (T*)dq, (TG*)dsrc, (TG*)ddest, l.Zk, l.Zq, d.L, l.Lp, l.D, d.d, chunked ? 0 : 1, chunked ? 1 : d.r,
                     l.key_parts);
  return hipGetLastError();
}

template <class T>
hipError_t delta_t(const ua::RowsView& O, const ua::RowsView& dO, const ua::RowsView& sub, const ua::RowsView& lse_in,
                   float* delta, float* lse2, int d, int L, int Lp, int Z, hipStream_t s, int* masked_nz = nullptr, int c = 0) {
  const int vec = vector_ok(O, sizeof(T), d) && vector_ok(dO, sizeof(T), d) ? 1 : 0;
  hipLaunchKernelGGL((ua::k_delta<T>), dim3(Lp / 128, Z), dim3(256), 0, s, O, dO, sub, lse_in, delta, lse2, d, L, Lp, vec, masked_nz, c);
  return hipGetLastError();
}

// chunked with a chunk that is not a multiple of 64: key-chunk-stationary kernel over row-major working tensors (atomics);
// otherwise the key-stationary and query-stationary kernels over tiled working tensors
int run_bwd_common(const ua_desc& d, const Layout& l, char* wf, char* wb, bool chunked, const void* src, const void* dest, void* dkc,
                   void* dvc, void* dxq, void* dsrc, void* ddest, hipStream_t s, const float* delta_given = nullptr,
                   const float* lse2_given = nullptr, const void* dO_rows = nullptr) {
  const bool is_chunked = chunked;
  chunked = is_chunked && !fast_chunk(d);      // from here on: the atomics path
  if (chunked) {
    UA_PROF("k_zero", s);
    UA_HIP(zero_fill(wb + l.dQacc, (size_t)l.Zq * l.Lp * l.D * 4, s));
    UA_HIP(zero_fill(wb + l.dKdacc, (size_t)l.Zk * l.Lp * l.D * 4, s));
  }
  ua::BwdArgsV a{};
  a.Kp = wf + l.Kp; a.Vp = wf + l.Vp; a.KT = wf + l.KT; a.Qp = wf + l.Qp; a.QT = l.grad_tiles ? nullptr : wf + l.QT; a.dOp = wb + l.dOp;
  a.dOT = l.grad_tiles ? nullptr : wb + l.dOT; a.lsrc = (const float*)(wf + l.lsrc); a.ldest = (const float*)(wf + l.ldest);
  a.lse2 = lse2_given ? lse2_given : (const float*)(wf + l.lse2); a.delta = delta_given ? delta_given : (const float*)(wb + l.delta); a.C = (const float*)(wf + l.C);
  a.reach = (const int*)(wf + l.reach); a.minkey = (const int*)(wf + l.minkey);
  a.dQacc = (float*)(wb + l.dQacc); a.dKdacc = (float*)(wb + l.dKdacc); a.Dsuf = (float*)(wb + l.Dsuf);
  a.dKrow = (float*)(wb + l.dKrow);
  a.dVrow = (float*)(wb + l.dVrow); a.dsrc_raw = (float*)(wb + l.dsrc_raw);
  a.masked_nz = (const int*)(wb + l.masked_nz);
  a.dS_st = l.grad_tiles ? wb + l.dS_st : nullptr; a.dG_st = l.grad_tiles ? wb + l.dG_st : nullptr; a.Bt = l.tiles ? wf + l.Bt : nullptr;
  if (dO_rows) { a.dOp = dO_rows; a.dO_rows = 1; }      // the caller's upstream gradient, read in place by k_bwd_keys2
  a.R = d.r; a.L = d.L; a.Lp = l.Lp; a.c = is_chunked ? d.chunk : 128; a.nch = l.nch; a.chunked = is_chunked ? 1 : 0;
  a.skip_masked = (d.flags & UA_FLAG_SKIP_MASKED) ? 1 : 0;
  a.split_r = (!chunked && d.r > 1) ? 1 : 0;
  a.key_parts = l.key_parts;
  a.keys_variant = l.tiles ? tuned_variant(d, UA_TUNE_BWD_KEYS) : 0;
  a.pair = is_chunked ? tuned_variant(d, UA_TUNE_CHUNKED_PAIR) : 0;
  // bf16 tile exchange with one query group: the two kernels write the caller's gradients themselves.  The chunked
  // operator qualifies when the caller asserts that nothing flows to (query, later chunk) pairs, so that the query side is
  // known here to run from the tiles.
  const bool from_tiles = l.tiles || (is_chunked && l.grad_tiles && (d.flags & UA_FLAG_SKIP_MASKED));
  const bool direct = from_tiles && d.r == 1 && !gates_f32(d);
  a.direct = direct ? 1 : 0; a.d_out = d.d; a.dk_out = dkc; a.dv_out = dvc; a.dsrc_out = dsrc; a.ddest_out = ddest;
  a.src_in = src; a.dest_in = dest;
  {
    UA_PROF("k_bwd_keys", s);
    UA_HIP(ua::launch_bwd_keys(d.dtype, l.D, a, l.Zk, chunked ? 1 : 0, s));
  }
  if (!chunked) {
    UA_PROF("k_bwd_queries", s);
    // chunked operator with tiles: both are enqueued, the flag k_delta left on the device decides which one works
    if (l.grad_tiles) UA_HIP(ua::launch_bwd_queries_from_tiles(l.D, a, dxq, d.d, l.Zq, s, tuned_variant(d, UA_TUNE_BWD_QUERIES)));
    if (!from_tiles) UA_HIP(ua::launch_bwd_queries(d.dtype, l.D, a, dxq, d.d, l.Zk, s));
  }
  if (direct) return UA_OK;
  UA_PROF("k_bwd_finish", s);
  if (d.dtype == UA_BF16 && gates_f32(d)) UA_HIP((finish_t<ua::bf16, float>(l, d, wf, wb, chunked, src, dest, dkc, dvc, dxq, dsrc, ddest, s)));
  else if (d.dtype == UA_BF16) UA_HIP((finish_t<ua::bf16, ua::bf16>(l, d, wf, wb, chunked, src, dest, dkc, dvc, dxq, dsrc, ddest, s)));
  else UA_HIP((finish_t<float, float>(l, d, wf, wb, chunked, src, dest, dkc, dvc, dxq, dsrc, ddest, s)));
  return UA_OK;
}

}  // namespace

namespace {
// times launch(variant) for every variant of the slot (one warm-up, the fastest of six timed launches each) and
// records the fastest; the events are destroyed on every path
template <class F>
int tune_slot(const ua_desc& d, int slot, hipStream_t s, F launch) {
  const int n = n_variants(d, slot);
  if (n <= 1) return UA_OK;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    if (e0) (void)hipEventDestroy(e0);
    return fail(UA_ELAUNCH, "hipEventCreate failed");
  }
  int best = -1, rc = UA_OK;
  float best_ms = 1e30f;
  for (int v = 0; v < n && rc == UA_OK; ++v) {
    for (int rep = 0; rep < 7 && rc == UA_OK; ++rep) {
      if (hipEventRecord(e0, s) != hipSuccess) { rc = fail(UA_ELAUNCH, "hipEventRecord failed"); break; }
      const int e = launch(v);
      if (e == 1) break;                     // variant not applicable to this problem
      if (e != UA_OK) { rc = e; break; }
      float ms = 0.f;
      if (hipEventRecord(e1, s) != hipSuccess || hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) {
        rc = fail(UA_ELAUNCH, "timing variant %d of slot %d failed", v, slot);
        break;
      }
      if (rep > 0 && ms < best_ms) { best_ms = ms; best = v; }
    }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != UA_OK) return rc;
  if (best >= 0) {
    std::lock_guard<std::mutex> g(g_tune_mu);
    g_tune[tune_key(d, slot)] = best;
  }
  return UA_OK;
}
}  // namespace

extern "C" {

int ua_version(void) { return 2; }
#ifndef UA_SOURCE_HASH
#define UA_SOURCE_HASH "unknown"
#endif
const char* ua_source_hash(void) { return UA_SOURCE_HASH; }
const char* ua_last_error(void) { return g_err; }

size_t ua_workspace_bytes(const ua_desc* desc, int op) {
  if (op < UA_OP_FWD || op > UA_OP_FUSED_BWD_SCRATCH) { fail(UA_EINVAL, "unknown op %d", op); return 0; }
  const bool chunked = (op == UA_OP_FWD || op == UA_OP_BWD || op == UA_OP_BWD_SCRATCH);
  if (check_desc(desc, chunked) != UA_OK) return 0;
  const Layout l = make_layout(*desc, chunked);
  if (op == UA_OP_FWD || op == UA_OP_FUSED_FWD) return l.fwd_end;
  if (op == UA_OP_BWD_SCRATCH || op == UA_OP_FUSED_BWD_SCRATCH) return l.total - l.fwd_end;
  return l.total;
}

int ua_fused_fwd(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
                 const void* static_dest, void* O, float* lse, void* ws, size_t ws_bytes, ua_stream_t stream) {
  if (int e = check_desc(desc, false)) return e;
  const Layout l = make_layout(*desc, false);
  if (int e = check_common(kc, vc, xq, static_src, static_dest, ws, ws_bytes, l.fwd_end)) return e;
  if (!O || !lse) return fail(UA_EINVAL, "null output tensor");
  char* wf = (char*)ws;
  hipStream_t s = (hipStream_t)stream;
  if (int e = pack_inputs(*desc, l, false, kc, vc, xq, static_src, static_dest, wf, s)) return e;
  return run_fused_fwd_kernels(*desc, l, wf, O, lse, s);
}

// ---- forward for callers that cannot allocate: scratch in a device array of the library itself ----------------
// One copy of the array exists per GPU, at its own address; the name below is only a host-side handle, the address
// comes from hipGetSymbolAddress with that GPU current and is what the kernels receive.
static __device__ __align__(256) unsigned char scratch[UA_NOALLOC_SCRATCH_BYTES];
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};
int scratch_of_current_device(void** out) {
  int dev = -1;
  UA_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(UA_EINVAL, "device index %d out of range", dev);
  std::lock_guard<std::mutex> g(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    UA_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(UA_ELAUNCH, "hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return UA_OK;
}
}  // namespace

size_t ua_noalloc_scratch_bytes(void) { return UA_NOALLOC_SCRATCH_BYTES; }

int ua_fused_fwd_noalloc(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
                         const void* static_dest, void* O, float* lse, ua_stream_t stream) {
  if (int e = check_desc(desc, false)) return e;
  const Layout l = make_layout(*desc, false);
  if (l.fwd_end > (size_t)UA_NOALLOC_SCRATCH_BYTES)
    return fail(UA_EWORKSPACE, "problem needs %zu bytes of scratch, the built-in array holds %zu: use ua_fused_fwd with a workspace",
                l.fwd_end, (size_t)UA_NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (int e = scratch_of_current_device(&ws)) return e;
  // every region of the forward state is written before it is read (padding included), so nothing of the previous
  // call's contents has to be cleared
  return ua_fused_fwd(desc, kc, vc, xq, static_src, static_dest, O, lse, ws, UA_NOALLOC_SCRATCH_BYTES, stream);
}

int ua_fused_bwd(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
                 const void* static_dest, const void* O, const float* lse, const void* dO, void* dkc, void* dvc, void* dxq,
                 void* dsrc, void* ddest, void* fwd_state, void* ws, size_t ws_bytes, ua_stream_t stream) {
  if (int e = check_desc(desc, false)) return e;
  const Layout l = make_layout(*desc, false);
  if (int e = check_common(kc, vc, xq, static_src, static_dest, ws, ws_bytes, fwd_state ? l.total - l.fwd_end : l.total)) return e;
  if (!O || !lse || !dO || !dkc || !dvc || !dxq || !dsrc || !ddest) return fail(UA_EINVAL, "null tensor");
  char *wf, *wb;
  if (int e = bwd_bases(l, fwd_state, ws, &wf, &wb)) return e;
  hipStream_t s = (hipStream_t)stream;
  const ua_desc& d = *desc;
  if (!fwd_state) {
    if (int e = pack_inputs(d, l, false, kc, vc, xq, static_src, static_dest, wf, s)) return e;
    if (int e = launch_carry_for(d, l, wf, l.tiles ? tuned_variant(d, UA_TUNE_CARRY) : 0, s)) return e;
  }
  const long rowsz = (long)d.L * d.d;
  const ua::RowsView Ov = contiguous_view(O, rowsz, d.d), dOv = contiguous_view(dO, rowsz, d.d);
  const ua::RowsView lsev = contiguous_view(lse, d.L, 1), none = null_view();
  {
    UA_PROF("pack_dO+delta", s);
    UA_HIP(pack(d.dtype, l.D, dOv, wb + l.dOp, l.grad_tiles ? nullptr : wb + l.dOT, d.d, d.L, l.Lp, l.Zq, TR_PERM32, s));
    if (d.dtype == UA_BF16) UA_HIP(delta_t<ua::bf16>(Ov, dOv, none, lsev, (float*)(wb + l.delta), (float*)(wf + l.lse2), d.d, d.L, l.Lp, l.Zq, s));
    else UA_HIP(delta_t<float>(Ov, dOv, none, lsev, (float*)(wb + l.delta), (float*)(wf + l.lse2), d.d, d.L, l.Lp, l.Zq, s));
  }
  return run_bwd_common(d, l, wf, wb, false, static_src, static_dest, dkc, dvc, dxq, dsrc, ddest, s);
}

int ua_fwd(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
           const void* static_dest, const ua_chunked* out, void* denom, float* lse2_out, void* ws, size_t ws_bytes,
           ua_stream_t stream) {
  if (int e = check_desc(desc, true)) return e;
  const Layout l = make_layout(*desc, true);
  if (int e = check_common(kc, vc, xq, static_src, static_dest, ws, ws_bytes, l.fwd_end)) return e;
  if (!out || !out->ptr || !denom) return fail(UA_EINVAL, "null output tensor");
  char* wf = (char*)ws;
  hipStream_t s = (hipStream_t)stream;
  const ua_desc& d = *desc;
  float* lse2 = lse2_out ? lse2_out : (float*)(wf + l.lse2);     // the per-chunk normalisers, float32, log2 units
  // the workspace stays a complete forward state for ua_bwd also when the normalisers went to the caller's buffer
  auto mirror_lse2 = [&]() -> int {
    if (lse2_out) UA_HIP(hipMemcpyAsync(wf + l.lse2, lse2_out, (size_t)l.Zq * l.nch * l.Lp * 4, hipMemcpyDeviceToDevice, s));
    return UA_OK;
  };
  if (fast_chunk(d)) {
    if (int e = pack_inputs(d, l, false, kc, vc, xq, static_src, static_dest, wf, s)) return e;
    {
      UA_PROF("k_carry", s);
      UA_HIP(ua::launch_carry(d.dtype, l.D, wf + l.Kp, (const float*)(wf + l.lsrc), (const float*)(wf + l.ldest), (float*)(wf + l.C), l.Lp,
                              l.Zk, 1, nullptr, nullptr, d.r, (int*)(wf + l.reach), (int*)(wf + l.minkey), s));
    }
    UA_PROF("k_fwd_chunked", s);
    UA_HIP(ua::launch_fwd_chunked2(d.dtype, l.D, wf + l.Qp, wf + l.Kp, wf + l.Vp, wf + l.VT, (const float*)(wf + l.lsrc),
                                   (const float*)(wf + l.ldest), (const float*)(wf + l.C), (const int*)(wf + l.reach),
                                   (const int*)(wf + l.minkey), out->ptr, denom, lse2, out->stride_z, out->stride_t,
                                   out->stride_d, out->stride_i, d.r, d.L, l.Lp, d.d, d.chunk, l.nch, l.Zq, s,
                                   tuned_variant(d, UA_TUNE_CHUNKED_PAIR)));
    return mirror_lse2();
  }
  if (int e = pack_inputs(d, l, true, kc, vc, xq, static_src, static_dest, wf, s)) return e;
  UA_PROF("k_fwd_chunked", s);
  UA_HIP(ua::launch_fwd_chunked(d.dtype, l.D, wf + l.Qp, wf + l.Kp, wf + l.VT, (const float*)(wf + l.lsrc),
                                (const float*)(wf + l.ldest), out->ptr, denom, lse2, out->stride_z, out->stride_t, out->stride_d, out->stride_i, d.r, d.L,
                                l.Lp, d.d, d.chunk, l.nch, l.Zk, s));
  return mirror_lse2();
}

int ua_bwd(const ua_desc* desc, const ua_rows* kc, const ua_rows* vc, const ua_rows* xq, const void* static_src,
           const void* static_dest, const ua_chunked* out, const ua_chunked* g_out, const float* g_denom, void* dkc,
           void* dvc, void* dxq, void* dsrc, void* ddest, const float* delta, const float* lse2_in, void* fwd_state, void* ws,
           size_t ws_bytes, ua_stream_t stream) {
  if (int e = check_desc(desc, true)) return e;
  const Layout l = make_layout(*desc, true);
  if (int e = check_common(kc, vc, xq, static_src, static_dest, ws, ws_bytes, fwd_state ? l.total - l.fwd_end : l.total)) return e;
  if (!out || !out->ptr || !g_out || !g_out->ptr || !g_denom || !dkc || !dvc || !dxq || !dsrc || !ddest)
    return fail(UA_EINVAL, "null tensor");
  if (delta && !(desc->flags & UA_FLAG_SKIP_MASKED)) return fail(UA_EINVAL, "a precomputed delta needs UA_FLAG_SKIP_MASKED and a chunk that is a multiple of 64");
  char *wf, *wb;
  if (int e = bwd_bases(l, fwd_state, ws, &wf, &wb)) return e;
  hipStream_t s = (hipStream_t)stream;
  const ua_desc& d = *desc;
  const ua::RowsView outv = chunked_view(*out, l.nch);
  ua_chunked gmut = *g_out;
  const ua::RowsView gv = chunked_view(gmut, l.nch), none = null_view();
  // g_denom [zq][t][i] seen per z = zq*nch + i
  ua::RowsView gdv;
  gdv.p = g_denom; gdv.sb = (long)d.L * l.nch; gdv.sh = 0; gdv.sr = 0; gdv.sn = 1; gdv.so = 0; gdv.si = l.nch; gdv.sc = 1;
  gdv.inner = 1 << 30; gdv.H = 1; gdv.R = 1; gdv.N = l.nch;
  if (fast_chunk(d)) {
    if (!fwd_state) {
      // recompute the carries and the per-chunk normalisers (the partial outputs themselves are passed in)
      if (int e = pack_inputs(d, l, false, kc, vc, xq, static_src, static_dest, wf, s)) return e;
      UA_HIP(ua::launch_carry(d.dtype, l.D, wf + l.Kp, (const float*)(wf + l.lsrc), (const float*)(wf + l.ldest), (float*)(wf + l.C), l.Lp,
                              l.Zk, 1, nullptr, nullptr, d.r, (int*)(wf + l.reach), (int*)(wf + l.minkey), s));
      if (!lse2_in)
        UA_HIP(ua::launch_fwd_chunked2(d.dtype, l.D, wf + l.Qp, wf + l.Kp, wf + l.Vp, wf + l.VT, (const float*)(wf + l.lsrc),
                                       (const float*)(wf + l.ldest), (const float*)(wf + l.C), (const int*)(wf + l.reach),
                                       (const int*)(wf + l.minkey), nullptr, nullptr, (float*)(wf + l.lse2), 0, 0, 0, 0, d.r, d.L, l.Lp,
                                       d.d, d.chunk, l.nch, l.Zq, s, tuned_variant(d, UA_TUNE_CHUNKED_PAIR)));
    }
    bool in_place = false;
    {
      UA_PROF("pack_dO+delta", s);
      UA_HIP(zero_fill(wb + l.masked_nz, 256, s));
      // with UA_FLAG_SKIP_MASKED the flag stays 0: rows before their chunk are neither checked nor packed
      int* nz = (int*)(wb + l.masked_nz);
      int* detect = (d.flags & UA_FLAG_SKIP_MASKED) ? nullptr : nz;
      if (delta) { /* ua_merge_bwd left it: neither out nor g_out is read for it */ }
      else if (d.dtype == UA_BF16) UA_HIP(delta_t<ua::bf16>(outv, gv, gdv, none, (float*)(wb + l.delta), nullptr, d.d, d.L, l.Lp, l.Zq * l.nch, s, detect, d.chunk));
      else UA_HIP(delta_t<float>(outv, gv, gdv, none, (float*)(wb + l.delta), nullptr, d.d, d.L, l.Lp, l.Zq * l.nch, s, detect, d.chunk));
      // With the tile exchange only the key-side kernel reads the upstream gradient, and when nothing flows to the
      // (query, later chunk) pairs (UA_FLAG_SKIP_MASKED) it can gather its tiles from the caller's tensor itself if that
      // is stored chunk-major in rows of exactly D elements: no packed copy (half of g_out read, as much written).
      in_place = l.grad_tiles && (d.flags & UA_FLAG_SKIP_MASKED) && d.d == l.D && d.L % 32 == 0 && g_out->stride_d == 1 &&
                 g_out->stride_t == d.d && g_out->stride_i == (int64_t)d.L * d.d && g_out->stride_z == (int64_t)l.nch * d.L * d.d &&
                 (uintptr_t)g_out->ptr % 16 == 0;
      if (!in_place)
        UA_HIP(pack(d.dtype, l.D, gv, wb + l.dOp, l.grad_tiles ? nullptr : wb + l.dOT, d.d, d.L, l.Lp, l.Zq * l.nch, TR_PERM32, s, nullptr, nz,
                    d.chunk));
    }
    return run_bwd_common(d, l, wf, wb, true, static_src, static_dest, dkc, dvc, dxq, dsrc, ddest, s, delta, lse2_in,
                          in_place ? g_out->ptr : nullptr);
  }
  if (delta) return fail(UA_EINVAL, "a precomputed delta needs UA_FLAG_SKIP_MASKED and a chunk that is a multiple of 64");
  if (!fwd_state) {
    // recompute the per-chunk normalisers (the partial outputs themselves are passed in)
    if (int e = pack_inputs(d, l, true, kc, vc, xq, static_src, static_dest, wf, s)) return e;
    if (!lse2_in)
      UA_HIP(ua::launch_fwd_chunked(d.dtype, l.D, wf + l.Qp, wf + l.Kp, wf + l.VT, (const float*)(wf + l.lsrc),
                                    (const float*)(wf + l.ldest), nullptr, nullptr, (float*)(wf + l.lse2), 0, 0, 0, 0, d.r, d.L, l.Lp, d.d, d.chunk, l.nch, l.Zk, s));
  }
  UA_HIP(ua::launch_carry(d.dtype, l.D, wf + l.Kp, (const float*)(wf + l.lsrc), (const float*)(wf + l.ldest),
                          (float*)(wf + l.C), l.Lp, l.Zk, 0, nullptr, nullptr, 1, nullptr, nullptr, s));
  UA_HIP(pack(d.dtype, l.D, gv, wb + l.dOp, wb + l.dOT, d.d, d.L, l.Lp, l.Zq * l.nch, TR_PERM16, s));
  if (d.dtype == UA_BF16) UA_HIP(delta_t<ua::bf16>(outv, gv, gdv, none, (float*)(wb + l.delta), nullptr, d.d, d.L, l.Lp, l.Zq * l.nch, s));
  else UA_HIP(delta_t<float>(outv, gv, gdv, none, (float*)(wb + l.delta), nullptr, d.d, d.L, l.Lp, l.Zq * l.nch, s));
  return run_bwd_common(d, l, wf, wb, true, static_src, static_dest, dkc, dvc, dxq, dsrc, ddest, s, nullptr, lse2_in);
}

// 16-byte accesses to every (row, chunk) slice of a chunked tensor, with d / V lanes per slice (a power of two <= 64)
static bool merge_vector_ok(const ua_chunked& c, int dtype, int d) {
  const long V = dtype == UA_BF16 ? 8 : 4;
  if (c.stride_d != 1 || d % V != 0) return false;
  const long lpr = d / V;
  if (lpr > 64 || (lpr & (lpr - 1)) != 0) return false;
  return (uintptr_t)c.ptr % 16 == 0 && c.stride_z % V == 0 && c.stride_t % V == 0 && c.stride_i % V == 0;
}

int ua_merge_fwd(int dtype, int64_t rows, int32_t L, int32_t d, int32_t n, const ua_chunked* mat, const void* vec,
                 void* result, ua_stream_t stream) {
  if (!mat || !mat->ptr || !vec || !result) return fail(UA_EINVAL, "null tensor");
  if (rows < 1 || L < 1 || d < 1 || n < 1 || n > ua::kMergeMaxN) return fail(UA_EINVAL, "bad merge shape rows=%ld L=%d d=%d n=%d", (long)rows, L, d, n);
  if (dtype != UA_F32 && dtype != UA_BF16) return fail(UA_EINVAL, "dtype %d unsupported", dtype);
  ua::ChunkedView m{mat->ptr, mat->stride_z, mat->stride_t, mat->stride_d, mat->stride_i};
  const dim3 grid((unsigned)((rows + 3) / 4));
  const size_t lds = 4 * (size_t)n * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  const bool vecp = merge_vector_ok(*mat, dtype, d) && (uintptr_t)result % 16 == 0;
#define UA_MERGE_FWD(T, VEC) hipLaunchKernelGGL((ua::k_merge_fwd<T, VEC>), grid, dim3(256), lds, s, m, (const T*)vec, (T*)result, (long)rows, L, d, n)
  if (dtype == UA_BF16) { if (vecp) UA_MERGE_FWD(ua::bf16, true); else UA_MERGE_FWD(ua::bf16, false); }
  else { if (vecp) UA_MERGE_FWD(float, true); else UA_MERGE_FWD(float, false); }
#undef UA_MERGE_FWD
  UA_HIP(hipGetLastError());
  return UA_OK;
}

int ua_merge_bwd(int dtype, int64_t rows, int32_t L, int32_t d, int32_t n, const ua_chunked* mat, const void* vec,
                 const void* g, const ua_chunked* d_mat, void* d_vec, float* delta, ua_stream_t stream) {
  if (!mat || !mat->ptr || !vec || !g || !d_mat || !d_mat->ptr || !d_vec) return fail(UA_EINVAL, "null tensor");
  if (rows < 1 || L < 1 || d < 1 || n < 1 || n > ua::kMergeMaxN) return fail(UA_EINVAL, "bad merge shape rows=%ld L=%d d=%d n=%d", (long)rows, L, d, n);
  if (dtype != UA_F32 && dtype != UA_BF16) return fail(UA_EINVAL, "dtype %d unsupported", dtype);
  ua::ChunkedView m{mat->ptr, mat->stride_z, mat->stride_t, mat->stride_d, mat->stride_i};
  ua::ChunkedView dm{d_mat->ptr, d_mat->stride_z, d_mat->stride_t, d_mat->stride_d, d_mat->stride_i};
  const dim3 grid((unsigned)((rows + 3) / 4));
  const size_t lds = 8 * (size_t)n * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  const bool vecp = merge_vector_ok(*mat, dtype, d) && merge_vector_ok(*d_mat, dtype, d) && (uintptr_t)g % 16 == 0;
  const int Lp = (int)align_up((size_t)L, 128);
#define UA_MERGE_BWD(T, VEC) hipLaunchKernelGGL((ua::k_merge_bwd<T, VEC>), grid, dim3(256), lds, s, m, (const T*)vec, (const T*)g, dm, (T*)d_vec, (long)rows, L, d, n, delta, Lp)
  if (dtype == UA_BF16) { if (vecp) UA_MERGE_BWD(ua::bf16, true); else UA_MERGE_BWD(ua::bf16, false); }
  else { if (vecp) UA_MERGE_BWD(float, true); else UA_MERGE_BWD(float, false); }
#undef UA_MERGE_BWD
  UA_HIP(hipGetLastError());
  return UA_OK;
}

// ---- stand-alone decay bias (affinity scores) ------------------------------------------------
namespace {
struct AffLayout { int D, Lp, Z; bool tiles; size_t Kp, KT, lsrc, ldest, fwd_end, DL, Wst, row, colp, gs_row, gs_col, total; };
AffLayout make_aff_layout(const ua_desc& d) {
  AffLayout l{};
  l.D = d.d <= 64 ? 64 : 128;
  l.Lp = (int)align_up((size_t)d.L, 128);
  l.Z = d.b * d.h;
  const size_t esz = d.dtype == UA_BF16 ? 2 : 4;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const size_t kbytes = (size_t)l.Z * l.Lp * l.D * esz;
  l.Kp = take(kbytes); l.KT = take(kbytes);
  l.lsrc = take((size_t)l.Z * l.Lp * 4); l.ldest = take((size_t)l.Z * l.Lp * 4);
  l.fwd_end = off;
  // bf16 with rows of daff that can be 16-byte aligned: the backward exchanges bf16 tiles over the causal triangle
  // (2 bytes per pair) instead of a float L x L running sum
  l.tiles = d.dtype == UA_BF16 && d.L % 8 == 0;
  l.DL = l.tiles ? 0 : take((size_t)l.Z * d.L * d.L * 4);
  l.Wst = l.tiles ? take((size_t)l.Z * ua::tri_tiles(l.Lp / 32) * 1024) : 0;
  l.row = take((size_t)l.Z * l.Lp * l.D * 4); l.colp = take((size_t)l.Z * l.Lp * l.D * 4);
  l.gs_row = take((size_t)l.Z * l.Lp * 4); l.gs_col = take((size_t)l.Z * l.Lp * 4);
  l.total = off;
  return l;
}
int aff_prepare(const ua_desc* desc, const ua_rows* k, const void* src, const void* dest, void* ws, size_t ws_bytes, bool bwd,
                AffLayout& l, hipStream_t s) {
  if (int e = check_desc(desc, false)) return e;
  if (desc->d > 128) return fail(UA_EINVAL, "head dim %d > 128 is not supported by the stand-alone bias", desc->d);
  l = make_aff_layout(*desc);
  if (!k || !k->ptr || !src || !dest) return fail(UA_EINVAL, "null input tensor");
  if (!ws) return fail(UA_EWORKSPACE, "null workspace");
  if ((uintptr_t)ws % 256 != 0) return fail(UA_EWORKSPACE, "workspace must be 256-byte aligned");
  const size_t need = bwd ? l.total : l.fwd_end;
  if (ws_bytes < need) return fail(UA_EWORKSPACE, "workspace has %zu bytes, %zu needed", ws_bytes, need);
  const ua_desc& d = *desc;
  char* w = (char*)ws;
  const ua::RowsView K = rows_view(*k, d.h, 1);
  UA_HIP(pack(d.dtype, l.D, K, w + l.Kp, w + l.KT, d.d, d.L, l.Lp, l.Z, TR_PERM32, s));
  const dim3 grid((l.Lp + 255) / 256, l.Z);
  if (d.dtype == UA_BF16)
    hipLaunchKernelGGL((ua::k_gates<ua::bf16>), grid, dim3(256), 0, s, (const ua::bf16*)src, (const ua::bf16*)dest,
                       (float*)(w + l.lsrc), (float*)(w + l.ldest), d.L, l.Lp);
  else
    hipLaunchKernelGGL((ua::k_gates<float>), grid, dim3(256), 0, s, (const float*)src, (const float*)dest,
                       (float*)(w + l.lsrc), (float*)(w + l.ldest), d.L, l.Lp);
  UA_HIP(hipGetLastError());
  return UA_OK;
}
}  // namespace

size_t ua_affinity_workspace_bytes(const ua_desc* desc, int backward) {
  if (check_desc(desc, false) != UA_OK) return 0;
  if (desc->d > 128) { fail(UA_EINVAL, "head dim %d > 128 is not supported by the stand-alone bias", desc->d); return 0; }
  const AffLayout l = make_aff_layout(*desc);
  return backward ? l.total : l.fwd_end;
}

int ua_affinity_fwd(const ua_desc* desc, const ua_rows* k, const void* src, const void* dest, void* aff, void* ws,
                    size_t ws_bytes, ua_stream_t stream) {
  AffLayout l;
  hipStream_t s = (hipStream_t)stream;
  if (!aff) return fail(UA_EINVAL, "null output tensor");
  if (int e = aff_prepare(desc, k, src, dest, ws, ws_bytes, false, l, s)) return e;
  char* w = (char*)ws;
  UA_HIP(ua::launch_aff_fwd(desc->dtype, l.D, w + l.Kp, (const float*)(w + l.lsrc), (const float*)(w + l.ldest), aff, desc->L, l.Lp,
                            l.Z, s, tuned_variant(*desc, UA_TUNE_AFF_PAIR)));
  return UA_OK;
}

int ua_affinity_bwd(const ua_desc* desc, const ua_rows* k, const void* src, const void* dest, const void* daff, void* dk,
                    void* dsrc, void* ddest, void* ws, size_t ws_bytes, ua_stream_t stream) {
  AffLayout l;
  hipStream_t s = (hipStream_t)stream;
  if (!daff || !dk || !dsrc || !ddest) return fail(UA_EINVAL, "null tensor");
  if (int e = aff_prepare(desc, k, src, dest, ws, ws_bytes, true, l, s)) return e;
  if (l.tiles && (uintptr_t)daff % 16 != 0) return fail(UA_EINVAL, "daff must be 16-byte aligned (bf16, L a multiple of 8)");
  char* w = (char*)ws;
  UA_HIP(ua::launch_aff_bwd(desc->dtype, l.D, w + l.Kp, w + l.KT, (const float*)(w + l.lsrc), (const float*)(w + l.ldest), daff,
                            (float*)(w + l.DL), (float*)(w + l.row), (float*)(w + l.colp), (float*)(w + l.gs_row),
                            (float*)(w + l.gs_col), src, dest, dk, dsrc, ddest, desc->L, l.Lp, desc->d, l.Z, s,
                            l.tiles ? w + l.Wst : nullptr, tuned_variant(*desc, UA_TUNE_AFF_PAIR)));
  return UA_OK;
}

void ua_prof_enable(int on) {
  std::lock_guard<std::mutex> g(g_prof_mu);
  g_prof_on = on != 0;
}
int ua_prof_collect(char* buf, size_t cap) {
  if (hipDeviceSynchronize() != hipSuccess) return fail(UA_ELAUNCH, "synchronize failed");
  std::lock_guard<std::mutex> g(g_prof_mu);
  std::map<std::string, std::pair<int, double>> acc;
  for (auto& r : g_prof) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, r.e0, r.e1) == hipSuccess) { auto& a = acc[r.name]; a.first += 1; a.second += ms; }
    (void)hipEventDestroy(r.e0); (void)hipEventDestroy(r.e1);
  }
  g_prof.clear();
  std::string out;
  char line[160];
  for (auto& kv : acc) { snprintf(line, sizeof(line), "%s:%d:%.6f;", kv.first.c_str(), kv.second.first, kv.second.second); out += line; }
  if (!buf || cap == 0) return (int)out.size();
  snprintf(buf, cap, "%s", out.c_str());
  return (int)out.size();
}

int ua_tune_variants(const ua_desc* desc, int slot) {
  if (!known_slot(slot)) return fail(UA_EINVAL, "unknown kernel slot %d", slot);
  if (int e = check_desc(desc, false)) return e;
  return n_variants(*desc, slot);
}
int ua_tune_get(const ua_desc* desc, int slot) {
  if (!desc) return -1;
  return tune_entry(*desc, slot);
}
int ua_tune_choice(const ua_desc* desc, int slot) {
  const int n = ua_tune_variants(desc, slot);
  if (n < 0) return n;
  return tuned_variant(*desc, slot);
}
int ua_tune_set(const ua_desc* desc, int slot, int variant) {
  const int n = ua_tune_variants(desc, slot);
  if (n < 0) return n;
  if (variant < -1 || variant >= n) return fail(UA_EINVAL, "variant %d out of range [-1,%d)", variant, n);
  std::lock_guard<std::mutex> g(g_tune_mu);
  if (variant < 0) g_tune.erase(tune_key(*desc, slot));
  else g_tune[tune_key(*desc, slot)] = variant;
  return UA_OK;
}

int ua_autotune(const ua_desc* desc, int op, void* ws, size_t ws_bytes, ua_stream_t stream) {
  if (op != UA_OP_FUSED_FWD && op != UA_OP_FUSED_BWD) return fail(UA_EINVAL, "ua_autotune tunes UA_OP_FUSED_FWD or UA_OP_FUSED_BWD (got %d)", op);
  if (int e = check_desc(desc, false)) return e;
  const ua_desc& d = *desc;
  Layout l = make_layout(d, false);
  if (!ws || (uintptr_t)ws % 256 != 0) return fail(UA_EWORKSPACE, "autotune needs the 256-byte aligned workspace the op ran on");
  if (ws_bytes < l.total) return fail(UA_EWORKSPACE, "autotune needs the backward-sized workspace (%zu bytes)", l.total);
  char* w = (char*)ws;
  char *wf = w, *wb = w;      // state and scratch in one buffer
  hipStream_t s = (hipStream_t)stream;
  // throw-away outputs live in the backward part of the workspace
  if (op == UA_OP_FUSED_FWD) {
    void* Otmp = wb + l.dOp;                  // [Zq][L][d] fits in [Zq][Lp][D]
    float* lsetmp = (float*)(wb + l.delta);
    if (l.tiles) {
      if (int e = tune_slot(d, UA_TUNE_FWD_TILES, s, [&](int v) { return launch_fwd_for(d, l, w, Otmp, lsetmp, v, s); })) return e;
      // the pre-pass rewrites the bias tiles, the reach table and the first-key table with the same values
      if (int e = tune_slot(d, UA_TUNE_CARRY, s, [&](int v) { return launch_carry_for(d, l, w, v, s); })) return e;
    } else {
      if (int e = tune_slot(d, UA_TUNE_FWD_RECOMPUTE, s, [&](int v) { return launch_fwd_for(d, l, w, Otmp, lsetmp, v, s); })) return e;
    }
    return UA_OK;
  }
  if (!l.tiles) return UA_OK;                // the recomputing backward has one variant per kernel
  // key side first (it reads the packed upstream gradient, which the query side's throw-away dQ then overwrites)
  auto bwd_args = [&](const Layout& ll) {
    ua::BwdArgsV a{};
    a.Kp = wf + ll.Kp; a.Vp = wf + ll.Vp; a.KT = wf + ll.KT; a.Qp = wf + ll.Qp; a.dOp = wb + ll.dOp;
    a.lsrc = (const float*)(wf + ll.lsrc); a.ldest = (const float*)(wf + ll.ldest); a.lse2 = (const float*)(wf + ll.lse2);
    a.delta = (const float*)(wb + ll.delta); a.C = (const float*)(wf + ll.C);
    a.reach = (const int*)(wf + ll.reach); a.minkey = (const int*)(wf + ll.minkey);
    a.dKdacc = (float*)(wb + ll.dKdacc); a.dKrow = (float*)(wb + ll.dKrow); a.dVrow = (float*)(wb + ll.dVrow);
    a.dsrc_raw = (float*)(wb + ll.dsrc_raw); a.masked_nz = (const int*)(wb + ll.masked_nz);
    a.dS_st = wb + ll.dS_st; a.dG_st = wb + ll.dG_st; a.Bt = wf + ll.Bt;
    a.R = d.r; a.L = d.L; a.Lp = ll.Lp; a.c = 128; a.nch = 1; a.key_parts = ll.key_parts;
    // one query group: the production path has both kernels write the caller's gradients from their epilogues and runs no
    // finish pass, so the slots are timed that way, with throw-away outputs in the scratch (dv over the dV partial sums,
    // dk over the column-side partial sums, the gate gradients over the dsrc partial sums; "gates" read from the log-gates)
    if (d.r == 1 && !gates_f32(d)) {
      a.direct = 1; a.d_out = d.d;
      a.dv_out = wb + ll.dVrow; a.dk_out = wb + ll.dKdacc; a.dsrc_out = wb + ll.dsrc_raw; a.ddest_out = wb + ll.dsrc_raw;
      a.src_in = wf + ll.lsrc; a.dest_in = wf + ll.ldest;
    }
    return a;
  };
  if (d.r > 1 && !(d.flags & UA_FLAG_SHARE_GROUPS)) {
    if (int e = tune_slot(d, UA_TUNE_BWD_PARTS, s, [&](int v) {
          const Layout ll = make_layout(d, false, nth_divisor(d.r, v));
          if (ll.total > ws_bytes) return 1;               // this many parts need a larger workspace: not timed
          const ua::BwdArgsV a = bwd_args(ll);
          UA_HIP(ua::launch_bwd_keys(d.dtype, ll.D, a, ll.Zk, 0, s));
          return (int)UA_OK;
        })) return e;
    l = make_layout(d, false);
    if (ws_bytes < l.total) return fail(UA_EWORKSPACE, "the chosen number of parts needs %zu bytes of workspace", l.total);
    // leave tiles that match the chosen layout for the query side
    { const ua::BwdArgsV a = bwd_args(l); UA_HIP(ua::launch_bwd_keys(d.dtype, l.D, a, l.Zk, 0, s)); }
  }
  if (d.r == 1) {
    // both variants leave the same tiles; the slot is timed on the production code path (results straight to the caller's
    // tensors are replaced by the partial-sum buffers of the scratch)
    if (int e = tune_slot(d, UA_TUNE_BWD_KEYS, s, [&](int v) {
          ua::BwdArgsV a = bwd_args(l);
          a.keys_variant = v;
          UA_HIP(ua::launch_bwd_keys(d.dtype, l.D, a, l.Zk, 0, s));
          return (int)UA_OK;
        })) return e;
  }
  {
    const ua::BwdArgsV a = bwd_args(l);
    void* dqtmp = wb + l.dOp;
    if (int e = tune_slot(d, UA_TUNE_BWD_QUERIES, s, [&](int v) {
          UA_HIP(ua::launch_bwd_queries_from_tiles(l.D, a, dqtmp, d.d, l.Zq, s, v));
          return (int)UA_OK;
        })) return e;
  }
  return UA_OK;
}

}  // extern "C"
