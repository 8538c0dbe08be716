// Shared device helpers for the Universal Attention kernels (gfx950 / CDNA4, wave64).
//
// Tile convention used by every kernel in this library
// ----------------------------------------------------
// All pairwise quantities (key s, query t) are produced by v_mfma_f32_32x32x* as
// 32x32 blocks in the orientation  D[t, s] = X_t . Y_s^T :
//     A operand = 32 rows of X (query side),   lane (l%32) <-> row t, 8 k-values per lane
//     B operand = 32 rows of Y (key side),     lane (l%32) <-> col s, 8 k-values per lane
//     result    = f32x16 per lane: lane <-> key s = l%32, register v <-> query
//                 t = 8*(v/4) + 4*(l/32) + (v%4)
// so one lane owns ONE key and 16 of the 32 queries of the block.  The decay bias is
// a cumulative sum over queries for a fixed key, i.e. an in-lane scan plus one
// exchange with lane^32.  A result block re-enters the matrix core as a B operand
// (K index = t, N index = s) with no data movement: registers 8q..8q+7 are exactly
// the 8 k-values of k-chunk q under the k-permutation
//     t(q, hi, e) = 16q + 8*(e/4) + 4*hi + (e%4),
// provided the A operand of that product is fetched with the same permutation
// (two 4-element pieces of a [feature][t] tile).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ua {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __bf16 bf16;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kAMax = (float)(1.0 - 1e-6);      // upper clamp of the affinity (forward and backward)
constexpr float kPruneLog2 = 48.0f;               // softmax weights provably below 2^-48 are dropped when pruning
constexpr float kAMinBwd = 1e-6f;                 // lower clamp used only in the backward divisor
// marker stored in the log2-unit normaliser buffer for a (query, chunk) pair with no visible key
constexpr float kNoKeyLse = 3.0e38f;
constexpr float kNegFill = -1e12f;                // bias of a (key, query) pair with key > query
constexpr int kPad16 = 16;                        // bytes of padding per LDS row

// ---------------------------------------------------------------------------------
// MFMA operand fragment: 8 consecutive k-values of one row/column
// ---------------------------------------------------------------------------------
template <class T> struct alignas(16) Frag { T v[8]; };

__device__ __forceinline__ void mma(f32x16& c, const Frag<bf16>& a, const Frag<bf16>& b) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
// fp32: lane (row, hi) supplies k = hi of each 32x32x2 step; with 8 values per lane at
// k = 16q + 8*hi + e the e-th step contracts {16q+e, 16q+8+e}.
__device__ __forceinline__ void mma(f32x16& c, const Frag<float>& a, const Frag<float>& b) {
#pragma unroll
  for (int e = 0; e < 8; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[e], b.v[e], c, 0, 0, 0);
}

// 16x16 tiles (v_mfma_f32_16x16x32_bf16 / 16x16x4_f32): A lane l = row l%16, k-values 8*(l/16)..+7 of a
// 32-wide k-step; B lane l = column l%16, same k-values; result f32x4: lane <-> column l%16, register v <->
// row 4*(l/16) + v.  In the [t, s] orientation a lane therefore owns one key and 4 of the 16 queries of a tile.
typedef __attribute__((ext_vector_type(4))) float f32x4;
__device__ __forceinline__ void mma16(f32x4& c, const Frag<bf16>& a, const Frag<bf16>& b) {
  c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ void mma16(f32x4& c, const Frag<float>& a, const Frag<float>& b) {
#pragma unroll
  for (int e = 0; e < 8; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[e], b.v[e], c, 0, 0, 0);
}

template <class T> __device__ __forceinline__ T cvt(float x);
template <> __device__ __forceinline__ float cvt<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16 cvt<bf16>(float x) { return (bf16)x; }

// k-chunk q (0 or 1) of a result block as a B operand (see header comment)
template <class T> __device__ __forceinline__ Frag<T> as_operand(const f32x16& c, int q) {
  Frag<T> f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f.v[e] = cvt<T>(c[8 * q + e]);
  return f;
}

// two 16x16 result tiles covering 32 consecutive queries (tile i: t = 16i + 4g + v) as ONE B operand of a
// product contracting over those 32 queries: element e of lane group g is query 16*(e/4) + 4g + e%4
template <class T> __device__ __forceinline__ Frag<T> as_operand16(const f32x4& x0, const f32x4& x1) {
  Frag<T> f;
#pragma unroll
  for (int e = 0; e < 4; ++e) { f.v[e] = cvt<T>(x0[e]); f.v[4 + e] = cvt<T>(x1[e]); }
  return f;
}
// column of position t (inside its group of 32) in the transposed working tensors read by such products:
// the 8 k-values of lane group g are then 8 CONSECUTIVE elements starting at 8g
__host__ __device__ __forceinline__ constexpr int perm32(int t) { return (t & ~31) | (((t >> 2) & 3) << 3) | (((t >> 4) & 1) << 2) | (t & 3); }

// 8 contiguous elements (global or LDS); p must be 16-byte aligned
template <class T> __device__ __forceinline__ Frag<T> ld8(const T* p) {
  Frag<T> f;
  if constexpr (sizeof(T) == 2) {
    *reinterpret_cast<uint4*>(&f) = *reinterpret_cast<const uint4*>(p);
  } else {
    reinterpret_cast<uint4*>(&f)[0] = reinterpret_cast<const uint4*>(p)[0];
    reinterpret_cast<uint4*>(&f)[1] = reinterpret_cast<const uint4*>(p)[1];
  }
  return f;
}
// two 4-element pieces p[0..3], p[8..11] (the permuted-t A operand; p points at t = 16q + 4*hi)
template <class T> __device__ __forceinline__ Frag<T> ld4x2(const T* p) {
  Frag<T> f;
  if constexpr (sizeof(T) == 2) {
    reinterpret_cast<uint2*>(&f)[0] = *reinterpret_cast<const uint2*>(p);
    reinterpret_cast<uint2*>(&f)[1] = *reinterpret_cast<const uint2*>(p + 8);
  } else {
    reinterpret_cast<uint4*>(&f)[0] = *reinterpret_cast<const uint4*>(p);
    reinterpret_cast<uint4*>(&f)[1] = *reinterpret_cast<const uint4*>(p + 8);
  }
  return f;
}

// LDS row stride (elements) of a tile with `cols` payload columns
template <class T> __host__ __device__ constexpr int lds_stride(int cols) { return cols + kPad16 / (int)sizeof(T); }

// cooperative copy of a [rows][cols] tile, global (row stride gstride) -> LDS (row stride lstride)
template <class T>
__device__ __forceinline__ void stage_tile(T* __restrict__ lds, const T* __restrict__ g, int rows, int cols,
                                           long gstride, int lstride, int tid, int nthreads) {
  constexpr int V = 16 / (int)sizeof(T);
  const int vec_per_row = cols / V;
  for (int i = tid; i < rows * vec_per_row; i += nthreads) {
    int r = i / vec_per_row, c = (i - r * vec_per_row) * V;
    *reinterpret_cast<uint4*>(lds + r * lstride + c) = *reinterpret_cast<const uint4*>(g + (long)r * gstride + c);
  }
}

// ---------------------------------------------------------------------------------
// Asynchronous tile staging: global_load_lds_dwordx4 moves 16 bytes per lane from an arbitrary
// global address straight into LDS at (wave-uniform base + 16*lane), without passing through
// registers.  A padded LDS tile is therefore filled by NINSTR instructions of 1 KB each; the
// lanes that fall on padding slots re-read a payload chunk.  Each wave issues instructions
// w, w+NWAVES, ... and keeps the per-lane source offsets of its instructions in registers.
// ---------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// A [ROWS][COLS] operand tile in LDS, filled by asynchronous global->LDS loads in units of 16-byte chunks, and
// read as MFMA operands: lane l takes the 8 k-values of k-group 4q + l/16 of row 16*blk + l%16.
//
// CM = true (the fused kernels): k-group-major order, element (row, k-group kg, e) at ((kg*ROWS + row)*8 + e).
// The 16 lanes that ds_read_b128 serves together (one k-group, 16 consecutive rows) then read 256 CONTIGUOUS
// bytes.  Measured on this part: that costs clearly less than 16 chunks scattered over 16 rows, even when the
// scattered chunks are bank-conflict free.  The working tensors in HBM use the same order tile by tile
// (nat_off / tr_off below), so a tile is one contiguous block on both sides of the copy.
//
// CM = false (carry pre-pass of the chunked mode, which reads row-major working tensors): row-major rows;
// bf16 rows are unpadded with payload chunk c of row r stored at position c ^ swz(r) (bank-conflict free),
// fp32 rows keep one padding chunk.
template <class T, int ROWS, int COLS, bool CM = true> struct Tile;
template <class T, int ROWS, int COLS> struct Tile<T, ROWS, COLS, true> {
  static constexpr bool CONTIG = true;
  static constexpr int BYTES = ROWS * COLS * (int)sizeof(T);
  static constexpr int NINSTR = BYTES / 1024;
  static_assert(BYTES % 1024 == 0, "a tile is copied in units of 1 KB");
  __device__ __forceinline__ static int at(int blk, int col, int q, int g) { return ((4 * q + g) * ROWS + 16 * blk + col) * 8; }
};
template <class T, int ROWS, int COLS> struct Tile<T, ROWS, COLS, false> {
  static constexpr bool CONTIG = false;
  static constexpr bool SWZ = sizeof(T) == 2;
  static constexpr int STRIDE = SWZ ? COLS : COLS + kPad16 / (int)sizeof(T);   // elements per row
  static constexpr int CPR = STRIDE * (int)sizeof(T) / 16;             // 16-byte chunks per row
  static constexpr int CPP = COLS * (int)sizeof(T) / 16;               // payload chunks per row
  static constexpr int NINSTR = (ROWS * CPR + 63) / 64;
  static constexpr int BYTES = NINSTR * 1024;                          // LDS footprint
  static_assert(!SWZ || CPP == 4 || CPP == 8 || CPP == 16, "swizzle is defined for rows of 4, 8 or 16 chunks");
  __host__ __device__ static constexpr int swz(int r) { return CPP >= 8 ? (r & (CPP - 1)) : ((r >> 1) & (CPP - 1)); }
  __device__ __forceinline__ static int at(int blk, int col, int q, int g) {
    if constexpr (SWZ) {
      if constexpr (CPP >= 8) return (16 * blk + col) * STRIDE + (((4 * q + g) ^ (col & (CPP - 1))) << 3);
      else return (16 * blk + col) * STRIDE + (((g ^ (col >> 1)) & 3) << 3);          // 32-wide rows: q == 0
    } else {
      return (16 * blk + col) * STRIDE + 32 * q + 8 * g;
    }
  }
};
// element offsets inside the tiled working tensors of the fused kernels (Lp is a multiple of 32):
//   natural    [Z][Lp/32][D/8][32 positions][8 features]     element (position row, feature dd)
//   transposed [Z][Lp/32][4][D features][8 positions]         element (feature dd, column p of tile `tile`)
template <int D> __host__ __device__ __forceinline__ constexpr long nat_off(long z, int Lp, int row, int dd) {
  return ((z * (Lp >> 5) + (row >> 5)) * (D / 8) + (dd >> 3)) * 256 + ((row & 31) << 3) + (dd & 7);
}
template <int D> __host__ __device__ __forceinline__ constexpr long tr_off(long z, int Lp, int dd, int tile, int p) {
  return ((z * (Lp >> 5) + tile) * 4 + (p >> 3)) * (D * 8) + dd * 8 + (p & 7);
}

template <class TILE, int NWAVES> struct Stager {
  static constexpr int PER = (TILE::NINSTR + NWAVES - 1) / NWAVES;
  int off[PER];
  // gstride_bytes: distance between consecutive rows of the tile in global memory (row-major tiles only)
  __device__ __forceinline__ void init(int w, int lane, long gstride_bytes, int rows) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int n = (w + k * NWAVES) * 64 + lane;
      if constexpr (TILE::CONTIG) {
        off[k] = n * 16;
      } else {
        int row = n / TILE::CPR, c = n - row * TILE::CPR;
        row = row < rows ? row : rows - 1;
        if constexpr (TILE::SWZ) c ^= TILE::swz(row);
        else c = c < TILE::CPP ? c : TILE::CPP - 1;
        off[k] = (int)(row * gstride_bytes) + c * 16;
      }
    }
  }
  __device__ __forceinline__ void issue(void* lds_tile, const void* gtile, int w) const {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = w + k * NWAVES;
      if (TILE::NINSTR % NWAVES == 0 || i < TILE::NINSTR)
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const char*>(gtile) + off[k],
                                         (lds_ptr_t)(reinterpret_cast<char*>(lds_tile) + i * 1024), 16, 0, 0);
    }
  }
};
// Workgroups go to the 8 XCDs round-robin in dispatch order (x fastest).  This map hands every XCD whole heads
// (grid y), in the same x order, so that the tiles which all workgroups of a head stream hit in that XCD's L2
// instead of being fetched once per XCD.  Falls back to the identity when the head count is not a multiple of 8.
__device__ __forceinline__ void xcd_map(int& bx, int& by) {
  const int gx = gridDim.x, gy = gridDim.y;
  bx = blockIdx.x; by = blockIdx.y;
  if ((gy & 7) == 0) {
    const int n = bx + gx * by, slot = n >> 3;
    by = (n & 7) + 8 * (slot / gx);
    bx = slot % gx;
  }
}
// CUs of the current device (launchers choose between one and two work items per workgroup by it)
inline int device_cus() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    return n > 0 ? n : 256;
  }();
  return cus;
}

// The tensors of 1 KB tiles the 16-bit kernels exchange only hold the causal triangle, row after row:
//   bias tiles:      row = 32-query block tb, key tiles j = 0 .. 2 tb + 1          -> the row starts at tile tb (tb + 1)
//   gradient tiles:  row = 16-query tile tq,  32-key halves h = 0 .. tq / 2        -> the row starts at tile tri_grad_row(tq)
//                    (stand-alone bias op; the fused operator groups its gradient tiles, see grp_tile)
// Both triangles have nT32 (nT32 + 1) tiles per head (nT32 = Lp / 32); consumers read whole steps and may run a few tiles
// past the end of a row (into the next rows; past the last row of a head into the slack).
__host__ __device__ __forceinline__ constexpr long tri_bias_row(long tb) { return tb * (tb + 1); }
__host__ __device__ __forceinline__ constexpr long tri_grad_row(long tq) { return (tq >> 1) * ((tq >> 1) + 1) + ((tq & 1) ? (tq >> 1) + 1 : 0); }
__host__ __device__ __forceinline__ constexpr long tri_tiles(long nT32) { return nT32 * (nT32 + 1) + 8; }
// The score / decay gradient tiles of the fused operator are grouped by the workgroup that consumes them (k_bwd_queries3:
// 8 query tiles = 128 queries): group J = tq / 8 holds, for every 32-key half h = 0 .. 4 J + 3, the eight tiles of its
// query tiles next to one another, so that the eight waves of the consumer read 8 KB contiguous per tensor and step.
// (Halves beyond a query tile's own diagonal are never written nor used.)
__host__ __device__ __forceinline__ constexpr long grp_tile(long tq, long h) { return 16 * (tq >> 3) * ((tq >> 3) + 1) + 8 * h + (tq & 7); }
__host__ __device__ __forceinline__ constexpr long grp_tiles(long nT32) { return 16 * (nT32 >> 2) * ((nT32 >> 2) + 1) + 8; }

__device__ __forceinline__ void wait_async_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Column order of the transposed ([feature][position]) working tensors: inside every group of 16
// positions bits 2 and 3 are swapped, so that the 8 k-values a lane needs for the permuted-t operand
// (t = 16q + 8(e/4) + 4hi + e%4) are 8 CONSECUTIVE elements starting at 16q + 8hi.
__host__ __device__ __forceinline__ constexpr int perm16(int t) { return (t & ~12) | ((t & 4) << 1) | ((t & 8) >> 1); }

// ---------------------------------------------------------------------------------
// lane exchanges (DPP within rows of 16 lanes, v_permlane{16,32}_swap across rows)
// ---------------------------------------------------------------------------------
__device__ __forceinline__ float xor_lane(float v, int mask) { return __shfl_xor(v, mask, 64); }

template <int CTRL> __device__ __forceinline__ float dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppRor4 = 0x124, kDppRor8 = 0x128;
// values of lanes l and l^16 (resp. l^32): one of the two results is the lane's own value, the other its partner's
// (vector elements are copied to scalars before the bit cast: a bit cast applied to r[1] directly reads r[0])
__device__ __forceinline__ void swap16(float v, float& a, float& b) {
  auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, v), __builtin_bit_cast(unsigned, v), false, false);
  const unsigned r0 = r[0], r1 = r[1];
  a = __builtin_bit_cast(float, r0); b = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ void swap32(float v, float& a, float& b) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, v), __builtin_bit_cast(unsigned, v), false, false);
  const unsigned r0 = r[0], r1 = r[1];
  a = __builtin_bit_cast(float, r0); b = __builtin_bit_cast(float, r1);
}

// all-reduce over the 32 lanes that share l/32 (i.e. over the 32 keys of a block)
__device__ __forceinline__ float allmax32(float v) {
  v = fmaxf(v, dpp<kDppXor1>(v)); v = fmaxf(v, dpp<kDppXor2>(v)); v = fmaxf(v, dpp<kDppRor4>(v)); v = fmaxf(v, dpp<kDppRor8>(v));
  float a, b; swap16(v, a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float allsum32(float v) {
  v += dpp<kDppXor1>(v); v += dpp<kDppXor2>(v); v += dpp<kDppRor4>(v); v += dpp<kDppRor8>(v);
  float a, b; swap16(v, a, b);
  return a + b;
}

// query index inside a 32-block of register v of lane-half hi
__device__ __forceinline__ constexpr int t_of(int v, int hi) { return 8 * (v >> 2) + 4 * hi + (v & 3); }

// Inclusive prefix sum over the 32 queries of a block (per key = per lane pair l, l^32).
// On return x[v] = sum_{t' <= t(v)} x_in[t'];  returns the block total.
__device__ __forceinline__ float block_prefix(f32x16& x, int hi) {
  const float him = hi ? 1.f : 0.f;
  float run = 0.f;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    x[4 * g + 1] += x[4 * g]; x[4 * g + 2] += x[4 * g + 1]; x[4 * g + 3] += x[4 * g + 2];
    float lo, up;                       // group sums of the hi=0 lane and of the hi=1 lane of this key
    swap32(x[4 * g + 3], lo, up);
    const float off = __builtin_fmaf(him, lo, run);   // the hi=1 piece follows the hi=0 piece
#pragma unroll
    for (int e = 0; e < 4; ++e) x[4 * g + e] += off;
    run += lo + up;
  }
  return run;
}
// Inclusive suffix sum: x[v] = sum_{t' >= t(v)} x_in[t'];  returns the block total.
__device__ __forceinline__ float block_suffix(f32x16& x, int hi) {
  const float lom = hi ? 0.f : 1.f;
  float run = 0.f;
#pragma unroll
  for (int g = 3; g >= 0; --g) {
    x[4 * g + 2] += x[4 * g + 3]; x[4 * g + 1] += x[4 * g + 2]; x[4 * g] += x[4 * g + 1];
    float lo, up;
    swap32(x[4 * g], lo, up);
    const float off = __builtin_fmaf(lom, up, run);   // the hi=1 piece of group g lies after the hi=0 piece
#pragma unroll
    for (int e = 0; e < 4; ++e) x[4 * g + e] += off;
    run += lo + up;
  }
  return run;
}

// ---------------------------------------------------------------------------------
// Wave-private staging of a [32 keys][16 queries] tile: written from result-tile registers (lane = key, its 4
// consecutive queries: ONE store) and read back transposed as the A operand (row = query, k = the 32 keys) of a
// product contracting over those keys.  bf16 uses ds_read_tr16_b64 (two reads per operand); fp32 has no
// transposing read and keeps a [16 queries][32 keys] tile written element by element.
// ---------------------------------------------------------------------------------
typedef short v4s16 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s16* lds_v4s16_t;
template <class T> struct StageT;
template <> struct StageT<bf16> {
  static constexpr int BYTES = 1024;
  // 32-byte rows (one per key).  Two swizzles, both measured on the LDS pipe of this part (cycles per wave instruction,
  // eight waves issuing): the two 128-byte halves of odd 256-byte blocks are swapped, so that the transposing reads of
  // lane groups 0 and 1 (keys 0-3 and 8-11) fall on different banks (2.5 instead of 4.0); and the four 8-byte pieces of
  // a row are rotated by bits 2-3 of the row, without which the 8-byte stores of `put` (16 rows 32 bytes apart per lane
  // group) take 16 cycles instead of the 6.7 a store of 512 contiguous bytes takes.
  __device__ __forceinline__ static int addr(int row, int byte) {
    return (row * 32 + (byte ^ (((row >> 2) & 3) << 3))) ^ (((row >> 3) & 1) << 7);
  }
  // x[v] = value at (query 4g + v, key `row`)
  __device__ __forceinline__ static void put(char* base, int row, int g, const f32x4& x) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    bf16x4 p;
#pragma unroll
    for (int v = 0; v < 4; ++v) p[v] = (bf16)x[v];
    *reinterpret_cast<bf16x4*>(base + addr(row, 8 * g)) = p;
  }
  __device__ __forceinline__ static Frag<bf16> get(char* base, int lane) {
    const int i = lane & 15, G = lane >> 4;
    const v4s16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s16_t)(base + addr(8 * G + (i >> 2), 8 * (i & 3))));
    const v4s16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s16_t)(base + addr(8 * G + 4 + (i >> 2), 8 * (i & 3))));
    Frag<bf16> f;
    reinterpret_cast<v4s16*>(&f)[0] = lo;
    reinterpret_cast<v4s16*>(&f)[1] = hi;
    return f;
  }
};
template <> struct StageT<float> {
  static constexpr int STRIDE = 36, BYTES = 16 * STRIDE * 4;
  __device__ __forceinline__ static void put(char* base, int row, int g, const f32x4& x) {
    float* p = reinterpret_cast<float*>(base);
#pragma unroll
    for (int v = 0; v < 4; ++v) p[(4 * g + v) * STRIDE + row] = x[v];
  }
  __device__ __forceinline__ static Frag<float> get(char* base, int lane) {
    return ld8(reinterpret_cast<const float*>(base) + (lane & 15) * STRIDE + 8 * (lane >> 4));
  }
};

// ---- scans over the 32 queries of two 16x16 tiles (lane = key l%16, lane group g = l/16 holds t = 4g+v) ----
struct GroupMasks { float g1, g2, n1, n2; };    // g1 = g&1, g2 = g>>1 as floats, n* their complements
__device__ __forceinline__ GroupMasks group_masks(int lane) {
  const int g = lane >> 4;
  GroupMasks m;
  m.g1 = (g & 1) ? 1.f : 0.f; m.g2 = (g & 2) ? 1.f : 0.f; m.n1 = 1.f - m.g1; m.n2 = 1.f - m.g2;
  return m;
}
// s = per-lane sum of its 4 queries; before = sum over lane groups holding EARLIER queries, after = LATER ones,
// total = all four groups
__device__ __forceinline__ void group_scan(float s, const GroupMasks& m, float& before, float& after, float& total) {
  float a, b;
  swap16(s, a, b);                   // a: group with g&1 == 0 of the pair, b: the other
  float lo, up;
  swap32(a + b, lo, up);             // lo: groups {0,1}, up: groups {2,3}
  before = __builtin_fmaf(m.g1, a, m.g2 * lo);
  after = __builtin_fmaf(m.n1, b, m.n2 * up);
  total = lo + up;
}
// inclusive prefix over t = 0..31 (x0: queries 0..15, x1: 16..31); returns the total
__device__ __forceinline__ float prefix32(f32x4& x0, f32x4& x1, const GroupMasks& m) {
  x0[1] += x0[0]; x0[2] += x0[1]; x0[3] += x0[2];
  x1[1] += x1[0]; x1[2] += x1[1]; x1[3] += x1[2];
  float b0, a0, t0, b1, a1, t1;
  group_scan(x0[3], m, b0, a0, t0);
  group_scan(x1[3], m, b1, a1, t1);
  b1 += t0;
#pragma unroll
  for (int v = 0; v < 4; ++v) { x0[v] += b0; x1[v] += b1; }
  return t0 + t1;
}
// inclusive suffix: x[t] = sum_{t' >= t}; returns the total, t1 = total of the second tile (queries 16..31)
__device__ __forceinline__ float suffix32(f32x4& x0, f32x4& x1, const GroupMasks& m, float& t1) {
  x0[2] += x0[3]; x0[1] += x0[2]; x0[0] += x0[1];
  x1[2] += x1[3]; x1[1] += x1[2]; x1[0] += x1[1];
  float b0, a0, t0, b1, a1;
  group_scan(x0[0], m, b0, a0, t0);
  group_scan(x1[0], m, b1, a1, t1);
  a0 += t1;
#pragma unroll
  for (int v = 0; v < 4; ++v) { x0[v] += a0; x1[v] += a1; }
  return t0 + t1;
}
// ---- the same scans on the matrix core (16-bit operands) --------------------------------------------------------
// A running sum over the 32 queries of a block is a product with a triangular 0/1 matrix: with the block's values as
// the B operand of as_operand16 (k index = query, column = key) and the matrix as the A operand (row = query u inside
// tile i), the result tile has the layout of the input tiles and the carry enters as the accumulator.  Three matrix
// instructions (two tiles and the block total through a matrix of ones) replace about 40 vector instructions of the
// in-lane adds and lane exchanges above; the summands are rounded to the operand precision, the sums are float32.
// query position of element e of lane group g in an as_operand16 fragment
__device__ __forceinline__ constexpr int operand16_query(int g, int e) { return e < 4 ? 4 * g + e : 16 + 4 * g + (e - 4); }
struct ScanOps { Frag<bf16> tri[2], ones; };
// SUFFIX = false: row u of tile i sums the queries <= 16 i + u (inclusive prefix); true: the queries >= 16 i + u
template <bool SUFFIX> __device__ __forceinline__ ScanOps scan_operands(int lane) {
  const int u = lane & 15, g = lane >> 4;
  ScanOps o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int q = operand16_query(g, e);
#pragma unroll
    for (int i = 0; i < 2; ++i) o.tri[i].v[e] = (bf16)((SUFFIX ? q >= 16 * i + u : q <= 16 * i + u) ? 1.0f : 0.0f);
    o.ones.v[e] = (bf16)1.0f;
  }
  return o;
}
// y[i] = carry + running sums of the block (values in xb), carry += block total; every register of carry holds the same value
__device__ __forceinline__ void scan32_mma(const ScanOps& o, const Frag<bf16>& xb, f32x4& carry, f32x4 (&y)[2]) {
  y[0] = carry; y[1] = carry;
  mma16(y[0], o.tri[0], xb);
  mma16(y[1], o.tri[1], xb);
  mma16(carry, o.ones, xb);
}

// the 4 per-query values of lane group g inside a 16-query tile, from a float array indexed by query
__device__ __forceinline__ f32x4 load_t4(const float* __restrict__ p16, int g) {
  const float4 x = *reinterpret_cast<const float4*>(p16 + 4 * g);
  return (f32x4){x.x, x.y, x.z, x.w};
}
// all-reduce over the 16 lanes of a lane group (the 16 keys of a tile)
__device__ __forceinline__ float allmax16(float v) {
  v = fmaxf(v, dpp<kDppXor1>(v)); v = fmaxf(v, dpp<kDppXor2>(v)); v = fmaxf(v, dpp<kDppRor4>(v)); v = fmaxf(v, dpp<kDppRor8>(v));
  return v;
}
__device__ __forceinline__ float allsum16(float v) {
  v += dpp<kDppXor1>(v); v += dpp<kDppXor2>(v); v += dpp<kDppRor4>(v); v += dpp<kDppRor8>(v);
  return v;
}

// ---------------------------------------------------------------------------------
// affinity  A = relu(g)^(2/3) src_s^(1/3) dest_t^(1/3)  with g = k_s.k_t, evaluated as
// exp2(2/3 log2 g + lab), lab = (log2 src_s + log2 dest_t)/3   (log2(0) = -inf -> A = 0).
// ---------------------------------------------------------------------------------
__device__ __forceinline__ float log2_relu(float g) { return __builtin_amdgcn_logf(fmaxf(g, 0.f)); }
__device__ __forceinline__ float affinity(float lg, float lab) {
  return __builtin_amdgcn_exp2f(__builtin_fmaf(lg, 2.0f / 3.0f, lab));
}
// dG from the gradient dl of l = log2(1 - A) (log2 units folded by the caller):
//   dA = dl / (clamp(A, 1e-6, 1-1e-6) - 1), zero where A exceeds the clamp;  dG = dA (2/3) A / G
// as ONE reciprocal of (3/2)(clamp(A) - 1) G.  grelu = relu(G); where it is 0, A is 0 and so is the result.
__device__ __forceinline__ float decay_grad(float dl, float a, float grelu) {
  const float den15 = __builtin_fmaf(__builtin_amdgcn_fmed3f(a, kAMinBwd, kAMax), 1.5f, -1.5f);
  const float r = __builtin_amdgcn_rcpf(den15 * fmaxf(grelu, 1.0e-30f));
  return (a <= kAMax) ? (dl * a) * r : 0.f;
}
__device__ __forceinline__ float log2_one_minus(float a) { return __builtin_amdgcn_logf(1.0f - fminf(a, kAMax)); }
constexpr float kGatePad = -1.0e4f;   // log-gate of padded rows: makes their affinity exactly 0

// the 16 per-query values of a 32-block that a lane needs (t = 8g + 4hi + e), from a float[32]
__device__ __forceinline__ void load_t16(const float* __restrict__ p32, int hi, float (&out)[16]) {
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const float4 x = *reinterpret_cast<const float4*>(p32 + 8 * g + 4 * hi);
    out[4 * g] = x.x; out[4 * g + 1] = x.y; out[4 * g + 2] = x.z; out[4 * g + 3] = x.w;
  }
}

}  // namespace ua
