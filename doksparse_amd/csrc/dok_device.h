// Device-side building blocks shared by every kernel of libdokhip: integer types, the key
// hash, wave64 helpers and the kernel-argument form of a table.
//
// Execution model used throughout: one workgroup = 256 threads = 4 wave64s.  Each lane
// "owns" one batch row (its key, its result).  A 128-byte bucket is probed by a *group* of 16
// adjacent lanes, each lane loading one 8-byte word, so a wave inspects four buckets per
// load instruction and a bucket costs exactly one 128-byte line.  The group works through
// the rows its 16 lanes own one at a time; the row being served is broadcast with a lane
// shuffle, matches are found with a wave ballot, and the owning lane takes the result.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/dokhip.h"

typedef unsigned long long u64;
typedef long long i64;
typedef unsigned int u32;
typedef unsigned short u16;
typedef unsigned char u8;

#define DOK_TPB 256          // threads per workgroup
#define DOK_NONE32 0xffffffffu
// Most dimensions of a coordinate table whose keys are LINEARISED coordinates (one 8-byte key on
// the packed layout), and of the index spaces its fused indexing kernels take: their descriptor
// arrays have this many entries and their loops unroll to it.  Tables of more dimensions (up to
// DOK_MAX_DIMS), or of 2^63 elements and more, keep their coordinates as multi-word keys.
#define DOK_LIN_DIMS 8

// Batch kernels walk the rows in tiles of DOK_TPB; a workgroup takes tiles blockIdx.x,
// blockIdx.x + gridDim.x, ...  The host launches one workgroup per tile for kernels without
// counters and a fixed, machine-filling grid for kernels that count (fresh inserts, removals,
// hits): a wave then adds to the table header once, after its last tile, instead of once per
// tile - a million same-address atomics would otherwise serialise the whole kernel.
#define DOK_TILE_LOOP(n_rows)                                          \
  const i64 n_tiles_ = ((i64)(n_rows) + DOK_TPB - 1) / DOK_TPB;        \
  for (i64 tile_ = blockIdx.x; tile_ < n_tiles_; tile_ += gridDim.x)
#define DOK_TILE_ROW() (tile_ * DOK_TPB + (i64)threadIdx.x)

// Kernel-argument copy of dok_table_t plus what the host precomputes from it.
struct DevTable {
  u64 *buckets;
  i64 *header;
  u64 nb;                    // physical buckets
  u64 seed;
  int key_bytes;
  int value_bytes;
  int lin_ndim;
  int pad_;
  i64 lin_dims[DOK_MAX_DIMS];        // (a multi-word coordinate table uses all of them)
  i64 lin_strides[DOK_LIN_DIMS];   // row-major strides of lin_dims
  u64 lin_magic[DOK_LIN_DIMS];     // division by lin_strides[d] as multiply + shift (dok_div_stride);
  int lin_shift[DOK_LIN_DIMS];     // set by the host for strides above 1
};

// n / d for the stride d that (magic, shift) were made for (host: div_magic in dokhip.hip).  The
// round-up method of Granlund and Montgomery in its branch-free form: q = hi64(magic * n),
// n / d = (((n - q) >> 1) + q) >> shift.  A 64-bit divide costs some 150 instructions here, and
// the read-out of a coordinate table divides once per dimension and entry.
__device__ __forceinline__ u64 dok_div_stride(u64 n, u64 magic, int shift) {
  const u64 q = __umul64hi(magic, n);
  return (((n - q) >> 1) + q) >> shift;
}

// Kernel-argument form of dok_index_t (+ optional source-value view), for tensors and index spaces
// of up to MAXD dimensions.  The descriptor travels by value and the kernels read it with scalar
// loads, each of which a use waits for: with arrays for 8 dimensions (8 x 8 selector strides) a
// gather of a few thousand elements spends 4 of its 12 microseconds there, so tensors of up to 4
// dimensions indexed over up to 4 axes - nearly all - take the small form.
template <int MAXD>
struct DevIndexT {
  static constexpr int DIMS = MAXD;
  int ndim;
  int sel_ndim;
  i64 n_elems;
  i64 shape[MAXD];
  i64 estride[MAXD];               // C-contiguous strides of `shape`
  const i64 *sel[MAXD];            // NULL: the coordinate is sbase + offset itself
  i64 sbase[MAXD];
  i64 sstride[MAXD][MAXD];
  const void *src;
  i64 vstride[MAXD];
};
typedef DevIndexT<DOK_LIN_DIMS> DevIndex;
typedef DevIndexT<4> DevIndex4;

__device__ __forceinline__ u64 dok_fmix64(u64 x) {
  x ^= x >> 33; x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

// Multiply-high range reduction: maps a hash uniformly onto [0, nb) without division.  A table
// has fewer than 2^32 buckets, so the upper half of the hash and one 32 x 32 -> 64 bit multiply do.
__device__ __forceinline__ u32 dok_reduce(u64 h, u64 nb) { return (u32)(((h >> 32) * (u64)(u32)nb) >> 32); }

__device__ __forceinline__ u64 dok_ballot(bool p) { return __ballot(p); }

__device__ __forceinline__ u64 dok_shfl64(u64 v, int src) { return __shfl(v, src, 64); }
__device__ __forceinline__ u32 dok_shfl32(u32 v, int src) { return __shfl(v, src, 64); }

// Loads that must observe what other workgroups (possibly on another XCD, behind another L2)
// wrote earlier in the same kernel.
__device__ __forceinline__ u64 dok_load_coherent(const u64 *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void dok_store_coherent(u64 *p, u64 v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One add per wave instead of one per lane.
__device__ __forceinline__ void dok_wave_add(i64 *counter, bool flag, i64 sign = 1) {
  u64 m = dok_ballot(flag);
  if (m != 0 && (threadIdx.x & 63) == 0) atomicAdd((u64 *)counter, (u64)(sign * (i64)__popcll(m)));
}
__device__ __forceinline__ void dok_wave_add_n(i64 *counter, int v) {
  // sum of a small per-lane int (either sign) over the wave, one atomic per wave
  #pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  if (v != 0 && (threadIdx.x & 63) == 0) atomicAdd((u64 *)counter, (u64)(i64)v);
}

// The same over a whole workgroup: one atomic per workgroup and counter instead of one per wave.
// The adds of a kernel all go to the same few header words and are served one after the other
// (about 10 ns each), which a small batch would otherwise wait for longer than for its rows.
// Every thread of the workgroup must get here (the function holds barriers: no call after a
// per-wave early return).
template <int N>
__device__ __forceinline__ void dok_block_add(i64 *const (&counter)[N], const int (&value)[N]) {
  __shared__ int part[16][N];
  const int wave = threadIdx.x >> 6, n_waves = (blockDim.x + 63) >> 6;
  #pragma unroll
  for (int k = 0; k < N; k++) {
    int v = value[k];
    #pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if ((threadIdx.x & 63) == 0) part[wave][k] = v;
  }
  __syncthreads();
  if (threadIdx.x < N) {
    int sum = 0;
    for (int w = 0; w < n_waves; w++) sum += part[w][threadIdx.x];
    if (sum != 0) atomicAdd((u64 *)counter[threadIdx.x], (u64)(i64)sum);
  }
  __syncthreads();           // `part` may be written again by a later call
}
__device__ __forceinline__ void dok_block_add1(i64 *c0, int v0) {
  i64 *const c[1] = {c0}; const int v[1] = {v0};
  dok_block_add<1>(c, v);
}
__device__ __forceinline__ void dok_block_add2(i64 *c0, int v0, i64 *c1, int v1) {
  i64 *const c[2] = {c0, c1}; const int v[2] = {v0, v1};
  dok_block_add<2>(c, v);
}
__device__ __forceinline__ void dok_block_add3(i64 *c0, int v0, i64 *c1, int v1, i64 *c2, int v2) {
  i64 *const c[3] = {c0, c1, c2}; const int v[3] = {v0, v1, v2};
  dok_block_add<3>(c, v);
}

// Zero `words` 8-byte words (a multiple of 4) and the table header.
__global__ __launch_bounds__(DOK_TPB) void dok_fill_kernel(u64 *p, i64 words, i64 *header) {
  const i64 i = ((i64)blockIdx.x * DOK_TPB + threadIdx.x) * 4;
  if (i + 3 < words) {
    ulonglong2 z; z.x = 0; z.y = 0;
    ((ulonglong2 *)(p + i))[0] = z;
    ((ulonglong2 *)(p + i))[1] = z;
  }
  if (blockIdx.x == 0 && threadIdx.x < DOK_HEADER_WORDS) header[threadIdx.x] = 0;
}

// Measurement aid: every group of LANES adjacent lanes loads pseudo-random, naturally aligned
// granules of LANES * 8 bytes of the bucket array (8 bytes per lane, eight independent loads in
// flight) and folds what it read into one word per granule.  With 16 lanes this is the access
// pattern of a lookup with the probing taken out - one 128-byte bucket line per row - so its rate is
// the practical ceiling of the lookup kernels on a given table; 8 and 4 lanes answer what a probe
// of half or a quarter of a line would cost instead.
template <int LANES>
__global__ __launch_bounds__(DOK_TPB) void dok_line_gather_kernel(const u64 *__restrict__ lines, u64 n_granules,
                                                                  i64 n, u64 seed, u32 *__restrict__ out) {
  const int l = threadIdx.x & (LANES - 1);
  const i64 group = ((i64)blockIdx.x * DOK_TPB + threadIdx.x) / LANES;
  const i64 n_groups = ((i64)gridDim.x * DOK_TPB) / LANES;
  for (i64 base = group * 8; base < n; base += n_groups * 8) {
    u64 v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const u64 gi = dok_reduce(dok_fmix64((u64)(base + u) ^ seed), n_granules);
      v[u] = lines[gi * LANES + l];
    }
#pragma unroll
    for (int u = 0; u < 8; u++) {
      u32 x = (u32)v[u] ^ (u32)(v[u] >> 32);
#pragma unroll
      for (int o = LANES / 2; o > 0; o >>= 1) x ^= __shfl_xor(x, o, LANES);
      if (l == 0 && base + u < n) out[base + u] = x;
    }
  }
}

// Row-major linearisation of an int64 coordinate row; false if any coordinate is outside
// [0, dim).  Negative coordinates are not wrapped (the reference does not wrap them either).
// The loops run to the compile-time maximum under a uniform guard, so that they unroll; the
// coordinates are loaded first and used afterwards, so that the loads of a row overlap.  (The
// streaming kernels of the bulk path, where the loads of many rows must overlap, have a loader
// of their own.)
__device__ __forceinline__ bool dok_linearise(const DevTable &t, const i64 *row, u64 &key) {
  i64 c[DOK_LIN_DIMS];
  #pragma unroll
  for (int d = 0; d < DOK_LIN_DIMS; d++) {
    c[d] = 0;
    if (d < t.lin_ndim) c[d] = row[d];               // loads only: they overlap
  }
  bool ok = true;
  u64 k = 0;
  #pragma unroll
  for (int d = 0; d < DOK_LIN_DIMS; d++) {
    if (d < t.lin_ndim) {
      ok = ok && ((u64)c[d] < (u64)t.lin_dims[d]);
      k += (u64)c[d] * (u64)t.lin_strides[d];
    }
  }
  key = k;
  return ok;
}

// Key formats of the batch buffers handed to the packed-layout kernels.  The format is a
// template argument so that kernels of plain tables never touch (or hold in scalar registers)
// the sixteen dimension / stride words of the descriptor.
#define DOK_KF_RAW  0   // key_bytes (1, 2, 4, 8) raw bytes per row, zero-extended to 8
#define DOK_KF_ROWS 1   // coordinate table, row-major:    keys[i * ndim + d]
#define DOK_KF_COLS 2   // coordinate table, column-major: keys[d * n + i]   (COO "indices")
#define DOK_KF_U64  3   // keys already in table form: one 8-byte word per row, whatever key_bytes is
#define DOK_KF_TABLE 4  // (bulk rehash only) the "batch" is another packed table: row i is word i of
                        // its bucket array; the words that are live key slots are the rows
#define DOK_KF_LIN  5   // (bulk path only) linearised coordinates, one 8-byte word per row; all ones =
                        // a row whose coordinates lie outside the table

// Key of batch row i (of n) as an 8-byte integer; false if a coordinate is out of range.
template <int KF>
__device__ __forceinline__ bool dok_load_key8(const DevTable &t, const void *keys, i64 i, i64 n, u64 &key) {
  if (KF == DOK_KF_ROWS) return dok_linearise(t, (const i64 *)keys + i * t.lin_ndim, key);
  if (KF == DOK_KF_U64) { key = ((const u64 *)keys)[i]; return true; }
  if (KF == DOK_KF_COLS) {
    i64 c[DOK_LIN_DIMS];
    #pragma unroll
    for (int d = 0; d < DOK_LIN_DIMS; d++) {
      c[d] = 0;
      if (d < t.lin_ndim) c[d] = ((const i64 *)keys)[(i64)d * n + i];
    }
    bool ok = true;
    u64 k = 0;
    #pragma unroll
    for (int d = 0; d < DOK_LIN_DIMS; d++) {
      if (d < t.lin_ndim) {
        ok = ok && ((u64)c[d] < (u64)t.lin_dims[d]);
        k += (u64)c[d] * (u64)t.lin_strides[d];
      }
    }
    key = k;
    return ok;
  }
  switch (t.key_bytes) {
    case 8: key = ((const u64 *)keys)[i]; break;
    case 4: key = ((const u32 *)keys)[i]; break;
    case 2: key = ((const u16 *)keys)[i]; break;
    default: key = ((const u8 *)keys)[i]; break;
  }
  return true;
}

// The inverse, for the read-out: row i of an output holding `cap` rows.
template <int KF>
__device__ __forceinline__ void dok_store_key8(const DevTable &t, void *keys_out, i64 i, i64 cap, u64 key) {
  if (KF != DOK_KF_RAW) {
    u64 rem = key;
    for (int d = 0; d < t.lin_ndim; d++) {
      const u64 s = (u64)t.lin_strides[d];
      const u64 c = s == 1 ? rem : dok_div_stride(rem, t.lin_magic[d], t.lin_shift[d]);
      rem -= c * s;
      if (KF == DOK_KF_ROWS) ((i64 *)keys_out)[i * t.lin_ndim + d] = (i64)c;
      else ((i64 *)keys_out)[(i64)d * cap + i] = (i64)c;
    }
    return;
  }
  switch (t.key_bytes) {
    case 8: ((u64 *)keys_out)[i] = key; break;
    case 4: ((u32 *)keys_out)[i] = (u32)key; break;
    case 2: ((u16 *)keys_out)[i] = (u16)key; break;
    default: ((u8 *)keys_out)[i] = (u8)key; break;
  }
}

template <int V> struct ValT;
template <> struct ValT<1> { typedef u8 type; };
template <> struct ValT<2> { typedef u16 type; };
template <> struct ValT<4> { typedef u32 type; };
template <> struct ValT<8> { typedef u64 type; };

template <int V> __device__ __forceinline__ u64 dok_load_val(const void *values, i64 i) {
  return (u64)((const typename ValT<V>::type *)values)[i];
}
template <int V> __device__ __forceinline__ void dok_store_val(void *values, i64 i, u64 v) {
  ((typename ValT<V>::type *)values)[i] = (typename ValT<V>::type)v;
}

// Coordinate selected by index vector idx[] of the broadcast index space along every tensor
// dimension, linearised: read each selector through its strides (stride 0 = broadcast axis).
// `voff` receives the element offset into the source view.  Loops run to the compile-time
// maximum with uniform guards so that idx[] stays in registers; the host zeroes the strides of
// unused axes.
template <class IX>
__device__ __forceinline__ bool dok_gather_at(const DevTable &t, const IX &ix,
                                              const i64 (&idx)[IX::DIMS], u64 &key, i64 &voff) {
  constexpr int DIMS = IX::DIMS;
  // The small form runs its stride loops without guards: the unused strides are zero, and nothing
  // then stands between the descriptor's scalar loads and the head of the kernel.
  constexpr bool GUARD = DIMS > 4;
  // first every dimension's selector is read, then the values are used: a use next to its load
  // would make the loads of the dimensions wait for one another
  i64 g[DIMS];
  #pragma unroll
  for (int d = 0; d < DIMS; d++) {
    g[d] = 0;
    if (!GUARD || d < ix.ndim) {
      i64 off = 0;
      #pragma unroll
      for (int j = 0; j < DIMS; j++)
        if (!GUARD || j < ix.sel_ndim) off += idx[j] * ix.sstride[d][j];
      const i64 *sp = ix.sel[d];
      g[d] = off;
      if (sp) g[d] = sp[off];
    }
  }
  bool ok = true;
  u64 k = 0;
  #pragma unroll
  for (int d = 0; d < DIMS; d++) {
    if (d < ix.ndim) {
      const i64 c = ix.sbase[d] + g[d];
      ok = ok && ((u64)c < (u64)t.lin_dims[d]);
      k += (u64)c * (u64)t.lin_strides[d];
    }
  }
  i64 vo = 0;
  #pragma unroll
  for (int j = 0; j < DIMS; j++)
    if (!GUARD || j < ix.sel_ndim) vo += idx[j] * ix.vstride[j];
  voff = vo;
  key = k;
  return ok;
}

// The same for element e (row-major offset) of the index space: unravel e over `shape` first.
template <class IX>
__device__ __forceinline__ bool dok_gather_key(const DevTable &t, const IX &ix, i64 e,
                                               u64 &key, i64 &voff) {
  constexpr int DIMS = IX::DIMS;
  constexpr bool GUARD = DIMS > 4;           // (the divisors of unused axes are 1)
  i64 idx[DIMS];
  if (ix.n_elems <= 0x7fffffffLL) {
    u32 rem = (u32)e;
    #pragma unroll
    for (int j = 0; j < DIMS; j++) {
      idx[j] = 0;
      if (!GUARD || j < ix.sel_ndim) {
        u32 s = (u32)ix.estride[j];
        u32 q = rem / s;
        rem -= q * s;
        idx[j] = q;
      }
    }
  } else {
    u64 rem = (u64)e;
    #pragma unroll
    for (int j = 0; j < DIMS; j++) {
      idx[j] = 0;
      if (j < ix.sel_ndim) {
        u64 s = (u64)ix.estride[j];
        u64 q = rem / s;
        rem -= q * s;
        idx[j] = (i64)q;
      }
    }
  }
  return dok_gather_at(t, ix, idx, key, voff);
}
