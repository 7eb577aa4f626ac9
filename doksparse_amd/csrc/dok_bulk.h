// Bulk insert for the packed layout: partition the batch by table range, then merge each range
// in LDS.
//
// The ordinary insert (p8_set_kernel) pays one returning 64-bit atomic in HBM per row, and the
// rate of those atomics - not memory bandwidth - is what bounds it.  When a batch holds more
// than about one row per bucket of the table it is cheaper to stream the whole table through
// the LDS once:
//
//   1. the table is cut into ranges of DOK_BULK_R consecutive buckets; the range of a row is
//      (home bucket) / DOK_BULK_R;
//   2. two scatter passes (first by range / 256 (range / 1024 for very large tables), then by
//      range inside each first-level bin) move every (key, value) row next to the other rows of
//      its range.  Nothing is counted beforehand: every bin owns a region of fixed capacity in the
//      pass's output - the rows a uniform hash sends there on average plus six (first level) resp.
//      five (ranges) standard deviations - and a workgroup that has staged a tile of rows in LDS, ordered by bin,
//      reserves the run of each bin with ONE atomic add on that bin's fill counter (a few hundred
//      atomics per tile of thousands of rows, issued while the tile is being staged, so their
//      latency is hidden).  Rows that find their bin's region full (batches with very many
//      equal keys) go to a spill list that the ordinary insert works through at the end;
//   3. one workgroup per range copies the range's buckets into LDS, places the range's rows
//      there and streams the buckets back (a table that holds nothing yet is not read: the
//      copy starts empty, and the clear of the table is saved as well);
//   4. rows whose chain runs out of a workgroup's block of ranges are placed in the next block's
//      first ranges by a small follow-up kernel, once those ranges are final;
//   5. the handful of rows left (overflow of the per-range lists, keys that may sit at far
//      displacements) are handed, packed, to the ordinary insert, which runs last.
//
// The two levels address 1024 x 1024 ranges = 2^28 buckets.  A larger table is worked through in
// windows of that many buckets, steps 2 to 5 once per window: the first scatter reads the whole
// batch each time and keeps the rows whose range lies in the window.  The rows that run out of a
// window's last range are placed by step 5's ordinary insert, in the next window's buckets before
// that window's merge - so the merge of a table of several windows always reads its ranges.
//
// Every step is exact for any input: a bin that receives more rows than its region holds spills
// the surplus, and a batch whose rows all fall into one range merely degrades to step 5's
// ordinary insert.
#pragma once
#include "dok_packed8.h"

#define DOK_BULK_RLOG 8                     // log2 of the buckets per range: 256 buckets = 32 KiB
#define DOK_BULK_R (1 << DOK_BULK_RLOG)
#define DOK_BULK_SUBLOG 8                   // log2 of the ranges per first-level bin ...
#define DOK_BULK_SUBLOG_WIDE 10             // ... and for tables of more than 1024 << 8 ranges
#define DOK_BULK_MAXBIG 1024                // first-level bins at most
#define DOK_BULK_WINDOW ((u64)DOK_BULK_MAXBIG << DOK_BULK_SUBLOG_WIDE)   // ranges one run of the passes takes: 2^28 buckets
// Threads per scatter workgroup.  One workgroup per CU with the large tiles either way (a tile
// fills the LDS); 16 waves instead of 8 make the second pass, whose workgroups take one or two
// tiles each, 12 % faster and the first pass over plain keys 3 %; the first pass over coordinate
// rows or over a table's buckets (more registers per row, more loads per row) loses with them.
#define DOK_BULK_TPB_FEW 512
#define DOK_BULK_TPB_MANY 1024
constexpr int bulk_tpb(int level, int key_format, int coord_dims) {
  return level == 1 && (coord_dims > 0 || key_format == DOK_KF_TABLE) ? DOK_BULK_TPB_FEW : DOK_BULK_TPB_MANY;
}
// Rows per scatter tile.  A tile is staged in LDS whole (8 + V + 2 bytes per row), and the larger
// it is, the longer the runs of rows that leave for one bin: for 8-byte keys with 4-byte values
// one workgroup per CU with a tile that nearly fills the LDS beats two with half the tile
// (scatter of 64M rows: 0.57 -> 0.47 ms).  All sizes are measured choices.
#define DOK_BULK_T 8192                     // first pass (up to 1024 bins: 12 KiB of bin arrays)
#define DOK_BULK_T1V8 6144                  //   ... with 8-byte values
#define DOK_BULK_T2 10240                   // second pass
#define DOK_BULK_T2S 4096                   //   ... with 1- and 2-byte values when a workgroup's stretch is short
                                            //   (three workgroups per CU with small tiles are faster then)
#define DOK_BULK_T2S_BELOW 16384            //   ... which is: fewer rows than this per workgroup
#define DOK_BULK_T2V8 8192                  //   ... with 8-byte values
#define DOK_BULK_CTPB 1024                  // threads per workgroup of the count kernels: they only stream
                                            // keys, and the bytes in flight per CU bound their rate
#define DOK_BULK_GRID 1024                  // most workgroups the first pass and the merge are given

// Device view of the caller's workspace.
struct BulkWs {
  u64 *keysA, *keysB;       // [n] each: rows after the first / second scatter
  void *valsA, *valsB;      // [n] values of value_bytes each
  u32 *big_cnt;             // [n_big]             rows reserved so far in first-level bin b, whose region is
                            //                     keysA[b * big_cap, (b + 1) * big_cap)
  u32 *part_cnt;            // [n_big << sublog]   the same for range p: keysB[p * part_cap, (p + 1) * part_cap)
  u64 *spill_keys;          // [spill_cap] rows that found their bin's region full
  void *spill_vals;
  u32 *spill_cnt;           // [1]
  u32 *def_cnt;             // [GRID] rows each merge workgroup handed to the ordinary insert
  u32 *meta_cnt;            // [GRID] displacement marks each merge workgroup left to be applied
  u32 *edge_cnt;            // [GRID] rows each merge workgroup could not place in the last range of its block
  u32 n_big, n_part;        // first-level bins and ranges OF THE CURRENT WINDOW (see range_base)
  u32 range_base;           // A table of more than 2^28 buckets is worked through in windows of
                            // DOK_BULK_WINDOW ranges, one run of the passes per window: range_base is the
                            // window's first range; range numbers inside the passes are relative to it,
  u32 first_window;         // and the rows outside the window are skipped by the first scatter.  first_window:
                            // this run also looks after what belongs to no range (side-slot keys, row counts)
  u32 sublog;               // log2 of the ranges per first-level bin
  u32 g1;                   // workgroups of the first pass (a multiple of 64, at most DOK_BULK_GRID)
  u32 ch;                   // stretches (workgroups) per first-level bin in the second pass
  u32 big_cap, part_cap;    // rows a first-level bin's / a range's region holds
  u32 spill_cap;
  i64 share;                // rows per workgroup in the first pass
};

// The rows of first-level bin b / of range p that the passes have delivered.
__device__ __forceinline__ u32 bulk_big_n(const BulkWs &ws, u32 b) {
  const u32 c = ws.big_cnt[b];
  return c < ws.big_cap ? c : ws.big_cap;
}
__device__ __forceinline__ u32 bulk_part_n(const BulkWs &ws, u32 p) {
  const u32 c = ws.part_cnt[p];
  return c < ws.part_cap ? c : ws.part_cap;
}

// Exclusive prefix sum of one value per thread over the workgroup (blockDim.x a multiple of 64,
// at most 1024).  `wsum` is LDS scratch of 16 words.  Ends with a barrier.
__device__ __forceinline__ u32 bulk_block_scan(u32 v, u32 *wsum, u32 &total) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  u32 inc = v;
  #pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const u32 up = __shfl_up(inc, o, 64);
    if (lane >= o) inc += up;
  }
  if (lane == 63) wsum[wv] = inc;
  __syncthreads();
  u32 pre = 0, tot = 0;
  for (int k = 0; k < nw; k++) {
    const u32 s = wsum[k];
    if (k < wv) pre += s;
    tot += s;
  }
  total = tot;
  __syncthreads();
  return pre + inc - v;
}

__device__ __forceinline__ u32 bulk_range_of(u64 key, const DevTable &t) {
  return p8_home(key ^ DOK_P8_XOR, t) >> DOK_BULK_RLOG;
}

// Row i of the batch, in two steps: bulk_fetch only loads, bulk_finish turns what was loaded into
// the key.  A kernel issues the fetches of all the rows it holds before it finishes any of them,
// so that their loads are in flight together (a load is not moved across the branch that guards
// its row, and a use inside that branch would wait for it right there).
// ND: the number of dimensions of a coordinate source - a compile-time constant, so that no
// branch separates the loads of one row either; 0 for the other sources.
template <int KF, int ND> struct BulkRaw { u64 w[ND > 0 ? ND : 1]; };

template <int KF, int ND>
__device__ __forceinline__ void bulk_fetch(const DevTable &t, const void *keys, i64 i, i64 n, BulkRaw<KF, ND> &r) {
  if constexpr (KF == DOK_KF_ROWS) {
    #pragma unroll
    for (int d = 0; d < ND; d++) r.w[d] = ((const u64 *)keys)[i * ND + d];
  } else if constexpr (KF == DOK_KF_COLS) {
    #pragma unroll
    for (int d = 0; d < ND; d++) r.w[d] = ((const u64 *)keys)[(i64)d * n + i];
  } else if constexpr (KF == DOK_KF_TABLE) {
    // word i of the source table's buckets; only the first S words of a bucket are key slots
    r.w[0] = 0;
    if ((int)(i & 15) < 120 / (8 + t.value_bytes)) r.w[0] = ((const u64 *)keys)[i];
  } else if constexpr (KF == DOK_KF_RAW) {
    dok_load_key8<DOK_KF_RAW>(t, keys, i, n, r.w[0]);
  } else {
    r.w[0] = ((const u64 *)keys)[i];                  // DOK_KF_U64, DOK_KF_LIN
  }
}

// Returns 1 = row, 0 = no row here, 2 = the row's coordinates lie outside the table.
template <int KF, int ND>
__device__ __forceinline__ int bulk_finish(const DevTable &t, const BulkRaw<KF, ND> &r, u64 &key) {
  if constexpr (KF == DOK_KF_ROWS || KF == DOK_KF_COLS) {
    bool ok = true;
    u64 k = 0;
    #pragma unroll
    for (int d = 0; d < ND; d++) {
      ok &= r.w[d] < (u64)t.lin_dims[d];
      k += r.w[d] * (u64)t.lin_strides[d];
    }
    key = k;
    return ok ? 1 : 2;
  } else if constexpr (KF == DOK_KF_TABLE) {
    key = r.w[0] ^ DOK_P8_XOR;                        // EMPTY, TOMB and the words that are no slots: no row
    return r.w[0] >= 2 ? 1 : 0;
  } else if constexpr (KF == DOK_KF_LIN) {
    key = r.w[0];
    return key == ~0ULL ? 2 : 1;
  } else {
    key = r.w[0];
    return 1;
  }
}

// The stretch of rows that workgroup `w` of a pass owns.
__device__ __forceinline__ void bulk_stretch1(const BulkWs &ws, i64 n, u32 w, i64 &lo, i64 &hi) {
  lo = (i64)w * ws.share;
  hi = lo + ws.share;
  if (hi > n) hi = n;
  if (lo > hi) lo = hi;
}
__device__ __forceinline__ void bulk_stretch2(const BulkWs &ws, u32 b, u32 c, i64 &lo, i64 &hi) {
  const i64 lo0 = (i64)b * ws.big_cap, hi0 = lo0 + bulk_big_n(ws, b);
  const i64 len = (hi0 - lo0 + ws.ch - 1) / ws.ch;
  lo = lo0 + (i64)c * len;
  hi = lo + len;
  if (hi > hi0) hi = hi0;
  if (lo > hi) lo = hi;
}

// ---- set-up: every fill counter to zero (and, for a build, the table header) ------------------------
__global__ __launch_bounds__(DOK_TPB) void bulk_init_kernel(BulkWs ws, i64 *header) {
  const u32 n_parts = ws.n_big << ws.sublog;
  for (u32 i = blockIdx.x * DOK_TPB + threadIdx.x; i < n_parts; i += gridDim.x * DOK_TPB) ws.part_cnt[i] = 0;
  if (blockIdx.x == 0) {
    for (u32 i = threadIdx.x; i < ws.n_big; i += DOK_TPB) ws.big_cnt[i] = 0;
    if (threadIdx.x == 0) ws.spill_cnt[0] = 0;
    if (header && threadIdx.x < DOK_HEADER_WORDS) header[threadIdx.x] = 0;
  }
}

// ---- coordinate rows of three and more dimensions are linearised once, into keysB (free until the
// second scatter), so that the first scatter reads 8 bytes per row and holds one word per row in
// registers instead of the coordinates; all ones marks a row outside the table's coordinate space.
template <int KF, int ND>
__global__ __launch_bounds__(DOK_BULK_CTPB) void bulk_linearise_kernel(DevTable t, const void *__restrict__ keys, i64 n,
                                                                      BulkWs ws) {
  constexpr int U = ND <= 4 ? 4 : 2;
  i64 lo, hi;
  bulk_stretch1(ws, n, blockIdx.x, lo, hi);
  for (i64 i0 = lo + threadIdx.x; i0 < hi; i0 += U * DOK_BULK_CTPB) {
    BulkRaw<KF, ND> raw[U] = {};
    #pragma unroll
    for (int u = 0; u < U; u++) {
      const i64 i = i0 + u * DOK_BULK_CTPB;
      if (i < hi) bulk_fetch<KF, ND>(t, keys, i, n, raw[u]);
    }
    #pragma unroll
    for (int u = 0; u < U; u++) {
      const i64 i = i0 + u * DOK_BULK_CTPB;
      u64 key = 0;
      if (i < hi) ws.keysB[i] = bulk_finish<KF, ND>(t, raw[u], key) == 1 ? key : ~0ULL;
    }
  }
}

// ---- scatter: LEVEL 1 moves the caller's rows into first-level bins (keysA/valsA), LEVEL 2 moves
// the rows of each first-level bin into their ranges (keysB/valsB) ---------------------------------
// REMOVE: the rows are keys to be removed - no values travel with them, a key that lives in a side
// slot of the header is removed on the spot, rows outside the coordinate space are dropped silently.
template <int V, int KF, int LEVEL, int SL = DOK_BULK_SUBLOG, int ND = 0, bool SMALLT = false, bool REMOVE = false>
__global__ __launch_bounds__(bulk_tpb(LEVEL, KF, ND)) void bulk_scatter_kernel(DevTable t, const void *__restrict__ keys_in,
                                                                    const void *__restrict__ vals_in, i64 n, BulkWs ws) {
  typedef typename ValT<V>::type VT;
  constexpr int T = LEVEL == 1 ? (V == 8 ? DOK_BULK_T1V8 : DOK_BULK_T)
                               : (V == 8 ? DOK_BULK_T2V8 : SMALLT ? DOK_BULK_T2S : DOK_BULK_T2);
  constexpr int TPB = bulk_tpb(LEVEL, KF, ND);
  static_assert(T % TPB == 0, "every thread stages the same number of rows");
  constexpr int RPT = T / TPB;
  constexpr int NB = LEVEL == 1 ? DOK_BULK_MAXBIG : (1 << SL);
  constexpr int BPT = NB >= TPB ? NB / TPB : 1;   // consecutive bins per thread
  __shared__ u32 cnt[NB], off[NB], gbase[NB];
  __shared__ u16 room[NB];                  // rows of a bin's run that its region still holds (a tile has < 65535 rows)
  __shared__ u64 skeys[T];
  __shared__ VT svals[T];
  __shared__ u16 sbins[T];                  // bin of every staged row (saves a second hash)
  __shared__ u32 wsum[16];
  const int tid = threadIdx.x;
  int n_fresh = 0, n_oob = 0;

  // this workgroup's stretch of the input; the fill counters and the region size of its output bins
  i64 lo0, hi0;
  const void *kin = keys_in, *vin = vals_in;
  u64 *out_keys;
  VT *out_vals;
  u32 *fill;                                // fill[bin]: rows reserved so far in the bin's region
  u32 first_bin, n_bins, cap;               // (global number of this workgroup's bin 0; bins in use; region size)
  if (LEVEL == 1) {
    bulk_stretch1(ws, n, blockIdx.x, lo0, hi0);
    out_keys = ws.keysA;
    out_vals = (VT *)ws.valsA;
    fill = ws.big_cnt; first_bin = 0; n_bins = ws.n_big; cap = ws.big_cap;
  } else {
    const u32 b = blockIdx.x / ws.ch, c = blockIdx.x % ws.ch;
    bulk_stretch2(ws, b, c, lo0, hi0);
    kin = ws.keysA;
    vin = ws.valsA;
    out_keys = ws.keysB;
    out_vals = (VT *)ws.valsB;
    first_bin = b * NB; fill = ws.part_cnt + first_bin; n_bins = NB; cap = ws.part_cap;
  }

  // The rows of a tile sit in registers from their load to their place in the LDS staging area;
  // the next tile's loads are issued as soon as the registers are free, so that they are in
  // flight during the write-out of this tile, and are only turned into keys (finish_tile) at the
  // top of the next round.  st[j]: 0 no row, 1 row, 2 row outside the table's coordinate space.
  u64 k[RPT];
  VT v[RPT];                                // (as loaded: widening a 1- or 2-byte value would be a use,
  int st[RPT];                              // and a use inside a row's guard waits for the load there)
  // what was fetched and is not finished yet: the coordinates of a coordinate source; the one word
  // of any other source waits in k[j] itself
  constexpr bool COORDS = ND > 0;
  BulkRaw<KF, ND> raw[COORDS ? RPT : 1];
  auto load_tile = [&](i64 lo) {
    const i64 hi = lo + T < hi0 ? lo + T : hi0;
    #pragma unroll
    for (int j = 0; j < RPT; j++) {
      const i64 i = lo + j * TPB + tid;
      k[j] = 0; v[j] = 0;
      if (COORDS) raw[COORDS ? j : 0] = BulkRaw<KF, ND>{};
      if (i < hi) {
        if constexpr (COORDS) {
          bulk_fetch<KF, ND>(t, kin, i, n, raw[j]);
        } else {
          BulkRaw<KF, ND> r;
          bulk_fetch<KF, ND>(t, kin, i, n, r);
          k[j] = r.w[0];
        }
        if (REMOVE) {
        } else if (KF == DOK_KF_TABLE) {              // value i & 15 of bucket i >> 4 of the source
          if ((int)(i & 15) < P8<V>::S)
            v[j] = *(const VT *)((const char *)kin + (i >> 4) * 128 + 8 * P8<V>::S + V * (i & 15));
        } else {
          v[j] = ((const VT *)vin)[i];
        }
      }
    }
  };
  auto finish_tile = [&](i64 lo) {
    const i64 hi = lo + T < hi0 ? lo + T : hi0;
    #pragma unroll
    for (int j = 0; j < RPT; j++) {
      st[j] = 0;
      if (lo + j * TPB + tid < hi) {
        if constexpr (COORDS) {
          st[j] = bulk_finish<KF, ND>(t, raw[j], k[j]);
        } else {
          BulkRaw<KF, ND> r;
          r.w[0] = k[j];
          st[j] = bulk_finish<KF, ND>(t, r, k[j]);
        }
      }
    }
  };
  if (lo0 < hi0) load_tile(lo0);

  for (i64 lo = lo0; lo < hi0; lo += T) {
    #pragma unroll
    for (int q = 0; q < BPT; q++)
      if (tid * BPT + q < NB) cnt[tid * BPT + q] = 0;
    finish_tile(lo);
    __syncthreads();

    // bins of the tile's rows and their ranks inside the bins
    int bn[RPT];
    u32 rk[RPT];
    #pragma unroll
    for (int j = 0; j < RPT; j++) {
      bn[j] = -1; rk[j] = 0;
      if (st[j] == 2 && !REMOVE && ws.first_window) n_oob++;
      if (st[j] == 1) {
        if (LEVEL == 1 && (k[j] ^ DOK_P8_XOR) < 2) {
          if (!ws.first_window) {
          } else if (REMOVE) n_fresh -= atomicExch((u64 *)&t.header[DOK_H_SIDE_STATE + (k[j] ^ DOK_P8_XOR)], 0ULL) != 0;
          else n_fresh += p8_side_set(t, k[j] ^ DOK_P8_XOR, (u64)v[j]);
        } else {
          const u32 r = bulk_range_of(k[j], t) - ws.range_base;        // (a row before the window wraps to a huge number)
          if (LEVEL == 2) bn[j] = (int)(r & (NB - 1));
          else if (r < ws.n_part) bn[j] = (int)(r >> ws.sublog);
        }
      }
    }
    #pragma unroll
    for (int j = 0; j < RPT; j++)
      if (bn[j] >= 0) rk[j] = atomicAdd(&cnt[bn[j]], 1u);
    __syncthreads();

    // bin offsets inside the tile; the run of every bin is reserved in the bin's region with one
    // atomic add on its fill counter, whose result is only needed for the write-out below
    u32 c[BPT], got[BPT], csum = 0;
    #pragma unroll
    for (int q = 0; q < BPT; q++) {
      const u32 bin = tid * BPT + q;
      c[q] = bin < NB ? cnt[bin] : 0u;
      csum += c[q];
      got[q] = 0;
      if (c[q] != 0 && bin < n_bins) got[q] = atomicAdd(&fill[bin], c[q]);
    }
    u32 total;
    u32 ex = bulk_block_scan(csum, wsum, total);
    #pragma unroll
    for (int q = 0; q < BPT; q++) {
      if (tid * BPT + q < NB) off[tid * BPT + q] = ex;
      ex += c[q];
    }
    __syncthreads();

    #pragma unroll
    for (int j = 0; j < RPT; j++) {
      if (bn[j] >= 0) {
        const u32 pos = off[bn[j]] + rk[j];
        skeys[pos] = k[j];
        svals[pos] = v[j];
        sbins[pos] = (u16)bn[j];
      }
    }
    if (lo + T < hi0) load_tile(lo + T);
    #pragma unroll
    for (int q = 0; q < BPT; q++) {
      const u32 bin = tid * BPT + q;
      if (bin < NB) {
        gbase[bin] = (first_bin + bin) * cap + got[q];       // (fits 32 bits: checked with the plan)
        const u32 left = got[q] < cap ? cap - got[q] : 0u;
        room[bin] = (u16)(left < 0xffffu ? left : 0xffffu);
      }
    }
    __syncthreads();

    #pragma unroll
    for (int j = 0; j < RPT; j++) {
      const u32 pos = tid + j * TPB;
      if (pos < total) {
        const u32 b = sbins[pos];
        const u32 r = pos - off[b];
        if (r < room[b]) {
          out_keys[gbase[b] + r] = skeys[pos];
          if (!REMOVE) out_vals[gbase[b] + r] = svals[pos];
        } else {
          // the bin's region is full: the row goes to the ordinary insert
          const u32 at = atomicAdd(ws.spill_cnt, 1u);
          if (at < ws.spill_cap) {
            ws.spill_keys[at] = skeys[pos];
            if (!REMOVE) ((VT *)ws.spill_vals)[at] = svals[pos];
          }
        }
      }
    }
    // the barriers at the top of the next tile order these reads before the next writes
  }
  if (LEVEL == 1) {
    dok_wave_add_n(&t.header[DOK_H_NELEM], n_fresh);
    dok_wave_add_n(&t.header[DOK_H_NOOB], n_oob);
  }
}

// ---- merge: one workgroup per range -----------------------------------------------------------
// The range's buckets sit in LDS word-major (word w of local bucket lb at tb[w * LD + lb], LD odd),
// so that threads reading one word of scattered buckets spread over the banks.  The range's rows
// are taken in chunks of DOK_BULK_C, every thread keeping its DOK_BULK_C / R rows in registers.
// Per chunk, first every row LOOKS at its home bucket, then (after a barrier) the rows WRITE:
//   - the key is in the bucket: the value is overwritten (values are never read here, so this
//     needs no barrier);
//   - otherwise the row marks a fingerprint of its key in a per-bucket bitmap that lives as long
//     as the range.  If the mark was already there, an equal key may be among the range's rows,
//     and the row goes on the range's list;
//   - if the bucket has an EMPTY slot, the probe chain of every key whose home it is ends right
//     here, so the key is new (the same holds for a bucket of keys and tombstones whose
//     displacement map is empty): the new rows of a bucket (their keys are distinct, thanks to the
//     marks) draw a rank and the r-th of them takes the r-th free slot, tombstones first, with
//     plain stores;
//   - rows whose rank lies beyond the free slots, and rows whose home bucket has no EMPTY slot,
//     go on the list as well.
// After the last chunk the listed rows (a tenth of the rows at load factor 0.9) are placed all at
// once, without walking their chains: lookup through the home bucket's displacement map, one row
// per key through a small hash set, free slots through a bitmap and per-bucket tickets (see
// there).  Rows that find no room up to the range's last bucket move on to the next range of the
// same workgroup, or - out of the block's last range - to bulk_edge_kernel; rows that found no
// room on the list, and a few awkward cases, are handed to the ordinary insert.
#define DOK_BULK_C (6 * DOK_BULK_R)
#define DOK_BULK_FPW 8                          // 32-bit fingerprint words per bucket
#define DOK_BULK_LIST (2 * DOK_BULK_R)          // capacity of a range's list

// Register type of a row's value in the merge: see there.
template <int V> struct BulkValReg { typedef u32 type; };
template <> struct BulkValReg<8> { typedef u64 type; };

// n-th (0-based) set bit of m (m has more than n set bits).
__device__ __forceinline__ int bulk_nth_bit(u32 m, u32 n) {
  for (u32 i = 0; i < n; i++) m &= m - 1;
  return __builtin_ctz(m);
}

// FRESH: the table's buckets hold nothing yet, not even the EMPTY pattern.  The merge then takes
// every range as empty instead of reading it and writes every range, also those without rows, so
// neither a clear of the table nor its read is paid for.
template <int V, bool FRESH>
__global__ __launch_bounds__(DOK_BULK_R, 3) void bulk_merge_kernel(DevTable t, BulkWs ws) {
  typedef typename ValT<V>::type VT;
  constexpr int S = P8<V>::S;
  constexpr int R = DOK_BULK_R;
  constexpr int LD = R + 1;
  constexpr int C = DOK_BULK_C;
  constexpr int RPT = C / R;
  __shared__ u64 tb[16 * LD];
  __shared__ u32 fresh_cnt[R];
  __shared__ __align__(8) u32 marks[R * DOK_BULK_FPW];
  __shared__ u64 lkey[DOK_BULK_LIST];
  __shared__ VT lval[DOK_BULK_LIST];
  __shared__ u8 lflag[DOK_BULK_LIST];       // 1: the row met a fingerprint mark (an equal key may be around)
  __shared__ u32 lpend[DOK_BULK_LIST];      // carried rows: marked displacements still to be looked at
  __shared__ u32 freemap[DOK_BULK_R / 32];  // buckets that still have an unclaimed free slot
  __shared__ u32 fmask[DOK_BULK_R];         // per bucket: EMPTY slots (low half), tombstones (high half)
  __shared__ int red[R / 64];
  __shared__ u32 n_def;             // rows this workgroup has deferred so far
  __shared__ u32 n_list;            // rows on the list of the current range
  __shared__ u32 n_carry;           // listed rows whose chain ran on into the next range
  __shared__ u32 n_meta;            // displacement marks noted down for the kernel after the merge
  __shared__ u32 range_live;        // the current range's buckets hold something (a key, a tombstone, a mark)
  __shared__ u32 n_edge;            // rows that leave the block's last range (see bulk_edge_kernel)
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  int n_fresh = 0;
  // A workgroup merges a block of consecutive ranges; their rows are one contiguous stretch of
  // keysB, and the rows it defers go, packed, to the same stretch of keysA - no shared cursor.
  const u32 per = (ws.n_part + gridDim.x - 1) / gridDim.x;
  const u32 p_lo = blockIdx.x * per < ws.n_part ? blockIdx.x * per : ws.n_part;
  const u32 p_hi = p_lo + per < ws.n_part ? p_lo + per : ws.n_part;
  const u32 def_base = p_lo * ws.part_cap, blk_end = p_hi * ws.part_cap;
  if (tid == 0) { n_def = 0; n_carry = 0; n_meta = 0; range_live = 0; n_edge = 0; }
  __syncthreads();

  for (u32 p = p_lo; p < p_hi; p++) {
    const u32 lo = p * ws.part_cap, hi = lo + bulk_part_n(ws, p);
    const u32 carried = n_carry;                     // rows handed on by the range before (they sit
                                                     // at the head of the list already)
    if (!FRESH && lo == hi && carried == 0) continue;   // nothing to do in this range
    const u64 b0 = ((u64)p + ws.range_base) << DOK_BULK_RLOG;
    const u64 left = t.nb - b0;
    const u32 nbk = left < (u64)R ? (u32)left : (u32)R;
    ulonglong2 *g = (ulonglong2 *)(t.buckets + b0 * 16);
    if (FRESH && lo == hi && carried == 0) {
      ulonglong2 z; z.x = 0; z.y = 0;
      for (u32 u = tid; u < nbk * 8; u += R) g[u] = z;
      continue;
    }
    ulonglong2 x[8];                                 // this thread's share of the range: 8 x 16 bytes
    #pragma unroll
    for (int q = 0; q < 8; q++) {
      x[q].x = 0; x[q].y = 0;
      if (!FRESH && (u32)(tid + q * R) < nbk * 8) x[q] = g[tid + q * R];
    }
    if (lo == hi) {
      // only carried rows: the chunk loop below, which otherwise stores the bucket copy, is empty
      #pragma unroll
      for (int q = 0; q < 8; q++) {
        const u32 u = tid + q * R, lb = u >> 3, w = (u & 7) * 2;
        if (u < nbk * 8) { tb[w * LD + lb] = x[q].x; tb[(w + 1) * LD + lb] = x[q].y; }
      }
      if (FRESH) fmask[tid] = 0;
      if (tid == 0) n_list = carried;
    }
    // `fr`: the range holds nothing, so its rows need not look at slots (see the look below).  Known
    // at compile time for a fresh table, found out while the copy is staged otherwise (upserts
    // into a cleared or sparsely filled table).
    bool fr = FRESH;
    for (u32 c0 = lo; c0 < hi; c0 += C) {
      const u32 c1 = c0 + C < hi ? c0 + C : hi;
      u64 k[RPT];
      // Values of one and two bytes are fetched as the aligned 32-bit word of valsB that holds
      // them and cut out where they are used: narrowing right after the load would be a use
      // inside the row's guard, and the loads of the chunk's rows would no longer overlap.
      typedef typename BulkValReg<V>::type VR;
      VR v[RPT];
      const u32 vsh = V < 4 ? ((c0 + (u32)tid) & (4 / V - 1)) * 8 * V : 0;   // (the same for every j: R is a multiple of 4)
#define BULK_VAL(j) ((VT)(V < 4 ? (VR)(v[j] >> vsh) : v[j]))
      bool on[RPT];
      #pragma unroll
      for (int j = 0; j < RPT; j++) {
        const u32 i = c0 + j * R + tid;
        on[j] = i < c1;
        k[j] = 0; v[j] = 0;
        if (on[j]) {
          k[j] = ws.keysB[i];
          v[j] = V < 4 ? (VR)((const u32 *)ws.valsB)[i / (V < 4 ? 4 / V : 1)] : (VR)((const VT *)ws.valsB)[i];
        }
      }
      if (c0 == lo) {
        // the bucket loads were issued before the row loads: both are in flight together
        #pragma unroll
        for (int q = 0; q < 8; q++) {
          const u32 u = tid + q * R, lb = u >> 3, w = (u & 7) * 2;
          if (u < nbk * 8) { tb[w * LD + lb] = x[q].x; tb[(w + 1) * LD + lb] = x[q].y; }
        }
        if (!FRESH) {
          u64 nz = 0;
          #pragma unroll
          for (int q = 0; q < 8; q++) nz |= x[q].x | x[q].y;
          if (nz) range_live = 1;
        }
        #pragma unroll
        for (int q = 0; q < DOK_BULK_FPW; q++) marks[q * R + tid] = 0;
        fmask[tid] = 0;                              // (empty range) slots filled so far, per bucket
        if (tid == 0) n_list = carried;
      }
      if (!FRESH) fresh_cnt[tid] = 0;
      // the bucket copy / the last chunk's writes are complete (an empty range's slots are only
      // written in the chunks, never read, so there only the first chunk has to wait - for the
      // zeroes of the empty copy)
      if (!fr || c0 == lo) __syncthreads();
      if (!FRESH && c0 == lo) fr = range_live == 0;

      // look: act[j] = 0 nothing left to do, 1 write key and value into `slot`, 2 defer
      int act[RPT], slot[RPT];
      u32 lh[RPT];
      #pragma unroll
      for (int j = 0; j < RPT; j++) {
        act[j] = 0; slot[j] = 0; lh[j] = 0;
        if (on[j]) {
          const u64 sk = k[j] ^ DOK_P8_XOR;
          const u64 h = dok_fmix64(sk ^ t.seed);
          lh[j] = dok_reduce(h, t.nb) - (u32)b0;
          if (fr) {
            // Nothing is in the range yet: a row that sets a new fingerprint mark carries a key
            // no earlier row of the range has, and takes the next slot of its bucket - no slot
            // is read or compared.  Rows that meet a mark, or a full bucket, go on the list.
            const u32 fp = (u32)h & (32 * DOK_BULK_FPW - 1), bit = 1u << (fp & 31);
            const u32 seen = atomicOr(&marks[lh[j] * DOK_BULK_FPW + (fp >> 5)], bit);
            bool listed = true;
            if (!(seen & bit)) {
              const u32 r = atomicAdd(&fmask[lh[j]], 1u);
              if (r < (u32)S) {
                tb[r * LD + lh[j]] = sk;
                *(VT *)((char *)(tb + (S + ((r * V) >> 3)) * LD + lh[j]) + ((r * V) & 7)) = BULK_VAL(j);
                n_fresh++;
                listed = false;
              }
            }
            // A row that met a mark may repeat the key of an earlier row.  A few such rows per wave
            // are the normal case (fingerprints collide) and go on the list, whose pass sorts
            // them out.  Many of them mean a batch with many equal keys, which would flood the
            // list: then they look into their bucket right here and, where the key is in it by
            // now, overwrite its value.  (The test is per wave, so the usual batch does not pay
            // for the reads of this branch.)
            if (__popcll(dok_ballot((seen & bit) != 0)) >= 8 && (seen & bit)) {
              u32 gm = 0;
              #pragma unroll
              for (int s = 0; s < S; s++) gm |= (u32)(((volatile u64 *)tb)[s * LD + lh[j]] == sk) << s;
              if (gm) {
                const int s = __builtin_ctz(gm);
                *(VT *)((char *)(tb + (S + ((s * V) >> 3)) * LD + lh[j]) + ((s * V) & 7)) = BULK_VAL(j);
                listed = false;
              }
            }
            if (listed) {
              const u32 e = atomicAdd(&n_list, 1u);
              if (e < DOK_BULK_LIST) { lkey[e] = k[j]; lval[e] = BULK_VAL(j); lflag[e] = (seen & bit) ? 1 : 0; }
              else act[j] = 2;
            }
            continue;
          }
          u32 gm = 0, ge = 0, gt = 0;
          #pragma unroll
          for (int s = 0; s < S; s++) {
            const u64 w = tb[s * LD + lh[j]];
            gm |= (u32)(w == sk) << s;
            ge |= (u32)(w == DOK_P8_EMPTY) << s;
            gt |= (u32)(w == DOK_P8_TOMB) << s;
          }
          if (gm) {
            const int s = __builtin_ctz(gm);
            *(VT *)((char *)(tb + (S + ((s * V) >> 3)) * LD + lh[j]) + ((s * V) & 7)) = BULK_VAL(j);
          } else {
            bool listed = true;
            const u32 fp = (u32)h & (32 * DOK_BULK_FPW - 1), bit = 1u << (fp & 31);
            const u32 seen = atomicOr(&marks[lh[j] * DOK_BULK_FPW + (fp >> 5)], bit);
            // The key is new if its chain ends in this bucket: the bucket has an EMPTY slot, or -
            // in a bucket of keys and tombstones only - its displacement map is empty, so no key
            // whose home it is lives anywhere else.
            if (!(seen & bit) && (ge || (gt && tb[DOK_P8_META * LD + lh[j]] == 0))) {
              const u32 r = atomicAdd(&fresh_cnt[lh[j]], 1u);
              const u32 nt = __popc(gt);
              if (r < nt + __popc(ge)) {
                listed = false;
                act[j] = 1;
                slot[j] = r < nt ? bulk_nth_bit(gt, r) : bulk_nth_bit(ge, r - nt);
              }
            }
            if (listed) {
              // onto the range's list while there is room, else to the ordinary insert
              const u32 e = atomicAdd(&n_list, 1u);
              if (e < DOK_BULK_LIST) { lkey[e] = k[j]; lval[e] = BULK_VAL(j); lflag[e] = (seen & bit) ? 1 : 0; }
              else act[j] = 2;
            }
          }
        }
      }
      if (!fr) __syncthreads();
      // write
      #pragma unroll
      for (int j = 0; j < RPT; j++) {
        if (act[j] == 1) {
          const int s = slot[j];
          tb[s * LD + lh[j]] = k[j] ^ DOK_P8_XOR;
          *(VT *)((char *)(tb + (S + ((s * V) >> 3)) * LD + lh[j]) + ((s * V) & 7)) = BULK_VAL(j);
          n_fresh++;
        }
        // deferred rows: one LDS atomic per wave, then a packed global write
        const u64 dm = dok_ballot(act[j] == 2);
        if (dm) {
          u32 base = 0;
          if (lane == 0) base = atomicAdd(&n_def, (u32)__popcll(dm));
          base = dok_shfl32(base, 0);
          if (act[j] == 2) {
            const u32 at = def_base + base + (u32)__popcll(dm & ((1ULL << lane) - 1ULL));
            ws.keysA[at] = k[j];
            dok_store_val<V>(ws.valsA, (i64)at, (u64)BULK_VAL(j));
          }
        }
      }
#undef BULK_VAL
    }
    __syncthreads();

    // The listed rows, one thread each, all at once.  They do not walk their chains:
    //   - where the key can sit is on record: besides the home bucket, at the displacements the
    //     home bucket's map marks (the rows placed so far have set their marks in the LDS copy);
    //   - rows that do not find their key pass a small hash set (in the memory of the fingerprint
    //     marks, which are done with) that lets one row per key through - the value of that row
    //     stands for the equal keys of the batch;
    //   - what is left are distinct new keys, which fight over free slots only.  A new key
    //     belongs into the first bucket from its home on that has a free slot (a tombstone, else
    //     an EMPTY slot; every bucket before it then has no EMPTY slot, which is the placement
    //     rule).  A bitmap of the buckets with free slots left finds that bucket, and a ticket
    //     counter per bucket hands out exactly as many tickets as it has free slots, so failed
    //     claims do not pile up and every bucket whose tickets are gone ends up full.
    // A row that finds no free bucket up to the range's end is handed on to the next range, which
    // this workgroup merges next (it is then known to be new and the only one of its key: its home
    // lies before the range, lhome < 0, and it takes the first free slot from bucket 0 on).  Rows
    // of the block's last range, carried rows that cross a second range and rows whose key may
    // sit beyond the range's end go to the ordinary insert instead.
    u64 *hset = (u64 *)marks;
    constexpr u32 HSET = R * DOK_BULK_FPW / 2;
    {
      u32 ge = 0, gt = 0;
      if (fr) {
        // slots 0 .. filled-1 hold keys, the rest is EMPTY (the count may have run past S)
        const u32 f = fmask[tid] < (u32)S ? fmask[tid] : (u32)S;
        if ((u32)tid < nbk) ge = ((1u << S) - 1u) & ~((1u << f) - 1u);
      } else if ((u32)tid < nbk) {
        #pragma unroll
        for (int s = 0; s < S; s++) {
          const u64 w = tb[s * LD + tid];
          ge |= (u32)(w == DOK_P8_EMPTY) << s;
          gt |= (u32)(w == DOK_P8_TOMB) << s;
        }
      }
      fmask[tid] = ge | (gt << 16);
      const int nfree = __popc(ge) + __popc(gt);
      fresh_cnt[tid] = (u32)nfree;                   // from here on: tickets for the bucket's free slots
      const u64 fm = dok_ballot(nfree != 0);
      if (lane == 0) { freemap[(tid >> 6) * 2] = (u32)fm; freemap[(tid >> 6) * 2 + 1] = (u32)(fm >> 32); }
      #pragma unroll
      for (u32 q = 0; q < HSET / R; q++) hset[q * R + tid] = 0;
      if (tid == 0) n_carry = 0;                     // every thread has read it at the top of the range
    }
    __syncthreads();
    const u32 total = n_list < (u32)DOK_BULK_LIST ? n_list : (u32)DOK_BULK_LIST;
    for (u32 e = tid; e < total; e += R) {
      const u64 key = lkey[e];
      const VT val = lval[e];
      const u64 sk = key ^ DOK_P8_XOR;
      const u64 h = dok_fmix64(sk ^ t.seed);
      const i64 home = (i64)dok_reduce(h, t.nb);
      const int lhome = (int)(home - (i64)b0);        // negative for a carried row
      bool done = false, beyond = false;
      u32 pend = 0;                                   // marked displacements that lie past this range
      if (lhome >= 0) {
        const u64 mw = ((volatile u64 *)tb)[DOK_P8_META * LD + lhome];
        // bit 0 stands for the home bucket here: the look has checked it, but a row that met a
        // fingerprint mark may find the key there by now
        // (a key that was ever placed away from this bucket has its filter bit set here; without
        // the bit there is nothing to look for beyond the home bucket)
        const bool maybe_away = ((u32)(mw >> 32) & p8_fbit(h)) != 0;
        u32 mk = (maybe_away ? ((u32)mw & ~1u) : 0u) | (u32)lflag[e];
        const u32 far_hi = (maybe_away && ((u32)mw & 1u)) ? ((u32)(mw >> 32) & 0xffu) : 0u;
        u32 d = 0;
        while (true) {
          if (mk) { d = (u32)__builtin_ctz(mk); mk &= mk - 1; }
          else if (d < 32 && far_hi >= 32) d = 32;
          else if (d >= 32 && d < far_hi) d++;
          else break;
          const u32 lb = (u32)lhome + d;
          if (lb >= nbk) {
            // the key may sit in the next range: the row goes there with the marks left to check
            // (far displacements are left to the ordinary insert)
            if (d < 32 && far_hi == 0) pend = mk | (1u << d);
            else beyond = true;
            break;
          }
          u32 gm = 0;
          #pragma unroll
          for (int s = 0; s < S; s++) gm |= (u32)(tb[s * LD + lb] == sk) << s;
          if (gm) {
            const int s = __builtin_ctz(gm);
            *(VT *)((char *)(tb + (S + ((s * V) >> 3)) * LD + lb) + ((s * V) & 7)) = val;
            done = true;
            break;
          }
        }
        // a saturated record of the largest displacement: the key may sit further on still
        if (!done && far_hi == DOK_P8_FARCAP) beyond = true;
        if (!done && !beyond) {
          // one row per key goes on
          u32 i = (u32)(h >> 8) & (HSET - 1);
          while (true) {
            const u64 old = atomicCAS(&hset[i], 0ULL, sk);
            if (old == 0) break;
            if (old == sk) { done = true; break; }
            i = (i + 1) & (HSET - 1);
          }
        }
      } else {
        // a carried row: the buckets its home marks and the range before did not hold
        u32 mk = lpend[e];
        while (mk) {
          const u32 d = (u32)__builtin_ctz(mk);
          mk &= mk - 1;
          const int lbs = lhome + (int)d;
          if (lbs < 0) continue;
          const u32 lb = (u32)lbs;
          if (lb >= nbk) { beyond = true; break; }
          u32 gm = 0;
          #pragma unroll
          for (int s = 0; s < S; s++) gm |= (u32)(tb[s * LD + lb] == sk) << s;
          if (gm) {
            const int s = __builtin_ctz(gm);
            *(VT *)((char *)(tb + (S + ((s * V) >> 3)) * LD + lb) + ((s * V) & 7)) = val;
            done = true;
            break;
          }
        }
      }
      if (done) continue;
      // (A row with marks left to check is not placed here even if the range has room: its key
      // may sit further on.  Its home marks a bucket past the range's end, so no bucket from its
      // home to that end has an EMPTY slot, then or now, and a place in the next range keeps
      // its chain whole.)
      u32 from = lhome < 0 ? 0u : (u32)lhome;
      while (!beyond && pend == 0) {
        // first bucket at or after `from` with a free slot left
        u32 T = DOK_NONE32;
        for (u32 wi = from >> 5; wi < (u32)(R / 32); wi++) {
          u32 m = ((volatile u32 *)freemap)[wi];
          if (wi == (from >> 5)) m &= ~0u << (from & 31);
          if (m) { T = wi * 32 + (u32)__builtin_ctz(m); break; }
        }
        if (T == DOK_NONE32) break;                   // the chain leaves the range
        const int ticket = atomicSub((int *)&fresh_cnt[T], 1);
        if (ticket <= 1) atomicAnd(&freemap[T >> 5], ~(1u << (T & 31)));   // the last one is out
        if (ticket <= 0) { from = T + 1; continue; }
        // The ticket stands for one of the free slots the bucket had when the tickets were
        // counted: the k-th row to arrive takes the k-th of them, tombstones first.  Nobody else
        // writes that slot, so a store does (rows checking this bucket for their own, different
        // key may read it before or after).
        {
          const u32 fm = fmask[T], ge = fm & 0xffffu, gt = fm >> 16;
          const u32 nt = __popc(gt);
          const u32 k = nt + __popc(ge) - (u32)ticket;
          const int ts = k < nt ? bulk_nth_bit(gt, k) : bulk_nth_bit(ge, k - nt);
          __hip_atomic_store(&tb[ts * LD + T], sk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          *(VT *)((char *)(tb + (S + ((ts * V) >> 3)) * LD + T) + ((ts * V) & 7)) = val;
          const u32 td = (u32)((int)T - lhome);
          if (td > 0 && lhome >= 0) {
            p8_mark(tb + DOK_P8_META * LD + lhome, td, p8_fbit(h), 0);
          } else if (td > 0) {
            // A carried row: its home bucket went back to HBM with plain stores a moment ago,
            // and an atomic on that line from inside this kernel is not ordered against
            // them.  The mark (with the key's filter bit) is noted down (in the part of keysB this
            // workgroup has consumed) and applied by the kernel that runs after the merge.
            const u32 mi = atomicAdd(&n_meta, 1u);
            ws.keysB[def_base + mi] = ((u64)home << 32) | ((u64)p8_fidx(h) << 24) | (u64)(td & 0xffffffu);
          }
          n_fresh++;
          done = true;
        }
        break;
      }
      if (!done) {
        bool carry = !beyond && p + 1 < p_hi && lhome >= 0;
        if (carry) {
          const u32 c = atomicAdd(&n_carry, 1u);
          if (c < (u32)R && total + c < (u32)DOK_BULK_LIST) { lkey[total + c] = key; lval[total + c] = val; lpend[total + c] = pend; }
          else carry = false;                         // n_carry is clamped below
        }
        if (!carry) {
          // Rows that have looked at every bucket their home marks, are the only row of their key
          // and found no room up to the end of the block's LAST range continue in the next
          // block's first range: bulk_edge_kernel places them there once this kernel is through.
          // They are listed from the top of the workgroup's stretch downwards; everything else
          // goes, from the bottom upwards, to the ordinary insert.
          const bool edge = p + 1 == p_hi && p_hi < ws.n_part && !beyond && pend == 0 && (lhome >= 0 || lpend[e] == 0);
          const u32 at = edge ? blk_end - 1 - atomicAdd(&n_edge, 1u) : def_base + atomicAdd(&n_def, 1u);
          ws.keysA[at] = key;
          dok_store_val<V>(ws.valsA, (i64)at, (u64)val);
        }
      }
    }
    __syncthreads();
    {
      // the carried rows move to the head of the list, where the next range expects them
      u32 nc = n_carry;
      if (nc > (u32)R) nc = R;
      if (total + nc > (u32)DOK_BULK_LIST) nc = DOK_BULK_LIST - total;
      u64 ck = 0; VT cv = 0; u32 cp = 0;
      if ((u32)tid < nc) { ck = lkey[total + tid]; cv = lval[total + tid]; cp = lpend[total + tid]; }
      __syncthreads();
      if ((u32)tid < nc) { lkey[tid] = ck; lval[tid] = cv; lpend[tid] = cp; }
      __syncthreads();
      if (tid == 0) { n_carry = nc; range_live = 0; }
    }
    __syncthreads();

    for (u32 u = tid; u < nbk * 8; u += R) {
      const u32 lb = u >> 3, w = (u & 7) * 2;
      ulonglong2 y;
      y.x = tb[w * LD + lb];
      y.y = tb[(w + 1) * LD + lb];
      g[u] = y;
    }
    __syncthreads();
  }

  // one header update per workgroup
  #pragma unroll
  for (int o = 32; o > 0; o >>= 1) n_fresh += __shfl_xor(n_fresh, o, 64);
  if ((tid & 63) == 0) red[tid >> 6] = n_fresh;
  __syncthreads();
  if (tid == 0) {
    int sum = 0;
    for (int w = 0; w < R / 64; w++) sum += red[w];
    if (sum) atomicAdd((u64 *)&t.header[DOK_H_NELEM], (u64)(i64)sum);
    ws.def_cnt[blockIdx.x] = n_def;
    ws.meta_cnt[blockIdx.x] = n_meta;
    ws.edge_cnt[blockIdx.x] = n_edge;
  }
}

// ---- rows that left a block's last range ------------------------------------------------------------
// Launched with the merge kernel's grid, after it.  Workgroup w takes the rows merge workgroup w
// listed as leaving the last range of its block - new keys, one row each, with no free slot from
// their home bucket to the block's end - and places them in the next block's first range (and the
// one after, if the blocks are that long), whose buckets are final by now: the same bitmap and
// tickets as in the merge, on an LDS copy of the range.  The workgroups touch disjoint ranges.
// Rows that find no room there either join the rows for the ordinary insert.
template <int V>
__global__ __launch_bounds__(DOK_BULK_R) void bulk_edge_kernel(DevTable t, BulkWs ws) {
  typedef typename ValT<V>::type VT;
  constexpr int S = P8<V>::S;
  constexpr int R = DOK_BULK_R;
  constexpr int LD = R + 1;
  __shared__ u64 tb[16 * LD];
  __shared__ u32 tickets[R], fmask[R], freemap[R / 32];
  __shared__ u32 n_left, n_note, n_a;
  const int tid = threadIdx.x, lane = tid & 63;
  const u32 per = (ws.n_part + gridDim.x - 1) / gridDim.x;
  const u32 p_lo = blockIdx.x * per < ws.n_part ? blockIdx.x * per : ws.n_part;
  const u32 p_hi = p_lo + per < ws.n_part ? p_lo + per : ws.n_part;
  const u32 n_rows = ws.edge_cnt[blockIdx.x];
  // (more rows than threads: left to the ordinary insert, which reads the list as it is)
  if (n_rows == 0 || n_rows > (u32)R || p_hi >= ws.n_part) return;
  const u32 def_base = p_lo * ws.part_cap, top = p_hi * ws.part_cap;
  const u32 note_base = def_base + ws.meta_cnt[blockIdx.x], a_base = def_base + ws.def_cnt[blockIdx.x];
  bool have = (u32)tid < n_rows;
  u64 key = 0, sk = 0, home = 0, fidx = 0;
  VT val = 0;
  if (have) {
    key = ws.keysA[top - 1 - tid];
    val = (VT)dok_load_val<V>(ws.valsA, (i64)(top - 1 - tid));
    sk = key ^ DOK_P8_XOR;
    const u64 h = p8_hash(sk, t);
    home = dok_reduce(h, t.nb);
    fidx = p8_fidx(h);
  }
  if (tid == 0) { n_note = 0; n_a = 0; }
  int n_fresh = 0;
  const u32 guests = per < 2 ? per : 2;
  for (u32 gi = 0; gi < guests && p_hi + gi < ws.n_part; gi++) {
    const u32 p = p_hi + gi;
    const u64 b0 = ((u64)p + ws.range_base) << DOK_BULK_RLOG;
    const u64 left = t.nb - b0;
    const u32 nbk = left < (u64)R ? (u32)left : (u32)R;
    ulonglong2 *g = (ulonglong2 *)(t.buckets + b0 * 16);
    for (u32 u = tid; u < nbk * 8; u += R) {
      const ulonglong2 x = g[u];
      const u32 lb = u >> 3, w = (u & 7) * 2;
      tb[w * LD + lb] = x.x; tb[(w + 1) * LD + lb] = x.y;
    }
    if (tid == 0) n_left = 0;
    __syncthreads();
    {
      u32 ge = 0, gt = 0;
      if ((u32)tid < nbk) {
        #pragma unroll
        for (int s = 0; s < S; s++) {
          const u64 w = tb[s * LD + tid];
          ge |= (u32)(w == DOK_P8_EMPTY) << s;
          gt |= (u32)(w == DOK_P8_TOMB) << s;
        }
      }
      fmask[tid] = ge | (gt << 16);
      const int nfree = __popc(ge) + __popc(gt);
      tickets[tid] = (u32)nfree;
      const u64 fm = dok_ballot(nfree != 0);
      if (lane == 0) { freemap[(tid >> 6) * 2] = (u32)fm; freemap[(tid >> 6) * 2 + 1] = (u32)(fm >> 32); }
    }
    __syncthreads();
    if (have) {
      u32 from = 0;
      while (true) {
        u32 T = DOK_NONE32;
        for (u32 wi = from >> 5; wi < (u32)(R / 32); wi++) {
          u32 m = ((volatile u32 *)freemap)[wi];
          if (wi == (from >> 5)) m &= ~0u << (from & 31);
          if (m) { T = wi * 32 + (u32)__builtin_ctz(m); break; }
        }
        if (T == DOK_NONE32) break;
        const int ticket = atomicSub((int *)&tickets[T], 1);
        if (ticket <= 1) atomicAnd(&freemap[T >> 5], ~(1u << (T & 31)));
        if (ticket <= 0) { from = T + 1; continue; }
        const u32 fm = fmask[T], ge = fm & 0xffffu, gt = fm >> 16;
        const u32 nt = __popc(gt);
        const u32 k = nt + __popc(ge) - (u32)ticket;
        const int ts = k < nt ? bulk_nth_bit(gt, k) : bulk_nth_bit(ge, k - nt);
        tb[ts * LD + T] = sk;
        *(VT *)((char *)(tb + (S + ((ts * V) >> 3)) * LD + T) + ((ts * V) & 7)) = val;
        // the displacement mark belongs to a bucket of another range: noted for the kernel that follows
        const u64 td = b0 + T - home;
        ws.keysB[note_base + atomicAdd(&n_note, 1u)] = (home << 32) | (fidx << 24) | (td & 0xffffffULL);
        n_fresh++;
        have = false;
        break;
      }
      if (have) atomicAdd(&n_left, 1u);
    }
    __syncthreads();
    for (u32 u = tid; u < nbk * 8; u += R) {
      const u32 lb = u >> 3, w = (u & 7) * 2;
      ulonglong2 y;
      y.x = tb[w * LD + lb];
      y.y = tb[(w + 1) * LD + lb];
      g[u] = y;
    }
    const u32 still = n_left;
    __syncthreads();
    if (still == 0) break;
  }
  // what is left joins the rows for the ordinary insert (the list above has been read in full, so
  // its place may be written over)
  if (have) {
    const u32 at = a_base + atomicAdd(&n_a, 1u);
    ws.keysA[at] = key;
    dok_store_val<V>(ws.valsA, (i64)at, (u64)val);
  }
  dok_wave_add_n(&t.header[DOK_H_NELEM], n_fresh);
  __syncthreads();
  if (tid == 0) {
    ws.def_cnt[blockIdx.x] += n_a;
    ws.meta_cnt[blockIdx.x] += n_note;
    ws.edge_cnt[blockIdx.x] = 0;
  }
}

// ---- the rows the merge handed back: ordinary insert ---------------------------------------------
// Launched with the merge kernel's grid: workgroup w inserts the rows merge workgroup w deferred.
template <int V>
__global__ __launch_bounds__(DOK_TPB, DOK_STREAM_WAVES) void bulk_deferred_kernel(DevTable t, BulkWs ws) {
  const u32 per = (ws.n_part + gridDim.x - 1) / gridDim.x;
  const u32 p_lo = blockIdx.x * per < ws.n_part ? blockIdx.x * per : ws.n_part;
  const i64 base = (i64)p_lo * ws.part_cap;
  // displacement marks the merge could not set itself (see there)
  const u32 n_marks = ws.meta_cnt[blockIdx.x];
  for (u32 i = threadIdx.x; i < n_marks; i += DOK_TPB) {
    // home bucket (32 bits) | the key's filter bit number (8) | displacement (24)
    const u64 note = ws.keysB[base + i];
    p8_mark(t.buckets + (note >> 32) * 16 + DOK_P8_META, (u32)note & 0xffffffu, 256u << ((u32)(note >> 24) & 0xffu), 0);
  }
  // the rows from the bottom of the stretch, and - if bulk_edge_kernel has not taken them - the
  // rows listed from its top downwards
  const u32 p_hi = p_lo + per < ws.n_part ? p_lo + per : ws.n_part;
  const i64 top = (i64)p_hi * ws.part_cap;
  // ... and this workgroup's share of the rows that found their bin's region full
  const i64 n_sp_all = ws.spill_cnt[0] < ws.spill_cap ? ws.spill_cnt[0] : ws.spill_cap;
  const i64 sp_per = (n_sp_all + gridDim.x - 1) / gridDim.x;
  const i64 sp_lo = sp_per * blockIdx.x < n_sp_all ? sp_per * blockIdx.x : n_sp_all;
  const i64 n_sp = sp_lo + sp_per < n_sp_all ? sp_per : n_sp_all - sp_lo;
  const i64 n_a = ws.def_cnt[blockIdx.x], n_e = n_a + ws.edge_cnt[blockIdx.x], n = n_e + n_sp;
  if (blockIdx.x == 0 && threadIdx.x == 0) t.header[DOK_H_NSPILL] = n_sp_all;
  const i64 waves = DOK_TPB / 64, wave = threadIdx.x >> 6;
  const i64 share = (n + waves - 1) / waves;
  i64 lo = wave * share, hi = lo + share;
  if (hi > n) hi = n;
  if (lo > hi) lo = hi;
  const u64 *keys = ws.keysA;
  const void *vals = ws.valsA;
  p8_stream_insert_rows<V>(t, lo, hi, nullptr, [&](i64 i, u64 &key, u64 &val) -> int {
    if (i >= n_e) {
      key = ws.spill_keys[sp_lo + (i - n_e)];
      val = dok_load_val<V>(ws.spill_vals, sp_lo + (i - n_e));
      return 0;
    }
    const i64 at = i < n_a ? base + i : top - 1 - (i - n_a);
    key = keys[at];
    val = dok_load_val<V>(vals, at);
    return 0;
  });
}

// ---- bulk removal ---------------------------------------------------------------------------------
// The keys of a large removal, partitioned by the range of their home bucket like the rows of a bulk
// insert, meet their buckets in table order: a workgroup works through the ranges of its block, its
// lookups read every bucket line of a range once (and mostly from the caches, the rows of a range
// arriving together), and the tombstones of a line leave the GPU as one write-back - where the
// per-row kernel pays a random line read and a partial write per key.
// Equal keys of a batch have one home, so they meet in one workgroup, which lets exactly one of them
// count: a bit per slot of the range in LDS.  (A key found outside the range of its home - placed
// far from it, near the range's end - is settled by a compare-and-swap on the slot instead.)
#define DOK_BULK_RM_CHUNK 2048                      // keys of a range sorted and looked up at a time
template <int V>
__global__ __launch_bounds__(DOK_TPB) void bulk_remove_kernel(DevTable t, BulkWs ws) {
  constexpr int CH = DOK_BULK_RM_CHUNK, RPT = CH / DOK_TPB;
  static_assert(DOK_BULK_R == DOK_TPB, "one counter of the bucket sort per thread");
  __shared__ u32 taken[DOK_BULK_R * 16 / 32];       // one bit per (bucket of the range, word of the bucket)
  __shared__ u64 skeys[CH];                         // the chunk's keys in bucket order
  __shared__ u32 cnt[DOK_BULK_R], off[DOK_BULK_R], wsum[16];
  const int tid = threadIdx.x;
  const u32 per = (ws.n_part + gridDim.x - 1) / gridDim.x;
  const u32 p_lo = blockIdx.x * per < ws.n_part ? blockIdx.x * per : ws.n_part;
  const u32 p_hi = p_lo + per < ws.n_part ? p_lo + per : ws.n_part;
  int n_removed = 0;
  // The work items are (range, chunk of its keys); the keys of the next item are loaded into
  // registers while the current one is looked up.
  u32 p = p_lo, c0 = 0;
  while (p < p_hi && bulk_part_n(ws, p) == 0) p++;
  u64 k[RPT];
  auto load_keys = [&](u32 pp, u32 cc) {
    const u32 n_pp = bulk_part_n(ws, pp);
    const u64 *rows = ws.keysB + (u64)pp * ws.part_cap + cc;
    const u32 mm = n_pp - cc < (u32)CH ? n_pp - cc : (u32)CH;
    #pragma unroll
    for (int j = 0; j < RPT; j++) {
      const u32 i = (u32)j * DOK_TPB + tid;
      k[j] = i < mm ? rows[i] : 0;
    }
  };
  if (p < p_hi) load_keys(p, 0);
  while (p < p_hi) {
    const u32 n_p = bulk_part_n(ws, p);
    const u64 b0 = ((u64)p + ws.range_base) << DOK_BULK_RLOG;
    if (c0 == 0)
      for (int q = tid; q < DOK_BULK_R * 16 / 32; q += DOK_TPB) taken[q] = 0;
    u32 pn = p, cn = c0 + CH;                          // the item after this one
    if (cn >= n_p) {
      cn = 0; pn = p + 1;
      while (pn < p_hi && bulk_part_n(ws, pn) == 0) pn++;
    }
    {
      const u32 m = n_p - c0 < (u32)CH ? n_p - c0 : (u32)CH;
      // The keys of a range arrive in no order.  Sorted by home bucket (a counting sort in LDS),
      // the keys of one bucket sit in neighbouring lanes, so every bucket line is fetched once, by
      // one wave instruction, instead of once per key and whenever a key's turn comes.
      cnt[tid] = 0;
      u32 lb[RPT], rk[RPT];
      __syncthreads();
      #pragma unroll
      for (int j = 0; j < RPT; j++) {
        const u32 i = (u32)j * DOK_TPB + tid;
        lb[j] = 0; rk[j] = 0;
        if (i < m) {
          lb[j] = (p8_home(k[j] ^ DOK_P8_XOR, t) - (u32)b0) & (DOK_BULK_R - 1);
          rk[j] = atomicAdd(&cnt[lb[j]], 1u);
        }
      }
      __syncthreads();
      u32 total;
      const u32 ex = bulk_block_scan(cnt[tid], wsum, total);
      off[tid] = ex;
      __syncthreads();
      #pragma unroll
      for (int j = 0; j < RPT; j++)
        if ((u32)j * DOK_TPB + tid < m) skeys[off[lb[j]] + rk[j]] = k[j];
      __syncthreads();
      if (pn < p_hi) load_keys(pn, cn);                 // (in flight during the lookups below)
      for (u32 i0 = 0; i0 < m; i0 += DOK_TPB) {
        const u32 i = i0 + tid;
        const bool active = i < m;
        const u64 sk = (active ? skeys[i] : 0) ^ DOK_P8_XOR;
        bool found = false, removed = false;
        u64 val = 0;
        u32 sb = 0; int ss = 0, nprobe = 0;
        const u64 h = p8_hash(sk, t);
        const u32 home = active ? dok_reduce(h, t.nb) : 0u;
        // Every lane reads the key words of its own key's home bucket (neighbouring lanes read the
        // same line: the keys are in bucket order): a dozen instructions per key, where the
        // cooperative probe of p8_lookup - made for keys in no order, one line per 16 lanes and
        // round - takes some forty and would bound this kernel by instruction issue.  Only a key that
        // is not in its home bucket although the bucket's metadata says it may sit further on takes
        // the general lookup.
        bool more = false;
        {
          const ulonglong2 *hb = (const ulonglong2 *)(t.buckets + (u64)home * 16);
          ulonglong2 w[8];
          #pragma unroll
          for (int q = 0; q < 8; q++) w[q] = hb[q];
          u32 gm = 0;
          #pragma unroll
          for (int q = 0; q < 8; q++) {
            if (2 * q < P8<V>::S) gm |= (u32)(w[q].x == sk) << (2 * q);
            if (2 * q + 1 < P8<V>::S) gm |= (u32)(w[q].y == sk) << (2 * q + 1);
          }
          const u64 meta = w[7].y;
          if (active && gm) { found = true; sb = home; ss = __builtin_ctz(gm); }
          more = active && !gm && (u32)meta != 0 && ((u32)(meta >> 32) & p8_fbit(h)) != 0;
        }
        if (dok_ballot(more) != 0) {
          bool f2 = false;
          u32 sb2 = 0; int ss2 = 0;
          p8_lookup<V, false>(t.buckets, t.nb, sk, more ? home : 0u, p8_fbit(h), more, f2, val, sb2, ss2, nprobe);
          if (more && f2) { found = true; sb = sb2; ss = ss2; }
        }
        if (found) {
          const u64 lbk = (u64)sb - b0;
          if (lbk < (u64)DOK_BULK_R) {
            const u32 bit = (u32)lbk * 16 + (u32)ss;
            removed = !(atomicOr(&taken[bit >> 5], 1u << (bit & 31)) & (1u << (bit & 31)));
            if (removed) t.buckets[(u64)sb * 16 + ss] = DOK_P8_TOMB;
          } else {
            removed = atomicCAS(t.buckets + (u64)sb * 16 + ss, sk, DOK_P8_TOMB) == sk;
          }
        }
        n_removed += removed;
      }
      __syncthreads();                                // skeys, cnt and (next range) the bits are reused
    }
    p = pn; c0 = cn;
  }
  dok_block_add1(&t.header[DOK_H_NELEM], -n_removed);
}

// The keys that found their bin's region full during the partition (batches with very many equal
// keys), after everything else: one compare-and-swap per row found.
template <int V>
__global__ __launch_bounds__(DOK_TPB) void bulk_remove_spill_kernel(DevTable t, BulkWs ws) {
  const i64 n = ws.spill_cnt[0] < ws.spill_cap ? ws.spill_cnt[0] : ws.spill_cap;
  int n_removed = 0;
  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool active = i < n;
    const u64 sk = (active ? ws.spill_keys[i] : 0) ^ DOK_P8_XOR;
    bool found = false, removed = false;
    u64 val = 0;
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V>(t.buckets, t.nb, sk, active ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), active, found, val, sb, ss, nprobe);
    if (found) removed = atomicCAS(t.buckets + (u64)sb * 16 + ss, sk, DOK_P8_TOMB) == sk;
    n_removed += removed;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) t.header[DOK_H_NSPILL] = n;
  dok_block_add1(&t.header[DOK_H_NELEM], -n_removed);
}

// Batch keys of any format as one 8-byte word per row in keysB (all ones: a row outside the
// coordinate space), for the first scatter of a removal.
template <int KF>
__global__ __launch_bounds__(DOK_TPB) void bulk_keys_to_words_kernel(DevTable t, const void *__restrict__ keys, i64 n, BulkWs ws) {
  for (i64 i = (i64)blockIdx.x * DOK_TPB + threadIdx.x; i < n; i += (i64)gridDim.x * DOK_TPB) {
    u64 key = 0;
    ws.keysB[i] = dok_load_key8<KF>(t, keys, i, n, key) ? key : ~0ULL;
  }
}

// ---- host side -----------------------------------------------------------------------------------
struct BulkPlan {
  u64 n_part_all;            // ranges of the whole table
  u32 n_windows;             // runs of the passes: windows of DOK_BULK_WINDOW ranges
  u32 n_part, n_big;         // ranges / first-level bins of a (full) window
  u32 sublog, ch, g1, gm;
  u32 big_cap, part_cap, spill_cap;
  i64 share;
  size_t o_keysA, o_keysB, o_valsA, o_valsB, o_big_cnt, o_part_cnt, o_spill_keys, o_spill_vals, o_spill_cnt,
         o_def_cnt, o_meta_cnt, o_edge_cnt, bytes;
};

// Rows the region of a bin holds that receives `mean` rows on average (the hash spreads the rows
// uniformly over the buckets, so a bin's share is binomial): the mean plus `sigmas` standard
// deviations and a little, a multiple of `unit`, and never more than all the rows.
static inline u64 bulk_region_rows(double mean, double sigmas, u64 unit, u64 all_rows) {
  u64 cap = (u64)(mean + sigmas * __builtin_sqrt(mean) + 2.0 * (double)unit) + 1;
  if (cap > all_rows) cap = all_rows;
  return (cap + unit - 1) / unit * unit;
}

static inline size_t bulk_align(size_t x) { return (x + 255) & ~(size_t)255; }

// False when the bulk path cannot take this table / batch (the caller then uses the ordinary
// insert).
// n = rows of the input that are looked at, n_cap = most rows that can turn out to be real (the
// two differ for a table source, where most words are not key slots).
static bool bulk_plan(const DevTable &d, i64 n, BulkPlan &p, u32 g1 = DOK_BULK_GRID, u32 gm = DOK_BULK_GRID,
                      i64 n_cap = -1) {
  if (n_cap < 0) n_cap = n;
  if (n < 1 || n > 0x7fff0000LL) return false;
  p.g1 = g1;
  const u64 n_part_all = (d.nb + DOK_BULK_R - 1) >> DOK_BULK_RLOG;
  p.n_part_all = n_part_all;
  p.n_windows = (u32)((n_part_all + DOK_BULK_WINDOW - 1) / DOK_BULK_WINDOW);     // (at most 16: a table has < 2^32 buckets)
  const u64 n_part = n_part_all < DOK_BULK_WINDOW ? n_part_all : DOK_BULK_WINDOW;
  p.sublog = n_part <= ((u64)DOK_BULK_MAXBIG << DOK_BULK_SUBLOG) ? DOK_BULK_SUBLOG : DOK_BULK_SUBLOG_WIDE;
  const u64 n_big = (n_part + (1u << p.sublog) - 1) >> p.sublog;
  p.n_part = (u32)n_part;
  p.n_big = (u32)n_big;
  // second pass: about 4096 workgroups in all, 16 to 256 per first-level bin
  u32 ch = 16;
  while (ch < 256 && (u64)ch * n_big < 4096) ch *= 2;
  p.ch = ch;
  // first pass: equal stretches, whole tiles
  const i64 tiles = (n + DOK_BULK_T - 1) / DOK_BULK_T;
  p.share = ((tiles + g1 - 1) / g1) * DOK_BULK_T;
  p.gm = p.n_part < gm ? p.n_part : gm;
  const size_t parts = (size_t)n_big << p.sublog;
  // Regions: a first-level bin covers (256 << sublog) of the nb buckets, a range 256 of them.  Six
  // resp. five standard deviations of slack: a region that still overflows (one range in a million
  // at five) spills a few rows to the ordinary insert.
  const double buckets = (double)d.nb;
  const double f_big = (double)((u64)DOK_BULK_R << p.sublog) / buckets, f_part = (double)DOK_BULK_R / buckets;
  const u64 big_cap = bulk_region_rows((double)n_cap * (f_big < 1.0 ? f_big : 1.0), 6.0, 64, (u64)n_cap);
  const u64 part_cap = bulk_region_rows((double)n_cap * (f_part < 1.0 ? f_part : 1.0), 5.0, 16, (u64)n_cap);
  const u64 rowsA_1 = (u64)n_big * big_cap, rowsB = (u64)parts * part_cap;
  if (rowsA_1 >= 0xffff0000ULL || rowsB >= 0xffff0000ULL) return false;      // positions are 32 bits
  // keysA also serves the merge as scratch, addressed like keysB; keysB first holds the linearised
  // keys of a coordinate source (n rows)
  const u64 rowsA = rowsA_1 > rowsB ? rowsA_1 : rowsB;
  const u64 rowsB2 = (d.lin_ndim >= 3 && rowsB < (u64)n) ? (u64)n : rowsB;
  p.big_cap = (u32)big_cap; p.part_cap = (u32)part_cap;
  p.spill_cap = (u32)n_cap;                                                   // (every row may spill: n_cap < 2^31)
  size_t o = 0;
  p.o_keysA = o; o = bulk_align(o + 8 * (size_t)rowsA);
  p.o_keysB = o; o = bulk_align(o + 8 * (size_t)rowsB2);
  p.o_valsA = o; o = bulk_align(o + (size_t)d.value_bytes * (size_t)rowsA);
  p.o_valsB = o; o = bulk_align(o + (size_t)d.value_bytes * (size_t)rowsB);
  p.o_spill_keys = o; o = bulk_align(o + 8 * (size_t)p.spill_cap);
  p.o_spill_vals = o; o = bulk_align(o + (size_t)d.value_bytes * (size_t)p.spill_cap);
  p.o_big_cnt = o; o = bulk_align(o + 4 * (size_t)DOK_BULK_MAXBIG);
  p.o_part_cnt = o; o = bulk_align(o + 4 * parts);
  p.o_spill_cnt = o; o = bulk_align(o + 4);
  p.o_def_cnt = o; o = bulk_align(o + 4 * DOK_BULK_GRID);
  p.o_meta_cnt = o; o = bulk_align(o + 4 * DOK_BULK_GRID);
  p.o_edge_cnt = o; o = bulk_align(o + 4 * DOK_BULK_GRID);
  p.bytes = o;
  return true;
}

// Device view of the workspace for window `win` of the table.
static void bulk_bind(const BulkPlan &p, void *workspace, BulkWs &ws, u32 win = 0) {
  char *w = (char *)workspace;
  ws.keysA = (u64 *)(w + p.o_keysA);
  ws.keysB = (u64 *)(w + p.o_keysB);
  ws.valsA = w + p.o_valsA;
  ws.valsB = w + p.o_valsB;
  ws.big_cnt = (u32 *)(w + p.o_big_cnt);
  ws.part_cnt = (u32 *)(w + p.o_part_cnt);
  ws.spill_keys = (u64 *)(w + p.o_spill_keys);
  ws.spill_vals = w + p.o_spill_vals;
  ws.spill_cnt = (u32 *)(w + p.o_spill_cnt);
  ws.big_cap = p.big_cap;
  ws.part_cap = p.part_cap;
  ws.spill_cap = p.spill_cap;
  ws.def_cnt = (u32 *)(w + p.o_def_cnt);
  ws.meta_cnt = (u32 *)(w + p.o_meta_cnt);
  ws.edge_cnt = (u32 *)(w + p.o_edge_cnt);
  const u64 base = (u64)win * DOK_BULK_WINDOW;
  const u64 parts = p.n_part_all - base < DOK_BULK_WINDOW ? p.n_part_all - base : DOK_BULK_WINDOW;
  ws.range_base = (u32)base;
  ws.first_window = win == 0;
  ws.n_part = (u32)parts;
  ws.n_big = (u32)((parts + (1u << p.sublog) - 1) >> p.sublog);
  ws.sublog = p.sublog;
  ws.g1 = p.g1;
  ws.ch = p.ch;
  ws.share = p.share;
}

// Persistent kernels get exactly as many workgroups as the device holds at once, so that no
// workgroup waits for a slot while others have already finished their share.
static int bulk_cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
    else cus = 256;
  }
  return cus;
}
template <class K>
static u32 bulk_resident(K kernel, int block, u32 limit, u32 multiple) {
  int occ = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, block, 0) != hipSuccess || occ < 1) occ = 1;
  u64 g = (u64)occ * (u64)bulk_cu_count();
  if (g > limit) g = limit;
  g -= g % multiple;
  return g < multiple ? multiple : (u32)g;
}

template <int V, int KF>
static bool bulk_plan_for(const DevTable &d, i64 n, BulkPlan &p, i64 n_cap = -1) {
  static u32 g1 = 0, gm = 0;
  if (g1 == 0) {
    constexpr int ND = (KF == DOK_KF_COLS || KF == DOK_KF_ROWS) ? 2 : 0;   // (the dimensions do not change the LDS use)
    g1 = bulk_resident(bulk_scatter_kernel<V, KF, 1, DOK_BULK_SUBLOG, ND>, bulk_tpb(1, KF, ND), DOK_BULK_GRID, 64);
    gm = bulk_resident(bulk_merge_kernel<V, false>, DOK_BULK_R, DOK_BULK_GRID, 1);
  }
  return bulk_plan(d, n, p, g1, gm, n_cap);
}

// The two reserved key patterns live in the table header, not in a bucket.
__global__ void bulk_side_slots_kernel(DevTable src, DevTable dst) {
  if (threadIdx.x < 2 && src.header[DOK_H_SIDE_STATE + threadIdx.x] != 0) {
    dst.header[DOK_H_SIDE_STATE + threadIdx.x] = 1;
    dst.header[DOK_H_SIDE_VALUE + threadIdx.x] = src.header[DOK_H_SIDE_VALUE + threadIdx.x];
    atomicAdd((u64 *)&dst.header[DOK_H_NELEM], 1ULL);
  }
}

// FRESH: the table's memory is uninitialised (see bulk_merge_kernel); the header is zeroed here.
// ND: dimensions of a coordinate source (KF rows or columns), else 0.
template <int V, int KF, int ND, bool FRESH>
static void bulk_launch_nd(const DevTable &d, const void *keys, const void *values, i64 n, const BulkPlan &p,
                           void *workspace, hipStream_t s) {
  for (u32 win = 0; win < p.n_windows; win++) {
  BulkWs ws;
  bulk_bind(p, workspace, ws, win);
  bulk_init_kernel<<<64, DOK_TPB, 0, s>>>(ws, FRESH && win == 0 ? d.header : nullptr);
  // coordinate rows of three and more dimensions are linearised first (see bulk_linearise_kernel)
  constexpr bool LIN = ND >= 3;
  if constexpr (LIN) {
    bulk_linearise_kernel<KF, ND><<<p.g1, DOK_BULK_CTPB, 0, s>>>(d, keys, n, ws);
    bulk_scatter_kernel<V, DOK_KF_LIN, 1><<<p.g1, bulk_tpb(1, DOK_KF_LIN, 0), 0, s>>>(d, ws.keysB, values, n, ws);
  } else {
    bulk_scatter_kernel<V, KF, 1, DOK_BULK_SUBLOG, ND><<<p.g1, bulk_tpb(1, KF, ND), 0, s>>>(d, keys, values, n, ws);
  }
  // narrow values: small second-pass tiles when the workgroups' stretches are short
  const bool smallt = V <= 2 && n / ((i64)p.n_big * p.ch * p.n_windows) < DOK_BULK_T2S_BELOW;
  if (p.sublog == DOK_BULK_SUBLOG) {
    if (smallt) bulk_scatter_kernel<V, DOK_KF_U64, 2, DOK_BULK_SUBLOG, 0, V <= 2><<<ws.n_big * p.ch, bulk_tpb(2, DOK_KF_U64, 0), 0, s>>>(d, nullptr, nullptr, n, ws);
    else bulk_scatter_kernel<V, DOK_KF_U64, 2><<<ws.n_big * p.ch, bulk_tpb(2, DOK_KF_U64, 0), 0, s>>>(d, nullptr, nullptr, n, ws);
  } else {
    bulk_scatter_kernel<V, DOK_KF_U64, 2, DOK_BULK_SUBLOG_WIDE><<<ws.n_big * p.ch, bulk_tpb(2, DOK_KF_U64, 0), 0, s>>>(d, nullptr, nullptr, n, ws);
  }
  const u32 gm = ws.n_part < p.gm ? ws.n_part : p.gm;
  bulk_merge_kernel<V, FRESH><<<gm, DOK_BULK_R, 0, s>>>(d, ws);
  if (gm > 1) bulk_edge_kernel<V><<<gm, DOK_BULK_R, 0, s>>>(d, ws);
  bulk_deferred_kernel<V><<<gm, DOK_TPB, 0, s>>>(d, ws);
  }
}

template <int V, int KF, bool FRESH = false>
static void bulk_launch(const DevTable &d, const void *keys, const void *values, i64 n, const BulkPlan &p,
                        void *workspace, hipStream_t s) {
  if constexpr (KF == DOK_KF_COLS || KF == DOK_KF_ROWS) {
    switch (d.lin_ndim) {                              // 1 .. DOK_LIN_DIMS, checked with the descriptor
      case 1: return bulk_launch_nd<V, KF, 1, FRESH>(d, keys, values, n, p, workspace, s);
      case 2: return bulk_launch_nd<V, KF, 2, FRESH>(d, keys, values, n, p, workspace, s);
      case 3: return bulk_launch_nd<V, KF, 3, FRESH>(d, keys, values, n, p, workspace, s);
      case 4: return bulk_launch_nd<V, KF, 4, FRESH>(d, keys, values, n, p, workspace, s);
      case 5: return bulk_launch_nd<V, KF, 5, FRESH>(d, keys, values, n, p, workspace, s);
      case 6: return bulk_launch_nd<V, KF, 6, FRESH>(d, keys, values, n, p, workspace, s);
      case 7: return bulk_launch_nd<V, KF, 7, FRESH>(d, keys, values, n, p, workspace, s);
      default: return bulk_launch_nd<V, KF, 8, FRESH>(d, keys, values, n, p, workspace, s);
    }
  } else {
    bulk_launch_nd<V, KF, 0, FRESH>(d, keys, values, n, p, workspace, s);
  }
}

// Bulk removal of n keys (key rows in the table's batch format; no per-row flags).
template <int V>
static void bulk_launch_remove(const DevTable &d, const void *keys, i64 n, const BulkPlan &p, void *workspace, hipStream_t s) {
  for (u32 win = 0; win < p.n_windows; win++) {
  BulkWs ws;
  bulk_bind(p, workspace, ws, win);
  bulk_init_kernel<<<64, DOK_TPB, 0, s>>>(ws, nullptr);
  // (the scatters move no values: their instantiation for one-byte values serves every table)
  if (d.lin_ndim == 0 && d.key_bytes == 8) {
    bulk_scatter_kernel<1, DOK_KF_U64, 1, DOK_BULK_SUBLOG, 0, false, true><<<p.g1, bulk_tpb(1, DOK_KF_U64, 0), 0, s>>>(d, keys, nullptr, n, ws);
  } else {
    const unsigned g = (unsigned)((n + DOK_TPB - 1) / DOK_TPB < 8192 ? (n + DOK_TPB - 1) / DOK_TPB : 8192);
    if (d.lin_ndim > 0) bulk_keys_to_words_kernel<DOK_KF_ROWS><<<g, DOK_TPB, 0, s>>>(d, keys, n, ws);
    else bulk_keys_to_words_kernel<DOK_KF_RAW><<<g, DOK_TPB, 0, s>>>(d, keys, n, ws);
    bulk_scatter_kernel<1, DOK_KF_LIN, 1, DOK_BULK_SUBLOG, 0, false, true><<<p.g1, bulk_tpb(1, DOK_KF_LIN, 0), 0, s>>>(d, ws.keysB, nullptr, n, ws);
  }
  if (p.sublog == DOK_BULK_SUBLOG)
    bulk_scatter_kernel<1, DOK_KF_U64, 2, DOK_BULK_SUBLOG, 0, false, true><<<ws.n_big * p.ch, bulk_tpb(2, DOK_KF_U64, 0), 0, s>>>(d, nullptr, nullptr, n, ws);
  else
    bulk_scatter_kernel<1, DOK_KF_U64, 2, DOK_BULK_SUBLOG_WIDE, 0, false, true><<<ws.n_big * p.ch, bulk_tpb(2, DOK_KF_U64, 0), 0, s>>>(d, nullptr, nullptr, n, ws);
  const u32 grid = ws.n_part < 2048u ? ws.n_part : 2048u;
  bulk_remove_kernel<V><<<grid, DOK_TPB, 0, s>>>(d, ws);
  bulk_remove_spill_kernel<V><<<256, DOK_TPB, 0, s>>>(d, ws);
  }
}
