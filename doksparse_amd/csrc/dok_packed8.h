// Packed layout: keys of at most 8 bytes, values of 1, 2, 4 or 8 bytes.
//
// A 128-byte bucket holds S = 128 / (8 + V) slots:
//     words 0 .. S-1           the S stored key words (8 bytes each)
//     bytes 8*S .. 8*S + V*S   the S values, value s at byte 8*S + V*s
// (V=4: 10 slots, V=8: 8, V=2: 12, V=1: 14).  The stored key word is  key XOR DOK_P8_XOR,
// and the two words 0 and 1 mean EMPTY and TOMBSTONE, so a cleared table is all zero bytes and
// the slot word itself is the target of the claiming 64-bit compare-and-swap: an insert is one
// CAS plus one value store into the same line.  The two keys whose stored word would be 0 or 1
// live in two side slots of the table header instead (state word + value word each).
//
// Probing is linear over buckets.  A chain ends at the first bucket that still has an EMPTY
// slot; a bucket never regains an EMPTY slot (remove leaves a TOMBSTONE), so a key that was
// placed past a full bucket stays reachable.
#pragma once
#include "dok_device.h"

#define DOK_P8_XOR   0x9E3779B97F4A7C15ULL
#define DOK_P8_EMPTY 0ULL
#define DOK_P8_TOMB  1ULL
#define DOK_H_SIDE_STATE 8    // header words 8,9: side slot occupied (0/1)
#define DOK_H_SIDE_VALUE 10   // header words 10,11: side slot values

template <int V> struct P8 {
  static constexpr int S = 128 / (8 + V);
  __device__ static __forceinline__ u64 extract(u64 vword, int s) {
    if (V == 8) return vword;
    return (vword >> (((s * V) & 7) * 8)) & ((1ULL << (8 * (V & 7))) - 1ULL);
  }
  __device__ static __forceinline__ int value_word(int s) { return S + ((s * V) >> 3); }
  __device__ static __forceinline__ void store(u64 *bucket, int s, u64 v) {
    typedef typename ValT<V>::type T;
    *(T *)((char *)bucket + 8 * S + V * s) = (T)v;
  }
};

__device__ __forceinline__ u32 p8_home(u64 sk, const DevTable &t) {
  return dok_reduce(dok_fmix64(sk ^ t.seed), t.nb);
}

// ---- cooperative lookup -------------------------------------------------------------------
// In: per-lane stored key `sk`, home bucket `b`, `pend` (row needs a table probe).
// Out: found / value for the lane's own row; slot_b / slot_s locate the matching slot;
// nprobe counts the buckets visited for the lane's row.
//
// Phase 1 serves the home bucket of each of the group's 16 rows.  It is written as "issue U
// loads, then resolve U rounds" with no branch in between, so that a wave keeps U*4 bucket
// lines in flight; everything a round decides is folded into the owner lane with selects.
// Phase 2 walks the few rows whose home bucket was full and held no match, one row per group
// per turn.
#define DOK_P8_U 8
template <int V>
__device__ __forceinline__ void p8_lookup(const u64 *__restrict__ buckets, u64 nb, u64 sk, u32 b,
                                          bool pend, bool &found, u64 &val, u32 &slot_b,
                                          int &slot_s, int &nprobe) {
  constexpr int S = P8<V>::S;
  const int lane = threadIdx.x & 63;
  const int gbase = lane & 48;
  const int l = lane & 15;
  const bool inb = l < S;
  const u32 home = b;
  slot_b = home;

  const u64 pend0 = dok_ballot(pend);
  if (pend0 != 0) {
    const u32 gp = (u32)(pend0 >> gbase) & 0xffffu;      // pending rows of this group
    #pragma unroll
    for (int r0 = 0; r0 < 16; r0 += DOK_P8_U) {
      u64 w[DOK_P8_U];
      #pragma unroll
      for (int u = 0; u < DOK_P8_U; u++) {
        const int r = r0 + u;
        const u32 qb = dok_shfl32(home, gbase + r);
        const bool has = (gp >> r) & 1u;
        w[u] = buckets[(u64)(has ? qb : 0u) * 16 + l];
      }
      #pragma unroll
      for (int u = 0; u < DOK_P8_U; u++) {
        const int r = r0 + u;
        const bool has = (gp >> r) & 1u;
        const u64 q = dok_shfl64(sk, gbase + r);
        const u64 bm = dok_ballot(has && inb && w[u] == q);
        const u64 be = dok_ballot(has && inb && w[u] == DOK_P8_EMPTY);
        const u32 gm = (u32)(bm >> gbase) & 0xffffu;
        const u32 ge = (u32)(be >> gbase) & 0xffffu;
        const int s = gm ? __builtin_ctz(gm) : 0;
        const u64 vword = dok_shfl64(w[u], gbase + P8<V>::value_word(s));
        const bool mine = has && l == r;
        const bool hit = mine && gm != 0;
        found = found || hit;
        val = hit ? P8<V>::extract(vword, s) : val;
        slot_s = hit ? s : slot_s;
        pend = pend && !(mine && (gm | ge) != 0);
      }
    }
  }
  nprobe += (pend0 >> lane) & 1ULL;

  // Phase 2
  u64 iters = 1;
  if (pend) b = (home + 1 == nb) ? 0u : home + 1;
  if (pend && nb == 1) pend = false;
  u64 pm = dok_ballot(pend);
  while (pm != 0) {
    const u32 sub = (u32)(pm >> gbase) & 0xffffu;
    const bool has = sub != 0;
    const int r = has ? __builtin_ctz(sub) : 0;
    const int j = gbase + r;
    const u64 q = dok_shfl64(sk, j);
    const u32 qb = dok_shfl32(b, j);
    const u64 w = buckets[(u64)(has ? qb : 0u) * 16 + l];
    const u64 bm = dok_ballot(has && inb && w == q);
    const u64 be = dok_ballot(has && inb && w == DOK_P8_EMPTY);
    const u32 gm = (u32)(bm >> gbase) & 0xffffu;
    const u32 ge = (u32)(be >> gbase) & 0xffffu;
    const int s = gm ? __builtin_ctz(gm) : 0;
    const u64 vword = dok_shfl64(w, gbase + P8<V>::value_word(s));
    if (has && l == r) {
      nprobe++;
      if (gm) {
        found = true; val = P8<V>::extract(vword, s); slot_b = b; slot_s = s; pend = false;
      } else if (ge) {
        pend = false;
      } else {
        b = (b + 1 == nb) ? 0u : b + 1;
        if (++iters >= nb) pend = false;      // walked the whole ring: absent
      }
    }
    pm = dok_ballot(pend);
  }
}

// Side-slot lookup for the two reserved stored words.
__device__ __forceinline__ bool p8_side_get(const DevTable &t, u64 sk, u64 &val) {
  if (t.header[DOK_H_SIDE_STATE + sk] != 0) { val = (u64)t.header[DOK_H_SIDE_VALUE + sk]; return true; }
  return false;
}

// ---- cooperative upsert -------------------------------------------------------------------
// In: per-lane stored key, value, `pend`.  Out: st (1 placed / 0 table full), fresh (took a new
// slot).  All table reads are device-coherent: other workgroups insert into the same buckets
// during the kernel.  The claim is one CAS on the slot's key word; whoever loses re-examines:
// if the winner wrote the same key (equal keys inside one batch) the loser is done and the
// winner's value stands, otherwise it restarts from its home bucket.
template <int V>
__device__ __forceinline__ void p8_insert(u64 *buckets, u64 nb, u64 sk, u64 val, u32 home,
                                          bool pend, int &st, int &fresh) {
  constexpr int S = P8<V>::S;
  const int lane = threadIdx.x & 63;
  const int gbase = lane & 48;
  const int l = lane & 15;
  const bool inb = l < S;
  u32 b = home;
  u32 tomb_b = DOK_NONE32;
  int tomb_s = 0;
  u64 iters = 0;

  u64 pm = dok_ballot(pend);
  while (pm != 0) {
    const u32 sub = (u32)(pm >> gbase) & 0xffffu;
    const bool has = sub != 0;
    const int r = has ? __builtin_ctz(sub) : 0;
    const int j = gbase + r;
    const u64 q = dok_shfl64(sk, j);
    const u32 qb = dok_shfl32(b, j);
    const u64 w = dok_load_coherent(buckets + (u64)(has ? qb : 0u) * 16 + l);
    const u64 bm = dok_ballot(has && inb && w == q);
    const u64 be = dok_ballot(has && inb && w == DOK_P8_EMPTY);
    const u64 bt = dok_ballot(has && inb && w == DOK_P8_TOMB);
    const u32 gm = (u32)(bm >> gbase) & 0xffffu;
    const u32 ge = (u32)(be >> gbase) & 0xffffu;
    const u32 gt = (u32)(bt >> gbase) & 0xffffu;
    if (has && l == r) {
      if (gm) {
        // key present: overwrite its value in place
        P8<V>::store(buckets + (u64)b * 16, __builtin_ctz(gm), val);
        st = 1; pend = false;
      } else {
        if (tomb_b == DOK_NONE32 && gt) { tomb_b = b; tomb_s = __builtin_ctz(gt); }
        const bool ring_done = (ge == 0) && (++iters >= nb);
        if (ge || ring_done) {
          // chain end: the key is absent.  Take the first tombstone seen on the way, else the
          // first empty slot of this bucket.
          if (tomb_b == DOK_NONE32 && ge == 0) {
            st = 0; pend = false;                       // no free slot anywhere
          } else {
            u32 tb; int ts; u64 expect;
            if (tomb_b != DOK_NONE32) { tb = tomb_b; ts = tomb_s; expect = DOK_P8_TOMB; }
            else { tb = b; ts = __builtin_ctz(ge); expect = DOK_P8_EMPTY; }
            u64 *tp = buckets + (u64)tb * 16;
            const u64 old = atomicCAS(tp + ts, expect, sk);
            if (old == expect) {
              P8<V>::store(tp, ts, val);
              st = 1; fresh = 1; pend = false;
            } else if (old == sk) {
              st = 1; pend = false;                     // an equal key of this batch won the slot
            } else {
              b = home; tomb_b = DOK_NONE32; iters = 0; // somebody else's key: look again
            }
          }
        } else {
          b = (b + 1 == nb) ? 0u : b + 1;
        }
      }
    }
    pm = dok_ballot(pend);
  }
}

// Side-slot upsert for a reserved stored word.
__device__ __forceinline__ int p8_side_set(const DevTable &t, u64 sk, u64 val) {
  const u64 old = atomicExch((u64 *)&t.header[DOK_H_SIDE_STATE + sk], 1ULL);
  dok_store_coherent((u64 *)&t.header[DOK_H_SIDE_VALUE + sk], val);
  return old == 0;
}

// ---- kernels ------------------------------------------------------------------------------

template <int V, bool STATS>
__global__ __launch_bounds__(DOK_TPB) void p8_get_kernel(DevTable t, const void *__restrict__ keys, i64 n,
                                                         void *__restrict__ values, u8 *__restrict__ found_out,
                                                         u64 fallback) {
  const i64 i = (i64)blockIdx.x * DOK_TPB + threadIdx.x;
  const bool active = i < n;
  u64 key = 0;
  const bool ok = active && dok_load_key8(t, keys, i, key);
  const u64 sk = key ^ DOK_P8_XOR;
  bool found = false;
  u64 val = fallback;
  bool pend = ok;
  if (ok && sk < 2) { found = p8_side_get(t, sk, val); pend = false; }
  u32 sb = 0; int ss = 0, nprobe = 0;
  p8_lookup<V>(t.buckets, t.nb, sk, pend ? p8_home(sk, t) : 0u, pend, found, val, sb, ss, nprobe);
  if (active) {
    dok_store_val<V>(values, i, val);
    found_out[i] = found ? 1 : 0;
  }
  if (STATS) {
    dok_wave_add_n(&t.header[DOK_H_NPROBE], nprobe);
    dok_wave_add(&t.header[DOK_H_NOPS], active);
  }
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_set_kernel(DevTable t, const void *__restrict__ keys,
                                                         const void *__restrict__ values, i64 n,
                                                         u8 *__restrict__ stored) {
  const i64 i = (i64)blockIdx.x * DOK_TPB + threadIdx.x;
  const bool active = i < n;
  u64 key = 0;
  const bool ok = active && dok_load_key8(t, keys, i, key);
  const u64 sk = key ^ DOK_P8_XOR;
  const u64 val = ok ? dok_load_val<V>(values, i) : 0;
  int st = 0, fresh = 0;
  bool pend = ok;
  if (ok && sk < 2) { fresh = p8_side_set(t, sk, val); st = 1; pend = false; }
  p8_insert<V>(t.buckets, t.nb, sk, val, pend ? p8_home(sk, t) : 0u, pend, st, fresh);
  if (active && stored) stored[i] = (u8)st;
  dok_wave_add(&t.header[DOK_H_NELEM], fresh != 0);
  dok_wave_add(&t.header[DOK_H_NFULL], ok && st == 0);
  dok_wave_add(&t.header[DOK_H_NOOB], active && !ok);
}

// Tombstone the matching slot with a CAS so that equal keys in one batch remove it once.
template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_remove_kernel(DevTable t, const void *__restrict__ keys, i64 n,
                                                            u8 *__restrict__ removed_out) {
  const i64 i = (i64)blockIdx.x * DOK_TPB + threadIdx.x;
  const bool active = i < n;
  u64 key = 0;
  const bool ok = active && dok_load_key8(t, keys, i, key);
  const u64 sk = key ^ DOK_P8_XOR;
  bool found = false, removed = false;
  u64 val = 0;
  bool pend = ok;
  if (ok && sk < 2) {
    removed = atomicExch((u64 *)&t.header[DOK_H_SIDE_STATE + sk], 0ULL) != 0;
    pend = false;
  }
  u32 sb = 0; int ss = 0, nprobe = 0;
  p8_lookup<V>(t.buckets, t.nb, sk, pend ? p8_home(sk, t) : 0u, pend, found, val, sb, ss, nprobe);
  if (found) removed = atomicCAS(t.buckets + (u64)sb * 16 + ss, sk, DOK_P8_TOMB) == sk;
  if (active && removed_out) removed_out[i] = removed ? 1 : 0;
  dok_wave_add(&t.header[DOK_H_NELEM], removed, -1);
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_count_kernel(DevTable t, const void *__restrict__ keys, i64 n,
                                                           i64 *count) {
  const i64 i = (i64)blockIdx.x * DOK_TPB + threadIdx.x;
  const bool active = i < n;
  u64 key = 0;
  const bool ok = active && dok_load_key8(t, keys, i, key);
  const u64 sk = key ^ DOK_P8_XOR;
  bool found = false;
  u64 val = 0;
  bool pend = ok;
  if (ok && sk < 2) { found = p8_side_get(t, sk, val); pend = false; }
  u32 sb = 0; int ss = 0, nprobe = 0;
  p8_lookup<V>(t.buckets, t.nb, sk, pend ? p8_home(sk, t) : 0u, pend, found, val, sb, ss, nprobe);
  dok_wave_add(count, found);
}

// ---- table scans: read-out, rehash, densify ------------------------------------------------
// Each wave walks DOK_CHUNK consecutive buckets, four per step (one per 16-lane group), so the
// live entries of a chunk are met in slot order and a per-chunk prefix sum gives every entry a
// stable output row.
#define DOK_CHUNK 256

template <int V>
__device__ __forceinline__ bool p8_scan_load(const DevTable &t, i64 b, u64 &w) {
  const int l = threadIdx.x & 15;
  const bool valid = b < (i64)t.nb;
  w = valid ? t.buckets[(u64)b * 16 + l] : 0;
  return valid && l < P8<V>::S && w >= 2;
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_chunk_count_kernel(DevTable t, i64 *chunk_counts, i64 n_chunks) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const int lane = threadIdx.x & 63;
  i64 cnt = 0;
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live = p8_scan_load<V>(t, wid * DOK_CHUNK + s * 4 + (lane >> 4), w);
    cnt += __popcll(dok_ballot(live));
  }
  if (lane == 0) chunk_counts[wid] = cnt;
}

// Exclusive prefix sum of counts[0..n) in place by one workgroup; counts[n] receives the sum.
// total_out[0] = sum + number of occupied side slots.
__global__ __launch_bounds__(1024) void dok_scan_kernel(i64 *counts, i64 n, const i64 *header, i64 *total_out) {
  __shared__ i64 wsum[16];
  __shared__ i64 carry_s;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (i64 base = 0; base < n; base += 1024) {
    const i64 idx = base + tid;
    const i64 v = idx < n ? counts[idx] : 0;
    i64 inc = v;
    #pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const i64 up = __shfl_up(inc, o, 64);
      if (lane >= o) inc += up;
    }
    if (lane == 63) wsum[wv] = inc;
    __syncthreads();
    i64 wpre = 0;
    for (int k = 0; k < wv; k++) wpre += wsum[k];
    const i64 carry = carry_s;
    if (idx < n) counts[idx] = carry + wpre + inc - v;
    __syncthreads();
    if (tid == 1023) carry_s = carry + wpre + inc;
    __syncthreads();
  }
  if (tid == 0) {
    const i64 total = carry_s;
    counts[n] = total;
    i64 side = 0;
    if (header) side = (header[DOK_H_SIDE_STATE] != 0) + (header[DOK_H_SIDE_STATE + 1] != 0);
    total_out[0] = total + side;
  }
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_chunk_write_kernel(DevTable t, const i64 *chunk_offsets, i64 n_chunks,
                                                                 void *keys_out, void *values_out, i64 cap) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const int lane = threadIdx.x & 63;
  const int gbase = lane & 48, l = lane & 15;
  i64 base = chunk_offsets[wid];
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live = p8_scan_load<V>(t, wid * DOK_CHUNK + s * 4 + (lane >> 4), w);
    const u64 m = dok_ballot(live);
    const int vw = l < P8<V>::S ? P8<V>::value_word(l) : 15;
    const u64 vword = dok_shfl64(w, gbase + vw);
    const i64 row = base + __popcll(m & ((1ULL << lane) - 1ULL));
    if (live && row < cap) {
      if (keys_out) dok_store_key8(t, keys_out, row, w ^ DOK_P8_XOR);
      if (values_out) dok_store_val<V>(values_out, row, P8<V>::extract(vword, l));
    }
    base += __popcll(m);
  }
  // the two side slots come last
  if (wid == 0 && lane == 0 && t.lin_ndim == 0) {
    i64 row = chunk_offsets[n_chunks];
    for (u64 k = 0; k < 2; k++) {
      if (t.header[DOK_H_SIDE_STATE + k] != 0) {
        if (row < cap) {
          if (keys_out) dok_store_key8(t, keys_out, row, k ^ DOK_P8_XOR);
          if (values_out) dok_store_val<V>(values_out, row, (u64)t.header[DOK_H_SIDE_VALUE + k]);
        }
        row++;
      }
    }
  }
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_rehash_kernel(DevTable src, DevTable dst, i64 n_chunks) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const int lane = threadIdx.x & 63;
  const int gbase = lane & 48, l = lane & 15;
  int n_fresh = 0, n_full = 0;
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live = p8_scan_load<V>(src, wid * DOK_CHUNK + s * 4 + (lane >> 4), w);
    const int vw = l < P8<V>::S ? P8<V>::value_word(l) : 15;
    const u64 val = P8<V>::extract(dok_shfl64(w, gbase + vw), l);
    int st = 0, fresh = 0;
    p8_insert<V>(dst.buckets, dst.nb, w, val, live ? p8_home(w, dst) : 0u, live, st, fresh);
    n_fresh += fresh;
    n_full += (live && st == 0);
  }
  dok_wave_add_n(&dst.header[DOK_H_NELEM], n_fresh);
  dok_wave_add_n(&dst.header[DOK_H_NFULL], n_full);
  if (wid == 0 && lane == 0) {
    for (int k = 0; k < 2; k++) {
      if (src.header[DOK_H_SIDE_STATE + k] != 0) {
        dst.header[DOK_H_SIDE_STATE + k] = 1;
        dst.header[DOK_H_SIDE_VALUE + k] = src.header[DOK_H_SIDE_VALUE + k];
        atomicAdd((u64 *)&dst.header[DOK_H_NELEM], 1ULL);
      }
    }
  }
}

// dense[key] = value for every live entry of a coordinate-keyed table (key = row-major offset).
template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_to_dense_kernel(DevTable t, void *dense, i64 n_chunks, i64 volume) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const int lane = threadIdx.x & 63;
  const int gbase = lane & 48, l = lane & 15;
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live = p8_scan_load<V>(t, wid * DOK_CHUNK + s * 4 + (lane >> 4), w);
    const int vw = l < P8<V>::S ? P8<V>::value_word(l) : 15;
    const u64 vword = dok_shfl64(w, gbase + vw);
    const u64 key = w ^ DOK_P8_XOR;
    if (live && key < (u64)volume) dok_store_val<V>(dense, (i64)key, P8<V>::extract(vword, l));
  }
}

// ---- DOK indexing kernels: gather coordinate -> linear key -> table op ----------------------

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_getitem_kernel(DevTable t, DevIndex ix, void *__restrict__ out) {
  const i64 e = (i64)blockIdx.x * DOK_TPB + threadIdx.x;
  const bool active = e < ix.n_elems;
  u64 key = 0; i64 voff = 0;
  const bool ok = active && dok_gather_key(t, ix, e, key, voff);
  const u64 sk = key ^ DOK_P8_XOR;
  bool found = false;
  u64 val = 0;
  u32 sb = 0; int ss = 0, nprobe = 0;
  p8_lookup<V>(t.buckets, t.nb, sk, ok ? p8_home(sk, t) : 0u, ok, found, val, sb, ss, nprobe);
  if (active) dok_store_val<V>(out, e, val);
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_setitem_kernel(DevTable t, DevIndex ix) {
  const i64 e = (i64)blockIdx.x * DOK_TPB + threadIdx.x;
  const bool active = e < ix.n_elems;
  u64 key = 0; i64 voff = 0;
  const bool ok = active && dok_gather_key(t, ix, e, key, voff);
  const u64 sk = key ^ DOK_P8_XOR;
  const u64 val = ok ? dok_load_val<V>(ix.src, voff) : 0;
  int st = 0, fresh = 0;
  p8_insert<V>(t.buckets, t.nb, sk, val, ok ? p8_home(sk, t) : 0u, ok, st, fresh);
  dok_wave_add(&t.header[DOK_H_NELEM], fresh != 0);
  dok_wave_add(&t.header[DOK_H_NFULL], ok && st == 0);
  dok_wave_add(&t.header[DOK_H_NOOB], active && !ok);
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_countitems_kernel(DevTable t, DevIndex ix, i64 *count) {
  const i64 e = (i64)blockIdx.x * DOK_TPB + threadIdx.x;
  const bool active = e < ix.n_elems;
  u64 key = 0; i64 voff = 0;
  const bool ok = active && dok_gather_key(t, ix, e, key, voff);
  const u64 sk = key ^ DOK_P8_XOR;
  bool found = false;
  u64 val = 0;
  u32 sb = 0; int ss = 0, nprobe = 0;
  p8_lookup<V>(t.buckets, t.nb, sk, ok ? p8_home(sk, t) : 0u, ok, found, val, sb, ss, nprobe);
  dok_wave_add(count, found);
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_zeroitems_kernel(DevTable t, DevIndex ix) {
  const i64 e = (i64)blockIdx.x * DOK_TPB + threadIdx.x;
  const bool active = e < ix.n_elems;
  u64 key = 0; i64 voff = 0;
  const bool ok = active && dok_gather_key(t, ix, e, key, voff);
  const u64 sk = key ^ DOK_P8_XOR;
  bool found = false, removed = false;
  u64 val = 0;
  u32 sb = 0; int ss = 0, nprobe = 0;
  p8_lookup<V>(t.buckets, t.nb, sk, ok ? p8_home(sk, t) : 0u, ok, found, val, sb, ss, nprobe);
  if (found) removed = atomicCAS(t.buckets + (u64)sb * 16 + ss, sk, DOK_P8_TOMB) == sk;
  dok_wave_add(&t.header[DOK_H_NELEM], removed, -1);
}
