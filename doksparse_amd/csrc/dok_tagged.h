// Tagged layout: keys and values of any width with 8*(1 + ceil(K/8) + ceil(V/8)) <= 128.
//
// A slot is W = 1 + KW + VW consecutive 8-byte words of a bucket:
//     word 0            tag / lock word   (the only word ever CAS'd)
//     words 1 .. KW     the key bytes, zero padded to 8*KW
//     then VW words     the value bytes, zero padded to 8*VW
// and a 128-byte bucket holds S = 16 / W slots.  Tag values:
//     0                  EMPTY
//     1                  TOMBSTONE
//     (h & ~3) | 2       BUSY: claimed by a writer of a key whose 62-bit tag hash is h; key and
//                        value words are being written
//     (h & ~3) | 3       FULL: key and value words are valid
// Identity is always the full key: a tag match only selects the slots whose key words are then
// compared, lane-parallel, against the query (each lane of the group holds one word of the
// bucket and compares it with the word it should be).
//
// Query keys are staged in LDS as zero-padded words, one row per thread of the workgroup, so
// that any lane of a group can fetch "word p of the row being served".
#pragma once
#include "dok_device.h"

#define DOK_TG_EMPTY 0ULL
#define DOK_TG_TOMB  1ULL
#define DOK_TG_MAXW  15
// Ordering of "write the slot's key and value words" before "publish the FULL tag".  The data
// words are written with agent-scope atomic stores, which gfx950 performs write-through to the
// level every XCD shares; what remains to be ensured is that those stores have completed before
// the tag store is issued, i.e. a wait for the wave's outstanding memory operations.  A
// workgroup-scope release fence compiles to exactly that wait.  (An agent-scope release fence
// adds a write-back of the whole L2, which exists for plain stores - there are none here - and
// costs ten times the kernel's run time when issued once per inserted row.)
#ifndef DOK_TG_RELEASE
#define DOK_TG_RELEASE() __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup")
#endif

struct TgGeom {
  int KW, VW, W, S;
  int K, V;
  int unit_k, unit_v;      // largest power of two (<= 8) dividing K resp. V: the access granule
  u64 fallback[DOK_TG_MAXW];
};

// Word k (8 bytes, zero padded past `nbytes`) of a byte row whose address is `unit`-aligned.
__device__ __forceinline__ u64 tg_load_word(const u8 *row, int k, int nbytes, int unit) {
  const int base = 8 * k;
  u64 w = 0;
  if (unit == 8) {
    w = *(const u64 *)(row + base);
  } else if (unit == 4) {
    w = *(const u32 *)(row + base);
    if (base + 4 < nbytes) w |= (u64)(*(const u32 *)(row + base + 4)) << 32;
  } else if (unit == 2) {
    for (int q = 0; q < 4; q++)
      if (base + 2 * q < nbytes) w |= (u64)(*(const u16 *)(row + base + 2 * q)) << (16 * q);
  } else {
    for (int q = 0; q < 8; q++)
      if (base + q < nbytes) w |= (u64)row[base + q] << (8 * q);
  }
  return w;
}

__device__ __forceinline__ void tg_store_word(u8 *row, int k, int nbytes, int unit, u64 w) {
  const int base = 8 * k;
  if (unit == 8) {
    *(u64 *)(row + base) = w;
  } else if (unit == 4) {
    *(u32 *)(row + base) = (u32)w;
    if (base + 4 < nbytes) *(u32 *)(row + base + 4) = (u32)(w >> 32);
  } else if (unit == 2) {
    for (int q = 0; q < 4; q++)
      if (base + 2 * q < nbytes) *(u16 *)(row + base + 2 * q) = (u16)(w >> (16 * q));
  } else {
    for (int q = 0; q < 8; q++)
      if (base + q < nbytes) row[base + q] = (u8)(w >> (8 * q));
  }
}

// Per-thread preparation shared by all tagged batch kernels: stage the row's key words in LDS,
// hash them, derive the home bucket and the FULL tag.
__device__ __forceinline__ void tg_stage(const DevTable &t, const TgGeom &g, const u8 *keys, i64 i,
                                         bool active, u64 *lds_keys, u32 &home, u64 &tag_full) {
  u64 h = t.seed;
  const u8 *row = keys + (size_t)i * g.K;
  for (int k = 0; k < g.KW; k++) {
    const u64 w = active ? tg_load_word(row, k, g.K, g.unit_k) : 0;
    lds_keys[threadIdx.x * g.KW + k] = w;
    h = dok_fmix64(h ^ w) + 0x9E3779B97F4A7C15ULL * (u64)(k + 1);
  }
  const u64 h1 = dok_fmix64(h);
  home = dok_reduce(h1, t.nb);
  tag_full = (dok_fmix64(h1 ^ 0xD6E8FEB86659FD93ULL) & ~3ULL) | 3ULL;
}

// Lane geometry inside a 16-lane group.
struct TgLane {
  int lane, gbase, l, slot, p;
  bool valid, is_tag, is_key, is_val;
  u32 slotmask;
  __device__ __forceinline__ TgLane(const TgGeom &g) {
    lane = threadIdx.x & 63;
    gbase = lane & 48;
    l = lane & 15;
    slot = l / g.W;
    p = l - slot * g.W;
    valid = slot < g.S;
    is_tag = valid && p == 0;
    is_key = valid && p >= 1 && p <= g.KW;
    is_val = valid && p > g.KW;
    slotmask = ((1u << g.W) - 1u) << (slot * g.W);
  }
};

// Group-wide view of one bucket for the row being served.
struct TgView {
  u32 hit;      // bit at the tag lane of every slot that is FULL with this row's key
  u32 tagonly;  // bit at the tag lane of every slot whose tag equals the row's FULL tag
  u32 busy;     // ... whose tag is the row's BUSY tag
  u32 empty, tomb;
};

__device__ __forceinline__ TgView tg_inspect(const TgGeom &g, const TgLane &L, bool has, u64 w,
                                             u64 qfull, const u64 *lds_row) {
  u64 expect = qfull;
  if (L.is_key) expect = lds_row[L.p - 1];
  const bool eq = L.valid && (L.is_val || w == expect);
  const u32 geq = (u32)(dok_ballot(has && eq) >> L.gbase) & 0xffffu;
  const bool slot_hit = L.valid && ((geq & L.slotmask) == L.slotmask);
  TgView v;
  v.hit = (u32)(dok_ballot(has && slot_hit && L.is_tag) >> L.gbase) & 0xffffu;
  v.tagonly = (u32)(dok_ballot(has && L.is_tag && w == qfull) >> L.gbase) & 0xffffu;
  v.busy = (u32)(dok_ballot(has && L.is_tag && w == (qfull & ~1ULL)) >> L.gbase) & 0xffffu;
  v.empty = (u32)(dok_ballot(has && L.is_tag && w == DOK_TG_EMPTY) >> L.gbase) & 0xffffu;
  v.tomb = (u32)(dok_ballot(has && L.is_tag && w == DOK_TG_TOMB) >> L.gbase) & 0xffffu;
  return v;
}

// mode 0: get (write value or fallback + flag), 1: count, 2: remove.
// Rows are taken in tiles of DOK_TPB (see DOK_TILE_LOOP); a wave only ever reads the LDS rows its
// own lanes staged, so the tiles need no workgroup barrier between them.
template <int MODE, bool STATS>
__global__ __launch_bounds__(DOK_TPB) void tg_lookup_kernel(DevTable t, TgGeom g, const u8 *__restrict__ keys, i64 n,
                                                            u8 *__restrict__ values, u8 *__restrict__ flags,
                                                            i64 *count) {
  extern __shared__ u64 lds[];
  u64 *lds_keys = lds;                          // [DOK_TPB][KW]
  u64 *lds_fb = lds + DOK_TPB * g.KW;           // [VW]
  if (MODE == 0 && threadIdx.x < g.VW) lds_fb[threadIdx.x] = g.fallback[threadIdx.x];
  __syncthreads();
  const TgLane L(g);
  const int wave_row0 = threadIdx.x & ~63;      // first LDS row of this wave
  int n_found = 0, n_removed = 0, n_probe = 0, n_ops = 0;

  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool active = i < n;
    u32 b; u64 tag_full;
    tg_stage(t, g, keys, i, active, lds_keys, b, tag_full);
    const i64 wave_i0 = i - L.lane;             // batch row of lane 0
    bool pend = active, found = false, removed = false;
    u64 iters = 0;

    u64 pm = dok_ballot(pend);
    while (pm != 0) {
      const u32 sub = (u32)(pm >> L.gbase) & 0xffffu;
      const bool has = sub != 0;
      const int r = has ? __builtin_ctz(sub) : 0;
      const int j = L.gbase + r;
      const u32 qb = dok_shfl32(b, j);
      const u64 qfull = dok_shfl64(tag_full, j);
      const u64 w = t.buckets[(u64)(has ? qb : 0u) * 16 + L.l];
      const TgView v = tg_inspect(g, L, has, w, qfull, lds_keys + (wave_row0 + j) * g.KW);
      const bool resolved = v.hit != 0 || v.empty != 0;
      if (MODE == 0 && has && resolved) {
        // the value lanes of the matching slot (or, on a miss, of slot 0 with the fallback)
        // write the output row directly
        const int hit_slot = v.hit ? (__builtin_ctz(v.hit) / g.W) : 0;
        if (L.is_val && L.slot == hit_slot) {
          const int k = L.p - 1 - g.KW;
          const u64 word = v.hit ? w : lds_fb[k];
          tg_store_word(values + (size_t)(wave_i0 + j) * g.V, k, g.V, g.unit_v, word);
        }
      }
      if (has && L.l == r) {
        n_probe++;
        if (v.hit) {
          found = true; pend = false;
          if (MODE == 2) {
            u64 *tagp = t.buckets + (u64)b * 16 + __builtin_ctz(v.hit);
            removed = atomicCAS(tagp, qfull, DOK_TG_TOMB) == qfull;
          }
        } else if (v.empty) {
          pend = false;
        } else {
          b = (b + 1 == t.nb) ? 0u : b + 1;
          if (++iters >= t.nb) {
            pend = false;
            if (MODE == 0) {
              // full ring without an empty slot: absent; the owner writes the fallback itself
              for (int k = 0; k < g.VW; k++)
                tg_store_word(values + (size_t)i * g.V, k, g.V, g.unit_v, lds_fb[k]);
            }
          }
        }
      }
      pm = dok_ballot(pend);
    }
    if (MODE == 0 && active) flags[i] = found ? 1 : 0;
    if (MODE == 2 && active && flags) flags[i] = removed ? 1 : 0;
    n_found += found;
    n_removed += removed;
    n_ops += active;
  }
  if (MODE == 1) dok_wave_add_n(count, n_found);
  if (MODE == 2) dok_wave_add_n(&t.header[DOK_H_NELEM], -n_removed);
  if (STATS) {
    dok_wave_add_n(&t.header[DOK_H_NPROBE], n_probe);
    dok_wave_add_n(&t.header[DOK_H_NOPS], n_ops);
  }
}

// Upsert.  Protocol per row (owner lane acts, the group inspects):
//   * slot FULL with the row's key  -> lock it (CAS FULL->BUSY), rewrite the value words,
//     publish FULL again.  Losing that CAS means an equal key of this batch holds the lock:
//     its value stands and this row is done.
//   * a slot BUSY with the row's tag -> its key is not readable yet: look again next turn.
//   * a slot FULL with the row's tag but other key words -> look once more after an acquire
//     fence (the key words may have been read before the writer's stores landed); a second
//     mismatch is a genuine tag collision and the slot is skipped.
//   * chain end (bucket with an EMPTY slot, or the ring walked) -> claim the first tombstone
//     seen, else the first empty slot: CAS ->BUSY, write key and value words, release fence,
//     publish FULL.  Losing the claim restarts the walk from the home bucket.
// A BUSY holder finishes in straight-line code inside one loop turn, so waiting rows always
// see it released.
__global__ __launch_bounds__(DOK_TPB) void tg_set_kernel(DevTable t, TgGeom g, const u8 *__restrict__ keys,
                                                         const u8 *__restrict__ values, i64 n,
                                                         u8 *__restrict__ stored) {
  extern __shared__ u64 lds[];
  u64 *lds_keys = lds;
  const TgLane L(g);
  const int wave_row0 = threadIdx.x & ~63;
  const u64 *krow = lds_keys + threadIdx.x * g.KW;
  int n_fresh = 0, n_full = 0;

  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool active = i < n;
    u32 home; u64 tag_full;
    tg_stage(t, g, keys, i, active, lds_keys, home, tag_full);
    u32 b = home, tomb_b = DOK_NONE32;
    int tomb_w = 0;
    bool pend = active, confirm = false;
    int st = 0, fresh = 0;
    u64 iters = 0;
    const u8 *vrow = values + (size_t)i * g.V;

    // Turns: in every turn the current bucket of EVERY pending row of the wave is inspected (the
    // loads of eight rows per group in flight together), then all owner lanes act at once - the
    // claims, the slot writes and the publishing stores of a whole wave overlap instead of
    // following one another row by row.  The first turn looks at the home buckets and settles
    // most rows; rows that walk on (bucket full, a lost claim, a slot that is being written, a
    // tag collision) stay pending for the next turn.
    u64 pm = dok_ballot(pend);
    while (pm != 0) {
      if (dok_ballot(confirm) != 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      const u32 sub = (u32)(pm >> L.gbase) & 0xffffu;          // this group's pending rows
      u32 any = (u32)pm | (u32)(pm >> 32);
      any = (any | (any >> 16)) & 0xffffu;                      // row numbers pending in some group
      TgView v;
      v.hit = v.tagonly = v.busy = v.empty = v.tomb = 0;
      #pragma unroll
      for (int r0 = 0; r0 < 16; r0 += 8) {
        if (((any >> r0) & 0xffu) == 0) continue;
        u64 w[8];
        #pragma unroll
        for (int u = 0; u < 8; u++) {
          const u32 qb = dok_shfl32(b, L.gbase + r0 + u);
          w[u] = 0;
          if ((sub >> (r0 + u)) & 1u) w[u] = dok_load_coherent(t.buckets + (u64)qb * 16 + L.l);
        }
        #pragma unroll
        for (int u = 0; u < 8; u++) {
          if (!((any >> (r0 + u)) & 1u)) continue;
          const int j = L.gbase + r0 + u;
          const u64 qfull = dok_shfl64(tag_full, j);
          const TgView x = tg_inspect(g, L, ((sub >> (r0 + u)) & 1u) != 0, w[u], qfull, lds_keys + (wave_row0 + j) * g.KW);
          if (L.l == r0 + u) v = x;
        }
      }
      if (pend) {
        u64 *bucket = t.buckets + (u64)b * 16;
        const u64 qfull = tag_full, qbusy = tag_full & ~1ULL;
        if (v.hit) {
          u64 *slot = bucket + __builtin_ctz(v.hit);
          if (atomicCAS(slot, qfull, qbusy) == qfull) {
            for (int k = 0; k < g.VW; k++)
              dok_store_coherent(slot + 1 + g.KW + k, tg_load_word(vrow, k, g.V, g.unit_v));
            DOK_TG_RELEASE();
            dok_store_coherent(slot, qfull);
          }
          st = 1; pend = false;
        } else if (v.busy) {
          // wait for the holder to publish
        } else if ((v.tagonly & ~v.hit) != 0 && !confirm) {
          confirm = true;
        } else {
          confirm = false;
          if (tomb_b == DOK_NONE32 && v.tomb) { tomb_b = b; tomb_w = __builtin_ctz(v.tomb); }
          const bool ring_done = (v.empty == 0) && (++iters >= t.nb);
          if (v.empty || ring_done) {
            if (tomb_b == DOK_NONE32 && v.empty == 0) {
              st = 0; pend = false;                         // no free slot anywhere
            } else {
              u64 *slot; u64 expect;
              if (tomb_b != DOK_NONE32) { slot = t.buckets + (u64)tomb_b * 16 + tomb_w; expect = DOK_TG_TOMB; }
              else { slot = bucket + __builtin_ctz(v.empty); expect = DOK_TG_EMPTY; }
              if (atomicCAS(slot, expect, qbusy) == expect) {
                for (int k = 0; k < g.KW; k++) dok_store_coherent(slot + 1 + k, krow[k]);
                for (int k = 0; k < g.VW; k++)
                  dok_store_coherent(slot + 1 + g.KW + k, tg_load_word(vrow, k, g.V, g.unit_v));
                DOK_TG_RELEASE();
                dok_store_coherent(slot, qfull);
                st = 1; fresh = 1; pend = false;
              } else {
                b = home; tomb_b = DOK_NONE32; iters = 0;   // lost the claim: walk again
              }
            }
          } else {
            b = (b + 1 == t.nb) ? 0u : b + 1;
          }
        }
      }
      pm = dok_ballot(pend);
    }
    if (active && stored) stored[i] = (u8)st;
    n_fresh += fresh;
    n_full += (active && st == 0);
  }
  dok_wave_add_n(&t.header[DOK_H_NELEM], n_fresh);
  dok_wave_add_n(&t.header[DOK_H_NFULL], n_full);
}

// ---- read-out ---------------------------------------------------------------------------------
#ifndef DOK_CHUNK
#define DOK_CHUNK 256
#endif

__device__ __forceinline__ bool tg_scan_load(const DevTable &t, const TgLane &L, i64 b, u64 &w) {
  const bool valid = b < (i64)t.nb;
  w = t.buckets[(u64)(valid ? b : (i64)t.nb - 1) * 16 + L.l];
  return valid && L.is_tag && (w & 3ULL) == 3ULL;
}

__global__ __launch_bounds__(DOK_TPB) void tg_chunk_count_kernel(DevTable t, TgGeom g, i64 *chunk_counts, i64 n_chunks) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const TgLane L(g);
  i64 cnt = 0;
  #pragma unroll 8
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live = tg_scan_load(t, L, wid * DOK_CHUNK + s * 4 + (L.lane >> 4), w);
    cnt += __popcll(dok_ballot(live));
  }
  if (L.lane == 0) chunk_counts[wid] = cnt;
}

__global__ __launch_bounds__(DOK_TPB) void tg_chunk_write_kernel(DevTable t, TgGeom g, const i64 *chunk_offsets,
                                                                 i64 n_chunks, u8 *keys_out, u8 *values_out, i64 cap) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const TgLane L(g);
  i64 base = chunk_offsets[wid];
  #pragma unroll 8
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live_tag = tg_scan_load(t, L, wid * DOK_CHUNK + s * 4 + (L.lane >> 4), w);
    const u64 m = dok_ballot(live_tag);
    // every lane of a live slot learns the slot's output row from the tag lane's position
    const int tag_lane = L.gbase + L.slot * g.W;
    const bool slot_live = L.valid && ((m >> tag_lane) & 1ULL);
    const i64 row = base + __popcll(m & ((1ULL << tag_lane) - 1ULL));
    if (slot_live && row < cap) {
      if (L.is_key && keys_out) tg_store_word(keys_out + (size_t)row * g.K, L.p - 1, g.K, g.unit_k, w);
      if (L.is_val && values_out) tg_store_word(values_out + (size_t)row * g.V, L.p - 1 - g.KW, g.V, g.unit_v, w);
    }
    base += __popcll(m);
  }
}

// ---- host launchers -----------------------------------------------------------------------------

static int tg_pow2_unit(int n) { return n % 8 == 0 ? 8 : n % 4 == 0 ? 4 : n % 2 == 0 ? 2 : 1; }

static int tg_geom(const DevTable &d, const void *fallback, TgGeom &g) {
  memset(&g, 0, sizeof(g));
  g.K = d.key_bytes; g.V = d.value_bytes;
  g.KW = (g.K + 7) / 8; g.VW = (g.V + 7) / 8;
  g.W = 1 + g.KW + g.VW;
  if (g.W > 16) return DOK_EUNSUPPORTED;
  g.S = 16 / g.W;
  g.unit_k = tg_pow2_unit(g.K);
  g.unit_v = tg_pow2_unit(g.V);
  if (fallback) memcpy(g.fallback, fallback, g.V);
  return DOK_OK;
}

static bool tg_aligned(const void *p, int unit) { return ((uintptr_t)p & (uintptr_t)(unit - 1)) == 0; }

static size_t tg_lds_bytes(const TgGeom &g) { return (size_t)(DOK_TPB * g.KW + g.VW) * 8; }

static int tg_launch_get(const DevTable &d, const void *keys, i64 n, void *values, const void *fallback,
                         u8 *found, bool stats, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, fallback, g);
  if (rc) return rc;
  if (!tg_aligned(keys, g.unit_k) || !tg_aligned(values, g.unit_v)) return DOK_EINVAL;
  const unsigned grid = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  const unsigned cgrid = grid < 2048u ? grid : 2048u;
  if (stats)
    tg_lookup_kernel<0, true><<<cgrid, DOK_TPB, tg_lds_bytes(g), s>>>(d, g, (const u8 *)keys, n, (u8 *)values, found, nullptr);
  else
    tg_lookup_kernel<0, false><<<grid, DOK_TPB, tg_lds_bytes(g), s>>>(d, g, (const u8 *)keys, n, (u8 *)values, found, nullptr);
  return DOK_OK;
}

// Most workgroups of the kernels that loop over tiles and end with one atomic per wave on a
// counter.  Few workgroups keep those atomics cheap (same-address atomics serialise at ~12 ns
// each), many even out the long probe chains of a loaded table; measured on 32M float32[3] ->
// int64[5] rows at load factors 0.5 / 0.9: count 1.58 / 10.2 ms with 2048 workgroups,
// 1.46 / 5.6 ms with 8192; set 9.6 / 22.7 ms with 2048, 9.0 / 15.4 ms with 32768; remove of 8M
// 0.68 / 1.10 ms with 2048, 1.65 / 2.35 ms with 32768.
#ifndef DOK_TG_COUNT_GRID
#define DOK_TG_COUNT_GRID 8192u
#endif
#ifndef DOK_TG_REMOVE_GRID
#define DOK_TG_REMOVE_GRID 2048u
#endif
#ifndef DOK_TG_SET_GRID
#define DOK_TG_SET_GRID 32768u
#endif
static int tg_launch_count(const DevTable &d, const void *keys, i64 n, i64 *count, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  if (!tg_aligned(keys, g.unit_k)) return DOK_EINVAL;
  const unsigned grid = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  tg_lookup_kernel<1, false><<<(grid < DOK_TG_COUNT_GRID ? grid : DOK_TG_COUNT_GRID), DOK_TPB, tg_lds_bytes(g), s>>>(d, g, (const u8 *)keys, n, nullptr, nullptr, count);
  return DOK_OK;
}

static int tg_launch_remove(const DevTable &d, const void *keys, i64 n, u8 *removed, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  if (!tg_aligned(keys, g.unit_k)) return DOK_EINVAL;
  const unsigned grid = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  tg_lookup_kernel<2, false><<<(grid < DOK_TG_REMOVE_GRID ? grid : DOK_TG_REMOVE_GRID), DOK_TPB, tg_lds_bytes(g), s>>>(d, g, (const u8 *)keys, n, nullptr, removed, nullptr);
  return DOK_OK;
}

static int tg_launch_set(const DevTable &d, const void *keys, const void *values, i64 n, u8 *stored, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  if (!tg_aligned(keys, g.unit_k) || !tg_aligned(values, g.unit_v)) return DOK_EINVAL;
  const unsigned grid = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  tg_set_kernel<<<(grid < DOK_TG_SET_GRID ? grid : DOK_TG_SET_GRID), DOK_TPB, tg_lds_bytes(g), s>>>(d, g, (const u8 *)keys, (const u8 *)values, n, stored);
  return DOK_OK;
}

static int tg_launch_compact(const DevTable &d, i64 *offs, i64 n_chunks, void *keys_out, void *values_out,
                             i64 cap, i64 *count_out, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  if ((keys_out && !tg_aligned(keys_out, g.unit_k)) || (values_out && !tg_aligned(values_out, g.unit_v)))
    return DOK_EINVAL;
  const unsigned grid = (unsigned)((n_chunks + 3) / 4);
  tg_chunk_count_kernel<<<grid, DOK_TPB, 0, s>>>(d, g, offs, n_chunks);
  dok_scan_kernel<<<1, 1024, 0, s>>>(offs, n_chunks, nullptr, count_out);
  if (keys_out || values_out)
    tg_chunk_write_kernel<<<grid, DOK_TPB, 0, s>>>(d, g, offs, n_chunks, (u8 *)keys_out, (u8 *)values_out, cap);
  return DOK_OK;
}
