// Tagged layout: keys and values of any width with 8*(1 + ceil(K/8) + ceil(V/8)) <= 128.
//
// A slot is W = 1 + KW + VW consecutive 8-byte words of a bucket:
//     word 0            low half:  tag / lock (the only 32 bits ever CAS'd)
//                       high half: bucket metadata (slot 0 only, see below; zero elsewhere)
//     words 1 .. KW     the key bytes, zero padded to 8*KW
//     then VW words     the value bytes, zero padded to 8*VW
// and a 128-byte bucket holds S = 16 / W slots.  Tag values (32 bits):
//     0                  EMPTY
//     1                  TOMBSTONE
//     (f & ~3) | 2       BUSY: claimed by a writer of a key whose 30-bit fingerprint is f; key and
//                        value words are being written
//     (f & ~3) | 3       FULL: key and value words are valid
// Identity is always the full key: a tag match only selects the slots whose key words are then
// compared, lane-parallel, against the query (each lane of the group holds one word of the
// bucket and compares it with the word it should be).
//
// Metadata (high half of word 0 of the bucket) describes the keys whose HOME is this bucket, like
// the metadata word of the packed layout:
//     bits 1..23   displacement map: bit d set = some key was placed d buckets past this one
//     bit 0        a key was placed 24 or more buckets past this one ...
//     bits 24..31  ... and the largest such displacement, 255 standing for "255 or more"
// Buckets of two or more slots also keep a filter in the (otherwise unused) high half of slot 1's
// tag word: every key placed away from this bucket sets the one of 32 bits its hash selects.
// Placement is linear probing over buckets (first free slot of the walk, a tombstone before an
// EMPTY slot; a bucket never regains an EMPTY slot), so a lookup visits the home bucket and then
// exactly the marked displacements - independent loads, no chain walk; with no mark set, or with
// the key's filter bit clear, the home bucket alone decides a miss.  Only beyond 254 buckets does
// a lookup walk on until it meets a bucket with an EMPTY slot.
//
// The rows a wave works on are staged in LDS as zero-padded words, one row per thread of the
// workgroup, so that any lane of a group can fetch "word p of the row being served".
#pragma once
#include "dok_device.h"
#include "dok_packed8.h"

#define DOK_TG_EMPTY 0u
#define DOK_TG_TOMB  1u
#define DOK_TG_MAXW  15
#define DOK_TG_NEAR  23                  // displacements with a bit of their own
#define DOK_TG_NEARMASK 0x00fffffeu
#define DOK_TG_FARCAP 255u               // stored largest far displacement saturates here

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

// ---- where the rows of a batch come from ---------------------------------------------------------
// Every kernel of this layout stages the rows it works on in LDS (key words at krow[1 .. KW], value
// words at vrow[0 .. VW)); a *row source* says how row i gets there.  stage() returns 0 = a row,
// 1 = the row addresses nothing inside the table's coordinate space (set kernels count it in
// header[DOK_H_NOOB]; lookups treat it as absent), 2 = skip the row silently.  vrow may be NULL
// (lookups).  A table with lin_ndim > 0 holds int64 coordinate rows - the key format of the
// reference's SparseDOKTensor (sparse_dok_tensor.py:45-69) - and its sources check every
// coordinate against lin_dims.

// Key rows and value rows as contiguous byte rows: the batched map entry points.
struct TgRows {
  const u8 *keys, *values;
  __device__ __forceinline__ int stage(const DevTable &t, const TgGeom &g, i64 i, u64 *krow, u64 *vrow) const {
    const u8 *kin = keys + (size_t)i * g.K;
    for (int k = 0; k < g.KW; k++) krow[1 + k] = tg_load_word(kin, k, g.K, g.unit_k);
    if (vrow) {
      const u8 *vin = values + (size_t)i * g.V;
      for (int k = 0; k < g.VW; k++) vrow[k] = tg_load_word(vin, k, g.V, g.unit_v);
    }
    bool ok = true;
    for (int d = 0; d < t.lin_ndim; d++) ok = ok && krow[1 + d] < (u64)t.lin_dims[d];
    return ok ? 0 : 1;
  }
};

// Coordinates the way a COO tensor holds them: indices[d * n + i]; values[i] (coordinate tables).
struct TgCols {
  const i64 *indices;
  i64 n;
  const u8 *values;
  __device__ __forceinline__ int stage(const DevTable &t, const TgGeom &g, i64 i, u64 *krow, u64 *vrow) const {
    // (a coordinate lands in the row's LDS word as it arrives and is checked there: nothing depends on
    // a load before the last one has been issued)
    for (int d = 0; d < g.KW; d++) krow[1 + d] = (u64)indices[(i64)d * n + i];
    if (vrow)
      for (int k = 0; k < g.VW; k++) vrow[k] = tg_load_word(values + (size_t)i * g.V, k, g.V, g.unit_v);
    bool ok = true;
    for (int d = 0; d < g.KW; d++) ok = ok && krow[1 + d] < (u64)t.lin_dims[d];
    return ok ? 0 : 1;
  }
};

// Kernel-argument form of dok_index_t for tables of up to DOK_MAX_DIMS dimensions (+ optional
// source-value view, + the source entries of a sparse-valued scatter).
struct DevIndexW {
  int ndim, sel_ndim;
  i64 n_elems;
  i64 shape[DOK_MAX_DIMS];
  i64 estride[DOK_MAX_DIMS];       // C-contiguous strides of `shape`
  const i64 *sel[DOK_MAX_DIMS];    // NULL: the coordinate is sbase + offset itself
  i64 sbase[DOK_MAX_DIMS];
  i64 sstride[DOK_MAX_DIMS][DOK_MAX_DIMS];
  const void *src;
  i64 vstride[DOK_MAX_DIMS];
};

// The selectors applied: on entry krow[1 + d] holds the element offset into dimension d's selector,
// on exit the coordinate.  Four dimensions at a time, their loads issued before the first is used.
__device__ __forceinline__ bool tg_apply_selectors(const DevTable &t, const DevIndexW &ix, u64 *krow) {
  bool ok = true;
  for (int d0 = 0; d0 < ix.ndim; d0 += 4) {
    i64 c[4];
    #pragma unroll
    for (int u = 0; u < 4; u++) {
      c[u] = 0;
      if (d0 + u < ix.ndim) {
        const i64 off = (i64)krow[1 + d0 + u];
        const i64 *sp = ix.sel[d0 + u];
        c[u] = sp ? sp[off] : off;
      }
    }
    #pragma unroll
    for (int u = 0; u < 4; u++) {
      if (d0 + u < ix.ndim) {
        const i64 x = c[u] + ix.sbase[d0 + u];
        ok = ok && (u64)x < (u64)t.lin_dims[d0 + u];
        krow[1 + d0 + u] = (u64)x;
      }
    }
  }
  return ok;
}

// Element e of the broadcast index space of an indexing expression: the fused form of the
// reference's stack + transpose of the broadcast selectors (sparse_dok_tensor.py:302-311) and of the
// accessor arithmetic of its DOK kernels (tensor_accessor.cu:50-87).  e is unravelled over the index
// space; the offsets into the selectors accumulate in the row's own LDS words (the number of
// dimensions is a run-time value here, and registers cannot be indexed by one).
struct TgIndexSrc {
  DevIndexW ix;
  __device__ __forceinline__ int stage(const DevTable &t, const TgGeom &g, i64 e, u64 *krow, u64 *vrow) const {
    for (int d = 0; d < ix.ndim; d++) krow[1 + d] = 0;
    i64 vo = 0;
    u64 rem = (u64)e;
    const bool small = ix.n_elems <= 0x7fffffffLL;
    for (int j = 0; j < ix.sel_ndim; j++) {
      u64 q;
      if (small) { const u32 st = (u32)ix.estride[j]; const u32 q32 = (u32)rem / st; rem = (u32)rem - q32 * st; q = q32; }
      else { const u64 st = (u64)ix.estride[j]; q = rem / st; rem -= q * st; }
      vo += (i64)q * ix.vstride[j];
      for (int d = 0; d < ix.ndim; d++) {
        const i64 st = ix.sstride[d][j];
        if (st) krow[1 + d] += q * (u64)st;          // (most strides are 0: a selector varies along few axes)
      }
    }
    const bool ok = tg_apply_selectors(t, ix, krow);
    if (vrow) vrow[0] = tg_load_word((const u8 *)ix.src + (size_t)vo * g.V, 0, g.V, g.V);
    return ok ? 0 : 1;
  }
};

// Source entry k of a sparse-valued scatter: index vector src_indices[j * n_src + k] over the axes of
// the index space, value src_values[k]; entries that are zero under nonzero_mask are skipped
// (reference: sparse_dok_set_items_sparse_v1, sparse_dok_tensor_impl.cu:163-211).
struct TgSparseSrc {
  DevIndexW ix;
  const i64 *src_indices;
  const u8 *src_values;
  i64 n_src;
  u64 nonzero_mask;
  __device__ __forceinline__ int stage(const DevTable &t, const TgGeom &g, i64 k, u64 *krow, u64 *vrow) const {
    const u64 val = tg_load_word(src_values + (size_t)k * g.V, 0, g.V, g.V);
    if ((val & nonzero_mask) == 0) return 2;
    for (int d = 0; d < ix.ndim; d++) krow[1 + d] = 0;
    bool inside = true;
    for (int j = 0; j < ix.sel_ndim; j++) {
      const u64 q = (u64)src_indices[(i64)j * n_src + k];
      inside = inside && q < (u64)ix.shape[j];
      for (int d = 0; d < ix.ndim; d++) {
        const i64 st = ix.sstride[d][j];
        if (st) krow[1 + d] += q * (u64)st;
      }
    }
    if (!inside) return 1;                            // (before any selector is read at such an offset)
    if (vrow) vrow[0] = val;
    return tg_apply_selectors(t, ix, krow) ? 0 : 1;
  }
};

// LDS row of a staged batch row: word 0 = the row's FULL tag (low half), words 1 .. KW = the
// zero-padded key words - exactly what the tag lane and the key lanes of a matching slot hold, so
// lane p of a slot compares its bucket word with word p of the row.
__device__ __forceinline__ int tg_rs(const TgGeom &g) { return g.KW + 1; }

// Hash the key words already staged at krow[1 .. KW]; stores the FULL tag at krow[0].
__device__ __forceinline__ void tg_hash_row(const DevTable &t, const TgGeom &g, u64 *krow,
                                            u32 &home, u32 &tag_full) {
  u64 h = t.seed;
  for (int k = 0; k < g.KW; k++) h = dok_fmix64(h ^ krow[1 + k]) + 0x9E3779B97F4A7C15ULL * (u64)(k + 1);
  const u64 h1 = dok_fmix64(h);
  home = dok_reduce(h1, t.nb);                       // upper half of the hash
  tag_full = ((u32)h1 & ~3u) | 3u;                   // lower half
  krow[0] = (u64)tag_full;
}
// The key's bit in its home bucket's filter (from the fingerprint bits of its tag).
__device__ __forceinline__ u32 tg_fbit(u32 tag_full) { return 1u << ((tag_full >> 2) & 31u); }

// Lane geometry inside a 16-lane group.
struct TgLane {
  int lane, gbase, l, slot, p, tag_lane;
  bool valid, is_tag, is_key, is_val;
  bool upper; int sh;        // where the group's 16 ballot bits sit (see P8Lane)
  __device__ __forceinline__ TgLane(const TgGeom &g) {
    lane = threadIdx.x & 63;
    gbase = lane & 48;
    l = lane & 15;
    slot = l / g.W;
    p = l - slot * g.W;
    tag_lane = slot * g.W;
    valid = slot < g.S;
    is_tag = valid && p == 0;
    is_key = valid && p >= 1 && p <= g.KW;
    is_val = valid && p > g.KW;
    upper = lane >= 32;
    sh = lane & 16;
  }
  __device__ __forceinline__ u32 grp(u64 m) const {
    const u32 x = upper ? (u32)(m >> 32) : (u32)m;
    return (x >> sh) & 0xffffu;
  }
};

// Wave-uniform lane masks of the geometry, made once per kernel.
struct TgMasks {
  u64 tagm;      // valid tag lanes
  u64 notkey;    // every lane that is not a key lane
  u32 kmask;     // KW + 1 ones: the tag lane and the key lanes of one slot
  __device__ __forceinline__ TgMasks(const TgGeom &g, const TgLane &L) {
    tagm = dok_ballot(L.is_tag);
    notkey = ~dok_ballot(L.is_key);
    kmask = (1u << (g.KW + 1)) - 1u;
  }
};

// Which slots of the buckets the wave just loaded (one per group, word `w` per lane) hold the key
// of the row each group is serving: `expect` is the lane's word of that row (tag lanes: the FULL
// tag, key lanes: the key word; other lanes: anything).  Returns a wave mask with a bit at the tag
// lane of every matching slot.  Two compares, one shift and one compare per lane; the rest is
// scalar mask arithmetic.
__device__ __forceinline__ u64 tg_match64(const TgLane &L, const TgMasks &M, u64 w, u64 expect) {
  const u64 mlo = __builtin_amdgcn_ballot_w64((u32)w == (u32)expect);
  const u64 mhi = __builtin_amdgcn_ballot_w64((u32)(w >> 32) == (u32)(expect >> 32));
  const u64 m = mlo & (mhi | M.notkey);              // tag lanes: low half only (the high half is metadata)
  const u32 bits = (u32)(m >> L.lane) & M.kmask;
  return __builtin_amdgcn_ballot_w64(bits == M.kmask) & M.tagm;
}

__device__ __forceinline__ u32 tg_wrap(u32 home, u32 d, u64 nb) {
  const u64 b = (u64)home + d;
  return (u32)(b >= nb ? b - nb : b);
}

// mode 0: get (write value or fallback + flag), 1: count, 2: remove, 3: remove of a batch that
// holds no key twice (the tombstone is a plain store instead of a compare-and-swap).
// Rows are taken in tiles of DOK_TPB (see DOK_TILE_LOOP); a wave only ever reads the LDS rows its
// own lanes staged, so the tiles need no workgroup barrier between them.
// Phase 1 serves the home bucket of each of a group's 16 rows as "issue 8 loads, resolve 8
// rounds"; a round is a handful of instructions (tg_match64), and the value lanes of a matching
// slot write the output row straight from the bucket words they hold.  Rows without a match are
// finished by their owner lane: with no displacement marked in the home bucket's metadata (passed
// on through LDS by the lane that held it) it writes the fallback row.  Phase 2 serves the rows
// whose home bucket carries displacement marks and held no match, four rows per group and turn,
// each at its next marked bucket.
// UV: the access granule of the value rows (8 or 4) as a compile-time constant, or 0 = g.unit_v:
// with it each of the 16 unrolled rounds carries one store instead of a switch over the four
// granules (4 % at 16M lookups of 40-byte values).
// MODE 4 (sparse-valued gather): as get, but the value of every row found goes, under the key i,
// into `out`, a packed table of VP-byte values (i = the element's offset in the index space).
// Src: where the rows come from (see the row sources above).
template <int MODE, bool STATS, int UV, class Src, int VP = 0>
__device__ __forceinline__ void tg_lookup_body(const DevTable &t, const TgGeom &g, const Src &src, i64 n,
                                               u8 *__restrict__ values, u8 *__restrict__ flags,
                                               i64 *count, const u8 *__restrict__ fallback_dev,
                                               const DevTable *out) {
  extern __shared__ u64 lds[];
  const int RS = tg_rs(g);
  u64 *lds_rows = lds;                          // [DOK_TPB][1 + KW]
  u64 *lds_fb = lds + DOK_TPB * RS;             // [VW]
  u32 *lds_meta = (u32 *)(lds_fb + g.VW);       // [DOK_TPB][2]: metadata and filter of each row's home bucket
  u8 *lds_out = (u8 *)(lds_meta + DOK_TPB * 2); // [DOK_TPB][V]: the tile's output rows (get)
  // the fallback row: part of the geometry argument, or - fallback_dev set - read from device memory
  constexpr bool VALUES = MODE == 0 || MODE == 4;   // the value rows of the hits are staged in lds_out
  if (VALUES && threadIdx.x < g.VW)
    lds_fb[threadIdx.x] = fallback_dev ? tg_load_word(fallback_dev, threadIdx.x, g.V, UV ? UV : g.unit_v)
                                       : g.fallback[threadIdx.x];
  __syncthreads();
  const TgLane L(g);
  const TgMasks M(g, L);
  const int unit_v = UV ? UV : g.unit_v;
  const int wave_row0 = threadIdx.x & ~63;      // first LDS row of this wave
  // the word of the served row this lane compares its bucket word with: word p of the row for the
  // tag and key lanes (any word for the others)
  const int my_word = (L.is_tag || L.is_key) ? L.p : 0;
  const u64 *exp0 = lds_rows + (wave_row0 + L.gbase) * RS + my_word;   // round r: exp0[r * RS]
  const int tl = L.gbase + L.tag_lane;          // wave lane of this lane's slot's tag
  // lane 0 of a group holds the bucket's metadata, lane W (slot 1's tag lane) its filter
  const bool has_filter = g.S >= 2;
  const bool meta_lane = L.l == 0 || (has_filter && L.l == g.W);
  u32 *meta_out = lds_meta + (wave_row0 + L.gbase) * 2 + (L.l != 0);   // round r: meta_out[2 * r]
  int n_found = 0, n_removed = 0, n_probe = 0, n_ops = 0, n_fresh = 0, n_full = 0;

  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool inside = i < n;                  // the tile's rows inside the batch
    u64 *krow = lds_rows + threadIdx.x * RS;
    // `active`: a row that is looked up (rows addressing nothing inside the coordinate space are absent)
    const bool active = inside && src.stage(t, g, i, krow, nullptr) == 0;
    u32 home, qfull;
    tg_hash_row(t, g, krow, home, qfull);
    if (!active) home = 0;
    const i64 wave_i0 = i - L.lane;             // batch row of lane 0
    u8 *out_g = lds_out + (size_t)(wave_row0 + L.gbase) * g.V;   // (staged) output row of the group's row 0
    u64 my_hit64 = 0;

    const u64 am = dok_ballot(active);
    const u64 im = dok_ballot(inside);
    if (am != 0) {
      #pragma unroll
      for (int r0 = 0; r0 < 16; r0 += 8) {
        u64 w[8];
        #pragma unroll
        for (int u = 0; u < 8; u++) {
          const u32 qb = dok_shfl32(home, L.gbase + r0 + u);
          w[u] = t.buckets[(u64)qb * 16 + L.l];
        }
        #pragma unroll
        for (int u = 0; u < 8; u++) {
          const int r = r0 + u;
          // lanes of the groups whose row r is a real row
          const u64 tr = (am >> r) & 0x0001000100010001ULL;
          const u64 on64 = (tr << 16) - tr;
          const u64 hit64 = tg_match64(L, M, w[u], exp0[r * RS]) & on64;
          if (VALUES && L.is_val && ((hit64 >> tl) & 1ULL))
            tg_store_word(out_g + (size_t)r * g.V, L.p - 1 - g.KW, g.V, unit_v, w[u]);
          // the bucket's metadata and filter are left in LDS for the row's owner
          if (meta_lane) meta_out[2 * r] = (u32)(w[u] >> 32);
          my_hit64 = L.l == r ? hit64 : my_hit64;
        }
      }
    }
    const u32 my_hit = L.grp(my_hit64);
    bool found = active && my_hit != 0;
    u32 sb = home, sw = my_hit ? (u32)__builtin_ctz(my_hit) : 0u;
    n_probe += active;
    // rows without a match: the home bucket's metadata decides between "absent" and "look on"
    u32 my_meta = 0;
    if (active && !found) {
      my_meta = lds_meta[threadIdx.x * 2];
      // a key placed away from its home has set its filter bit there
      if (has_filter && !(lds_meta[threadIdx.x * 2 + 1] & tg_fbit(qfull))) my_meta = 0;
    }
    bool open = active && !found && my_meta != 0;
    if (VALUES && inside && !found && !open) {
      for (int k = 0; k < g.VW; k++)
        tg_store_word(lds_out + (size_t)threadIdx.x * g.V, k, g.V, unit_v, lds_fb[k]);
    }

    // phase 2: the marked displacements, then (rare) the far ones
    u32 cand = open ? (my_meta & DOK_TG_NEARMASK) : 0u;
    bool far = open && (my_meta & 1u);
    const u32 far_max = my_meta >> 24;
    u32 far_d = DOK_TG_NEAR + 1;
    u64 pm = dok_ballot(open);
    while (pm != 0) {
      const u32 d0 = cand ? (u32)__builtin_ctz(cand) : far_d;
      const u32 b0 = tg_wrap(home, d0, t.nb);
      u32 rest = L.grp(pm);
      int rr[4];
      bool hs[4];
      u64 w[4];
      #pragma unroll
      for (int k = 0; k < 4; k++) {
        hs[k] = rest != 0;
        rr[k] = hs[k] ? __builtin_ctz(rest) : 0;
        rest &= rest - 1;
        const u32 qb = dok_shfl32(b0, L.gbase + rr[k]);
        w[k] = t.buckets[(u64)(hs[k] ? qb : 0u) * 16 + L.l];
      }
      bool act = false;
      u32 h = 0, e = 0;
      #pragma unroll
      for (int k = 0; k < 4; k++) {
        const u64 hit64 = tg_match64(L, M, w[k], exp0[rr[k] * RS]) & dok_ballot(hs[k]);
        const u32 em = L.grp(dok_ballot(hs[k] && L.is_tag && (u32)w[k] == DOK_TG_EMPTY));
        if (VALUES && L.is_val && ((hit64 >> tl) & 1ULL))
          tg_store_word(out_g + (size_t)rr[k] * g.V, L.p - 1 - g.KW, g.V, unit_v, w[k]);
        const bool mine = hs[k] && L.l == rr[k];
        act = act || mine;
        h = mine ? L.grp(hit64) : h;
        e = mine ? em : e;
      }
      if (act) {
        n_probe++;
        if (h) {
          found = true; open = false;
          sb = b0; sw = (u32)__builtin_ctz(h);
        } else {
          if (cand) cand &= cand - 1;
          else {
            if (far_max == DOK_TG_FARCAP && e) far = false;     // beyond the recorded range the chain ends at an EMPTY slot
            far_d++;
          }
          open = cand != 0 || (far && (far_max == DOK_TG_FARCAP ? (u64)far_d < t.nb : far_d <= far_max));
          if (!open && VALUES) {
            for (int k = 0; k < g.VW; k++)
              tg_store_word(lds_out + (size_t)threadIdx.x * g.V, k, g.V, unit_v, lds_fb[k]);
          }
        }
      }
      pm = dok_ballot(open);
    }
    bool removed = false;
    if (MODE == 2 && found)
      removed = atomicCAS((u32 *)(t.buckets + (u64)sb * 16 + sw), qfull, DOK_TG_TOMB) == qfull;
    if (MODE == 3 && found) { *(u32 *)(t.buckets + (u64)sb * 16 + sw) = DOK_TG_TOMB; removed = true; }
    if (MODE == 0 && im != 0) {
      // the wave's output rows leave LDS as one contiguous stretch
      const int ne = __popcll(im) * (g.V / unit_v);
      const u8 *src = lds_out + (size_t)wave_row0 * g.V;
      u8 *dst = values + (size_t)wave_i0 * g.V;
      for (int e = L.lane; e < ne; e += 64) {
        if (unit_v == 8) ((u64 *)dst)[e] = ((const u64 *)src)[e];
        else if (unit_v == 4) ((u32 *)dst)[e] = ((const u32 *)src)[e];
        else if (unit_v == 2) ((u16 *)dst)[e] = ((const u16 *)src)[e];
        else dst[e] = src[e];
      }
    }
    if (MODE == 0 && inside && flags) flags[i] = found ? 1 : 0;
    if ((MODE == 2 || MODE == 3) && inside && flags) flags[i] = removed ? 1 : 0;
    if constexpr (MODE == 4) {
      // every row found goes into `out` under the key i, by the packed layout's cooperative insert
      // (the whole wave takes part; its rows' values sit in the wave's own lds_out rows)
      const u64 ok2 = (u64)i ^ DOK_P8_XOR;
      const u64 val = found ? tg_load_word(lds_out + (size_t)threadIdx.x * g.V, 0, g.V, unit_v) : 0;
      const u64 h2 = p8_hash(ok2, *out);
      int st = 0, fresh = 0;
      p8_insert<VP>(out->buckets, out->nb, ok2, val, found ? dok_reduce(h2, out->nb) : 0u, p8_fbit(h2), found, st, fresh);
      n_fresh += fresh;
      n_full += (found && st == 0);
    }
    n_found += found;
    n_removed += removed;
    n_ops += inside;
  }
  if constexpr (MODE == 4)
    dok_block_add2(&out->header[DOK_H_NELEM], n_fresh, &out->header[DOK_H_NFULL], n_full);
  else if (MODE == 1 || MODE == 2 || MODE == 3 || STATS)
    dok_block_add3(MODE == 1 ? count : &t.header[DOK_H_NELEM], MODE == 1 ? n_found : -n_removed,
                   &t.header[DOK_H_NPROBE], STATS ? n_probe : 0, &t.header[DOK_H_NOPS], STATS ? n_ops : 0);
}

template <int MODE, bool STATS, int UV, class Src>
__global__ __launch_bounds__(DOK_TPB) void tg_lookup_kernel(DevTable t, TgGeom g, Src src, i64 n,
                                                            u8 *__restrict__ values, u8 *__restrict__ flags,
                                                            i64 *count, const u8 *__restrict__ fallback_dev) {
  tg_lookup_body<MODE, STATS, UV, Src>(t, g, src, n, values, flags, count, fallback_dev, nullptr);
}

// Sparse-valued gather from a multi-word coordinate table into a packed one keyed by the index space.
template <int VP>
__global__ __launch_bounds__(DOK_TPB) void tg_getitem_sparse_kernel(DevTable t, TgGeom g, TgIndexSrc src, DevTable out) {
  tg_lookup_body<4, false, 0, TgIndexSrc, VP>(t, g, src, src.ix.n_elems, nullptr, nullptr, nullptr, nullptr, &out);
}

// Record in the home bucket's metadata that a key was placed d > 0 buckets further on, and (W > 0:
// the bucket has a filter, in slot 1's tag word) the key's filter bit.
__device__ __forceinline__ void tg_mark(u64 *home_bucket, u32 d, u32 md_seen, int W, u32 fbit, u32 filt_seen) {
  u32 *meta = (u32 *)home_bucket + 1;
  if (W > 0 && !(filt_seen & fbit)) atomicOr((u32 *)(home_bucket + W) + 1, fbit);
  if (d <= DOK_TG_NEAR) {
    if (!((md_seen >> d) & 1u)) atomicOr(meta, 1u << d);
    return;
  }
  const u32 dm = d < DOK_TG_FARCAP ? d : DOK_TG_FARCAP;
  u32 old = __hip_atomic_load(meta, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  for (;;) {
    u32 mx = old >> 24;
    if (dm > mx) mx = dm;
    const u32 nw = (old & 0x00ffffffu) | (mx << 24) | 1u;
    if (nw == old) break;
    const u32 prev = atomicCAS(meta, old, nw);
    if (prev == old) break;
    old = prev;
  }
}

#define DOK_TG_MAXS 5            // most slots a bucket can have (W >= 3)

// Upsert of the (up to 64) rows a wave has staged in LDS: lane x owns LDS row threadIdx.x (tag and
// key words in lds_rows, value words in lds_vals).  Every lane inspects the current bucket of its
// own row by itself - it reads just the S tag words (slot 0's comes with the bucket metadata) and,
// only where a tag equals its own, that slot's key words - so a turn costs a few loads per row and
// no cross-lane work.  Protocol per row:
//   * a slot FULL with the row's key -> lock it (CAS FULL->BUSY), rewrite the value words,
//     publish FULL again.  Losing that CAS means an equal key of this batch holds the lock:
//     its value stands and this row is done.
//   * a slot BUSY with the row's tag -> its key is not readable yet: look again next turn.
//   * a slot FULL with the row's tag but other key words -> look once more after an acquire
//     fence; a second mismatch is a genuine fingerprint collision and the slot is skipped.
//   * otherwise the row's place is the first free slot of its walk (a tombstone of that bucket
//     before an EMPTY slot).  That the key does not sit further on is established through the
//     home bucket's displacement map, as in the packed layout: the marked buckets beyond the
//     chosen slot are looked at, then the slot is claimed (CAS -> BUSY).  A lost claim makes the
//     row look at that bucket again.
// The slots won in a turn are then written by the groups, one row per round: lane p of the group
// stores word p of the slot, so a slot costs one contiguous store instead of W scattered ones;
// after a wait for those stores the owners publish FULL together.  The data words are written
// with agent-scope atomic stores (write-through to the level all XCDs share); a BUSY holder
// finishes in straight-line code inside one loop turn, so waiting rows always see it released.
__device__ __forceinline__ void tg_insert_rows(const DevTable &t, const TgGeom &g, const TgLane &L,
                                               const u64 *lds_rows, const u64 *lds_vals, u32 home, u32 qfull,
                                               bool pend, int &st, int &fresh) {
  const int RS = tg_rs(g);
  const int wave_row0 = threadIdx.x & ~63;
  const u64 *krow = lds_rows + threadIdx.x * RS;
  if (!pend) home = 0;
  const u32 qbusy = qfull & ~1u;
  const u32 fbit = tg_fbit(qfull);
  const bool has_filter = g.S >= 2;
  u32 cur = 0, md_home = 0, filt_home = 0;        // displacement inspected this turn; home metadata and filter
  bool chosen = false, slot_tomb = false, confirm = false, far_unb = false;
  u32 slot_d = 0, slot_w = 0, chk = 0, far_next = 0, far_to = 0;

  u64 pm = dok_ballot(pend);
  while (pm != 0) {
    if (dok_ballot(confirm) != 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    const u32 b = pend ? tg_wrap(home, cur, t.nb) : 0u;
    u64 *bucket = t.buckets + (u64)b * 16;

    // ---- every owner looks at the tags of its bucket
    u64 tw[DOK_TG_MAXS];
    #pragma unroll
    for (int s = 0; s < DOK_TG_MAXS; s++) {
      tw[s] = 0;
      if (s < g.S && pend) tw[s] = dok_load_coherent(bucket + s * g.W);
    }
    const u32 md = (u32)(tw[0] >> 32);
    u32 candm = 0, emptym = 0, tombm = 0;          // one bit per slot
    bool busy = false;
    #pragma unroll
    for (int s = 0; s < DOK_TG_MAXS; s++) {
      if (s < g.S) {
        const u32 t32 = (u32)tw[s];
        candm |= (u32)(t32 == qfull) << s;
        busy = busy || t32 == qbusy;
        emptym |= (u32)(t32 == DOK_TG_EMPTY) << s;
        tombm |= (u32)(t32 == DOK_TG_TOMB) << s;
      }
    }
    // slots with the row's tag: compare the key words
    int hit_s = -1;
    bool tagonly = false;
    if (pend) {
      u32 c = candm;
      while (c != 0 && hit_s < 0) {
        const int s = __builtin_ctz(c);
        c &= c - 1;
        bool eq = true;
        for (int k = 0; k < g.KW; k++) eq = eq && dok_load_coherent(bucket + s * g.W + 1 + k) == krow[1 + k];
        if (eq) hit_s = s; else tagonly = true;
      }
    }

    bool wr = false, wr_fresh = false;
    u32 wr_b = 0, wr_w = 0;
    if (pend) {
      if (hit_s >= 0) {
        const u32 sw = (u32)(hit_s * g.W);
        if (atomicCAS((u32 *)(bucket + sw), qfull, qbusy) == qfull) { wr = true; wr_b = b; wr_w = sw; }
        st = 1; pend = false;
      } else if (busy) {
        // wait for the holder to publish
      } else if (tagonly && !confirm) {
        confirm = true;
      } else {
        confirm = false;
        if (!chosen) {
          if (cur == 0) { md_home = md; filt_home = (u32)(tw[1] >> 32); }
          if (tombm | emptym) {
            chosen = true;
            slot_tomb = tombm != 0;
            slot_d = cur;
            slot_w = (u32)(__builtin_ctz(tombm ? tombm : emptym) * g.W);
            chk = cur < DOK_TG_NEAR ? (md_home & DOK_TG_NEARMASK & ~((2u << cur) - 1u)) : 0u;
            far_unb = (md_home & 1u) && (md_home >> 24) == DOK_TG_FARCAP;
            far_to = (md_home & 1u) ? (far_unb ? 0xffffffffu : (md_home >> 24)) : 0u;
            far_next = cur + 1 > DOK_TG_NEAR + 1u ? cur + 1 : DOK_TG_NEAR + 1u;
            // without the key's filter bit in its home bucket the key was never placed elsewhere
            if (has_filter && !(filt_home & fbit)) { chk = 0; far_to = 0; }
          } else if ((u64)cur + 1 >= t.nb) {
            st = 0; pend = false;                          // no free slot anywhere
          } else {
            cur++;
          }
        } else if (far_unb && cur > DOK_TG_NEAR && emptym) {
          far_to = 0;                                      // beyond the recorded range the chain ends at an EMPTY slot
        }
        if (pend && chosen) {
          bool claim = false;
          if (chk) { cur = (u32)__builtin_ctz(chk); chk &= chk - 1; }
          else if (far_next <= far_to && (u64)far_next < t.nb) cur = far_next++;
          else claim = true;
          if (claim) {
            const u32 tb = tg_wrap(home, slot_d, t.nb);
            u32 *tagp = (u32 *)(t.buckets + (u64)tb * 16 + slot_w);
            const u32 expect = slot_tomb ? DOK_TG_TOMB : DOK_TG_EMPTY;
            if (atomicCAS(tagp, expect, qbusy) == expect) {
              wr = true; wr_fresh = true; wr_b = tb; wr_w = slot_w;
              st = 1; fresh = 1; pend = false;
              if (slot_d > 0) tg_mark(t.buckets + (u64)home * 16, slot_d, md_home, has_filter ? g.W : 0, fbit, filt_home);
            } else {
              chosen = false; cur = slot_d;                // somebody took the slot: look at that bucket again
            }
          }
        }
      }
    }

    // ---- the slots won in this turn: payload by the groups, then the owners publish
    const u64 wm = dok_ballot(wr);
    if (wm != 0) {
      const u32 wsub = L.grp(wm);
      u32 wany = (u32)wm | (u32)(wm >> 32);
      wany = (wany | (wany >> 16)) & 0xffffu;
      #pragma unroll
      for (int r = 0; r < 16; r++) {
        if (!((wany >> r) & 1u)) continue;
        const int j = L.gbase + r;
        const u32 qb = dok_shfl32(wr_b, j), qw = dok_shfl32(wr_w, j);
        const int first = dok_shfl32((u32)wr_fresh, j) ? 1 : 1 + g.KW;
        if (((wsub >> r) & 1u) && L.l >= first && L.l < g.W) {
          const u64 word = L.l <= g.KW ? lds_rows[(wave_row0 + j) * RS + L.l]
                                       : lds_vals[(wave_row0 + j) * g.VW + L.l - 1 - g.KW];
          dok_store_coherent(t.buckets + (u64)qb * 16 + qw + L.l, word);
        }
      }
      // the payload stores have completed before any tag is published
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (wr) __hip_atomic_store((u32 *)(t.buckets + (u64)wr_b * 16 + wr_w), qfull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    pm = dok_ballot(pend);
  }
}

// Placement of rows whose keys are all different and absent from the table, into a table without
// tombstones that nothing else touches while the kernel runs: the destination of a rehash.
// Slots then only ever go from EMPTY to FULL, so no key is compared and no slot is locked: a row
// claims the first EMPTY slot of its walk (CAS EMPTY -> FULL; a stale view of a taken slot only
// costs a failed claim) and the group writes the payload with plain stores - one compare-and-swap
// and one store per row where the upsert protocol takes three write-through transactions.
__device__ __forceinline__ void tg_place_rows(const DevTable &t, const TgGeom &g, const TgLane &L,
                                              const u64 *lds_rows, const u64 *lds_vals, u32 home, u32 qfull,
                                              bool pend, int &st) {
  const int RS = tg_rs(g);
  const int wave_row0 = threadIdx.x & ~63;
  if (!pend) home = 0;
  const u32 fbit = tg_fbit(qfull);
  const bool has_filter = g.S >= 2;
  u32 cur = 0, md_home = 0, filt_home = 0;
  u64 pm = dok_ballot(pend);
  while (pm != 0) {
    bool wr = false;
    u32 wr_b = 0, wr_w = 0;
    if (pend) {
      const u32 b = tg_wrap(home, cur, t.nb);
      u64 *bucket = t.buckets + (u64)b * 16;
      u32 emptym = 0;
      #pragma unroll
      for (int s = 0; s < DOK_TG_MAXS; s++) {
        if (s < g.S) {
          const u64 tw = bucket[s * g.W];
          emptym |= (u32)((u32)tw == DOK_TG_EMPTY) << s;
          if (cur == 0 && s == 0) md_home = (u32)(tw >> 32);
          if (cur == 0 && s == 1) filt_home = (u32)(tw >> 32);
        }
      }
      while (emptym != 0 && !wr) {
        const int s = __builtin_ctz(emptym);
        emptym &= emptym - 1;
        if (atomicCAS((u32 *)(bucket + s * g.W), DOK_TG_EMPTY, qfull) == DOK_TG_EMPTY) {
          wr = true; wr_b = b; wr_w = (u32)(s * g.W);
        }
      }
      if (wr) {
        st = 1; pend = false;
        if (cur > 0) tg_mark(t.buckets + (u64)home * 16, cur, md_home, has_filter ? g.W : 0, fbit, filt_home);
      } else if ((u64)cur + 1 >= t.nb) {
        st = 0; pend = false;                              // no free slot anywhere
      } else {
        cur++;
      }
    }
    // the slots won in this turn: lane p of the row's group stores word p
    const u64 wm = dok_ballot(wr);
    if (wm != 0) {
      const u32 wsub = L.grp(wm);
      u32 wany = (u32)wm | (u32)(wm >> 32);
      wany = (wany | (wany >> 16)) & 0xffffu;
      #pragma unroll
      for (int r = 0; r < 16; r++) {
        if (!((wany >> r) & 1u)) continue;
        const int j = L.gbase + r;
        const u32 qb = dok_shfl32(wr_b, j), qw = dok_shfl32(wr_w, j);
        if (((wsub >> r) & 1u) && L.l >= 1 && L.l < g.W) {
          const u64 word = L.l <= g.KW ? lds_rows[(wave_row0 + j) * RS + L.l]
                                       : lds_vals[(wave_row0 + j) * g.VW + L.l - 1 - g.KW];
          t.buckets[(u64)qb * 16 + qw + L.l] = word;
        }
      }
    }
    pm = dok_ballot(pend);
  }
}

// ---- insert with ONE compare-and-swap per new row (batches with a workspace) ------------------------
// The protocol above costs a new row three write transactions (claim, payload, publish) because a
// row with the same key on another XCD must never read a half-written slot.  tg_fast_rows drops
// that guarantee and does not need it: a new row claims an EMPTY slot with one compare-and-swap
// EMPTY -> FULL and its group writes the payload with plain stores, and a row that cannot tell
// what it sees is DEFERRED - put on a list in the caller's workspace - and inserted by the protocol
// above in a second launch, when everything the first one wrote is visible.  Rules per row:
//   * a slot with the row's tag: compare the key words.  Equal: the key is present (or an equal row
//     of this batch has just claimed the slot: same bytes either way) - the value, a single 8-byte
//     word, is overwritten with one store, which cannot tear.  Not equal: a payload in flight or a
//     fingerprint collision: defer.
//   * a tag BUSY with the row's fingerprint: a tombstone being re-used (below): look again.
//   * otherwise the first free slot of the walk, after the displacement checks of tg_insert_rows.
//     EMPTY: claim -> FULL, payload by plain stores.  A TOMBSTONE keeps the key words of the entry
//     that was removed, which a concurrent row could mistake for a payload, so it is claimed the
//     slow way (BUSY, write-through payload, publish).  A claim lost to the row's own tag: defer.
//   * a row with a key word that is zero is deferred at once.  Zero is what the key words of a
//     never-used slot hold, and the words of a payload in flight become visible in any order: a slot
//     claimed by another key of the same fingerprint shows, word by word, either that key's word or
//     zero.  A row without a zero word can only find "the key words equal mine" when every word has
//     arrived and the keys are equal, so the comparison is exact.
// Only values of one word can be overwritten without a lock, so this form serves tables with
// VW == 1 (every coordinate table).  FRESH - the table held nothing when the kernel started, so
// whatever a row meets was claimed by this kernel - compares nothing, overwrites nothing (a slot with
// the row's tag: defer) and serves any widths.  (Claiming without looking first - one compare-and-swap
// per slot tried, the returned tag telling what holds it - was measured and is slower: 32M rows of 52
// bytes at load factor 0.5 take 3.4 ms against 3.05 ms, at 0.75 5.3 against 3.6 ms: a returning
// atomic costs more than the loads of a bucket's tags.  Looking at one slot first, the one the tag
// picks, and at the whole bucket only if that one is taken, changes little either way: 3.69 / 4.43 ms
// for the same rows, 1.11 against 1.18 ms for 10M rows of a 2-D coordinate table with four slots per
// bucket.  The claim and the payload store bound the kernel, not the look.)
template <bool FRESH>
__device__ __forceinline__ void tg_fast_rows(const DevTable &t, const TgGeom &g, const TgLane &L,
                                             const u64 *lds_rows, const u64 *lds_vals, u32 home, u32 qfull,
                                             bool pend, int &st, int &fresh, bool &deferred) {
  const int RS = tg_rs(g);
  const int wave_row0 = threadIdx.x & ~63;
  const u64 *krow = lds_rows + threadIdx.x * RS;
  if (!FRESH && pend) {
    bool zero_word = false;
    for (int k = 0; k < g.KW; k++) zero_word = zero_word || krow[1 + k] == 0;
    if (zero_word) { deferred = true; pend = false; }
  }
  if (!pend) home = 0;
  const u32 qbusy = qfull & ~1u;
  const u32 fbit = tg_fbit(qfull);
  const bool has_filter = g.S >= 2;
  u32 cur = 0, md_home = 0, filt_home = 0;
  bool chosen = false, slot_tomb = false, far_unb = false;
  u32 slot_d = 0, slot_w = 0, chk = 0, far_next = 0, far_to = 0;

  u64 pm = dok_ballot(pend);
  while (pm != 0) {
    const u32 b = pend ? tg_wrap(home, cur, t.nb) : 0u;
    u64 *bucket = t.buckets + (u64)b * 16;
    bool wr = false, wr_slow = false;
    u32 wr_b = 0, wr_w = 0;
    u64 tw[DOK_TG_MAXS];
    #pragma unroll
    for (int s = 0; s < DOK_TG_MAXS; s++) {
      tw[s] = 0;
      if (s < g.S && pend) tw[s] = dok_load_coherent(bucket + s * g.W);
    }
    const u32 md = (u32)(tw[0] >> 32);
    u32 candm = 0, emptym = 0, tombm = 0;
    bool busy = false;
    #pragma unroll
    for (int s = 0; s < DOK_TG_MAXS; s++) {
      if (s < g.S) {
        const u32 t32 = (u32)tw[s];
        candm |= (u32)(t32 == qfull) << s;
        busy = busy || t32 == qbusy;
        emptym |= (u32)(t32 == DOK_TG_EMPTY) << s;
        tombm |= (u32)(t32 == DOK_TG_TOMB) << s;
      }
    }
    if (pend) {
      if (candm) {
        // (FRESH: whatever carries this fingerprint was claimed by this kernel, its payload may be in
        // flight: nothing to compare)
        bool hit = false;
        u32 c = FRESH ? 0u : candm;
        while (c != 0 && !hit) {
          const int s = __builtin_ctz(c);
          c &= c - 1;
          bool eq = true;
          for (int k = 0; k < g.KW; k++) eq = eq && dok_load_coherent(bucket + s * g.W + 1 + k) == krow[1 + k];
          if (eq) {
            bucket[s * g.W + 1 + g.KW] = lds_vals[threadIdx.x * g.VW];       // (VW == 1: one word, one store)
            hit = true;
          }
        }
        if (hit) st = 1; else deferred = true;
        pend = false;
      } else if (busy) {
        // a tombstone being re-used by a row of this fingerprint: its holder publishes within its turn
      } else {
        if (!chosen) {
          if (cur == 0) { md_home = md; filt_home = (u32)(tw[1] >> 32); }
          if (tombm | emptym) {
            chosen = true;
            slot_tomb = tombm != 0;
            slot_d = cur;
            slot_w = (u32)(__builtin_ctz(tombm ? tombm : emptym) * g.W);
            chk = cur < DOK_TG_NEAR ? (md_home & DOK_TG_NEARMASK & ~((2u << cur) - 1u)) : 0u;
            far_unb = (md_home & 1u) && (md_home >> 24) == DOK_TG_FARCAP;
            far_to = (md_home & 1u) ? (far_unb ? 0xffffffffu : (md_home >> 24)) : 0u;
            far_next = cur + 1 > DOK_TG_NEAR + 1u ? cur + 1 : DOK_TG_NEAR + 1u;
            if (has_filter && !(filt_home & fbit)) { chk = 0; far_to = 0; }
            if (FRESH) { chk = 0; far_to = 0; }               // nothing was in the table: nothing to find further on
          } else if ((u64)cur + 1 >= t.nb) {
            st = 0; pend = false;                              // no free slot anywhere
          } else {
            cur++;
          }
        } else if (far_unb && cur > DOK_TG_NEAR && emptym) {
          far_to = 0;
        }
        if (pend && chosen) {
          bool claim = false;
          if (chk) { cur = (u32)__builtin_ctz(chk); chk &= chk - 1; }
          else if (far_next <= far_to && (u64)far_next < t.nb) cur = far_next++;
          else claim = true;
          if (claim) {
            const u32 tb = tg_wrap(home, slot_d, t.nb);
            u32 *tagp = (u32 *)(t.buckets + (u64)tb * 16 + slot_w);
            const u32 expect = slot_tomb ? DOK_TG_TOMB : DOK_TG_EMPTY;
            const u32 old = atomicCAS(tagp, expect, slot_tomb ? qbusy : qfull);
            if (old == expect) {
              wr = true; wr_slow = slot_tomb; wr_b = tb; wr_w = slot_w;
              st = 1; fresh = 1; pend = false;
              if (slot_d > 0) tg_mark(t.buckets + (u64)home * 16, slot_d, md_home, has_filter ? g.W : 0, fbit, filt_home);
            } else if ((old | 1u) == qfull) {
              deferred = true; pend = false;                   // a row with this fingerprint took the slot
            } else {
              chosen = false; cur = slot_d;                    // somebody else's key: look at that bucket again
            }
          }
        }
      }
    }

    // ---- the slots won in this turn: lane p of the row's group stores word p of the payload
    const u64 wm = dok_ballot(wr);
    if (wm != 0) {
      const u32 wsub = L.grp(wm);
      u32 wany = (u32)wm | (u32)(wm >> 32);
      wany = (wany | (wany >> 16)) & 0xffffu;
      #pragma unroll
      for (int r = 0; r < 16; r++) {
        if (!((wany >> r) & 1u)) continue;
        const int j = L.gbase + r;
        const u32 qb = dok_shfl32(wr_b, j), qw = dok_shfl32(wr_w, j);
        const bool slow = dok_shfl32((u32)wr_slow, j) != 0;
        if (((wsub >> r) & 1u) && L.l >= 1 && L.l < g.W) {
          const u64 word = L.l <= g.KW ? lds_rows[(wave_row0 + j) * RS + L.l]
                                       : lds_vals[(wave_row0 + j) * g.VW + L.l - 1 - g.KW];
          u64 *dst = t.buckets + (u64)qb * 16 + qw + L.l;
          if (slow) dok_store_coherent(dst, word); else *dst = word;
        }
      }
      if (dok_ballot(wr_slow) != 0) {
        // re-used tombstones: the payload has completed before the tag is published
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (wr_slow) __hip_atomic_store((u32 *)(t.buckets + (u64)wr_b * 16 + wr_w), qfull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    pm = dok_ballot(pend);
  }
}

// Workspace of the fast insert: a counter and the list of the deferred rows' numbers.
struct TgDeferList {
  u64 *count;        // [1] (cleared by tg_defer_clear_kernel)
  i64 *rows;         // [cap]
  i64 cap;
};
__global__ void tg_defer_clear_kernel(TgDeferList dl) { if (threadIdx.x == 0) dl.count[0] = 0; }

template <class Src, bool FRESH>
__global__ __launch_bounds__(DOK_TPB) void tg_fast_set_kernel(DevTable t, TgGeom g, Src src, i64 n, TgDeferList dl) {
  extern __shared__ u64 lds[];
  const int RS = tg_rs(g);
  u64 *lds_rows = lds;
  u64 *lds_vals = lds + DOK_TPB * RS;
  const TgLane L(g);
  int n_fresh = 0, n_full = 0, n_oob = 0;
  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool inside = i < n;
    u64 *krow = lds_rows + threadIdx.x * RS;
    const int code = inside ? src.stage(t, g, i, krow, lds_vals + threadIdx.x * g.VW) : 2;
    const bool active = code == 0;
    n_oob += code == 1;
    u32 home, qfull;
    tg_hash_row(t, g, krow, home, qfull);
    int st = 0, fresh = 0;
    bool deferred = false;
    tg_fast_rows<FRESH>(t, g, L, lds_rows, lds_vals, home, qfull, active, st, fresh, deferred);
    // the deferred rows of the wave go on the list with one atomic
    const u64 dm = dok_ballot(deferred);
    if (dm != 0) {
      u64 base = 0;
      if (L.lane == 0) base = atomicAdd(dl.count, (u64)__popcll(dm));
      base = dok_shfl64(base, 0);
      const i64 at = (i64)base + __popcll(dm & ((1ULL << L.lane) - 1ULL));
      if (deferred && at < dl.cap) dl.rows[at] = i;
    }
    n_fresh += fresh;
    n_full += (active && !deferred && st == 0);
  }
  dok_block_add3(&t.header[DOK_H_NELEM], n_fresh, &t.header[DOK_H_NFULL], n_full, &t.header[DOK_H_NOOB], n_oob);
}

// Second launch of the fast insert: the deferred rows, by the ordinary protocol.
template <class Src>
__global__ __launch_bounds__(DOK_TPB) void tg_deferred_kernel(DevTable t, TgGeom g, Src src, TgDeferList dl) {
  extern __shared__ u64 lds[];
  const int RS = tg_rs(g);
  u64 *lds_rows = lds;
  u64 *lds_vals = lds + DOK_TPB * RS;
  const TgLane L(g);
  const i64 n = (i64)dl.count[0] < dl.cap ? (i64)dl.count[0] : dl.cap;
  int n_fresh = 0, n_full = 0;
  DOK_TILE_LOOP(n) {
    const i64 k = DOK_TILE_ROW();
    const bool inside = k < n;
    u64 *krow = lds_rows + threadIdx.x * RS;
    const bool active = inside && src.stage(t, g, dl.rows[k], krow, lds_vals + threadIdx.x * g.VW) == 0;
    u32 home, qfull;
    tg_hash_row(t, g, krow, home, qfull);
    int st = 0, fresh = 0;
    tg_insert_rows(t, g, L, lds_rows, lds_vals, home, qfull, active, st, fresh);
    n_fresh += fresh;
    n_full += (active && st == 0);
  }
  dok_block_add2(&t.header[DOK_H_NELEM], n_fresh, &t.header[DOK_H_NFULL], n_full);
}

// Upsert of the rows a source delivers (see the row sources above).
template <class Src>
__global__ __launch_bounds__(DOK_TPB) void tg_set_kernel(DevTable t, TgGeom g, Src src, i64 n, u8 *__restrict__ stored) {
  extern __shared__ u64 lds[];
  const int RS = tg_rs(g);
  u64 *lds_rows = lds;                          // [DOK_TPB][1 + KW]
  u64 *lds_vals = lds + DOK_TPB * RS;           // [DOK_TPB][VW]
  const TgLane L(g);
  int n_fresh = 0, n_full = 0, n_oob = 0;

  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool inside = i < n;
    u64 *krow = lds_rows + threadIdx.x * RS;
    const int code = inside ? src.stage(t, g, i, krow, lds_vals + threadIdx.x * g.VW) : 2;
    const bool active = code == 0;
    n_oob += code == 1;
    u32 home, qfull;
    tg_hash_row(t, g, krow, home, qfull);
    int st = 0, fresh = 0;
    tg_insert_rows(t, g, L, lds_rows, lds_vals, home, qfull, active, st, fresh);
    if (inside && stored) stored[i] = (u8)(active ? st : 0);
    n_fresh += fresh;
    n_full += (active && st == 0);
  }
  dok_block_add3(&t.header[DOK_H_NELEM], n_fresh, &t.header[DOK_H_NFULL], n_full, &t.header[DOK_H_NOOB], n_oob);
}

// ---- table scans: read-out and rehash (chunks of DOK_CHUNK buckets, as in the packed layout) --------

__device__ __forceinline__ bool tg_scan_load(const DevTable &t, const TgLane &L, i64 b, u64 &w) {
  const bool valid = b < (i64)t.nb;
  w = t.buckets[(u64)(valid ? b : (i64)t.nb - 1) * 16 + L.l];
  return valid && L.is_tag && ((u32)w & 3u) == 3u;
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

// COLS: the key words are coordinates and go out the way a COO tensor holds them, word d of entry
// `row` at keys_out[d * cap + row].
template <bool COLS>
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
    const int tag_lane = L.gbase + L.tag_lane;
    const bool slot_live = L.valid && ((m >> tag_lane) & 1ULL);
    const i64 row = base + __popcll(m & ((1ULL << tag_lane) - 1ULL));
    if (slot_live && row < cap) {
      if (L.is_key && keys_out) {
        if (COLS) ((u64 *)keys_out)[(i64)(L.p - 1) * cap + row] = w;
        else tg_store_word(keys_out + (size_t)row * g.K, L.p - 1, g.K, g.unit_k, w);
      }
      if (L.is_val && values_out) tg_store_word(values_out + (size_t)row * g.V, L.p - 1 - g.KW, g.V, g.unit_v, w);
    }
    base += __popcll(m);
  }
}

// dense[row-major offset of the coordinates] = value for every live entry of a coordinate table
// (strides: row-major element strides of the dense tensor).  The key lanes of a slot hold one
// coordinate each; the slot's tag lane collects them with lane shuffles.
struct TgDenseStrides { i64 s[DOK_MAX_DIMS]; };
__global__ __launch_bounds__(DOK_TPB) void tg_to_dense_kernel(DevTable t, TgGeom g, TgDenseStrides strides, u8 *dense,
                                                              i64 n_chunks) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const TgLane L(g);
  const int tag_lane = L.gbase + L.tag_lane;
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live_tag = tg_scan_load(t, L, wid * DOK_CHUNK + s * 4 + (L.lane >> 4), w);
    u64 off = 0;
    bool ok = true;
    for (int k = 0; k < g.KW; k++) {
      const u64 c = dok_shfl64(w, (tag_lane + 1 + k) & 63);
      ok = ok && c < (u64)t.lin_dims[k];
      off += c * (u64)strides.s[k];
    }
    const u64 val = dok_shfl64(w, (tag_lane + 1 + g.KW) & 63);
    if (live_tag && ok) tg_store_word(dense + (size_t)off * g.V, 0, g.V, g.V, val);
  }
}

// Re-insert every live entry of `src` into `dst` (same widths, cleared by the caller).  A wave
// scans a chunk of the source four buckets per step; the lanes that hold the words of a live slot
// put them into the wave's LDS rows, packed, and whenever the rows of another step might not fit
// any more the wave inserts what it has gathered.
__global__ __launch_bounds__(DOK_TPB) void tg_rehash_kernel(DevTable src, DevTable dst, TgGeom g, i64 n_chunks) {
  extern __shared__ u64 lds[];
  const int RS = tg_rs(g);
  u64 *lds_rows = lds;
  u64 *lds_vals = lds + DOK_TPB * RS;
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  const TgLane L(g);
  const int wave_row0 = threadIdx.x & ~63;
  int n_fresh = 0, n_full = 0;
  if (wid < n_chunks) {
    int cnt = 0;
    for (int s = 0; s < DOK_CHUNK / 4; s++) {
      u64 w;
      const bool live_tag = tg_scan_load(src, L, wid * DOK_CHUNK + s * 4 + (L.lane >> 4), w);
      const u64 m = dok_ballot(live_tag);
      const int tag_lane = L.gbase + L.tag_lane;
      const bool slot_live = L.valid && ((m >> tag_lane) & 1ULL);
      const int row = wave_row0 + cnt + __popcll(m & ((1ULL << tag_lane) - 1ULL));
      if (slot_live && L.is_key) lds_rows[row * RS + L.p] = w;
      if (slot_live && L.is_val) lds_vals[row * g.VW + L.p - 1 - g.KW] = w;
      cnt += __popcll(m);
      if (cnt + 4 * g.S > 64 || s == DOK_CHUNK / 4 - 1) {
        const bool pend = L.lane < cnt;
        u32 home, qfull;
        tg_hash_row(dst, g, lds_rows + threadIdx.x * RS, home, qfull);
        int st = 0;
        tg_place_rows(dst, g, L, lds_rows, lds_vals, home, qfull, pend, st);
        n_fresh += (pend && st == 1);
        n_full += (pend && st == 0);
        cnt = 0;
      }
    }
  }
  dok_wave_add_n(&dst.header[DOK_H_NELEM], n_fresh);
  dok_wave_add_n(&dst.header[DOK_H_NFULL], n_full);
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

static size_t tg_lds_lookup(const TgGeom &g) { return (size_t)(DOK_TPB * (g.KW + 1) + g.VW + DOK_TPB + (DOK_TPB * g.V + 7) / 8) * 8; }
static size_t tg_lds_insert(const TgGeom &g) { return (size_t)DOK_TPB * (g.KW + 1 + g.VW) * 8; }

// Most workgroups of the kernels that loop over tiles and end with one atomic per wave on a
// counter: few workgroups keep those atomics cheap (same-address atomics serialise at ~12 ns
// each), many even out the differing amounts of work of the tiles.
#define DOK_TG_COUNT_GRID 8192u
#define DOK_TG_REMOVE_GRID 4096u
#define DOK_TG_SET_GRID 32768u

// Launch of the lookup kernel for one mode and row source.  fallback: host pointer to the fallback row
// (NULL = zeros); fb_dev: device pointer to it instead.
template <class Src>
static int tg_launch_get(const DevTable &d, const Src &src, i64 n, void *values, const void *fallback,
                         const void *fb_dev, u8 *found, bool stats, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, fallback, g);
  if (rc) return rc;
  if (!tg_aligned(values, g.unit_v)) return DOK_EINVAL;
  if (fb_dev && !tg_aligned(fb_dev, g.unit_v)) return DOK_EINVAL;
  const u8 *fbd = (const u8 *)fb_dev;
  const unsigned grid = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  const unsigned cgrid = grid < 2048u ? grid : 2048u;
  if (stats)
    tg_lookup_kernel<0, true, 0, Src><<<cgrid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, n, (u8 *)values, found, nullptr, fbd);
  else if (g.unit_v == 8)
    tg_lookup_kernel<0, false, 8, Src><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, n, (u8 *)values, found, nullptr, fbd);
  else if (g.unit_v == 4)
    tg_lookup_kernel<0, false, 4, Src><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, n, (u8 *)values, found, nullptr, fbd);
  else
    tg_lookup_kernel<0, false, 0, Src><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, n, (u8 *)values, found, nullptr, fbd);
  return DOK_OK;
}

template <class Src>
static int tg_launch_count(const DevTable &d, const Src &src, i64 n, i64 *count, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  const unsigned grid = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  tg_lookup_kernel<1, false, 0, Src><<<(grid < DOK_TG_COUNT_GRID ? grid : DOK_TG_COUNT_GRID), DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, n, nullptr, nullptr, count, nullptr);
  return DOK_OK;
}

template <class Src>
static int tg_launch_remove(const DevTable &d, const Src &src, i64 n, u8 *removed, bool unique, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  const unsigned tiles = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  const unsigned grid = tiles < DOK_TG_REMOVE_GRID ? tiles : DOK_TG_REMOVE_GRID;
  if (unique)
    tg_lookup_kernel<3, false, 0, Src><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, n, nullptr, removed, nullptr, nullptr);
  else
    tg_lookup_kernel<2, false, 0, Src><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, n, nullptr, removed, nullptr, nullptr);
  return DOK_OK;
}

template <class Src>
static int tg_launch_set(const DevTable &d, const Src &src, i64 n, u8 *stored, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  const unsigned grid = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  tg_set_kernel<Src><<<(grid < DOK_TG_SET_GRID ? grid : DOK_TG_SET_GRID), DOK_TPB, tg_lds_insert(g), s>>>(d, g, src, n, stored);
  return DOK_OK;
}

// Workspace bytes of the fast insert for n rows, and its layout.
static i64 tg_fast_workspace_bytes(i64 n) { return 256 + 8 * n; }
// Whether the fast insert serves this table (fresh = it holds nothing: every width; else one-word values).
static bool tg_fast_serves(const DevTable &d, bool fresh) { return fresh || d.value_bytes <= 8; }

// fresh: the table has just been cleared (or is cleared here: `clear`), nothing else is in it.
template <class Src>
static int tg_launch_set_fast(const DevTable &d, const Src &src, i64 n, bool fresh, void *workspace, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  TgDeferList dl;
  dl.count = (u64 *)workspace;
  dl.rows = (i64 *)((char *)workspace + 256);
  dl.cap = n;
  const unsigned tiles = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  const unsigned grid = tiles < DOK_TG_SET_GRID ? tiles : DOK_TG_SET_GRID;
  tg_defer_clear_kernel<<<1, 64, 0, s>>>(dl);
  if (fresh) tg_fast_set_kernel<Src, true><<<grid, DOK_TPB, tg_lds_insert(g), s>>>(d, g, src, n, dl);
  else tg_fast_set_kernel<Src, false><<<grid, DOK_TPB, tg_lds_insert(g), s>>>(d, g, src, n, dl);
  // (the deferred rows are few - equal keys inside the batch, re-used fingerprints - and the grid is
  // sized for a list that nobody knows yet: its workgroups find the count on the device)
  tg_deferred_kernel<Src><<<(tiles < 1024u ? tiles : 1024u), DOK_TPB, tg_lds_insert(g), s>>>(d, g, src, dl);
  return DOK_OK;
}

// Key / value row pointers of a batch call, checked against the access granules of the widths.
static int tg_rows(const DevTable &d, const void *keys, const void *values, TgRows &r) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  if (!tg_aligned(keys, g.unit_k) || (values && !tg_aligned(values, g.unit_v))) return DOK_EINVAL;
  r.keys = (const u8 *)keys;
  r.values = (const u8 *)values;
  return DOK_OK;
}

static int tg_launch_getitem_sparse(const DevTable &d, const TgIndexSrc &src, const DevTable &out, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  const i64 n = src.ix.n_elems;
  const unsigned tiles = (unsigned)((n + DOK_TPB - 1) / DOK_TPB);
  const unsigned grid = tiles < 2048u ? tiles : 2048u;
  switch (out.value_bytes) {
    case 1: tg_getitem_sparse_kernel<1><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, out); break;
    case 2: tg_getitem_sparse_kernel<2><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, out); break;
    case 4: tg_getitem_sparse_kernel<4><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, out); break;
    default: tg_getitem_sparse_kernel<8><<<grid, DOK_TPB, tg_lds_lookup(g), s>>>(d, g, src, out); break;
  }
  return DOK_OK;
}

static int tg_launch_rehash(const DevTable &a, const DevTable &b, i64 n_chunks, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(a, nullptr, g);
  if (rc) return rc;
  tg_rehash_kernel<<<(unsigned)((n_chunks + 3) / 4), DOK_TPB, tg_lds_insert(g), s>>>(a, b, g, n_chunks);
  return DOK_OK;
}

// cols: coordinate table, keys go out as [ndim][cap] int64 (see tg_chunk_write_kernel)
static int tg_launch_compact(const DevTable &d, i64 *offs, i64 n_chunks, void *keys_out, void *values_out,
                             i64 cap, i64 *count_out, bool cols, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  if ((keys_out && !tg_aligned(keys_out, cols ? 8 : g.unit_k)) || (values_out && !tg_aligned(values_out, g.unit_v)))
    return DOK_EINVAL;
  const unsigned grid = (unsigned)((n_chunks + 3) / 4);
  tg_chunk_count_kernel<<<grid, DOK_TPB, 0, s>>>(d, g, offs, n_chunks);
  dok_scan_kernel<<<1, 1024, 0, s>>>(offs, n_chunks, nullptr, count_out);
  if (keys_out || values_out) {
    if (cols) tg_chunk_write_kernel<true><<<grid, DOK_TPB, 0, s>>>(d, g, offs, n_chunks, (u8 *)keys_out, (u8 *)values_out, cap);
    else tg_chunk_write_kernel<false><<<grid, DOK_TPB, 0, s>>>(d, g, offs, n_chunks, (u8 *)keys_out, (u8 *)values_out, cap);
  }
  return DOK_OK;
}

static int tg_launch_to_dense(const DevTable &d, void *dense, i64 n_chunks, hipStream_t s) {
  TgGeom g;
  int rc = tg_geom(d, nullptr, g);
  if (rc) return rc;
  if (!tg_aligned(dense, g.V)) return DOK_EINVAL;
  TgDenseStrides st;
  memset(&st, 0, sizeof(st));
  i64 vol = 1;
  for (int k = d.lin_ndim - 1; k >= 0; k--) { st.s[k] = vol; vol *= d.lin_dims[k]; }
  tg_to_dense_kernel<<<(unsigned)((n_chunks + 3) / 4), DOK_TPB, 0, s>>>(d, g, st, (u8 *)dense, n_chunks);
  return DOK_OK;
}
