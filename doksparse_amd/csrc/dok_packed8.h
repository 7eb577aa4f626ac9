// Packed layout: keys of at most 8 bytes, values of 1, 2, 4 or 8 bytes.
//
// A 128-byte bucket holds S = 120 / (8 + V) slots and one metadata word:
//     words 0 .. S-1           the S stored key words (8 bytes each)
//     bytes 8*S .. 8*S + V*S   the S values, value s at byte 8*S + V*s
//     word 15                  metadata about the keys whose HOME is this bucket:
//                              bits 1..31  displacement map: bit d set = some key was placed d
//                                          buckets past this one
//                              bit 0       a key was placed 32 or more buckets past this one
//                              bits 32..39 the largest such far displacement, 255 standing for
//                                          "255 or more" (the walk then ends at the first bucket
//                                          with an EMPTY slot)
//                              bits 40..63 filter: every key placed away from this bucket sets the
//                                          bit its hash selects; a lookup whose bit is clear
//                                          cannot be a displaced key and ends at the home bucket
// (V=4: 10 slots, V=8: 7, V=2: 12, V=1: 13).  The stored key word is  key XOR DOK_P8_XOR,
// and the two words 0 and 1 mean EMPTY and TOMBSTONE, so a cleared table is all zero bytes and
// the slot word itself is the target of the claiming 64-bit compare-and-swap: an insert is one
// CAS plus one value store into the same line.  The two keys whose stored word would be 0 or 1
// live in two side slots of the table header instead (state word + value word each).
//
// Placement is linear probing over buckets: a new key goes to the first tombstone on its chain,
// else to the first empty slot, where the chain h, h+1, ... ends at the first bucket that still
// has an EMPTY slot (a bucket never regains one: remove leaves a TOMBSTONE).  A lookup does not
// walk that chain: after the home bucket it visits exactly the displacements marked in the home
// bucket's map, and those loads do not depend on each other.  Most home buckets never
// overflowed, so most misses are decided by the home bucket alone, also in a nearly full table.
#pragma once
#include "dok_device.h"

#define DOK_P8_XOR   0x9E3779B97F4A7C15ULL
#define DOK_P8_EMPTY 0ULL
#define DOK_P8_TOMB  1ULL
#define DOK_P8_META  15       // word index of the bucket metadata
#define DOK_H_SIDE_STATE 8    // header words 8,9: side slot occupied (0/1)
#define DOK_H_SIDE_VALUE 10   // header words 10,11: side slot values

template <int V> struct P8 {
  static constexpr int S = 120 / (8 + V);
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

// Hash of a stored key word.  Its upper half picks the home bucket, its lower half the filter bit.
__device__ __forceinline__ u64 p8_hash(u64 sk, const DevTable &t) { return dok_fmix64(sk ^ t.seed); }
__device__ __forceinline__ u32 p8_home(u64 sk, const DevTable &t) { return dok_reduce(p8_hash(sk, t), t.nb); }

#define DOK_P8_FARCAP 255u
#define DOK_P8_FBITS 24
// The key's bit among bits 8..31 of the metadata word's upper half.
__device__ __forceinline__ u32 p8_fidx(u64 h) { return (((u32)h & 0xffffu) * DOK_P8_FBITS) >> 16; }
__device__ __forceinline__ u32 p8_fbit(u64 h) { return 256u << p8_fidx(h); }

// Record in the home bucket's metadata word (global memory or an LDS copy) that a key with filter
// bit `fbit` was placed d > 0 buckets further on.  `seen`: a view of the word taken earlier (0 if
// none) - what it already shows need not be written again.
__device__ __forceinline__ void p8_mark(u64 *meta, u32 d, u32 fbit, u64 seen) {
  const u64 want = ((u64)fbit << 32) | (d < 32 ? 1ULL << d : 1ULL);
  if ((seen & want) != want) atomicOr(meta, want);
  if (d >= 32) {
    u32 *hi = (u32 *)meta + 1;
    const u32 dm = d < DOK_P8_FARCAP ? d : DOK_P8_FARCAP;
    u32 old = *(volatile u32 *)hi;
    while ((old & 0xffu) < dm) {
      const u32 prev = atomicCAS(hi, old, (old & ~0xffu) | dm);
      if (prev == old) break;
      old = prev;
    }
  }
}

// Keeps the compiler from hoisting the 16 per-round "is this my row" masks out of the tile loop
// (32 scalar registers that then spill) and from interleaving the rounds (which keeps every
// round's ballot masks alive at once).
#define DOK_OPAQUE(v) asm volatile("" : "+v"(v))
#define DOK_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// ---- shared pieces of the cooperative probe ---------------------------------------------------

// Lane geometry of the 16-lane probe groups of a wave64.
struct P8Lane {
  int lane, gbase, l;
  bool upper;        // lane >= 32: the group's ballot bits sit in the high word
  int sh;            // bit offset of the group inside that word (0 or 16)
  __device__ __forceinline__ P8Lane() {
    lane = threadIdx.x & 63;
    gbase = lane & 48;
    l = lane & 15;
    upper = lane >= 32;
    sh = lane & 16;
  }
  // the 16 ballot bits that belong to this lane's group
  __device__ __forceinline__ u32 group(u64 m) const {
    const u32 x = upper ? (u32)(m >> 32) : (u32)m;
    return (x >> sh) & 0xffffu;
  }
};

// One probe of one bucket by one group: which slots hold `q`, which are EMPTY / TOMBSTONE.
// Masks are restricted to the S key lanes on the scalar side.
template <int V> struct P8Probe {
  static constexpr u64 KEY_LANES = ((1ULL << P8<V>::S) - 1ULL) * 0x0001000100010001ULL;
  u32 gm, ge, gt;
  __device__ __forceinline__ void match(const P8Lane &L, u64 w, u64 q) {
    gm = L.group(__builtin_amdgcn_ballot_w64(w == q) & KEY_LANES);
    ge = L.group(__builtin_amdgcn_ballot_w64(w == DOK_P8_EMPTY) & KEY_LANES);
  }
  __device__ __forceinline__ void tombs(const P8Lane &L, u64 w) {
    gt = L.group(__builtin_amdgcn_ballot_w64(w == DOK_P8_TOMB) & KEY_LANES);
  }
  // index of the matching slot, 16 if none
  __device__ __forceinline__ int slot() const { return __builtin_ctz(gm | 0x10000u); }
};

// Which free slot of a bucket a key claims.  Each key scans the slots in a cyclic order of its
// own (start = a cheap hash of the key), so that rows racing for one bucket mostly claim
// different slots.  Equal keys share the order, and because free slots only become fewer while
// an insert kernel runs, the first free slot in a fixed order is the same for every view that
// still shows it free: equal keys of one batch always end up competing for one slot, never
// claiming two.
template <int V> __device__ __forceinline__ int p8_slot_start(u64 sk) {
  const u32 x = ((u32)sk ^ (u32)(sk >> 32)) * 0x9E3779B1u;
  return (int)(((x >> 16) * (u32)P8<V>::S) >> 16);
}
__device__ __forceinline__ int p8_pick(u32 free_mask, int start) {   // free_mask != 0
  const u32 from = free_mask >> start;
  return from ? start + __builtin_ctz(from) : __builtin_ctz(free_mask);
}

// ---- cooperative lookup -------------------------------------------------------------------
// In: per-lane stored key `sk`, home bucket `b` (0 for rows that need no probe), `pend` (row
// needs a table probe).  Out: found / value for the lane's own row; slot_b / slot_s locate the
// matching slot; nprobe counts the buckets visited for the lane's row.
//
// Phase 1 serves the home bucket of each of the group's 16 rows.  It is written as "issue U
// loads, then resolve U rounds" with no branch in between, so that a wave keeps U*4 bucket
// lines in flight; everything a round decides is folded into the owner lane with selects
// (rows that need no probe are carried through it and their outcome discarded).
// Phase 2 serves the rows whose home bucket carries overflow marks: per turn every group takes
// up to DOK_P8_WL of its open rows and loads the next two marked buckets of each (independent
// loads), folds the outcomes into the owners, which then act together.  Two rows per turn
// measured best: most turns have few open rows and wider turns only add instructions.
#define DOK_P8_U 8
#define DOK_P8_WL 2  // rows per group per phase-2 turn of the lookup
#define DOK_P8_WI 4  // rows per group per phase-2 turn of the insert
// WANT_VALUE = false: the caller only needs to know whether and where the key is (removal, counts);
// the value is then not read, which takes one dependent load off every hit.
template <int V, bool WANT_VALUE = true>
__device__ __forceinline__ void p8_lookup(const u64 *__restrict__ buckets, u64 nb, u64 sk, u32 b, u32 fbit,
                                          bool pend, bool &found, u64 &val, u32 &slot_b,
                                          int &slot_s, int &nprobe) {
  const P8Lane L;
  const int gbase = L.gbase;
  int l = L.l;
  DOK_OPAQUE(l);
  const u32 home = b;
  u32 meta = 0, mhi = 0;        // the home bucket's metadata word
  bool open = false;            // row still unresolved after its home bucket
  slot_b = home;

  if (dok_ballot(pend) != 0) {
    // per-owner outcome of the row's own round, kept as plain words (lane-mask booleans would
    // occupy a scalar register pair per round)
    u32 my_gm = 0, my_ge = 0;
    u64 my_v = 0;
    #pragma unroll
    for (int r0 = 0; r0 < 16; r0 += DOK_P8_U) {
      u64 w[DOK_P8_U];
      #pragma unroll
      for (int u = 0; u < DOK_P8_U; u++) {
        const u32 qb = dok_shfl32(home, gbase + r0 + u);
        w[u] = buckets[(u64)qb * 16 + l];
      }
      #pragma unroll
      for (int u = 0; u < DOK_P8_U; u++) {
        const int r = r0 + u;
        const u64 q = dok_shfl64(sk, gbase + r);
        P8Probe<V> pr;
        pr.match(L, w[u], q);
        const u64 mw = dok_shfl64(w[u], gbase + DOK_P8_META);
        const bool mine = l == r;
        my_gm = mine ? pr.gm : my_gm;
        my_ge = mine ? pr.ge : my_ge;
        meta = mine ? (u32)mw : meta;
        mhi = mine ? (u32)(mw >> 32) : mhi;
        DOK_SCHED_FENCE();
      }
    }
    const bool hit1 = pend && my_gm != 0;
    const int s1 = __builtin_ctz(my_gm | 0x10000u);
    // the bucket line was fetched a moment ago: the owner reads the value of the matching slot
    // from it (cheaper than shuffling a value out of the group in every round)
    if (WANT_VALUE && hit1) {
      typedef typename ValT<V>::type T;
      my_v = *(const T *)((const char *)(buckets + (u64)home * 16) + 8 * P8<V>::S + V * s1);
    }
    if (pend) { found = hit1; slot_s = s1; if (hit1) val = my_v; }
    // a key placed away from its home has set its filter bit there: with the bit clear the
    // home bucket alone decides, whatever other keys it has sent on
    open = pend && my_gm == 0 && meta != 0 && (mhi & fbit) != 0;
    nprobe += pend;
  }

  // Phase 2: rows whose home bucket carries overflow marks.  `cand` holds the displacements still
  // to be visited; the far walk (displacements >= 32, rare even in a 97 % full table) follows.
  u32 cand = open ? (meta & ~1u) : 0u;
  bool far = open && (meta & 1u);
  u32 far_d = 32, far_max = mhi & 0xffu;
  // a saturated record: the far walk goes on to the first bucket with an EMPTY slot (or once round)
  const bool far_unb = far_max == DOK_P8_FARCAP;
  if (far_unb) far_max = nb > 0xffffffffULL ? 0xffffffffu : (u32)nb - 1u;
  bool hit2 = false;
  u64 pm = dok_ballot(open);
  while (pm != 0) {
    // every open row offers its next two buckets
    u32 d0 = 0, d1 = 0;
    if (open) {
      if (cand) {
        d0 = __builtin_ctz(cand);
        const u32 c2 = cand & (cand - 1);
        if (c2) d1 = __builtin_ctz(c2);
        else if (far && far_d <= far_max) d1 = far_d;
      } else {
        d0 = far_d;
        if (far_d + 1 <= far_max) d1 = far_d + 1;
      }
    }
    u64 t0 = (u64)home + d0, t1 = (u64)home + d1;
    const u32 b0 = (u32)(t0 >= nb ? t0 - nb : t0), b1 = (u32)(t1 >= nb ? t1 - nb : t1);
    u32 rest = L.group(pm);
    int rr[DOK_P8_WL];
    bool hs[DOK_P8_WL], h1[DOK_P8_WL];
    u64 w0[DOK_P8_WL], w1[DOK_P8_WL];
    #pragma unroll
    for (int k = 0; k < DOK_P8_WL; k++) {
      hs[k] = rest != 0;
      rr[k] = hs[k] ? __builtin_ctz(rest) : 0;
      rest &= rest - 1;
      const u32 qb0 = dok_shfl32(b0, gbase + rr[k]);
      const u32 qb1 = dok_shfl32(b1, gbase + rr[k]);
      h1[k] = hs[k] && dok_shfl32(d1, gbase + rr[k]) != 0;
      w0[k] = buckets[(u64)(hs[k] ? qb0 : 0u) * 16 + l];
      w1[k] = buckets[(u64)(h1[k] ? qb1 : 0u) * 16 + l];
    }
    bool act = false;
    u32 gm0 = 0, gm1 = 0, gee = 0;
    #pragma unroll
    for (int k = 0; k < DOK_P8_WL; k++) {
      const u64 q = dok_shfl64(sk, gbase + rr[k]);
      P8Probe<V> p0, p1;
      p0.match(L, w0[k], q);
      p1.match(L, w1[k], q);
      const bool mine = hs[k] && l == rr[k];
      act = act || mine;
      gm0 = mine ? p0.gm : gm0;
      gm1 = mine ? (h1[k] ? p1.gm : 0u) : gm1;
      gee = mine ? (p0.ge | (h1[k] ? p1.ge : 0u)) : gee;
    }
    if (act) {
      nprobe += 1 + (d1 != 0);
      if (gm0 | gm1) {
        hit2 = true; open = false;
        slot_b = gm0 ? b0 : b1;
        slot_s = __builtin_ctz(gm0 ? gm0 : gm1);
      } else {
        if (far_unb && cand == 0 && gee != 0) far = false;   // an EMPTY slot ends the unrecorded part of the chain
        // drop the visited displacements
        if (cand) {
          cand &= cand - 1;
          if (d1 != 0) { if (cand) cand &= cand - 1; else far_d++; }
        } else {
          far_d += 1 + (d1 != 0);
        }
        open = cand != 0 || (far && far_d <= far_max);
      }
    }
    pm = dok_ballot(open);
  }
  if (hit2) {
    typedef typename ValT<V>::type T;
    found = true;
    if (WANT_VALUE) val = *(const T *)((const char *)(buckets + (u64)slot_b * 16) + 8 * P8<V>::S + V * slot_s);
  }
}

// Side-slot lookup for the two reserved stored words.
__device__ __forceinline__ bool p8_side_get(const DevTable &t, u64 sk, u64 &val) {
  if (t.header[DOK_H_SIDE_STATE + sk] != 0) { val = (u64)t.header[DOK_H_SIDE_VALUE + sk]; return true; }
  return false;
}

// ---- cooperative upsert -------------------------------------------------------------------
// In: per-lane stored key, value, home bucket (0 for rows that need no probe), `pend`.
// Out: st (1 placed / 0 table full), fresh (took a new slot).
//
// The claim is one CAS on the slot's key word; whoever loses re-examines: if the winner wrote
// the same key (equal keys inside one batch) the loser is done and the winner's value stands,
// otherwise it walks again.  A key absent from the table takes the first tombstone on its chain,
// else the first empty slot of the chain-end bucket.  Because slots only ever move
// EMPTY/TOMBSTONE -> key inside a set kernel, two rows with the same key can never both win a
// claim: the later one either sees the earlier one's key or competes for the same slot.  The
// same monotonicity makes a stale (cached) view of a bucket harmless - it can only show a slot
// as free that is in fact taken, and the CAS then fails - so phase 1 uses plain loads; the
// retry loop reads device-coherently.
//
// Phase 1 inspects the home bucket of all 64 rows (batched loads as in the lookup), then the
// whole wave issues its CAS / value stores together.  Phase 2 is the general walk for rows whose
// home bucket was full or whose claim was lost, DOK_P8_WI rows per group per turn, the owners
// acting together.  A key placed d > 0 buckets past its home raises the home bucket's recorded largest
// displacement to d.
template <int V>
__device__ __forceinline__ void p8_insert(u64 *buckets, u64 nb, u64 sk, u64 val, u32 home, u32 fbit,
                                          bool pend, int &st, int &fresh) {
  const P8Lane L;
  const int gbase = L.gbase;
  int l = L.l;
  DOK_OPAQUE(l);

  int act1 = 0;                 // 0 walk on, 1 overwrite slot, 2 claim slot
  int slot = 0;
  u32 my_pick = 0;              // match mask, else tombstone mask, else empty mask of the home bucket
  bool tomb_here = false;       // the chosen slot of the home bucket is a tombstone
  u32 md_home = 0;

  if (dok_ballot(pend) != 0) {
    #pragma unroll
    for (int r0 = 0; r0 < 16; r0 += DOK_P8_U) {
      u64 w[DOK_P8_U];
      #pragma unroll
      for (int u = 0; u < DOK_P8_U; u++) {
        const u32 qb = dok_shfl32(home, gbase + r0 + u);
        w[u] = buckets[(u64)qb * 16 + l];
      }
      #pragma unroll
      for (int u = 0; u < DOK_P8_U; u++) {
        const int r = r0 + u;
        const u64 q = dok_shfl64(sk, gbase + r);
        P8Probe<V> pr;
        pr.match(L, w[u], q);
        pr.tombs(L, w[u]);
        const u32 md = dok_shfl32((u32)w[u], gbase + DOK_P8_META);
        const bool mine = l == r;
        const int a = pr.gm ? 1 : (pr.ge ? 2 : 0);
        const u32 pick = pr.gm ? pr.gm : (pr.gt ? pr.gt : pr.ge);
        act1 = mine ? a : act1;
        my_pick = mine ? pick : my_pick;
        tomb_here = mine ? (pr.gm == 0 && pr.gt != 0) : tomb_here;
        md_home = mine ? md : md_home;
        DOK_SCHED_FENCE();
      }
    }
  }

  const int start = p8_slot_start<V>(sk);
  if (act1 == 1) slot = __builtin_ctz(my_pick);
  else if (my_pick) slot = p8_pick(my_pick, start);
  u64 *hb = buckets + (u64)home * 16;
  u32 b = home, d = 0;
  u32 tomb_b = DOK_NONE32, tomb_d = 0;
  int tomb_s = 0;
  u64 iters = 0;
  if (pend && act1 == 1) {
    P8<V>::store(hb, slot, val);
    st = 1; pend = false;
  } else if (pend && act1 == 2) {
    const u64 expect = tomb_here ? DOK_P8_TOMB : DOK_P8_EMPTY;
    const u64 old = atomicCAS(hb + slot, expect, sk);
    if (old == expect) { P8<V>::store(hb, slot, val); st = 1; fresh = 1; pend = false; }
    else if (old == sk) { st = 1; pend = false; }
    // else: lost to another key; phase 2 starts over at the home bucket
  } else if (pend) {
    // home bucket full without a match: walk on, remembering its first tombstone
    if (tomb_here) { tomb_b = home; tomb_s = slot; tomb_d = 0; }
    b = (home + 1 == nb) ? 0u : home + 1;
    d = 1; iters = 1;
  }

  u64 pm = dok_ballot(pend);
  while (pm != 0) {
    u32 rest = L.group(pm);
    int rr[DOK_P8_WI];
    bool hs[DOK_P8_WI];
    u64 w[DOK_P8_WI];
    #pragma unroll
    for (int k = 0; k < DOK_P8_WI; k++) {
      hs[k] = rest != 0;
      rr[k] = hs[k] ? __builtin_ctz(rest) : 0;
      rest &= rest - 1;
      const u32 qb = dok_shfl32(b, gbase + rr[k]);
      w[k] = dok_load_coherent(buckets + (u64)(hs[k] ? qb : 0u) * 16 + l);
    }
    bool act = false;
    u32 gm = 0, ge = 0, gt = 0;
    #pragma unroll
    for (int k = 0; k < DOK_P8_WI; k++) {
      const u64 q = dok_shfl64(sk, gbase + rr[k]);
      P8Probe<V> pr;
      pr.match(L, w[k], q);
      pr.tombs(L, w[k]);
      const bool mine = hs[k] && l == rr[k];
      act = act || mine;
      gm = mine ? pr.gm : gm;
      ge = mine ? pr.ge : ge;
      gt = mine ? pr.gt : gt;
    }
    if (act) {
      if (gm) {
        // key present: overwrite its value in place
        P8<V>::store(buckets + (u64)b * 16, __builtin_ctz(gm), val);
        st = 1; pend = false;
      } else {
        if (tomb_b == DOK_NONE32 && gt) { tomb_b = b; tomb_s = p8_pick(gt, start); tomb_d = d; }
        const bool ring_done = (ge == 0) && (++iters >= nb);
        if (ge || ring_done) {
          // chain end: the key is absent
          if (tomb_b == DOK_NONE32 && ge == 0) {
            st = 0; pend = false;                       // no free slot anywhere
          } else {
            u32 tb, td; int ts; u64 expect;
            if (tomb_b != DOK_NONE32) { tb = tomb_b; ts = tomb_s; td = tomb_d; expect = DOK_P8_TOMB; }
            else { tb = b; ts = p8_pick(ge, start); td = d; expect = DOK_P8_EMPTY; }
            u64 *tp = buckets + (u64)tb * 16;
            const u64 old = atomicCAS(tp + ts, expect, sk);
            if (old == expect) {
              P8<V>::store(tp, ts, val);
              // mark the displacement and the key's filter bit in the home bucket's metadata
              if (td > 0) p8_mark(hb + DOK_P8_META, td, fbit, 0);
              st = 1; fresh = 1; pend = false;
            } else if (old == sk) {
              st = 1; pend = false;                     // an equal key of this batch won the slot
            } else {
              b = home; d = 0; tomb_b = DOK_NONE32; iters = 0;   // somebody else's key: look again
            }
          }
        } else {
          b = (b + 1 == nb) ? 0u : b + 1;
          d++;
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
template <int V, bool STATS, int KF>
__global__ __launch_bounds__(DOK_TPB) void p8_get_kernel(DevTable t, const void *__restrict__ keys, i64 n,
                                                         void *__restrict__ values, u8 *__restrict__ found_out,
                                                         u64 fallback, const void *__restrict__ fallback_dev) {
  // the fallback value: an immediate, or - fallback_dev set - read from device memory by the kernel
  // itself, as the reference's kernel reads its fallback array
  if (fallback_dev) fallback = dok_load_val<V>(fallback_dev, 0);
  int n_probe = 0, n_ops = 0;
  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool active = i < n;
    u64 key = 0;
    const bool ok = active && dok_load_key8<KF>(t, keys, i, n, key);
    const u64 sk = key ^ DOK_P8_XOR;
    bool found = false;
    u64 val = fallback;
    bool pend = ok;
    if (ok && sk < 2) { found = p8_side_get(t, sk, val); pend = false; }
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V>(t.buckets, t.nb, sk, pend ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), pend, found, val, sb, ss, nprobe);
    if (active) {
      dok_store_val<V>(values, i, val);
      found_out[i] = found ? 1 : 0;
    }
    n_probe += nprobe;
    n_ops += active;
  }
  if (STATS) {
    dok_block_add2(&t.header[DOK_H_NPROBE], n_probe, &t.header[DOK_H_NOPS], n_ops);
  }
}

#define DOK_STREAM_WAVES 8   // waves per SIMD the streaming kernels are compiled for
// Streaming insert.  Every lane carries one row at some point of its walk (bucket home + d); a
// pass loads the current bucket of all 64 rows (batched as in phase 1 of p8_insert), the owners
// decide and claim together, and lanes whose row is finished take the next rows of the wave's
// contiguous share [wave * rows_per_wave, (wave + 1) * rows_per_wave) of the n rows.  A row that
// has to walk on therefore costs the wave one more bucket load in a later pass instead of a turn
// of its own, and the number of bucket lines in flight does not drop when the table is nearly
// full (at load factor 0.9 this is 1.3x faster than tile-wise p8_insert).  All loads are
// device-coherent, so a row that lost its claim to another key simply looks again, from the
// bucket of the slot it lost, in the next pass.
// A row's place is the first free slot of its walk (a tombstone of that bucket before an EMPTY
// slot), as in p8_insert.  That the key is not in the table further on is not established by
// walking to the chain's end - in a table with many tombstones that end is far away - but
// through the home bucket's displacement map: a key with this home can only sit at a marked
// displacement, so the marked buckets beyond the chosen slot are looked at and then the slot is
// claimed.  (Without removals there are none: the first free slot is the chain's end.)
//
// `src(i, key, val)` produces row i: 0 = insert key -> val, 1 = the row addresses nothing inside
// the table's coordinate space (counted, reported as not stored), 2 = skip the row silently.
// The header counters are updated once per workgroup at the end (dok_block_add3: every thread of
// the workgroup has to reach the end of this function, exactly once per kernel).
// The core works through the rows [next, end) that the caller assigns to this wave.
// RETRY: see the claim below; switched on where it costs no registers (it takes three more in the
// indexing kernel, which already spills).
template <int V, bool RETRY = false, class Src>
__device__ __forceinline__ void p8_stream_insert_rows(const DevTable &t, i64 next, i64 end,
                                                      u8 *__restrict__ stored, Src src) {
  const P8Lane L;
  const int gbase = L.gbase;
  int l = L.l;
  DOK_OPAQUE(l);
  u64 *const buckets = t.buckets;
  const u64 nb = t.nb;

  int n_fresh = 0, n_full = 0, n_oob = 0;
  bool act = false;
  u64 sk = 0, val = 0;
  i64 idx = 0;
  u32 home = 0, fbit = 0, d = 0, md_home = 0, far_home = 0;
  // once the walk has met a free slot: the slot, and what is left to look at before the claim
  bool chosen = false, slot_tomb = false, far_unb = false;
  u32 slot_d = 0, cd = 0, chk = 0, far_next = 0, far_to = 0;
  int slot_s = 0;

  for (;;) {
    // ---- lanes without a row take the next rows of the wave's share
    const u64 freem = dok_ballot(!act);
    if (!act) {
      const int rank = __builtin_amdgcn_mbcnt_hi((u32)(freem >> 32), __builtin_amdgcn_mbcnt_lo((u32)freem, 0u));
      const i64 i = next + rank;
      if (i < end) {
        u64 key = 0;
        const int code = src(i, key, val);
        sk = key ^ DOK_P8_XOR;
        if (code == 1) {
          n_oob++;
          if (stored) stored[i] = 0;
        } else if (code == 0) {
          if (sk < 2) {
            n_fresh += p8_side_set(t, sk, val);
            if (stored) stored[i] = 1;
          } else {
            const u64 h = p8_hash(sk, t);
            act = true; idx = i; home = dok_reduce(h, nb); fbit = p8_fbit(h); d = 0; chosen = false;
          }
        }
      }
    }
    next += __popcll(freem);
    if (next > end) next = end;
    if (dok_ballot(act) == 0) {
      if (next >= end) break;
      continue;
    }

    // ---- one pass: the current bucket of every row (the next bucket of its walk, or - once it
    // has chosen a slot - the next bucket its home marks beyond that slot)
    const u32 dcur = chosen ? cd : d;
    u32 b = 0;
    if (act) {
      const u64 bb = (u64)home + dcur;
      b = (u32)(bb >= nb ? bb - nb : bb);
    }
    u32 gm = 0, ge = 0, gt = 0, md = 0, mh = 0;
    const u64 actm = dok_ballot(act);
    const u32 rows_on = L.group(actm);               // lanes without a row load nothing
    u32 rounds_on = (u32)actm | (u32)(actm >> 32);   // rounds in which no group has a row are skipped
    rounds_on = (rounds_on | (rounds_on >> 16)) & 0xffffu;
    #pragma unroll
    for (int r0 = 0; r0 < 16; r0 += DOK_P8_U) {
      u64 w[DOK_P8_U];
      #pragma unroll
      for (int u = 0; u < DOK_P8_U; u++) {
        w[u] = 0;
        if ((rounds_on >> (r0 + u)) & 1u) {
          const u32 qb = dok_shfl32(b, gbase + r0 + u);
          if ((rows_on >> (r0 + u)) & 1u) w[u] = dok_load_coherent(buckets + (u64)qb * 16 + l);
        }
      }
      #pragma unroll
      for (int u = 0; u < DOK_P8_U; u++) {
        const int r = r0 + u;
        if (!((rounds_on >> r) & 1u)) continue;
        const u64 q = dok_shfl64(sk, gbase + r);
        P8Probe<V> pr;
        pr.match(L, w[u], q);
        pr.tombs(L, w[u]);
        const u64 mw = dok_shfl64(w[u], gbase + DOK_P8_META);
        const bool mine = l == r;
        gm = mine ? pr.gm : gm;
        ge = mine ? pr.ge : ge;
        gt = mine ? pr.gt : gt;
        md = mine ? (u32)mw : md;
        mh = mine ? (u32)(mw >> 32) : mh;
        DOK_SCHED_FENCE();
      }
    }

    // ---- the owners act together
    if (act) {
      int st = -1;                                   // -1 the row goes on, 0 failed, 1 stored
      bool claim = false;
      if (gm) {
        P8<V>::store(buckets + (u64)b * 16, __builtin_ctz(gm), val);
        st = 1;
      } else if (!chosen) {
        if (d == 0) { md_home = md; far_home = mh; }
        if (gt | ge) {
          // The first free slot of the walk is the row's place (a tombstone of the bucket before
          // an EMPTY slot).  The key may still sit further on: exactly at the displacements the
          // home bucket marks, so those beyond this bucket are looked at before the claim.
          const int start = p8_slot_start<V>(sk);
          chosen = true;
          slot_tomb = gt != 0;
          slot_d = d;
          slot_s = p8_pick(gt ? gt : ge, start);
          chk = d < 31 ? (md_home & ~((2u << d) - 1u)) : 0u;
          far_next = d + 1 > 32u ? d + 1 : 32u;
          far_to = (md_home & 1u) ? (far_home & 0xffu) : 0u;
          far_unb = far_to == DOK_P8_FARCAP;
          if (far_unb) far_to = nb > 0xffffffffULL ? 0xffffffffu : (u32)nb - 1u;
          // without the key's filter bit in its home bucket the key was never placed elsewhere
          if (!(far_home & fbit)) { chk = 0; far_to = 0; }
        } else if ((u64)d + 1 >= nb) {
          st = 0;                                    // no free slot anywhere
        } else {
          d++;
        }
      }
      else if (far_unb && cd >= 32u && ge) {
        far_to = 0;                                    // an EMPTY slot ends the unrecorded part of the chain
      }
      if (st < 0 && chosen) {
        if (chk) { cd = (u32)__builtin_ctz(chk); chk &= chk - 1; }
        else if (far_next <= far_to) cd = far_next++;
        else claim = true;
      }
      if (claim) {
        const u32 td = slot_d;
        const u64 expect = slot_tomb ? DOK_P8_TOMB : DOK_P8_EMPTY;
        const u64 tbb = (u64)home + td;
        u64 *tp = buckets + (tbb >= nb ? tbb - nb : tbb) * 16;
        u64 old = atomicCAS(tp + slot_s, expect, sk);
        if (RETRY && dcur == td) {
          // The claim follows the choice in the same pass (nothing marked to look at first), so the
          // pass's view of the slot's bucket is still at hand: a slot lost to another key is
          // followed at once by the other free slots of the same kind that the view showed, in the
          // order every row of this key tries them, instead of by another pass that loads the
          // bucket again.  (Rows that arrive at one bucket together - a batch that is large
          // against a small table - otherwise pay a load and a claim, one after the other, per
          // lost slot.)
          u32 cand = (slot_tomb ? gt : ge) & ~(1u << slot_s);
          while (old != expect && old != sk && cand != 0) {
            slot_s = p8_pick(cand, p8_slot_start<V>(sk));
            cand &= ~(1u << slot_s);
            old = atomicCAS(tp + slot_s, expect, sk);
          }
        }
        if (old == expect) {
          P8<V>::store(tp, slot_s, val);
          if (td > 0) p8_mark(buckets + (u64)home * 16 + DOK_P8_META, td, fbit, ((u64)far_home << 32) | md_home);
          st = 1; n_fresh++;
        } else if (old == sk) {
          st = 1;                                    // an equal key of this batch won the slot
        } else {
          // somebody else's key took the slot.  Every bucket before the slot's own held
          // neither a free slot nor this key when the row passed it, and buckets only fill up,
          // so the row need not go back further than that bucket
          chosen = false;
          d = td;
        }
      }
      if (st >= 0) {
        if (stored) stored[idx] = (u8)st;
        n_full += (st == 0);
        act = false;
      }
    }
  }
  dok_block_add3(&t.header[DOK_H_NELEM], n_fresh, &t.header[DOK_H_NFULL], n_full, &t.header[DOK_H_NOOB], n_oob);
}

// Rows [0, n) split into one contiguous share per wave of the grid.
template <int V, bool RETRY = false, class Src>
__device__ __forceinline__ void p8_stream_insert(const DevTable &t, i64 n, i64 rows_per_wave,
                                                 u8 *__restrict__ stored, Src src) {
  const i64 wave = ((i64)blockIdx.x * DOK_TPB + threadIdx.x) >> 6;
  i64 next = wave * rows_per_wave;
  i64 end = next + rows_per_wave;
  if (end > n) end = n;
  if (next > end) next = end;
  p8_stream_insert_rows<V, RETRY>(t, next, end, stored, src);
}

template <int V, int KF>
__global__ __launch_bounds__(DOK_TPB, DOK_STREAM_WAVES) void p8_set_kernel(DevTable t, const void *__restrict__ keys,
                                                         const void *__restrict__ values, i64 n,
                                                         u8 *__restrict__ stored, i64 rows_per_wave) {
  p8_stream_insert<V, KF == DOK_KF_RAW>(t, n, rows_per_wave, stored, [&](i64 i, u64 &key, u64 &val) -> int {
    if (!dok_load_key8<KF>(t, keys, i, n, key)) return 1;
    val = dok_load_val<V>(values, i);
    return 0;
  });
}

// Tombstone the matching slot: with a CAS, so that equal keys in one batch remove it once, or -
// UNIQUE: the caller vouches that the batch holds no key twice - with a plain store, as the
// reference does after its host-side unique (one returning atomic in HBM less per row).
template <int V, int KF, bool UNIQUE>
__global__ __launch_bounds__(DOK_TPB) void p8_remove_kernel(DevTable t, const void *__restrict__ keys, i64 n,
                                                            u8 *__restrict__ removed_out) {
  int n_removed = 0;
  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool active = i < n;
    u64 key = 0;
    const bool ok = active && dok_load_key8<KF>(t, keys, i, n, key);
    const u64 sk = key ^ DOK_P8_XOR;
    bool found = false, removed = false;
    u64 val = 0;
    bool pend = ok;
    if (ok && sk < 2) {
      removed = atomicExch((u64 *)&t.header[DOK_H_SIDE_STATE + sk], 0ULL) != 0;
      pend = false;
    }
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V, false>(t.buckets, t.nb, sk, pend ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), pend, found, val, sb, ss, nprobe);
    if (found) {
      if (UNIQUE) { t.buckets[(u64)sb * 16 + ss] = DOK_P8_TOMB; removed = true; }
      else removed = atomicCAS(t.buckets + (u64)sb * 16 + ss, sk, DOK_P8_TOMB) == sk;
    }
    if (active && removed_out) removed_out[i] = removed ? 1 : 0;
    n_removed += removed;
  }
  dok_block_add1(&t.header[DOK_H_NELEM], -n_removed);
}

template <int V, int KF>
__global__ __launch_bounds__(DOK_TPB) void p8_count_kernel(DevTable t, const void *__restrict__ keys, i64 n,
                                                           i64 *count) {
  int n_found = 0;
  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool active = i < n;
    u64 key = 0;
    const bool ok = active && dok_load_key8<KF>(t, keys, i, n, key);
    const u64 sk = key ^ DOK_P8_XOR;
    bool found = false;
    u64 val = 0;
    bool pend = ok;
    if (ok && sk < 2) { found = p8_side_get(t, sk, val); pend = false; }
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V, false>(t.buckets, t.nb, sk, pend ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), pend, found, val, sb, ss, nprobe);
    n_found += found;
  }
  dok_block_add1(count, n_found);
}

// The keys of the batch that are present get their values overwritten; the others are only counted
// (missing[0] += their number) and nothing is inserted.  A batch of nothing but present keys - the
// usual update of a map - is then done in one pass at the rate of a lookup, with no compare-and-swap.
// (Equal keys in the batch store into one slot, each store a whole value.)
template <int V, int KF>
__global__ __launch_bounds__(DOK_TPB) void p8_update_kernel(DevTable t, const void *__restrict__ keys,
                                                            const void *__restrict__ values, i64 n, i64 *missing) {
  int n_missing = 0;
  DOK_TILE_LOOP(n) {
    const i64 i = DOK_TILE_ROW();
    const bool active = i < n;
    u64 key = 0;
    const bool ok = active && dok_load_key8<KF>(t, keys, i, n, key);
    const u64 sk = key ^ DOK_P8_XOR;
    const u64 mine = ok ? dok_load_val<V>(values, i) : 0;
    bool found = false;
    u64 val = 0;
    bool pend = ok;
    if (ok && sk < 2) {
      found = t.header[DOK_H_SIDE_STATE + sk] != 0;
      if (found) t.header[DOK_H_SIDE_VALUE + sk] = (i64)mine;
      pend = false;
    }
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V, false>(t.buckets, t.nb, sk, pend ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), pend, found, val, sb, ss, nprobe);
    if (pend && found) P8<V>::store(t.buckets + (u64)sb * 16, ss, mine);
    n_missing += active && !found;             // (a row outside the coordinate space is not present either)
  }
  dok_block_add1(missing, n_missing);
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
  // unconditional load (clamped) so that the unrolled scan loops keep several in flight
  w = t.buckets[(u64)(valid ? b : (i64)t.nb - 1) * 16 + l];
  return valid && l < P8<V>::S && w >= 2;
}

template <int V>
__global__ __launch_bounds__(DOK_TPB) void p8_chunk_count_kernel(DevTable t, i64 *chunk_counts, i64 n_chunks) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const int lane = threadIdx.x & 63;
  i64 cnt = 0;
  #pragma unroll 8
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
  // eight consecutive counts per thread and round: the rounds are serial (barriers, a carry), so
  // fewer and fatter ones
  for (i64 base = 0; base < n; base += 8 * 1024) {
    const i64 i0 = base + (i64)tid * 8;
    i64 v[8], sum = 0;
    #pragma unroll
    for (int k = 0; k < 8; k++) v[k] = i0 + k < n ? counts[i0 + k] : 0;
    #pragma unroll
    for (int k = 0; k < 8; k++) { const i64 x = v[k]; v[k] = sum; sum += x; }
    i64 inc = sum;
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
    const i64 excl = carry + wpre + inc - sum;
    #pragma unroll
    for (int k = 0; k < 8; k++)
      if (i0 + k < n) counts[i0 + k] = excl + v[k];
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

template <int V, int KF>
__global__ __launch_bounds__(DOK_TPB) void p8_chunk_write_kernel(DevTable t, const i64 *chunk_offsets, i64 n_chunks,
                                                                 void *keys_out, void *values_out, i64 cap) {
  const i64 wid = (i64)blockIdx.x * (DOK_TPB / 64) + (threadIdx.x >> 6);
  if (wid >= n_chunks) return;
  const int lane = threadIdx.x & 63;
  const int gbase = lane & 48, l = lane & 15;
  i64 base = chunk_offsets[wid];
  #pragma unroll 8
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live = p8_scan_load<V>(t, wid * DOK_CHUNK + s * 4 + (lane >> 4), w);
    const u64 m = dok_ballot(live);
    const int vw = l < P8<V>::S ? P8<V>::value_word(l) : 15;
    const u64 vword = dok_shfl64(w, gbase + vw);
    const i64 row = base + __popcll(m & ((1ULL << lane) - 1ULL));
    if (live && row < cap) {
      if (keys_out) dok_store_key8<KF>(t, keys_out, row, cap, w ^ DOK_P8_XOR);
      if (values_out) dok_store_val<V>(values_out, row, P8<V>::extract(vword, l));
    }
    base += __popcll(m);
  }
  // the two side slots come last
  if (KF == DOK_KF_RAW && wid == 0 && lane == 0) {
    i64 row = chunk_offsets[n_chunks];
    for (u64 k = 0; k < 2; k++) {
      if (t.header[DOK_H_SIDE_STATE + k] != 0) {
        if (row < cap) {
          if (keys_out) dok_store_key8<KF>(t, keys_out, row, cap, k ^ DOK_P8_XOR);
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
  #pragma unroll 8
  for (int s = 0; s < DOK_CHUNK / 4; s++) {
    u64 w;
    const bool live = p8_scan_load<V>(src, wid * DOK_CHUNK + s * 4 + (lane >> 4), w);
    const int vw = l < P8<V>::S ? P8<V>::value_word(l) : 15;
    const u64 val = P8<V>::extract(dok_shfl64(w, gbase + vw), l);
    int st = 0, fresh = 0;
    const u64 h = p8_hash(w, dst);
    p8_insert<V>(dst.buckets, dst.nb, w, val, live ? dok_reduce(h, dst.nb) : 0u, p8_fbit(h), live, st, fresh);
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
  #pragma unroll 8
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

template <int V, class IX>
__global__ __launch_bounds__(DOK_TPB) void p8_getitem_kernel(DevTable t, IX ix, void *__restrict__ out) {
  DOK_TILE_LOOP(ix.n_elems) {
    const i64 e = DOK_TILE_ROW();
    const bool active = e < ix.n_elems;
    u64 key = 0; i64 voff = 0;
    const bool ok = active && dok_gather_key(t, ix, e, key, voff);
    const u64 sk = key ^ DOK_P8_XOR;
    bool found = false;
    u64 val = 0;
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V>(t.buckets, t.nb, sk, ok ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), ok, found, val, sb, ss, nprobe);
    if (active) dok_store_val<V>(out, e, val);
  }
}

template <int V, class IX>
__global__ __launch_bounds__(DOK_TPB, DOK_STREAM_WAVES) void p8_setitem_kernel(DevTable t, IX ix, i64 rows_per_wave) {
  p8_stream_insert<V>(t, ix.n_elems, rows_per_wave, nullptr, [&](i64 e, u64 &key, u64 &val) -> int {
    i64 voff = 0;
    if (!dok_gather_key(t, ix, e, key, voff)) return 1;
    val = dok_load_val<V>(ix.src, voff);
    return 0;
  });
}

template <int V, class IX>
__global__ __launch_bounds__(DOK_TPB) void p8_countitems_kernel(DevTable t, IX ix, i64 *count) {
  int n_found = 0;
  DOK_TILE_LOOP(ix.n_elems) {
    const i64 e = DOK_TILE_ROW();
    const bool active = e < ix.n_elems;
    u64 key = 0; i64 voff = 0;
    const bool ok = active && dok_gather_key(t, ix, e, key, voff);
    const u64 sk = key ^ DOK_P8_XOR;
    bool found = false;
    u64 val = 0;
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V, false>(t.buckets, t.nb, sk, ok ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), ok, found, val, sb, ss, nprobe);
    n_found += found;
  }
  dok_block_add1(count, n_found);
}

template <int V, class IX>
__global__ __launch_bounds__(DOK_TPB) void p8_zeroitems_kernel(DevTable t, IX ix) {
  int n_removed = 0;
  DOK_TILE_LOOP(ix.n_elems) {
    const i64 e = DOK_TILE_ROW();
    const bool active = e < ix.n_elems;
    u64 key = 0; i64 voff = 0;
    const bool ok = active && dok_gather_key(t, ix, e, key, voff);
    const u64 sk = key ^ DOK_P8_XOR;
    bool found = false, removed = false;
    u64 val = 0;
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V, false>(t.buckets, t.nb, sk, ok ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), ok, found, val, sb, ss, nprobe);
    if (found) removed = atomicCAS(t.buckets + (u64)sb * 16 + ss, sk, DOK_P8_TOMB) == sk;
    n_removed += removed;
  }
  dok_block_add1(&t.header[DOK_H_NELEM], -n_removed);
}

// Sparse-valued getitem: every element of the index space whose coordinate is stored in `t` is
// inserted into `out`, a coordinate-keyed table over the index space itself (key = e).
template <int V, class IX>
__global__ __launch_bounds__(DOK_TPB) void p8_getitem_sparse_kernel(DevTable t, IX ix, DevTable out) {
  int n_fresh = 0, n_full = 0;
  DOK_TILE_LOOP(ix.n_elems) {
    const i64 e = DOK_TILE_ROW();
    const bool active = e < ix.n_elems;
    u64 key = 0; i64 voff = 0;
    const bool ok = active && dok_gather_key(t, ix, e, key, voff);
    const u64 sk = key ^ DOK_P8_XOR;
    bool found = false;
    u64 val = 0;
    u32 sb = 0; int ss = 0, nprobe = 0;
    const u64 h = p8_hash(sk, t);
    p8_lookup<V>(t.buckets, t.nb, sk, ok ? dok_reduce(h, t.nb) : 0u, p8_fbit(h), ok, found, val, sb, ss, nprobe);
    const u64 ok2 = (u64)e ^ DOK_P8_XOR;
    int st = 0, fresh = 0;
    const u64 h2 = p8_hash(ok2, out);
    p8_insert<V>(out.buckets, out.nb, ok2, val, found ? dok_reduce(h2, out.nb) : 0u, p8_fbit(h2), found, st, fresh);
    n_fresh += fresh;
    n_full += (found && st == 0);
  }
  dok_block_add2(&out.header[DOK_H_NELEM], n_fresh, &out.header[DOK_H_NFULL], n_full);
}

// Sparse-valued setitem: source entry k has index vector src_indices[j*n_src + k] (j over the
// axes of the index space) and value src_values[k]; entries whose value is zero under
// `nonzero_mask` (all ones for integers, sign bit cleared for floating values) are skipped.
template <int V, class IX>
__global__ __launch_bounds__(DOK_TPB, DOK_STREAM_WAVES) void p8_setitem_sparse_kernel(DevTable t, IX ix,
                                                                    const i64 *__restrict__ src_indices,
                                                                    const void *__restrict__ src_values,
                                                                    i64 n_src, u64 nonzero_mask,
                                                                    i64 rows_per_wave) {
  p8_stream_insert<V>(t, n_src, rows_per_wave, nullptr, [&](i64 k, u64 &key, u64 &val) -> int {
    i64 idx[IX::DIMS];
    bool inside = true;
    #pragma unroll
    for (int j = 0; j < IX::DIMS; j++) {
      idx[j] = 0;
      if (j < ix.sel_ndim) {
        idx[j] = src_indices[(i64)j * n_src + k];
        inside = inside && ((u64)idx[j] < (u64)ix.shape[j]);
      }
    }
    val = dok_load_val<V>(src_values, k);
    if ((val & nonzero_mask) == 0) return 2;
    i64 voff = 0;
    return (inside && dok_gather_at(t, ix, idx, key, voff)) ? 0 : 1;
  });
}
