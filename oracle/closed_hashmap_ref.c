/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * CPU restatement, in plain C, of the algorithm of the reference's batched
 * closed-hashing hashmap and of the DOK kernels that run on it.  It exists so
 * that (a) the HIP path can be checked against an independent implementation
 * of the reference semantics on the same seeded inputs and (b) the benchmark
 * can time "the reference algorithm on the host cores" beside the GPU number.
 * Nothing in the shipped package may link, load or call this file.
 *
 * What is restated (paths relative to the reference checkout):
 *   sparse_dok/components/cuda/closed_hashmap_impl_class.cu
 *       get_hash :87-96, get_uuid :98-107, exists :253-278, get :280-312,
 *       set :368-427 (incl. CAS helpers :183-209), remove :459-484
 *   sparse_dok/components/cuda/closed_hashmap_impl.cu
 *       closed_hashmap_get :7-85, closed_hashmap_set :88-156,
 *       closed_hashmap_remove :159-220   (one "thread" per key row)
 *   sparse_dok/components/cuda/tensor_accessor.cu
 *       get_offset :50-58, get_index_from_offset :82-87
 *   sparse_dok/components/cuda/sparse_dok_tensor_impl.cu
 *       sparse_dok_count_items :4-56, sparse_dok_zero_items :59-108,
 *       sparse_dok_get_items :111-160, sparse_dok_set_items_sparse_v1 :163-211,
 *       sparse_dok_set_items_dense :271-313
 *
 * Table layout is the reference's structure-of-arrays:
 *   uuid[B] int64 (-1 empty, -3 removed), keys[B][key_bytes], values[B][value_bytes].
 *
 * Deliberate, documented differences from the reference device code:
 *   1. Key identity.  The reference matches a slot on the 63-bit secondary
 *      hash ("uuid") alone and so confuses two keys whose uuids collide.
 *      Here a slot matches only if uuid AND the stored key bytes are equal;
 *      a uuid alias is probed past.  Results therefore equal a dictionary
 *      keyed by the key row's bytes.
 *   2. Key word fed to the hash.  The device code casts the key element
 *      numerically to int64 (floats truncate).  Here the element's bit
 *      pattern, sign-extended, is used (as the reference's host-side
 *      get_hash does, cuda_closed_hashmap.py:278-300); the float
 *      "minus zero -> plus zero" substitution of that host code is applied to
 *      the hash word only, never to identity.
 *   3. llabs(INT64_MIN) is mapped to 0 instead of staying negative.
 *   4. Slot addresses are 64-bit (the reference truncates to int in the CAS
 *      helpers, :184,198).
 *   5. key_perm is the identity (permuted views are outside this restatement).
 *
 * Parity pins (see tests/test_oracle_*.py): hash functions against an
 * arbitrary-precision evaluation and closed-form special cases; get/set/remove
 * against a Python dict model on random and adversarial sequences; slot
 * placement against hand-derived known answers for tiny tables (collision
 * chains, tombstone reuse, wrap-around, full table).
 *
 * Threading: the batch drivers take n_threads.  n_threads == 1 gives the
 * sequential semantics used for parity (a later row of a batch overwrites an
 * earlier equal key).  n_threads > 1 uses OpenMP and an atomic CAS on uuid[],
 * as the device code does; like the device code it requires the keys of one
 * set batch to be distinct.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef int64_t ll_t;

#define REF_EMPTY   ((ll_t)-1)
#define REF_REMOVED ((ll_t)-3)

typedef struct {
  ll_t n_buckets;        /* B: number of slots                                  */
  int32_t key_size;      /* elements per key row                                */
  int32_t key_elem_bytes;/* 1,2,4 or 8                                          */
  int32_t key_is_float;  /* 1: apply the minus-zero substitution to hash words  */
  int32_t value_bytes;   /* bytes per value row                                 */
  const ll_t *prime1, *prime2, *alpha1, *alpha2, *beta1, *beta2; /* [key_size]  */
  ll_t *uuid;            /* [B]                                                 */
  uint8_t *keys;         /* [B][key_size*key_elem_bytes]                        */
  uint8_t *values;       /* [B][value_bytes]                                    */
} ref_table_t;

/* ---- key element -> 64-bit hash word --------------------------------------*/
static inline ll_t ref_key_word(const ref_table_t *t, const uint8_t *key, int i) {
  ll_t w;
  switch (t->key_elem_bytes) {
    case 1: { int8_t v;  memcpy(&v, key + i, 1);      w = v; if (t->key_is_float && v == INT8_MIN)  w = 0; break; }
    case 2: { int16_t v; memcpy(&v, key + 2 * i, 2);  w = v; if (t->key_is_float && v == INT16_MIN) w = 0; break; }
    case 4: { int32_t v; memcpy(&v, key + 4 * i, 4);  w = v; if (t->key_is_float && v == INT32_MIN) w = 0; break; }
    default:{ int64_t v; memcpy(&v, key + 8 * i, 8);  w = v; if (t->key_is_float && v == INT64_MIN) w = 0; break; }
  }
  return w;
}

/* wrapping int64 arithmetic, spelled through uint64 so it is defined in C */
static inline ll_t wmul(ll_t a, ll_t b) { return (ll_t)((uint64_t)a * (uint64_t)b); }
static inline ll_t wadd(ll_t a, ll_t b) { return (ll_t)((uint64_t)a + (uint64_t)b); }
static inline ll_t wabs(ll_t a) { return a == INT64_MIN ? 0 : (a < 0 ? -a : a); }

/* closed_hashmap_impl_class.cu:87-96 : prod_i ((key_i*alpha_i + beta_i) % prime_i), C-sign %, then |.| */
static ll_t ref_universal(const ref_table_t *t, const uint8_t *key,
                          const ll_t *alpha, const ll_t *beta, const ll_t *prime) {
  ll_t h = wadd(wmul(ref_key_word(t, key, 0), alpha[0]), beta[0]) % prime[0];
  for (int i = 1; i < t->key_size; i++)
    h = wmul(h, wadd(wmul(ref_key_word(t, key, i), alpha[i]), beta[i]) % prime[i]);
  return wabs(h);
}

ll_t ref_get_hash(const ref_table_t *t, const uint8_t *key) {   /* :87-96 */
  return ref_universal(t, key, t->alpha1, t->beta1, t->prime1);
}
ll_t ref_get_uuid(const ref_table_t *t, const uint8_t *key) {   /* :98-107 */
  return ref_universal(t, key, t->alpha2, t->beta2, t->prime2);
}

static inline int ref_key_bytes(const ref_table_t *t) { return t->key_size * t->key_elem_bytes; }

static inline int ref_slot_is(const ref_table_t *t, ll_t addr, ll_t uuid, const uint8_t *key) {
  return t->uuid[addr] == uuid &&
         memcmp(t->keys + (size_t)addr * ref_key_bytes(t), key, ref_key_bytes(t)) == 0;
}

static inline ll_t ref_load_uuid(const ref_table_t *t, ll_t addr) {
  return __atomic_load_n(&t->uuid[addr], __ATOMIC_ACQUIRE);
}

/* :253-278 (exists) and :280-312 (get): walk from h1 until EMPTY; tombstones are walked past */
ll_t ref_find(const ref_table_t *t, const uint8_t *key, ll_t *probes) {
  ll_t h = ref_get_hash(t, key), u = ref_get_uuid(t, key), B = t->n_buckets;
  for (ll_t i = 0; i < B; i++) {
    ll_t addr = (h + i) % B;
    ll_t c = ref_load_uuid(t, addr);
    if (probes) (*probes)++;
    if (c == REF_EMPTY) break;
    if (c == u && ref_slot_is(t, addr, u, key)) return addr;
  }
  return -1;
}

static inline void ref_write(const ref_table_t *t, ll_t addr, const uint8_t *key, const uint8_t *value) {
  memcpy(t->keys + (size_t)addr * ref_key_bytes(t), key, ref_key_bytes(t));
  memcpy(t->values + (size_t)addr * t->value_bytes, value, t->value_bytes);
}

static inline int ref_cas(const ref_table_t *t, ll_t addr, ll_t expect, ll_t desired) {   /* :183-209 */
  return __atomic_compare_exchange_n(&t->uuid[addr], &expect, desired, 0, __ATOMIC_ACQ_REL, __ATOMIC_ACQUIRE);
}

/* :368-427.  Returns 1 stored into a fresh slot, 2 overwrote an existing key, 0 table full. */
int ref_set(const ref_table_t *t, const uint8_t *key, const uint8_t *value) {
  ll_t start = ref_get_hash(t, key), u = ref_get_uuid(t, key), B = t->n_buckets;
  ll_t first_removed = -1;
  /* phase 1 (:378-407) */
  for (ll_t i = 0; i < B; i++) {
    ll_t addr = (start + i) % B;
    ll_t c = ref_load_uuid(t, addr);
    if (c == u && ref_slot_is(t, addr, u, key)) { ref_write(t, addr, key, value); return 2; }
    if (c == REF_REMOVED && first_removed == -1) first_removed = addr;
    if (c == REF_EMPTY) {
      if (first_removed == -1) {
        /* the key bytes must be in place before uuid is published to concurrent probers */
        if (ref_cas(t, addr, REF_EMPTY, -2 /* claimed, not yet published */)) {
          ref_write(t, addr, key, value);
          __atomic_store_n(&t->uuid[addr], u, __ATOMIC_RELEASE);
          return 1;
        }
        /* lost the race for this slot: keep walking (:398-402) */
      } else {
        break;
      }
    }
  }
  /* phase 2 (:409-425): from the first tombstone, take the first tombstone or empty slot */
  if (first_removed != -1) {
    for (ll_t i = 0; i < B; i++) {
      ll_t addr = (first_removed + i) % B;
      if (ref_cas(t, addr, REF_REMOVED, -2) || ref_cas(t, addr, REF_EMPTY, -2)) {
        ref_write(t, addr, key, value);
        __atomic_store_n(&t->uuid[addr], u, __ATOMIC_RELEASE);
        return 1;
      }
    }
  }
  return 0;
}

/* :459-484 */
int ref_remove(const ref_table_t *t, const uint8_t *key) {
  ll_t addr = ref_find(t, key, NULL);
  if (addr < 0) return 0;
  __atomic_store_n(&t->uuid[addr], REF_REMOVED, __ATOMIC_RELEASE);
  return 1;
}

/* ---- batch drivers: closed_hashmap_impl.cu kernels, one iteration per "thread" ------------*/

static void ref_set_threads(int n_threads) {
#ifdef _OPENMP
  if (n_threads > 0) omp_set_num_threads(n_threads);
#else
  (void)n_threads;
#endif
}

/* closed_hashmap_get :7-85.  values_out must be pre-filled with the fallback row by the caller
 * (closed_hashmap_impl.py:103-109); only hits are written.  Returns total slot probes. */
ll_t ref_batch_get(const ref_table_t *t, const uint8_t *keys, ll_t n,
                   uint8_t *values_out, uint8_t *found, int n_threads) {
  const int kb = ref_key_bytes(t), vb = t->value_bytes;
  ll_t probes = 0;
  ref_set_threads(n_threads);
  #pragma omp parallel for schedule(static) reduction(+:probes) if (n_threads != 1)
  for (ll_t r = 0; r < n; r++) {
    ll_t p = 0;
    ll_t addr = ref_find(t, keys + (size_t)r * kb, &p);
    probes += p;
    found[r] = addr >= 0;
    if (addr >= 0) memcpy(values_out + (size_t)r * vb, t->values + (size_t)addr * vb, vb);
  }
  return probes;
}

/* closed_hashmap_set :88-156.  stored[r] = 1 fresh slot, 2 overwrite, 0 table full.
 * Returns the number of fresh slots taken. */
ll_t ref_batch_set(const ref_table_t *t, const uint8_t *keys, const uint8_t *values, ll_t n,
                   uint8_t *stored, int n_threads) {
  const int kb = ref_key_bytes(t), vb = t->value_bytes;
  ll_t fresh = 0;
  ref_set_threads(n_threads);
  #pragma omp parallel for schedule(static) reduction(+:fresh) if (n_threads != 1)
  for (ll_t r = 0; r < n; r++) {
    int s = ref_set(t, keys + (size_t)r * kb, values + (size_t)r * vb);
    if (stored) stored[r] = (uint8_t)s;
    fresh += (s == 1);
  }
  return fresh;
}

/* closed_hashmap_remove :159-220.  Returns the number removed. */
ll_t ref_batch_remove(const ref_table_t *t, const uint8_t *keys, ll_t n,
                      uint8_t *removed, int n_threads) {
  const int kb = ref_key_bytes(t);
  ll_t cnt = 0;
  ref_set_threads(n_threads);
  #pragma omp parallel for schedule(static) reduction(+:cnt) if (n_threads != 1)
  for (ll_t r = 0; r < n; r++) {
    int s = ref_remove(t, keys + (size_t)r * kb);
    if (removed) removed[r] = (uint8_t)s;
    cnt += s;
  }
  return cnt;
}

/* slot of each key or -1 (test helper for the placement known-answers) */
void ref_batch_find(const ref_table_t *t, const uint8_t *keys, ll_t n, ll_t *slots) {
  const int kb = ref_key_bytes(t);
  for (ll_t r = 0; r < n; r++) slots[r] = ref_find(t, keys + (size_t)r * kb, NULL);
}

void ref_batch_hash(const ref_table_t *t, const uint8_t *keys, ll_t n, ll_t *h1, ll_t *h2) {
  const int kb = ref_key_bytes(t);
  for (ll_t r = 0; r < n; r++) {
    h1[r] = ref_get_hash(t, keys + (size_t)r * kb);
    h2[r] = ref_get_uuid(t, keys + (size_t)r * kb);
  }
}

/* ---- DOK kernels --------------------------------------------------------------------------*/

#define REF_MAX_DIMS 16

/* One strided view: tensor_accessor.cu:1-121.  Strides are in elements; 0 = broadcast. */
typedef struct {
  const void *data;
  ll_t sizes[REF_MAX_DIMS];
  ll_t strides[REF_MAX_DIMS];
} ref_accessor_t;

/* tensor_accessor.cu:82-87 : idx[j] = (offset / stride_j) % size_j over the selector-element space */
static inline void ref_unravel(const ll_t *sizes, const ll_t *strides, int sel_ndim, ll_t off, ll_t *idx) {
  for (int j = 0; j < sel_ndim; j++) idx[j] = (off / strides[j]) % sizes[j];
}
/* tensor_accessor.cu:50-58 */
static inline ll_t ref_offset(const ref_accessor_t *a, int sel_ndim, const ll_t *idx) {
  ll_t o = 0;
  for (int j = 0; j < sel_ndim; j++) o += idx[j] * a->strides[j];
  return o;
}

static inline void ref_gather_coord(const ref_accessor_t *sel, int ndim, int sel_ndim,
                                    const ll_t *idx, ll_t *coord) {
  for (int d = 0; d < ndim; d++)
    coord[d] = ((const ll_t *)sel[d].data)[ref_offset(&sel[d], sel_ndim, idx)];
}

/* sparse_dok_count_items :4-56.  The table's keys are int64[ndim] coordinate rows.
 * elem_sizes/elem_strides describe the selector-element space (C-contiguous strides of the
 * broadcast shape).  Returns how many selector elements address a stored coordinate. */
ll_t ref_dok_count_items(const ref_table_t *t, const ref_accessor_t *sel, int ndim, int sel_ndim,
                         const ll_t *elem_sizes, const ll_t *elem_strides, ll_t n_elems, int n_threads) {
  ll_t cnt = 0;
  ref_set_threads(n_threads);
  #pragma omp parallel for schedule(static) reduction(+:cnt) if (n_threads != 1)
  for (ll_t e = 0; e < n_elems; e++) {
    ll_t idx[REF_MAX_DIMS], coord[REF_MAX_DIMS];
    ref_unravel(elem_sizes, elem_strides, sel_ndim, e, idx);
    ref_gather_coord(sel, ndim, sel_ndim, idx, coord);
    cnt += ref_find(t, (const uint8_t *)coord, NULL) >= 0;
  }
  return cnt;
}

/* sparse_dok_set_items_dense :271-313.  src is the strided source-value view (same broadcast
 * shape); every element is stored, zeros included.  Returns the number of fresh slots. */
ll_t ref_dok_set_items_dense(const ref_table_t *t, const ref_accessor_t *sel, const ref_accessor_t *src,
                             int ndim, int sel_ndim, const ll_t *elem_sizes, const ll_t *elem_strides,
                             ll_t n_elems, int n_threads) {
  const int vb = t->value_bytes;
  ll_t fresh = 0;
  ref_set_threads(n_threads);
  #pragma omp parallel for schedule(static) reduction(+:fresh) if (n_threads != 1)
  for (ll_t e = 0; e < n_elems; e++) {
    ll_t idx[REF_MAX_DIMS], coord[REF_MAX_DIMS];
    ref_unravel(elem_sizes, elem_strides, sel_ndim, e, idx);
    ref_gather_coord(sel, ndim, sel_ndim, idx, coord);
    const uint8_t *v = (const uint8_t *)src->data + (size_t)ref_offset(src, sel_ndim, idx) * vb;
    fresh += ref_set(t, (const uint8_t *)coord, v) == 1;
  }
  return fresh;
}

/* Lookup half of SparseDOKTensor.__getitem__ (sparse_dok_tensor.py:302-315) without the
 * stack/transpose copies: gather the coordinate of each selector element and read its value
 * (zero when absent) into the C-contiguous dense output; found (may be NULL) gets the hit flags. */
void ref_dok_get_items_dense(const ref_table_t *t, const ref_accessor_t *sel, int ndim, int sel_ndim,
                             const ll_t *elem_sizes, const ll_t *elem_strides, ll_t n_elems,
                             uint8_t *out, uint8_t *found, int n_threads) {
  const int vb = t->value_bytes;
  ref_set_threads(n_threads);
  #pragma omp parallel for schedule(static) if (n_threads != 1)
  for (ll_t e = 0; e < n_elems; e++) {
    ll_t idx[REF_MAX_DIMS], coord[REF_MAX_DIMS];
    ref_unravel(elem_sizes, elem_strides, sel_ndim, e, idx);
    ref_gather_coord(sel, ndim, sel_ndim, idx, coord);
    ll_t addr = ref_find(t, (const uint8_t *)coord, NULL);
    if (addr >= 0) memcpy(out + (size_t)e * vb, t->values + (size_t)addr * vb, vb);
    else memset(out + (size_t)e * vb, 0, vb);
    if (found) found[e] = addr >= 0;
  }
}

/* sparse_dok_zero_items :59-108: remove the coordinate of every selector element.
 * Returns the number removed. */
ll_t ref_dok_zero_items(const ref_table_t *t, const ref_accessor_t *sel, int ndim, int sel_ndim,
                        const ll_t *elem_sizes, const ll_t *elem_strides, ll_t n_elems) {
  ll_t cnt = 0;
  for (ll_t e = 0; e < n_elems; e++) {
    ll_t idx[REF_MAX_DIMS], coord[REF_MAX_DIMS];
    ref_unravel(elem_sizes, elem_strides, sel_ndim, e, idx);
    ref_gather_coord(sel, ndim, sel_ndim, idx, coord);
    cnt += ref_remove(t, (const uint8_t *)coord);
  }
  return cnt;
}

/* sparse_dok_get_items :111-160: every selector element whose coordinate is stored is inserted
 * into `out`, keyed by its index vector in the selector space (sel_ndim int64 words). */
void ref_dok_get_items(const ref_table_t *t, const ref_table_t *out, const ref_accessor_t *sel,
                       int ndim, int sel_ndim, const ll_t *elem_sizes, const ll_t *elem_strides,
                       ll_t n_elems) {
  for (ll_t e = 0; e < n_elems; e++) {
    ll_t idx[REF_MAX_DIMS], coord[REF_MAX_DIMS];
    ref_unravel(elem_sizes, elem_strides, sel_ndim, e, idx);
    ref_gather_coord(sel, ndim, sel_ndim, idx, coord);
    ll_t addr = ref_find(t, (const uint8_t *)coord, NULL);
    if (addr >= 0) ref_set(out, (const uint8_t *)idx, t->values + (size_t)addr * t->value_bytes);
  }
}

/* sparse_dok_set_items_sparse_v1 :163-211: src_indices is [sel_ndim][n_src] (index vectors in the
 * selector space), src_values [n_src]; each nonzero source value is stored at the coordinate
 * its index vector selects.  "Nonzero" is the numeric test of the device code: for floating
 * values minus zero counts as zero (value_is_float).  Returns the number of fresh slots. */
ll_t ref_dok_set_items_sparse_v1(const ref_table_t *t, const ref_accessor_t *sel, int ndim, int sel_ndim,
                                 const ll_t *src_indices, const uint8_t *src_values, ll_t n_src,
                                 int value_is_float) {
  const int vb = t->value_bytes;
  ll_t fresh = 0;
  for (ll_t k = 0; k < n_src; k++) {
    ll_t idx[REF_MAX_DIMS], coord[REF_MAX_DIMS];
    for (int j = 0; j < sel_ndim; j++) idx[j] = src_indices[(size_t)j * n_src + k];
    const uint8_t *v = src_values + (size_t)k * vb;
    int nonzero = 0;
    for (int q = 0; q < vb; q++) {
      uint8_t byte = v[q];
      if (value_is_float && q == vb - 1) byte &= 0x7f;      /* little endian: sign bit last */
      nonzero |= byte != 0;
    }
    if (!nonzero) continue;
    ref_gather_coord(sel, ndim, sel_ndim, idx, coord);
    fresh += ref_set(t, (const uint8_t *)coord, v) == 1;
  }
  return fresh;
}

int ref_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
