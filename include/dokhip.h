/*
 * dokhip.h - C ABI of libdokhip.so: a batched open-addressing hash table and the
 * dictionary-of-keys (DOK) sparse-tensor indexing kernels that run on it, written
 * for AMD gfx950 (MI355X).
 *
 * Conventions
 *   - Every pointer documented as "device" is a HIP device pointer owned by the
 *     caller.  The library never allocates or frees device memory; scratch space
 *     is passed in.  Batch buffers are row-major and contiguous.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Calls
 *     enqueue work and return; they do not synchronise.  Operations on one table
 *     must be ordered on one stream (or by events); distinct tables are independent.
 *     Kernels run on the GPU the stream belongs to, whichever GPU is current in the
 *     calling thread (the null stream: on the current one); every buffer of a call must
 *     live on that GPU.
 *   - Return value: DOK_OK or a negative DOK_E* code.  No call throws or aborts.
 *   - Flags (`found`, `stored`, `removed`) are one byte per row, 0 or 1.
 *
 * Each entry point names the interface of the reference implementation
 * (DeMoriarty/DOKSparse, paths relative to its checkout) that it stands in for.
 */
#ifndef DOKHIP_H
#define DOKHIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DOK_OK            0
#define DOK_EINVAL       -1   /* bad argument (null pointer, negative count, misaligned buffer)   */
#define DOK_EUNSUPPORTED -2   /* key/value width the table layouts cannot hold                   */
#define DOK_ELAUNCH      -3   /* the HIP runtime refused a launch; see dok_last_hip_error()      */
#define DOK_ETOOLARGE    -4   /* the table needs more scratch than dok_map_compact_static owns   */

#define DOK_BUCKET_BYTES  128
#define DOK_MAX_DIMS      14  /* most dimensions of a coordinate table and of an index space     */

/* Table header: DOK_HEADER_WORDS int64 words in device memory, zeroed by dok_table_clear.     */
#define DOK_HEADER_WORDS  16
#define DOK_H_NELEM       0   /* live entries (set adds fresh inserts, remove subtracts)          */
#define DOK_H_NFULL       1   /* rows a set could not place because every bucket was full         */
#define DOK_H_NPROBE      2   /* buckets visited, accumulated by the *_stats entry points         */
#define DOK_H_NOOB        3   /* rows whose coordinates fell outside lin_dims (skipped)           */
#define DOK_H_NOPS        4   /* rows processed by the *_stats entry points                       */
#define DOK_H_NSPILL      5   /* rows the last bulk insert handed to the per-row insert because
                                 their range's region of the partition was full (statistics)       */
/* words 8..11: side slots for the two 8-byte key patterns the packed layout reserves            */

/* Physical layouts (chosen from the key/value widths by dok_layout_of). */
#define DOK_LAYOUT_PACKED8 1  /* key <= 8 bytes (1,2,4,8), value 1,2,4 or 8 bytes: the key word
                                 itself is the CAS-claimed slot word; S = 120/(8+V) slots per bucket
                                 and one metadata word                                            */
#define DOK_LAYOUT_TAGGED  2  /* any widths with 8*(1+ceil(K/8)+ceil(V/8)) <= 128: an 8-byte
                                 tag/lock word per slot, then the key words, then the value words */

typedef struct dok_table {
  void    *buckets;            /* device, 128-byte aligned, n_phys_buckets * 128 bytes            */
  int64_t *header;             /* device, DOK_HEADER_WORDS int64                                  */
  int64_t  n_phys_buckets;     /* 1 .. 2^32-1                                                     */
  uint64_t seed;               /* hash seed; placement depends on it, results do not              */
  int32_t  key_bytes;          /* bytes per key row as stored                                     */
  int32_t  value_bytes;        /* bytes per value row                                             */
  int32_t  lin_ndim;           /* 0: key rows are raw bytes.  n>0: a COORDINATE TABLE - key rows
                                  handed to the entry points are n int64 coordinates inside
                                  lin_dims (the key format of the reference's SparseDOKTensor,
                                  sparse_dok_tensor.py:45-69); rows outside lin_dims are skipped
                                  (lookups: absent; inserts: counted in header[DOK_H_NOOB]).
                                  key_bytes says how they are stored:
                                    8      linearised row-major into one 8-byte key (packed
                                           layout).  Needs n <= 8 and prod(lin_dims) < 2^63, else
                                           DOK_EUNSUPPORTED.
                                    8 * n  (n >= 2) the coordinate rows themselves, as multi-word
                                           keys (n <= DOK_MAX_DIMS, any lin_dims).
                                  value_bytes must be 1, 2, 4 or 8 (one tensor element).           */
  int32_t  reserved_;
  int64_t  lin_dims[DOK_MAX_DIMS];
} dok_table_t;

/* A strided int64 (selector) or value (source) view over the broadcast index space.
 * Strides are in elements; 0 means the axis is broadcast.  For index vector idx[] the element
 * offset is off = sum_j idx[j]*strides[j].  A selector yields the coordinate
 * base + data[off], or, when data is NULL, base + off: an integer selector is {NULL, value, all
 * strides 0}, a slice start:stop on result axis a is {NULL, start, strides[a] = 1} - neither
 * needs a device tensor.  For a source-value view data must be set and base is ignored. */
typedef struct dok_view {
  const void *data;                    /* device, or NULL (selectors only)                       */
  int64_t     base;
  int64_t     strides[DOK_MAX_DIMS];
} dok_view_t;

/* The broadcast index space of one advanced-indexing expression plus one selector per
 * tensor dimension: what SparseDOKTensor._handle_selectors (sparse_dok_tensor.py:220-300)
 * produces and get_tensor_accessor_argument_array (util.py:295-310) packs for the kernels. */
typedef struct dok_index {
  int32_t    ndim;                     /* tensor dimensions = number of selectors                */
  int32_t    sel_ndim;                 /* dimensions of the broadcast index space: at most
                                          DOK_MAX_DIMS; on a table of linearised keys at most 8
                                          (else DOK_EUNSUPPORTED)                                */
  int64_t    shape[DOK_MAX_DIMS];      /* broadcast shape                                        */
  dok_view_t sel[DOK_MAX_DIMS];        /* int64 selector views, one per tensor dimension         */
} dok_index_t;

/* ---- layout helpers (host only, no GPU needed) ------------------------------------------ */

/* Layout id for the widths, or DOK_EUNSUPPORTED.  *slots_per_bucket may be NULL. */
int dok_layout_of(int32_t key_bytes, int32_t value_bytes, int32_t *slots_per_bucket);

/* Physical bucket count that gives at least `capacity` slots. */
int64_t dok_phys_buckets_for(int64_t capacity, int32_t key_bytes, int32_t value_bytes);

/* Text of the last HIP error a launch hit on this thread ("" if none). */
const char *dok_last_hip_error(void);

/* ---- table lifetime --------------------------------------------------------------------- */

/* Mark every slot empty and zero the header.
 * Reference: CudaClosedHashmap.__init__ filling _uuid with -1 (cuda_closed_hashmap.py:40). */
int dok_table_clear(const dok_table_t *t, void *stream);

/* ---- batched map operations -------------------------------------------------------------- */

/* values_out[r] = value of keys[r] if present else the fallback row; found[r] = present.
 * `fallback` is a HOST pointer to value_bytes bytes (NULL = zeros).
 * Reference: closed_hashmap_get (closed_hashmap_impl.cu:7-85) together with the fallback
 * pre-fill of ClosedHashmapImplCuda.get (closed_hashmap_impl.py:50-145). */
int dok_map_get(const dok_table_t *t, const void *keys, int64_t n,
                void *values_out, const void *fallback, uint8_t *found, void *stream);

/* dok_map_get with the fallback row in DEVICE memory (value_bytes bytes, aligned like a value
 * row; never NULL): the kernel reads it, so the host neither copies nor synchronises, and a call
 * captured into a HIP graph sees the row's current contents at every replay.
 * Reference: the `fallback` array argument of closed_hashmap_get (closed_hashmap_impl.cu:7-23),
 * a device tensor made by ClosedHashmapImplCuda.get (closed_hashmap_impl.py:103-109). */
int dok_map_get_dev_fallback(const dok_table_t *t, const void *keys, int64_t n,
                             void *values_out, const void *fallback_dev, uint8_t *found,
                             void *stream);

/* Same as dok_map_get, and adds the buckets visited / rows processed to header[DOK_H_NPROBE/NOPS]. */
int dok_map_get_stats(const dok_table_t *t, const void *keys, int64_t n,
                      void *values_out, const void *fallback, uint8_t *found, void *stream);

/* Upsert.  A key present is overwritten in place; a key absent takes the first tombstone on
 * its probe chain, else the first empty slot.  Equal keys inside one batch end up in ONE slot
 * holding one of their values.  header[DOK_H_NELEM] grows by the number of fresh inserts.
 * stored (may be NULL): 1 = placed, 0 = table full or coordinate out of range.
 * Reference: closed_hashmap_set (closed_hashmap_impl.cu:88-156, ClosedHashmap::set
 * closed_hashmap_impl_class.cu:368-427); the in-kernel count replaces the host-side
 * "get, unique, count" pre-pass of CudaClosedHashmap.set (cuda_closed_hashmap.py:350-384). */
int dok_map_set(const dok_table_t *t, const void *keys, const void *values, int64_t n,
                uint8_t *stored, void *stream);

/* Bulk upsert: the same result as dok_map_set (stored == NULL) for a batch that is large
 * against the table - rule of thumb: more than one row per physical bucket.  Instead of one
 * compare-and-swap in HBM per row, the batch is partitioned by table range (two scatter passes
 * through `workspace`, each bin of a pass owning a region of fixed capacity there) and every
 * range of buckets is merged in LDS, so the table is streamed through the GPU once.  Rows whose
 * bin's region is full (batches with very many equal keys) take the per-row insert at the end;
 * header[DOK_H_NSPILL] says how many.
 * On the multi-word layout the bulk entry points run another fast form: a new row claims its slot
 * with ONE compare-and-swap and plain stores (dok_map_set: claim, payload and publish are three
 * write transactions); a row that meets its own fingerprint in flight - equal keys inside the batch,
 * mostly - is put on a list in the workspace and inserted by a second launch.  That form serves
 * tables with values of at most 8 bytes (every coordinate table) and, for dok_map_build_bulk /
 * dok_coo_build_bulk, any widths; other tables take the dok_map_set kernel, same result.
 *   dok_bulk_workspace_bytes: device bytes dok_map_set_bulk / dok_coo_set_bulk need for n rows;
 *     0 if the bulk path cannot take this table or n (packed layout: n >= 2^31: use
 *     dok_map_set), negative on a bad table.  A table of more than 2^28 buckets (32 GiB) is
 *     worked through in windows of 2^28 buckets, one run of the passes per window, each reading
 *     the whole batch and keeping the rows of its window; dok_map_build_bulk then clears the table
 *     first and merges into it like dok_map_set_bulk.
 *     (packed layout: about 3.4 times the bytes of the batch - two partition buffers with slack
 *     and the spill list - plus 4 bytes per 256 buckets of the table; multi-word layout: 8 n + 256).
 *   workspace: device, 256-byte aligned, at least that many bytes; contents need no
 *     initialisation and are garbage afterwards.  Calls sharing one workspace must be ordered.
 * Reference: the same closed_hashmap_set launch as dok_map_set, at the batch sizes of
 * SparseDOKTensor.__init__ / from_sparse_coo (sparse_dok_tensor.py:59-69) and of
 * CudaClosedHashmap.rehash (cuda_closed_hashmap.py:456-468). */
int64_t dok_bulk_workspace_bytes(const dok_table_t *t, int64_t n);
int dok_map_set_bulk(const dok_table_t *t, const void *keys, const void *values, int64_t n,
                     void *workspace, int64_t workspace_bytes, void *stream);

/* dok_table_clear followed by dok_map_set_bulk, in one pass: the bucket memory and the header
 * of t need no initialisation, every bucket and header word is written (n >= 1).  The merge takes
 * each range of buckets as empty instead of reading it, so neither the clear nor the read of the
 * table is paid for.
 * Reference: the first set after the table allocation - CudaClosedHashmap.set on a new map
 * fills uuid with the EMPTY marker and then launches closed_hashmap_set
 * (cuda_closed_hashmap.py:36-53, 321-384), as SparseDOKTensor.__init__ does for a COO source
 * (sparse_dok_tensor.py:59-69). */
int dok_map_build_bulk(const dok_table_t *t, const void *keys, const void *values, int64_t n,
                       void *workspace, int64_t workspace_bytes, void *stream);

/* Tombstone each present key; header[DOK_H_NELEM] shrinks by the number removed.  Equal keys
 * in one batch: exactly one row reports 1.
 * Reference: closed_hashmap_remove (closed_hashmap_impl.cu:159-220, ClosedHashmap::remove
 * closed_hashmap_impl_class.cu:459-484). */
int dok_map_remove(const dok_table_t *t, const void *keys, int64_t n,
                   uint8_t *removed, void *stream);

/* dok_map_remove for a batch in which no key occurs twice - what the reference's kernel is given,
 * because CudaClosedHashmap.remove passes its keys through unique(dim=0) first
 * (cuda_closed_hashmap.py:438) and the kernel then stores the REMOVED marker without any atomic
 * (closed_hashmap_impl_class.cu:459-484).  The tombstone is a plain store here as well, which
 * saves one returning atomic in HBM per row.  With a key twice in the batch both rows would
 * report 1 and header[DOK_H_NELEM] would shrink twice: use dok_map_remove for such batches. */
int dok_map_remove_unique(const dok_table_t *t, const void *keys, int64_t n,
                          uint8_t *removed, void *stream);

/* dok_map_remove without per-row flags for a batch that is large against the table (rule of
 * thumb: a million keys and more, more than one per physical bucket): the keys are partitioned by
 * table range through `workspace` (dok_bulk_workspace_bytes(t, n) bytes, 256-byte aligned, as for
 * dok_map_set_bulk) and every range's keys are looked up together, so the table is read in order
 * and each bucket line written back once.  Equal keys inside the batch count once.  Packed layout
 * only (else DOK_EUNSUPPORTED: use dok_map_remove).
 * Reference: closed_hashmap_remove (closed_hashmap_impl.cu:159-220) at the batch sizes of
 * `del hashmap[keys]` (cuda_closed_hashmap.py:476-477), which discards the flags. */
int dok_map_remove_bulk(const dok_table_t *t, const void *keys, int64_t n, void *workspace,
                        int64_t workspace_bytes, void *stream);

/* count[0] += number of rows whose key is present.  count is a device int64.
 * Reference: ClosedHashmap::exists (closed_hashmap_impl_class.cu:253-278). */
int dok_map_count_existing(const dok_table_t *t, const void *keys, int64_t n,
                           int64_t *count, void *stream);

/* Overwrite the values of the rows whose key is present and count the others:
 * missing[0] += number of rows whose key is absent (a device int64); nothing is inserted.
 * What a caller runs before an upsert whose growth decision needs the number of new keys anyway
 * (the reference's get + unique pre-pass, cuda_closed_hashmap.py:350-366): when the answer is 0 -
 * a batch that only updates existing keys - the upsert is already done, at the rate of a lookup.
 * Otherwise follow with dok_map_set of the whole batch (the rows already written are written
 * again; equal keys keep one whole value either way).  Packed layout only (DOK_EUNSUPPORTED
 * otherwise: use dok_map_count_existing).
 * Reference: the overwrite branch of ClosedHashmap::set (closed_hashmap_impl_class.cu:383-388). */
int dok_map_update_existing(const dok_table_t *t, const void *keys, const void *values, int64_t n,
                            int64_t *missing, void *stream);

/* ---- read-out ----------------------------------------------------------------------------- */

/* Bytes of device scratch dok_map_compact needs for this table. */
int64_t dok_compact_scratch_bytes(const dok_table_t *t);

/* Write the live entries in slot order: keys_out[i] (key_bytes each; lin_ndim int64
 * coordinates each when lin_ndim > 0) and values_out[i].  Either output may be NULL.  Two
 * calls on an unchanged table give the same order.  `capacity_rows` bounds the rows written;
 * count_out[0] (device int64) receives the number of live entries.
 * Reference: nonempty_mask / keys() / values() (cuda_closed_hashmap.py:157-172). */
int dok_map_compact(const dok_table_t *t, void *keys_out, void *values_out,
                    int64_t capacity_rows, int64_t *count_out, void *scratch, void *stream);

/* dok_map_compact for callers that cannot provide scratch memory because they cannot allocate:
 * code under HIP graph capture, serving loops and harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  The scratch is a device array of DOK_STATIC_SCRATCH_BYTES that
 * the library itself holds on every GPU it runs on (dok_static_scratch_bytes() returns that
 * size); the call allocates and frees nothing.  Same outputs, in the same order, as
 * dok_map_compact on the same table.
 *   - A table whose dok_compact_scratch_bytes exceeds that size (more than 2^28 buckets) is
 *     refused with DOK_ETOOLARGE before anything is launched: use dok_map_compact.
 *   - All calls on one GPU share the one array: calls that may overlap (different streams,
 *     different host threads) race and must be ordered by the caller. */
#define DOK_STATIC_SCRATCH_BYTES ((8 << 20) + 256)
int64_t dok_static_scratch_bytes(void);
int dok_map_compact_static(const dok_table_t *t, void *keys_out, void *values_out,
                           int64_t capacity_rows, int64_t *count_out, void *stream);

/* Re-insert every live entry of src into dst (same key/value widths; dst may have another size
 * or seed).  dst must be EMPTY: cleared by the caller (dok_table_clear) and not written by anything
 * else while the call runs.  On the multi-word layout the entries are placed without comparing
 * keys (src holds no key twice, an empty dst none at all), so a dst that already holds entries
 * would end up with keys stored twice and a wrong entry count; the packed layout happens to
 * upsert, which callers must not rely on.
 * Reference: CudaClosedHashmap.rehash (cuda_closed_hashmap.py:456-468). */
int dok_map_rehash(const dok_table_t *src, const dok_table_t *dst, void *stream);

/* dok_map_rehash through the bulk path (see dok_map_build_bulk): the live entries of src are
 * partitioned by range of dst and merged in LDS.  Unlike dok_map_rehash, dst need NOT be
 * cleared: its bucket memory and header may be uninitialised and are overwritten in full
 * (whatever dst held is gone).  Needs a caller-owned workspace of
 * dok_rehash_bulk_workspace_bytes(src, dst) bytes (0 = not available for these tables, use
 * dok_map_rehash).  Worth it when src holds several entries per bucket of dst and millions of
 * them.
 * Reference: CudaClosedHashmap.rehash (cuda_closed_hashmap.py:456-468). */
int64_t dok_rehash_bulk_workspace_bytes(const dok_table_t *src, const dok_table_t *dst);
int dok_map_rehash_bulk(const dok_table_t *src, const dok_table_t *dst, void *workspace,
                        int64_t workspace_bytes, void *stream);

/* ---- COO bridge (coordinate tables: lin_ndim > 0, either key format) ------------------------ */

/* dok_map_set for coordinates given the way a COO tensor holds them: indices is
 * [lin_ndim][n] int64 (coordinate d of entry i at indices[d*n + i]).  No per-row flag.
 * Reference: SparseDOKTensor.__init__ / from_sparse_coo, which transpose and copy the indices
 * before the set (sparse_dok_tensor.py:66-69, 71-84). */
int dok_coo_set(const dok_table_t *t, const int64_t *indices, const void *values, int64_t n,
                void *stream);

/* dok_coo_set through the bulk path (see dok_map_set_bulk). */
int dok_coo_set_bulk(const dok_table_t *t, const int64_t *indices, const void *values, int64_t n,
                     void *workspace, int64_t workspace_bytes, void *stream);

/* dok_coo_set into uninitialised table memory (see dok_map_build_bulk). */
int dok_coo_build_bulk(const dok_table_t *t, const int64_t *indices, const void *values, int64_t n,
                       void *workspace, int64_t workspace_bytes, void *stream);

/* dok_map_compact emitting COO layout: indices_out is [lin_ndim][capacity] int64, values_out
 * [capacity].  Either output may be NULL; count_out[0] receives the number of live entries.
 * Reference: SparseDOKTensor.indices()/values()/to_sparse_coo (sparse_dok_tensor.py:156-203). */
int dok_coo_compact(const dok_table_t *t, int64_t *indices_out, void *values_out, int64_t capacity,
                    int64_t *count_out, void *scratch, void *stream);

/* ---- DOK indexing (coordinate tables: lin_ndim > 0, either key format) ---------------------- */

/* out[e] = value stored at the coordinate the selectors give for element e of the broadcast
 * index space, or zero; out is C-contiguous with value_bytes per element.
 * Reference: SparseDOKTensor.__getitem__ (sparse_dok_tensor.py:302-315): stack + transpose +
 * closed_hashmap_get with fallback 0, fused into one pass. */
int dok_getitem_dense(const dok_table_t *t, const dok_index_t *ix, void *out, void *stream);

/* Upsert src[e] at the coordinate of every element e (zeros are stored too).
 * Reference: sparse_dok_set_items_dense (sparse_dok_tensor_impl.cu:271-313). */
int dok_setitem_dense(const dok_table_t *t, const dok_index_t *ix, const dok_view_t *src,
                      void *stream);

/* dok_setitem_dense for large scatters into a table of coordinate rows (key_bytes = 8 * lin_ndim):
 * the fast insert of the multi-word layout (see dok_map_set_bulk), which needs a workspace of
 * dok_bulk_workspace_bytes(t, number of elements of the index space) bytes, 256-byte aligned.  On a
 * table of linearised keys the call is dok_setitem_dense and the workspace is not used.
 * Reference: sparse_dok_set_items_dense (sparse_dok_tensor_impl.cu:271-313). */
int dok_setitem_dense_bulk(const dok_table_t *t, const dok_index_t *ix, const dok_view_t *src,
                           void *workspace, int64_t workspace_bytes, void *stream);

/* count[0] += number of elements whose coordinate is stored.
 * Reference: sparse_dok_count_items (sparse_dok_tensor_impl.cu:4-56). */
int dok_count_items(const dok_table_t *t, const dok_index_t *ix, int64_t *count, void *stream);

/* Tombstone the coordinate of every element; header[DOK_H_NELEM] shrinks accordingly.
 * Reference: sparse_dok_zero_items (sparse_dok_tensor_impl.cu:59-108). */
int dok_zero_items(const dok_table_t *t, const dok_index_t *ix, void *stream);

/* Sparse-valued gather: every element e of the index space whose coordinate is stored in t is
 * inserted into `out` under the key e.  `out` is a cleared coordinate-keyed table whose
 * lin_dims are the broadcast shape of ix and whose value_bytes equal t's.  `out` must hold
 * linearised keys (key_bytes 8), else DOK_EUNSUPPORTED; t may be of either key format.
 * Reference: sparse_dok_get_items (sparse_dok_tensor_impl.cu:111-160). */
int dok_getitem_sparse(const dok_table_t *t, const dok_index_t *ix, const dok_table_t *out,
                       void *stream);

/* Sparse-valued scatter: source entry k has index vector src_indices[j*n_src + k] (j over the
 * axes of the index space, device int64) and value src_values[k]; every entry whose value,
 * ANDed with nonzero_mask, is not zero is upserted at the coordinate its index vector selects
 * (nonzero_mask: all ones for integer values, sign bit cleared for floating values, so that
 * minus zero counts as zero).
 * Reference: sparse_dok_set_items_sparse_v1 (sparse_dok_tensor_impl.cu:163-211). */
int dok_setitem_sparse(const dok_table_t *t, const dok_index_t *ix, const int64_t *src_indices,
                       const void *src_values, int64_t n_src, uint64_t nonzero_mask, void *stream);

/* dense[linear coordinate] = value for every live entry; `dense` holds prod(lin_dims) elements
 * of value_bytes (fewer than 2^62 elements) and must be zero-filled by the caller.
 * Reference: SparseDOKTensor.to_dense (sparse_dok_tensor.py:195-209). */
int dok_to_dense(const dok_table_t *t, void *dense, void *stream);

/* Measurement aid with no counterpart in the reference: out[i] = a checksum of one
 * pseudo-randomly chosen 128-byte bucket line, for i in [0, n) - the memory access pattern of
 * dok_map_get with the probing removed.  Its rate (lines per second) is the practical ceiling
 * for lookups on this table; the benchmark reports it beside the published HBM peak. */
int dok_line_gather(const dok_table_t *t, int64_t n, uint64_t seed, uint32_t *out, void *stream);

/* The same with granules of 128, 64 or 32 bytes (naturally aligned pieces of the bucket array, read
 * by 16, 8 or 4 lanes): what a probe of half or a quarter of a bucket line would cost.  No
 * counterpart in the reference. */
int dok_line_gather_granule(const dok_table_t *t, int64_t n, uint64_t seed, int32_t granule_bytes,
                            uint32_t *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DOKHIP_H */
