// libdokhip: host side of the C ABI declared in include/dokhip.h.  Validates arguments,
// turns the caller's descriptors into kernel-argument structs, picks the kernel instantiation
// from the table's widths and enqueues it on the caller's stream.  Nothing here allocates
// device memory or synchronises.
#include <hip/hip_runtime.h>
#include <string.h>
#include <atomic>
#include "dok_device.h"
#include "dok_packed8.h"
#include "dok_tagged.h"
#include "dok_bulk.h"

// Scratch of dok_map_compact_static: device memory that belongs to the library, so that the call
// needs no buffer from its caller.  Every GPU the library runs on holds its own copy of the array,
// at its own address, from the moment the code object is loaded until the process ends.  In host
// code this name is only a handle for hipGetSymbolAddress - never a pointer to hand to a kernel.
static __device__ __align__(256) unsigned char dok_static_scratch[DOK_STATIC_SCRATCH_BYTES];
static_assert(DOK_STATIC_SCRATCH_BYTES >= (((1LL << 28) / DOK_CHUNK) + 1) * 8, "serves tables of up to 2^28 buckets");

namespace {

thread_local char g_last_error[256] = "";

// Device address of dok_static_scratch on each GPU, resolved at the first call on that GPU.
constexpr int kMaxDevices = 64;
std::atomic<void *> g_static_scratch[kMaxDevices];

int static_scratch_of_current_device(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess && (dev < 0 || dev >= kMaxDevices)) e = hipErrorInvalidDevice;
  void *p = nullptr;
  if (e == hipSuccess) {
    p = g_static_scratch[dev].load(std::memory_order_acquire);
    if (!p) {
      // (two threads may both get here: they obtain the same address)
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(dok_static_scratch));
      if (e == hipSuccess && !p) e = hipErrorInvalidSymbol;
      if (e == hipSuccess) g_static_scratch[dev].store(p, std::memory_order_release);
    }
  }
  if (e != hipSuccess) {
    strncpy(g_last_error, hipGetErrorString(e), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = 0;
    return DOK_ELAUNCH;
  }
  *out = p;
  return DOK_OK;
}

// Makes the device of the caller's stream current for the duration of a call (kernels launch on
// the current device; a process that drives several GPUs may call with another one current).
// The null stream belongs to whatever device is current, so there is nothing to switch then.
// A process that sees one GPU (the usual one-process-per-GPU set-up) skips the query, which costs
// 2 to 3 microseconds per call.
int visible_devices() {
  static std::atomic<int> count{0};
  int c = count.load(std::memory_order_relaxed);
  if (c == 0) {
    if (hipGetDeviceCount(&c) != hipSuccess || c < 1) c = 1;
    count.store(c, std::memory_order_relaxed);
  }
  return c;
}
struct DeviceScope {
  int prev = -1;
  bool switched = false;
  explicit DeviceScope(hipStream_t s) {
    hipDevice_t dev = -1;
    if (s != nullptr && visible_devices() > 1 && hipStreamGetDevice(s, &dev) == hipSuccess &&
        hipGetDevice(&prev) == hipSuccess && prev != (int)dev)
      switched = hipSetDevice((int)dev) == hipSuccess;
  }
  ~DeviceScope() {
    if (switched) (void)hipSetDevice(prev);
  }
  DeviceScope(const DeviceScope &) = delete;
  DeviceScope &operator=(const DeviceScope &) = delete;
};

int note_launch() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    strncpy(g_last_error, hipGetErrorString(e), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = 0;
    return DOK_ELAUNCH;
  }
  return DOK_OK;
}

bool is_pow2_le8(int v) { return v == 1 || v == 2 || v == 4 || v == 8; }

int layout_of(int kb, int vb, int *slots) {
  if (kb <= 0 || vb <= 0) return DOK_EUNSUPPORTED;
  if (is_pow2_le8(kb) && is_pow2_le8(vb)) {
    if (slots) *slots = 120 / (8 + vb);    // word 15 of a packed bucket is metadata
    return DOK_LAYOUT_PACKED8;
  }
  const int w = 1 + (kb + 7) / 8 + (vb + 7) / 8;
  if (w > 16) return DOK_EUNSUPPORTED;
  if (slots) *slots = 16 / w;
  return DOK_LAYOUT_TAGGED;
}

// Multiplier and shift that divide a 64-bit integer by d >= 2 (see dok_div_stride).
static void div_magic(u64 d, u64 &magic, int &shift) {
  const int fl = 63 - __builtin_clzll(d);
  if ((d & (d - 1)) == 0) { magic = 0; shift = fl - 1; return; }      // power of two: q = 0, n >> 1 >> (fl - 1)
  const unsigned __int128 num = (unsigned __int128)1 << (64 + fl);     // d > 2^fl, so the quotient fits 64 bits
  u64 m = (u64)(num / d);
  const u64 rem = (u64)(num % d);
  m += m;
  const u64 twice = rem + rem;
  if (twice >= d || twice < rem) m += 1;
  magic = m + 1;
  shift = fl;
}

// Validate a table descriptor and build its kernel-argument form.
// A coordinate table (lin_ndim > 0) states its key format through key_bytes: 8 = the coordinates are
// linearised into one 8-byte key (packed layout; at most DOK_LIN_DIMS dimensions and fewer than 2^63
// elements), 8 * lin_ndim = the int64 coordinate rows themselves are the keys (multi-word layout).
int make_dev_table(const dok_table_t *t, DevTable &d, int &layout) {
  if (!t || !t->buckets || !t->header) return DOK_EINVAL;
  if (t->n_phys_buckets < 1 || t->n_phys_buckets > 0xffffffffLL) return DOK_EINVAL;
  if (((uintptr_t)t->buckets & 127) != 0 || ((uintptr_t)t->header & 7) != 0) return DOK_EINVAL;
  if (t->lin_ndim < 0 || t->lin_ndim > DOK_MAX_DIMS) return DOK_EINVAL;
  const bool rows = t->lin_ndim > 0 && (t->lin_ndim > 1 || t->key_bytes != 8) && t->key_bytes == 8 * t->lin_ndim;
  if (t->lin_ndim > 0 && !rows && t->key_bytes != 8) return DOK_EINVAL;
  layout = layout_of(t->key_bytes, t->value_bytes, nullptr);
  if (layout < 0) return layout;
  if (rows && layout != DOK_LAYOUT_TAGGED) return DOK_EUNSUPPORTED;
  if (t->lin_ndim > 0 && !is_pow2_le8(t->value_bytes)) return DOK_EUNSUPPORTED;   // one tensor element per entry
  memset(&d, 0, sizeof(d));
  d.buckets = (u64 *)t->buckets;
  d.header = (i64 *)t->header;
  d.nb = (u64)t->n_phys_buckets;
  d.seed = t->seed;
  d.key_bytes = t->key_bytes;
  d.value_bytes = t->value_bytes;
  d.lin_ndim = t->lin_ndim;
  for (int k = 0; k < t->lin_ndim; k++) {
    if (t->lin_dims[k] < 0) return DOK_EINVAL;
    d.lin_dims[k] = t->lin_dims[k];
  }
  if (t->lin_ndim > 0 && !rows) {
    if (t->lin_ndim > DOK_LIN_DIMS) return DOK_EUNSUPPORTED;
    // volume must fit in 63 bits so that a linear key never meets the reserved patterns
    unsigned __int128 vol = 1;
    for (int k = t->lin_ndim - 1; k >= 0; k--) {
      d.lin_strides[k] = (i64)vol;
      if (vol > 1) div_magic((u64)vol, d.lin_magic[k], d.lin_shift[k]);
      vol *= (unsigned __int128)(t->lin_dims[k] > 0 ? t->lin_dims[k] : 1);
      if (vol >> 63) return DOK_EUNSUPPORTED;
    }
  }
  return DOK_OK;
}

// Validate an index descriptor against the table; build its kernel-argument form: DevIndex for the
// fused kernels of the packed layout, DevIndexW (more dimensions) for the multi-word layout.
template <class DI, int MAXD>
int make_dev_index(const DevTable &t, const dok_index_t *ix, const dok_view_t *src, DI &d) {
  if (!ix || t.lin_ndim == 0) return DOK_EINVAL;
  if (ix->ndim != t.lin_ndim) return DOK_EINVAL;
  if (ix->sel_ndim < 0 || ix->sel_ndim > DOK_MAX_DIMS) return DOK_EINVAL;
  if (ix->sel_ndim > MAXD || ix->ndim > MAXD) return DOK_EUNSUPPORTED;
  memset(&d, 0, sizeof(d));
  d.ndim = ix->ndim;
  d.sel_ndim = ix->sel_ndim;
  unsigned __int128 n = 1;
  for (int j = ix->sel_ndim - 1; j >= 0; j--) {
    if (ix->shape[j] < 0) return DOK_EINVAL;
    d.shape[j] = ix->shape[j];
    d.estride[j] = n ? (i64)n : 1;          // never 0: it is a divisor in the unravel
    n *= (unsigned __int128)ix->shape[j];
    if (n >> 62) return DOK_EINVAL;
  }
  d.n_elems = (i64)n;
  for (int j = ix->sel_ndim; j < MAXD; j++) d.estride[j] = 1;      // (divisors of the unused axes)
  for (int k = 0; k < ix->ndim; k++) {
    d.sel[k] = (const i64 *)ix->sel[k].data;
    d.sbase[k] = ix->sel[k].base;
    for (int j = 0; j < ix->sel_ndim; j++) {
      if (ix->sel[k].strides[j] < 0) return DOK_EINVAL;
      d.sstride[k][j] = ix->sel[k].strides[j];
    }
  }
  if (src) {
    if (!src->data && d.n_elems > 0) return DOK_EINVAL;
    d.src = src->data;
    for (int j = 0; j < ix->sel_ndim; j++) {
      if (src->strides[j] < 0) return DOK_EINVAL;
      d.vstride[j] = src->strides[j];
    }
  }
  return DOK_OK;
}
int make_dev_index(const DevTable &t, const dok_index_t *ix, const dok_view_t *src, DevIndex &d) {
  return make_dev_index<DevIndex, DOK_LIN_DIMS>(t, ix, src, d);
}
int make_dev_index(const DevTable &t, const dok_index_t *ix, const dok_view_t *src, DevIndex4 &d) {
  return make_dev_index<DevIndex4, 4>(t, ix, src, d);
}
// Whether the small descriptor form serves this index.
inline bool small_index(const dok_index_t *ix) { return ix && ix->ndim <= 4 && ix->sel_ndim >= 0 && ix->sel_ndim <= 4; }
int make_dev_index(const DevTable &t, const dok_index_t *ix, const dok_view_t *src, DevIndexW &d) {
  return make_dev_index<DevIndexW, DOK_MAX_DIMS>(t, ix, src, d);
}
// The two kinds of coordinate table.
inline bool is_lin(const DevTable &d, int layout) { return d.lin_ndim > 0 && layout == DOK_LAYOUT_PACKED8; }
inline bool is_coord_rows(const DevTable &d, int layout) { return d.lin_ndim > 0 && layout == DOK_LAYOUT_TAGGED; }

// One workgroup per tile of DOK_TPB rows (kernels without counters) ...
inline unsigned grid_for(i64 n) { return (unsigned)((n + DOK_TPB - 1) / DOK_TPB); }
// ... or a fixed grid that fills the machine (8 workgroups on each of 256 CUs) and loops over the
// tiles, for kernels that end with per-wave atomics on the table header.
#define DOK_COUNT_GRID 2048
inline unsigned grid_counting(i64 n) {
  const i64 tiles = (n + DOK_TPB - 1) / DOK_TPB;
  return (unsigned)(tiles < DOK_COUNT_GRID ? tiles : DOK_COUNT_GRID);
}
// Contiguous share of a batch that each wave of a streaming kernel works through.
inline i64 rows_per_wave(i64 n, unsigned grid) {
  const i64 waves = (i64)grid * (DOK_TPB / 64);
  return (n + waves - 1) / waves;
}
inline i64 chunks_of(const DevTable &d) { return ((i64)d.nb + DOK_CHUNK - 1) / DOK_CHUNK; }
inline unsigned chunk_grid(i64 n_chunks) { return (unsigned)((n_chunks + 3) / 4); }

u64 fallback_word(const void *fallback, int vb) {
  u64 f = 0;
  if (fallback) memcpy(&f, fallback, vb);
  return f;
}

// Rows per launch are bounded so that the 32-bit grid dimension cannot overflow.
const i64 kMaxRows = (i64)0x7fffffff * DOK_TPB;

#define P8_DISPATCH(vb, CALL)        \
  switch (vb) {                      \
    case 1: { constexpr int V = 1; CALL; } break; \
    case 2: { constexpr int V = 2; CALL; } break; \
    case 4: { constexpr int V = 4; CALL; } break; \
    default: { constexpr int V = 8; CALL; } break; \
  }
// the same, also binding KF (key format of the batch buffer) for the kernels that read key rows
#define P8_DISPATCH_LIN(vb, lin, CALL)                                          \
  if (lin) { constexpr int KF = DOK_KF_ROWS; P8_DISPATCH(vb, CALL) }            \
  else { constexpr int KF = DOK_KF_RAW; P8_DISPATCH(vb, CALL) }

// The fused kernels of the packed layout, for either size of the index descriptor.
template <class IX>
int getitem_dense_lin(const DevTable &d, const dok_index_t *ix, void *out, hipStream_t s) {
  IX di;
  int rc = make_dev_index(d, ix, nullptr, di);
  if (rc) return rc;
  if (di.n_elems == 0) return DOK_OK;
  if (!out || di.n_elems > kMaxRows) return DOK_EINVAL;
  const DeviceScope on_stream_device(s);
  P8_DISPATCH(d.value_bytes, (p8_getitem_kernel<V, IX><<<grid_for(di.n_elems), DOK_TPB, 0, s>>>(d, di, out)));
  return note_launch();
}
template <class IX>
int setitem_dense_lin(const DevTable &d, const dok_index_t *ix, const dok_view_t *src, hipStream_t s) {
  IX di;
  int rc = make_dev_index(d, ix, src, di);
  if (rc) return rc;
  if (di.n_elems == 0) return DOK_OK;
  if (di.n_elems > kMaxRows) return DOK_EINVAL;
  const DeviceScope on_stream_device(s);
  const unsigned grid = grid_counting(di.n_elems);
  P8_DISPATCH(d.value_bytes, (p8_setitem_kernel<V, IX><<<grid, DOK_TPB, 0, s>>>(d, di, rows_per_wave(di.n_elems, grid))));
  return note_launch();
}
template <class IX>
int count_items_lin(const DevTable &d, const dok_index_t *ix, int64_t *count, hipStream_t s) {
  IX di;
  int rc = make_dev_index(d, ix, nullptr, di);
  if (rc) return rc;
  if (di.n_elems == 0) return DOK_OK;
  if (!count || di.n_elems > kMaxRows) return DOK_EINVAL;
  const DeviceScope on_stream_device(s);
  P8_DISPATCH(d.value_bytes, (p8_countitems_kernel<V, IX><<<grid_counting(di.n_elems), DOK_TPB, 0, s>>>(d, di, (i64 *)count)));
  return note_launch();
}
template <class IX>
int zero_items_lin(const DevTable &d, const dok_index_t *ix, hipStream_t s) {
  IX di;
  int rc = make_dev_index(d, ix, nullptr, di);
  if (rc) return rc;
  if (di.n_elems == 0) return DOK_OK;
  if (di.n_elems > kMaxRows) return DOK_EINVAL;
  const DeviceScope on_stream_device(s);
  P8_DISPATCH(d.value_bytes, (p8_zeroitems_kernel<V, IX><<<grid_counting(di.n_elems), DOK_TPB, 0, s>>>(d, di)));
  return note_launch();
}
template <class IX>
int getitem_sparse_lin(const DevTable &d, const dok_index_t *ix, const DevTable &o, hipStream_t s) {
  IX di;
  int rc = make_dev_index(d, ix, nullptr, di);
  if (rc) return rc;
  if (o.lin_ndim != di.sel_ndim) return DOK_EINVAL;
  for (int j = 0; j < di.sel_ndim; j++) if (o.lin_dims[j] != di.shape[j]) return DOK_EINVAL;
  if (di.n_elems == 0) return DOK_OK;
  if (di.n_elems > kMaxRows) return DOK_EINVAL;
  const DeviceScope on_stream_device(s);
  P8_DISPATCH(d.value_bytes, (p8_getitem_sparse_kernel<V, IX><<<grid_counting(di.n_elems), DOK_TPB, 0, s>>>(d, di, o)));
  return note_launch();
}
template <class IX>
int setitem_sparse_lin(const DevTable &d, const dok_index_t *ix, const int64_t *src_indices,
                              const void *src_values, int64_t n_src, uint64_t nonzero_mask, hipStream_t s) {
  IX di;
  int rc = make_dev_index(d, ix, nullptr, di);
  if (rc) return rc;
  if (n_src == 0) return DOK_OK;
  if (!src_values || (!src_indices && di.sel_ndim > 0)) return DOK_EINVAL;
  const DeviceScope on_stream_device(s);
  const unsigned grid = grid_counting(n_src);
  P8_DISPATCH(d.value_bytes, (p8_setitem_sparse_kernel<V, IX><<<grid, DOK_TPB, 0, s>>>(
      d, di, (const i64 *)src_indices, src_values, n_src, nonzero_mask, rows_per_wave(n_src, grid))));
  return note_launch();
}

}  // namespace

extern "C" {

int dok_layout_of(int32_t key_bytes, int32_t value_bytes, int32_t *slots_per_bucket) {
  return layout_of(key_bytes, value_bytes, slots_per_bucket);
}

int64_t dok_phys_buckets_for(int64_t capacity, int32_t key_bytes, int32_t value_bytes) {
  int slots = 0;
  const int lay = layout_of(key_bytes, value_bytes, &slots);
  if (lay < 0) return lay;
  if (capacity < 1) capacity = 1;
  return (capacity + slots - 1) / slots;
}

const char *dok_last_hip_error(void) { return g_last_error; }

int dok_table_clear(const dok_table_t *t, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  // a fill kernel rather than a memset node, so that the call can be captured into a graph
  const i64 words = (i64)d.nb * 16;
  dok_fill_kernel<<<(unsigned)((words / 4 + DOK_TPB - 1) / DOK_TPB), DOK_TPB, 0, s>>>(d.buckets, words, d.header);
  return note_launch();
}

// Shared body of the get entry points.  fallback: host pointer (NULL = zeros); fb_dev: device
// pointer that the kernel reads instead.
static int map_get(const dok_table_t *t, const void *keys, int64_t n, void *values_out, const void *fallback,
                   const void *fb_dev, uint8_t *found, bool stats, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (n < 0 || n > kMaxRows) return DOK_EINVAL;
  if (n == 0) return DOK_OK;
  if (!keys || !values_out || !found) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  if (layout == DOK_LAYOUT_PACKED8) {
    if (fb_dev && ((uintptr_t)fb_dev & (uintptr_t)(d.value_bytes - 1)) != 0) return DOK_EINVAL;
    const u64 fb = fallback_word(fallback, d.value_bytes);
    if (stats) {
      P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, (p8_get_kernel<V, true, KF><<<grid_counting(n), DOK_TPB, 0, s>>>(d, keys, n, values_out, found, fb, fb_dev)));
    } else {
      P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, (p8_get_kernel<V, false, KF><<<grid_for(n), DOK_TPB, 0, s>>>(d, keys, n, values_out, found, fb, fb_dev)));
    }
  } else {
    TgRows r;
    rc = tg_rows(d, keys, nullptr, r);
    if (!rc) rc = tg_launch_get(d, r, n, values_out, fallback, fb_dev, found, stats, s);
    if (rc) return rc;
  }
  return note_launch();
}

int dok_map_get(const dok_table_t *t, const void *keys, int64_t n, void *values_out,
                const void *fallback, uint8_t *found, void *stream) {
  return map_get(t, keys, n, values_out, fallback, nullptr, found, false, stream);
}

int dok_map_get_dev_fallback(const dok_table_t *t, const void *keys, int64_t n, void *values_out,
                             const void *fallback_dev, uint8_t *found, void *stream) {
  if (!fallback_dev) return DOK_EINVAL;
  return map_get(t, keys, n, values_out, nullptr, fallback_dev, found, false, stream);
}

int dok_map_get_stats(const dok_table_t *t, const void *keys, int64_t n, void *values_out,
                      const void *fallback, uint8_t *found, void *stream) {
  return map_get(t, keys, n, values_out, fallback, nullptr, found, true, stream);
}

int dok_map_set(const dok_table_t *t, const void *keys, const void *values, int64_t n,
                uint8_t *stored, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (n < 0 || n > kMaxRows) return DOK_EINVAL;
  if (n == 0) return DOK_OK;
  if (!keys || !values) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  if (layout == DOK_LAYOUT_PACKED8) {
    const unsigned grid = grid_counting(n);
    P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, (p8_set_kernel<V, KF><<<grid, DOK_TPB, 0, s>>>(d, keys, values, n, stored, rows_per_wave(n, grid))));
  } else {
    TgRows r;
    rc = tg_rows(d, keys, values, r);
    if (!rc) rc = tg_launch_set(d, r, n, stored, s);
    if (rc) return rc;
  }
  return note_launch();
}

int dok_coo_set(const dok_table_t *t, const int64_t *indices, const void *values, int64_t n, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (d.lin_ndim == 0) return DOK_EINVAL;
  if (n < 0 || n > kMaxRows) return DOK_EINVAL;
  if (n == 0) return DOK_OK;
  if (!indices || !values) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  if (layout == DOK_LAYOUT_PACKED8) {
    constexpr int KF = DOK_KF_COLS;
    const unsigned grid = grid_counting(n);
    P8_DISPATCH(d.value_bytes, (p8_set_kernel<V, KF><<<grid, DOK_TPB, 0, s>>>(d, indices, values, n, nullptr, rows_per_wave(n, grid))));
  } else {
    if (((uintptr_t)indices & 7) != 0 || ((uintptr_t)values & (uintptr_t)(d.value_bytes - 1)) != 0) return DOK_EINVAL;
    const TgCols c{(const i64 *)indices, n, (const u8 *)values};
    rc = tg_launch_set(d, c, n, nullptr, s);
    if (rc) return rc;
  }
  return note_launch();
}

int64_t dok_bulk_workspace_bytes(const dok_table_t *t, int64_t n) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (layout != DOK_LAYOUT_PACKED8) return n >= 1 && n <= kMaxRows ? tg_fast_workspace_bytes(n) : 0;
  BulkPlan p;
  if (!bulk_plan(d, n, p)) return 0;
  return (int64_t)p.bytes;
}

// Shared body of the bulk entry points; `cols` selects the column-major coordinate format,
// `fresh` the build into uninitialised table memory.
static int set_bulk(const dok_table_t *t, const void *keys, const void *values, int64_t n, bool cols, bool fresh,
                    void *workspace, int64_t workspace_bytes, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (cols && d.lin_ndim == 0) return DOK_EINVAL;
  if (n < 0) return DOK_EINVAL;
  if (n == 0) return fresh ? DOK_EINVAL : DOK_OK;      // a build writes the table: it needs rows
  if (!keys || !values || !workspace) return DOK_EINVAL;
  if (layout != DOK_LAYOUT_PACKED8) {
    // multi-word layout: the insert with one compare-and-swap per new row and a list of deferred rows
    if (n > kMaxRows || ((uintptr_t)workspace & 255) != 0 || workspace_bytes < tg_fast_workspace_bytes(n)) return DOK_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    const DeviceScope on_stream_device(s);
    if (fresh) {
      const i64 words = (i64)d.nb * 16;
      dok_fill_kernel<<<(unsigned)((words / 4 + DOK_TPB - 1) / DOK_TPB), DOK_TPB, 0, s>>>(d.buckets, words, d.header);
    }
    if (cols) {
      if (((uintptr_t)keys & 7) != 0 || ((uintptr_t)values & (uintptr_t)(d.value_bytes - 1)) != 0) return DOK_EINVAL;
      const TgCols c{(const i64 *)keys, n, (const u8 *)values};
      rc = tg_fast_serves(d, fresh) ? tg_launch_set_fast(d, c, n, fresh, workspace, s) : tg_launch_set(d, c, n, nullptr, s);
    } else {
      TgRows r;
      rc = tg_rows(d, keys, values, r);
      if (!rc) rc = tg_fast_serves(d, fresh) ? tg_launch_set_fast(d, r, n, fresh, workspace, s) : tg_launch_set(d, r, n, nullptr, s);
    }
    if (rc) return rc;
    return note_launch();
  }
  BulkPlan p;
  if (!bulk_plan(d, n, p)) return DOK_EUNSUPPORTED;
  if (((uintptr_t)workspace & 255) != 0 || workspace_bytes < (int64_t)p.bytes) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  // the launch plan shares the workspace layout of the sizing plan above and only narrows the grids
  // A table of several windows (more than 2^28 buckets) is built as "clear, then upsert": the rows
  // that leave a window are placed in the next one before that one's merge, which therefore has to
  // read its ranges instead of taking them as empty.
  const bool build = fresh && p.n_windows == 1;
  if (fresh && !build) {
    const i64 words = (i64)d.nb * 16;
    dok_fill_kernel<<<(unsigned)((words / 4 + DOK_TPB - 1) / DOK_TPB), DOK_TPB, 0, s>>>(d.buckets, words, d.header);
  }
#define BULK_GO (bulk_plan_for<V, KF>(d, n, p),                                                    \
                 build ? bulk_launch<V, KF, true>(d, keys, values, n, p, workspace, s)             \
                       : bulk_launch<V, KF, false>(d, keys, values, n, p, workspace, s))
  if (cols) {
    constexpr int KF = DOK_KF_COLS;
    P8_DISPATCH(d.value_bytes, BULK_GO);
  } else if (d.lin_ndim == 0 && d.key_bytes == 8) {
    // 8-byte raw keys are already in table form: the loader without the width switch lets the
    // compiler keep a whole tile's loads in flight
    constexpr int KF = DOK_KF_U64;
    P8_DISPATCH(d.value_bytes, BULK_GO);
  } else {
    P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, BULK_GO);
  }
#undef BULK_GO
  return note_launch();
}

int dok_map_set_bulk(const dok_table_t *t, const void *keys, const void *values, int64_t n,
                     void *workspace, int64_t workspace_bytes, void *stream) {
  return set_bulk(t, keys, values, n, false, false, workspace, workspace_bytes, stream);
}

int dok_coo_set_bulk(const dok_table_t *t, const int64_t *indices, const void *values, int64_t n,
                     void *workspace, int64_t workspace_bytes, void *stream) {
  return set_bulk(t, indices, values, n, true, false, workspace, workspace_bytes, stream);
}

int dok_map_build_bulk(const dok_table_t *t, const void *keys, const void *values, int64_t n,
                       void *workspace, int64_t workspace_bytes, void *stream) {
  return set_bulk(t, keys, values, n, false, true, workspace, workspace_bytes, stream);
}

int dok_coo_build_bulk(const dok_table_t *t, const int64_t *indices, const void *values, int64_t n,
                       void *workspace, int64_t workspace_bytes, void *stream) {
  return set_bulk(t, indices, values, n, true, true, workspace, workspace_bytes, stream);
}

static int map_remove(const dok_table_t *t, const void *keys, int64_t n, uint8_t *removed, bool unique, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (n < 0 || n > kMaxRows) return DOK_EINVAL;
  if (n == 0) return DOK_OK;
  if (!keys) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  if (layout == DOK_LAYOUT_PACKED8) {
    if (unique) {
      P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, (p8_remove_kernel<V, KF, true><<<grid_counting(n), DOK_TPB, 0, s>>>(d, keys, n, removed)));
    } else {
      P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, (p8_remove_kernel<V, KF, false><<<grid_counting(n), DOK_TPB, 0, s>>>(d, keys, n, removed)));
    }
  } else {
    TgRows r;
    rc = tg_rows(d, keys, nullptr, r);
    if (!rc) rc = tg_launch_remove(d, r, n, removed, unique, s);
    if (rc) return rc;
  }
  return note_launch();
}

int dok_map_remove(const dok_table_t *t, const void *keys, int64_t n, uint8_t *removed, void *stream) {
  return map_remove(t, keys, n, removed, false, stream);
}

int dok_map_remove_unique(const dok_table_t *t, const void *keys, int64_t n, uint8_t *removed, void *stream) {
  return map_remove(t, keys, n, removed, true, stream);
}

int dok_map_remove_bulk(const dok_table_t *t, const void *keys, int64_t n, void *workspace, int64_t workspace_bytes,
                        void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (n < 0) return DOK_EINVAL;
  if (n == 0) return DOK_OK;
  if (!keys || !workspace) return DOK_EINVAL;
  BulkPlan p;
  if (layout != DOK_LAYOUT_PACKED8 || !bulk_plan(d, n, p)) return DOK_EUNSUPPORTED;
  if (((uintptr_t)workspace & 255) != 0 || workspace_bytes < (int64_t)p.bytes) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  { constexpr int KF = DOK_KF_U64;
    P8_DISPATCH(d.value_bytes, (bulk_plan_for<V, KF>(d, n, p), bulk_launch_remove<V>(d, keys, n, p, workspace, s))); }
  return note_launch();
}

int dok_map_count_existing(const dok_table_t *t, const void *keys, int64_t n, int64_t *count, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (n < 0 || n > kMaxRows) return DOK_EINVAL;
  if (n == 0) return DOK_OK;
  if (!keys || !count) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  if (layout == DOK_LAYOUT_PACKED8) {
    P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, (p8_count_kernel<V, KF><<<grid_counting(n), DOK_TPB, 0, s>>>(d, keys, n, (i64 *)count)));
  } else {
    TgRows r;
    rc = tg_rows(d, keys, nullptr, r);
    if (!rc) rc = tg_launch_count(d, r, n, (i64 *)count, s);
    if (rc) return rc;
  }
  return note_launch();
}

int dok_map_update_existing(const dok_table_t *t, const void *keys, const void *values, int64_t n,
                            int64_t *missing, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (layout != DOK_LAYOUT_PACKED8) return DOK_EUNSUPPORTED;
  if (n < 0 || n > kMaxRows) return DOK_EINVAL;
  if (n == 0) return DOK_OK;
  if (!keys || !values || !missing) return DOK_EINVAL;
  if (((uintptr_t)values & (uintptr_t)(d.value_bytes - 1)) != 0) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, (p8_update_kernel<V, KF><<<grid_counting(n), DOK_TPB, 0, s>>>(
      d, keys, values, n, (i64 *)missing)));
  return note_launch();
}

int64_t dok_compact_scratch_bytes(const dok_table_t *t) {
  if (!t || t->n_phys_buckets < 1) return DOK_EINVAL;
  const i64 n_chunks = (t->n_phys_buckets + DOK_CHUNK - 1) / DOK_CHUNK;
  return (n_chunks + 1) * 8;
}

int dok_map_compact(const dok_table_t *t, void *keys_out, void *values_out, int64_t capacity_rows,
                    int64_t *count_out, void *scratch, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (!count_out || !scratch || capacity_rows < 0) return DOK_EINVAL;
  if (((uintptr_t)scratch & 7) != 0) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  const i64 n_chunks = chunks_of(d);
  i64 *offs = (i64 *)scratch;
  if (layout == DOK_LAYOUT_PACKED8) {
    P8_DISPATCH(d.value_bytes, (p8_chunk_count_kernel<V><<<chunk_grid(n_chunks), DOK_TPB, 0, s>>>(d, offs, n_chunks)));
    dok_scan_kernel<<<1, 1024, 0, s>>>(offs, n_chunks, d.lin_ndim == 0 ? d.header : nullptr, (i64 *)count_out);
    if (keys_out || values_out) {
      P8_DISPATCH_LIN(d.value_bytes, d.lin_ndim > 0, (p8_chunk_write_kernel<V, KF><<<chunk_grid(n_chunks), DOK_TPB, 0, s>>>(d, offs, n_chunks, keys_out, values_out, capacity_rows)));
    }
  } else {
    rc = tg_launch_compact(d, offs, n_chunks, keys_out, values_out, capacity_rows, (i64 *)count_out, false, s);
    if (rc) return rc;
  }
  return note_launch();
}

int64_t dok_static_scratch_bytes(void) { return DOK_STATIC_SCRATCH_BYTES; }

int dok_map_compact_static(const dok_table_t *t, void *keys_out, void *values_out, int64_t capacity_rows,
                           int64_t *count_out, void *stream) {
  const int64_t need = dok_compact_scratch_bytes(t);
  if (need < 0) return (int)need;
  if (need > DOK_STATIC_SCRATCH_BYTES) return DOK_ETOOLARGE;     // before anything is launched
  const DeviceScope on_stream_device((hipStream_t)stream);      // (the scratch of the GPU the stream runs on)
  void *scratch = nullptr;
  int rc = static_scratch_of_current_device(&scratch);
  if (rc) return rc;
  // every word of the scratch that is read is written first (chunk counts, then their prefix
  // sums), so what an earlier call left behind does not matter
  return dok_map_compact(t, keys_out, values_out, capacity_rows, count_out, scratch, stream);
}

int dok_coo_compact(const dok_table_t *t, int64_t *indices_out, void *values_out, int64_t capacity,
                    int64_t *count_out, void *scratch, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (d.lin_ndim == 0) return DOK_EINVAL;
  if (!count_out || !scratch || capacity < 0) return DOK_EINVAL;
  if (((uintptr_t)scratch & 7) != 0) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  const i64 n_chunks = chunks_of(d);
  i64 *offs = (i64 *)scratch;
  if (layout != DOK_LAYOUT_PACKED8) {
    rc = tg_launch_compact(d, offs, n_chunks, indices_out, values_out, capacity, (i64 *)count_out, true, s);
    if (rc) return rc;
    return note_launch();
  }
  P8_DISPATCH(d.value_bytes, (p8_chunk_count_kernel<V><<<chunk_grid(n_chunks), DOK_TPB, 0, s>>>(d, offs, n_chunks)));
  dok_scan_kernel<<<1, 1024, 0, s>>>(offs, n_chunks, nullptr, (i64 *)count_out);
  if (indices_out || values_out) {
    constexpr int KF = DOK_KF_COLS;
    P8_DISPATCH(d.value_bytes, (p8_chunk_write_kernel<V, KF><<<chunk_grid(n_chunks), DOK_TPB, 0, s>>>(d, offs, n_chunks, indices_out, values_out, capacity)));
  }
  return note_launch();
}

int dok_map_rehash(const dok_table_t *src, const dok_table_t *dst, void *stream) {
  DevTable a, b; int la, lb;
  int rc = make_dev_table(src, a, la);
  if (rc) return rc;
  rc = make_dev_table(dst, b, lb);
  if (rc) return rc;
  if (a.key_bytes != b.key_bytes || a.value_bytes != b.value_bytes || a.lin_ndim != b.lin_ndim) return DOK_EINVAL;
  if (a.buckets == b.buckets) return DOK_EINVAL;
  for (int k = 0; k < a.lin_ndim; k++) if (a.lin_dims[k] != b.lin_dims[k]) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  const i64 n_chunks = chunks_of(a);
  if (la == DOK_LAYOUT_PACKED8) {
    P8_DISPATCH(a.value_bytes, (p8_rehash_kernel<V><<<chunk_grid(n_chunks), DOK_TPB, 0, s>>>(a, b, n_chunks)));
  } else {
    rc = tg_launch_rehash(a, b, n_chunks, s);
    if (rc) return rc;
  }
  return note_launch();
}

// Rows the source of a bulk rehash is scanned as (every 8-byte word of its buckets) and the most
// of them that can be live entries.
static void rehash_rows(const DevTable &a, i64 &n_in, i64 &n_cap) {
  n_in = (i64)a.nb * 16;
  n_cap = (i64)a.nb * (120 / (8 + a.value_bytes));
}

int64_t dok_rehash_bulk_workspace_bytes(const dok_table_t *src, const dok_table_t *dst) {
  DevTable a, b; int la, lb;
  int rc = make_dev_table(src, a, la);
  if (rc) return rc;
  rc = make_dev_table(dst, b, lb);
  if (rc) return rc;
  if (la != DOK_LAYOUT_PACKED8 || lb != DOK_LAYOUT_PACKED8) return 0;
  i64 n_in, n_cap;
  rehash_rows(a, n_in, n_cap);
  BulkPlan p;
  if (!bulk_plan(b, n_in, p, DOK_BULK_GRID, DOK_BULK_GRID, n_cap)) return 0;
  return (int64_t)p.bytes;
}

int dok_map_rehash_bulk(const dok_table_t *src, const dok_table_t *dst, void *workspace,
                        int64_t workspace_bytes, void *stream) {
  DevTable a, b; int la, lb;
  int rc = make_dev_table(src, a, la);
  if (rc) return rc;
  rc = make_dev_table(dst, b, lb);
  if (rc) return rc;
  if (a.key_bytes != b.key_bytes || a.value_bytes != b.value_bytes || a.lin_ndim != b.lin_ndim) return DOK_EINVAL;
  if (a.buckets == b.buckets || !workspace) return DOK_EINVAL;
  for (int k = 0; k < a.lin_ndim; k++) if (a.lin_dims[k] != b.lin_dims[k]) return DOK_EINVAL;
  if (la != DOK_LAYOUT_PACKED8) return DOK_EUNSUPPORTED;
  i64 n_in, n_cap;
  rehash_rows(a, n_in, n_cap);
  BulkPlan p;
  if (!bulk_plan(b, n_in, p, DOK_BULK_GRID, DOK_BULK_GRID, n_cap)) return DOK_EUNSUPPORTED;
  if (((uintptr_t)workspace & 255) != 0 || workspace_bytes < (int64_t)p.bytes) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  constexpr int KF = DOK_KF_TABLE;
  const bool build = p.n_windows == 1;           // (several windows: clear, then upsert - see set_bulk)
  if (!build) {
    const i64 words = (i64)b.nb * 16;
    dok_fill_kernel<<<(unsigned)((words / 4 + DOK_TPB - 1) / DOK_TPB), DOK_TPB, 0, s>>>(b.buckets, words, b.header);
  }
  P8_DISPATCH(b.value_bytes, (bulk_plan_for<V, KF>(b, n_in, p, n_cap),
                              build ? bulk_launch<V, KF, true>(b, a.buckets, nullptr, n_in, p, workspace, s)
                                    : bulk_launch<V, KF, false>(b, a.buckets, nullptr, n_in, p, workspace, s)));
  bulk_side_slots_kernel<<<1, 64, 0, s>>>(a, b);
  return note_launch();
}

// The DOK indexing entry points take both kinds of coordinate table: linearised keys on the packed
// layout (DevIndex, kernels of dok_packed8.h) and int64 coordinate rows on the multi-word layout
// (DevIndexW, the kernels of dok_tagged.h fed by an index source).
int dok_getitem_dense(const dok_table_t *t, const dok_index_t *ix, void *out, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (is_coord_rows(d, layout)) {
    TgIndexSrc src;
    rc = make_dev_index(d, ix, nullptr, src.ix);
    if (rc) return rc;
    if (src.ix.n_elems == 0) return DOK_OK;
    if (!out || src.ix.n_elems > kMaxRows) return DOK_EINVAL;
    const DeviceScope on_stream_device(s);
    rc = tg_launch_get(d, src, src.ix.n_elems, out, nullptr, nullptr, nullptr, false, s);
    if (rc) return rc;
    return note_launch();
  }
  return small_index(ix) ? getitem_dense_lin<DevIndex4>(d, ix, out, s) : getitem_dense_lin<DevIndex>(d, ix, out, s);
}

int dok_setitem_dense(const dok_table_t *t, const dok_index_t *ix, const dok_view_t *src, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (!src) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  if (is_coord_rows(d, layout)) {
    TgIndexSrc isrc;
    rc = make_dev_index(d, ix, src, isrc.ix);
    if (rc) return rc;
    if (isrc.ix.n_elems == 0) return DOK_OK;
    if (isrc.ix.n_elems > kMaxRows || ((uintptr_t)src->data & (uintptr_t)(d.value_bytes - 1)) != 0) return DOK_EINVAL;
    const DeviceScope on_stream_device(s);
    rc = tg_launch_set(d, isrc, isrc.ix.n_elems, nullptr, s);
    if (rc) return rc;
    return note_launch();
  }
  return small_index(ix) ? setitem_dense_lin<DevIndex4>(d, ix, src, s) : setitem_dense_lin<DevIndex>(d, ix, src, s);
}

int dok_setitem_dense_bulk(const dok_table_t *t, const dok_index_t *ix, const dok_view_t *src, void *workspace,
                           int64_t workspace_bytes, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (!is_coord_rows(d, layout)) return dok_setitem_dense(t, ix, src, stream);    // (no use for the workspace)
  if (!src || !workspace) return DOK_EINVAL;
  TgIndexSrc isrc;
  rc = make_dev_index(d, ix, src, isrc.ix);
  if (rc) return rc;
  const i64 n = isrc.ix.n_elems;
  if (n == 0) return DOK_OK;
  if (n > kMaxRows || ((uintptr_t)src->data & (uintptr_t)(d.value_bytes - 1)) != 0) return DOK_EINVAL;
  if (((uintptr_t)workspace & 255) != 0 || workspace_bytes < tg_fast_workspace_bytes(n)) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  rc = tg_launch_set_fast(d, isrc, n, false, workspace, s);
  if (rc) return rc;
  return note_launch();
}

int dok_count_items(const dok_table_t *t, const dok_index_t *ix, int64_t *count, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (is_coord_rows(d, layout)) {
    TgIndexSrc src;
    rc = make_dev_index(d, ix, nullptr, src.ix);
    if (rc) return rc;
    if (src.ix.n_elems == 0) return DOK_OK;
    if (!count || src.ix.n_elems > kMaxRows) return DOK_EINVAL;
    const DeviceScope on_stream_device(s);
    rc = tg_launch_count(d, src, src.ix.n_elems, (i64 *)count, s);
    if (rc) return rc;
    return note_launch();
  }
  return small_index(ix) ? count_items_lin<DevIndex4>(d, ix, count, s) : count_items_lin<DevIndex>(d, ix, count, s);
}

int dok_zero_items(const dok_table_t *t, const dok_index_t *ix, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (is_coord_rows(d, layout)) {
    TgIndexSrc src;
    rc = make_dev_index(d, ix, nullptr, src.ix);
    if (rc) return rc;
    if (src.ix.n_elems == 0) return DOK_OK;
    if (src.ix.n_elems > kMaxRows) return DOK_EINVAL;
    const DeviceScope on_stream_device(s);
    rc = tg_launch_remove(d, src, src.ix.n_elems, nullptr, false, s);
    if (rc) return rc;
    return note_launch();
  }
  return small_index(ix) ? zero_items_lin<DevIndex4>(d, ix, s) : zero_items_lin<DevIndex>(d, ix, s);
}

int dok_getitem_sparse(const dok_table_t *t, const dok_index_t *ix, const dok_table_t *out, void *stream) {
  DevTable d, o; int layout, lo;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  rc = make_dev_table(out, o, lo);
  if (rc) return rc;
  // `out` is keyed by the offsets into the index space: a table of linearised coordinates
  if (!is_lin(o, lo)) return o.lin_ndim > 0 ? DOK_EUNSUPPORTED : DOK_EINVAL;
  if (o.value_bytes != d.value_bytes || o.buckets == d.buckets) return DOK_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  if (is_coord_rows(d, layout)) {
    TgIndexSrc src;
    rc = make_dev_index(d, ix, nullptr, src.ix);
    if (rc) return rc;
    if (o.lin_ndim != src.ix.sel_ndim) return DOK_EINVAL;
    for (int j = 0; j < src.ix.sel_ndim; j++) if (o.lin_dims[j] != src.ix.shape[j]) return DOK_EINVAL;
    if (src.ix.n_elems == 0) return DOK_OK;
    if (src.ix.n_elems > kMaxRows) return DOK_EINVAL;
    const DeviceScope on_stream_device(s);
    rc = tg_launch_getitem_sparse(d, src, o, s);
    if (rc) return rc;
    return note_launch();
  }
  return small_index(ix) ? getitem_sparse_lin<DevIndex4>(d, ix, o, s) : getitem_sparse_lin<DevIndex>(d, ix, o, s);
}

int dok_setitem_sparse(const dok_table_t *t, const dok_index_t *ix, const int64_t *src_indices,
                       const void *src_values, int64_t n_src, uint64_t nonzero_mask, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (n_src < 0 || n_src > kMaxRows) return DOK_EINVAL;
  if (is_coord_rows(d, layout)) {
    TgSparseSrc src;
    rc = make_dev_index(d, ix, nullptr, src.ix);
    if (rc) return rc;
    if (n_src == 0) return DOK_OK;
    if (!src_values || (!src_indices && src.ix.sel_ndim > 0)) return DOK_EINVAL;
    if (((uintptr_t)src_indices & 7) != 0 || ((uintptr_t)src_values & (uintptr_t)(d.value_bytes - 1)) != 0) return DOK_EINVAL;
    src.src_indices = (const i64 *)src_indices;
    src.src_values = (const u8 *)src_values;
    src.n_src = n_src;
    src.nonzero_mask = nonzero_mask;
    const DeviceScope on_stream_device(s);
    rc = tg_launch_set(d, src, n_src, nullptr, s);
    if (rc) return rc;
    return note_launch();
  }
  return small_index(ix) ? setitem_sparse_lin<DevIndex4>(d, ix, src_indices, src_values, n_src, nonzero_mask, s)
                         : setitem_sparse_lin<DevIndex>(d, ix, src_indices, src_values, n_src, nonzero_mask, s);
}

int dok_to_dense(const dok_table_t *t, void *dense, void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (d.lin_ndim == 0 || !dense) return DOK_EINVAL;
  unsigned __int128 vol = 1;
  for (int k = 0; k < d.lin_ndim; k++) {
    vol *= (unsigned __int128)d.lin_dims[k];
    if (vol >> 62) return DOK_EINVAL;              // no such dense tensor exists
  }
  const i64 volume = (i64)vol;
  if (volume == 0) return DOK_OK;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  const i64 n_chunks = chunks_of(d);
  if (layout == DOK_LAYOUT_PACKED8) {
    P8_DISPATCH(d.value_bytes, (p8_to_dense_kernel<V><<<chunk_grid(n_chunks), DOK_TPB, 0, s>>>(d, dense, n_chunks, volume)));
  } else {
    rc = tg_launch_to_dense(d, dense, n_chunks, s);
    if (rc) return rc;
  }
  return note_launch();
}

int dok_line_gather_granule(const dok_table_t *t, int64_t n, uint64_t seed, int32_t granule_bytes, uint32_t *out,
                            void *stream) {
  DevTable d; int layout;
  int rc = make_dev_table(t, d, layout);
  if (rc) return rc;
  if (n < 0 || (n > 0 && !out)) return DOK_EINVAL;
  if (granule_bytes != 128 && granule_bytes != 64 && granule_bytes != 32) return DOK_EINVAL;
  if (n == 0) return DOK_OK;
  const int lanes = granule_bytes / 8;
  const u64 n_granules = d.nb * (u64)(128 / granule_bytes);
  if (n_granules > 0xffffffffULL) return DOK_EUNSUPPORTED;
  const i64 groups = (n + 7) / 8;
  i64 blocks = (groups * lanes + DOK_TPB - 1) / DOK_TPB;
  if (blocks > 16384) blocks = 16384;
  hipStream_t s = (hipStream_t)stream;
  const DeviceScope on_stream_device(s);
  const u64 *lines = (const u64 *)d.buckets;
  if (lanes == 16) dok_line_gather_kernel<16><<<(unsigned)blocks, DOK_TPB, 0, s>>>(lines, n_granules, n, seed, out);
  else if (lanes == 8) dok_line_gather_kernel<8><<<(unsigned)blocks, DOK_TPB, 0, s>>>(lines, n_granules, n, seed, out);
  else dok_line_gather_kernel<4><<<(unsigned)blocks, DOK_TPB, 0, s>>>(lines, n_granules, n, seed, out);
  return note_launch();
}

int dok_line_gather(const dok_table_t *t, int64_t n, uint64_t seed, uint32_t *out, void *stream) {
  return dok_line_gather_granule(t, n, seed, 128, out, stream);
}

}  // extern "C"
