// C ABI of libsba.so (declarations and the upstream functions each entry point replaces are
// in include/sba.h).  Host code only validates, sizes and launches.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>

#include "sba.h"
#include "sba_kernels.hpp"

namespace {

using namespace sba;

// Process-wide on purpose: PyTorch runs the backward on its own autograd thread.
std::atomic<int> g_timing{0};
std::atomic<int> g_dkdv_workgroups{0};   // sba_set_dkdv_workgroups
std::atomic<float> g_ms[3];

inline int cdiv_i(long long a, long long b) { return (int)((a + b - 1) / b); }

struct Sizes {
  int n_docs;        // documents the scheduler sees (fixed: batch)
  long long rows;    // batch * tokens
  int n_q_max, n_kv_max;
};

int check_problem(const sba_problem* p, bool fixed, Sizes* sz) {
  if (p == nullptr) return SBA_E_NULL;
  if (p->dtype != SBA_BF16 && p->dtype != SBA_F16) return SBA_E_DTYPE;
  if (p->head_dim != 32 && p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256) return SBA_E_HEAD_DIM;
  if (p->heads <= 0 || p->tokens < 0 || p->batch <= 0 || p->max_doc_len < 0) return SBA_E_SHAPE;
  if (fixed != ((p->flags & SBA_FIXED_LENGTH) != 0)) return SBA_E_SHAPE;
  if (fixed) {
    if (p->max_doc_len != p->tokens) return SBA_E_SHAPE;
  } else {
    if (p->batch != 1 || p->n_docs < 0) return SBA_E_SHAPE;
    if (p->n_docs > 0 && p->cu_seqlens == nullptr) return SBA_E_NULL;
  }
  sz->n_docs = fixed ? p->batch : p->n_docs;
  sz->rows = (long long)p->batch * p->tokens;
  sz->n_q_max = (int)(sz->rows / BM) + sz->n_docs + 1;
  sz->n_kv_max = (int)(sz->rows / BKV) + sz->n_docs + 1;
  return 0;
}

// Carry-table entries per head.  Fixed-length: exact.  Packed documents: the most any split of
// `tokens` tokens into n_docs documents of at most max_doc_len tokens can need.  A document
// occupies what its length rounded up to a multiple of 32 needs, and that need is convex in
// the length, so the worst split is as many longest documents as fit plus the rest, with every
// document's rounding (at most 31 tokens each) added to the token count.
long long table_entries_bound(const sba_problem* p, bool fixed) {
  if (fixed) return (long long)p->batch * tab_doc_entries(p->tokens);
  const long long tokens = (long long)p->tokens + 31ll * p->n_docs;
  long long lmax = (p->max_doc_len > 0 && p->max_doc_len < p->tokens) ? p->max_doc_len : p->tokens;
  lmax = (lmax + 31) & ~31ll;
  if (lmax <= 0) return 0;
  return (tokens / lmax) * tab_doc_entries((int)lmax) + tab_doc_entries((int)(tokens % lmax));
}

// Grid bounds of the dk/dv pass.  The second group of the key-tile list holds at most TAIL_TILES
// tiles of every document.  The first group holds ceil(L / BKV) - 1 tiles of a document of more
// than TAIL_TILES * BKV tokens and none of a shorter one: at most rows / BKV in all and, with the
// declared longest document, at most that many per document.  The declaration is checked on the
// device: a longer document makes every backward kernel return and the outputs NaN.
int declared_max_doc_len(const sba_problem* p, bool fixed) {
  return (fixed || p->max_doc_len <= 0 || p->max_doc_len > p->tokens) ? p->tokens : p->max_doc_len;
}
struct BwdBounds { int n_long_max, n_tail_max; };
BwdBounds backward_bounds(const sba_problem* p, bool fixed, const Sizes& sz) {
  const int max_doc_len = declared_max_doc_len(p, fixed);
  const long long per_doc = (max_doc_len + BKV - 1) / BKV - kv_tail_tiles(max_doc_len);
  BwdBounds b;
  b.n_long_max = (int)std::min<long long>(sz.rows / BKV, per_doc * sz.n_docs);
  b.n_tail_max = (int)std::min<long long>(sz.n_kv_max, (long long)TAIL_TILES * sz.n_docs);
  return b;
}

size_t schedule_bytes(const Sizes& sz) {
  size_t words = SCHED_HDR + TILE_WORDS * ((size_t)sz.n_q_max + sz.n_kv_max) + 6 * (size_t)sz.n_docs + 2;
  return (words * sizeof(int) + 255) & ~(size_t)255;
}

int check_view(const sba_view* v, bool need_ptr) {
  if (v == nullptr) return SBA_E_NULL;
  if (need_ptr && v->ptr == nullptr) return SBA_E_NULL;
  return 0;
}

// 16-byte vector loads/stores need every row start aligned: strides multiple of 8 elements.
// Tile loads address a (document, head) slice with 32-bit byte offsets: the token stride must
// keep every row of the slice (plus one tile of slack) below 2 GiB.
int check_mat(const sba_view* v, const sba_problem* p) {
  int e = check_view(v, true);
  if (e) return e;
  if ((v->stride_b % 8) || (v->stride_h % 8) || (v->stride_t % 8) || ((uintptr_t)v->ptr % 16)) return SBA_E_STRIDE;
  if (v->stride_t < p->head_dim) return SBA_E_STRIDE;
  if (((long long)p->tokens + 8 * BM) * v->stride_t * 2 >= (1ll << 31)) return SBA_E_SHAPE;
  return 0;
}

View to_view(const sba_view* v) {
  View r;
  r.ptr = v ? (char*)v->ptr : nullptr;
  r.sb = v ? v->stride_b : 0;
  r.sh = v ? v->stride_h : 0;
  r.st = v ? v->stride_t : 0;
  return r;
}

// The counter words at the end of a table workspace of `table_bytes` bytes.
unsigned* work_words(float* table, size_t table_bytes) {
  return reinterpret_cast<unsigned*>(table) + (table_bytes / sizeof(unsigned) - WORK_WORDS);
}

// Compute units of the current device (0 if it cannot be asked: launches then take one workgroup per item).
int device_cus() {
  static std::atomic<int> cached[64];   // by device ordinal; 0 = not asked yet
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if ((n = cached[dev].load(std::memory_order_relaxed)) > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

int check_arch() {
  static int cached = -1;   // immutable once set
  if (cached >= 0) return cached ? 0 : SBA_E_ARCH;
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return SBA_E_ARCH;
  cached = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
  return cached ? 0 : SBA_E_ARCH;
}

// Brackets one compute launch with HIP events on the caller's stream.  Nothing waits here: the
// pair is parked and resolved when sba_last_kernel_ms asks for it, so that timed kernels follow
// one another on the device exactly as untimed ones do.
struct EventPair {
  hipEvent_t e0 = nullptr, e1 = nullptr;
};
std::mutex g_ev_mutex;
EventPair g_ev[3];

struct Timer {
  EventPair ev;
  hipStream_t s;
  int which;
  bool on;
  Timer(int which_, hipStream_t s_, bool allowed = true) : s(s_), which(which_), on(allowed && g_timing.load() != 0) {
    if (on) {
      on = hipEventCreate(&ev.e0) == hipSuccess && hipEventCreate(&ev.e1) == hipSuccess;
      if (on) (void)hipEventRecord(ev.e0, s);
    }
  }
  ~Timer() {
    EventPair done = ev;   // (timing off, or creation failed half-way: nothing to park)
    if (on) {
      (void)hipEventRecord(ev.e1, s);
      std::lock_guard<std::mutex> lock(g_ev_mutex);
      done = g_ev[which];
      g_ev[which] = ev;
    }
    if (done.e0) (void)hipEventDestroy(done.e0);
    if (done.e1) (void)hipEventDestroy(done.e1);
  }
};

// `table_bytes`: size of EACH carry table handed in (ignored when none is).
int fill_common(const sba_problem* p, bool fixed, const Sizes& sz, const void* schedule, size_t sched_bytes,
                bool with_table, size_t table_bytes, KArgs* a) {
  if (schedule == nullptr) return SBA_E_NULL;
  if (reinterpret_cast<uintptr_t>(schedule) & 15) return SBA_E_STRIDE;   // kernels read the header as one 16-byte word
  if (sched_bytes < schedule_bytes(sz)) return SBA_E_WORKSPACE;
  a->tab_stride = -1;
  if (with_table) {
    // (the last WORK_WORDS words of a table workspace are the work counters of the call's persistent launches)
    if (table_bytes < WORK_WORDS * sizeof(unsigned)) return SBA_E_WORKSPACE;
    table_bytes -= WORK_WORDS * sizeof(unsigned);
    a->tab_stride = (int64_t)(table_bytes / sizeof(float) / (size_t)p->heads) & ~(int64_t)31;   // heads start on 128-byte lines
    // fixed-length needs are known here; packed documents are checked on the device against
    // what the scheduler found (kernels refuse to run, outputs are filled with NaN)
    if (fixed && a->tab_stride < table_entries_bound(p, true)) return SBA_E_WORKSPACE;
    if (a->tab_stride <= 0) return SBA_E_WORKSPACE;
  }
  a->sched = reinterpret_cast<const int*>(schedule);
  a->kv_list_off = SCHED_HDR + TILE_WORDS * sz.n_q_max;
  a->n_kv_alloc = sz.n_kv_max;
  a->heads = p->heads;
  a->tokens = p->tokens;
  a->fuse = (p->flags & SBA_FUSE_REMAINDER) ? 1 : 0;
  a->inv_temp = p->inv_temp;
  a->c = p->inv_temp * 1.4426950408889634f;
  return 0;
}

int forward(const sba_problem* p, bool fixed, const void* schedule, size_t sched_bytes, const sba_view* q,
            const sba_view* k, const sba_view* v, const sba_view* o, const sba_view* rem, float* stick,
            size_t table_bytes, float* weights, size_t weights_bytes, void* stream, bool timed = true) {
  Sizes sz;
  int e = check_problem(p, fixed, &sz);
  if (e) return e;
  const bool table_only = (p->flags & SBA_TABLE_ONLY) != 0;   // nothing but the carry table is written; v, o, rem are not looked at
  if (table_only && (stick == nullptr || weights != nullptr)) return SBA_E_NULL;
  if ((e = check_mat(q, p)) || (e = check_mat(k, p))) return e;
  if (!table_only && ((e = check_mat(v, p)) || (e = check_mat(o, p)) || (e = check_view(rem, true)))) return e;
  if (weights != nullptr &&
      weights_bytes / sizeof(float) < (size_t)p->batch * p->heads * (size_t)p->tokens * (size_t)p->tokens)
    return SBA_E_WORKSPACE;
  KArgs a;
  std::memset(&a, 0, sizeof(a));
  if ((e = fill_common(p, fixed, sz, schedule, sched_bytes, stick != nullptr, table_bytes, &a))) return e;
  if ((e = check_arch())) return e;
  if (sz.rows == 0) return 0;
  a.q = to_view(q); a.k = to_view(k);
  if (table_only) a.v = a.o = a.rem = to_view(k);   // (placeholders: the kernel touches none of them)
  else { a.v = to_view(v); a.o = to_view(o); a.rem = to_view(rem); }
  a.stick = stick;
  a.weights = weights;
  a.clear_spare = fixed ? 0 : 1;
  a.nan_pair = p->dtype == SBA_F16 ? 0x7e007e00u : 0x7fc07fc0u;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipError_t he = hipSuccess;
  {   // (packed input without a single document still launches: the spare workgroups clear the outputs)
    Timer tm(0, s, timed);
    he = (p->dtype == SBA_F16 ? f16::launch_fwd : bf16::launch_fwd)(a, p->head_dim, (p->flags & SBA_ATTEND_CURRENT) != 0,
                    (p->flags & SBA_PRODUCT_SPACE) != 0, weights != nullptr ? 1 : (table_only ? 2 : 0), sz.n_q_max, s);
  }
  return (int)he;
}

int backward(const sba_problem* p, bool fixed, const void* schedule, size_t sched_bytes, const sba_view* q,
             const sba_view* k, const sba_view* v, const sba_view* go, const sba_view* grem, const float* stick,
             float* gtab, size_t table_bytes, const sba_view* dq, const sba_view* dk, const sba_view* dv,
             void* stream) {
  Sizes sz;
  int e = check_problem(p, fixed, &sz);
  if (e) return e;
  if ((e = check_mat(q, p)) || (e = check_mat(k, p)) || (e = check_mat(v, p)) || (e = check_mat(go, p)) ||
      (e = check_mat(dq, p)) || (e = check_mat(dk, p)) || (e = check_mat(dv, p)))
    return e;
  if (stick == nullptr || gtab == nullptr) return SBA_E_NULL;
  KArgs a;
  std::memset(&a, 0, sizeof(a));
  if ((e = fill_common(p, fixed, sz, schedule, sched_bytes, true, table_bytes, &a))) return e;
  if ((e = check_arch())) return e;
  if (sz.rows == 0) return 0;
  a.q = to_view(q); a.k = to_view(k); a.v = to_view(v); a.go = to_view(go);
  a.grem = to_view(grem);
  a.dq = to_view(dq); a.dk = to_view(dk); a.dv = to_view(dv);
  a.stick = const_cast<float*>(stick);
  a.gtab = gtab;
  // The main kernel of the dk/dv pass fills a compute unit with one workgroup.  With many more key tiles than
  // compute units it is launched once per compute unit and walks the tiles itself (see work_next in
  // sba_device.hpp); with few it pays more for the hand-over between tiles than the hardware does for a
  // fresh workgroup (measured: 960 tiles on 256 compute units, 124 against 118 us).
  const int forced = g_dkdv_workgroups.load();
  a.work = work_words(gtab, table_bytes);
  a.resident = forced > 0 ? std::max(8, forced & ~7) : (forced < 0 ? 0 : device_cus());
  a.min_items_each = forced > 0 ? 1 : 8;
  a.max_doc_len = declared_max_doc_len(p, fixed);
  const BwdBounds bb = backward_bounds(p, fixed, sz);
  const int n_long_max = bb.n_long_max, n_tail_max = bb.n_tail_max;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool ac = (p->flags & SBA_ATTEND_CURRENT) != 0, prod = (p->flags & SBA_PRODUCT_SPACE) != 0;
  a.clear_spare = fixed ? 0 : 1;
  a.nan_pair = p->dtype == SBA_F16 ? 0x7e007e00u : 0x7fc07fc0u;
  hipError_t he = hipSuccess;
  {
    Timer tm(1, s);
    he = (p->dtype == SBA_F16 ? f16::launch_bwd_dq : bf16::launch_bwd_dq)(a, p->head_dim, ac, prod, sz.n_q_max, s);
  }
  if (he == hipSuccess && sz.n_docs > 0) {
    Timer tm(2, s);
    he = (p->dtype == SBA_F16 ? f16::launch_bwd_dkdv : bf16::launch_bwd_dkdv)(a, p->head_dim, ac, prod, n_long_max, n_tail_max, s);
  }
  return (int)he;
}

// Schedule workspace of sba_varlen_fwd_static: one array per GPU, inside the code object, so the
// entry point needs no allocation.  In host code the name `scratch` is only a handle for
// hipGetSymbolAddress; kernels get the device address looked up once per device.
static __device__ __align__(256) unsigned char scratch[SBA_STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[MAX_DEVICES];

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void** out) {
  int dev = 0;
  hipError_t he = hipGetDevice(&dev);
  if (he != hipSuccess) return (int)he;
  if (dev < 0 || dev >= MAX_DEVICES) return SBA_E_ARCH;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    he = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (he != hipSuccess) return (int)he;
    if (ptr == nullptr) return SBA_E_NULL;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // every thread computes the same address
  }
  *out = ptr;
  return 0;
}

}  // namespace

extern "C" {

int sba_version(void) { return SBA_VERSION; }

const char* sba_error_string(int code) {
  switch (code) {
    case 0: return "ok";
    case SBA_E_NULL: return "a required pointer is NULL";
    case SBA_E_HEAD_DIM: return "head_dim must be 32, 64, 128 or 256";
    case SBA_E_DTYPE: return "unsupported element type (SBA_BF16 or SBA_F16)";
    case SBA_E_SHAPE: return "negative or inconsistent sizes";
    case SBA_E_STRIDE: return "pointer or stride breaks 16-byte row alignment";
    case SBA_E_WORKSPACE: return "workspace too small";
    case SBA_E_ARCH: return "current device is not gfx950 (MI355X)";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
  }
}

size_t sba_schedule_bytes(const sba_problem* p) {
  Sizes sz;
  const bool fixed = p != nullptr && (p->flags & SBA_FIXED_LENGTH) != 0;
  if (check_problem(p, fixed, &sz)) return 0;
  return schedule_bytes(sz);
}

size_t sba_table_bytes(const sba_problem* p) {
  Sizes sz;
  const bool fixed = p != nullptr && (p->flags & SBA_FIXED_LENGTH) != 0;
  if (check_problem(p, fixed, &sz)) return 0;
  return (size_t)p->heads * (size_t)table_entries_bound(p, fixed) * sizeof(float) + WORK_WORDS * sizeof(unsigned);
}

size_t sba_table_bytes_for_lengths(const sba_problem* p, const int64_t* doc_lengths, int n_lengths) {
  Sizes sz;
  const bool fixed = p != nullptr && (p->flags & SBA_FIXED_LENGTH) != 0;
  if (check_problem(p, fixed, &sz) || (n_lengths > 0 && doc_lengths == nullptr)) return 0;
  if (fixed) return sba_table_bytes(p);
  long long entries = 0;
  for (int i = 0; i < n_lengths; ++i) {
    if (doc_lengths[i] < 0 || doc_lengths[i] > p->tokens) return 0;
    entries += tab_doc_entries((int)doc_lengths[i]);
  }
  if (entries > 0x7fffffffll) return 0;   // a document's base must fit the scheduler's int32 field
  return (size_t)p->heads * (size_t)(entries > 0 ? entries : 32) * sizeof(float)   // never empty: one 128-byte line per head
         + WORK_WORDS * sizeof(unsigned);
}

int sba_build_schedule(const sba_problem* p, void* schedule, size_t schedule_size, void* stream) {
  Sizes sz;
  const bool fixed = p != nullptr && (p->flags & SBA_FIXED_LENGTH) != 0;
  int e = check_problem(p, fixed, &sz);
  if (e) return e;
  if (schedule == nullptr) return SBA_E_NULL;
  if (schedule_size < schedule_bytes(sz)) return SBA_E_WORKSPACE;
  if ((e = check_arch())) return e;
  SchedArgs a;
  a.cu = fixed ? nullptr : p->cu_seqlens;
  a.cu_is64 = (p->flags & SBA_CU_INT64) ? 1 : 0;
  a.n_docs = sz.n_docs;
  a.tokens = p->tokens;
  a.n_q_max = sz.n_q_max;
  a.n_kv_max = sz.n_kv_max;
  a.out = reinterpret_cast<int*>(schedule);
  return (int)launch_schedule(a, reinterpret_cast<hipStream_t>(stream));
}

int sba_varlen_fwd(const sba_problem* p, const void* schedule, size_t schedule_size, const sba_view* q,
                   const sba_view* k, const sba_view* v, const sba_view* o, const sba_view* rem,
                   float* stick_table, size_t table_size, void* stream) {
  return forward(p, false, schedule, schedule_size, q, k, v, o, rem, stick_table, table_size, nullptr, 0, stream);
}

int sba_attn_fwd(const sba_problem* p, const void* schedule, size_t schedule_size, const sba_view* q,
                 const sba_view* k, const sba_view* v, const sba_view* o, const sba_view* rem,
                 float* stick_table, size_t table_size, void* stream) {
  return forward(p, true, schedule, schedule_size, q, k, v, o, rem, stick_table, table_size, nullptr, 0, stream);
}

int sba_varlen_fwd_weights(const sba_problem* p, const void* schedule, size_t schedule_size, const sba_view* q,
                           const sba_view* k, const sba_view* v, const sba_view* o, const sba_view* rem,
                           float* stick_table, size_t table_size, float* weights, size_t weights_size,
                           void* stream) {
  if (weights == nullptr) return SBA_E_NULL;
  return forward(p, false, schedule, schedule_size, q, k, v, o, rem, stick_table, table_size, weights, weights_size,
                 stream);
}

int sba_attn_fwd_weights(const sba_problem* p, const void* schedule, size_t schedule_size, const sba_view* q,
                         const sba_view* k, const sba_view* v, const sba_view* o, const sba_view* rem,
                         float* stick_table, size_t table_size, float* weights, size_t weights_size,
                         void* stream) {
  if (weights == nullptr) return SBA_E_NULL;
  return forward(p, true, schedule, schedule_size, q, k, v, o, rem, stick_table, table_size, weights, weights_size,
                 stream);
}

int sba_varlen_bwd(const sba_problem* p, const void* schedule, size_t schedule_size, const sba_view* q,
                   const sba_view* k, const sba_view* v, const sba_view* grad_o, const sba_view* grad_rem,
                   const float* stick_table, float* grad_table, size_t table_size, const sba_view* dq,
                   const sba_view* dk, const sba_view* dv, void* stream) {
  return backward(p, false, schedule, schedule_size, q, k, v, grad_o, grad_rem, stick_table, grad_table, table_size,
                  dq, dk, dv, stream);
}

int sba_attn_bwd(const sba_problem* p, const void* schedule, size_t schedule_size, const sba_view* q,
                 const sba_view* k, const sba_view* v, const sba_view* grad_o, const sba_view* grad_rem,
                 const float* stick_table, float* grad_table, size_t table_size, const sba_view* dq,
                 const sba_view* dk, const sba_view* dv, void* stream) {
  return backward(p, true, schedule, schedule_size, q, k, v, grad_o, grad_rem, stick_table, grad_table, table_size,
                  dq, dk, dv, stream);
}

int sba_varlen_fwd_static(const sba_problem* p, const sba_view* q, const sba_view* k, const sba_view* v,
                          const sba_view* o, const sba_view* rem, void* stream) {
  Sizes sz;
  int e = check_problem(p, false, &sz);
  if (e) return e;
  if (schedule_bytes(sz) > (size_t)SBA_STATIC_SCRATCH_BYTES) return SBA_E_WORKSPACE;
  if ((e = check_arch())) return e;
  void* sched = nullptr;
  if ((e = static_scratch(&sched))) return e;
  // The scheduler rewrites the header and every list entry the kernels will use; nothing of
  // the previous call's contents is read, so nothing needs clearing.
  if ((e = sba_build_schedule(p, sched, SBA_STATIC_SCRATCH_BYTES, stream))) return e;
  return forward(p, false, sched, SBA_STATIC_SCRATCH_BYTES, q, k, v, o, rem, nullptr, 0, nullptr, 0, stream,
                 /*timed=*/false);   // (timing creates events)
}

int sba_launch_geometry(const sba_problem* p, sba_geometry* out) {
  Sizes sz;
  const bool fixed = p != nullptr && (p->flags & SBA_FIXED_LENGTH) != 0;
  int e = check_problem(p, fixed, &sz);
  if (e) return e;
  if (out == nullptr) return SBA_E_NULL;
  const BwdBounds bb = backward_bounds(p, fixed, sz);
  const DkdvGrid g = dkdv_grid(has_dkdv_tail_kernel(p->head_dim), bb.n_long_max, bb.n_tail_max, sz.n_kv_max);
  out->query_list_tiles = sz.n_q_max;
  out->key_list_tiles = sz.n_kv_max;
  out->query_list_word = SCHED_HDR;
  out->key_list_word = SCHED_HDR + TILE_WORDS * sz.n_q_max;
  out->tile_words = TILE_WORDS;
  out->schedule_words = (long long)(schedule_bytes(sz) / sizeof(int));
  out->fwd_tiles = sz.n_q_max;     // forward and dq pass: one workgroup per slot of the query-tile list and head
  out->dq_tiles = sz.n_q_max;
  out->long_tiles_bound = bb.n_long_max;
  out->tail_tiles_bound = bb.n_tail_max;
  out->dkdv_main_tiles = g.main_tiles;
  out->dkdv_tail_tiles = g.tail_tiles;
  return 0;
}

void sba_set_timing(int on) { g_timing.store(on); }
void sba_set_dkdv_workgroups(int n) { g_dkdv_workgroups.store(n); }
float sba_last_kernel_ms(int which) {
  if (which < 0 || which >= 3) return 0.f;
  std::lock_guard<std::mutex> lock(g_ev_mutex);
  const EventPair& ev = g_ev[which];
  float ms = 0.f;
  if (ev.e0 != nullptr && ev.e1 != nullptr && hipEventSynchronize(ev.e1) == hipSuccess &&
      hipEventElapsedTime(&ms, ev.e0, ev.e1) == hipSuccess)
    g_ms[which].store(ms);
  return g_ms[which].load();
}

}  // extern "C"
