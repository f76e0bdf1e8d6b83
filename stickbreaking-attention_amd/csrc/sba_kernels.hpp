// Kernel argument block and launch prototypes shared by the translation units of libsba.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "sba_device.hpp"

namespace sba {

struct KArgs {
  View q, k, v, o, rem;        // forward tensors (rem has no head_dim axis)
  View go, grem, dq, dk, dv;   // backward tensors (grem.ptr may be null)
  const int* sched;            // schedule workspace
  int kv_list_off;             // int32 offset of the KV tile list inside `sched`
  int n_kv_alloc;              // tiles that list has room for (no launch may index it beyond)
  float* stick;                // carry table written by the forward (may be null in fwd): per (row, 32-key block) the
                               // stick left on entering the block; per-row plane: rem in fp32
  float* gtab;                 // gradient prefix table (backward scratch); per-row plane: the full d(rem)
  float* weights;              // forward, debug variant only: dense attention weights
                               // [batch][heads][tokens][tokens] (row = query token, column = key token)
  int heads;
  int tokens;                  // tokens per batch entry
  int fuse;                    // the output is o + rem * v (and grad_o is the gradient of that)
  int clear_spare;             // packed input: spare workgroups clear the rows that belong to no document (or fill
                               // everything with NaN when the launch is refused)
  unsigned nan_pair;           // two NaNs of the 16-bit element type
  int64_t tab_stride;          // carry-table entries per head the caller's tables hold
  int max_doc_len;             // backward: the longest document the caller declared (its grids are sized with it;
                               // the kernels refuse to run when the scheduler found a longer one)
  float c;                     // inv_temp * log2(e)
  float inv_temp;
  unsigned* work;              // work counters of the backward's persistent launch (WORK_WORDS words at the end of the
                               // gradient table; the dq pass clears them), or null: one workgroup per work item
  int n_items;                 // work items of this launch (what the grid would be with one workgroup per item)
  int resident;                // host side: workgroups of a persistent launch (0: never persistent)
  int min_items_each;          // host side: a launch is persistent when it has this many items per workgroup
};

// The argument block read afresh from the kernel-argument segment.  A persistent kernel calls this at
// the top of every work item with a pointer the compiler cannot see through: argument words it
// needs would otherwise be loaded once, ahead of the item loop, and stay in scalar registers across
// the whole loop (the block is 380 bytes; the loop bodies have no such room, and spilled scalar
// registers end up as vector registers spilled to scratch memory).
__device__ __forceinline__ KArgs fresh_args() {
  typedef const __attribute__((address_space(4))) unsigned long long* Words;
  Words w = (Words)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(w));
  static_assert(sizeof(KArgs) % 8 == 0, "copied in 8-byte words");
  union { KArgs a; unsigned long long u[sizeof(KArgs) / 8]; } out;
#pragma unroll
  for (unsigned i = 0; i < sizeof(KArgs) / 8; ++i) out.u[i] = w[i];
  // Pointers rebuilt from integer words are generic pointers to the compiler (64-bit flat addresses in
  // vector registers for every access); say again what it knows of pointers in a kernel's argument
  // list: they point into global memory.
  auto global = [](auto*& p) {
    typedef __attribute__((address_space(1))) char* GlobalBytes;
    p = reinterpret_cast<std::remove_reference_t<decltype(p)>>((char*)(GlobalBytes)(unsigned long long)p);
  };
  KArgs& a = out.a;
  global(a.q.ptr); global(a.k.ptr); global(a.v.ptr); global(a.o.ptr); global(a.rem.ptr);
  global(a.go.ptr); global(a.grem.ptr); global(a.dq.ptr); global(a.dk.ptr); global(a.dv.ptr);
  global(a.sched); global(a.stick); global(a.gtab); global(a.weights); global(a.work);
  return out.a;
}

// Grid of a launch over n_items work items: one workgroup per item, or -- when the caller has work counters and
// there are enough items for every workgroup of a persistent launch -- a.resident workgroups (a multiple of 8).
inline unsigned launch_grid(const KArgs& a, long long n_items) {
  const long long resident = a.resident & ~7;
  const bool persistent = a.work != nullptr && resident >= 8 && n_items > resident &&
                          n_items >= resident * (long long)a.min_items_each;
  return (unsigned)(persistent ? resident : n_items);
}

struct SchedArgs {
  const void* cu;   // null for fixed-length
  int cu_is64;
  int n_docs;       // documents (fixed: batch)
  int tokens;       // T per batch entry
  int n_q_max, n_kv_max;
  int* out;
};

hipError_t launch_schedule(const SchedArgs& a, hipStream_t s);

// Key-tile slots the two kernels of the dk/dv pass are launched over (one workgroup per slot and
// head).  Every workgroup of the main kernel reads the tile descriptor of its slot BEFORE it knows
// how many tiles the list really holds, so the main grid must never exceed the room of the list
// (n_kv_alloc); the tail kernel compares its slot with the true length first.  Head dimensions
// without a tail kernel give both groups of the list to the main kernel.
struct DkdvGrid { int main_tiles, tail_tiles; };
inline DkdvGrid dkdv_grid(bool has_tail_kernel, int n_long_max, int n_last_max, int n_kv_alloc) {
  DkdvGrid g;
  g.main_tiles = has_tail_kernel ? (n_long_max < n_kv_alloc ? n_long_max : n_kv_alloc)
                                 : (n_long_max + n_last_max < n_kv_alloc ? n_long_max + n_last_max : n_kv_alloc);
  g.tail_tiles = has_tail_kernel ? n_last_max : 0;
  return g;
}
inline bool has_dkdv_tail_kernel(int head_dim) { return head_dim <= 64; }

// One set of compute launchers per element type (sba_fwd.hip and sba_bwd.hip are compiled once
// for each, see SBA_ELEM_NS).
#ifdef SBA_ELEM_F16
#define SBA_INLINE_bf16
#define SBA_INLINE_f16 inline
#else
#define SBA_INLINE_bf16 inline
#define SBA_INLINE_f16
#endif
#define SBA_DECLARE_LAUNCHERS(NS)                                                                                \
  SBA_INLINE_##NS namespace NS {                                                                                 \
  hipError_t launch_fwd(const KArgs& a, int head_dim, bool attend_current, bool product, int mode,               \
                        int n_q_max, hipStream_t s);                                                             \
  hipError_t launch_bwd_dq(const KArgs& a, int head_dim, bool attend_current, bool product, int n_q_max,         \
                           hipStream_t s);                                                                       \
  hipError_t launch_bwd_dkdv(const KArgs& a, int head_dim, bool attend_current, bool product, int n_long_max,    \
                             int n_last_max, hipStream_t s);                                                     \
  }
SBA_DECLARE_LAUNCHERS(bf16)
SBA_DECLARE_LAUNCHERS(f16)
#undef SBA_DECLARE_LAUNCHERS

}  // namespace sba
