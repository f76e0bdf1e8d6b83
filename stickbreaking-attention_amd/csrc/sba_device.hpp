// Device-side building blocks shared by the forward and backward kernels (gfx950 only).
//
// Orientation used everywhere: the score tile is computed TRANSPOSED, S^T = K . Q^T, with the
// 32x32x16 bf16 MFMA.  In the accumulator layout of that instruction a lane owns ONE query
// (column n = lane % 32) and 16 of the 32 rows of the sub-block (rows 8*(i/4) + 4*h + i%4 for
// register i, h = lane / 32); the lane with the other h owns the other 16 rows of the same
// query.  Which key sits in which row is ours to choose (see kperm).  The running sums / products of stick-breaking attention run along the key axis, so
// they become in-register chains plus one exchange between the two half-waves
// (v_permlane32_swap) -- no LDS, no DPP row scans.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// The kernels are written once for a 16-bit element type and compiled twice: for bfloat16 (the
// default) and, with SBA_ELEM_F16 defined, for IEEE half.  Everything that depends on the element
// type lives in an inline namespace named after it, so the two compilations produce distinct
// symbols and one library holds both.
#ifdef SBA_ELEM_F16
#define SBA_ELEM_NS f16
#else
#define SBA_ELEM_NS bf16
#endif

namespace sba {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

constexpr int BM = 128;  // query rows per workgroup tile (4 waves x 32 rows)
constexpr int BN = 64;   // keys per KV tile staged in LDS by the dq pass
constexpr int BKV = 128;  // keys owned by one workgroup of the dk/dv pass
constexpr int BT = 32;   // keys per carry-table entry (one MFMA sub-block)
// The key-tile list has two groups.  The second holds the tiles that few queries follow, for which
// the dk/dv pass has a lighter kernel: every tile of a document of at most TAIL_TILES * BKV tokens,
// and the last tile of every longer document.  The first group holds the rest.
constexpr int TAIL_TILES = 2;
__host__ __device__ inline int kv_tail_tiles(int len) {   // key tiles of a document in the second group
  const int nkv = (len + BKV - 1) / BKV;
  return len <= TAIL_TILES * BKV ? nkv : 1;
}
constexpr int NT = 256;  // threads per workgroup

// Schedule workspace layout (int32 words).
constexpr int SCHED_STATUS = 0;
constexpr int SCHED_NQ = 1;      // number of query tiles
constexpr int SCHED_NKV = 2;     // number of KV tiles
constexpr int SCHED_TABLE = 3;   // carry-table entries per head the documents need (saturates at INT_MAX)
constexpr int SCHED_TOTAL = 4;   // tokens covered by the documents (0 when the input is rejected)
constexpr int SCHED_MAXLEN = 6;  // longest document found (read together with the next word: keep the pair 8-byte aligned)
constexpr int SCHED_NKV_LONG = 7; // key tiles of the first group of the key-tile list (see kv_tail_tiles)
constexpr int SCHED_HDR = 16;    // tile lists start here
constexpr int TILE_WORDS = 8;    // int32 words of one Tile

struct Tile {
  int tok_start;  // first token of the document inside the packed token axis (0 for fixed-length)
  int doc_len;
  int idx;        // tile index inside the document
  int batch;      // batch entry (0 for varlen)
  int tab_base;   // first carry-table entry of the document inside a head's share of the tables
  int rsv[3];
};

// Carry tables (fp32).  Inside a head's share every document owns a triangular area: for each
// 32-key block b the rows 32*b .. Lp-1 (the queries at or below the block; Lp = the length
// rounded up to a multiple of 32), blocks back to back, then one plane of Lp per-row values.
// Entry (b, row) sits at  tab_seg(L, b) + row  from the document's base: consecutive rows are
// consecutive floats and every block's rows start on a 128-byte boundary, so the 32 lanes that
// own 32 consecutive query rows read and write one aligned 128-byte line.
__host__ __device__ inline long long tab_block_off(int L, int b) { return 32ll * b * ((L + 31) >> 5) - 16ll * b * (b - 1); }
__host__ __device__ inline long long tab_seg(int L, int b) { return tab_block_off(L, b) - 32ll * b; }
__host__ __device__ inline long long tab_rowplane(int L) { return tab_block_off(L, (L + 31) >> 5); }
__host__ __device__ inline long long tab_doc_entries(int L) { return tab_rowplane(L) + 32ll * ((L + 31) >> 5); }
// The same offsets inside ONE document's area as 32-bit values (the scheduler refuses inputs whose
// tables exceed 2^31 - 1 entries per head): kernels address  uniform base + 32-bit lane offset.
__device__ __forceinline__ int tab_seg32(int L, int b) { return b * (32 * ((L + 31) >> 5) - 16 * (b + 1)); }
__device__ __forceinline__ int tab_rowplane32(int L) { const int nb = (L + 31) >> 5; return 16 * nb * (nb + 1); }

struct View {
  char* ptr;
  int64_t sb, sh, st;  // element strides
};

// Fills rows [row0, row1) of one head of a [heads, tokens, width] 16-bit tensor (width a multiple of
// 8 elements, rows 16-byte aligned) or of a per-row tensor (width 1) with a repeated 16-bit value.
__device__ inline void fill_rows16(const View& v, int head, int row0, int row1, int width, unsigned pair,
                                   int tid, int nthreads) {
  if (v.ptr == nullptr || row1 <= row0) return;
  unsigned short* base = reinterpret_cast<unsigned short*>(v.ptr) + head * v.sh;
  if (width == 1) {
    for (int r = row0 + tid; r < row1; r += nthreads) base[(int64_t)r * v.st] = (unsigned short)pair;
    return;
  }
  const int c8 = width / 8;
  const uint4 z = make_uint4(pair, pair, pair, pair);
  for (int i = tid; i < (row1 - row0) * c8; i += nthreads) {
    const int r = row0 + i / c8, c = i % c8;
    *reinterpret_cast<uint4*>(base + (int64_t)r * v.st + c * 8) = z;
  }
}

// Upstream leaves the rows of `o`, `dq`, `dk`, `dv` past cu_seqlens[-1] uninitialised (empty_like,
// sb_varlen_fwd.py:418) and relies on zeros_like elsewhere (sb_varlen_bwd.py:507-509).  Here the
// compute kernels write every row of every document exactly once, and the workgroups a launch has
// to spare clear the rest: the grid of a query-tile-owned kernel has one slot per 128 tokens more
// than the documents can use, so slot (tiles + j) takes the j-th block of 128 rows behind the last
// document.  When nothing else runs -- the scheduler rejected cu_seqlens, the carry tables are
// smaller than the documents need, a document is longer than declared -- every slot fills its
// own 128 rows of the token axis with NaN instead, so that the failure cannot pass for a result.
// Returns the rows this workgroup has to fill: [row0, row1), and with what.
__device__ inline void spare_rows(bool refused, int slot, int n_tiles, int total, int tokens, unsigned nan_pair,
                                  int& row0, int& row1, unsigned& pair) {
  row0 = refused ? slot * BM : total + (slot - n_tiles) * BM;
  row1 = min(row0 + BM, tokens);
  pair = refused ? nan_pair : 0u;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains every
// outstanding GLOBAL load (s_waitcnt vmcnt(0)), which would expose the full latency of the
// tile prefetches and table reads that are deliberately kept in flight across the barrier.
// The compiler still waits for each load's result before its first use.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---------------------------------------------------------------------------------------------
// Work queue of a persistent launch.
//
// The hardware deals the workgroups of a grid to the eight XCDs in turn (workgroup b runs on XCD
// b mod 8) and each XCD then works through its share alone.  The XCDs of one part do not run at
// the same speed (measured on the dk/dv pass: 0.875 to 1.0 us per step between the fastest and
// the slowest XCD of one MI355X), so with one workgroup per work item the launch ends when the
// slowest XCD is done with its eighth, the others idle for several percent of the kernel by then.
//
// A persistent launch therefore starts only as many workgroups as fit on the chip at once (`grid`,
// a multiple of 8) over n_items > grid work items numbered as blockIdx used to number them.
// Workgroup b begins with item b.  The remaining items form eight classes, item grid + c + 8 * pos
// being position pos of class c, dealt out through one counter per class (zero when the launch
// begins): a workgroup draws from the class of its own XCD (its items then share K/V or Q/dO rows
// with their neighbours behind that XCD's L2 exactly as before) and, once that class is exhausted,
// from the classes of the other XCDs.  Counters only grow and every draw either yields an item or
// finds its class exhausted, so every workgroup ends after at most n_items + 8 draws.
// ---------------------------------------------------------------------------------------------
constexpr int WORK_WORDS = 64;        // counter words reserved at the end of a table workspace (256 bytes)
constexpr int WORK_DQ = 0;            // first counter of: the forward or the dq pass,
constexpr int WORK_DKDV = 8;          //   the dk/dv pass,
constexpr int WORK_DKDV_TAIL = 16;    //   its kernel for the second group of key tiles
__host__ __device__ inline int work_positions(int n_items, int grid, int c) { return (n_items - grid - c + 7) >> 3; }   // may be <= 0
// One lane draws the next ticket of its class.  The draw goes out when the current item has only its epilogue left
// (a draw made when the item BEGINS would hand the following item to this workgroup however long the current one
// still takes, which is a static assignment in all but name) and is looked at after the epilogue, so its round trip
// is hidden.  Through inline assembly: the compiler would wait for the returned value right behind the instruction.
__device__ __forceinline__ unsigned work_draw(unsigned* ctr_of_class) {
  unsigned ticket, zero = 0u, one = 1u;
  asm volatile("global_atomic_add %0, %1, %2, %3 sc0" : "=&v"(ticket) : "v"(zero), "v"(one), "s"(ctr_of_class) : "memory");
  return ticket;
}
__device__ __forceinline__ void work_wait(unsigned& ticket) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(ticket)::"memory"); }
// The same lane: the item behind ticket `pos` of class `cls`, or the next item any other class still holds, or -1.
__device__ inline int work_next(unsigned* ctr, int cls, unsigned pos, int n_items, int grid) {
  if ((int)pos < work_positions(n_items, grid, cls)) return grid + cls + 8 * (int)pos;
  for (int k = 1; k < 8; ++k) {
    const int c = (cls + k) & 7;
    const int n_pos = work_positions(n_items, grid, c);
    if (n_pos <= 0 || (int)__hip_atomic_load(&ctr[c], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= n_pos) continue;
    const unsigned q = atomicAdd(&ctr[c], 1u);
    if ((int)q < n_pos) return grid + c + 8 * (int)q;
  }
  return -1;
}

inline namespace SBA_ELEM_NS {

#ifdef SBA_ELEM_F16
typedef _Float16 elem_t;
#else
typedef __bf16 elem_t;
#endif
typedef __attribute__((ext_vector_type(8))) elem_t el8;
typedef __attribute__((ext_vector_type(2))) elem_t el2;

__device__ __forceinline__ f32x16 mfma32(el8 a, el8 b, f32x16 c) {
#ifdef SBA_ELEM_F16
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#endif
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Round-to-nearest-even fp32 -> element pairs (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32 on gfx950).
__device__ __forceinline__ el2 cvt2(float a, float b) {
  f32x2 f = {a, b};
  return __builtin_convertvector(f, el2);
}

__device__ __forceinline__ el8 pack8(const float* p) {
  el2 a = cvt2(p[0], p[1]), b = cvt2(p[2], p[3]), c = cvt2(p[4], p[5]), d = cvt2(p[6], p[7]);
  el8 r;
  r[0] = a[0]; r[1] = a[1]; r[2] = b[0]; r[3] = b[1];
  r[4] = c[0]; r[5] = c[1]; r[6] = d[0]; r[7] = d[1];
  return r;
}

__device__ __forceinline__ el8 zero8() {
  el8 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = (elem_t)0.0f;
  return r;
}

// Both half-waves' values of `t`: lo = the value held by lane (n, h=0), hi = by lane (n, h=1).
__device__ __forceinline__ void both_halves(float t, float& lo, float& hi) {
  unsigned u = __builtin_bit_cast(unsigned, t);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  lo = __builtin_bit_cast(float, (unsigned)r[0]);
  hi = __builtin_bit_cast(float, (unsigned)r[1]);
}

// LDS transpose read (ds_read_b64_tr_b16).  Inside each block of 16 lanes, lane r receives,
// for j = 0..3, element (r % 4) of the four 16-bit values addressed by lane (4*j + r/4).
// With lane i pointing at row (base + i/4), column (col0 + 4*(i%4)) of a row-major tile, lane
// r ends up with rows base..base+3 of column col0 + r: four consecutive contraction indices
// for the matrix column that lane owns in an MFMA operand.
__device__ __forceinline__ s16x4 lds_tr4(const unsigned short* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
}

// MFMA operand (8 contraction slots per lane) gathered from a ROW-MAJOR LDS tile whose rows
// are the contraction index.  `p0` / `p1` address rows 0..3 / 4..7 of the lane's 8-row group
// as described for lds_tr4.
__device__ __forceinline__ el8 lds_tr8(const unsigned short* p0, const unsigned short* p1) {
  s16x4 a = lds_tr4(p0), b = lds_tr4(p1);
  s16x8 r = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
  return __builtin_bit_cast(el8, r);
}

__device__ __forceinline__ el8 lds_row8(const unsigned short* p) {
  return *reinterpret_cast<const el8*>(p);
}

// ---------------------------------------------------------------------------------------------
// Key ownership.  Row m of the S^T MFMA is fed with key  kperm(m) = 16*((m>>2)&1) + 4*(m>>3) + (m&3)
// of the sub-block (the lane that supplies A-operand row m simply loads that key), so that in
// the accumulator the lane with half-wave index h owns the 16 CONSECUTIVE keys 16*h + i
// (register i).  Running sums / products along the keys are then one in-register chain plus a
// single exchange between the half-waves.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int kperm(int m) { return ((m & 4) << 2) | ((m >> 3) << 2) | (m & 3); }

// ex[i] <- base * product of r over keys newer than key(i) (exclusive).  Returns base * all.
__device__ __forceinline__ float suffix_prod32_excl(const float (&r)[16], float (&ex)[16], int h,
                                                    float base) {
  const float t = (((r[0] * r[1]) * (r[2] * r[3])) * ((r[4] * r[5]) * (r[6] * r[7]))) *
                  (((r[8] * r[9]) * (r[10] * r[11])) * ((r[12] * r[13]) * (r[14] * r[15])));
  float lo, hi;
  both_halves(t, lo, hi);
  // keys of the h=1 lane (16..31) are newer than those of the h=0 lane
  ex[15] = h == 0 ? base * hi : base;
#pragma unroll
  for (int i = 14; i >= 0; --i) ex[i] = ex[i + 1] * r[i + 1];
  return base * (lo * hi);
}

// v[i] <- base + sum of v over keys >= key(i).  Returns the plain total over the 32 keys.
__device__ __forceinline__ float suffix_sum32(float (&v)[16], int h, float base) {
  const float t = (((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]))) +
                  (((v[8] + v[9]) + (v[10] + v[11])) + ((v[12] + v[13]) + (v[14] + v[15])));
  float lo, hi;
  both_halves(t, lo, hi);
  v[15] += h == 0 ? base + hi : base;
#pragma unroll
  for (int i = 14; i >= 0; --i) v[i] += v[i + 1];
  return lo + hi;
}

// ---------------------------------------------------------------------------------------------
// Stick-breaking weights of one 32-key sub-block for the lane's query.
//
//   x      raw q.k accumulators (S^T layout, register i = key 16*h + i), c = inv_temp * log2(e)
//   k0     document-local index of the sub-block's first key
//   qrow   document-local index of the lane's query
//   carry  stick left after all visible keys NEWER than this sub-block:
//          LOG space: log2 of it (<= 0);  PRODUCT space: the value itself.  Updated in place.
//   p      out: weights A[q, key(i)]
//   beta   out (NEED_BETA): 1 - sigmoid(z) (the fraction of the stick a key leaves), 1 where masked
//   ends   out (PRODUCT space, optional): the stick on entering this lane's newest key and
//          after its oldest key, {ex[15], ex[0] * r[0]}; their difference is the lane's sum of p
//
// Restates compute_block of the upstream Triton kernel
// (stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:26-78): base-2 softplus
// (sb_varlen/softplus.py:34-51), band mask with masked log(1-beta) forced to 0, reverse
// inclusive running sum inside the block plus the carried total, exp2.  The running sum is
// kept in fp32 registers instead of upstream's bf16 triangular matmul.
// ---------------------------------------------------------------------------------------------
template <bool AC, bool PROD, bool BAND, bool NEED_BETA>
__device__ __forceinline__ void stick_weights(const f32x16& x, float c, int k0, int qrow, int h,
                                              float& carry, float (&p)[16], float (&beta)[16],
                                              float* ends = nullptr) {
  // visible keys of a band sub-block: key < qrow (<= with attend_current)  <=>  i < lim
  const int lim = qrow - k0 - 16 * h + (AC ? 1 : 0);
  if constexpr (PROD) {
    // r = 1 - beta.  With ex[i] = stick left after the keys newer than key(i), the stick left
    // after key(i) itself is ex[i] * r[i] = ex[i-1], so the weight is a difference of
    // consecutive chain values: p[i] = ex[i] - ex[i-1].  A masked key has r = 1, which makes
    // its p and beta vanish without further masking.
    float r[16], ex[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float e = fast_exp2(c * x[i]);   // overflow -> inf -> r = 0, beta = 1: still right
      r[i] = fast_rcp(1.0f + e);
      if (BAND && !(i < lim)) r[i] = 1.0f;
    }
    carry = suffix_prod32_excl(r, ex, h, carry);
    const float after = ex[0] * r[0];
    p[0] = ex[0] - after;
#pragma unroll
    for (int i = 1; i < 16; ++i) p[i] = ex[i] - ex[i - 1];
    if (ends != nullptr) { ends[0] = ex[15]; ends[1] = after; }
    if (NEED_BETA) {
#pragma unroll
      for (int i = 0; i < 16; ++i) beta[i] = r[i];
    }
  } else {
    float xs[16], sp[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      // clamping the logit at 126 (log2 units) keeps 2^x finite; sigmoid is 1 - 2^-126 there
      xs[i] = fminf(c * x[i], 126.0f);
      const float t = 1.0f + fast_exp2(xs[i]);
      sp[i] = fast_log2(t);                  // base-2 softplus = -log2(1 - beta)
      if (NEED_BETA) beta[i] = fast_rcp(t);
      if (BAND && !(i < lim)) { sp[i] = 0.0f; if (NEED_BETA) beta[i] = 1.0f; }
    }
    const float total = suffix_sum32(sp, h, -carry);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      p[i] = fast_exp2(xs[i] - sp[i]);
      if (BAND && !(i < lim)) p[i] = 0.0f;
    }
    carry -= total;
  }
}

// ---------------------------------------------------------------------------------------------
// Forward-only form of the product-space weights with a quarter of the reciprocals.
//
// With e = 2^z (the odds of taking the stick) and t = 1 + e, a key divides the stick by t and
// takes the difference: if A is the stick left on a key's older side, the stick on its newer
// side is A t and the key's weight is A t - A = A e -- a product, no cancellation.  For a group of
// four keys only ONE reciprocal is needed: the stick after the group's oldest key is (stick
// before the group) / (t0 t1 t2 t3); from there the group is walked towards its newest key with
// p_j = A_j e_j and A_{j+1} = A_j + p_j.  A transcendental costs about four ordinary
// instructions on this machine, so 16 exp2 + 4 rcp per lane beat 16 exp2 + 16 rcp.
// The backward kernels need r = 1/t for every key and keep the plain form (stick_weights).
//
// Where a product of four t would leave the fp32 range the odds are clamped at 2^30 (beta =
// 1 - 2^-30 there, which in fp32 is 1); a masked key has e = 0: its weight is exactly zero and it
// leaves the stick exactly as it was, so that nothing of a later token reaches the row.
// ---------------------------------------------------------------------------------------------
template <bool BAND, bool CLAMP>
__device__ __forceinline__ float stick_odds(const f32x16& x, float c, int lim, float (&e)[16], float (&inv)[4]) {
  // per group of four keys (register i = key 16*h + i, so a smaller i is an older key):
  // the odds e and inv = 1 / ((1 + e0) (1 + e1) (1 + e2) (1 + e3))
#pragma unroll
  for (int g = 0; g < 4; ++g) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = 4 * g + j;
      const float ej = fast_exp2(CLAMP ? fminf(c * x[i], 30.0f) : c * x[i]);
      e[i] = (BAND && !(i < lim)) ? 0.0f : ej;
    }
    float u = 1.0f + e[4 * g];
    u = fmaf(u, e[4 * g + 1], u);
    u = fmaf(u, e[4 * g + 2], u);
    u = fmaf(u, e[4 * g + 3], u);
    inv[g] = fast_rcp(u);
  }
  return (inv[0] * inv[1]) * (inv[2] * inv[3]);   // what this lane's 16 keys leave of a stick
}

template <bool AC, bool BAND>
__device__ __forceinline__ void stick_weights_fwd(const f32x16& x, float c, int k0, int qrow, int h,
                                                  float& carry, float (&p)[16]) {
  const int lim = qrow - k0 - 16 * h + (AC ? 1 : 0);   // visible keys of a band block: i < lim
  float e[16], inv[4];
  // The clamp is only ever needed when a group's product leaves the fp32 range (its reciprocal is
  // then 0 and the weights a * e would be 0 * inf or plain wrong; an infinite odd next to one that
  // underflowed to 0 even makes the product NaN): that shows as a lane total that is not a
  // positive number, so the odds are first formed without it -- sixteen instructions fewer per
  // block -- and the whole wave repeats them with the clamp in the rare block where some lane's
  // total is 0 or NaN (a stick that really underflows triggers it too: the repeat then merely
  // confirms the 0).
  float total = stick_odds<BAND, false>(x, c, lim, e, inv);
  if (__builtin_amdgcn_ballot_w64(!(total > 0.0f)) != 0) total = stick_odds<BAND, true>(x, c, lim, e, inv);
  float lo, hi;
  both_halves(total, lo, hi);
  // keys of the h=1 lane (16..31) are newer than those of the h=0 lane
  float s = h == 0 ? carry * hi : carry;
  // Newest group first: s becomes the stick on the older side of the group's oldest key.
#pragma unroll
  for (int g = 3; g >= 0; --g) {
    s *= inv[g];
    float a = s;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      p[4 * g + j] = a * e[4 * g + j];
      if (j < 3) a += p[4 * g + j];
    }
  }
  carry *= lo * hi;
}

// ---------------------------------------------------------------------------------------------
// Epilogue: one wave writes its 32 x D block of fp32 accumulators (lane = column n of a 32-wide
// block, register i = row 8*(i/4) + 4*h + i%4) to global memory as bf16.  Storing straight from
// that layout would take 16*D/32 two-byte stores per lane; instead the block goes through a
// wave-private LDS scratch of 32*D elements (2-byte LDS writes, 16-byte reads) and leaves as
// D/16 fully coalesced 16-byte stores per lane.  Wave-private: no workgroup barrier inside,
// but the caller must make sure nobody else still uses the scratch memory.
// ---------------------------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void store_block32(unsigned short* scratch, const f32x16 (&acc)[D / 32], float scale,
                                              elem_t* out, int64_t stride_t, int row0, int limit, int lane) {
  const int n = lane & 31, h = lane >> 5;
  elem_t* sc = reinterpret_cast<elem_t*>(scratch);
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 8 * (i >> 2) + 4 * h + (i & 3);
      sc[row * D + 32 * db + n] = (elem_t)(acc[db][i] * scale);
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own LDS writes have landed
  constexpr int C8 = D / 8;
#pragma unroll
  for (int j = 0; j < 32 * C8 / 64; ++j) {
    const int cidx = lane + 64 * j;
    const int row = cidx / C8, c8 = cidx % C8;
    const uint4 v = *reinterpret_cast<const uint4*>(scratch + row * D + c8 * 8);
    if (row0 + row < limit) *reinterpret_cast<uint4*>(out + (int64_t)(row0 + row) * stride_t + c8 * 8) = v;
  }
}

// Same, with a per-row multiple of another bf16 matrix added on the way out:
//   out[row] = acc[row] * scale + rowscale(row) * addend[row]
// (`rowscale(r)` = the fp32 factor of block row r, 0 <= r < 32, called once per 16-byte chunk).
// The accumulators are rounded to bf16 once in the scratch, the sum is formed in fp32 and
// rounded again: one rounding fewer than a caller adding the two bf16 tensors afterwards.
template <int D, class RowScale>
__device__ __forceinline__ void store_block32_axpy(unsigned short* scratch, const f32x16 (&acc)[D / 32], float scale,
                                                   elem_t* out, int64_t stride_t, int row0, int limit, int lane,
                                                   const elem_t* addend, int64_t addend_stride_t, RowScale rowscale) {
  const int n = lane & 31, h = lane >> 5;
  elem_t* sc = reinterpret_cast<elem_t*>(scratch);
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 8 * (i >> 2) + 4 * h + (i & 3);
      sc[row * D + 32 * db + n] = (elem_t)(acc[db][i] * scale);
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own LDS writes have landed
  constexpr int C8 = D / 8;
#pragma unroll
  for (int j = 0; j < 32 * C8 / 64; ++j) {
    const int cidx = lane + 64 * j;
    const int row = cidx / C8, c8 = cidx % C8;
    const bool ok = row0 + row < limit;
    const float f = rowscale(row);
    const el8 mine = *reinterpret_cast<const el8*>(scratch + row * D + c8 * 8);
    el8 other;
#pragma unroll
    for (int e = 0; e < 8; ++e) other[e] = (elem_t)0.0f;
    if (ok) other = *reinterpret_cast<const el8*>(addend + (int64_t)(row0 + row) * addend_stride_t + c8 * 8);
    float sum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = fmaf(f, (float)other[e], (float)mine[e]);
    if (ok) *reinterpret_cast<el8*>(out + (int64_t)(row0 + row) * stride_t + c8 * 8) = pack8(sum);
  }
}

// Is the 32-key sub-block starting at k0 entirely invisible / entirely visible to the 32
// queries starting at qw0?
template <bool AC>
__device__ __forceinline__ bool sub_skip(int k0, int qw0) {
  return AC ? (k0 > qw0 + 31) : (k0 >= qw0 + 31);
}
template <bool AC>
__device__ __forceinline__ bool sub_full(int k0, int qw0) {
  return AC ? (k0 + 31 <= qw0) : (k0 + 31 < qw0);
}

// ---------------------------------------------------------------------------------------------
// Global -> register tile loads through a buffer resource that covers exactly the rows of one
// (document, head) slice: rows at or past the end of the document fall outside the resource
// and the hardware returns zeros for them, so no branch and no 64-bit address arithmetic.
// ---------------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

struct Rows {
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned row_bytes;   // stride between consecutive tokens, in bytes
};

__device__ __forceinline__ Rows make_rows(const elem_t* base, int64_t stride_t, int n_rows) {
  Rows r;
  const uint64_t bytes = (uint64_t)n_rows * (uint64_t)stride_t * 2u;
  r.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<elem_t*>(base), 0,
                                             bytes > 0xffffffffull ? 0xffffffffu : (unsigned)bytes, 0x00020000);
  r.row_bytes = (unsigned)stride_t * 2u;
  return r;
}

__device__ __forceinline__ uint4 load16(const Rows& r, int row, int col_bytes) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r.rsrc, row * (int)r.row_bytes + col_bytes, 0, 0);
  return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ el8 load_frag(const Rows& r, int row, int col_bytes) {
  return __builtin_bit_cast(el8, load16(r, row, col_bytes));
}

// XOR swizzle of the 16-byte chunks of an UNPADDED row-major tile (row = D*2 bytes) that makes
// both access patterns of a dual-use tile bank-conflict free: row reads (16 consecutive rows,
// one chunk each) and transpose reads (4 consecutive rows, 64 contiguous bytes each).
template <int D>
__device__ __forceinline__ int swz(int row) {
  // (512-byte rows span the banks twice: the chunk's low four bits decide its banks, as with 256-byte rows)
  if constexpr (D >= 128) return ((row & 3) << 2) | ((row >> 2) & 3);
  else if constexpr (D == 64) { const int x = (row >> 1) & 7; return ((x & 1) << 2) | (x >> 1); }
  else return (row >> 2) & 3;   // 64-byte rows: four rows fill the banks, the next four take the next rotation
}

template <int D>
__device__ __forceinline__ int swz_off(int row, int chunk) {   // element offset of a 16-byte chunk
  return row * D + ((chunk ^ swz<D>(row)) << 3);
}

// Asynchronous global -> LDS copy of ROWS x D bf16 of a (document, head) slice into an unpadded,
// swizzled tile, issued by THREADS threads (buffer_load_dwordx4 ... lds).  One wave instruction
// moves 1 KiB: lane l fills the 16-byte LDS chunk number (first chunk of the instruction + l),
// so the swizzle (and the key permutation of key tiles) is applied on the GLOBAL side by
// choosing which chunk a lane fetches; rows past the end of the document arrive as zeros.
// Completion is tracked by vmcnt: wait for it, then barrier, before any wave reads the tile.
//
// Instruction j of wave w covers the tile rows  j * STEP + w * RPI .. + RPI - 1  (RPI = rows per
// instruction, STEP = rows all waves cover together).  STEP is a multiple of 16, which the
// swizzle does not see, and the key permutation turns "+ STEP rows" into a fixed row offset, so
// ONE per-lane byte offset serves every instruction: the rest of the address is scalar.
// One wave instruction of such a copy (buffer_load_dwordx4 ... lds): lane l fetches the 16 bytes at
// byte offset voff + soff of the buffer and the hardware writes them to LDS at dst + 16 * l.
//
// Issued through inline assembly on purpose.  The compiler's wait-count pass knows that the
// builtin form of this instruction writes LDS and, unable to tell one tile slot from another,
// puts `s_waitcnt vmcnt(0)` in front of the next LDS read it cannot prove disjoint -- that is,
// in front of the reads of the CURRENT tile, right after the copy of a LATER tile was issued --
// which makes every tile step wait out a full round trip to memory and turns the prefetch rings
// of the kernels into plain synchronous loads.  Through inline assembly the copy is invisible to
// that pass, and the counted waits the kernels place themselves (wait_loads<N>, then a barrier,
// before any wave reads a slot) are the only ones left.  Those are REQUIRED for correctness:
// nothing else orders an LDS read after the copy that fills its slot.
__device__ __forceinline__ void async_copy16(__amdgpu_buffer_rsrc_t rsrc, const unsigned short* dst, int voff, int soff) {
  const unsigned lds_addr = __builtin_amdgcn_readfirstlane((unsigned)(size_t)dst);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               ::"s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory", "m0");
}

template <int D, int ROWS, int THREADS, bool KEYS>
struct TileCopy {
  static constexpr int C8 = D / 8;
  static constexpr int NCH = ROWS * C8 / THREADS;
  static constexpr int RPI = 64 / C8;                 // rows one wave instruction covers
  static constexpr int STEP = (THREADS / 64) * RPI;   // rows one instruction of every wave covers
  // 512-byte rows with four loading waves: STEP is 8, the swizzle of a row repeats every 16 rows, so the
  // instructions with odd j need a second per-lane offset (the swizzle's bit 1 flipped)
  static constexpr bool TWO_PHASE = STEP == 8;
  static_assert(ROWS * C8 % THREADS == 0, "tile must split evenly over the loading threads");
  static_assert(TWO_PHASE ? (D == 256 && RPI == 2)
                          : (STEP % 16 == 0 && (NCH == 1 || STEP == 16 || STEP % 32 == 0)), "row step must be invisible to the swizzle");
  int voff;       // byte offset of this lane's chunk in instruction 0, relative to the tile's first row
  int voff_odd;   // TWO_PHASE: the same for instructions with odd j (relative to that instruction's first row)
  int wave;

  // source row offset of instruction j relative to instruction 0
  static constexpr int row_delta(int j) {
    // STEP == 8: bits 3 and 4 of the tile row become bits 2 and 3 of the permuted key (see kperm)
    if (TWO_PHASE) return KEYS ? 32 * (j >> 2) + 4 * (j & 3) : j * STEP;
    if (!KEYS || STEP % 32 == 0) return j * STEP;
    // STEP == 16: bit 4 of the tile row becomes bit 3 of the permuted key (see kperm)
    return 32 * (j >> 1) + 8 * (j & 1);
  }

  // gtid = index of the thread inside the group of THREADS loading threads
  __device__ __forceinline__ void init(int gtid, unsigned row_bytes) {
    wave = __builtin_amdgcn_readfirstlane(gtid >> 6);
    const int lane = gtid & 63;
    const int m = wave * RPI + lane / C8, phys = lane % C8;
    const int logical = phys ^ swz<D>(m);
    const int src = KEYS ? ((m & ~31) | kperm(m & 31)) : m;
    voff = src * (int)row_bytes + logical * 16;
    voff_odd = src * (int)row_bytes + (phys ^ swz<D>(m + 8)) * 16;
  }

  // `rows_needed` (uniform): instructions whose rows all lie at or beyond it are skipped; the tile
  // rows they would have filled keep whatever they held.
  __device__ __forceinline__ void issue(const Rows& r, int row0, unsigned short* lds_tile, int rows_needed = ROWS) const {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      if (!KEYS && j * STEP >= rows_needed) continue;
      const int soff = __builtin_amdgcn_readfirstlane((row0 + row_delta(j)) * (int)r.row_bytes);
#ifdef SBA_BUILTIN_DMA
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          r.rsrc, (__attribute__((address_space(3))) void*)(lds_tile + (j * STEP + wave * RPI) * D), 16,
          TWO_PHASE && (j & 1) ? voff_odd : voff, soff, 0, 0);
#else
      async_copy16(r.rsrc, lds_tile + (j * STEP + wave * RPI) * D, TWO_PHASE && (j & 1) ? voff_odd : voff, soff);
#endif
    }
  }
};

// Wait until at most N of this wave's global loads (including asynchronous tile copies) are
// still in flight.
// (s_waitcnt immediate of gfx9: vmcnt in bits 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at
// their maxima = not waited for.)  Emitted through the builtin, not inline assembly, so that the
// compiler's own wait-count bookkeeping sees the wait: after a wait_loads<0>() it knows that none
// of ITS loads is outstanding and places no further vmcnt waits of its own -- which, with the
// asynchronous copies invisible to it, would otherwise wait for copies that were meant to stay in
// flight (a wait for "at most k of my loads" is a wait for "at most k of ALL loads").
template <int N>
__device__ __forceinline__ void wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");
}

}  // inline namespace SBA_ELEM_NS
}  // namespace sba
