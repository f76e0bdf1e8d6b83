// Backward kernels.
//
// Upstream computes dq, dk and dv in ONE query-tile-owned kernel and accumulates the dk/dv
// partial tiles of different query tiles through a spin lock in global memory
// (`_backward_one_row` and `locked_add`, stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:
// 297-481 and :12-54).  On MI355X fp32 global atomics sustain about 1.35 TB/s of payload,
// which at 128-row query tiles is several times the whole time budget of the backward, so the
// accumulation is reorganised into two kernels that need no atomics and no locks at all:
//
//   bwd_dq_kernel    query-tile owned (like the forward).  Walks the keys from 0 to the
//                    diagonal, forms dz and accumulates dq in registers.  On the way it
//                    records, per (row, 32-key sub-block), the running prefix
//                    C = sum_{keys before the sub-block} G in `gtab`.
//   bwd_dkdv_kernel  KV-tile owned.  Loops over the query tiles at or below its keys, takes
//                    the stick carry (table written by the forward) and the G prefix (table
//                    written by bwd_dq_kernel) of each sub-block, recomputes p and dz and
//                    accumulates dk and dv in registers; every output element is written once.
//                    (bwd_dkdv_tail_kernel: the same for the key tiles that few queries follow.)
//
// Per-score math (upstream sb_varlen_bwd.py:439-453):
//   G = A * (do.v - drem),  C = inclusive running sum of G over keys,  dz = G - beta * C,
//   dq = s * dz K,  dk = s * dz^T Q,  dv = A^T do.
#include <algorithm>
#include <type_traits>

#include "sba_kernels.hpp"

namespace sba {
inline namespace SBA_ELEM_NS {

// One 32-key sub-block for the 32 queries of a wave, in two phases so that the do.v^T
// accumulators need not be live while the weights are formed:
//   grad_weights  p and r = 1 - beta from the raw scores and the stick carry at the sub-block's newer edge
//   grad_dz       dz = G - beta C with G = p (do.v - drem) and the running prefix C of G
//                 (carry_c: in = prefix before the sub-block, out = after it)
// p and dz leave as bf16 A-operand fragments: slot s of fragment [tt] is key 16*h + 8*tt + s.
template <bool AC, bool PROD>
__device__ __forceinline__ void grad_weights(const f32x16& x, float c, int k0, int qw0, int qrow, int h,
                                             float carry_e, float (&p)[16], float (&bt)[16], float (&ends)[2]) {
  if (sub_full<AC>(k0, qw0)) {
    stick_weights<AC, PROD, false, true>(x, c, k0, qrow, h, carry_e, p, bt, ends);
  } else {
    stick_weights<AC, PROD, true, true>(x, c, k0, qrow, h, carry_e, p, bt, ends);
  }
}

// With G = p (do.v - drem), C the inclusive running sum of G along the keys and r = 1 - beta:
//   dz = G - beta C = r C - (C - G) = r * C[i] - C[i-1],
// so neither G nor beta is formed: the running sum is an fma chain and dz one more fma.  A
// masked key has p = 0 and r = 1, which gives dz = 0 exactly.
//
// In product space the subtraction of drem disappears as well.  With ex[i] the stick left on
// entering key i (so that p[i] = ex[i] - ex[i-1] and r[i] * ex[i] = ex[i-1]) define
// D[i] = C[i] + drem * ex[i].  Then
//   D[i] - D[i-1] = p[i] (do.v - drem) + drem p[i] = p[i] do.v          (one fma, no subtraction)
//   r[i] D[i] - D[i-1] = r[i] C[i] - C[i-1] + drem (r[i] ex[i] - ex[i-1]) = dz[i],
// so the chain runs on do.v directly and starts from C + drem * (stick after the lane's oldest
// key); the lane's total of G is sum(p do.v) - drem * sum(p) with sum(p) = ends[0] - ends[1].
template <bool PROD>
__device__ __forceinline__ void grad_dz(const float (&p)[16], const float (&r)[16], const f32x16& da,
                                        const float (&ends)[2], int h, float& carry_c, float dr,
                                        el8 (&zf)[2]) {
  float dz[16];
  if constexpr (PROD) {
    float t0 = 0.0f, t1 = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) { t0 = fmaf(p[i], da[i], t0); t1 = fmaf(p[i + 1], da[i + 1], t1); }
    const float total = fmaf(-dr, ends[0] - ends[1], t0 + t1);   // this lane's sum of G
    float lo, hi;
    both_halves(total, lo, hi);
    const float cstart = h == 1 ? carry_c + lo : carry_c;        // keys of the h=0 lane come first
    float dprev = fmaf(dr, ends[1], cstart);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float d = fmaf(p[i], da[i], dprev);
      dz[i] = fmaf(r[i], d, -dprev);
      dprev = d;
    }
    carry_c += lo + hi;
  } else {
    float dA[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) dA[i] = da[i] - dr;
    // this lane's total of G (two partial chains), then both half-waves' totals
    float t0 = 0.0f, t1 = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) { t0 = fmaf(p[i], dA[i], t0); t1 = fmaf(p[i + 1], dA[i + 1], t1); }
    float lo, hi;
    both_halves(t0 + t1, lo, hi);
    float cprev = h == 1 ? carry_c + lo : carry_c;   // keys of the h=0 lane come first
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float c = fmaf(p[i], dA[i], cprev);
      dz[i] = fmaf(r[i], c, -cprev);
      cprev = c;
    }
    carry_c += lo + hi;
  }
  zf[0] = pack8(dz);
  zf[1] = pack8(dz + 8);
}

// -------------------------------------------------------------------------------------------
// dq pass
// -------------------------------------------------------------------------------------------
// (head_dim 256: the tiles take 128 KiB, one workgroup per CU, one wave per SIMD with 512 registers)
template <int D, bool AC, bool PROD>
__global__ void __launch_bounds__(NT, D > 128 ? 1 : 2) bwd_dq_kernel(const KArgs a) {
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int TILE = BN * D;   // elements of one K or V tile (unpadded, swizzled)
  // K (row reads for the scores, transpose reads for dq) and V (row reads) tiles,
  // double-buffered, filled by asynchronous global -> LDS copies.
  __shared__ __attribute__((aligned(16))) unsigned short Ks[2 * TILE];
  __shared__ __attribute__((aligned(16))) unsigned short Vs[2 * TILE];
  __shared__ float Cst[NT / 64][32];   // per wave: a table value waiting for the next tile's top

  // Header words and this workgroup's tile are fetched together (the grid never exceeds the
  // allocated list, so the tile read is safe before the count is known): one round trip.
  const int* sched = a.sched;
  const int slot = blockIdx.x / a.heads;
  const int head = blockIdx.x - slot * a.heads;
  const int4 hdr = *reinterpret_cast<const int4*>(sched);   // status, query tiles, key tiles, table entries needed
  const Tile t = reinterpret_cast<const Tile*>(sched + SCHED_HDR)[slot];
  asm volatile("" ::"s"(t.tok_start), "s"(t.doc_len), "s"(t.idx), "s"(t.batch), "s"(t.tab_base));   // keep the tile read above the branch
  const bool refused = hdr.x != 0 || hdr.w > a.tab_stride || sched[SCHED_MAXLEN] > a.max_doc_len;
  // the dk/dv pass that follows on the same stream hands out its work items through these counters
  if (a.work != nullptr && blockIdx.x == 0 && threadIdx.x < WORK_WORDS) a.work[threadIdx.x] = 0u;
  if (refused || slot >= hdr.y) {
    if (a.clear_spare) {     // for the dk/dv pass as well, which has no slots to spare
      int row0, row1;
      unsigned pair;
      spare_rows(refused, slot, hdr.y, sched[SCHED_TOTAL], a.tokens, a.nan_pair, row0, row1, pair);
      fill_rows16(a.dq, head, row0, row1, D, pair, threadIdx.x, NT);
      fill_rows16(a.dk, head, row0, row1, D, pair, threadIdx.x, NT);
      fill_rows16(a.dv, head, row0, row1, D, pair, threadIdx.x, NT);
    }
    return;
  }

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, n = lane & 31, h = lane >> 5;
  const int m0 = t.idx * BM;
  const int qw0 = m0 + 32 * w;
  const int qrow = qw0 + n;
  const bool qvalid = qrow < t.doc_len;

  const int64_t tok0 = t.tok_start;
  const elem_t* qb = reinterpret_cast<const elem_t*>(a.q.ptr) + t.batch * a.q.sb + head * a.q.sh + tok0 * a.q.st;
  const elem_t* kb = reinterpret_cast<const elem_t*>(a.k.ptr) + t.batch * a.k.sb + head * a.k.sh + tok0 * a.k.st;
  const elem_t* vb = reinterpret_cast<const elem_t*>(a.v.ptr) + t.batch * a.v.sb + head * a.v.sh + tok0 * a.v.st;
  const elem_t* gob = reinterpret_cast<const elem_t*>(a.go.ptr) + t.batch * a.go.sb + head * a.go.sh + tok0 * a.go.st;
  elem_t* dqb = reinterpret_cast<elem_t*>(a.dq.ptr) + t.batch * a.dq.sb + head * a.dq.sh + tok0 * a.dq.st;
  const Rows qrows = make_rows(qb, a.q.st, t.doc_len);
  const Rows grows = make_rows(gob, a.go.st, t.doc_len);
  const Rows krows = make_rows(kb, a.k.st, t.doc_len);
  const Rows vrows = make_rows(vb, a.v.st, t.doc_len);

  TileCopy<D, BN, NT, true> kcopy, vcopy;
  kcopy.init(tid, krows.row_bytes);
  vcopy.init(tid, vrows.row_bytes);
  kcopy.issue(krows, 0, Ks);
  vcopy.issue(vrows, 0, Vs);

  el8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    qf[ks] = load_frag(qrows, qrow, 32 * ks + 16 * h);
    dof[ks] = load_frag(grows, qrow, 32 * ks + 16 * h);
  }
  // d(rem) of this lane's row.  When the caller consumed o + rem * v, the gradient arriving for
  // that sum also reaches rem, through the row's own value vector: d(rem) += do . v_row.
  float dr = 0.0f;
  if (a.grem.ptr != nullptr && qvalid) {
    const elem_t* grb = reinterpret_cast<const elem_t*>(a.grem.ptr) + t.batch * a.grem.sb + head * a.grem.sh + tok0 * a.grem.st;
    dr = (float)grb[(int64_t)qrow * a.grem.st];
  }
  if (a.fuse) {
    float dot = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const el8 vown = load_frag(vrows, qrow, 32 * ks + 16 * h);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot = fmaf((float)dof[ks][e], (float)vown[e], dot);
    }
    float lo, hi;
    both_halves(dot, lo, hi);
    dr += lo + hi;
  }

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) dqacc[db][i] = 0.0f;
  float carry_c = 0.0f;

  const int last_key = min(m0 + BM - 1, t.doc_len - 1);
  const int kt_last = last_key / BN;
  // Offsets (elements) inside a tile: row reads of chunk 2*ks + h of LDS row n, and transpose
  // reads of rows 8*u + 4*h + i/4 (+ 32*sb + 16*tt), columns 32*db + 16*blk + 4*(i%4).
  const int i16 = lane & 15, blk = (lane >> 4) & 1;
  int roff[KS], toff[2][DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) roff[ks] = swz_off<D>(n, 2 * ks + h);
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int r = 8 * u + 4 * h + (i16 >> 2);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int col = 32 * db + 16 * blk + 4 * (i16 & 3);
      toff[u][db] = swz_off<D>(r, col >> 3) + (col & 7);
    }
  }
  // the document's area of the two tables (uniform); a lane adds its row and a block's 32-bit offset
  const int64_t tab0 = (int64_t)head * a.tab_stride + t.tab_base;
  const float* stick = a.stick + tab0;
  float* gtab = a.gtab + tab0;
  // the dk/dv pass takes d(rem) from the last plane of the gradient table
  if (qvalid && h == 0) gtab[(unsigned)(tab_rowplane32(t.doc_len) + qrow)] = dr;

  // stick carries of the two sub-blocks of a tile (neutral where the sub-block is skipped)
  auto carries = [&](int kt, float (&ce)[2]) {
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      ce[sb] = PROD ? 1.0f : 0.0f;
      if (qvalid && kt <= kt_last && !sub_skip<AC>(kt * BN + 32 * sb, qw0)) ce[sb] = stick[(unsigned)(tab_seg32(t.doc_len, 2 * kt + sb) + qrow)];
    }
  };
  float ce[2], ce_next[2];
  carries(0, ce);
  int pend_ix = -1;         // table entry of a prefix that is still to be stored (same for the whole wave)

  // One tile step; the buffer index is a compile-time constant so that every LDS address is a
  // fixed register plus an immediate.
  auto tile = [&](auto buf_tag, const int kt) {
    constexpr int buf = decltype(buf_tag)::value;
    // tile kt has landed and every wave is done with the tile before it
    wait_loads<0>();
    lds_barrier();
    // Table stores only ever go out here, at the top of a tile: the vmcnt wait above also waits
    // for the acknowledgement of stores (well over a thousand cycles), so a store issued in the
    // middle of a tile would stall the top of the next one.  The prefix of the second sub-block
    // therefore waits in LDS (no register to spare) until the next tile begins.
    if (pend_ix >= 0) {
      if (qvalid && h == 0) gtab[(unsigned)(pend_ix + qrow)] = Cst[w][n];
      pend_ix = -1;
    }
    // the next tile's carries go out before its tile copy; neither is waited for in this step
    carries(kt + 1, ce_next);
    if (kt < kt_last) {
      kcopy.issue(krows, (kt + 1) * BN, Ks + (buf ^ 1) * TILE);
      vcopy.issue(vrows, (kt + 1) * BN, Vs + (buf ^ 1) * TILE);
    }
    const unsigned short* Kt = Ks + buf * TILE;
    const unsigned short* Vt = Vs + buf * TILE;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const int k0 = kt * BN + 32 * sb;
      if (sub_skip<AC>(k0, qw0)) continue;
      const int tix = tab_seg32(t.doc_len, 2 * kt + sb);   // (uniform)
      if (sb == 0) {
        if (qvalid && h == 0) gtab[(unsigned)(tix + qrow)] = carry_c;
      } else {
        pend_ix = tix;
        if (h == 0) Cst[w][n] = carry_c;
      }
      // LDS latency under load is several hundred cycles, so every group of operand reads is
      // issued one phase before the MFMAs that consume it: V rows before the weights are
      // formed, the transposed K columns before dz is formed.
      float p[16], bt[16], ends[2] = {0.0f, 0.0f};
      el8 vfr[KS];
      {
        f32x16 x;
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = 0.0f;
        el8 kfr[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kfr[ks] = lds_row8(Kt + 32 * sb * D + roff[ks]);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) x = mfma32(kfr[ks], qf[ks], x);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) vfr[ks] = lds_row8(Vt + 32 * sb * D + roff[ks]);
        __builtin_amdgcn_sched_barrier(0);
        grad_weights<AC, PROD>(x, a.c, k0, qw0, qrow, h, ce[sb], p, bt, ends);
      }
      el8 zf[2];
      el8 ktr[2][DB];
      {
        f32x16 da;
#pragma unroll
        for (int i = 0; i < 16; ++i) da[i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) da = mfma32(vfr[ks], dof[ks], da);
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
          const unsigned short* krow = Kt + (32 * sb + 16 * tt) * D;
#pragma unroll
          for (int db = 0; db < DB; ++db) ktr[tt][db] = lds_tr8(krow + toff[0][db], krow + toff[1][db]);
        }
        __builtin_amdgcn_sched_barrier(0);
        grad_dz<PROD>(p, bt, da, ends, h, carry_c, dr, zf);
      }
      // dq += dz . K  (K as the B operand: transpose reads along keys)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int db = 0; db < DB; ++db) dqacc[db] = mfma32(zf[tt], ktr[tt][db], dqacc[db]);
    }
    ce[0] = ce_next[0];
    ce[1] = ce_next[1];
  };
  for (int kt = 0;;) {
    tile(std::integral_constant<int, 0>{}, kt);
    if (++kt > kt_last) break;
    tile(std::integral_constant<int, 1>{}, kt);
    if (++kt > kt_last) break;
  }

  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  if (pend_ix >= 0 && qvalid && h == 0) gtab[(unsigned)(pend_ix + qrow)] = Cst[w][n];
  lds_barrier();   // every wave is done with the K/V tiles: their memory becomes the dq staging area
  store_block32<D>(Ks + w * 32 * D, dqacc, a.inv_temp, dqb, a.dq.st, qw0, t.doc_len, lane);
}

// -------------------------------------------------------------------------------------------
// dk / dv pass.  One workgroup owns 128 keys of one (document, head) and walks the queries that
// can see them, 32 at a time.  Its 8 waves are specialised:
//
//   waves 0-3  "score" waves, one 32-key block each: recompute the 32x32 block of p and dz of
//              step i (K and V fragments live in registers) and stage them in LDS.
//              Software-pipelined: the two MFMA chains (q.k and do.v) of block i+1 are issued
//              while the VALU works on block i.
//   waves 4-7  "product" waves: accumulate dv = p^T dO and dk = dz^T Q of step i-1 from the
//              staged blocks (each owns 64 keys x D of one of the two outputs), and do all the
//              global -> LDS staging of the Q/dO tiles, four steps ahead.
//
// p/dz staging is double-buffered and the Q/dO tiles sit in a ring of eight slots (in step i:
// slot i-1 feeds the products, slot i+1 the score chains, slots i+2..i+4 are in flight), so a
// step needs a single workgroup barrier and a tile has three steps to arrive.
// -------------------------------------------------------------------------------------------
constexpr int NT2 = 512;
// Head dimensions for which the second group of key tiles (a handful of steps each, most of them on or
// near the diagonal) goes to bwd_dkdv_tail_kernel instead.
template <int D> struct TailKernel { static constexpr bool value = D <= 64; };
constexpr int BQ = 32;     // queries per step of the dk/dv pass
constexpr int RING = 6;    // Q/dO tile slots: tiles i-1 (products) .. i+4 (in flight) of step i
constexpr int AHEAD = 4;   // a tile is requested this many steps before the products use it + 1

template <int D, bool AC, bool PROD>
__global__ void __launch_bounds__(NT2, 1) bwd_dkdv_kernel(const KArgs a) {
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int NPT = NT2 / 2;                 // threads of one role
  constexpr int QTILE = BQ * D;     // elements of one Q or dO tile (swizzled, unpadded)
  constexpr int PTILE = BQ * BKV;   // elements of one staged p or dz block [query][key]
  // Q and dO tiles: row reads (score operands) and transpose reads (dk/dv operands).
  __shared__ __attribute__((aligned(16))) unsigned short Qs[RING * QTILE];
  __shared__ __attribute__((aligned(16))) unsigned short Gs[RING * QTILE];
  // p and dz staged [query][key]: 16-byte row writes, transpose reads.
  __shared__ __attribute__((aligned(16))) unsigned short Ps[2 * PTILE];
  __shared__ __attribute__((aligned(16))) unsigned short Zs[2 * PTILE];
  __shared__ int mbox[2][8];        // persistent launch, by item parity: the tile descriptor of the item after the current one
                                    // (five words) and, in word 7, that item (-1: none)

  // A work item is one key tile of one head: item = slot * heads + head, the number blockIdx.x has
  // when the launch takes one workgroup per item.  Header words and the first item's tile are
  // fetched together (the grid never exceeds the allocated list, so the tile read is safe before
  // the count is known): one round trip.
  const int* sched = a.sched;
  const Tile* const kv_list = reinterpret_cast<const Tile*>(sched + a.kv_list_off);
  const int4 hdr = *reinterpret_cast<const int4*>(sched);   // status, query tiles, key tiles, table entries needed
  const Tile t_first = kv_list[blockIdx.x / a.heads];
  asm volatile("" ::"s"(t_first.tok_start), "s"(t_first.doc_len), "s"(t_first.idx), "s"(t_first.batch), "s"(t_first.tab_base));   // keep the tile read above the branch
  // with a kernel of their own for the documents' last key tiles, this one stops where they begin
  const int2 hdr2 = *reinterpret_cast<const int2*>(sched + SCHED_MAXLEN);   // longest document, key tiles of the first group
  const int n_mine = TailKernel<D>::value ? hdr2.y : hdr.z;
  const int n_items = n_mine * a.heads;
  if (hdr.x != 0 || (int)blockIdx.x >= n_items || hdr.w > a.tab_stride || hdr2.x > a.max_doc_len) return;
  // Persistent launch (see work_next): fewer workgroups than items; every workgroup goes on to further
  // items, and the end of one item (last products, conversion and stores of dk / dv by the product waves)
  // overlaps the beginning of the next (tile descriptor, K / V fragments, first Q / dO tiles and table rows,
  // all requested by the score waves, which have nothing else to do by then).
  const bool persistent = a.work != nullptr && (int)gridDim.x < a.n_items;   // (uniform)
  unsigned* const ctr = a.work + WORK_DKDV;
  const int cls = blockIdx.x & 7;

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, n = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, blk = (lane >> 4) & 1;
  // Waves w and w + 4 of a workgroup share a SIMD: every SIMD gets one score wave and one product wave.
  // (Pairing the score waves on two SIMDs and the product waves on the other two was measured: 1.10 against 0.97 ms.)
  const bool scorer = w < 4;
  const int rw = w & 3;                              // index of the wave inside its role
  const int ptid = rw * 64 + lane;                   // index of the thread inside its role

  // What identifies an item (all uniform); each role derives the rest where it needs it.
  struct Item { int tok_start, doc_len, kt, batch, tab_base, head; };
  auto describe = [&](int item, const Tile& t) {
    const int slot = item / a.heads;
    Item it;
    it.tok_start = t.tok_start; it.doc_len = t.doc_len; it.kt = t.idx; it.batch = t.batch; it.tab_base = t.tab_base;
    it.head = item - slot * a.heads;
    return it;
  };
  auto rows_of = [](const View& v, const Item& it) {
    return make_rows(reinterpret_cast<const elem_t*>(v.ptr) + it.batch * v.sb + it.head * v.sh + (int64_t)it.tok_start * v.st,
                     v.st, it.doc_len);
  };
  Item cur = describe(blockIdx.x, t_first);
  // The item after the current one and its tile descriptor, as the first score wave left them in `mbox` (every wave,
  // behind the barrier of the current item's last step).
  auto next_item = [&](int parity, Item& it) {
    if (!persistent) return -1;
    const int nx = __builtin_amdgcn_readfirstlane(mbox[parity][7]);
    if (nx < 0) return -1;
    Tile t;
    t.tok_start = __builtin_amdgcn_readfirstlane(mbox[parity][0]);
    t.doc_len = __builtin_amdgcn_readfirstlane(mbox[parity][1]);
    t.idx = __builtin_amdgcn_readfirstlane(mbox[parity][2]);
    t.batch = __builtin_amdgcn_readfirstlane(mbox[parity][3]);
    t.tab_base = __builtin_amdgcn_readfirstlane(mbox[parity][4]);
    it = describe(nx, t);
    return nx;
  };
  // Both roles copy Q / dO tiles into the ring.  The product waves copy every tile from tile AHEAD on, AHEAD steps
  // ahead of its use, and the first AHEAD tiles of a workgroup's first item; the score waves copy the first AHEAD
  // tiles of every later item, at a time when the product waves are still busy with the item before.
  // (a 32 x 32 tile is one instruction each for two waves: the other two request nothing, wait
  // for nothing and meet the copies at the barrier)
  constexpr int CT = D == 32 ? NPT / 2 : NPT;   // threads of a role that copy tiles
  const bool copier = ptid < CT;                // (uniform per wave)
  using Copy = TileCopy<D, BQ, CT, false>;
  constexpr int LOADS_PER_TILE = 2 * Copy::NCH;

  // The two roles run separate copies of the step loop (same barrier count) so that neither
  // carries the other's registers.
  // A score wave issues about three times as many instructions per step as the product wave it
  // shares a SIMD with and is the critical path of a step, so it gets the issue priority; the
  // product wave fills the slots the score wave leaves (measured: 5 % faster than the reverse).
  if (scorer) {
    __builtin_amdgcn_s_setprio(3);
    const int sb = rw;                          // 32-key block of this wave
    const int qr = n;                           // this lane's query row inside a tile
    el8 kf[KS], vf[KS];                      // MFMA row n holds key k0 + kperm(n)
    // of the current item
    int k0, q_first, nsteps, doc_len, row4, last4;
    float rem_own;
    __amdgpu_buffer_rsrc_t stick_rs, gtab_rs, drem_rs;
    // `request` only issues the loads; nothing consumes (and therefore waits for) a loaded value
    // until `settle`, a whole step or more after the request.
    struct Raw { float e, g, d; };
    auto request = [&](int step, Raw& r) {
      const int off = min(row4 + step * (4 * BQ), last4);
      r.e = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(stick_rs, off, 0, 0));
      r.g = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(gtab_rs, off, 0, 0));
      r.d = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(drem_rs, off, 0, 0));
    };
    auto settle = [&](int step, const Raw& r, float& ce, float& cc, float& d_r) {
      (void)step;
      ce = r.e;
      cc = r.g;
      d_r = r.d;
    };
    // work queue of a persistent launch (see `queue` below)
    unsigned ticket = 0;
    int tile_word = -1;
    const bool keeper = persistent && rw == 0;     // (uniform)
    int queue_from = 0x7fffffff;                   // of the current item: the step of the draw (never, for the other waves)
    int late_tiles = 0;                            // of the current item: tiles this wave copied that may land after its first barrier
    Raw r0, r1, r2;
    // Everything of an item that comes from global memory, requested in one go: the first AHEAD Q / dO
    // tiles, the K and V fragments of this wave's keys and the carries of the first three steps.  For
    // every item but a workgroup's first this happens right after the score waves' last step of the
    // item before, while the product waves finish that one.
    auto open_item = [&](const KArgs& a, const Item& it, bool with_tiles) {
      // (Inside the item loop the argument block is read afresh, see the call, and the lane indices are opaque
      // here: the views and the per-lane address parts would otherwise be formed once, ahead of the item loop,
      // and held in registers all through the steps, which have none to spare.)
      int n = lane & 31, h = lane >> 5;
      asm volatile("" : "+v"(n), "+v"(h));
      doc_len = it.doc_len;
      q_first = it.kt * BKV;                                  // first query that can see the tile
      k0 = q_first + 32 * sb;
      nsteps = (doc_len - q_first + BQ - 1) / BQ;             // >= 1
      // A block that starts past the end of the document is never visible to a query; its table
      // reads are redirected to the document's last block so that they stay inside the document's
      // table area, and their values are never used.  (Rows above a block's first row, read by the
      // first steps of the later blocks, fall into the preceding block's rows: in bounds, unused.)
      const int tblock = min((BKV / 32) * it.kt + sb, (doc_len - 1) / 32);
      const int64_t tab_row0 = (int64_t)it.head * a.tab_stride + it.tab_base;
      const int64_t tab = tab_row0 + tab_seg32(doc_len, tblock);
      const int64_t tab_rowval = tab_row0 + tab_rowplane32(doc_len);   // per-row plane: rem (stick table), d(rem) (gradient table, written by the dq pass)
      // Fused output o + rem * v: its gradient reaches v_j directly as rem_j * do_j.  The queries of
      // step `sb` are this wave's own keys, so that term is dv = P^T dO with rem_j added on the
      // diagonal of P (which is otherwise zero, or p_jj with attend_current), at no extra traffic.
      rem_own = 0.0f;
      if (a.fuse && k0 + n < doc_len) rem_own = a.stick[tab_rowval + k0 + n];
      // Per-row carries of a step.  The three runs of rows this wave reads (its block's rows of the two
      // tables and the per-row plane of the gradient table) are buffer resources, so that a lane
      // addresses them with a 32-bit byte offset: two vector instructions per step instead of 64-bit
      // address arithmetic per load.  The row is clamped into the document; rows past its end then
      // carry the values of its last row, which is harmless: their Q and dO rows are zero (the tile
      // copies fill them with zeros), so whatever finite p and dz they produce adds nothing to dk, dv.
      const unsigned run_bytes = (unsigned)doc_len * 4u;   // (rows of one block: at most doc_len)
      stick_rs = __builtin_amdgcn_make_buffer_rsrc(a.stick + tab, 0, run_bytes, 0x00020000);
      gtab_rs = __builtin_amdgcn_make_buffer_rsrc(a.gtab + tab, 0, run_bytes, 0x00020000);
      drem_rs = __builtin_amdgcn_make_buffer_rsrc(a.gtab + tab_rowval, 0, run_bytes, 0x00020000);
      row4 = 4 * (q_first + qr);
      last4 = 4 * (doc_len - 1);
      // In the order of need: the carries of the first steps (small), tiles 0 and 1 and the fragments (all wanted
      // at the item's first barrier), then the tiles of steps 1 and 2, which only have to arrive one and two steps
      // later (`late_tiles`, see `guard`).
      request(0, r0);
      request(1, r1);
      request(2, r2);
      const Rows qrows = rows_of(a.q, it), grows = rows_of(a.go, it);
      Copy qcopy, gcopy;      // (formed here, once per item: a score wave has no register to keep them in)
      qcopy.init(64 * rw + 32 * h + n, qrows.row_bytes);
      gcopy.init(64 * rw + 32 * h + n, grows.row_bytes);
      auto tiles = [&](int from, int to) {
        if (!(copier && with_tiles)) return;
#pragma unroll
        for (int sft = from; sft < to; ++sft)
          if (sft < nsteps) {
            qcopy.issue(qrows, q_first + sft * BQ, Qs + sft * QTILE);
            gcopy.issue(grows, q_first + sft * BQ, Gs + sft * QTILE);
          }
      };
      tiles(0, 2);
      {
        const Rows krows = rows_of(a.k, it), vrows = rows_of(a.v, it);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          kf[ks] = load_frag(krows, k0 + kperm(n), 32 * ks + 16 * h);
          vf[ks] = load_frag(vrows, k0 + kperm(n), 32 * ks + 16 * h);
        }
      }
      tiles(2, AHEAD);
      late_tiles = with_tiles ? max(min(AHEAD, nsteps) - 2, 0) : 0;
      if (keeper) queue_from = max(nsteps - 5, 0);
    };
    // The row-read offsets of this lane inside a tile (chunk 2*ks + h of row qr).
    int roff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) roff[ks] = swz_off<D>(qr, 2 * ks + h);
    auto chains = [&](int slot8, f32x16& x, f32x16& da) {
      const unsigned short* Qt = Qs + slot8 * QTILE;
      const unsigned short* Gt = Gs + slot8 * QTILE;
#pragma unroll
      for (int j = 0; j < 16; ++j) { x[j] = 0.0f; da[j] = 0.0f; }
      // all operand reads first, so the chains are not paced by LDS latency
      el8 qfr[KS], gfr[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) { qfr[ks] = lds_row8(Qt + roff[ks]); gfr[ks] = lds_row8(Gt + roff[ks]); }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        x = mfma32(kf[ks], qfr[ks], x);
        da = mfma32(vf[ks], gfr[ks], da);
      }
    };
    // Ahead of the barrier that ends step 0 (step 1) of an item whose first tiles this wave copied: its part of
    // tile 2 (tile 3), read behind that barrier, has landed.  What was requested after it -- tile 3 and the
    // carries of step 3, or the carries of steps 3 and 4 -- may stay in flight (loads return in the order issued).
    static_assert(AHEAD == 4, "the late tiles are tiles 2 and 3");
    auto guard = [&](int i) {
      if (late_tiles == 0 || i > 1) return;
      if (i == 0) {
        if (late_tiles == 2) wait_loads<LOADS_PER_TILE + 3>();
        else wait_loads<3>();
      } else if (late_tiles == 2) {
        wait_loads<6>();
      }
    };
    auto stage = [&](int parity, const el8 (&pf)[2], const el8 (&zf)[2]) {
      // p and dz as [query][key]: fragment tt is 8 consecutive keys = one 16-byte chunk
      unsigned short* Pt = Ps + parity * PTILE;
      unsigned short* Zt = Zs + parity * PTILE;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const int chunk = 4 * sb + 2 * h + tt;
        *reinterpret_cast<el8*>(Pt + swz_off<BKV>(qr, chunk)) = pf[tt];
        *reinterpret_cast<el8*>(Zt + swz_off<BKV>(qr, chunk)) = zf[tt];
      }
    };

    // Carries are requested three steps before the step that uses them, into three register sets
    // used in turn (a table read takes longer than one step), and settled when that step begins.
    float carry_e, carry_c, dr;
    // One step: (xc, dc) hold the finished chains of block i; the chains of block i+1 go into
    // (xn, dn).  Called with the two accumulator pairs swapped on alternate steps, so nothing
    // is copied between steps.  DIAG = one of the first steps, whose queries may sit on or
    // above this wave's keys (masks, possible skip); every later step is one straight-line
    // block in which the MFMA chains of block i+1 are interleaved with the VALU work on block i.
    auto step = [&](auto diag_tag, int i, f32x16& xc, f32x16& dc, f32x16& xn, f32x16& dn, Raw& set) {
      constexpr bool DIAG = decltype(diag_tag)::value;
      settle(i, set, carry_e, carry_c, dr);   // requested three steps ago
      request(i + 3, set);
      chains((i + 1) % RING, xn, dn);
      el8 pf[2], zf[2];
      const int qw0 = q_first + i * BQ;
      const int qrow = qw0 + n;
      if (DIAG && sub_skip<AC>(k0, qw0)) {
        pf[0] = zero8(); pf[1] = zero8(); zf[0] = zero8(); zf[1] = zero8();
      } else {
        float p[16], bt[16], ends[2] = {0.0f, 0.0f};
        if (DIAG) grad_weights<AC, PROD>(xc, a.c, k0, qw0, qrow, h, carry_e, p, bt, ends);
        else stick_weights<AC, PROD, false, true>(xc, a.c, k0, qrow, h, carry_e, p, bt, ends);
        pf[0] = pack8(p);
        pf[1] = pack8(p + 8);
        if (DIAG && a.fuse && qw0 == k0) {
          float pd[16];
#pragma unroll
          for (int j = 0; j < 16; ++j) pd[j] = p[j] + (16 * h + j == n ? rem_own : 0.0f);
          pf[0] = pack8(pd);
          pf[1] = pack8(pd + 8);
        }
        grad_dz<PROD>(p, bt, dc, ends, h, carry_c, dr, zf);
      }
      stage(i & 1, pf, zf);
      if constexpr (DIAG) guard(i);
      lds_barrier();
    };
    // The same step for the product-space carry away from the diagonal, hand-pipelined: the
    // VALU work on block i is cut into 8 chunks and the 2*KS chain MFMAs of block i+1 are
    // issued between them (operand reads two chunks ahead), each position pinned with a
    // scheduling barrier so that the matrix core runs underneath the VALU stream.
    // SLOT >= 0: the ring slot of tile i+1 (and with it the p/dz buffer, SLOT and i have opposite
    // parity) is a compile-time constant, so every LDS address is a fixed register plus an
    // immediate; SLOT < 0: taken from i at run time.
    // BAND: one of the first steps, whose queries may sit on or above this wave's keys: a key the query must not
    // see gets r = 1, which makes its p and its dz exactly zero and leaves the stick as it was.
    auto bulk = [&](auto band_tag, auto slot_tag, int i, f32x16& xc, f32x16& dc, f32x16& xn, f32x16& dn, Raw& set) {
      constexpr bool BAND = decltype(band_tag)::value;
      constexpr int SLOT = decltype(slot_tag)::value;
      constexpr int NCHUNK = 8, PER = 2 * KS / NCHUNK;
      settle(i, set, carry_e, carry_c, dr);   // requested three steps ago
      request(i + 3, set);
      const int slot8 = SLOT >= 0 ? SLOT : ((i + 1) % RING);
      const int parity = SLOT >= 0 ? ((SLOT + 1) & 1) : (i & 1);
      const unsigned short* Qt = Qs + slot8 * QTILE;
      const unsigned short* Gt = Gs + slot8 * QTILE;
#pragma unroll
      for (int j = 0; j < 16; ++j) { xn[j] = 0.0f; dn[j] = 0.0f; }
      // Operand reads run LEAD chunks ahead of the MFMAs that consume them (LDS latency under
      // load is longer than one chunk of VALU work), through a small rotating set of registers.
      constexpr int LEAD = 2;
      el8 fr[LEAD + 1][PER];
      auto pre = [&](int c) {
        if (c >= NCHUNK) return;
#pragma unroll
        for (int m = 0; m < PER; ++m) {
          const int k = c * PER + m;   // even: q.k chain step k/2, odd: do.v chain step k/2
          fr[c % (LEAD + 1)][m] = lds_row8(((k & 1) ? Gt : Qt) + roff[k >> 1]);
        }
      };
      auto post = [&](int c) {
#pragma unroll
        for (int m = 0; m < PER; ++m) {
          const int k = c * PER + m;
          if (k & 1) dn = mfma32(vf[k >> 1], fr[c % (LEAD + 1)][m], dn);
          else xn = mfma32(kf[k >> 1], fr[c % (LEAD + 1)][m], xn);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      // The step opens with vector work only: right after the barrier the product waves fetch the
      // p / dz fragments this wave's neighbours just staged, and they are the ones the next barrier
      // waits for -- the score waves' own operand reads join one chunk later.
      float r[16], ex[16], p[16];
      const int qw0 = q_first + i * BQ;
      const int lim = qw0 + n - k0 - 16 * h + (AC ? 1 : 0);   // (BAND) visible keys of this lane: j < lim
      // chunks 0, 1: r = 1 - beta of the 16 keys
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        r[j] = fast_rcp(1.0f + fast_exp2(a.c * xc[j]));
        if (BAND && !(j < lim)) r[j] = 1.0f;
      }
      __builtin_amdgcn_sched_barrier(0);
      pre(0);
      pre(1);
#pragma unroll
      for (int j = 8; j < 16; ++j) {
        r[j] = fast_rcp(1.0f + fast_exp2(a.c * xc[j]));
        if (BAND && !(j < lim)) r[j] = 1.0f;
      }
      __builtin_amdgcn_sched_barrier(0);
      // chunk 2: stick left after the newer keys
      pre(2);
      carry_e = suffix_prod32_excl(r, ex, h, carry_e);
      post(0);
      // chunk 3: weights and their bf16 fragments
      pre(3);
      const float after = ex[0] * r[0];       // stick left after this lane's oldest key
      p[0] = ex[0] - after;
#pragma unroll
      for (int j = 1; j < 16; ++j) p[j] = ex[j] - ex[j - 1];
      el8 pf[2], zf[2];
      if (BAND && a.fuse && qw0 == k0) {      // (see rem_own)
        float pd[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) pd[j] = p[j] + (16 * h + j == n ? rem_own : 0.0f);
        pf[0] = pack8(pd);
        pf[1] = pack8(pd + 8);
      } else {
        pf[0] = pack8(p);
        pf[1] = pack8(p + 8);
      }
      post(1);
      // chunk 4: this lane's total of G = sum(p do.v) - drem sum(p), sum(p) = ex[15] - after
      pre(4);
      float t0 = 0.0f, t1 = 0.0f;
#pragma unroll
      for (int j = 0; j < 16; j += 2) { t0 = fmaf(p[j], dc[j], t0); t1 = fmaf(p[j + 1], dc[j + 1], t1); }
      float lo, hi;
      both_halves(fmaf(-dr, ex[15] - after, t0 + t1), lo, hi);
      // chunks 5, 6: D = C + drem * stick runs on do.v directly (see grad_dz); dz = r D[i] - D[i-1]
      float dprev = fmaf(dr, after, h == 1 ? carry_c + lo : carry_c);
      post(2);
      float dz[16];
      pre(5);
#pragma unroll
      for (int j = 0; j < 8; ++j) { const float dj = fmaf(p[j], dc[j], dprev); dz[j] = fmaf(r[j], dj, -dprev); dprev = dj; }
      post(3);
      pre(6);
#pragma unroll
      for (int j = 8; j < 16; ++j) { const float dj = fmaf(p[j], dc[j], dprev); dz[j] = fmaf(r[j], dj, -dprev); dprev = dj; }
      post(4);
      // chunk 7: dz fragments and staging
      pre(7);
      zf[0] = pack8(dz);
      zf[1] = pack8(dz + 8);
      stage(parity, pf, zf);
      post(5);
      post(6);
      post(7);
      if constexpr (BAND) guard(i);
      lds_barrier();
    };
    auto later = [&](auto slot_tag, int i, f32x16& xc, f32x16& dc, f32x16& xn, f32x16& dn, Raw& set) {
      if constexpr (PROD && D >= 64) bulk(std::false_type{}, slot_tag, i, xc, dc, xn, dn, set);   // (its eight chunks need 2 * KS >= 8 chain steps)
      else step(std::false_type{}, i, xc, dc, xn, dn, set);
    };
    auto first = [&](int i, f32x16& xc, f32x16& dc, f32x16& xn, f32x16& dn, Raw& set) {
      if constexpr (PROD && D >= 64) {
        // (A block none of whose keys the step's queries may see goes the plain way, which stages zeros without
        // looking at the carries: the table rows such a step reads are rows of other blocks or rows that nobody
        // ever wrote, and whatever they hold -- a NaN, say -- must not get anywhere.)
        if (sub_skip<AC>(k0, q_first + i * BQ)) {
          settle(i, set, carry_e, carry_c, dr);
          request(i + 3, set);
          chains((i + 1) % RING, xn, dn);
          const el8 zero[2] = {zero8(), zero8()};
          stage(i & 1, zero, zero);
          guard(i);
          lds_barrier();
        } else {
          bulk(std::true_type{}, std::integral_constant<int, -1>{}, i, xc, dc, xn, dn, set);
        }
      } else {
        step(std::true_type{}, i, xc, dc, xn, dn, set);
      }
    };
    // Work queue of a persistent launch, kept by the first score wave ahead of the steps: the draw goes out five
    // steps before the item ends; two steps before the end its answer is taken and the tile descriptor of the
    // next item requested (one word per lane); ahead of the last step both go into `mbox`, where every wave finds
    // them behind that step's barrier -- no wave ever waits for the queue or for the descriptor.  A score wave's
    // only other global loads in a step are the three of `request`, and loads return in the order issued: "at
    // most 3 * (steps since the draw) outstanding" says that the draw has returned.
    auto queue = [&](int i, int parity) {
      if (i < queue_from) return;                  // (all a step away from the item's end pays for the queue: one comparison)
      const int drawn = queue_from, resolved = max(nsteps - 2, 0);
      if (i == drawn && lane == 0) ticket = work_draw(ctr + cls);
      if (i == resolved) {
        const int since = resolved - drawn;
        if (since >= 3) wait_loads<9>();
        else if (since == 2) wait_loads<6>();
        else if (since == 1) wait_loads<3>();
        else wait_loads<0>();
        int nx = -1;
        if (lane == 0) {
          work_wait(ticket);     // (nothing left to wait for: ties the value to the waits above)
          nx = work_next(ctr, cls, ticket, n_items, gridDim.x);
        }
        nx = __builtin_amdgcn_readfirstlane(nx);
        tile_word = nx;
        if (nx >= 0 && lane < 7) tile_word = reinterpret_cast<const int*>(kv_list + nx / a.heads)[lane];
      }
      if (i == nsteps - 1 && lane < 8) mbox[parity][lane] = tile_word;
    };
    open_item(a, cur, false);     // (a workgroup's first item: the product waves, idle so far, copy its first tiles)
#pragma unroll 1
    for (int m = 0;; ++m) {
      // the carries, tiles 0 and 1 and the fragments have arrived (not necessarily the late tiles, requested last)
      if (late_tiles == 2) wait_loads<2 * LOADS_PER_TILE>();
      else if (late_tiles == 1) wait_loads<LOADS_PER_TILE>();
      else wait_loads<0>();
      lds_barrier();                        // every score wave's part of tiles 0 .. AHEAD-1 is in slots 0 .. AHEAD-1
      f32x16 xa, da, xb, db;
      chains(0, xa, da);
      // the first BKV/BQ = 4 steps can touch the diagonal of some wave's block
      queue(0, m & 1);
      first(0, xa, da, xb, db, r0);
      if (nsteps > 1) { queue(1, m & 1); first(1, xb, db, xa, da, r1); }
      if (nsteps > 2) { queue(2, m & 1); first(2, xa, da, xb, db, r2); }
      if (nsteps > 3) { queue(3, m & 1); first(3, xb, db, xa, da, r0); }
      // Whole turns of the ring with static slots (the ring, the two staging buffers, the two
      // accumulator pairs and the three carry sets all repeat with period six: at i = 4 + 6m tile
      // i+1 sits in slot 5 and the carries in set 1), then the remaining steps with run-time slots.
      using std::integral_constant;
      int i = BKV / BQ;
      // (the queue's business all falls into an item's last five steps: the turns before them run without it, as one
      // straight-line block)
      const int spare = persistent ? 5 : 0;
#pragma unroll 1
      for (; i + RING + spare <= nsteps; i += RING) {
        later(integral_constant<int, 5>{}, i, xa, da, xb, db, r1);
        later(integral_constant<int, 0>{}, i + 1, xb, db, xa, da, r2);
        later(integral_constant<int, 1>{}, i + 2, xa, da, xb, db, r0);
        later(integral_constant<int, 2>{}, i + 3, xb, db, xa, da, r1);
        later(integral_constant<int, 3>{}, i + 4, xa, da, xb, db, r2);
        later(integral_constant<int, 4>{}, i + 5, xb, db, xa, da, r0);
      }
      // The item's last steps (five to ten after long runs), with the queue's business between them and ring slots
      // taken from i at run time: one copy of the step per place in the period of six, walked until the steps run out.
      // (i = 4 + 6m here: accumulator pair a and carry set 1 are next)
#pragma unroll 1
      for (;; i += RING) {
        if (i >= nsteps) break;
        queue(i, m & 1);     later(integral_constant<int, -1>{}, i, xa, da, xb, db, r1);
        if (i + 1 >= nsteps) break;
        queue(i + 1, m & 1); later(integral_constant<int, -1>{}, i + 1, xb, db, xa, da, r2);
        if (i + 2 >= nsteps) break;
        queue(i + 2, m & 1); later(integral_constant<int, -1>{}, i + 2, xa, da, xb, db, r0);
        if (i + 3 >= nsteps) break;
        queue(i + 3, m & 1); later(integral_constant<int, -1>{}, i + 3, xb, db, xa, da, r1);
        if (i + 4 >= nsteps) break;
        queue(i + 4, m & 1); later(integral_constant<int, -1>{}, i + 4, xa, da, xb, db, r2);
        if (i + 5 >= nsteps) break;
        queue(i + 5, m & 1); later(integral_constant<int, -1>{}, i + 5, xb, db, xa, da, r0);
      }
      // This wave is done with the item's tiles and with its K / V fragments: the next item's global
      // reads go out now, while the product waves form the last products and convert and store dk / dv.
      const int next = next_item(m & 1, cur);
      if (next < 0) break;
      open_item(fresh_args(), cur, true);
    }
  } else {
    __builtin_amdgcn_s_setprio(0);
    const int mat = (rw >> 1) & 1, half = rw & 1;   // (dv | dk) x 64 keys (two 32-key blocks); all D columns
    f32x16 acc[2][DB];
#pragma unroll
    for (int kb2 = 0; kb2 < 2; ++kb2)
#pragma unroll
      for (int j = 0; j < DB; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[kb2][j][i] = 0.0f;
    // Transpose-read offsets (elements).  Rows are queries 16*ks + 8*h + 4*u + i/4; the swizzle
    // depends on the row modulo 16 only, so one offset serves every ks.
    int xoff[2][2], yoff[2][DB];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int r = 8 * h + 4 * u + (i16 >> 2);
#pragma unroll
      for (int kb2 = 0; kb2 < 2; ++kb2) {
        const int xc = 64 * half + 32 * kb2 + 16 * blk + 4 * (i16 & 3);   // key column (elements)
        xoff[u][kb2] = swz_off<BKV>(r, xc >> 3) + (xc & 7);
      }
#pragma unroll
      for (int j = 0; j < DB; ++j) {
        const int yc = 32 * j + 16 * blk + 4 * (i16 & 3);           // d column (elements)
        yoff[u][j] = swz_off<D>(r, yc >> 3) + (yc & 7);
      }
    }
    Copy qcopy, gcopy;
    qcopy.init(ptid, (unsigned)a.q.st * 2u);
    gcopy.init(ptid, (unsigned)a.go.st * 2u);
    // of the current item
    Rows qrows = rows_of(a.q, cur), grows = rows_of(a.go, cur);
    int q_first = cur.kt * BKV;
    int nsteps = (cur.doc_len - q_first + BQ - 1) / BQ;
    auto fetch = [&](int step) {
      if (!copier) return;
      qcopy.issue(qrows, q_first + step * BQ, Qs + (step % RING) * QTILE);
      gcopy.issue(grows, q_first + step * BQ, Gs + (step % RING) * QTILE);
    };
    // The LDS is the busiest unit of this kernel (every step moves about 140 KB through it), and
    // a product wave that fetched all its operands after the barrier would spend half the step
    // issuing reads.  Only the staged p / dz fragments have to wait for the barrier: the Q / dO
    // fragments of a step come from a tile that landed long before, so they are read one
    // iteration ahead, between the MFMAs of the previous step.
    auto read_y = [&](int step, el8 (&bf)[2][DB], int ks) {
      const unsigned short* Yt = (mat ? Qs : Gs) + (step % RING) * QTILE;
#pragma unroll
      for (int j = 0; j < DB; ++j) bf[ks][j] = lds_tr8(Yt + yoff[0][j] + 16 * ks * D, Yt + yoff[1][j] + 16 * ks * D);
    };
    auto finish = [&](int i) {
      // Tile i+2 (read by the score waves in step i+1) has landed before anyone passes the
      // barrier: only the tiles requested after it may still be in flight (loads return in order).
      // The first AHEAD tiles are the score waves' (landed before the item's first barrier), and the
      // item's last two barriers guard no tile.
      if (i + 2 >= AHEAD && i + 2 < nsteps) {
        const int after = min(i + AHEAD, nsteps - 1) - (i + 2);
        if (after >= 2) wait_loads<2 * LOADS_PER_TILE>();
        else if (after == 1) wait_loads<LOADS_PER_TILE>();
        else wait_loads<0>();
      }
      lds_barrier();
    };
    // iteration i >= 1: products of step i - 1 with the Q / dO fragments in `cur`; the fragments of
    // step i go into `nxt` (past the last step they come from an idle ring slot and are never used)
    auto iter = [&](int i, el8 (&cur)[2][DB], el8 (&nxt)[2][DB]) {
      if (i + AHEAD < nsteps) fetch(i + AHEAD);
      // acc[key, d] += sum over the 32 queries of step i-1 of X[query][key] * Y[query][d]
      const unsigned short* Xt = (mat ? Zs : Ps) + ((i - 1) & 1) * PTILE;
      el8 af[2][2];
#pragma unroll
      for (int ks = 0; ks < BQ / 16; ++ks)
#pragma unroll
        for (int kb2 = 0; kb2 < 2; ++kb2)
          af[ks][kb2] = lds_tr8(Xt + xoff[0][kb2] + 16 * ks * BKV, Xt + xoff[1][kb2] + 16 * ks * BKV);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < BQ / 16; ++ks) {
#pragma unroll
        for (int kb2 = 0; kb2 < 2; ++kb2)
#pragma unroll
          for (int j = 0; j < DB; ++j) acc[kb2][j] = mfma32(af[ks][kb2], cur[ks][j], acc[kb2][j]);
        read_y(i, nxt, ks);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (i < nsteps) finish(i);     // (nothing follows the item's last products that another wave could disturb)
    };
#pragma unroll
    for (int sft = 0; sft < AHEAD; ++sft)
      if (sft < nsteps) fetch(sft);          // (of the workgroup's first item; the score waves copy these tiles of every later one)
    wait_loads<0>();
#pragma unroll 1
    for (int m = 0;; ++m) {
      lds_barrier();                        // the item's first barrier: tiles 0 .. AHEAD-1 are in the ring
      el8 ya[2][DB], yb[2][DB];
      if (AHEAD < nsteps) fetch(AHEAD);
      read_y(0, ya, 0);
      read_y(0, ya, 1);
      finish(0);
#pragma unroll 1
      for (int i = 1; i <= nsteps; i += 2) {
        iter(i, ya, yb);
        if (i + 1 <= nsteps) iter(i + 1, yb, ya);
      }
      // dk / dv leave through ring slots 4 and 5, which nothing uses between the barrier of the item's last
      // score step and the next item's first barrier (the score waves are filling slots 0 .. AHEAD-1 with the
      // next item's first tiles by now; the staging buffers may still be feeding another product wave's last
      // products).  This wave reaches that barrier only after the stores below.
      static_assert(AHEAD + 2 <= RING, "two ring slots free for the output staging");
      Item nxt = cur;
      const int next = next_item(m & 1, nxt);
      const KArgs a = fresh_args();          // (see open_item)
      int lane_e = lane;
      asm volatile("" : "+v"(lane_e));
      const View& ov = mat ? a.dk : a.dv;
      elem_t* outb = reinterpret_cast<elem_t*>(ov.ptr) + cur.batch * ov.sb + cur.head * ov.sh + (int64_t)cur.tok_start * ov.st;
      unsigned short* scratch = (rw & 2 ? Gs : Qs) + (AHEAD + (rw & 1)) * QTILE;
#pragma unroll
      for (int kb2 = 0; kb2 < 2; ++kb2) {
        store_block32<D>(scratch, acc[kb2], mat ? a.inv_temp : 1.0f, outb, ov.st, cur.kt * BKV + 64 * half + 32 * kb2,
                         cur.doc_len, lane_e);
#pragma unroll
        for (int j = 0; j < DB; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[kb2][j][e] = 0.0f;
      }
      if (next < 0) break;
      cur = nxt;
      qrows = rows_of(a.q, cur);
      grows = rows_of(a.go, cur);
      q_first = cur.kt * BKV;
      nsteps = (cur.doc_len - q_first + BQ - 1) / BQ;
    }
  }
}

// -------------------------------------------------------------------------------------------
// dk / dv of the second group of key tiles (kv_tail_tiles): at most TAIL_TILES * BKV queries see such a
// tile.  For packed short documents that is the whole dk/dv pass, and the eight-wave pipeline
// above spends nearly all of such a tile on its prologue, its barriers and its epilogue with one
// workgroup per CU.  Here a workgroup is four independent waves: wave w owns the 32 keys of block
// w, recomputes p and dz of the query blocks at or after it exactly as a score wave does, turns
// its own 32x32 blocks around through a private piece of LDS and accumulates its own rows of dk
// and dv.  One barrier (after the Q / dO rows have landed), two workgroups per CU.
//
// STREAM: the same four independent waves on EVERY key tile, whatever number of queries follows
// it: the Q / dO rows then come 64 at a time through two LDS buffers, with one barrier per 64
// rows (one per 32 rows costs a quarter more time: the waves wait for one another at each).
// This is the whole dk/dv pass of head_dim 256, where a wave's K and V fragments (128 registers)
// and the accumulators of ONE of dk and dv (128) with the chains' own temporaries need the
// register file of a SIMD to themselves: one workgroup per CU, one wave per SIMD, nothing to
// split into roles, and two passes over the queries, dv first and dk second (both outputs'
// accumulators at once leave the chains no accumulation registers: 150 to 210 spilled values,
// whether or not the V fragments wait in LDS instead).
// -------------------------------------------------------------------------------------------
template <int D> struct StreamKernel { static constexpr bool value = D > 128; };

template <int D, bool AC, bool PROD, bool STREAM>
__global__ void __launch_bounds__(NT, D > 128 ? 1 : 2) bwd_dkdv_tail_kernel(const KArgs a) {
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int SEG = 64;                             // STREAM: query rows per buffer
  constexpr int QROWS = STREAM ? 2 * SEG : TAIL_TILES * BKV;   // rows the buffers hold (not STREAM: every query that can follow the tile's first key)
  __shared__ __attribute__((aligned(16))) unsigned short Qs[QROWS * D];   // Q rows from the tile's first key on (swizzled like every tile)
  __shared__ __attribute__((aligned(16))) unsigned short Gs[QROWS * D];   // dO rows
  __shared__ __attribute__((aligned(16))) unsigned short St[NT / 64][2][32 * 32];   // per wave: p and dz of one block, [query][key]

  const int* sched = a.sched;
  const int4 hdr = *reinterpret_cast<const int4*>(sched);   // status, query tiles, key tiles, table entries needed
  const int2 hdr2 = *reinterpret_cast<const int2*>(sched + SCHED_MAXLEN);   // longest document, key tiles of the first group
  if (hdr.x != 0 || hdr.w > a.tab_stride || hdr2.x > a.max_doc_len) return;
  const int which = blockIdx.x / a.heads;
  const int head = blockIdx.x - which * a.heads;
  const int slot = STREAM ? which : hdr2.y + which;   // STREAM: both groups of the list
  if (slot >= hdr.z) return;
  const Tile t = reinterpret_cast<const Tile*>(sched + a.kv_list_off)[slot];
  const int kt = t.idx;
  const int L = t.doc_len;

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, n = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, blk = (lane >> 4) & 1;

  const int64_t tok0 = t.tok_start;
  const elem_t* qb = reinterpret_cast<const elem_t*>(a.q.ptr) + t.batch * a.q.sb + head * a.q.sh + tok0 * a.q.st;
  const elem_t* kb = reinterpret_cast<const elem_t*>(a.k.ptr) + t.batch * a.k.sb + head * a.k.sh + tok0 * a.k.st;
  const elem_t* vb = reinterpret_cast<const elem_t*>(a.v.ptr) + t.batch * a.v.sb + head * a.v.sh + tok0 * a.v.st;
  const elem_t* gob = reinterpret_cast<const elem_t*>(a.go.ptr) + t.batch * a.go.sb + head * a.go.sh + tok0 * a.go.st;
  const Rows qrows = make_rows(qb, a.q.st, L);
  const Rows grows = make_rows(gob, a.go.st, L);
  const Rows krows = make_rows(kb, a.k.st, L);
  const Rows vrows = make_rows(vb, a.v.st, L);

  const int q_first = kt * BKV;                      // first query that can see the tile
  const int nblk = (L - q_first + 31) / 32;          // query blocks behind the tile's first key (not STREAM: 1 .. QROWS / 32)
  // all of those Q and dO rows at once, or the first block of them (rows past the document arrive as zeros)
  TileCopy<D, STREAM ? SEG : QROWS, NT, false> qcopy, gcopy;
  qcopy.init(tid, qrows.row_bytes);
  gcopy.init(tid, grows.row_bytes);
  qcopy.issue(qrows, q_first, Qs, STREAM ? SEG : 32 * nblk);      // (32 or 64 rows per instruction of all waves: whole query blocks)
  gcopy.issue(grows, q_first, Gs, STREAM ? SEG : 32 * nblk);
  // Wave w of workgroup b takes key block (w + b) mod 4: the block with the most queries behind it
  // is the first one, and two workgroups that share a CU should not both put it on the same SIMD.
  const int kblk = (w + blockIdx.x) & (BKV / 32 - 1);
  const int k0 = q_first + 32 * kblk;                // this wave's keys
  const bool active = k0 < L;
  el8 kf[KS], vf[KS];                                // MFMA row n holds key k0 + kperm(n)
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    kf[ks] = load_frag(krows, k0 + kperm(n), 32 * ks + 16 * h);
    vf[ks] = load_frag(vrows, k0 + kperm(n), 32 * ks + 16 * h);
  }
  // A block that starts past the end of the document is never visible; its table reads are
  // redirected into the document's area and never used.
  const int tblock = min((BKV / 32) * kt + kblk, (L - 1) / 32);
  const int64_t tab_row0 = (int64_t)head * a.tab_stride + t.tab_base;
  const int64_t tab = tab_row0 + tab_seg32(L, tblock);
  const int64_t tab_rowval = tab_row0 + tab_rowplane32(L);
  struct Raw { float e, g, d; };
  auto request = [&](int qblk, Raw& r) {             // the carries of a query block, clamped into the document
    const int qrow = q_first + 32 * qblk + n;
    const int qc = qrow < L ? qrow : L - 1;
    r.e = a.stick[tab + qc];
    r.g = a.gtab[tab + qc];
    r.d = a.gtab[tab_rowval + qc];
  };
  Raw cur, nxt;
  request(kblk, cur);
  float rem_own = 0.0f;       // fused output: rem_j * do_j reaches dv_j through the diagonal of P (see above)
  if (a.fuse && k0 + n < L) rem_own = a.stick[tab_rowval + k0 + n];

  int roff[KS], xoff[2], yoff[2][DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) roff[ks] = swz_off<D>(n, 2 * ks + h);
  // The private p / dz blocks have rows of 64 bytes (4 chunks).  A transpose read takes 4 whole
  // consecutive rows, which are 256 contiguous bytes whatever the order of the chunks inside a row;
  // the 16-byte row writes of 16 lanes are spread over the banks by rotating the chunks with row/4.
  auto blk_off = [](int row, int chunk) { return row * 32 + ((chunk ^ ((row >> 2) & 3)) << 3); };
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int r = 8 * h + 4 * u + (i16 >> 2);
    const int xc = 16 * blk + 4 * (i16 & 3);                    // key column inside the block (elements)
    xoff[u] = blk_off(r, xc >> 3) + (xc & 7);
#pragma unroll
    for (int j = 0; j < DB; ++j) {
      const int yc = 32 * j + 16 * blk + 4 * (i16 & 3);         // d column (elements)
      yoff[u][j] = swz_off<D>(r, yc >> 3) + (yc & 7);
    }
  }
  if constexpr (!STREAM) {
    wait_loads<0>();
    lds_barrier();            // the only barrier: every wave's part of the Q / dO rows has landed
    if (!active) return;
  }

  unsigned short* Pt = St[w][0];
  unsigned short* Zt = St[w][1];
  // Query block qblk, whose Q / dO rows begin at buffer row lrow0.  WHAT: 0 = p alone and its
  // products into `acc` (dv), 1 = dz alone and its products into `acc` (dk), 2 = both, dk into `acc2`.
  auto block = [&](auto what_tag, f32x16 (&acc)[DB], f32x16 (&acc2)[DB], const int qblk, const int lrow0) {
    constexpr int WHAT = decltype(what_tag)::value;
    constexpr bool DV = WHAT != 1, DK = WHAT != 0;
    request(qblk + 1, nxt);                           // (clamped; unused past the last block)
    const int qw0 = q_first + 32 * qblk;
    const int qrow = qw0 + n;
    const bool ok = qrow < L;
    float carry_e = ok ? cur.e : (PROD ? 1.0f : 0.0f);
    float carry_c = ok ? cur.g : 0.0f;
    const float dr = ok ? cur.d : 0.0f;
    f32x16 x, da;
#pragma unroll
    for (int j = 0; j < 16; ++j) { x[j] = 0.0f; da[j] = 0.0f; }
    {
      const unsigned short* Qt = Qs + lrow0 * D;
      const unsigned short* Gt = Gs + lrow0 * D;
      // (head_dim 256: four contraction steps at a time, so that the operand fragments of a whole
      // chain are never in registers at once)
      constexpr int CH = D > 128 ? 4 : KS;
#pragma unroll
      for (int c0 = 0; c0 < KS; c0 += CH) {
        el8 qfr[CH], gfr[CH];
#pragma unroll
        for (int ks = 0; ks < CH; ++ks) {
          qfr[ks] = lds_row8(Qt + roff[c0 + ks]);
          if constexpr (DK) gfr[ks] = lds_row8(Gt + roff[c0 + ks]);
        }
#pragma unroll
        for (int ks = 0; ks < CH; ++ks) {
          x = mfma32(kf[c0 + ks], qfr[ks], x);
          if constexpr (DK) da = mfma32(vf[c0 + ks], gfr[ks], da);
        }
        if constexpr (D > 128) __builtin_amdgcn_sched_barrier(0);
      }
    }
    el8 pf[2], zf[2];
    {
      float p[16], bt[16], ends[2] = {0.0f, 0.0f};
      grad_weights<AC, PROD>(x, a.c, k0, qw0, qrow, h, carry_e, p, bt, ends);
      if constexpr (DV) {
        if (a.fuse && qblk == kblk) {
          float pd[16];
#pragma unroll
          for (int j = 0; j < 16; ++j) pd[j] = p[j] + (16 * h + j == n ? rem_own : 0.0f);
          pf[0] = pack8(pd);
          pf[1] = pack8(pd + 8);
        } else {
          pf[0] = pack8(p);
          pf[1] = pack8(p + 8);
        }
      }
      if constexpr (DK) grad_dz<PROD>(p, bt, da, ends, h, carry_c, dr, zf);
    }
    // turn the block around: [query][key] rows in, key-major MFMA operands out
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      if constexpr (DV) *reinterpret_cast<el8*>(Pt + blk_off(n, 2 * h + tt)) = pf[tt];
      if constexpr (DK) *reinterpret_cast<el8*>(Zt + blk_off(n, 2 * h + tt)) = zf[tt];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own writes have landed
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      el8 ap, az;
      if constexpr (DV) ap = lds_tr8(Pt + xoff[0] + 16 * ks * 32, Pt + xoff[1] + 16 * ks * 32);
      if constexpr (DK) az = lds_tr8(Zt + xoff[0] + 16 * ks * 32, Zt + xoff[1] + 16 * ks * 32);
      const unsigned short* Gr = Gs + (lrow0 + 16 * ks) * D;
      const unsigned short* Qr = Qs + (lrow0 + 16 * ks) * D;
#pragma unroll
      for (int j = 0; j < DB; ++j) {
        if constexpr (DV) acc[j] = mfma32(ap, lds_tr8(Gr + yoff[0][j], Gr + yoff[1][j]), acc[j]);
        if constexpr (WHAT == 1) acc[j] = mfma32(az, lds_tr8(Qr + yoff[0][j], Qr + yoff[1][j]), acc[j]);
        if constexpr (WHAT == 2) acc2[j] = mfma32(az, lds_tr8(Qr + yoff[0][j], Qr + yoff[1][j]), acc2[j]);
        if constexpr (D > 128) { if (j % 4 == 3) __builtin_amdgcn_sched_barrier(0); }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the reads are done before the next block overwrites the piece
    cur = nxt;
  };
  auto clear = [&](f32x16 (&acc)[DB]) {
#pragma unroll
    for (int j = 0; j < DB; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[j][i] = 0.0f;
  };
  elem_t* dvb = reinterpret_cast<elem_t*>(a.dv.ptr) + t.batch * a.dv.sb + head * a.dv.sh + tok0 * a.dv.st;
  elem_t* dkb = reinterpret_cast<elem_t*>(a.dk.ptr) + t.batch * a.dk.sb + head * a.dk.sh + tok0 * a.dk.st;
  if constexpr (!STREAM) {
    f32x16 acc_v[DB], acc_k[DB];
    clear(acc_v);
    clear(acc_k);
    // query blocks at or after the key block (those before it see none of these keys)
#pragma unroll 1
    for (int qblk = kblk; qblk < nblk; ++qblk) block(std::integral_constant<int, 2>{}, acc_v, acc_k, qblk, 32 * qblk);
    // the private piece becomes the output scratch (at most its size)
    static_assert(STREAM || 2 * 32 * 32 >= 32 * D, "the staging piece of a wave doubles as its output scratch");
    store_block32<D>(Pt, acc_v, 1.0f, dvb, a.dv.st, k0, L, lane);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    store_block32<D>(Pt, acc_k, a.inv_temp, dkb, a.dk.st, k0, L, lane);
  } else {
    // Two passes over the queries, dv first and dk second; the scores are formed in each.
    // Segment s (SEG query rows) sits in buffer s & 1.  At its top every wave is done with segment s - 1,
    // whose buffer takes the rows of segment s + 1 while this one is worked on.
    static_assert(!STREAM || (QROWS >= 64 && NT / 64 == 4), "a quarter of the first 64 rows of the two buffers per wave for its output");
    unsigned short* const scratch = (w & 2 ? Gs : Qs) + (w & 1) * 32 * D;
    constexpr int BPS = SEG / 32;                     // query blocks per segment
    const int nseg = (nblk + BPS - 1) / BPS;
    auto pass = [&](auto what_tag) {
      f32x16 acc[DB];
      clear(acc);
#pragma unroll 1
      for (int sgm = 0; sgm < nseg; ++sgm) {
        wait_loads<0>();
        lds_barrier();
        if (sgm + 1 < nseg) {
          qcopy.issue(qrows, q_first + (sgm + 1) * SEG, Qs + ((sgm + 1) & 1) * SEG * D);
          gcopy.issue(grows, q_first + (sgm + 1) * SEG, Gs + ((sgm + 1) & 1) * SEG * D);
        }
#pragma unroll
        for (int b = 0; b < BPS; ++b) {
          const int qblk = BPS * sgm + b;
          if (active && qblk >= kblk && qblk < nblk) block(what_tag, acc, acc, qblk, (sgm & 1) * SEG + 32 * b);
        }
      }
      lds_barrier();            // every wave is done with the buffers: they become the output staging
      if (active) {
        if constexpr (decltype(what_tag)::value == 0) store_block32<D>(scratch, acc, 1.0f, dvb, a.dv.st, k0, L, lane);
        else store_block32<D>(scratch, acc, a.inv_temp, dkb, a.dk.st, k0, L, lane);
      }
    };
    pass(std::integral_constant<int, 0>{});
    lds_barrier();              // and buffers again: the first block's rows once more
    qcopy.issue(qrows, q_first, Qs, SEG);
    gcopy.issue(grows, q_first, Gs, SEG);
    request(kblk, cur);
    pass(std::integral_constant<int, 1>{});
  }
}

// Explicit instantiations: every (head_dim, attend_current, carry space) variant the launchers use.
template __global__ void bwd_dq_kernel<32, false, false>(const KArgs);
template __global__ void bwd_dq_kernel<32, false, true>(const KArgs);
template __global__ void bwd_dq_kernel<32, true, false>(const KArgs);
template __global__ void bwd_dq_kernel<32, true, true>(const KArgs);
template __global__ void bwd_dq_kernel<64, false, false>(const KArgs);
template __global__ void bwd_dq_kernel<64, false, true>(const KArgs);
template __global__ void bwd_dq_kernel<64, true, false>(const KArgs);
template __global__ void bwd_dq_kernel<64, true, true>(const KArgs);
template __global__ void bwd_dq_kernel<128, false, false>(const KArgs);
template __global__ void bwd_dq_kernel<128, false, true>(const KArgs);
template __global__ void bwd_dq_kernel<128, true, false>(const KArgs);
template __global__ void bwd_dq_kernel<128, true, true>(const KArgs);
template __global__ void bwd_dq_kernel<256, false, false>(const KArgs);
template __global__ void bwd_dq_kernel<256, false, true>(const KArgs);
template __global__ void bwd_dq_kernel<256, true, false>(const KArgs);
template __global__ void bwd_dq_kernel<256, true, true>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<256, false, false, true>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<256, false, true, true>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<256, true, false, true>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<256, true, true, true>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<32, false, false, false>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<32, false, true, false>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<32, true, false, false>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<32, true, true, false>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<64, false, false, false>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<64, false, true, false>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<64, true, false, false>(const KArgs);
template __global__ void bwd_dkdv_tail_kernel<64, true, true, false>(const KArgs);
template __global__ void bwd_dkdv_kernel<32, false, false>(const KArgs);
template __global__ void bwd_dkdv_kernel<32, false, true>(const KArgs);
template __global__ void bwd_dkdv_kernel<32, true, false>(const KArgs);
template __global__ void bwd_dkdv_kernel<32, true, true>(const KArgs);
template __global__ void bwd_dkdv_kernel<64, false, false>(const KArgs);
template __global__ void bwd_dkdv_kernel<64, false, true>(const KArgs);
template __global__ void bwd_dkdv_kernel<64, true, false>(const KArgs);
template __global__ void bwd_dkdv_kernel<64, true, true>(const KArgs);
template __global__ void bwd_dkdv_kernel<128, false, false>(const KArgs);
template __global__ void bwd_dkdv_kernel<128, false, true>(const KArgs);
template __global__ void bwd_dkdv_kernel<128, true, false>(const KArgs);
template __global__ void bwd_dkdv_kernel<128, true, true>(const KArgs);

template <int D>
static hipError_t launch_dq_d(const KArgs& a, bool ac, bool prod, int n_q_max, hipStream_t s) {
  const dim3 grid((unsigned)n_q_max * (unsigned)a.heads), block(NT);
  if (ac) {
    if (prod) hipLaunchKernelGGL((bwd_dq_kernel<D, true, true>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((bwd_dq_kernel<D, true, false>), grid, block, 0, s, a);
  } else {
    if (prod) hipLaunchKernelGGL((bwd_dq_kernel<D, false, true>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((bwd_dq_kernel<D, false, false>), grid, block, 0, s, a);
  }
  return hipGetLastError();
}

// n_long_max / n_last_max: upper bounds on the key tiles of the first / second group of the list.
template <int D, bool STREAM>
static void launch_dkdv_four_waves(const KArgs& a, bool ac, bool prod, unsigned tiles, hipStream_t s) {
  const dim3 grid(tiles * (unsigned)a.heads), block(NT);
  if (ac) {
    if (prod) hipLaunchKernelGGL((bwd_dkdv_tail_kernel<D, true, true, STREAM>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((bwd_dkdv_tail_kernel<D, true, false, STREAM>), grid, block, 0, s, a);
  } else {
    if (prod) hipLaunchKernelGGL((bwd_dkdv_tail_kernel<D, false, true, STREAM>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((bwd_dkdv_tail_kernel<D, false, false, STREAM>), grid, block, 0, s, a);
  }
}

// n_long_max / n_last_max: upper bounds on the key tiles of the first / second group of the list.
template <int D>
static hipError_t launch_dkdv_d(const KArgs& a_in, bool ac, bool prod, int n_long_max, int n_last_max, hipStream_t s) {
  static_assert(TailKernel<D>::value == (D <= 64), "has_dkdv_tail_kernel() states the same rule for the host");
  KArgs a = a_in;
  const DkdvGrid g = dkdv_grid(TailKernel<D>::value, n_long_max, n_last_max, a.n_kv_alloc);
  const unsigned n_main = (unsigned)g.main_tiles;
  if constexpr (StreamKernel<D>::value) {
    // every key tile of both groups to the four independent waves, queries streamed
    if (n_main > 0) launch_dkdv_four_waves<D, true>(a, ac, prod, n_main, s);
  } else {
    if (n_main > 0) {
      a.n_items = (int)(n_main * (unsigned)a.heads);
      const dim3 grid(launch_grid(a, a.n_items)), block(NT2);
      if (ac) {
        if (prod) hipLaunchKernelGGL((bwd_dkdv_kernel<D, true, true>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((bwd_dkdv_kernel<D, true, false>), grid, block, 0, s, a);
      } else {
        if (prod) hipLaunchKernelGGL((bwd_dkdv_kernel<D, false, true>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((bwd_dkdv_kernel<D, false, false>), grid, block, 0, s, a);
      }
    }
    if constexpr (TailKernel<D>::value) {
      if (g.tail_tiles > 0) launch_dkdv_four_waves<D, false>(a, ac, prod, (unsigned)g.tail_tiles, s);
    }
  }
  return hipGetLastError();
}

hipError_t launch_bwd_dq(const KArgs& a, int head_dim, bool ac, bool prod, int n_q_max, hipStream_t s) {
  if (head_dim == 256) return launch_dq_d<256>(a, ac, prod, n_q_max, s);
  if (head_dim == 128) return launch_dq_d<128>(a, ac, prod, n_q_max, s);
  if (head_dim == 64) return launch_dq_d<64>(a, ac, prod, n_q_max, s);
  return launch_dq_d<32>(a, ac, prod, n_q_max, s);
}

hipError_t launch_bwd_dkdv(const KArgs& a, int head_dim, bool ac, bool prod, int n_long_max, int n_last_max,
                           hipStream_t s) {
  if (head_dim == 256) return launch_dkdv_d<256>(a, ac, prod, n_long_max, n_last_max, s);
  if (head_dim == 128) return launch_dkdv_d<128>(a, ac, prod, n_long_max, n_last_max, s);
  if (head_dim == 64) return launch_dkdv_d<64>(a, ac, prod, n_long_max, n_last_max, s);
  return launch_dkdv_d<32>(a, ac, prod, n_long_max, n_last_max, s);
}

}  // inline namespace SBA_ELEM_NS
}  // namespace sba
