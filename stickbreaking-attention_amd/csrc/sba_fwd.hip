// Forward kernel: one 128-row query tile of one (document, head) per workgroup, KV tiles of
// 32 keys walked from the causal diagonal back to the start of the document.
//
// Replaces upstream `_forward` / `_forward_one_row`
// (stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:81-215, :231-410) and the fixed-length
// wrapper (stickbreaking_attention/sb_attn/sb_fwd.py:15-136).
#include "sba_kernels.hpp"

#include <type_traits>

namespace sba {
inline namespace SBA_ELEM_NS {

// MODE 1 (WOUT): also write the attention weights (fp32, before their bf16 rounding) into a dense
// [tokens x tokens] matrix per (batch, head) -- upstream's `return_attention` debug output
// (sb_varlen_fwd.py:195-202).  MODE 2 (TAB): write the carry table and nothing else -- no V tiles,
// no P.V products, no o, no rem -- for a backward whose forward kept no table.  Separate
// instantiations, so the production kernel (MODE 0) carries none of it.
// head_dim 256: the ring takes 96 KiB, so one workgroup per CU and one wave per SIMD, with the whole register
// file (512 registers per lane) for its 64 registers of Q fragments and 128 of accumulators.
template <int D, bool AC, bool PROD, int MODE>
__global__ void __launch_bounds__(NT, D > 128 ? 1 : 3) fwd_kernel(const KArgs a) {
  constexpr bool WOUT = MODE == 1, TAB = MODE == 2;
  constexpr int KS = D / 16;     // contraction steps of K.Q^T
  constexpr int DB = D / 32;     // 32-wide output column blocks of P.V
  constexpr int BF = 32;         // keys per staged tile: one MFMA sub-block
  constexpr int TILE = BF * D;   // elements of one K or V tile (unpadded, swizzled)
  // K and V tiles of 32 keys in a three-slot ring filled by asynchronous global -> LDS copies:
  // 48 KiB per workgroup at head_dim 128, so three workgroups share a CU.
  __shared__ __attribute__((aligned(16))) unsigned short smem[6 * TILE];
  unsigned short* const Ks = smem;              // three K tiles
  unsigned short* const Vs = smem + 3 * TILE;   // three V tiles

  // Header words and this workgroup's tile are fetched together (the grid never exceeds the
  // allocated list, so the tile read is safe before the count is known): one round trip.
  const int* sched = a.sched;
  const int slot = blockIdx.x / a.heads;
  const int head = blockIdx.x - slot * a.heads;
  const int4 hdr = *reinterpret_cast<const int4*>(sched);   // status, query tiles, key tiles, table entries needed
  const Tile t = reinterpret_cast<const Tile*>(sched + SCHED_HDR)[slot];
  asm volatile("" ::"s"(t.tok_start), "s"(t.doc_len), "s"(t.idx), "s"(t.batch));   // keep the tile read above the branch
  const bool refused = hdr.x != 0 || (a.stick != nullptr && hdr.w > a.tab_stride);
  if (refused || slot >= hdr.y) {
    if (a.clear_spare && !TAB) {
      int row0, row1;
      unsigned pair;
      spare_rows(refused, slot, hdr.y, sched[SCHED_TOTAL], a.tokens, a.nan_pair, row0, row1, pair);
      fill_rows16(a.o, head, row0, row1, D, pair, threadIdx.x, NT);
      fill_rows16(a.rem, head, row0, row1, 1, pair, threadIdx.x, NT);
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
  elem_t* ob = reinterpret_cast<elem_t*>(a.o.ptr) + t.batch * a.o.sb + head * a.o.sh + tok0 * a.o.st;
  elem_t* rb = reinterpret_cast<elem_t*>(a.rem.ptr) + t.batch * a.rem.sb + head * a.rem.sh + tok0 * a.rem.st;
  const Rows qrows = make_rows(qb, a.q.st, t.doc_len);
  const Rows krows = make_rows(kb, a.k.st, t.doc_len);
  const Rows vrows = make_rows(vb, a.v.st, t.doc_len);

  const int last_key = min(m0 + BM - 1, t.doc_len - 1);
  const int kt_last = last_key / BF;

  // Q^T operand fragments: lane (n, h) holds Q[qrow][16*ks + 8*h .. +7] (zeros past the document).
  el8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) qf[ks] = load_frag(qrows, qrow, 32 * ks + 16 * h);

  // Three-stage ring of K/V tiles: two tiles are in flight while one is consumed.
  // (a 32 x 32 tile is one instruction each for two waves: the other two request nothing, wait for
  // nothing and meet the copies at the barrier)
  constexpr int CT = D == 32 ? NT / 2 : NT;   // threads that copy tiles
  const bool copier = tid < CT;               // (uniform per wave)
  TileCopy<D, BF, CT, true> kcopy, vcopy;
  kcopy.init(tid, krows.row_bytes);
  vcopy.init(tid, vrows.row_bytes);
  constexpr int LOADS_PER_TILE = (TAB ? 1 : 2) * TileCopy<D, BF, CT, true>::NCH;
  if (copier) {
    kcopy.issue(krows, kt_last * BF, Ks);
    if (!TAB) vcopy.issue(vrows, kt_last * BF, Vs);
    if (kt_last >= 1) {
      kcopy.issue(krows, (kt_last - 1) * BF, Ks + TILE);
      if (!TAB) vcopy.issue(vrows, (kt_last - 1) * BF, Vs + TILE);
    }
  }

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[db][i] = 0.0f;
  float carry = PROD ? 1.0f : 0.0f;

  // Offsets (elements) inside a tile.  K: row read of chunk 2*ks + h of LDS row n (= MFMA row n).
  // V: transpose reads of rows 8*u + 4*h + i/4 (+ 16*tt), columns 32*db + 16*blk + 4*(i%4).
  const int i16 = lane & 15, blk = (lane >> 4) & 1;
  int koff[KS], voff[2][DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff[ks] = swz_off<D>(n, 2 * ks + h);
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int r = 8 * u + 4 * h + (i16 >> 2);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int col = 32 * db + 16 * blk + 4 * (i16 & 3);
      voff[u][db] = swz_off<D>(r, col >> 3) + (col & 7);
    }
  }
  // the document's triangular table area; a lane adds its row and a block's 32-bit offset
  float* stick = a.stick == nullptr ? nullptr : a.stick + (int64_t)head * a.tab_stride + t.tab_base;   // (uniform)

  // One tile step; the ring slot is a compile-time constant so every LDS address is a fixed
  // register plus an immediate.
  auto tile = [&](auto slot_c, const int kt) {
    constexpr int SLOT = decltype(slot_c)::value;
    constexpr int REFILL = (SLOT + 2) % 3;   // slot of tile kt + 1, free once every wave is past it
    // Tile kt has landed when only the loads of tile kt - 1 (issued after it, returning in
    // order) can still be in flight; stores in between only make the wait stricter.
    if (kt >= 1) wait_loads<LOADS_PER_TILE>(); else wait_loads<0>();
    lds_barrier();
    if (kt >= 2 && copier) {
      kcopy.issue(krows, (kt - 2) * BF, Ks + REFILL * TILE);
      if (!TAB) vcopy.issue(vrows, (kt - 2) * BF, Vs + REFILL * TILE);
    }
    const unsigned short* Kt = Ks + SLOT * TILE;
    const unsigned short* Vt = Vs + SLOT * TILE;
    const int k0 = kt * BF;
    if (sub_skip<AC>(k0, qw0)) return;
    // stick left on entering this block: what both backward kernels start it from
    if (stick != nullptr && h == 0 && qvalid) stick[(unsigned)(tab_seg32(t.doc_len, kt) + qrow)] = carry;
    f32x16 x;
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = 0.0f;
    {
      el8 kfr[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kfr[ks] = lds_row8(Kt + koff[ks]);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) x = mfma32(kfr[ks], qf[ks], x);
    }
    float p[16];
    if constexpr (PROD) {
      if (sub_full<AC>(k0, qw0)) stick_weights_fwd<AC, false>(x, a.c, k0, qrow, h, carry, p);
      else stick_weights_fwd<AC, true>(x, a.c, k0, qrow, h, carry, p);
    } else {
      float unused[16];
      if (sub_full<AC>(k0, qw0)) stick_weights<AC, PROD, false, false>(x, a.c, k0, qrow, h, carry, p, unused);
      else stick_weights<AC, PROD, true, false>(x, a.c, k0, qrow, h, carry, p, unused);
    }
    if constexpr (WOUT) {
      // this lane: query qrow, keys k0 + 16*h + i; masked positions already hold 0
      if (qvalid) {
        float* wrow = a.weights + (((int64_t)t.batch * a.heads + head) * a.tokens + tok0 + qrow) * a.tokens + tok0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = k0 + 16 * h + i;
          if (key < t.doc_len) wrow[key] = p[i];
        }
      }
    }
    if constexpr (TAB) return;
    // P as the A operand of O = P.V: slot s of step tt is key 16*h + 8*tt + s, which the
    // permuted tile keeps in LDS row 16*tt + 8*(s/4) + 4*h + s%4.
    el8 vfr[2][DB];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const unsigned short* vrow = Vt + 16 * tt * D;
#pragma unroll
      for (int db = 0; db < DB; ++db) vfr[tt][db] = lds_tr8(vrow + voff[0][db], vrow + voff[1][db]);
    }
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const el8 pf = pack8(p + 8 * tt);
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] = mfma32(pf, vfr[tt][db], oacc[db]);
    }
  };

  // The Q fragments and both tiles have landed.  (A full wait, so that the compiler's bookkeeping
  // holds no load of its own when the loop begins: a wait it placed inside the loop for the Q
  // fragments would, from the second step on, wait for the tile copies issued in between.)
  wait_loads<0>();
  for (int kt = kt_last;;) {
    tile(std::integral_constant<int, 0>{}, kt);
    if (--kt < 0) break;
    tile(std::integral_constant<int, 1>{}, kt);
    if (--kt < 0) break;
    tile(std::integral_constant<int, 2>{}, kt);
    if (--kt < 0) break;
  }

  // epilogue: rem = what is left of the stick; o rows in the accumulator layout
  const float r = PROD ? carry : fast_exp2(carry);
  if (h == 0 && qvalid) {
    if (!TAB) rb[(int64_t)qrow * a.rem.st] = (elem_t)r;
    // rem in full precision for the backward of the fused output (last plane of the table)
    if (stick != nullptr) stick[(unsigned)(tab_rowplane32(t.doc_len) + qrow)] = r;
  }
  if constexpr (TAB) return;
  lds_barrier();   // every wave is done with the K/V tiles: their memory becomes the o staging area
  if (a.fuse) {
    // what every caller computes next (upstream tests/test_varlen.py:101): o + rem * v
    store_block32_axpy<D>(smem + w * 32 * D, oacc, 1.0f, ob, a.o.st, qw0, t.doc_len, lane, vb, a.v.st,
                          [&](int row) { return __shfl(r, row, 64); });
  } else {
    store_block32<D>(smem + w * 32 * D, oacc, 1.0f, ob, a.o.st, qw0, t.doc_len, lane);
  }
}

// Explicit instantiations: every (head_dim, attend_current, carry space) variant the launchers use.
template __global__ void fwd_kernel<32, false, false, 0>(const KArgs);
template __global__ void fwd_kernel<32, false, false, 1>(const KArgs);
template __global__ void fwd_kernel<32, false, true, 0>(const KArgs);
template __global__ void fwd_kernel<32, false, true, 1>(const KArgs);
template __global__ void fwd_kernel<32, true, false, 0>(const KArgs);
template __global__ void fwd_kernel<32, true, false, 1>(const KArgs);
template __global__ void fwd_kernel<32, true, true, 0>(const KArgs);
template __global__ void fwd_kernel<32, true, true, 1>(const KArgs);
template __global__ void fwd_kernel<64, false, false, 0>(const KArgs);
template __global__ void fwd_kernel<64, false, false, 1>(const KArgs);
template __global__ void fwd_kernel<64, false, true, 0>(const KArgs);
template __global__ void fwd_kernel<64, false, true, 1>(const KArgs);
template __global__ void fwd_kernel<64, true, false, 0>(const KArgs);
template __global__ void fwd_kernel<64, true, false, 1>(const KArgs);
template __global__ void fwd_kernel<64, true, true, 0>(const KArgs);
template __global__ void fwd_kernel<64, true, true, 1>(const KArgs);
template __global__ void fwd_kernel<128, false, false, 0>(const KArgs);
template __global__ void fwd_kernel<128, false, false, 1>(const KArgs);
template __global__ void fwd_kernel<128, false, true, 0>(const KArgs);
template __global__ void fwd_kernel<128, false, true, 1>(const KArgs);
template __global__ void fwd_kernel<128, true, false, 0>(const KArgs);
template __global__ void fwd_kernel<128, true, false, 1>(const KArgs);
template __global__ void fwd_kernel<128, true, true, 0>(const KArgs);
template __global__ void fwd_kernel<128, true, true, 1>(const KArgs);

template __global__ void fwd_kernel<32, false, false, 2>(const KArgs);
template __global__ void fwd_kernel<32, false, true, 2>(const KArgs);
template __global__ void fwd_kernel<32, true, false, 2>(const KArgs);
template __global__ void fwd_kernel<32, true, true, 2>(const KArgs);
template __global__ void fwd_kernel<64, false, false, 2>(const KArgs);
template __global__ void fwd_kernel<64, false, true, 2>(const KArgs);
template __global__ void fwd_kernel<64, true, false, 2>(const KArgs);
template __global__ void fwd_kernel<64, true, true, 2>(const KArgs);
template __global__ void fwd_kernel<128, false, false, 2>(const KArgs);
template __global__ void fwd_kernel<128, false, true, 2>(const KArgs);
template __global__ void fwd_kernel<128, true, false, 2>(const KArgs);
template __global__ void fwd_kernel<128, true, true, 2>(const KArgs);
template __global__ void fwd_kernel<256, false, false, 0>(const KArgs);
template __global__ void fwd_kernel<256, false, false, 1>(const KArgs);
template __global__ void fwd_kernel<256, false, true, 0>(const KArgs);
template __global__ void fwd_kernel<256, false, true, 1>(const KArgs);
template __global__ void fwd_kernel<256, true, false, 0>(const KArgs);
template __global__ void fwd_kernel<256, true, false, 1>(const KArgs);
template __global__ void fwd_kernel<256, true, true, 0>(const KArgs);
template __global__ void fwd_kernel<256, true, true, 1>(const KArgs);
template __global__ void fwd_kernel<256, false, false, 2>(const KArgs);
template __global__ void fwd_kernel<256, false, true, 2>(const KArgs);
template __global__ void fwd_kernel<256, true, false, 2>(const KArgs);
template __global__ void fwd_kernel<256, true, true, 2>(const KArgs);

template <int D, int MODE>
static hipError_t launch_fwd_d(const KArgs& a, bool ac, bool prod, int n_q_max, hipStream_t s) {
  const dim3 grid((unsigned)n_q_max * (unsigned)a.heads), block(NT);
  if (ac) {
    if (prod) hipLaunchKernelGGL((fwd_kernel<D, true, true, MODE>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((fwd_kernel<D, true, false, MODE>), grid, block, 0, s, a);
  } else {
    if (prod) hipLaunchKernelGGL((fwd_kernel<D, false, true, MODE>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((fwd_kernel<D, false, false, MODE>), grid, block, 0, s, a);
  }
  return hipGetLastError();
}

// mode: 0 = o and rem (and the table when one is given), 1 = the attention weights as well, 2 = the table alone
hipError_t launch_fwd(const KArgs& a, int head_dim, bool ac, bool prod, int mode, int n_q_max, hipStream_t s) {
  if (mode == 1) {
    if (head_dim == 256) return launch_fwd_d<256, 1>(a, ac, prod, n_q_max, s);
    if (head_dim == 128) return launch_fwd_d<128, 1>(a, ac, prod, n_q_max, s);
    if (head_dim == 64) return launch_fwd_d<64, 1>(a, ac, prod, n_q_max, s);
    return launch_fwd_d<32, 1>(a, ac, prod, n_q_max, s);
  }
  if (mode == 2) {
    if (head_dim == 256) return launch_fwd_d<256, 2>(a, ac, prod, n_q_max, s);
    if (head_dim == 128) return launch_fwd_d<128, 2>(a, ac, prod, n_q_max, s);
    if (head_dim == 64) return launch_fwd_d<64, 2>(a, ac, prod, n_q_max, s);
    return launch_fwd_d<32, 2>(a, ac, prod, n_q_max, s);
  }
  if (head_dim == 256) return launch_fwd_d<256, 0>(a, ac, prod, n_q_max, s);
  if (head_dim == 128) return launch_fwd_d<128, 0>(a, ac, prod, n_q_max, s);
  if (head_dim == 64) return launch_fwd_d<64, 0>(a, ac, prod, n_q_max, s);
  return launch_fwd_d<32, 0>(a, ac, prod, n_q_max, s);
}

}  // inline namespace SBA_ELEM_NS
}  // namespace sba
