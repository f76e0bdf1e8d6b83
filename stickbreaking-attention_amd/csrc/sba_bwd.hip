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
//
// Per-score math (upstream sb_varlen_bwd.py:439-453):
//   G = A * (do.v - drem),  C = inclusive running sum of G over keys,  dz = G - beta * C,
//   dq = s * dz K,  dk = s * dz^T Q,  dv = A^T do.
#include "sba_kernels.hpp"

namespace sba {

// One 32-key sub-block for the 32 queries of a wave, given the raw score and do.v^T
// accumulators: p, beta from the stick carry at the sub-block's newer edge, G, then dz with
// the running prefix of G (carry_c: in = prefix before the sub-block, out = after it).
// Emits p and dz as bf16 A-operand fragments: slot s of fragment [tt] is key 16*h + 8*tt + s.
template <bool AC, bool PROD, bool NEED_P>
__device__ __forceinline__ void grad_block(const f32x16& x, const f32x16& da, float c, int k0, int qw0,
                                           int qrow, int h, float carry_e, float& carry_c, float dr,
                                           bf16x8 (&pf)[2], bf16x8 (&zf)[2]) {
  float p[16], bt[16];
  if (sub_full<AC>(k0, qw0)) {
    stick_weights<AC, PROD, false, true>(x, c, k0, qrow, h, carry_e, p, bt);
  } else {
    stick_weights<AC, PROD, true, true>(x, c, k0, qrow, h, carry_e, p, bt);
  }
  if (NEED_P) {
    pf[0] = pack8(p);
    pf[1] = pack8(p + 8);
  }
  float g[16], cs[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) { g[i] = p[i] * (da[i] - dr); cs[i] = g[i]; }
  carry_c += prefix_sum32(cs, h, carry_c);
  float dz[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) dz[i] = g[i] - bt[i] * cs[i];
  zf[0] = pack8(dz);
  zf[1] = pack8(dz + 8);
}

// -------------------------------------------------------------------------------------------
// dq pass
// -------------------------------------------------------------------------------------------
template <int D, bool AC, bool PROD>
__global__ void __launch_bounds__(NT, 2) bwd_dq_kernel(const KArgs a) {
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int KROW = D + 8;    // K, V copies for row reads (operands of the score products)
  constexpr int TROW = D + 32;   // second K copy for transpose reads (operand of dq)
  constexpr int NCH = BN * (D / 8) / NT;
  __shared__ __attribute__((aligned(16))) unsigned short Ks[BN * KROW];
  __shared__ __attribute__((aligned(16))) unsigned short Kt[BN * TROW];
  __shared__ __attribute__((aligned(16))) unsigned short Vs[BN * KROW];

  const int* sched = a.sched;
  if (sched[SCHED_STATUS] != 0) return;
  const int slot = blockIdx.x / a.heads;
  const int head = blockIdx.x - slot * a.heads;
  if (slot >= sched[SCHED_NQ]) return;
  const Tile t = reinterpret_cast<const Tile*>(sched + SCHED_HDR)[slot];

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, n = lane & 31, h = lane >> 5;
  const int m0 = t.idx * BM;
  const int qw0 = m0 + 32 * w;
  const int qrow = qw0 + n;
  const bool qvalid = qrow < t.doc_len;

  const int64_t tok0 = t.tok_start;
  const __bf16* qb = reinterpret_cast<const __bf16*>(a.q.ptr) + t.batch * a.q.sb + head * a.q.sh + tok0 * a.q.st;
  const __bf16* kb = reinterpret_cast<const __bf16*>(a.k.ptr) + t.batch * a.k.sb + head * a.k.sh + tok0 * a.k.st;
  const __bf16* vb = reinterpret_cast<const __bf16*>(a.v.ptr) + t.batch * a.v.sb + head * a.v.sh + tok0 * a.v.st;
  const __bf16* gob = reinterpret_cast<const __bf16*>(a.go.ptr) + t.batch * a.go.sb + head * a.go.sh + tok0 * a.go.st;
  __bf16* dqb = reinterpret_cast<__bf16*>(a.dq.ptr) + t.batch * a.dq.sb + head * a.dq.sh + tok0 * a.dq.st;
  const int64_t grow = (int64_t)t.batch * a.tokens + tok0 + qrow;
  const Rows qrows = make_rows(qb, a.q.st, t.doc_len);
  const Rows grows = make_rows(gob, a.go.st, t.doc_len);
  const Rows krows = make_rows(kb, a.k.st, t.doc_len);
  const Rows vrows = make_rows(vb, a.v.st, t.doc_len);

  bf16x8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    qf[ks] = load_frag(qrows, qrow, 32 * ks + 16 * h);
    dof[ks] = load_frag(grows, qrow, 32 * ks + 16 * h);
  }
  float dr = 0.0f;
  if (a.grem.ptr != nullptr && qvalid) {
    const __bf16* grb = reinterpret_cast<const __bf16*>(a.grem.ptr) + t.batch * a.grem.sb + head * a.grem.sh + tok0 * a.grem.st;
    dr = (float)grb[(int64_t)qrow * a.grem.st];
  }

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) dqacc[db][i] = 0.0f;
  float carry_c = 0.0f;

  const int last_key = min(m0 + BM - 1, t.doc_len - 1);
  const int kt_last = last_key / BN;
  const int i16 = lane & 15, blk = (lane >> 4) & 1;
  const int ktr = (4 * h + (i16 >> 2)) * TROW + 16 * blk + 4 * (i16 & 3);
  const int64_t tab0 = (int64_t)head * a.n_tt * a.rows_total + grow;
  const float* stick = a.stick + tab0;
  float* gtab = a.gtab + tab0;

  uint4 kreg[NCH], vreg[NCH];
  load_tile<D, BN, NT, true>(krows, 0, kreg);
  load_tile<D, BN, NT, true>(vrows, 0, vreg);

  for (int kt = 0; kt <= kt_last; ++kt) {
    __syncthreads();
    store_tile_padded<D, BN, NT, KROW>(Ks, kreg);
    store_tile_padded<D, BN, NT, TROW>(Kt, kreg);
    store_tile_padded<D, BN, NT, KROW>(Vs, vreg);
    __syncthreads();
    if (kt < kt_last) {
      load_tile<D, BN, NT, true>(krows, (kt + 1) * BN, kreg);
      load_tile<D, BN, NT, true>(vrows, (kt + 1) * BN, vreg);
    }
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const int k0 = kt * BN + 32 * sb;
      if (sub_skip<AC>(k0, qw0)) continue;
      const int64_t tix = (int64_t)(2 * kt + sb) * a.rows_total;
      float carry_e = PROD ? 1.0f : 0.0f;
      if (qvalid) {
        carry_e = stick[tix];
        if (h == 0) gtab[tix] = carry_c;
      }
      f32x16 x, da;
#pragma unroll
      for (int i = 0; i < 16; ++i) { x[i] = 0.0f; da[i] = 0.0f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        x = mfma32(lds_row8(Ks + (32 * sb + n) * KROW + 16 * ks + 8 * h), qf[ks], x);
        da = mfma32(lds_row8(Vs + (32 * sb + n) * KROW + 16 * ks + 8 * h), dof[ks], da);
      }
      bf16x8 pf[2], zf[2];
      grad_block<AC, PROD, false>(x, da, a.c, k0, qw0, qrow, h, carry_e, carry_c, dr, pf, zf);
      // dq += dz . K  (K as the B operand: transpose reads along keys)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const unsigned short* krow = Kt + ktr + (32 * sb + 16 * tt) * TROW;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const bf16x8 kf = lds_tr8(krow + 32 * db, krow + 8 * TROW + 32 * db);
          dqacc[db] = mfma32(zf[tt], kf, dqacc[db]);
        }
      }
    }
  }

#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = qw0 + 8 * (i >> 2) + 4 * h + (i & 3);
      if (row < t.doc_len) dqb[(int64_t)row * a.dq.st + 32 * db + n] = (__bf16)(dqacc[db][i] * a.inv_temp);
    }
  }
}

// -------------------------------------------------------------------------------------------
// dk / dv pass: 8 waves; wave (qg, sb) scores the 32 queries of group qg against the 32 keys
// of sub-block sb (K and V fragments stay in registers for the whole kernel), stages p and dz
// through LDS, then every wave accumulates two 32x32 blocks of dk or dv over all 128 queries.
// -------------------------------------------------------------------------------------------
constexpr int NT2 = 512;

template <int D, bool AC, bool PROD>
__global__ void __launch_bounds__(NT2, 1) bwd_dkdv_kernel(const KArgs a) {
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int NCHQ = BM * (D / 8) / NT2;
  constexpr int DBW = DB / 2;   // d-blocks per wave in the dk/dv products
  // Q and dO tiles: row reads (score operands) and transpose reads (dk/dv operands) -> swizzled.
  __shared__ __attribute__((aligned(16))) unsigned short Qs[BM * D];
  __shared__ __attribute__((aligned(16))) unsigned short Gs[BM * D];
  // p and dz staged [query][key]: 16-byte row writes, transpose reads -> swizzled, 64-key rows.
  __shared__ __attribute__((aligned(16))) unsigned short Ps[BM * BN];
  __shared__ __attribute__((aligned(16))) unsigned short Zs[BM * BN];

  const int* sched = a.sched;
  if (sched[SCHED_STATUS] != 0) return;
  const int slot = blockIdx.x / a.heads;
  const int head = blockIdx.x - slot * a.heads;
  if (slot >= sched[SCHED_NKV]) return;
  const Tile t = reinterpret_cast<const Tile*>(sched + a.kv_list_off)[slot];
  const int kt = t.idx;

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, n = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, blk = (lane >> 4) & 1;
  const int qg = w >> 1, sb = w & 1;
  const int k0 = kt * BN + 32 * sb;

  const int64_t tok0 = t.tok_start;
  const __bf16* qb = reinterpret_cast<const __bf16*>(a.q.ptr) + t.batch * a.q.sb + head * a.q.sh + tok0 * a.q.st;
  const __bf16* kb = reinterpret_cast<const __bf16*>(a.k.ptr) + t.batch * a.k.sb + head * a.k.sh + tok0 * a.k.st;
  const __bf16* vb = reinterpret_cast<const __bf16*>(a.v.ptr) + t.batch * a.v.sb + head * a.v.sh + tok0 * a.v.st;
  const __bf16* gob = reinterpret_cast<const __bf16*>(a.go.ptr) + t.batch * a.go.sb + head * a.go.sh + tok0 * a.go.st;
  const __bf16* grb = a.grem.ptr == nullptr ? nullptr
      : reinterpret_cast<const __bf16*>(a.grem.ptr) + t.batch * a.grem.sb + head * a.grem.sh + tok0 * a.grem.st;
  const Rows qrows = make_rows(qb, a.q.st, t.doc_len);
  const Rows grows = make_rows(gob, a.go.st, t.doc_len);
  const Rows krows = make_rows(kb, a.k.st, t.doc_len);
  const Rows vrows = make_rows(vb, a.v.st, t.doc_len);

  // K and V A-operand fragments of this wave's 32 keys: MFMA row n holds key k0 + kperm(n).
  bf16x8 kf[KS], vf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    kf[ks] = load_frag(krows, k0 + kperm(n), 32 * ks + 16 * h);
    vf[ks] = load_frag(vrows, k0 + kperm(n), 32 * ks + 16 * h);
  }

  // Output ownership in the products: matrix (dv / dk), 32-key block, pair of d-blocks.
  const int mat = w >> 2, kb32 = (w >> 1) & 1, dbp = w & 1;
  f32x16 acc[DBW];
#pragma unroll
  for (int j = 0; j < DBW; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.0f;
  const unsigned short* Xs = mat ? Zs : Ps;   // dz^T or p^T as the A operand
  const unsigned short* Ys = mat ? Qs : Gs;   // Q or dO as the B operand

  // Transpose-read offsets (elements).  Rows are queries 16*ks + 8*h + 4*u + i/4; the swizzle
  // depends on the row modulo 16 only, so it is the same for every ks.
  int xoff[2], yoff[2][DBW];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int r = 8 * h + 4 * u + (i16 >> 2);
    const int xc = 32 * kb32 + 16 * blk + 4 * (i16 & 3);          // key column (elements)
    xoff[u] = swz_off<BN>(r, xc >> 3) + (xc & 7);
#pragma unroll
    for (int j = 0; j < DBW; ++j) {
      const int yc = 32 * (DBW * dbp + j) + 16 * blk + 4 * (i16 & 3);   // d column (elements)
      yoff[u][j] = swz_off<D>(r, yc >> 3) + (yc & 7);
    }
  }
  // Row-read offsets of this lane's query row for the score operands (chunk 2*ks + h).
  const int qr = 32 * qg + n;
  const int64_t tab_head = (int64_t)head * a.n_tt * a.rows_total + (int64_t)t.batch * a.tokens + tok0;
  const int64_t tix_sb = (int64_t)(2 * kt + sb) * a.rows_total;

  const int qt_first = (kt * BN) / BM;
  const int qt_last = (t.doc_len - 1) / BM;
  uint4 qreg[NCHQ], greg[NCHQ];
  load_tile<D, BM, NT2, false>(qrows, qt_first * BM, qreg);
  load_tile<D, BM, NT2, false>(grows, qt_first * BM, greg);

  for (int qt = qt_first; qt <= qt_last; ++qt) {
    const int m0 = qt * BM;
    __syncthreads();   // previous step's products have consumed Qs, Gs, Ps, Zs
    store_tile_swizzled<D, BM, NT2>(Qs, qreg);
    store_tile_swizzled<D, BM, NT2>(Gs, greg);
    __syncthreads();
    if (qt < qt_last) {
      load_tile<D, BM, NT2, false>(qrows, m0 + BM, qreg);
      load_tile<D, BM, NT2, false>(grows, m0 + BM, greg);
    }

    const int qw0 = m0 + 32 * qg;
    const int qrow = qw0 + n;
    bf16x8 pf[2], zf[2];
    if (sub_skip<AC>(k0, qw0)) {
      pf[0] = zero8(); pf[1] = zero8(); zf[0] = zero8(); zf[1] = zero8();
    } else {
      f32x16 x, da;
#pragma unroll
      for (int i = 0; i < 16; ++i) { x[i] = 0.0f; da[i] = 0.0f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        x = mfma32(kf[ks], lds_row8(Qs + swz_off<D>(qr, 2 * ks + h)), x);
        da = mfma32(vf[ks], lds_row8(Gs + swz_off<D>(qr, 2 * ks + h)), da);
      }
      float carry_e = PROD ? 1.0f : 0.0f, carry_c = 0.0f, dr = 0.0f;
      if (qrow < t.doc_len) {
        carry_e = a.stick[tab_head + qrow + tix_sb];
        carry_c = a.gtab[tab_head + qrow + tix_sb];
        if (grb != nullptr) dr = (float)grb[(int64_t)qrow * a.grem.st];
      }
      grad_block<AC, PROD, true>(x, da, a.c, k0, qw0, qrow, h, carry_e, carry_c, dr, pf, zf);
    }
    // stage p and dz as [query][key]: fragment tt is 8 consecutive keys = one 16-byte chunk
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const int chunk = 4 * sb + 2 * h + tt;
      *reinterpret_cast<bf16x8*>(Ps + swz_off<BN>(qr, chunk)) = pf[tt];
      *reinterpret_cast<bf16x8*>(Zs + swz_off<BN>(qr, chunk)) = zf[tt];
    }
    __syncthreads();
    // acc[key, d] += sum over the 128 queries of X[query][key] * Y[query][d]
#pragma unroll
    for (int ks = 0; ks < BM / 16; ++ks) {
      const bf16x8 af = lds_tr8(Xs + xoff[0] + 16 * ks * BN, Xs + xoff[1] + 16 * ks * BN);
#pragma unroll
      for (int j = 0; j < DBW; ++j) {
        const bf16x8 bf = lds_tr8(Ys + yoff[0][j] + 16 * ks * D, Ys + yoff[1][j] + 16 * ks * D);
        acc[j] = mfma32(af, bf, acc[j]);
      }
    }
  }

  const View& ov = mat ? a.dk : a.dv;
  __bf16* outb = reinterpret_cast<__bf16*>(ov.ptr) + t.batch * ov.sb + head * ov.sh + tok0 * ov.st;
  const float scale = mat ? a.inv_temp : 1.0f;
#pragma unroll
  for (int j = 0; j < DBW; ++j) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kt * BN + 32 * kb32 + 8 * (i >> 2) + 4 * h + (i & 3);
      if (key < t.doc_len) outb[(int64_t)key * ov.st + 32 * (DBW * dbp + j) + n] = (__bf16)(acc[j][i] * scale);
    }
  }
}

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

template <int D>
static hipError_t launch_dkdv_d(const KArgs& a, bool ac, bool prod, int n_kv_max, hipStream_t s) {
  const dim3 grid((unsigned)n_kv_max * (unsigned)a.heads), block(NT2);
  if (ac) {
    if (prod) hipLaunchKernelGGL((bwd_dkdv_kernel<D, true, true>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((bwd_dkdv_kernel<D, true, false>), grid, block, 0, s, a);
  } else {
    if (prod) hipLaunchKernelGGL((bwd_dkdv_kernel<D, false, true>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((bwd_dkdv_kernel<D, false, false>), grid, block, 0, s, a);
  }
  return hipGetLastError();
}

hipError_t launch_bwd_dq(const KArgs& a, int head_dim, bool ac, bool prod, int n_q_max, hipStream_t s) {
  if (head_dim == 128) return launch_dq_d<128>(a, ac, prod, n_q_max, s);
  return launch_dq_d<64>(a, ac, prod, n_q_max, s);
}

hipError_t launch_bwd_dkdv(const KArgs& a, int head_dim, bool ac, bool prod, int n_kv_max, hipStream_t s) {
  if (head_dim == 128) return launch_dkdv_d<128>(a, ac, prod, n_kv_max, s);
  return launch_dkdv_d<64>(a, ac, prod, n_kv_max, s);
}

}  // namespace sba
