// Backward kernels.
//
// Upstream computes dq, dk and dv in ONE query-tile-owned kernel and accumulates the dk/dv
// partial tiles of different query tiles through a spin lock in global memory
// (`_backward_one_row` and `locked_add`, stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:
// 297-481 and :12-54).  On MI355X fp32 global atomics sustain about 1.35 TB/s of payload,
// which at 128-row query tiles is several times the whole time budget of the backward, so the
// accumulation is reorganised into two kernels that need no atomics and no locks at all:
//
//   bwd_dq_kernel    query-tile owned (like the forward).  Walks the KV tiles from key 0 to
//                    the diagonal, forms dz and accumulates dq in registers.  On the way it
//                    records, per (row, KV tile), the running prefix C = sum_{keys before the
//                    tile} G in `gtab`.
//   bwd_dkdv_kernel  KV-tile owned.  Loops over the query tiles at or below its keys, takes
//                    the stick carry (table written by the forward) and the G prefix (table
//                    written by bwd_dq_kernel) at its tile boundary, recomputes p and dz and
//                    accumulates dk and dv in registers; every output element is written once.
//
// Per-score math (upstream sb_varlen_bwd.py:439-453):
//   G = A * (do.v - drem),  C = inclusive running sum of G over keys,  dz = G - beta * C,
//   dq = s * dz K,  dk = s * dz^T Q,  dv = A^T do.
#include "sba_kernels.hpp"

namespace sba {

// One 64-key tile for the 32 queries of a wave: recompute p, beta from the K tile in LDS and
// the stick carry at the tile's newer edge, G from the V tile, then dz with the running
// prefix of G.  Emits p and dz as bf16 MFMA A-operand fragments whose contraction slots are
// keys: slot s of fragment [sb][tt] is key 32*sb + 16*tt + 8*(s/4) + 4*h + s%4 of the tile.
template <int D, bool AC, bool PROD, int KROW, int VROW>
__device__ __forceinline__ void grad_tile(const unsigned short* Ks, const unsigned short* Vs,
                                          const bf16x8 (&qf)[D / 16], const bf16x8 (&dof)[D / 16],
                                          float c, int kt, int qw0, int qrow, int n, int h,
                                          float carry_e, float& carry_c, float dr,
                                          bf16x8 (&pf)[2][2], bf16x8 (&zf)[2][2], bool (&live)[2]) {
  constexpr int KS = D / 16;
  float G[2][16], Bt[2][16];
#pragma unroll
  for (int sb = 1; sb >= 0; --sb) {
    const int k0 = kt * BN + 32 * sb;
    live[sb] = !sub_skip<AC>(k0, qw0);
    if (!live[sb]) {
      pf[sb][0] = zero8(); pf[sb][1] = zero8();
      zf[sb][0] = zero8(); zf[sb][1] = zero8();
      continue;
    }
    f32x16 x, da;
#pragma unroll
    for (int i = 0; i < 16; ++i) { x[i] = 0.0f; da[i] = 0.0f; }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      x = mfma32(lds_row8(Ks + (32 * sb + n) * KROW + 16 * ks + 8 * h), qf[ks], x);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      da = mfma32(lds_row8(Vs + (32 * sb + n) * VROW + 16 * ks + 8 * h), dof[ks], da);
    }
    float p[16];
    if (sub_full<AC>(k0, qw0)) {
      stick_weights<AC, PROD, false, true>(x, c, k0, qrow, h, carry_e, p, Bt[sb]);
    } else {
      stick_weights<AC, PROD, true, true>(x, c, k0, qrow, h, carry_e, p, Bt[sb]);
    }
    pf[sb][0] = pack8(p);
    pf[sb][1] = pack8(p + 8);
#pragma unroll
    for (int i = 0; i < 16; ++i) G[sb][i] = p[i] * (da[i] - dr);
  }
#pragma unroll
  for (int sb = 0; sb < 2; ++sb) {
    if (!live[sb]) continue;
    float cs[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) cs[i] = G[sb][i];
    const float total = prefix_sum32(cs, h, carry_c);
    float dz[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) dz[i] = G[sb][i] - Bt[sb][i] * cs[i];
    carry_c += total;
    zf[sb][0] = pack8(dz);
    zf[sb][1] = pack8(dz + 8);
  }
}

// -------------------------------------------------------------------------------------------
// dq pass
// -------------------------------------------------------------------------------------------
template <int D, bool AC, bool PROD>
__global__ void __launch_bounds__(NT, 1) bwd_dq_kernel(const KArgs a) {
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int KROW = D + 8;   // K: row reads (scores) and transpose reads (dq)
  constexpr int VROW = D + 8;   // V: row reads only
  constexpr int NCH = BN * (D / 8) / NT;
  __shared__ __attribute__((aligned(16))) unsigned short Ks[BN * KROW];
  __shared__ __attribute__((aligned(16))) unsigned short Vs[BN * VROW];

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

  bf16x8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    qf[ks] = qvalid ? *reinterpret_cast<const bf16x8*>(qb + (int64_t)qrow * a.q.st + 16 * ks + 8 * h) : zero8();
    dof[ks] = qvalid ? *reinterpret_cast<const bf16x8*>(gob + (int64_t)qrow * a.go.st + 16 * ks + 8 * h) : zero8();
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
  const int ktr = (4 * h + (i16 >> 2)) * KROW + 16 * blk + 4 * (i16 & 3);

  uint4 kreg[NCH], vreg[NCH];
  load_rows_to_regs<D, BN, KROW>(kb, a.k.st, 0, t.doc_len, kreg);
  load_rows_to_regs<D, BN, VROW>(vb, a.v.st, 0, t.doc_len, vreg);

  for (int kt = 0; kt <= kt_last; ++kt) {
    __syncthreads();
    store_regs_to_lds<D, BN, KROW>(Ks, kreg);
    store_regs_to_lds<D, BN, VROW>(Vs, vreg);
    __syncthreads();
    if (kt < kt_last) {
      load_rows_to_regs<D, BN, KROW>(kb, a.k.st, (kt + 1) * BN, t.doc_len, kreg);
      load_rows_to_regs<D, BN, VROW>(vb, a.v.st, (kt + 1) * BN, t.doc_len, vreg);
    }
    const int64_t tix = ((int64_t)head * a.n_tt + kt) * a.rows_total + grow;
    float carry_e = PROD ? 1.0f : 0.0f;
    if (qvalid) {
      carry_e = a.stick[tix];
      if (h == 0) a.gtab[tix] = carry_c;
    }
    bf16x8 pf[2][2], zf[2][2];
    bool live[2];
    grad_tile<D, AC, PROD, KROW, VROW>(Ks, Vs, qf, dof, a.c, kt, qw0, qrow, n, h, carry_e, carry_c, dr,
                                       pf, zf, live);
    // dq += dz . K  (K as the B operand: transpose reads along keys)
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      if (!live[sb]) continue;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const unsigned short* krow = Ks + ktr + (32 * sb + 16 * tt) * KROW;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const bf16x8 kf = lds_tr8(krow + 32 * db, krow + 8 * KROW + 32 * db);
          dqacc[db] = mfma32(zf[sb][tt], kf, dqacc[db]);
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
// dk / dv pass
// -------------------------------------------------------------------------------------------
template <int D, bool AC, bool PROD>
__global__ void __launch_bounds__(NT, 1) bwd_dkdv_kernel(const KArgs a) {
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int KROW = D + 8;    // K, V: row reads only
  constexpr int QROW = D + 8;    // Q, dO: row reads (operands of the score products) and
                                 // transpose reads (operands of dk / dv)
  constexpr int PROW = BN + 4;   // p / dz staged [query][key]: 8-byte row writes, transpose reads
  constexpr int NCHK = BN * (D / 8) / NT;
  constexpr int NCHQ = BM * (D / 8) / NT;
  __shared__ __attribute__((aligned(16))) unsigned short Ks[BN * KROW];
  __shared__ __attribute__((aligned(16))) unsigned short Vs[BN * KROW];
  __shared__ __attribute__((aligned(16))) unsigned short Qs[BM * QROW];
  __shared__ __attribute__((aligned(16))) unsigned short Gs[BM * QROW];
  __shared__ __attribute__((aligned(16))) unsigned short Ps[BM * PROW];
  __shared__ __attribute__((aligned(16))) unsigned short Zs[BM * PROW];

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

  const int64_t tok0 = t.tok_start;
  const __bf16* qb = reinterpret_cast<const __bf16*>(a.q.ptr) + t.batch * a.q.sb + head * a.q.sh + tok0 * a.q.st;
  const __bf16* kb = reinterpret_cast<const __bf16*>(a.k.ptr) + t.batch * a.k.sb + head * a.k.sh + tok0 * a.k.st;
  const __bf16* vb = reinterpret_cast<const __bf16*>(a.v.ptr) + t.batch * a.v.sb + head * a.v.sh + tok0 * a.v.st;
  const __bf16* gob = reinterpret_cast<const __bf16*>(a.go.ptr) + t.batch * a.go.sb + head * a.go.sh + tok0 * a.go.st;
  const __bf16* grb = a.grem.ptr == nullptr ? nullptr
      : reinterpret_cast<const __bf16*>(a.grem.ptr) + t.batch * a.grem.sb + head * a.grem.sh + tok0 * a.grem.st;

  {
    uint4 kreg[NCHK], vreg[NCHK];
    load_rows_to_regs<D, BN, KROW>(kb, a.k.st, kt * BN, t.doc_len, kreg);
    load_rows_to_regs<D, BN, KROW>(vb, a.v.st, kt * BN, t.doc_len, vreg);
    store_regs_to_lds<D, BN, KROW>(Ks, kreg);
    store_regs_to_lds<D, BN, KROW>(Vs, vreg);
  }

  // Output ownership: waves 0,1 accumulate dv, waves 2,3 dk; each owns 32 keys x D.
  const int mat = w >> 1, kb32 = w & 1;
  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.0f;

  const unsigned short* Xs = mat ? Zs : Ps;   // dz^T or p^T as the A operand
  const unsigned short* Ys = mat ? Qs : Gs;   // Q or dO as the B operand
  const int xtr = (8 * h + (i16 >> 2)) * PROW + 32 * kb32 + 16 * blk + 4 * (i16 & 3);
  const int ytr = (8 * h + (i16 >> 2)) * QROW + 16 * blk + 4 * (i16 & 3);

  const int qt_first = (kt * BN) / BM;
  const int qt_last = (t.doc_len - 1) / BM;
  for (int qt = qt_first; qt <= qt_last; ++qt) {
    const int m0 = qt * BM;
    __syncthreads();   // previous step's dk/dv products have consumed Qs, Gs, Ps, Zs
    {
      uint4 qreg[NCHQ];
      load_rows_to_regs<D, BM, QROW>(qb, a.q.st, m0, t.doc_len, qreg);
      store_regs_to_lds<D, BM, QROW>(Qs, qreg);
      load_rows_to_regs<D, BM, QROW>(gob, a.go.st, m0, t.doc_len, qreg);
      store_regs_to_lds<D, BM, QROW>(Gs, qreg);
    }
    __syncthreads();

    const int qw0 = m0 + 32 * w;
    const int qrow = qw0 + n;
    const bool qvalid = qrow < t.doc_len;
    bf16x8 qf[KS], dof[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = lds_row8(Qs + (32 * w + n) * QROW + 16 * ks + 8 * h);
      dof[ks] = lds_row8(Gs + (32 * w + n) * QROW + 16 * ks + 8 * h);
    }
    float carry_e = PROD ? 1.0f : 0.0f, carry_c = 0.0f, dr = 0.0f;
    if (qvalid) {
      const int64_t grow = (int64_t)t.batch * a.tokens + tok0 + qrow;
      const int64_t tix = ((int64_t)head * a.n_tt + kt) * a.rows_total + grow;
      carry_e = a.stick[tix];
      carry_c = a.gtab[tix];
      if (grb != nullptr) dr = (float)grb[(int64_t)qrow * a.grem.st];
    }
    bf16x8 pf[2][2], zf[2][2];
    bool live[2];
    grad_tile<D, AC, PROD, KROW, KROW>(Ks, Vs, qf, dof, a.c, kt, qw0, qrow, n, h, carry_e, carry_c, dr,
                                       pf, zf, live);
    // stage p and dz as [query][key]: each half fragment is 4 consecutive keys = 8 bytes
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const int col = 32 * sb + 16 * tt + 4 * h;
        const uint4 pv = __builtin_bit_cast(uint4, pf[sb][tt]);
        const uint4 zv = __builtin_bit_cast(uint4, zf[sb][tt]);
        unsigned short* prow = Ps + (32 * w + n) * PROW + col;
        unsigned short* zrow = Zs + (32 * w + n) * PROW + col;
        *reinterpret_cast<uint2*>(prow) = make_uint2(pv.x, pv.y);
        *reinterpret_cast<uint2*>(prow + 8) = make_uint2(pv.z, pv.w);
        *reinterpret_cast<uint2*>(zrow) = make_uint2(zv.x, zv.y);
        *reinterpret_cast<uint2*>(zrow + 8) = make_uint2(zv.z, zv.w);
      }
    }
    __syncthreads();
    // acc[key, d] += sum over the 128 queries of X[query][key] * Y[query][d]
#pragma unroll
    for (int ks = 0; ks < BM / 16; ++ks) {
      const unsigned short* xr = Xs + xtr + 16 * ks * PROW;
      const bf16x8 af = lds_tr8(xr, xr + 4 * PROW);
      const unsigned short* yr = Ys + ytr + 16 * ks * QROW;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16x8 bf = lds_tr8(yr + 32 * db, yr + 4 * QROW + 32 * db);
        acc[db] = mfma32(af, bf, acc[db]);
      }
    }
  }

  const View& ov = mat ? a.dk : a.dv;
  __bf16* outb = reinterpret_cast<__bf16*>(ov.ptr) + t.batch * ov.sb + head * ov.sh + tok0 * ov.st;
  const float scale = mat ? a.inv_temp : 1.0f;
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kt * BN + 32 * kb32 + 8 * (i >> 2) + 4 * h + (i & 3);
      if (key < t.doc_len) outb[(int64_t)key * ov.st + 32 * db + n] = (__bf16)(acc[db][i] * scale);
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
  const dim3 grid((unsigned)n_kv_max * (unsigned)a.heads), block(NT);
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
