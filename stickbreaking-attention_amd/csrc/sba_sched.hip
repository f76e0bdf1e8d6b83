// Device-side tile scheduler: turns cu_seqlens into the tile lists the compute kernels index
// with blockIdx, without a device-to-host round trip.
//
// Upstream sizes its grid from the host-side `max_seqlens` and lets every program find its
// document from cu_seqlens, pairing a long and a short causal row of two heads per program
// (stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:281-296, :476-480).  Here documents are
// ranked longest first and each contributes exactly its own tiles, most expensive first, so
// no program is idle and the tail of the launch is made of the cheapest tiles.
#include "sba_kernels.hpp"

namespace sba {

constexpr int RANK_LIMIT = 4096;   // beyond this many documents the input order is kept

__device__ __forceinline__ int cdiv(int a, int b) { return (a + b - 1) / b; }

// Scratch (int32) behind the two tile lists, per document: start, len, order, qoff, kvoff, table base.
// SCHED_THREADS: workgroup size; a small one when there are few documents (every step of the scans
// and every phase boundary is a workgroup barrier, which costs by the wave).
template <int SCHED_THREADS>
__global__ void __launch_bounds__(SCHED_THREADS) sched_kernel(const SchedArgs a) {
  __shared__ int s_status, s_maxlen;
  __shared__ int s_scan_q[SCHED_THREADS], s_scan_kv[SCHED_THREADS], s_scan_ne[SCHED_THREADS];
  __shared__ long long s_scan_tab[SCHED_THREADS];
  // Lengths, ranking and tile-count prefixes of up to RANK_LIMIT documents are kept in LDS: the
  // ranking reads every length once per document and the tile emission searches the prefixes, and
  // with a few hundred documents those reads, taken from global memory one after the other, used to
  // be three quarters of this kernel's time.  Beyond RANK_LIMIT documents the same arrays in the
  // workspace are used.
  __shared__ int s_len[RANK_LIMIT], s_ord[RANK_LIMIT], s_qoff[RANK_LIMIT + 1], s_kvoff[RANK_LIMIT + 1];
  __shared__ int s_start[RANK_LIMIT], s_tab[RANK_LIMIT];
  const int tid = threadIdx.x;
  const int nd = a.n_docs;
  int* hdr = a.out;
  Tile* qtiles = reinterpret_cast<Tile*>(a.out + SCHED_HDR);
  Tile* kvtiles = qtiles + a.n_q_max;
  int* dstart = reinterpret_cast<int*>(kvtiles + a.n_kv_max);
  int* dlen = dstart + nd;
  int* order = dlen + nd;
  int* qoff = order + nd;         // nd + 1 entries
  int* kvoff = qoff + nd + 1;     // nd + 1 entries (key tiles of the first group)
  int* dtab = kvoff + nd + 1;     // first carry-table entry of each document (by document index)
  const bool fixed = a.cu == nullptr;
  const bool in_lds = nd <= RANK_LIMIT;
  int* const len_of = in_lds ? s_len : dlen;          // by document index
  int* const ranked = in_lds ? s_ord : order;         // rank -> document index
  int* const q_before = in_lds ? s_qoff : qoff;       // by rank: query tiles of the documents ranked before
  int* const kv_before = in_lds ? s_kvoff : kvoff;    // by rank: key tiles of the first group ranked before
  int* const start_of = in_lds ? s_start : dstart;    // by document index: first token
  int* const tab_of = in_lds ? s_tab : dtab;          // by document index: first carry-table entry

  if (tid == 0) { s_status = 0; s_maxlen = 0; }
  __syncthreads();

  // A. document bounds + validation
  for (int d = tid; d < nd; d += SCHED_THREADS) {
    long long st = 0, en = a.tokens;
    if (!fixed) {
      if (a.cu_is64) {
        const long long* cu = reinterpret_cast<const long long*>(a.cu);
        st = d ? cu[d - 1] : 0; en = cu[d];
      } else {
        const int* cu = reinterpret_cast<const int*>(a.cu);
        st = d ? cu[d - 1] : 0; en = cu[d];
      }
    }
    int len = 0;
    if (st < 0 || en < st || en > a.tokens) {
      atomicOr(&s_status, 1);   // SBA_STATUS_BAD_CU
      st = 0;
    } else {
      len = (int)(en - st);
    }
    dstart[d] = (int)st;
    if (in_lds) s_start[d] = (int)st;
    dlen[d] = len;
    if (in_lds) s_len[d] = len;
    atomicMax(&s_maxlen, len);
  }
  __syncthreads();

  // B. rank documents by length, longest first (ties by index)
  for (int d = tid; d < nd; d += SCHED_THREADS) {
    int r = d;
    if (!fixed && in_lds) {
      const int len = s_len[d];
      r = 0;
      for (int e = 0; e < nd; ++e) {
        const int le = s_len[e];
        r += (le > len) || (le == len && e < d);
      }
    }
    ranked[r] = d;
  }
  __syncthreads();

  // C. exclusive prefix of the tile counts in ranked order.  Key tiles are listed in two groups (see
  // kv_tail_tiles): first, document by document, the tiles that many queries follow; then the rest.
  // SCHED_NKV_LONG marks the boundary.
  const int per = cdiv(nd, SCHED_THREADS);
  int sq = 0, skv = 0, sne = 0;
  long long stab = 0;
  for (int j = 0; j < per; ++j) {
    const int i = tid * per + j;
    if (i < nd) {
      const int len = len_of[ranked[i]];
      sq += cdiv(len, BM);
      skv += cdiv(len, BKV) - kv_tail_tiles(len);
      sne += kv_tail_tiles(len);
      stab += tab_doc_entries(len);
    }
  }
  s_scan_q[tid] = sq;
  s_scan_kv[tid] = skv;
  s_scan_ne[tid] = sne;
  s_scan_tab[tid] = stab;
  __syncthreads();
  for (int off = 1; off < SCHED_THREADS; off <<= 1) {
    int vq = 0, vkv = 0, vne = 0;
    long long vtab = 0;
    if (tid >= off) { vq = s_scan_q[tid - off]; vkv = s_scan_kv[tid - off]; vne = s_scan_ne[tid - off]; vtab = s_scan_tab[tid - off]; }
    __syncthreads();
    s_scan_q[tid] += vq;
    s_scan_kv[tid] += vkv;
    s_scan_ne[tid] += vne;
    s_scan_tab[tid] += vtab;
    __syncthreads();
  }
  int bq = s_scan_q[tid] - sq, bkv = s_scan_kv[tid] - skv, bne = s_scan_ne[tid] - sne;
  long long btab = s_scan_tab[tid] - stab;
  const long long total_tab = s_scan_tab[SCHED_THREADS - 1];
  const int total_q = s_scan_q[SCHED_THREADS - 1], total_long = s_scan_kv[SCHED_THREADS - 1];
  const int total_kv = total_long + s_scan_ne[SCHED_THREADS - 1];
  // a document's table base must fit an int32 tile field; larger totals are reported through the
  // saturated header word and refused by every kernel that uses a table
  const bool tab_ok = total_tab <= 0x7fffffffll;
  const bool ok = s_status == 0;
  for (int j = 0; j < per; ++j) {
    const int i = tid * per + j;
    if (i < nd) {
      const int d = ranked[i];
      const int len = len_of[d];
      q_before[i] = bq; kv_before[i] = bkv;
      tab_of[d] = tab_ok ? (int)btab : 0;
      if (ok) {              // the document's last key tiles, in the second group (the older one first: more steps)
        const int nkv = cdiv(len, BKV), ntail = kv_tail_tiles(len);
        for (int j2 = 0; j2 < ntail; ++j2) {
          Tile t;
          t.tok_start = fixed ? 0 : start_of[d];
          t.doc_len = len;
          t.idx = nkv - ntail + j2;
          t.batch = fixed ? d : 0;
          t.tab_base = tab_ok ? (int)btab : 0;
          t.rsv[0] = t.rsv[1] = t.rsv[2] = 0;
          kvtiles[total_long + bne + j2] = t;
        }
      }
      bq += cdiv(len, BM);
      bkv += cdiv(len, BKV) - kv_tail_tiles(len);
      bne += kv_tail_tiles(len);
      btab += tab_doc_entries(len);
    }
  }
  if (tid == 0) { q_before[nd] = total_q; kv_before[nd] = total_long; }
  __syncthreads();

  // D. emit tiles: slot -> ranked document by binary search over the prefix
  // The hardware deals workgroups to the CUs round-robin in launch order (workgroups i and
  // i + number of CUs start on the same CU and run side by side), and hands out the rest as
  // slots free up.  Equal-length documents are therefore listed tile-major, the most expensive
  // tile of every document first: all expensive tiles start at once and the cheap ones fill
  // in behind them.  (Document-major order would put the same tile of every batch entry on
  // the same CU.)  Packed documents of different lengths stay document-major, which keeps the
  // K/V rows a workgroup's neighbours read in the caches.
  for (int s = tid; s < total_q && ok; s += SCHED_THREADS) {
    int d, within;   // document, position among its tiles in cost order
    if (fixed) {
      d = s % nd;
      within = s / nd;
    } else {
      int lo = 0, hi = nd;   // largest i with qoff[i] <= s
      while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (q_before[mid] <= s) lo = mid; else hi = mid; }
      d = ranked[lo];
      within = s - q_before[lo];
    }
    const int nq = cdiv(len_of[d], BM);
    Tile t;
    t.tok_start = fixed ? 0 : start_of[d];
    t.doc_len = len_of[d];
    t.idx = nq - 1 - within;             // newest (most expensive) query tile first
    t.batch = fixed ? d : 0;
    t.tab_base = tab_of[d];
    t.rsv[0] = t.rsv[1] = t.rsv[2] = 0;
    qtiles[s] = t;
  }
  // Key tiles stay document-major for every input: one workgroup per CU runs at a time, so the
  // hardware hands them out one by one as CUs free up, and neighbours that share a document
  // share its Q and dO rows in the caches.
  for (int s = tid; s < total_long && ok; s += SCHED_THREADS) {
    int lo = 0, hi = nd;
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (kv_before[mid] <= s) lo = mid; else hi = mid; }
    const int d = ranked[lo];
    Tile t;
    t.tok_start = fixed ? 0 : start_of[d];
    t.doc_len = len_of[d];
    t.idx = s - kv_before[lo];               // oldest keys are seen by the most queries: first
    t.batch = fixed ? d : 0;
    t.tab_base = tab_of[d];
    t.rsv[0] = t.rsv[1] = t.rsv[2] = 0;
    kvtiles[s] = t;
  }
  if (tid == 0) {
    hdr[SCHED_STATUS] = s_status;
    hdr[SCHED_NQ] = ok ? total_q : 0;
    hdr[SCHED_NKV] = ok ? total_kv : 0;
    hdr[SCHED_NKV_LONG] = ok ? total_long : 0;
    hdr[SCHED_MAXLEN] = s_maxlen;
    hdr[SCHED_TABLE] = tab_ok ? (int)total_tab : 0x7fffffff;
    hdr[SCHED_TOTAL] = (ok && nd > 0) ? dstart[nd - 1] + dlen[nd - 1] : 0;
  }
}

hipError_t launch_schedule(const SchedArgs& a, hipStream_t s) {
  if (a.n_docs <= 512) hipLaunchKernelGGL(sched_kernel<256>, dim3(1), dim3(256), 0, s, a);
  else hipLaunchKernelGGL(sched_kernel<1024>, dim3(1), dim3(1024), 0, s, a);
  return hipGetLastError();
}

}  // namespace sba
