/*
 * sba.h -- C ABI of libsba.so: stick-breaking attention for AMD Instinct MI355X (gfx950).
 *
 * Plain C, no torch types.  Every pointer is a DEVICE pointer unless stated otherwise; the
 * library never allocates, frees or synchronises: outputs and workspaces are owned by the
 * caller and all work is enqueued on the HIP stream handed in (a `hipStream_t` passed as
 * `void*`; NULL = the null stream).  Return value: 0 = ok, negative = SBA_E_* (bad argument,
 * nothing launched), positive = a hipError_t raised by a launch.
 *
 * The entry points replace the host launchers of the upstream Python package
 * (paths relative to the upstream repository root):
 *
 *   sba_varlen_fwd  <->  varlen_fwd / _compileable_forward
 *                        stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:413-522
 *   sba_varlen_bwd  <->  varlen_bwd / _compileable_backward
 *                        stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:484-641
 *   sba_attn_fwd    <->  _fwd / _compileable_fwd
 *                        stickbreaking_attention/sb_attn/sb_fwd.py:139-253
 *   sba_attn_bwd    <->  _bwd / _compileable_backward
 *                        stickbreaking_attention/sb_attn/sb_bwd.py:163-297
 *
 * Upstream lets PyTorch allocate outputs, the saved per-row statistic and the lock/count
 * workspaces and passes raw pointers plus explicit strides to the kernels; this ABI keeps
 * that ownership model.  What differs is the private state carried from forward to
 * backward: instead of one fp32 log-remainder per row (upstream `neg_log_acc`) the forward
 * fills a per-(row, 32-key block) carry table that both backward kernels consume, so the
 * backward needs neither locks nor atomics.  Every workspace is passed with its size in bytes;
 * an entry point never reads or writes past a size it was given: what the host can check comes
 * back as SBA_E_WORKSPACE, what only the device can know (the documents inside cu_seqlens) makes
 * the kernels return early and the outputs NaN.
 */
#ifndef SBA_H_
#define SBA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SBA_VERSION 213

/* error codes (negative returns) */
#define SBA_E_NULL      (-1)  /* a required pointer is NULL                         */
#define SBA_E_HEAD_DIM  (-2)  /* head_dim not in {32, 64, 128, 256}                 */
#define SBA_E_DTYPE     (-3)  /* dtype neither SBA_BF16 nor SBA_F16                 */
#define SBA_E_SHAPE     (-4)  /* negative / inconsistent sizes, or tokens*stride_t
                                 too large for 32-bit byte offsets (>= 2 GiB)       */
#define SBA_E_STRIDE    (-5)  /* a row start is not 16-byte aligned (stride % 8)    */
#define SBA_E_WORKSPACE (-6)  /* a workspace handed in is smaller than the problem
                                 needs: schedule, weights array, the tables of the
                                 fixed-length op, the static array of
                                 sba_varlen_fwd_static                              */
#define SBA_E_ARCH      (-7)  /* current device is not gfx950                       */

/* element types of q, k, v, grad_o, grad_rem and of every output (one type per call); the
 * matrix products run on the MFMA instruction of that type with fp32 accumulation */
#define SBA_BF16 1
#define SBA_F16  2

/* flags */
#define SBA_ATTEND_CURRENT 1u   /* a token may attend to itself (upstream attend_current) */
#define SBA_CU_INT64       2u   /* cu_seqlens holds int64 (else int32)                    */
#define SBA_FIXED_LENGTH   8u   /* the problem is the fixed-length op: `batch` documents of
                                   `tokens` tokens each, cu_seqlens ignored (sba_attn_*)   */
#define SBA_PRODUCT_SPACE  4u   /* carry the stick as a running product instead of a
                                   running log2 sum (same results to ~1e-6, fewer
                                   transcendentals); must match between fwd and bwd       */
#define SBA_FUSE_REMAINDER 16u  /* fold in what every upstream caller does next with the two
                                   outputs (tests/test_varlen.py:101, tests/test_attn.py:64):
                                   forward writes  o + rem[..., None] * v  into `o` (rem is
                                   still written); backward takes `grad_o` as the gradient
                                   of that sum and adds the terms it implies
                                   (d rem += grad_o . v per row, dv += rem * grad_o).  No
                                   upstream counterpart; must match between fwd and bwd    */
#define SBA_TABLE_ONLY     32u  /* forward entry points only: write the stick table and nothing
                                   else (v, o and rem are not looked at and may be null views;
                                   `stick_table` is required).  For a caller that kept no
                                   table between forward and backward -- the O(heads x tokens)
                                   footprint of upstream's neg_log_acc -- and rebuilds it in
                                   front of sba_*_bwd: same kernel, same bits, about 60 % of
                                   a forward's time.  No upstream counterpart             */

/* A strided view over [batch, heads, tokens, head_dim]; the last dimension is contiguous.
 * Strides are in ELEMENTS.  For packed variable-length input batch == 1 and stride_b is
 * ignored.  For per-row tensors (rem, grad_rem) the head_dim axis is absent. */
typedef struct sba_view {
  void*   ptr;
  int64_t stride_b;
  int64_t stride_h;
  int64_t stride_t;
} sba_view;

/* Problem description shared by all entry points. */
typedef struct sba_problem {
  int32_t  dtype;        /* SBA_BF16 or SBA_F16                                          */
  int32_t  head_dim;     /* 32, 64, 128 or 256                                           */
  int32_t  heads;        /* H                                                            */
  int32_t  batch;        /* B for the fixed-length op, 1 for varlen                      */
  int32_t  tokens;       /* T: tokens per batch entry (fixed) / total packed tokens      */
  int32_t  n_docs;       /* varlen: number of entries in cu_seqlens; fixed: ignored      */
  int32_t  max_doc_len;  /* upper bound on any document length (fixed: == tokens; 0 =
                            unknown, taken as `tokens`).  sba_table_bytes() sizes the
                            tables with it and the backward its launches; the device
                            checks it: a longer document makes the backward return
                            at once with NaN outputs (upstream silently drops rows
                            when its max_seqlens is too small, sb_varlen_fwd.py:478) */
  uint32_t flags;        /* SBA_ATTEND_CURRENT | SBA_CU_INT64 | SBA_PRODUCT_SPACE | ...  */
  float    inv_temp;     /* logit scale (upstream logit_scale / inv_temp)                */
  const void* cu_seqlens;/* varlen: inclusive cumulative document ends, WITHOUT a leading
                            zero (upstream strips it, sb_varlen/__init__.py:72-74)       */
} sba_problem;

/* ---- sizes ------------------------------------------------------------------------------ */

/* Bytes of the schedule workspace (tile lists + status words) for this problem. */
size_t sba_schedule_bytes(const sba_problem* p);

/* Bytes of ONE carry table.  A table holds, per head and per document of length L, one fp32 for
 * every (32-key block, query row at or below it) pair -- about L*L/64, L rounded up to a
 * multiple of 32 so that every block starts on a 128-byte line -- plus one per row (the
 * forward leaves rem there in fp32, the backward the complete gradient of rem) -- and, behind
 * all heads, 256 bytes of work counters: the dk/dv pass of a large problem is launched with one
 * workgroup per compute unit, and those workgroups draw their key tiles from counters kept at
 * the end of `grad_table` (cleared by the dq pass that precedes them; both sizes below include
 * the 256 bytes).  The forward fills `stick_table`; the backward additionally needs a
 * `grad_table` of the same size, which must not be shared by backward calls that run at the
 * same time.
 *   sba_table_bytes              no lengths needed: the most any documents of at most
 *                                max_doc_len tokens can need (exact for the fixed-length op);
 *   sba_table_bytes_for_lengths  exact, from the document lengths in HOST memory.
 * Tables may be larger than needed.  Tables that turn out too small for the documents in
 * cu_seqlens (a max_doc_len that under-states them) are detected on the device: nothing runs
 * and every output is filled with NaN (see SBA_STATUS_TABLE_TOO_SMALL). */
size_t sba_table_bytes(const sba_problem* p);
size_t sba_table_bytes_for_lengths(const sba_problem* p, const int64_t* doc_lengths, int n_lengths);

/* ---- schedule --------------------------------------------------------------------------- */

/* Builds, on the device, the list of 128-row query tiles and 128-key KV tiles from
 * cu_seqlens (documents sorted longest first, tiles of a document newest first), assigns every
 * document its area of the carry tables and validates cu_seqlens.  `schedule` must be 16-byte
 * aligned and `schedule_size` (its size in bytes) at least sba_schedule_bytes(), else
 * SBA_E_WORKSPACE.  The first int32 of the workspace is a status word (0 = ok, else
 * SBA_STATUS_*) and the fourth the number of table entries per head the documents need, both
 * readable by the caller after the stream has drained (the seventh: the longest document found).
 * Has no upstream counterpart as a
 * separate call: upstream derives the tile of a program from its grid index inside `_forward`
 * (sb_varlen_fwd.py:281-296). */
int sba_build_schedule(const sba_problem* p, void* schedule, size_t schedule_size, void* stream);

#define SBA_STATUS_OK               0
#define SBA_STATUS_BAD_CU           1   /* cu_seqlens not monotone or beyond `tokens`        */
#define SBA_STATUS_TABLE_TOO_SMALL  4   /* reported by the Python layer when the fourth header
                                           word exceeds the entries per head of the tables   */
#define SBA_STATUS_DOC_TOO_LONG     5   /* likewise when the seventh header word (the longest
                                           document found) exceeds max_doc_len               */

/* ---- forward ---------------------------------------------------------------------------- */

/* o[b,h,t,:] and rem[b,h,t] for every token: tokens that belong to no document (past the
 * last entry of cu_seqlens) are set to zero.  When the scheduler rejected cu_seqlens, or
 * `stick_table` is too small for the documents, no attention is computed and every element of
 * both outputs is NaN.  `stick_table` (`table_size` bytes) may be NULL when no backward will
 * follow.  `schedule_size` is checked against sba_schedule_bytes(). */
int sba_varlen_fwd(const sba_problem* p, const void* schedule, size_t schedule_size,
                   const sba_view* q, const sba_view* k, const sba_view* v,
                   const sba_view* o, const sba_view* rem,
                   float* stick_table, size_t table_size, void* stream);

int sba_attn_fwd(const sba_problem* p, const void* schedule, size_t schedule_size,
                 const sba_view* q, const sba_view* k, const sba_view* v,
                 const sba_view* o, const sba_view* rem,
                 float* stick_table, size_t table_size, void* stream);

/* Debug variants that additionally write the attention weights A[i,j] (fp32, before the bf16
 * rounding that feeds A.V) of every causal in-document pair into `weights`, a dense
 * [batch][heads][tokens][tokens] array of `weights_size` bytes (row = query token, column = key
 * token; packed variable-length input: batch == 1 and both indices are positions in the packed
 * sequence).  Elements outside the causal triangle of a document are not written: clear the
 * array first.  Replaces upstream's `return_attention=True` launches (sb_varlen_fwd.py:195-202,
 * :421-425; sb_attn/sb_fwd.py:147-151).  Quadratic memory; a separate, slower kernel
 * instantiation. */
int sba_varlen_fwd_weights(const sba_problem* p, const void* schedule, size_t schedule_size,
                           const sba_view* q, const sba_view* k, const sba_view* v,
                           const sba_view* o, const sba_view* rem,
                           float* stick_table, size_t table_size,
                           float* weights, size_t weights_size, void* stream);

int sba_attn_fwd_weights(const sba_problem* p, const void* schedule, size_t schedule_size,
                         const sba_view* q, const sba_view* k, const sba_view* v,
                         const sba_view* o, const sba_view* rem,
                         float* stick_table, size_t table_size,
                         float* weights, size_t weights_size, void* stream);

/* Forward of packed variable-length input for callers that cannot allocate device memory (code
 * running under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart upstream, where PyTorch allocates every buffer.  Same results as
 * sba_build_schedule + sba_varlen_fwd with stick_table == NULL (no backward can follow), but the
 * schedule workspace is a fixed array of SBA_STATIC_SCRATCH_BYTES bytes that lives inside the
 * library's code object on every GPU it runs on, from the first call until the process ends; the
 * call allocates and frees nothing.  Problems whose sba_schedule_bytes() exceed that size are
 * rejected with SBA_E_WORKSPACE (the array holds, for example, 262144 tokens in 4096 documents).
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams
 * or threads) race; serialise them.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress): make that call outside any graph capture. */
#define SBA_STATIC_SCRATCH_BYTES (512 * 1024)
int sba_varlen_fwd_static(const sba_problem* p,
                          const sba_view* q, const sba_view* k, const sba_view* v,
                          const sba_view* o, const sba_view* rem, void* stream);

/* ---- backward --------------------------------------------------------------------------- */

/* dq, dk, dv for every token (zero for tokens that belong to no document; NaN everywhere when
 * nothing could run, as in the forward, or when a document is longer than max_doc_len).  `schedule` and `stick_table` are the ones the forward
 * of the same problem and inputs filled; `grad_table` is scratch; `table_size` is the size in
 * bytes of EACH of the two tables.  grad_rem may have ptr == NULL (treated as zeros). */
int sba_varlen_bwd(const sba_problem* p, const void* schedule, size_t schedule_size,
                   const sba_view* q, const sba_view* k, const sba_view* v,
                   const sba_view* grad_o, const sba_view* grad_rem,
                   const float* stick_table, float* grad_table, size_t table_size,
                   const sba_view* dq, const sba_view* dk, const sba_view* dv,
                   void* stream);

int sba_attn_bwd(const sba_problem* p, const void* schedule, size_t schedule_size,
                 const sba_view* q, const sba_view* k, const sba_view* v,
                 const sba_view* grad_o, const sba_view* grad_rem,
                 const float* stick_table, float* grad_table, size_t table_size,
                 const sba_view* dq, const sba_view* dk, const sba_view* dv,
                 void* stream);

/* ---- misc ------------------------------------------------------------------------------- */

/* Launch geometry of a problem: host arithmetic only, nothing is launched and no device is
 * looked at.  It has no counterpart upstream (Triton computes its grids inside the launchers,
 * sb_varlen_fwd.py:476-480, sb_varlen_bwd.py:511-513); it exists so that a caller, and this
 * library's own CPU tests, can check that every tile descriptor a workgroup may read lies inside
 * the schedule workspace: the compute kernels read the descriptor of their slot before they know
 * how long the lists really are.
 *   forward / dq pass: `fwd_tiles` / `dq_tiles` slots of the query-tile list (room: query_list_tiles);
 *   dk/dv pass: `dkdv_main_tiles` slots of the key-tile list from its start (room: key_list_tiles),
 *   and `dkdv_tail_tiles` workgroups per head that compare their slot with the list's true length
 *   before they read it.  `long_tiles_bound` / `tail_tiles_bound` are the bounds on the two groups
 *   of the key-tile list the grids are derived from.  Offsets and sizes are in int32 words. */
typedef struct sba_geometry {
  int query_list_tiles, key_list_tiles;
  int query_list_word, key_list_word, tile_words;
  long long schedule_words;
  int fwd_tiles, dq_tiles;
  int long_tiles_bound, tail_tiles_bound;
  int dkdv_main_tiles, dkdv_tail_tiles;
} sba_geometry;
int sba_launch_geometry(const sba_problem* p, sba_geometry* out);

int         sba_version(void);
const char* sba_error_string(int code);

/* Benchmark instrumentation, NOT part of the re-entrant interface: with the switch on, every
 * compute launch is bracketed by HIP events on the caller's stream (event creation, no waiting:
 * timed kernels follow one another on the device as untimed ones do); sba_last_kernel_ms WAITS
 * for the most recent launch of the kernel asked for and returns its duration in milliseconds
 * (which: 0 = forward, 1 = backward dq pass, 2 = backward dk/dv pass).  One process-wide switch
 * and one process-wide set of results (the backward may run on PyTorch's autograd thread): do
 * not use with concurrent callers, under graph capture, or in production.  Off by default;
 * sba_varlen_fwd_static ignores it. */
void  sba_set_timing(int on);
float sba_last_kernel_ms(int which);

/* Test and tuning switch (no counterpart upstream, process-wide like the one above): the number of
 * workgroups the main kernel of the dk/dv pass is launched with when it has more key tiles
 * (times heads) than that to work through.  n > 0: exactly n rounded down to a multiple of 8 (at
 * least 8), however few tiles there are per workgroup; n = 0 (default): one per compute unit,
 * and only for problems with at least eight tiles per workgroup; n < 0: always one workgroup per
 * tile.  The results do not depend on it (every tile is computed by the same instructions in the
 * same order whichever workgroup takes it). */
void  sba_set_dkdv_workgroups(int n);

#ifdef __cplusplus
}
#endif
#endif /* SBA_H_ */
