/* C ABI of libsga_hip.so -- the MI355X (gfx950) kernels behind SGA's operator
 * boundary.  Plain device pointers, sizes, scalars and a hipStream_t passed
 * as void*; no allocation inside except where a function says so.  Every
 * function returns SGA_OK (0) or a negative code and never throws;
 * sga_last_error() gives the text for the calling thread.
 *
 * Each entry point names the reference interface it stands behind
 * (paths relative to wenqingqian/SGA).
 */
#ifndef SGA_HIP_H_
#define SGA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SGA_OK 0
#define SGA_ERR_ARG (-1)
#define SGA_ERR_LAUNCH (-2)
#define SGA_ERR_WORKSPACE (-3)

#define SGA_F32 0
#define SGA_BF16 1

/* score ids: sga/plugins/optimizer/adamw.py:75-80 (_TRITON_SCORE_MAP) */
#define SGA_SCORE_UPDATE 0
#define SGA_SCORE_ABS_G 1
#define SGA_SCORE_ABS_M 2
#define SGA_SCORE_COI 3
/* Two benchmark scores with NO counterpart in the reference's registry
 * (scores.py:93-116), accepted by the fused step and the replay re-selection
 * only: the residual-blind |g| (the recorded gradient alone ranks, while the
 * residual keeps accumulating) and the literal |g + r| / sqrt(v + eps). */
#define SGA_SCORE_ABS_G_BLIND 4
#define SGA_SCORE_GR_OVER_SQRT_V 5

/* grad-correct flags: constexprs of _grad_correct_kernel, adamw.py:88-106 */
#define SGA_GC_HAS_MASK 1
#define SGA_GC_APPLY_COEFF 2
#define SGA_GC_CLEAR 4
#define SGA_GC_FOLD 8
#define SGA_GC_LR_SPLIT 16
#define SGA_GC_ADAMS 32

/* tie semantics of the exact select */
#define SGA_TIE_ALL 0          /* |s| >= thresh, count >= k  (_histogram.py:194-200) */
#define SGA_TIE_LOWEST_INDEX 1 /* exactly k, ascending index (replay.py:559-572)    */

/* replay commit flags: constexprs of _k_adam, replay_kernels.py:163-168 */
#define SGA_RP_HAS_LAB 1
#define SGA_RP_ADAMS 2
#define SGA_RP_SPLIT 4

int sga_version(void);
const char* sga_last_error(void);

/* Per-segment hyper-parameters of a flat bucket (one ParamRecord each:
 * sga/plugins/optimizer/__init__.py:20-60).  All floats are the fp32
 * roundings of the Python doubles; om1 = f32(1-beta1), bc = f32(1-beta^step). */
typedef struct sga_segment {
  int64_t start;
  int64_t n;
  float lr, beta1, om1, beta2, om2, eps, wd, bc1, bc2;
  float pad_;
} sga_segment;

/* Result block written on the device by the select entry points. */
typedef struct sga_select_result {
  uint32_t thresh_bits; /* fp32 pattern of the k-th largest |score|        */
  uint32_t need;        /* ties to take at thresh (lowest index first)     */
  uint32_t n_gt;        /* count of |score| >  thresh                      */
  uint32_t n_eq;        /* count of |score| == thresh                      */
  uint32_t n_selected;  /* coordinates selected under the tie mode         */
  uint32_t nonfinite;   /* NaN/Inf lanes seen (selection is undefined > 0) */
  uint32_t status;      /* 0 ok; 1 k out of range; 2 fast path fell back;
                           3 single-sweep bracket missed (step invalid)    */
  uint32_t path;        /* low byte: 0 radix passes, 1 sampled bracket, 2 single
                           sweep; bit 8: an fp32 score array held a value < 0;
                           bit 9: an out-of-place single-sweep step was redone */
} sga_select_result;

/* ---- scheme-agnostic masked ops (sga/kernels.py) ------------------------ */

/* dst[idx[i]] = src[i]            -- scatter_selected, kernels.py:145-163 */
int sga_scatter_selected(float* dst, const int32_t* idx, const float* src,
                         int64_t k, int64_t n_dst, void* stream);

/* values[i] = grad[idx[i]]*factor; grad[idx[i]] = 0
 *                                 -- pack_selected, kernels.py:166-187.
 * values_dtype SGA_F32 or SGA_BF16 (round-to-nearest-even of the product). */
int sga_pack_selected(float* grad, const int32_t* idx, void* values,
                      int values_dtype, float factor, int64_t k,
                      int64_t n_grad, void* stream);

/* total[0] += sum(values^2), two-stage, fixed order
 *                 -- compact_norm_sq_contribution, kernels.py:252-268.
 * partials: workspace of sga_norm_partials(k) floats. */
int64_t sga_norm_partials(int64_t n);
int sga_compact_norm_sq(const float* values, int64_t k, float* partials,
                        float* total, void* stream);

/* Allocation-free variant of sga_compact_norm_sq.  It has no counterpart in
 * the reference (whose compact_norm_sq_contribution allocates its partials on
 * every call, kernels.py:264); it is for callers that cannot allocate device
 * memory or carry a workspace: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  The stage-1 partials live in an
 * 8 KiB array inside the library's device image, one copy per GPU, kept until
 * the process ends; the call allocates nothing and frees nothing.  Same
 * kernels, same grid and the same bits in total[0] as sga_compact_norm_sq.
 * k above SGA_NOALLOC_NORM_MAX_K is refused with SGA_ERR_ARG.  Every call on
 * a GPU shares that GPU's array: calls that overlap on one GPU (two streams,
 * two host threads) race; serialise them.  Nothing in the array has to be
 * cleared between calls (each call overwrites the slots it reads).  The first
 * call on a device looks the array's address up (hipGetSymbolAddress): make
 * it before a graph capture starts. */
#define SGA_NOALLOC_NORM_MAX_K 2147483647ll
int sga_compact_norm_sq_noalloc(const float* values, int64_t k, float* total,
                                void* stream);

/* total[0] += sum(grad[mask]^2)
 *                 -- masked_norm_sq_contribution, kernels.py:284-302.
 * Deterministic two-stage reduction (the reference uses a float atomic). */
int sga_masked_norm_sq(const float* grad, const uint8_t* mask, int64_t n,
                       float* partials, float* total, void* stream);

/* grad[i] *= coeff where mask[i] != 0 (mask NULL: everywhere) -- the explicit
 * clip scale of the masked clip service, engine.py:1172-1216
 * (`grad.mul_(coeff)`, `grad.view(-1)[m > 0] *= coeff`). */
int sga_scale_masked(float* grad, const uint8_t* mask, int64_t n, float coeff,
                     void* stream);

/* block gather / scatter  -- gather_selected_blocks / scatter_selected_blocks,
 * kernels.py:190-249 */
int sga_gather_selected_blocks(const float* grad, const uint8_t* mask,
                               const int32_t* block_idx, float* values,
                               int64_t kb, int x, float factor, int64_t n_grad,
                               void* stream);
int sga_scatter_selected_blocks(float* dst, const uint8_t* mask,
                                const int32_t* block_idx, const float* src,
                                int64_t kb, int x, int64_t n_dst, void* stream);

/* Block-granular selection helpers (x a power of two in [1, 1024]).
 * sga_block_reduce: out[b] = mean (mode 0) or max (mode 1) of |g| over the
 *   b-th x-element block of one view, tail block over its real length
 *   (_block_reduce_views, selection/_histogram.py:219-251).
 * sga_block_any: any_out[b] = block b of the span has a set mask byte
 *   (block_idx_from_mask, support.py:102-142).
 * sga_expand_blocks: out[i] = bmask[i / x], i < n
 *   (bm.repeat_interleave(x)[:n], _histogram.py:303-306). */
int sga_block_reduce(const float* g, int64_t n, int x, int mode, float* out,
                     void* stream);
int sga_block_any(const uint8_t* mask, int64_t n, int x, uint8_t* any_out,
                  void* stream);
int sga_expand_blocks(const uint8_t* bmask, int x, int64_t n, uint8_t* out,
                      void* stream);

/* ---- support: mask -> sorted int32 idx (sga/support.py:57-99) ----------- */

/* Phase 1: per-chunk set-byte counts + total.  chunk_counts has
 * sga_mask_chunks(n) uint32 entries and is turned into exclusive offsets;
 * total[0] (device, int64) receives k. */
int64_t sga_mask_chunks(int64_t n);
int sga_mask_count(const uint8_t* mask, int64_t n, uint32_t* chunk_counts,
                   int64_t* total, void* stream);
/* Phase 2: idx_out[..k) = ascending positions of the non-zero bytes. */
int sga_mask_fill(const uint8_t* mask, int64_t n, const uint32_t* chunk_offsets,
                  int32_t* idx_out, int64_t idx_capacity, void* stream);

/* ---- residual-aware AdamW (sga/plugins/optimizer/adamw.py) -------------- */

/* adamw_grad_correct / _grad_correct_kernel, adamw.py:88-213, 502-634.
 * emit_mode -1 = sparse step, 0..3 = full step writing that score into g.
 * flags: SGA_GC_*.  interval is the fold divisor (fp32 division).
 * SGA_GC_ADAMS selects the AdamS tail of adams.py:87-213, 392-504 (v rebuilt
 * from the pre-commit m, no bias corrections: bc1/bc2 are ignored). */
int sga_adamw_grad_correct(float* p, float* g, float* m, float* v,
                           const uint8_t* mask, int64_t n, float lr,
                           float beta1, float om1, float beta2, float om2,
                           float eps, float wd, float bc1, float bc2,
                           float coeff, float interval, float lr_inactive,
                           int emit_mode, int flags, void* stream);

/* The same commit over many records (one per parameter tensor) in ONE launch:
 * what SgaAdamW's per-record loop (adamw.py:869-905) issues as one kernel per
 * record.  recs: DEVICE table of n_recs records ordered by first_span; record
 * r covers spans [first_span, first_span + ceil(n / 4096)), total_spans is the
 * sum.  flags are per record (SGA_GC_*; a record without a mask carries none
 * of HAS_MASK / APPLY_COEFF / CLEAR / FOLD / LR_SPLIT), with the same legality
 * rules as sga_adamw_grad_correct -- checked by the host wrapper, the table
 * being device memory.  bc1 / bc2 must be 1 for SGA_GC_ADAMS records. */
typedef struct sga_gc_record {
  float* p;
  float* g;
  float* m;
  float* v;
  const uint8_t* mask;     /* NULL when the record has no mask */
  int64_t n;
  int64_t first_span;
  float lr, beta1, om1, beta2, om2, eps, wd, bc1, bc2, lr_inactive;
  int flags;
  int pad_;
} sga_gc_record;
int sga_adamw_grad_correct_multi(const sga_gc_record* recs, int n_recs,
                                 int64_t total_spans, float coeff,
                                 float interval, int emit_mode, void* stream);

/* adamw_grad_correct_compact, adamw.py:217-322, 637-792: the commit reads its
 * gradient from the bucket-level sorted (idx, values) by merge-join.
 * flags: SGA_GC_APPLY_COEFF | SGA_GC_FOLD | SGA_GC_ADAMS (adams.py:507-654).
 * dir_table may be NULL. */
int sga_adamw_grad_correct_compact(float* p, float* g, float* m, float* v,
                                   const int32_t* idx, const void* values,
                                   int values_dtype, int64_t rec_start,
                                   int64_t n, int64_t k_total, float lr,
                                   float beta1, float om1, float beta2,
                                   float om2, float eps, float wd, float bc1,
                                   float bc2, float coeff, float interval,
                                   int flags, const int32_t* dir_table,
                                   int64_t n_table, void* stream);

/* The compact commit over many records in ONE launch (the per-record loop of
 * adamw.py:907-947).  recs: DEVICE table ordered by first_span; idx / values /
 * table / k_total / n_table are the record's bucket's; flags:
 * SGA_GC_APPLY_COEFF | SGA_GC_FOLD | SGA_GC_ADAMS per record; every record's
 * values have the dtype values_dtype. */
typedef struct sga_gcc_record {
  float* p;
  float* g;
  float* m;
  float* v;
  const int32_t* idx;
  const void* values;
  const int32_t* table;    /* directory table or NULL */
  int64_t rec_start, n, k_total, n_table, first_span;
  float lr, beta1, om1, beta2, om2, eps, wd, bc1, bc2;
  int flags;
} sga_gcc_record;
int sga_adamw_grad_correct_compact_multi(const sga_gcc_record* recs, int n_recs,
                                         int64_t total_spans, int values_dtype,
                                         float coeff, float interval,
                                         void* stream);

/* build_dir_table, adamw.py:325-349, 472-499:
 * table[j] = lower_bound(idx, j*1024), j < n_table. */
int sga_build_dir_table(const int32_t* idx, int64_t k, int32_t* table,
                        int64_t n_table, void* stream);

/* ---- exact top-k selection --------------------------------------------- */

/* Workspace for every select entry point over n elements. */
size_t sga_select_workspace_bytes(int64_t n);

/* select_topk_flat / shard_select (replay.py:538-572, replay_fused.py:290-402)
 * and select_masks_histogram(mode="exact") (_histogram.py:161-201) on one
 * contiguous fp32 score array (sign is stripped).  Writes mask_out[n] (0/1)
 * and *result (device).  Runs entirely on the stream, no host sync. */
int sga_select_topk(const float* score, int64_t n, int64_t k, int tie_mode,
                    uint8_t* mask_out, sga_select_result* result, void* ws,
                    size_t ws_bytes, void* stream);

/* The same select over several disjoint runs (the online plugin's per-param
 * views, _histogram.py:97-112): begin, then per radix level one hist call per
 * run followed by one scan; then count per run, tile scan, mask per run.
 * tile_base is the run's first chunk index: runs are laid out back to back
 * in chunk space, each starting on a fresh 1024-element chunk. */
int sga_sel_begin(int64_t k, void* ws, size_t ws_bytes, void* stream);
int sga_sel_hist(const float* score, int64_t n, int level, void* ws,
                 size_t ws_bytes, void* stream);
int sga_sel_scan(int level, void* ws, size_t ws_bytes, void* stream);
int sga_sel_count(const float* score, int64_t n, int64_t tile_base, void* ws,
                  size_t ws_bytes, void* stream);
int sga_sel_tile_scan(int64_t n_tiles, int tie_mode, void* ws, size_t ws_bytes,
                      void* stream);
int sga_sel_mask(const float* score, int64_t n, int64_t tile_base,
                 int tie_mode, uint8_t* mask_out, void* ws, size_t ws_bytes,
                 void* stream);
int sga_sel_result(sga_select_result* result, void* ws, size_t ws_bytes,
                   void* stream);

/* Balanced / fast histogram select (_histogram.py:115-123, 203-216): the
 * histogram over a stride subsample, mask = top-bits >= crossing bin.
 * hist is int64[nbins] on the device and is ACCUMULATED into. */
int sga_hist_topbits(const float* score, int64_t n, int shift, int stride,
                     int phase, int64_t* hist, int nbins, uint32_t* nonfinite,
                     void* stream);
int sga_mask_topbits_ge(const float* score, int64_t n, int shift, int32_t bin,
                        uint8_t* mask_out, void* stream);

/* Adaptive-tau threshold mask (_adaptive.py:44-66): mask = |score| >= tau,
 * count[0] (device int64, may be NULL) += number of set bytes. */
int sga_mask_abs_ge(const float* score, int64_t n, float tau, uint8_t* mask_out,
                    int64_t* count, void* stream);

/* replay_kernels.py:372-414 building blocks with the same outputs. */
int sga_cand_extract_count(const float* score, int64_t n, int32_t bin,
                           uint32_t* chunk_counts, int64_t* total,
                           void* stream);
int sga_cand_extract_fill(const float* score, int64_t n, int32_t bin,
                          const uint32_t* chunk_offsets, float* cand,
                          int64_t cand_capacity, void* stream);
int sga_gt_eq(const float* score, int64_t n, float thresh, uint8_t* gt,
              uint8_t* eq, int32_t* counts2, void* stream);

/* ---- score formulas and replay commit (sga/replay_kernels.py) ----------- */

/* formula(name): out = score(w,m,v,g); absolute != 0 stores |score|.
 * scores.py:147-269 / replay_kernels.py:109-160.  flags: SGA_SF_ADAMS
 * substitutes v := m*m and bc := 1 (replay.py:486-505); SGA_SF_NO_WD leaves
 * the wd*w term of `update` out altogether (update_includes_wd=False,
 * scores.py:227-230: the score is then U(g) itself, also for -0 and for
 * non-finite w). */
#define SGA_SF_ADAMS 1
#define SGA_SF_NO_WD 2
int sga_score_formula(int score_id, const float* w, const float* m,
                      const float* v, const float* g, float* out, int64_t n,
                      float beta1, float om1, float beta2, float om2, float wd,
                      float bc1, float bc2, float eps, int absolute, int flags,
                      void* stream);

/* Branch-point score of the replay front select (replay_fused.py:1236-1265):
 * the same registry formula evaluated in double on fp32 inputs with double
 * scalars, out = fp32(|score|).  adams != 0: v := m*m, bc := 1.  include_wd
 * adds wd*w to the update score (the online cycle semantics). */
int sga_branch_score_f64(int score_id, const float* w, const float* m,
                         const float* v, const float* g, float* out, int64_t n,
                         double beta1, double beta2, double eps, double wd,
                         double bc1, double bc2, int adams, int include_wd,
                         void* stream);

/* opt_step_inplace / _k_adam, replay_kernels.py:163-216, 330-369 and
 * replay.py:674-744.  flags: SGA_RP_*. */
int sga_opt_step_inplace(const float* q, float* m, float* v, float* w,
                         float* lab, const uint8_t* inactive, int64_t n,
                         float beta1, float om1, float beta2, float om2,
                         float bc1, float bc2, float eps, float omlwd,
                         float neglr, float lr2, float lr, float lr_inactive,
                         float wd, int flags, void* stream);

/* ---- fused per-rank sparse step ----------------------------------------- */

/* One pass pair over a flat bucket: buf = resid + g; score; exact top-k
 * (lowest-index ties); idx/values pack; resid <- buf with selected coords
 * zeroed; sparse AdamW commit on p/m/v (engine order: engine.py:416-604,
 * pack kernels.py:166-187, commit adamw.py:637-724).
 * g_dtype / values_dtype: SGA_F32 | SGA_BF16.  mask_out may be NULL.
 * g may be NULL with g_dtype SGA_F32: resid then ALREADY holds g + r, the
 * reference's own buffer contract (backward accumulates into the buffer that
 * keeps the residual and the engine hands that buffer to the pack,
 * engine.py:453-470); nothing is added, buf = resid bit for bit, and the step
 * reads 4 B per coordinate less.  Refused for the residual-blind score, which
 * ranks the step's own gradient.  The same holds for every entry point of
 * this section (per bucket for sga_fused_sparse_step_multi).
 * idx_out / values_out need room for k entries.  segs is a DEVICE array.
 * flags: SGA_GC_ADAMS commits (and, for update / coi, scores) with the AdamS
 * tail (adams.py:87-213, 507-654: v rebuilt from the pre-commit m, no bias
 * corrections; bc1 / bc2 of the segments are ignored); SGA_GC_FOLD divides the
 * new residual by `interval` (residual mean before a boundary, adamw.py:199-204;
 * true division like adamw_torch.py:88-91).  Any other flag is refused: the
 * dual-lr split belongs to full steps (adamw.py:570-580). */
size_t sga_fused_workspace_bytes(int64_t n);
int sga_fused_sparse_step(const void* g, int g_dtype, float* resid, float* p,
                          float* m, float* v, int64_t n, int64_t k,
                          const sga_segment* segs, int n_segs, int score_id,
                          int32_t* idx_out, void* values_out, int values_dtype,
                          uint8_t* mask_out, float factor, float coeff,
                          int fast, int flags, float interval,
                          sga_select_result* result, void* ws,
                          size_t ws_bytes, void* stream);

/* The same step for several buckets in one call -- the per-bucket online path,
 * where every bucket of the optimizer selects its own top-k (engine.py:822-890;
 * bucket layout torch_pipelined_mask.py:91-138, torch_pipelined_index.py:490-520).
 * The buckets share dtypes, score and knobs; each has its own tensors, k,
 * segment table, outputs, result block and workspace
 * (sga_fused_workspace_bytes(n) bytes, 16-byte aligned, distinct per bucket).
 * Outputs are bucket by bucket what sga_fused_sparse_step gives.  The chain of
 * short dependent kernels around a select (sample, descents, check, candidate
 * settlement, chunk scan) runs ONCE for up to 8 buckets (the kernels take the
 * bucket from the grid's second dimension), only the data sweeps are launched
 * per bucket.  `buckets` is a HOST array, read before the call returns. */
typedef struct sga_fused_bucket {
  const void* g;
  float* resid;
  float* p;
  float* m;
  float* v;
  int64_t n;
  int64_t k;
  const sga_segment* segs;   /* DEVICE array */
  int n_segs;
  int pad_;
  int32_t* idx_out;
  void* values_out;
  uint8_t* mask_out;         /* may be NULL */
  sga_select_result* result; /* may be NULL */
  void* ws;
  size_t ws_bytes;
} sga_fused_bucket;
int sga_fused_sparse_step_multi(const sga_fused_bucket* buckets, int n_buckets,
                                int g_dtype, int score_id, int values_dtype,
                                float factor, float coeff, int fast, int flags,
                                float interval, void* stream);

/* Single-sweep variant of the fused step (no counterpart in the reference,
 * whose engine runs score, select, pack and commit as separate passes,
 * engine.py:416-604): g, resid, p, m, v are read ONCE.  The sampled bracket
 * around the k-th key is known before the sweep and decides all but a few
 * coordinates; those are committed in the sweep itself, the ones inside the
 * bracket afterwards from their records, and the pack is written in index
 * order from two bit planes.  Same arithmetic and outputs as
 * sga_fused_sparse_step whenever result->status == 0.  status == 3: the
 * bracket missed the k-th key after coordinates were committed on it -- the
 * step is then invalid and cannot be repaired (margins: 12 sigma of the
 * sample rank; `seed` moves the sample offsets so no fixed input can defeat
 * them).  Shapes the sweep does not take are done by the two-sweep step
 * behind the same call (n < 2^20, a bracket open below or too wide for the
 * candidate buffers); a plateau of equal keys inside the bracket is seen in
 * the sample BEFORE anything is committed and done by the radix passes.
 * ws: sga_fused_workspace_bytes(n); ws2: 256-byte aligned,
 * sga_fused_single_sweep_workspace_bytes(n, values_dtype) bytes (one staged
 * pack value per coordinate, 128 B of bit planes per 1024, candidate records). */
size_t sga_fused_single_sweep_workspace_bytes(int64_t n, int values_dtype);
int sga_fused_sparse_step_single_sweep(
    const void* g, int g_dtype, float* resid, float* p, float* m, float* v,
    int64_t n, int64_t k, const sga_segment* segs, int n_segs, int score_id,
    int32_t* idx_out, void* values_out, int values_dtype, uint8_t* mask_out,
    float factor, float coeff, int flags, float interval, uint32_t seed,
    sga_select_result* result, void* ws, size_t ws_bytes, void* ws2,
    size_t ws2_bytes, void* stream);
int sga_fused_sparse_step_single_sweep_packed(
    const void* g, int g_dtype, float* state, int64_t n, int64_t k,
    const sga_segment* segs, int n_segs, int score_id, int32_t* idx_out,
    void* values_out, int values_dtype, uint8_t* mask_out, float factor,
    float coeff, int flags, float interval, uint32_t seed,
    sga_select_result* result, void* ws, size_t ws_bytes, void* ws2,
    size_t ws2_bytes, void* stream);

/* Out-of-place single-sweep step (no counterpart in the reference): same
 * sweep, but the new resid / p / m / v go to OTHER arrays (ping-pong state:
 * swap the two sets after every step) and the inputs are only read.  Nothing
 * is lost when the bracket misses: the device then redoes the step from the
 * untouched inputs with the radix passes and the key-forming final sweep of
 * sga_fused_sparse_step, over whatever the sweep wrote.  result->status is 0
 * for every input (never 3), outputs equal sga_fused_sparse_step's bit for
 * bit, and bit 9 (0x200) of result->path says that the step was redone.  The
 * price is a second copy of the optimizer-side state (16 B per coordinate).
 * No output array may overlap an input or another output (refused).  The
 * packed twin takes two packed states (sga_packed_state_elems(n) floats each,
 * 16-byte aligned). */
int sga_fused_sparse_step_single_sweep_out(
    const void* g, int g_dtype, const float* resid, const float* p,
    const float* m, const float* v, float* resid_out, float* p_out,
    float* m_out, float* v_out, int64_t n, int64_t k, const sga_segment* segs,
    int n_segs, int score_id, int32_t* idx_out, void* values_out,
    int values_dtype, uint8_t* mask_out, float factor, float coeff, int flags,
    float interval, uint32_t seed, sga_select_result* result, void* ws,
    size_t ws_bytes, void* ws2, size_t ws2_bytes, void* stream);
int sga_fused_sparse_step_single_sweep_packed_out(
    const void* g, int g_dtype, const float* state, float* state_out,
    int64_t n, int64_t k, const sga_segment* segs, int n_segs, int score_id,
    int32_t* idx_out, void* values_out, int values_dtype, uint8_t* mask_out,
    float factor, float coeff, int flags, float interval, uint32_t seed,
    sga_select_result* result, void* ws, size_t ws_bytes, void* ws2,
    size_t ws2_bytes, void* stream);

/* Packed-state variant of the fused step for callers that let the library
 * lay out the optimizer-side state (no counterpart in the reference, whose
 * buffers are separate tensors): resid, p, m, v are interleaved in 64 KiB
 * records [resid[4096] | p[4096] | m[4096] | v[4096]], i.e. element i of
 * array a (0 resid, 1 p, 2 m, 3 v) is state[(i >> 12) * 16384 + a * 4096 +
 * (i & 4095)].  state holds sga_packed_state_elems(n) floats, 16-byte
 * aligned.  Same arithmetic, same outputs as sga_fused_sparse_step; the four
 * streams of a workgroup then always fall into different DRAM banks of one
 * physical page, which the device rewards with higher streaming efficiency.
 * sga_state_repack converts between the two layouts (unpack = 0: arrays ->
 * state, 1: state -> arrays; a NULL array is skipped). */
int64_t sga_packed_state_elems(int64_t n);
int sga_fused_sparse_step_packed(const void* g, int g_dtype, float* state,
                                 int64_t n, int64_t k, const sga_segment* segs,
                                 int n_segs, int score_id, int32_t* idx_out,
                                 void* values_out, int values_dtype,
                                 uint8_t* mask_out, float factor, float coeff,
                                 int fast, int flags, float interval,
                                 sga_select_result* result, void* ws,
                                 size_t ws_bytes, void* stream);
int sga_state_repack(float* resid, float* p, float* m, float* v, float* state,
                     int64_t n, int unpack, void* stream);

/* ---- fused offline-replay group step (sga/replay_fused.py:1607-1914) ------ */

/* One configuration's resident state for the current recorded step
 * (states[c][param] = {ms, vs, ws, res, sel}, replay_fused.py:1548-1567),
 * flattened over the shard.  sel / out_sel are masks kept as BIT PLANES
 * (sga_plane_words(n) uint32 each): per 1024-element chunk 32 words; element
 * i = c*1024 + it*256 + lane*4 + e is bit (lane & 31) of word
 * (i >> 8)*8 + 2*e + (lane >> 5) -- four wave64 ballots per 256 elements.
 * sga_mask_to_planes / sga_planes_to_mask convert from and to byte masks. */
typedef struct sga_replay_cfg {
  float* w;
  float* m;
  float* v;
  float* res;
  const uint32_t* sel;
  const uint32_t* out_sel; /* outgoing mask for the dual-lr split; NULL = sel */
  double lr_scale;        /* dual-lr scale, lr_inactive = lr * lr_scale      */
  int boundary;           /* si % T == 0                                     */
  int adams;              /* optimizer == "adams"                            */
  int split;              /* boundary dual-lr split active                   */
  int packed;             /* 1: res/w/m/v are the run bases state, state+4096,
                             state+8192, state+12288 of ONE packed state (the
                             layout of sga_fused_sparse_step_packed, array
                             order res, w, m, v); the same for every config  */
  int res_zero;           /* 1: the caller knows res is all zeros when this
                             step starts (first step, or the step after a
                             boundary): it is then neither read nor, at a
                             boundary, rewritten                              */
  int pad_;
} sga_replay_cfg;

/* Per-tensor hyper-parameters of the replay commit (ShardParams entries +
 * _lr_for_step + _bc_pair: replay_fused.py:251-271, replay.py:132-137).
 * lr / wd are kept in double so 1-lr*wd, -lr and lr*lr_scale round like the
 * reference's Python doubles; the rest are fp32 roundings. */
typedef struct sga_replay_segment {
  int64_t start, n;
  double lr, wd;
  float beta1, om1, beta2, om2, eps, bc1, bc2, wdf;
} sga_replay_segment;

/* pass 1 (replay_fused.py:1682-1743): qn2[c] = sum q_pre^2 over the shard
 * (fp32 products, double accumulation, fixed order), coef[c] in double and
 * fp32.  partials: sga_replay_partials() doubles.  cfgs is a HOST array. */
int64_t sga_replay_partials(void);
int sga_replay_pass1(const void* g, int g_dtype, int64_t n, float coef_dense,
                     double clip, const sga_replay_cfg* cfgs, int G,
                     double* partials, double* qn2, double* coef_d,
                     float* coef_f, void* stream);

/* pass 2 (replay_fused.py:1752-1825) for ONE boundary configuration:
 * score = |formula(w,m,v,(g/coef_dense + res)*coef)|, exact top-k with
 * lowest-index ties, written as a byte mask into sel_out.  The score is
 * never materialised.  segs: sga_segment table (beta, eps, wd, bc of the
 * upcoming commit); coef_f: device pointer to this configuration's coef. */
int sga_replay_reselect(const void* g, int g_dtype, const float* res,
                        const float* w, const float* m, const float* v,
                        int64_t n, int64_t k, const sga_segment* segs,
                        int n_segs, int score_id, const float* coef_f,
                        float coef_dense, int adams, int packed, int res_zero,
                        uint32_t* sel_out,
                        sga_select_result* result, void* ws, size_t ws_bytes,
                        void* stream);

/* The boundary re-selections of ONE recorded step in one call
 * (replay_fused.py:1752-1825 re-selects up to every configuration of the group
 * at a step): each job is what sga_replay_reselect takes for one
 * configuration, with a workspace of its own (distinct per job).  Up to 8 jobs
 * form a batch whose short select kernels run once for all of them (the
 * kernels take the job from the grid's second dimension); the kernels that
 * form keys (sample, radix fallback) run once per score among the jobs, the
 * score sweeps once per job.  Same outputs, job by job, as
 * sga_replay_reselect.  `jobs` is a HOST array, read before the call returns. */
typedef struct sga_reselect_job {
  const float* res;
  const float* w;
  const float* m;
  const float* v;
  int64_t k;
  int score_id;
  int adams;
  int res_zero;
  int pad_;
  const float* coef_f;       /* device pointer to this configuration's coef */
  uint32_t* sel_out;         /* bit planes, sga_plane_words(n) words        */
  sga_select_result* result; /* may be NULL                                 */
  void* ws;
  size_t ws_bytes;
} sga_reselect_job;
int sga_replay_reselect_multi(const void* g, int g_dtype, int64_t n,
                              const sga_segment* segs, int n_segs,
                              float coef_dense, int packed,
                              const sga_reselect_job* jobs, int n_jobs,
                              void* stream);

/* pass 2 under the `balanced-histogram` selection semantics
 * (replay_fused.py:405-489, 1805-1809; _histogram.py:115-123, 203-216): the
 * same on-the-fly score, selected like the online engine's approximate tier --
 * histogram of the top 16 bits of |score| over the stride-8 subsample of every
 * tensor's own grid (element j of tensor t is sampled when j = seg_phase[t]
 * (mod 8), seg_phase[t] = (-p_off) mod 8; NULL = all zero), crossing bin
 * b = searchsorted(cumsum(hist), rank), selection = top 16 bits >= b (the
 * whole crossing bin; the count is approximate by construction), written as
 * bit planes into sel_out.  rank is the caller's
 * max(1, round(n_sampled * (n_total - k + 1) / n_total)) (host integers, as
 * the reference computes it).  result: thresh_bits = the bin's lower edge,
 * n_selected = coordinates selected, path 3.  hist: device scratch of
 * sga_balanced_hist_words() uint32. */
int64_t sga_balanced_hist_words(void);
int sga_replay_reselect_balanced(const void* g, int g_dtype, const float* res,
                                 const float* w, const float* m, const float* v,
                                 int64_t n, int64_t rank, const sga_segment* segs,
                                 int n_segs, const int32_t* seg_phase,
                                 int score_id, const float* coef_f,
                                 float coef_dense, int adams, int packed,
                                 int res_zero, uint32_t* sel_out,
                                 sga_select_result* result, uint32_t* hist,
                                 void* ws, size_t ws_bytes, void* stream);

/* pass 3 (replay_fused.py:1836-1889): commit + residual for all G
 * configurations in one sweep (the gradient is read once).  coef_f: device
 * float[G] from pass 1.  segs: DEVICE array.  cfgs: HOST array. */
int sga_replay_pass3(const void* g, int g_dtype, int64_t n, float coef_dense,
                     const sga_replay_cfg* cfgs, int G, const float* coef_f,
                     const sga_replay_segment* segs, int n_segs, void* stream);

/* Dense reference step of the replay (dense_replay_dev, replay.py:848-926):
 * in-place AdamW/AdamS commit of the recorded gradient g over the whole flat
 * shard with per-tensor hyper-parameters from segs, lab += (lr*upd)^2 when lab
 * is not NULL, and recon2[0] = sum((g / coef_dense)^2) in double.  partials:
 * sga_replay_partials() doubles of workspace. */
int sga_dense_replay_step(const void* g, int g_dtype, float* w, float* m, float* v,
                          float* lab, int64_t n, const sga_replay_segment* segs,
                          int n_segs, int adams, double coef_dense, double* partials,
                          double* recon2, void* stream);

/* Bit-plane masks (layout above). */
int64_t sga_plane_words(int64_t n);
int sga_mask_to_planes(const uint8_t* mask, int64_t n, uint32_t* planes,
                       void* stream);
int sga_planes_to_mask(const uint32_t* planes, int64_t n, uint8_t* mask,
                       void* stream);

/* res /= T at fold boundaries (replay_fused.py:1632-1636), true division.
 * packed != 0: x is the run base of one array inside a packed state. */
int sga_div_inplace(float* x, int64_t n, float d, int packed, void* stream);

/* out[0] = sum (a-b)^2 in double (horizon numerators, :1890-1900).
 * partials: 1024 doubles.  a_packed != 0: a is the run base of one array
 * inside a packed state; b is always flat. */
int sga_sq_dist(const float* a, int a_packed, const float* b, int64_t n,
                double* partials, double* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SGA_HIP_H_ */
