/*
 * C ABI of the MI355X (gfx950) distillation-loss library, libdistill_hip.so.
 *
 * The reference (golololologol/LLM-Distillery) has no FFI layer: its loss path is
 * a chain of PyTorch eager ops called from Python.  Each entry point below names
 * the reference lines whose work it replaces.  Conventions shared by all GPU
 * entry points:
 *   - every pointer is a DEVICE pointer on the current HIP device unless the
 *     parameter comment says "host";
 *   - nothing is allocated, freed or retained; buffers belong to the caller;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*) and the call
 *     returns without synchronising;
 *   - strides are in ELEMENTS of the array's dtype;
 *   - the return value is DL_OK or a negative dl_status; no exception crosses
 *     the boundary.
 */
#ifndef DISTILL_HIP_H
#define DISTILL_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { DL_F32 = 0, DL_BF16 = 1, DL_F16 = 2 } dl_dtype;      /* floating storage types */
typedef enum { DL_I32 = 0, DL_I64 = 1 } dl_itype;                   /* index storage types     */
typedef enum { DL_FKL = 0, DL_RKL = 1, DL_JSD = 2 } dl_kind;        /* divergence              */

typedef enum {
  DL_OK = 0,
  DL_ERR_NULL = -1,     /* a required pointer is NULL                      */
  DL_ERR_DTYPE = -2,    /* unknown dtype / itype / kind                    */
  DL_ERR_SHAPE = -3,    /* negative or inconsistent sizes                  */
  DL_ERR_LIMIT = -4,    /* a size exceeds what the kernels support         */
  DL_ERR_LAUNCH = -5,   /* the HIP runtime refused the launch              */
  DL_ERR_ALIGN = -6,    /* a pointer/stride breaks a stated alignment rule */
  DL_ERR_WORKSPACE = -7, /* a required workspace is too small              */
  DL_ERR_SCRATCH = -8   /* dl_div_topk_static: the problem needs more scratch than the static array holds */
} dl_status;

#define DL_MAX_TOPK 2048      /* entries per row a sparse teacher may hold        */
#define DL_MAX_TEACHERS 8     /* teachers merged in one launch                    */
#define DL_MAX_HOST_CONVOS 64 /* conversations whose offsets may travel with a launch (dl_composite_*) */
/* dl_div_topk flags (OR them together) */
#define DL_TOPK_UNIQUE_IDS 1   /* no id occurs twice in a row                                          */
#define DL_TOPK_NO_WAIT 2      /* parts of a split row never wait for their partners: every part that  */
                               /* finds a record missing is finished by the second launch (exercises   */
                               /* that path; same results, slower)                                      */
#define DL_TOPK_FINE_PARTS 4   /* rows of 1025-16384 16-byte chunks are cut into parts of 1024 chunks   */
                               /* (up to 16 per row) where the workspace holds 20 bytes per row and    */
                               /* part + 16; else ignored                                               */
#define DL_TOPK_PARTS_SHIFT 8  /* bits 8-11: column parts a row of 65537-131072 two-byte (half as many */
#define DL_TOPK_PARTS(n) ((n) << DL_TOPK_PARTS_SHIFT)   /* four-byte) entries is cut into: 1, 2 or 4    */
                               /* (4 only where four parts of 32768 two-byte entries all hold columns); */
                               /* 0 = automatic                                                         */

/* Library ABI revision; bumped when a signature changes. */
int dl_abi_version(void);
/* Static, NUL-terminated description of a dl_status. */
const char* dl_status_string(int status);

/*
 * Forward or reverse KL against a sparse (top-K) teacher, loss and gradient in one sweep.
 * Replaces, for one launch over all token rows:
 *   classes/student/model.py:408,420-421   slice + .float() + /T, row select, teacher /T
 *   utils/finetuning_utils.py:88,91-92     log_softmax (student over V, teacher over K), gather
 *   utils/finetuning_utils.py:49-56,104-105  F.kl_div(log_target=True).sum(-1)   (kind FKL / RKL)
 *   classes/losses.py:77-78                the autograd replay of all of the above
 *
 * logits     [n_rows, V] (row stride `row_stride`), dtype `logits_dtype`, native model dtype.
 * row_map    [n_rows] int32: teacher row feeding logits row r; a value outside
 *            [0, n_teacher_rows) marks a masked/padded row (loss 0, gradient row zero-filled);
 *            NULL = identity.
 * t_val      [*, K] stored teacher log-probs (dtype `t_val_dtype`), t_idx [*, K] vocabulary ids
 *            (`t_idx_itype`); both K-contiguous.  t_cnt: optional int32 per teacher row, only the
 *            first t_cnt entries count (NULL = all K).  Ids outside [0, V) are ignored, and so are entries
 *            whose stored log-prob is -inf (zero mass: they do not belong to the teacher's support).
 *            The teacher is renormalised over its counted entries: log_softmax(t_val * inv_T_teacher).
 * row_loss   [n_rows] fp32 per-token divergence (optional, may be NULL).
 * grad       [n_rows, V] (stride `grad_stride`), same dtype as logits; receives
 *            d(sum_r row_loss[r]) / d logits * grad_scale (optional, NULL = forward only).
 * workspace  optional scratch of at least dl_div_topk_workspace_bytes(...) bytes, 16-byte aligned,
 *            contents irrelevant on entry and on return.  Rows too wide for one workgroup's share
 *            of the register file are cut into column parts that meet through it; without a
 *            workspace (NULL or too small) such rows take a slower one-workgroup-per-row kernel.
 *            Two launches that may overlap in time must not share a workspace.
 * flags      DL_TOPK_UNIQUE_IDS promises that no id occurs twice within a row (true for the output of
 *            torch.topk and of dl_merge_remap_topk); the kernel then skips its check for repeated ids
 *            (a few instructions per entry in the register kernels, a scan in the streaming one).  With
 *            the flag set and duplicates present, the gradient at a duplicated id is wrong.
 *            DL_TOPK_NO_WAIT and DL_TOPK_PARTS(n) are tuning / test hooks of the split-row kernels; they
 *            change neither results nor requirements.  The library keeps no state between calls.
 * K <= DL_MAX_TOPK.
 * Alignment: any V and any element-aligned pointers and row strides are taken (else DL_ERR_ALIGN).  Rows
 * on the 16-byte grid (16-byte aligned pointers, logits and gradient; row strides whole numbers of 16-byte
 * chunks) take the aligned register kernels whatever V is: a row that ends inside a chunk -- the crop
 * logits[:, :, :V] of a vocabulary padded to a multiple of 8 (4 for fp32) columns,
 * classes/student/model.py:408 -- moves like a whole one, one workgroup per row or cut into column parts,
 * and only its last chunk is stored element by element; nothing beyond column V is written.  The kernels
 * READ that chunk's 16 bytes whole: they begin inside the row and, aligned as they are, end inside the
 * row's stride or at least inside the memory page of the row's last column, so the read cannot fault; what
 * it brings in from beyond column V is discarded.  The same holds for dl_rowcoef_grad_topk and
 * dl_fkl_multi_teacher.  Other rows (an odd row stride, a column slice that starts off the grid) are still
 * moved 16 bytes at a time: forward-KL rows by unaligned accesses in the register kernels (one workgroup per
 * row of up to 4096 16-byte chunks, column parts beyond where a workspace came along -- which
 * dl_div_topk_workspace_bytes asks for from 4097 chunks on when V is not a whole number of chunks); wider ones
 * without a workspace, and dl_rowstats_topk / dl_rowcoef_grad_topk, by the aligned chunks inside
 * each row, provided that logits and gradient rows share their address modulo 16 (the same stride from
 * 16-byte aligned bases, or the gradient written over the logits; reverse KL: any gradient row), and
 * element by element otherwise.
 * grad may be the logits buffer itself (same pointer and stride): every kernel holds, or has
 * consumed, what it still needs of a row before it writes there.  The same holds for dl_div_dense
 * and dl_rkl_marginalised, not for dl_rowcoef_grad_topk.
 * With n_teacher_rows == 0 the teacher pointers may be NULL: every row then counts as masked
 * (the same holds for dl_div_dense, dl_rowstats_topk and dl_rowcoef_grad_topk).
 */
int dl_div_topk(int kind,
                const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                const int32_t* row_map,
                const void* t_val, int t_val_dtype, const void* t_idx, int t_idx_itype, int K,
                int64_t n_teacher_rows, const int32_t* t_cnt,
                float inv_T_student, float inv_T_teacher, float grad_scale,
                float* row_loss, void* grad, int64_t grad_stride,
                void* workspace, int64_t workspace_bytes, int flags, void* stream);

/* Scratch size dl_div_topk can make use of for this problem (0 = none needed).  Host-only. */
int64_t dl_div_topk_workspace_bytes(int kind, int logits_dtype, int64_t n_rows, int64_t V);

/*
 * dl_div_topk for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, results and kernels as dl_div_topk, without the workspace pair: the scratch of the
 * split-row kernels lives in a static device array of DL_STATIC_SCRATCH_BYTES that every GPU the
 * library runs on holds until the process ends.  The call allocates and frees nothing.
 * Limit: dl_div_topk_workspace_bytes(kind, logits_dtype, n_rows, V) <= DL_STATIC_SCRATCH_BYTES
 * (e.g. 52428 rows of 65537-131072 two-byte entries; narrower rows need no scratch and have no
 * limit), else DL_ERR_SCRATCH and nothing is launched.
 * All calls on one GPU share that GPU's array: calls that may overlap in time on one GPU (two
 * streams, two threads) race on it and must use dl_div_topk with workspaces of their own.  Calls
 * in stream order need no care: each call clears the part of the array it uses with a fill
 * kernel before its main launch.
 */
#define DL_STATIC_SCRATCH_BYTES (4 << 20)
int dl_div_topk_static(int kind,
                       const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                       const int32_t* row_map,
                       const void* t_val, int t_val_dtype, const void* t_idx, int t_idx_itype, int K,
                       int64_t n_teacher_rows, const int32_t* t_cnt,
                       float inv_T_student, float inv_T_teacher, float grad_scale,
                       float* row_loss, void* grad, int64_t grad_stride, int flags, void* stream);

/*
 * Forward KL (DL_FKL), reverse KL (DL_RKL) or Jensen-Shannon divergence (DL_JSD) against a dense
 * teacher, loss and gradient in one launch.  Replaces, with K = V:
 *   classes/student/model.py:408,420-421, utils/finetuning_utils.py:88,94 (both log_softmax),
 *   utils/finetuning_utils.py:49-56,104-105 (kl_div + sum), classes/losses.py:77-78 (autograd replay).
 * The reference's training side cannot run a dense teacher (it raises on indices=None) and has no
 * JSD, so the conventions are this library's: teacher entries of -inf logit carry zero mass and
 * contribute 0 to FKL/JSD; RKL renormalises the student over the teacher's support
 * {j : t_logits[j] > -inf}, as the reference renormalises it over the top-K ids; JSD is
 * 0.5 KL(P||M) + 0.5 KL(Q||M), natural log.
 * t_logits [n_teacher_rows, V] (stride t_stride): teacher logits or log-probs (any per-row constant
 * is irrelevant), scaled by inv_T_teacher.  Other arguments as for dl_div_topk.
 * Rows on the 16-byte grid (student, teacher and gradient; V a multiple of 8) are read once as far as
 * a workgroup's registers hold the pair (65536 columns of 16-bit rows, 32768 with an fp32 row) and
 * streamed in 16-byte chunks beyond that; rows off the grid take the same register kernels through
 * unaligned 16-byte accesses when student and teacher share a dtype and the pair fits, and a
 * kernel that streams them element by element otherwise.
 * Pointers and strides must be whole elements (else DL_ERR_ALIGN).
 */
int dl_div_dense(int kind,
                 const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                 const int32_t* row_map,
                 const void* t_logits, int t_dtype, int64_t t_stride, int64_t n_teacher_rows,
                 float inv_T_student, float inv_T_teacher, float grad_scale,
                 float* row_loss, void* grad, int64_t grad_stride, void* stream);

/*
 * dl_div_dense with a workspace: forward and reverse KL on rows that the registers of 512 threads do not hold
 * (more than 32768 columns of two 16-bit rows, 24576 of a 16-bit row against an fp32 one, 16384 of two fp32
 * rows) are cut evenly into 2 to 8 column parts, one workgroup of 256, 512 or 1024 threads each, which exchange
 * their maxima and sums through the workspace -- the split of dl_div_topk applied to the dense pair (same
 * reference lines as dl_div_dense).  Parts of different rows share a compute unit and hide each other's load,
 * arithmetic and store phases, which a workgroup that holds a whole pair of rows cannot.  Same arguments and
 * conventions as dl_div_dense, same results to fp32 rounding (the sums are taken part by part),
 * bit-reproducible from call to call.
 * workspace   at least dl_div_dense_workspace_bytes(...) bytes, 16-byte aligned, contents irrelevant on entry
 *             and on return; NULL or too small: exactly dl_div_dense.  Launches that may overlap in time must
 *             not share a workspace.  dl_div_dense_workspace_bytes returns 0 where rows are not cut (JSD,
 *             narrow or very wide rows, V not a multiple of 8, dtype pairs without a register kernel).
 * flags       DL_TOPK_NO_WAIT: the parts never wait for their partners; DL_TOPK_PARTS(1 / 2 / 3): parts of
 *             256 / 512 / 1024 threads wherever two or more come out (test and tuning hooks).
 */
int dl_div_dense_ws(int kind,
                    const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                    const int32_t* row_map,
                    const void* t_logits, int t_dtype, int64_t t_stride, int64_t n_teacher_rows,
                    float inv_T_student, float inv_T_teacher, float grad_scale,
                    float* row_loss, void* grad, int64_t grad_stride,
                    void* workspace, int64_t workspace_bytes, int flags, void* stream);

/* Scratch size dl_div_dense_ws can make use of for this problem (0 = none: rows are not cut).  Host-only. */
int64_t dl_div_dense_workspace_bytes(int kind, int logits_dtype, int t_dtype, int64_t n_rows, int64_t V);

/*
 * Phase 1 of the general (two-phase) path: per valid row r with teacher row t = row_map[r],
 *   lse[t]   = logsumexp_j(logits[r, j] * inv_T)                       (fp32, natural log)
 *   zk[t, k] = logits[r, t_idx[t, k]] * inv_T                          (fp32; 0 for ids outside [0, V))
 * Replaces classes/student/model.py:408,420 (slice, cast, /T, row select) and
 * utils/finetuning_utils.py:88,92 (full-vocabulary log_softmax + gather): the student log-probs
 * on the teacher's support are zk - lse.  Rows whose row_map entry is outside
 * [0, n_teacher_rows) are skipped (their lse / zk entries are not written).
 */
int dl_rowstats_topk(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                     const int32_t* row_map, const void* t_idx, int t_idx_itype, int K,
                     int64_t n_teacher_rows, float inv_T, float* lse, float* zk, void* stream);

/*
 * Phase 2: the gradient of any scalar L that depends on the logits only through phase 1's
 * outputs, given coef_lse[t] = dL/d lse[t] and coef_zk[t, k] = dL/d zk[t, k]:
 *   grad[r, j] = ( coef_lse[t] * softmax(logits[r] * inv_T)_j + sum_k coef_zk[t, k] [j == t_idx[t, k]] ) * inv_T
 * in the logits' dtype; masked rows are zero-filled.  `lse` is phase 1's output.
 * Replaces the autograd replay (classes/losses.py:77-78) of log_softmax + gather + index_select
 * + /T + cast.
 */
int dl_rowcoef_grad_topk(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                         const int32_t* row_map, const void* t_idx, int t_idx_itype, int K,
                         int64_t n_teacher_rows, float inv_T, const float* lse, const float* coef_lse,
                         const float* coef_zk, void* grad, int64_t grad_stride, void* stream);

/*
 * The K-wide half of the composite loss for all conversations of a batch, from phase 1's outputs.
 * Replaces utils/finetuning_utils.py:58-84 (abomination_loss, custom_ce_loss), :91 (teacher
 * log_softmax over K), :96-110 (CE, CE diff, forward / reverse KL per token, the two weighted means
 * and their average) and :112-122 (the nine values), and in backward the autograd replay of those
 * lines.  Conversation c owns rows [row_off[c], row_off[c+1]) of lse / zk / t_val / t_idx, labels
 * [label_off[c], label_off[c+1]) of `labels` (row i of the conversation carries label i; the caller
 * guarantees #labels == #rows - 1, the only case the reference's code runs without raising) and
 * entries [avoid_off[c], avoid_off[c+1]) of `avoid` (conversation-local rows excluded from the cross
 * entropy; entries outside [0, #labels) are ignored; avoid_itype DL_I32 or DL_I64).  The teacher rows
 * are renormalised over their K entries after scaling by inv_T_teacher.
 * row_off / label_off / avoid_off: [n_convos + 1] each; DEVICE arrays, or with offsets_on_host != 0
 * HOST arrays of at most DL_MAX_HOST_CONVOS conversations that are copied into the launch (no upload:
 * the reference calls its loss once per conversation, classes/student/model.py:415-427; labels /
 * avoid may then be NULL where a conversation set has none).
 * out [n_convos, 9] in the reference's key order: train_loss, custom loss, CE loss, kl_div,
 * reverse kl_div, weighted kl_div, weighted rev. kl_div, teacher CE loss, CE diff.
 * row_records (32 bytes per row) and row_coef (16 bytes per row, may be NULL when no gradient is
 * wanted) are caller-owned device buffers that carry the per-row state to dl_composite_backward.
 * The gradient of max(kl) is shared evenly among tied rows, as torch.max's is.
 */
int dl_composite_forward(const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                         float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                         const int64_t* labels, const void* avoid, int avoid_itype, const int32_t* row_off,
                         const int32_t* label_off, const int32_t* avoid_off, int offsets_on_host, int n_convos,
                         int64_t n_rows, float alpha, void* row_records, void* row_coef, float* out,
                         void* stream);

/*
 * dl_rowstats_topk and dl_composite_forward in one call.  Where every teacher row has its logits row (no row map,
 * n_teacher_rows == n_rows), K <= 1024 and a row holds at most 16384 16-byte chunks, phase 1 makes the rows'
 * records at its own tail -- the logits at the teacher's ids are in LDS when its sweep ends -- and the call is two
 * launches instead of three; otherwise it runs the launches of the two entry points it stands for.  Arguments,
 * reference lines and results as theirs (lse, zk, row_records, row_coef, out are all written; the records agree
 * with dl_composite_forward's to fp32 rounding: the sums over K are taken by a workgroup instead of a wave).
 */
int dl_composite_forward_fused(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                               const int32_t* row_map, int64_t n_teacher_rows, float inv_T, const void* t_val,
                               int t_val_dtype, float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                               const int64_t* labels, const void* avoid, int avoid_itype, const int32_t* row_off,
                               const int32_t* label_off, const int32_t* avoid_off, int offsets_on_host,
                               int n_convos, float alpha, float* lse, float* zk, void* row_records,
                               void* row_coef, float* out, void* stream);

/*
 * Backward of dl_composite_forward for upstream gradients g_train [n_convos] on each conversation's
 * train_loss: g_lse [n_rows] = dL/dlse and g_zk [n_rows, K] = dL/dzk, the inputs of
 * dl_rowcoef_grad_topk.  Replaces the autograd replay started at classes/losses.py:77-78.
 * row_off / offsets_on_host as for dl_composite_forward.
 */
int dl_composite_backward(const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                          float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                          const int32_t* row_off, int offsets_on_host, int n_convos, int64_t n_rows,
                          const void* row_records, const void* row_coef, const float* g_train, float* g_lse,
                          float* g_zk, void* stream);

/*
 * dl_composite_backward and dl_rowcoef_grad_topk in one launch: every column part of a row makes the row's K
 * coefficients and their sum itself (from the row's record, its conversation's coefficients and g_train) instead
 * of reading what a launch before it wrote (the reference's default shape, one conversation of 2048 x 32000
 * logits, is a few tens of microseconds of kernels per call: a launch saved counts there).  Same reference lines
 * and the same arguments with the same meaning as the two entry points it stands for (row_map / n_teacher_rows as
 * for dl_rowcoef_grad_topk: the K-wide arrays, the records and the offsets count teacher rows).  grad [n_rows, V] =
 * d(sum_c g_train[c] * train_loss[c]) / d logits, to fp32 rounding what the two entry points give (the sum over
 * the K coefficients is taken in another order); rows and alignment as for dl_rowcoef_grad_topk.
 */
int dl_composite_backward_fused(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                                int64_t V, const int32_t* row_map, int64_t n_teacher_rows, float inv_T,
                                const void* t_val, int t_val_dtype, float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                                const int32_t* row_off, int offsets_on_host, int n_convos, const float* lse,
                                const float* zk, const void* row_records, const void* row_coef,
                                const float* g_train, void* grad, int64_t grad_stride, void* stream);

/*
 * Teacher producer: per selected row, log_softmax over the V (cropped) columns, then the K largest
 * log-probs in descending order with their ids.  Replaces
 *   classes/teacher/inference_worker.py:73-80  (F.log_softmax(logits[:, :, :crop].float()) -> torch.topk)
 *   classes/teacher/result_processor_worker.py:27-35  (content-row selection, via row_list)
 *   classes/data_manager.py:306,312  (cast to the storage dtypes: out_dtype DL_F16, out_itype DL_I32)
 * No temperature is applied at collection time.  row_list (int32 [n_out], may be NULL = rows
 * 0..n_out-1) names the logits row behind each output row; an entry outside [0, n_rows) gives a
 * masked output row (log-probs -inf, ids -1) and touches no logits.  Entries with equal log-prob are
 * ordered by ascending id (the reference leaves tie order to torch.topk); logits are ranked by their
 * bit patterns, so a -0 ranks just below a +0.
 * K <= 1024, K <= V; V <= 262144 (131072 fp32); K * parts <= 4096 with parts = ceil(V / 32768)
 * (fp32: ceil(V / 16384)).  Any V and any element-aligned row pitch are taken, as by the reference;
 * V a multiple of 8 (4 for fp32) with 16-byte aligned rows selects the 16-byte loads.
 * workspace: device memory, 16-byte aligned, at least dl_teacher_topk_workspace_bytes(...) bytes
 * (per output row and 32768-column part: the part's best K candidates and its softmax statistics);
 * contents need no initialisation and mean nothing afterwards.  Two launches that may overlap in
 * time need different workspaces.
 */
int dl_teacher_topk(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                    const int32_t* row_list, int64_t n_out, int K,
                    void* out_val, int out_dtype, void* out_idx, int out_itype,
                    void* workspace, int64_t workspace_bytes, void* stream);
int64_t dl_teacher_topk_workspace_bytes(int logits_dtype, int64_t n_out, int64_t V, int K);

/*
 * Weighted merge of n_teachers sparse teachers with an optional vocabulary id map
 * (no reference counterpart; generalises classes/data_manager.py:231-240, which is unweighted,
 * pairwise and has no map).  Per row: mass = weights[j] * exp(t_vals[j][row, k]); the id goes
 * through id_map (int32 [Vt], teacher id -> student id, -1 = dropped; NULL = identity); entries
 * outside [0, Vs) are dropped; entries on the same id are summed in entry order (teacher 0 first).
 * Output, E = n_teachers * K columns per row: out_idx ascending ids (int32, -1 padding),
 * out_logmass = log(summed mass) (fp32, -inf padding), out_cnt = survivors per row.  Feed these to
 * dl_div_topk as (t_val = out_logmass, t_idx = out_idx, K = E, t_cnt = out_cnt): it renormalises.
 * t_vals / t_idxs / weights are HOST arrays of n_teachers device pointers / floats.
 * n_teachers <= DL_MAX_TEACHERS, n_teachers * K <= 4096.
 */
int dl_merge_remap_topk(int n_teachers, const void* const* t_vals, const void* const* t_idxs,
                        int val_dtype, int idx_itype, int K, const float* weights, int64_t n_rows,
                        const int32_t* id_map, int64_t Vt, int64_t Vs,
                        int32_t* out_idx, float* out_logmass, int32_t* out_cnt, void* stream);

/*
 * Forward KL against the weighted mixture of n_teachers sparse teachers, loss and gradient:
 * what dl_merge_remap_topk + dl_div_topk(DL_FKL) compute, without the sort and without the merged
 * row going through memory for every column part (no reference counterpart for weights and id map;
 * replaces, per training step, what the reference does at collection time in
 * classes/data_manager.py:231-240 plus utils/finetuning_utils.py:88,91-92,104 and the autograd
 * replay of classes/losses.py:77-78).
 * Per row: mass_e = weights[j] * exp(t_vals[j][row, k]); the id goes through id_map (int32 [Vt],
 * negative = dropped; NULL = identity); ids outside [0, V) are dropped; the teacher distribution is
 * Q_id = (sum of the masses on id) / (sum of all surviving masses) -- the renormalisation of
 * dl_div_topk at teacher temperature 1, the only one this entry point offers (for others merge first:
 * the power 1/T applies to the summed mass of an id).  row_loss = sum_id Q_id (log Q_id - log p_id),
 * grad = (softmax(logits * inv_T_student) - Q) * inv_T_student * grad_scale.  Sums over the entries of
 * one id are taken in fixed point: results do not depend on the order the hardware met them in.
 * Two launches: a K-wide one over the teacher rows (map, weigh, renormalise, deal the entries into
 * one bucket per column part of the loss kernel's rows, in the workspace), then dl_div_topk's loss
 * kernels, each workgroup reading only its own bucket.
 * t_vals / t_idxs / weights are HOST arrays of n_teachers device pointers / non-negative floats;
 * every teacher holds [n_teacher_rows, K] entries, K-contiguous.  flags: DL_TOPK_NO_WAIT,
 * DL_TOPK_PARTS as for dl_div_topk.  workspace: at least dl_fkl_multi_teacher_workspace_bytes(...)
 * bytes (same flags), 256-byte aligned, contents irrelevant on entry and on return; two launches
 * that may overlap in time need different workspaces.
 * Limits: n_teachers <= DL_MAX_TEACHERS, n_teachers * K <= DL_MAX_TOPK; logits and gradient rows on the
 * 16-byte grid (aligned pointers, strides whole numbers of chunks; V itself may end inside a chunk, see
 * dl_div_topk), else DL_ERR_ALIGN; V <= 262144 two-byte / 131072 four-byte columns, else
 * DL_ERR_LIMIT (dl_fkl_multi_teacher_workspace_bytes then returns 0).  In those cases nothing was
 * launched: call dl_merge_remap_topk + dl_div_topk.
 */
int dl_fkl_multi_teacher(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                         const int32_t* row_map, int n_teachers, const void* const* t_vals,
                         const void* const* t_idxs, int val_dtype, int idx_itype, int K,
                         int64_t n_teacher_rows, const float* weights, const int32_t* id_map, int64_t Vt,
                         float inv_T_student, float grad_scale, float* row_loss, void* grad, int64_t grad_stride,
                         void* workspace, int64_t workspace_bytes, int flags, void* stream);
int64_t dl_fkl_multi_teacher_workspace_bytes(int logits_dtype, int64_t n_rows, int64_t V, int n_teachers, int K,
                                             int64_t n_teacher_rows, int flags);

/*
 * The dataset manager's pairwise merge, classes/data_manager.py:198-261 (merge_topk): exp both
 * inputs, per row sum the masses of equal ids, keep the K largest in descending order, log.
 * Rows that only the longer input holds pass through in their stored order (:214-224,242-244).
 * Ties between equal masses go to the smaller id (the reference leaves them to torch.topk).
 * Outputs cover max(disk_rows, new_rows) rows: out_logmass fp32 [rows, K], out_idx int64 [rows, K].
 * 2 * K <= 4096.
 */
int dl_merge_topk_pair(const void* disk_val, const void* disk_idx, int64_t disk_rows,
                       const void* new_val, const void* new_idx, int64_t new_rows,
                       int val_dtype, int idx_itype, int K, int64_t V,
                       float* out_logmass, int64_t* out_idx, void* stream);

/*
 * Byte-trie longest-prefix map between two tokenizers (no reference counterpart; the reference
 * rejects cross-vocabulary distillation, collect_and_finetune.py:83-101).  HOST function, HOST
 * pointers.  Vocabularies are given as concatenated byte strings plus int64 offsets [n + 1].
 * out_t2s[t] = id of the student token whose bytes are the longest prefix of teacher token t
 * (duplicate student strings: the smallest id), else byte_fallback[first byte] if that table
 * (256 int32, may be NULL) holds an id >= 0, else -1; empty teacher tokens map to -1.
 */
int dl_trie_longest_prefix_map(const uint8_t* student_bytes, const int64_t* student_offsets, int64_t n_student,
                               const uint8_t* teacher_bytes, const int64_t* teacher_offsets, int64_t n_teacher,
                               const int32_t* byte_fallback, int32_t* out_t2s);

/*
 * CSR form of a teacher->student map (HOST function, HOST pointers): offsets int32 [n_student + 1],
 * indices int32 [n_teacher] (the first *n_mapped entries are used) listing, per student id, the
 * teacher ids mapped to it in ascending order; ids mapped to -1 are left out.
 */
int dl_csr_from_map(const int32_t* t2s, int64_t n_teacher, int64_t n_student, int32_t* offsets,
                    int32_t* indices, int64_t* n_mapped);

/*
 * Marginalisation plan (HOST function, HOST pointers; no reference counterpart): re-lays a
 * teacher->student map for the planned kernels, which add every marginal in a fixed order without
 * atomics: every accumulator word in LDS belongs to one thread of a 1024-thread workgroup.  Slot s
 * (< n_student) accumulates student id s; ids with far more than an even share of the teacher ids
 * get replica slots (n_student rounded up to 4, + j), *n_extra_out in all, folded into the id's
 * slot after the last tile as listed in `fold` (int32 triples: id, first replica slot, replica
 * count).  The teacher vocabulary is cut into tiles of *tile_out ids; for tile k and wave w, rows
 * (row_off[16k + w] & ~3) .. (row_off[16k + w + 1] & ~3) of `ent` (64 dwords per row) hold the
 * entries of the wave's 64 threads, per thread sorted by (slot, t), in one of two formats:
 *   general (bit 0 of row_off[16k + w] clear): batches of 8 entries per lane, 8 rows each, the
 *     entries of lane l in dwords [8l, 8l + 8) of the batch.  A thread adds up runs of entries of one
 *     slot and stores slot + running sum after every entry: bit 31 of an entry = first of its run,
 *     bits 15-30 = the slot on the run's last entry and the lane's spare slot (64 of them behind the
 *     replicas) on the others, bits 0-14 = 4 * (t - k * tile).  Padding = a first entry on the spare
 *     slot with offset 0, ahead of the lane's entries.
 *   packed (bit 0 set: every lane holds at most one run of at most 8 entries): 4 rows, the lane's 4
 *     dwords at [4l, 4l + 4), two 16-bit fields per dword, entries in order from the low field of
 *     dword 0; bits 2-15 of a field = 4 * (t - k * tile), or 4 * tile (words the kernels keep at
 *     zero) for padding, which comes first; the low two bits of the eight fields together are the
 *     slot: field 2j carries its bits 2j, 2j + 1, field 2j + 1 its bits 8 + 2j, 9 + 2j.
 * Between tiles a slot may change hands.
 * Call once with row_off = ent = fold = NULL to learn *tile_out, *ent_rows_out, *n_fold_out and
 * *n_extra_out, allocate row_off int32 [16 * ceil(n_teacher / tile) + 1], ent uint32
 * [64 * ent_rows] and fold int32 [3 * n_fold], call again.
 * DL_ERR_LIMIT: the student vocabulary is too wide for a plan (fp32 marginal + 64 spare slots + 16 KiB tile + 16 bytes must fit 159 KiB).
 */
int dl_marginal_plan_build(const int32_t* t2s, int64_t n_teacher, int64_t n_student, int* tile_out,
                           int32_t* row_off, uint32_t* ent, int64_t ent_rows_capacity, int64_t* ent_rows_out,
                           int32_t* fold, int64_t fold_capacity, int64_t* n_fold_out, int* n_extra_out);

/*
 * marg[r, s] = sum of probs[r, t] over the teacher ids t with t2s[t] == s (probs [n_rows, Vt] in
 * p_dtype, marg fp32 [n_rows, Vs]; out_log != 0 stores log(marg) instead).  With a plan
 * (plan_row_off / plan_ent / plan_fold device copies of dl_marginal_plan_build's arrays, plan_tile,
 * plan_n_fold and plan_n_extra its tile, fold count and replica count;
 * fp32 probabilities, 16-byte aligned rows) every sum is added in a fixed order: bit-reproducible.
 * Without (NULL, NULL, 0) it accumulates with LDS floating-point atomics: sums then agree to fp32
 * rounding, not bit for bit.
 */
int dl_marginalise_map(const void* probs, int p_dtype, int64_t p_stride, int64_t n_rows, int64_t Vt,
                       const int32_t* t2s, int64_t Vs,
                       const int32_t* plan_row_off, const uint32_t* plan_ent, int plan_tile,
                       const int32_t* plan_fold, int plan_n_fold, int plan_n_extra,
                       float* marg, int64_t marg_stride, int out_log, void* stream);

/*
 * Column subsets, for student vocabularies wider than the marginal that dl_rkl_marginalised can hold (36864 ids):
 * a teacher -> student map only ever reaches the student ids in its image, all other columns of a row lie off
 * the marginal's support (no loss term, zero gradient), so the fused kernel can run on the image alone.
 *   dl_gather_columns   dst[r, c] = src[r, cols[c]] for c < n_cols; cols[c] < 0 (padding) gives -inf.
 *   dl_expand_columns   dst[r, j] = src[r, col_src[j]] for j < V; col_src[j] < 0 (a column outside the subset) gives 0.
 * Raw 2- or 4-byte elements of `dtype`, no conversion.  cols int32 [n_cols], col_src int32 [V], both 16-byte
 * aligned; dst rows on the 16-byte grid, n_cols (gather) / V (expand) whole 16-byte chunks (else DL_ERR_ALIGN);
 * src rows of any stride.  n_rows <= 65535 per call.  Reference: none (serves the byte-trie reverse KL where the
 * student vocabulary is too wide for a marginal in LDS: 128256 ids).
 */
int dl_gather_columns(const void* src, int dtype, int64_t src_stride, int64_t n_rows, int64_t V, const int32_t* cols,
                      int64_t n_cols, void* dst, int64_t dst_stride, void* stream);
int dl_expand_columns(const void* src, int dtype, int64_t src_stride, int64_t n_rows, int64_t n_cols,
                      const int32_t* col_src, int64_t V, void* dst, int64_t dst_stride, void* stream);

/* The same marginal from the CSR form, each segment added in ascending teacher-id order (bit-reproducible). */
int dl_marginalise_csr(const void* probs, int p_dtype, int64_t p_stride, int64_t n_rows, int64_t Vt,
                       const int32_t* offsets, const int32_t* indices, int64_t Vs, float* marg,
                       int64_t marg_stride, int out_log, void* stream);

/*
 * Fused: marginalise the dense teacher row t_probs[row_map[r]] (over Vt teacher ids) into the Vs
 * student ids inside LDS, then reverse KL of the student logits[r] against
 * softmax(log(marginal) * inv_T_teacher), loss and gradient, with the conventions of dl_div_dense
 * (DL_RKL: student renormalised over the marginal's support).  The marginal never reaches memory.
 * Optional plan as for dl_marginalise_map (faster and bit-reproducible).
 * Vs <= 36864 (the fp32 marginal of one row must fit the CU's LDS), Vs % 8 == 0, logits / grad
 * rows 16-byte aligned (else DL_ERR_LIMIT / DL_ERR_ALIGN: use dl_marginalise_map + dl_div_dense).
 */
int dl_rkl_marginalised(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t Vs,
                        const int32_t* row_map, const void* t_probs, int p_dtype, int64_t p_stride,
                        int64_t n_teacher_rows, int64_t Vt, const int32_t* t2s,
                        const int32_t* plan_row_off, const uint32_t* plan_ent, int plan_tile,
                        const int32_t* plan_fold, int plan_n_fold, int plan_n_extra,
                        float inv_T_student, float inv_T_teacher, float grad_scale,
                        float* row_loss, void* grad, int64_t grad_stride, void* stream);

/*
 * dl_rkl_marginalised for a student vocabulary wider than the marginal the kernel can hold (Vs_full columns per
 * logits / gradient row, any width): a teacher -> student map only ever reaches the student ids in its image, and
 * every other column of a row lies off the marginal's support -- no loss term, zero gradient -- so the kernel
 * works on the image alone.  cols int32 [n_compact] names the image's columns, ascending, padded with -1 to a
 * multiple of 8 (n_compact <= 36864); col_src16 uint16 [Vs_full] gives every column its position in `cols`
 * (0xffff: outside the image); t2c int32 [Vt] maps teacher ids onto positions in `cols` (negative: dropped), and the
 * plan arrays are dl_marginal_plan_build's for (t2c, n_compact).  The kernel gathers the row's logits at `cols`
 * while the teacher row streams in, and writes the full-width gradient row from the compact one it holds in LDS:
 * every 16-byte chunk once.  Other arguments, conventions and results as dl_rkl_marginalised (the loss and the
 * gradient are those of the full vocabulary).  cols / col_src16 16-byte aligned, gradient rows on the 16-byte grid,
 * Vs_full a multiple of 8; the logits rows need element alignment only.  No counterpart in the reference
 * (the byte-trie reverse KL on maps that use few student ids, and on student vocabularies of 128256 ids).
 */
int dl_rkl_marginalised_compact(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t Vs_full,
                                const int32_t* cols, const uint16_t* col_src16, int64_t n_compact,
                                const int32_t* row_map,
                                const void* t_probs, int p_dtype, int64_t p_stride, int64_t n_teacher_rows, int64_t Vt,
                                const int32_t* t2c,
                                const int32_t* plan_row_off, const uint32_t* plan_ent, int plan_tile,
                                const int32_t* plan_fold, int plan_n_fold, int plan_n_extra,
                                float inv_T_student, float inv_T_teacher, float grad_scale,
                                float* row_loss, void* grad, int64_t grad_stride, void* stream);


/*
 * Deterministic sum of n fp32 values times `scale` into out[0] (fixed reduction tree,
 * double accumulation).  Replaces the `.mean()` of utils/finetuning_utils.py:54 /
 * the `+=` accumulation of classes/losses.py:43-47.
 */
int dl_reduce_sum(const float* values, int64_t n, float scale, float* out, void* stream);

/*
 * Plain 16-byte streaming copy of n_bytes (a multiple of 16; both pointers 16-byte aligned).
 * No reference counterpart: it is the calibration kernel of known traffic that the HBM
 * counters (FETCH_SIZE / WRITE_SIZE) of the loss kernels are scaled by.
 */
int dl_copy16(const void* src, void* dst, int64_t n_bytes, void* stream);

/*
 * Copy of n_rows rows of row_bytes (a multiple of 16; both pointers 16-byte aligned, rows dense) in
 * the access shape of the row kernels: every row is cut into column parts of threads x chunks
 * 16-byte chunks, one workgroup per part, each thread issuing all its loads and then all its stores.
 * No reference counterpart: the yardstick that says what a bare copy reaches in a kernel's shape.
 * (threads, chunks) one of (256, 2 / 4 / 8 / 12 / 16), (512, 4 / 8 / 16), (1024, 4 / 16), else
 * DL_ERR_LIMIT.  flags:
 *   DL_COPY_PARTS_ON_ONE_XCD  the parts of a row are placed 8 workgroup ids apart (as the split loss
 *                             kernels do); else row-major
 *   DL_COPY_WAVE_MAJOR        every wave owns `chunks` KiB in one piece (the loss kernels' layout);
 *                             else chunk c of a part belongs to thread c % threads
 *   DL_COPY_LDS_KB(n)         every workgroup also holds n KiB of LDS (n <= 64), which bounds the
 *                             workgroups per CU at 160 / n
 */
#define DL_COPY_PARTS_ON_ONE_XCD 1
#define DL_COPY_WAVE_MAJOR 2
#define DL_COPY_LDS_KB_SHIFT 8
#define DL_COPY_LDS_KB(n) ((n) << DL_COPY_LDS_KB_SHIFT)
int dl_copy_rows(const void* src, void* dst, int64_t n_rows, int64_t row_bytes, int threads, int chunks,
                 int flags, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DISTILL_HIP_H */
