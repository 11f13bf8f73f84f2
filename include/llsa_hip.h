/*
 * libllsa_hip.so -- C ABI of the MI355X (gfx950) implementation of the llsa_l1 / llsa_l2
 * hot path of SingleZombie/LLSA (log-linear sparse attention on Z-ordered tokens).
 *
 * The reference has no FFI: its boundary is a Python operator API whose launchers take
 * torch tensors and start Triton kernels (the modules of src/llsa/kernel/torch_op calling
 * those of src/llsa/kernel/triton).  Each entry point below replaces one of those launchers;
 * the comment on it names the launcher (file:line in the reference checkout).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is allocated here
 *   - tensors are bf16 (the MFMA kernels) unless a `dtype` argument says otherwise
 *   - strides are in ELEMENTS; the innermost (channel) stride is always 1 and every row
 *     start must be 16-byte aligned
 *   - the head dimension D is 64 and the block size is 16 in every attention/selection
 *     kernel (the only values the reference's configs use); llsa_mean_pool_* are general
 *   - indices are int32 block ids
 *   - work is enqueued on `stream` (a hipStream_t passed as void*); no host sync
 *   - return value: 0 on success, negative on a rejected argument or a launch error;
 *     llsa_last_error_string() describes the last failure on the calling thread
 *
 * Operand tiles ("xr", "xt" below).  The attention kernels do not read K/V/Q/dO row-major: a
 * (B,H,n,64) tensor is cut into blocks of 16 rows and every block (1024 elements) is stored
 * in the order the 64 lanes of a wave consume it as an MFMA operand, so that each operand
 * load is one contiguous, fully coalesced access.  Element (row t of the block, channel c):
 *   R tile (products that contract over channels: Q.K^T, dO.V^T)
 *        offset = ((c >> 3) * 16 + t) * 8 + (c & 7)
 *   T tile (products that contract over the block's 16 tokens: P.V, dS.K, P^T.dO, dS^T.Q)
 *        offset = (((c >> 4) * 4 + (t >> 2)) * 16 + (c & 15)) * 4 + (t & 3)
 * Tiled tensors are (B,H,n/16,1024) contiguous.  llsa_pool_pyramid_fwd writes them.  Only the
 * forward's P.V product reads T tiles from memory (of v and the pooled v); the backward
 * kernels fetch R tiles only and produce the token-major orientation on chip with the
 * transposing LDS read of gfx950.
 */
#ifndef LLSA_HIP_H
#define LLSA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LLSA_DTYPE_BF16 0
#define LLSA_DTYPE_F32 1

#define LLSA_ABI_VERSION 203     /* changes with every change of a signature or argument structure below */
int llsa_version(void);          /* LLSA_ABI_VERSION of the built library                                    */
const char* llsa_last_error_string(void);

/* ------------------------------------------------------------------------------------------
 * Pooling pyramid.  Replaces the 3 (l1) / 6 (l2) launches of mean_pool1d
 * (kernel/triton/mean_pool.py:129-148, called from torch_op/flash_sparse_attention_res_1.py:42-44
 * and ..._res_2.py:49-55) and, when `freq` is given, my_rope_fn on the same tensor
 * (kernel/triton/rope.py:100-127) in one pass over the input.  One launch serves up to 4
 * tensors.  Rounding follows the reference: the accumulator has the tensor dtype, summed in
 * token order.
 * With `gamma` the rows are first RMS-normalised over the 64 channels,
 *     x <- bf16( float(x) * rsqrt(mean(float(x)^2) + eps) * gamma ),
 * which is the qk-norm the reference's attention processor applies before the RoPE
 * (models/rope_dit_transformer_2d.py:215-219: attn.norm_q / attn.norm_k, diffusers' RMSNorm
 * with an fp32 weight, result cast back to the input dtype).
 * ---------------------------------------------------------------------------------------- */
typedef struct llsa_pool_item {
    const void* x;          /* (B,H,n,64) bf16, strides below                                   */
    int64_t sxb, sxh, sxn;
    int32_t n;              /* rows of this item, multiple of 16                                */
    int32_t rope;           /* rotate x with `freq` first                                       */
    void* y1;               /* (B,H,n/16,64)   mean over 16 rows, contiguous, or NULL           */
    void* y2;               /* (B,H,n/256,64)  mean over 16 rows of y1, or NULL (n % 256 == 0)  */
    void* xr;               /* (B,H,n/16,1024)  R tiles of (rotated) x, or NULL                 */
    void* xt;               /* (B,H,n/16,1024)  T tiles of (rotated) x, or NULL                 */
    void* y1r;              /* (B,H,n/256,1024) R tiles of y1, or NULL (n % 256 == 0)           */
    void* y1t;              /* (B,H,n/256,1024) T tiles of y1, or NULL (n % 256 == 0)           */
    void* xrot;             /* (B,H,n,64) contiguous copy of the normalised / rotated x, or NULL */
    const float* gamma;     /* (64) fp32 or NULL: RMS-normalise every row first (see below)     */
    float eps;
    int32_t reserved;       /* 0                                                                */
    void* y2r;              /* (B,H,n/4096,1024) R tiles of y2, or NULL (n % 4096 == 0)         */
    void* y2t;              /* (B,H,n/4096,1024) T tiles of y2, or NULL (n % 4096 == 0)         */
} llsa_pool_item;

int llsa_pool_pyramid_fwd(const llsa_pool_item* items, int n_items, const void* freq /* (n,64) bf16 or NULL */,
                          int B, int H, void* stream);

/* General mean_pool1d forward / backward, layout 'bhsc' (mean_pool.py:6-58,129-165); the
 * 'bsc' layout (mean_pool.py:61-110,168-206) is the same call with H = 1.  Any K dividing S,
 * any C, bf16 or fp32, arbitrary strides (4 element strides each). */
int llsa_mean_pool_fwd(const void* x, const int64_t* sx, void* y, const int64_t* sy,
                       int B, int H, int S, int C, int K, int dtype, void* stream);
int llsa_mean_pool_bwd(const void* dy, const int64_t* sdy, void* dx, const int64_t* sdx,
                       int B, int H, int S_out, int C, int K, int dtype, void* stream);

/* What autograd does after the operator's backward: out = rn(dx + rn(g1 / 16)) per token with
 * g1 = dy1 (l1) or rn(dy1 + rn(dy2 / 16)) (l2), i.e. mean_pool backward (mean_pool.py:150-165)
 * plus the gradient accumulation into k / v, in one pass; with `freq` the result is then
 * rotated back (rope.py:130-145).  out may alias dx. */
int llsa_pool_bwd_accum(const void* dx, const int64_t* sdx /*3*/, const void* dy1, const void* dy2 /* or NULL */,
                        void* out, const int64_t* sout /*3*/, const void* freq /* or NULL */,
                        int B, int H, int N, void* stream);

/* Backward of the RMS normalisation above: dy, x (B,H,N,64) bf16 with strides, gamma (64) fp32;
 * dx (B,H,N,64) bf16 = rstd * (g - xn * mean(g * xn)) with xn = x * rstd, g = dy * gamma, and
 * dgamma (64) fp32 = sum over all rows of dy * xn.  `partials` is scratch of
 * llsa_rmsnorm_bwd_partials(B,H,N) floats; the sum over rows is taken in a fixed order. */
int64_t llsa_rmsnorm_bwd_partials(int B, int H, int N);
int llsa_rmsnorm_bwd(const void* dy, const int64_t* sdy /*3*/, const void* x, const int64_t* sx /*3*/, const float* gamma,
                     float eps, void* dx, const int64_t* sdx /*3*/, float* dgamma, float* partials,
                     int B, int H, int N, void* stream);

/* The same backward with the partial sums in a static device array inside the library instead of a
 * caller-owned buffer.  It has no counterpart in the reference; it is for callers that cannot
 * allocate device memory: a step that is being captured into a HIP graph, a tight serving loop,
 * a harness that forbids hipMalloc.  Limits and rules:
 *   - B * H * ceil(N / 256) * 64 <= LLSA_STATIC_PARTIALS_MAX (1 MiB of fp32), else the call is
 *     rejected with an error that names the limit;
 *   - the first call on a device looks up the array's address there (no allocation, but do it
 *     once outside a graph capture); the device of `stream` must be the current device;
 *   - every call on one GPU uses the same array: calls that overlap on one GPU (two streams,
 *     two threads) race on it.  Calls on one stream are ordered and safe.
 * Results are bit-identical to llsa_rmsnorm_bwd's. */
#define LLSA_STATIC_PARTIALS_MAX 262144
int llsa_rmsnorm_bwd_static(const void* dy, const int64_t* sdy /*3*/, const void* x, const int64_t* sx /*3*/, const float* gamma,
                            float eps, void* dx, const int64_t* sdx /*3*/, float* dgamma,
                            int B, int H, int N, void* stream);

/* Token permutation at the model's entry and exit (models/rope_dit_transformer_2d.py:963-965,
 * 1028-1030: hidden_states[:, fwd_perm, :] and hidden_states[:, bwd_perm, :]), and the one after
 * the REPA pooling (:1020).  y[b, i, :] = x[b, index[i], :] for b < B, i < n_out; rows are
 * row_bytes long (a multiple of 16) and contiguous inside a batch, batches are x_batch_bytes /
 * y_batch_bytes apart.  index is int32 on the device; an entry outside [0, n_in) gives zeros.
 * The backward of a permutation is the same call with the inverse permutation. */
int llsa_gather_rows(const void* x, void* y, const int32_t* index, int B, int n_out, int n_in, int row_bytes,
                     int64_t x_batch_bytes, int64_t y_batch_bytes, void* stream);

/* 2-D RoPE rotation, forward and backward (rope.py:6-97,100-145).  freq is (S,64) with
 * [sin, cos] interleaved; arithmetic is rounded to bf16 after every operation. */
int llsa_rope_fwd(const void* x, const int64_t* sx /*3*/, const void* freq, void* y, const int64_t* sy /*3*/,
                  int B, int H, int S, void* stream);
int llsa_rope_bwd(const void* dy, const int64_t* sdy /*3*/, const void* freq, void* dx, const int64_t* sdx /*3*/,
                  int B, int H, int S, void* stream);

/* ------------------------------------------------------------------------------------------
 * Selection.
 * llsa_topk_dense replaces gen_sparse_indices (kernel/triton/topk.py:6-9): scores pq.pk^T are
 * rounded to bf16 when round_scores != 0 (the reference's matmul returns the input dtype),
 * top-T per row, descending, equal scores -> smaller index (torch.topk leaves that order
 * unspecified; this library fixes it).  pq, pk (B,H,n,64) contiguous, out (B,H,n,T) int32.
 * llsa_topk_sparse replaces compute_topk_indices_sparse (topk.py:172-197): the candidates of
 * the 16 rows of parent block G are the level-1 key blocks parent_idx[G][a]*16 + b; fp32
 * scores; descending, ties -> smaller index (topk.py:155-164).
 * ---------------------------------------------------------------------------------------- */
int llsa_topk_dense(const void* pq, const void* pk, int32_t* out_idx, int B, int H, int n, int T,
                    int round_scores, void* stream);
int llsa_topk_sparse(const void* pq, const void* pk, const int32_t* parent_idx, int32_t* out_idx,
                     int B, int H, int N1, int T, int T2, void* stream);
/* llsa_topk_dense on the parent level followed by llsa_topk_sparse under its result, in one launch
 * (every workgroup of the second selection first selects its own parent row): the same two results,
 * parent_out (B,H,N1/16,T2) and out_idx (B,H,N1,T).  pq_parent, pk_parent (B,H,N1/16,64) are the pooled
 * rows one level above pq, pk (B,H,N1,64).  N1/16 may not exceed llsa_topk_cascade_max_parents(). */
int llsa_topk_cascade(const void* pq_parent, const void* pk_parent, int32_t* parent_out, const void* pq, const void* pk,
                      int32_t* out_idx, int B, int H, int N1, int T, int T2, void* stream);
int llsa_topk_cascade_max_parents(void);

/* ------------------------------------------------------------------------------------------
 * The hierarchy.  Pooled level l = 1 .. levels: its tokens are means of 16^l input tokens and weigh
 * 16^l in the soft-max (token_weight, token_weight_2 of the reference for l = 1, 2).  A block of a
 * level is 16 of its tokens.  A query reads: the T fine blocks its query block selected (idx); at
 * every level l < levels the lvl[l-1].T blocks of that level which its group of 16^(l+1) queries
 * selected (lvl[l-1].sel -- the reference's p_indices is level 1 of llsa_l2); and every block of the
 * coarsest level.  levels = 1 is llsa_l1 (sparse_attention_res_1.py), levels = 2 llsa_l2
 * (sparse_attention_res_2.py); deeper hierarchies have no counterpart in the reference and continue
 * the scheme by induction on sparse_attention_res_2.py:94-149.  The coarsest level is walked in
 * groups of four blocks: N must be a multiple of 64 * 16^levels.  Indices outside their range are
 * clamped into it; a row of idx that names a block twice counts it twice in the forward and in dq
 * (as the reference's gather does) -- the K-side gradients need distinct entries, see
 * llsa_transpose_indices.
 * ---------------------------------------------------------------------------------------- */
#define LLSA_MAX_LEVELS 4
#define LLSA_POOLED_TOPK_MAX 56     /* the T of the pooled levels below the coarsest may add up to this much (forward and backward) */

typedef struct llsa_fwd_level {
    const void* kr;                            /* (B,H,N/16^(l+1),1024) R tiles of the level's pooled k    */
    const void* vt;                            /* (B,H,N/16^(l+1),1024) T tiles of the level's pooled v    */
    const int32_t* sel;                        /* (B,H,N/16^(l+1),T) blocks of this level selected by every group
                                                  of 16^(l+1) queries; NULL at the coarsest level          */
    int32_t T;                                 /* multiple of 4; ignored at the coarsest level             */
    float w;                                   /* weight of one token of this level (> 0)                  */
} llsa_fwd_level;

/* ------------------------------------------------------------------------------------------
 * Forward.  Replaces sparse_indices_attn_res_fwd (sparse_attention_res_1.py:123-150) when
 * levels == 1 and sparse_indices_attn_res_2_2_fwd (sparse_attention_res_2.py:166-199) when
 * levels == 2.
 * ---------------------------------------------------------------------------------------- */
typedef struct llsa_attn_fwd_args {
    const void* qr;                            /* (B,H,N/16,1024)   R tiles of q                  */
    const void* kr;                            /* (B,H,N/16,1024)   R tiles of k                  */
    const void* vt;                            /* (B,H,N/16,1024)   T tiles of v                  */
    const int32_t* idx;                        /* (B,H,N/16,T)   selected fine blocks             */
    void* o;        int64_t sob, soh, son;     /* (B,H,N,64) out                                  */
    float* lse;                                /* (B,H,N) out, m + log(l)                          */
    int32_t B, H, N, T, levels, reserved;
    llsa_fwd_level lvl[LLSA_MAX_LEVELS];       /* lvl[l - 1] = pooled level l                     */
} llsa_attn_fwd_args;

int llsa_attn_fwd(const llsa_attn_fwd_args* a, void* stream);

/* ------------------------------------------------------------------------------------------
 * Index transpose.  Replaces transpose_indices (kernel/triton/indices_transpose.py:104-109):
 * idx (B,H,Mb,T) -> offsets (B,H,Kb+1) with offsets[0] = 0 and flat (B,H,Mb*T); segment n of
 * flat lists the query blocks that selected key block n in ASCENDING order (the reference's
 * order is whatever its atomics produce).  Rows of idx must hold distinct values in [0, Kb): a
 * value named twice in a row collapses to one list entry and leaves the tail of the segment
 * undefined (nothing is read or written out of bounds).
 * With `inv` (B,H,Mb,T) the inverse is written too: inv[q][t] = position in flat of the entry
 * that (query block q, slot t) became.  llsa_attn_bwd needs it for the selections of the pooled
 * levels (lvl[].sel): the partial sums of a key block are stored at the positions of its list.
 * ---------------------------------------------------------------------------------------- */
int llsa_transpose_indices(const int32_t* idx, int32_t* offsets, int32_t* flat, int32_t* work /* or NULL */,
                           int32_t* inv /* or NULL */, int B, int H, int Mb, int Kb, int T, int chunk, void* stream);

/* The same for several index tensors of one operator call (the selections of all its levels) with as few launches as
 * possible: every job is what one llsa_transpose_indices call takes, all jobs share B and H.  When every job is small
 * enough for a workgroup to hold a bitmap of (key block, query block) in LDS -- roughly Mb * Kb <= 2^20 -- all of them
 * are done in ONE launch, already sorted; otherwise the large ones go job by job, as llsa_transpose_indices does them,
 * and so do the small ones whose bitmaps are more than 32 KB.  It has no counterpart of its own in
 * the reference, which calls transpose_indices once per index tensor (sparse_attention_res_2.py:593-594). */
typedef struct llsa_transpose_job {
    const int32_t* idx; int32_t* offsets; int32_t* flat; int32_t* work /* or NULL */; int32_t* inv /* or NULL */;
    int32_t Mb, Kb, T, chunk;
} llsa_transpose_job;
int llsa_transpose_indices_multi(const llsa_transpose_job* jobs, int n_jobs, int B, int H, void* stream);

/* Work list for the K-side backward kernels, written by llsa_transpose_indices when `work` is
 * given: every key block's segment is cut into chunks of at most `chunk` entries, one work item
 * per chunk, so that a key block selected by very many query blocks is spread over many waves
 * (the reference walks each segment serially, sparse_attention_res_1.py:300-322).  `work` is
 * (B,H,llsa_work_list_len(Mb,Kb,T,chunk)) int32, 16-byte aligned; llsa_attn_bwd needs the
 * work list of idx with chunk = llsa_fine_chunk(N) (the pooled levels need none).  Per (b,h), in int32:
 *   [0] items, [1] partial-sum slots, [2] key blocks with more than one chunk, [3] 0
 *   [4 + 4i ..]              item i = {key block, first entry in flat, entries, partial-sum slot or -1};
 *                            items with more than chunk/2 entries come first
 *   [4 + 4*max_items + 4j ..] j-th key block with more than one chunk = {key block, first slot, chunks, 0}
 *   then Kb ints (rounded up to a multiple of 4) that the transpose itself uses as scratch
 * with max_items = Mb*T/chunk + Kb; every key block has at least one item. */
int64_t llsa_work_list_len(int Mb, int Kb, int T, int chunk);
/* Entries per work item of the fine level for a sequence of N tokens: 64 up to N = 16384, where a step is short and a long
 * item would end it alone, 256 beyond, where fewer items and fewer partial sums count for more (N = 65536: -2 %,
 * N = 262144: -3 % of the step).  Never more than LLSA_CHUNK_FINE_MAX.  No counterpart in the reference, which walks a key
 * block's whole list in one program (sparse_attention_res_1.py:300-322). */
int llsa_fine_chunk(int N);
#define LLSA_CHUNK_FINE_MAX 256

/* ------------------------------------------------------------------------------------------
 * Backward.  Replaces sparse_indices_attn_res_scatter_bwd_v2 (sparse_attention_res_1.py:403-471)
 * and sparse_indices_attn_res_scatter_2_2_bwd_v2 (sparse_attention_res_2.py:578-681): the
 * delta pre-pass, dQ, dK/dV over the transposed index, the gradients of the pooled levels under
 * an ancestor's selection and of the dense coarsest level.  The k*scale temporaries of the
 * reference (:420-422) do not exist here.  Levels as in the forward; lvl[l-1].gw is the factor used
 * on the path to the level's own gradient: the reference uses 1 for the one level of llsa_l1
 * (sparse_attention_res_1.py:388-389) where its forward and its dq use token_weight, and the
 * weight itself everywhere in llsa_l2 (sparse_attention_res_2.py:478, :564).
 * ---------------------------------------------------------------------------------------- */
typedef struct llsa_bwd_level {
    const void* kr; const void* vr;              /* (B,H,N/16^(l+1),1024) R tiles of the level's pooled k, v      */
    const int32_t* sel;                          /* as in the forward; NULL at the coarsest level                  */
    const int32_t* off; const int32_t* inv;      /* transposed sel (Kb = N/16^(l+1)): offsets and inverse positions */
    void* dk; void* dv;                          /* (B,H,N/16^l,64) contiguous out: gradients of the pooled k, v    */
    int32_t T;
    float w, gw;
    int32_t reserved;
} llsa_bwd_level;

typedef struct llsa_attn_bwd_args {
    const void* dout; int64_t sdob, sdoh, sdon;  /* (B,H,N,64) upstream gradient                 */
    const void* o;    int64_t sob, soh, son;     /* (B,H,N,64) forward output                     */
    const float* lse;                            /* (B,H,N)                                       */
    const void* qr;  const void* kr;  const void* vr;   /* R tiles of q, k, v  (B,H,N/16,1024)    */
    const int32_t* idx;                          /* (B,H,N/16,T) selected fine blocks             */
    const int32_t* off;  const int32_t* flat;  const int32_t* work;    /* transposed idx  (Kb = N/16)     */
    void* dq; int64_t sdqb, sdqh, sdqn;
    void* dk; int64_t sdkb, sdkh, sdkn;
    void* dv; int64_t sdvb, sdvh, sdvn;
    void* workspace; int64_t workspace_bytes;    /* see llsa_attn_bwd_workspace_bytes             */
    const void* freq_dq;                         /* (N,64) or NULL: rotate dq back (fused rope)   */
    const void* freq_dk;                         /* (N,64) or NULL: rotate dk back; needs fold_pooled */
    int32_t B, H, N, T, levels;
    int32_t stages;                              /* 0 = everything; else a mask of LLSA_BWD_* (see below) */
    int32_t fold_pooled;                         /* 0: dk, dv are the fine-token gradients only, as the
                                                    reference's kernels return them (mean_pool1d's backward
                                                    and autograd add the pooled gradients afterwards).  1: dk, dv
                                                    also receive the pooled gradients of their blocks, with the
                                                    same bf16 roundings (= llsa_pool_bwd_accum, level by level),
                                                    and dk is rotated back with freq_dk                */
    int32_t reserved;
    llsa_bwd_level lvl[LLSA_MAX_LEVELS];         /* lvl[l - 1] = pooled level l                     */
} llsa_attn_bwd_args;

/* `stages` is a diagnostic for timing kernels one at a time: a mask other than 0 launches only the named kernels.
 * Every stage but LLSA_BWD_DQ reads what that stage left in the workspace (delta, the R tiles of dout), and the
 * reductions read partial sums the K-side stages left there: a mask is only meaningful on a workspace that a
 * complete call (stages = 0) with the same arguments has filled before, and only its duration is of use. */
#define LLSA_BWD_DQ 2       /* dq; also delta = rowsum(o * dout) and the R tiles of dout, which the
                               stages below read from the workspace                              */
#define LLSA_BWD_DKV 4      /* dK/dV of the fine tokens                                          */
#define LLSA_BWD_DPKV1 8    /* gradients of the pooled levels below the coarsest (levels >= 2)   */
#define LLSA_BWD_DENSE 16   /* dense coarsest pooled gradients (partials + reduction)            */
#define LLSA_BWD_NO_REDUCE 32 /* with an explicit mask: leave out the reductions of partial sums (results
                                 are then incomplete; for timing the K-side kernels alone)          */

/* topk: `levels` entries, topk[0] = T of the fine blocks, topk[l] = lvl[l-1].T for l < levels */
int64_t llsa_attn_bwd_workspace_bytes(int B, int H, int N, const int32_t* topk, int levels);
int llsa_attn_bwd(const llsa_attn_bwd_args* a, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LLSA_HIP_H */
