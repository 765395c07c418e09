/*
 * paraattn_hip.h -- C ABI of libparaattn_hip.so (gfx950 / MI355X).
 *
 * The reference (chengzeyi/ParaAttention) is pure Python: its attention ops end
 * in aten CUDA kernels and it has no FFI of its own.  This header is therefore
 * the binding surface a maintainer would target from the reference's op layer;
 * every entry point names the reference interface it stands in for.
 *
 * Conventions
 *  - All pointers are device pointers unless the name ends in _host.
 *  - Nothing here allocates or frees device memory and nothing synchronises:
 *    work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 *    null stream) and the call returns at once.  Outputs and workspaces belong
 *    to the caller and must stay alive until the stream work has run.
 *  - Functions return PA_OK (0) or a negative PA_ERR_* code and never throw or
 *    exit; pa_last_error() gives the text for the calling thread.
 *  - Strides are in elements.  The innermost (head_dim) stride must be 1.
 */
#ifndef PARAATTN_HIP_H
#define PARAATTN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* exported symbol (the library is built with hidden default visibility) */
#define PA_API __attribute__((visibility("default")))

#define PA_OK 0
#define PA_ERR_INVALID (-1)     /* bad argument (null pointer, negative size ...) */
#define PA_ERR_UNSUPPORTED (-2) /* shape / dtype / stride the kernels do not cover */
#define PA_ERR_LAUNCH (-3)      /* HIP reported an error at launch */
#define PA_ERR_WORKSPACE (-4)   /* workspace too small */

/* element types of activations */
#define PA_DTYPE_BF16 0
#define PA_DTYPE_F16 1
#define PA_DTYPE_F32 2

/* ABI version of this header (bumped on any signature change). */
PA_API int pa_abi_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
PA_API const char* pa_last_error(void);

/*
 * Tuning and test aids of the attention launches (no counterpart in the
 * reference, whose aten kernels choose their own variants).  Each knob starts
 * from an environment variable that is read once per process, at the first
 * launch; this call changes it afterwards, for all later launches of the
 * process:
 *   "no_pipe"      PARAATTN_NO_PIPE=1       1: the kernels without 32-bit offset limits
 *   "bm"           PARAATTN_BM=128|256      query rows per workgroup, 0 = chosen per launch
 *   "no_split"     PARAATTN_NO_SPLIT=1      1: no key-split tail
 *   "no_xcd_order" PARAATTN_NO_XCD_ORDER=1  1: block-sparse workgroups in plain order
 *   "bound"        PARAATTN_BOUND=0|1       0 / 1: never / always compute the score bound, -1 = by size
 *   "stream"       PARAATTN_STREAM=0|1      0 / 1: never / wherever possible the kernel with resident workgroups, -1 = by shape
 *   "stream_even"  PARAATTN_STREAM_EVEN=0|1 that kernel's tail cut into shares that begin at the same keys / into equal ranges, -1 = by size
 *   "stream_dyn"   PARAATTN_STREAM_DYN=0|2..6  that kernel's tail in equal ranges, one per workgroup / in that many rounds of ever
 *                                           shorter ranges which the workgroups draw from a counter as they run out of work (so
 *                                           that faster compute units take more), wherever two rounds fit; -1 = 4 rounds from 2048
 *                                           key-tile steps per workgroup on.  Needs 4x the workspace of equal ranges; a call whose
 *                                           workspace is smaller gets equal ranges.  Results do not depend on who drew what.
 *   "stream_solo"  PARAATTN_STREAM_SOLO=1   test aid: a launch all of whose pieces are cut into drawn ranges (fewer pieces than
 *                                           compute units) is computed by one workgroup, which draws every range in turn
 *   "sparse_pair"  PARAATTN_SPARSE_PAIR=1   1: pa_attn_fwd_blocksparse with 128-row query blocks puts two adjacent blocks into one
 *                                           256-row workgroup that walks the union of their key ranges (head_dim 128)
 *   "wave_rows"    PARAATTN_WAVE_ROWS=64    64: the kernel with resident workgroups runs as 4 wavefronts of 64 query rows (one per SIMD,
 *                                           half the LDS reads per flop) instead of 8 wavefronts of 32: the same results bit for
 *                                           bit, slower as measured, kept for comparison
 *   "sparse_order" PARAATTN_SPARSE_ORDER=0  0: block-sparse launches take the query blocks of a head in their own order instead of
 *                                           longest list of key ranges first (1, the default)
 *   "short_keys"   PARAATTN_SHORT_KEYS=0|1  0 / 1: never / wherever it applies the kernel for 449..512 keys per head (head_dim 128,
 *                                           dense), -1 = where a workgroup gets two query tiles or more
 * Returns PA_ERR_INVALID for an unknown name or value.
 */
PA_API int pa_set_tuning(const char* name, int value);

/*
 * Dense scaled-dot-product attention forward.
 *   out[b,h,i,:] = softmax_j(scale * q[b,h,i,:].k[b,h,j,:]) @ v[b,h,j,:]
 *   lse[b,h,i]   = log sum_j exp(scale * q.k)      (natural log, fp32)
 * with j over all keys, or, with is_causal != 0, over keys j <= i (torch's
 * is_causal: the lower-left triangle aligned at the top-left corner).
 * Stands in for para_attn.ops.attention_forward_with_lse
 * (src/para_attn/ops/__init__.py:112-179: the aten flash / efficient / cuDNN
 * forward + [:2]) and, with lse == NULL, for para_attn.ops.attention_forward
 * (src/para_attn/ops/__init__.py:204-223).
 *
 * q [B,H,Sq,D], k,v [B,H,Skv,D], out [B,H,Sq,D]: dtype bf16 or f16, strides
 * {batch, head, seq} in elements, head_dim stride 1, every row start 16-byte
 * aligned.  lse: contiguous fp32 [B,H,Sq] or NULL.  D == 128 (or 64).
 * kv_len: NULL, or int32 [B] device array giving, per batch element, how many
 * leading keys take part (the rest are ignored); this is how the sparse_kv op
 * (src/para_attn/ops/__init__.py:248-299) runs once its mask is a prefix.
 * is_causal: the op's argument of the same name (ops/__init__.py:117, 138).
 */
PA_API int pa_attn_fwd_lse(const void* q, const void* k, const void* v, void* out, float* lse,
                    int dtype, int B, int H, int Sq, int Skv, int D,
                    const int64_t q_strides[3], const int64_t k_strides[3],
                    const int64_t v_strides[3], const int64_t out_strides[3],
                    float scale, const int32_t* kv_len, int is_causal, void* stream);

/*
 * pa_attn_fwd_lse with a workspace lent by the caller.  The reference's op
 * (src/para_attn/ops/__init__.py:112-157) ends in an aten kernel that takes its
 * scratch from torch's allocator; this library allocates nothing, so the caller
 * brings it.  With a workspace of at least pa_attn_fwd_workspace_bytes() bytes
 * (device memory, 16-byte aligned, contents irrelevant before and after) the
 * head_dim-128 kernels cut the query tiles that do not fill a round of the
 * chip's compute units into ranges of key tiles, one per compute unit, and fold
 * their partial results with the same log-sum-exp merge as pa_merge_lse, which
 * removes the idle tail of the launch.
 * On launches of 1e12 flop and more the first 8 KB of the workspace hold a bound
 * of the scores, computed on the device from the largest row norms of q and k
 * (two small launches that read q and k once): where no score can leave
 * [-60, 60] in the log2 domain (models that normalise q and k sit near 16) the
 * kernel variant without a running maximum runs, about 4 % faster; otherwise,
 * and always without a workspace, the variant with it.  Both are launched, and
 * the one the device-side flag does not select returns at once, so nothing is
 * read back by the host.
 * A null or short workspace is not an error: the tail is then cut into as many
 * ranges as the workspace holds, or not at all (as pa_attn_fwd_lse runs).
 * Results are the same to rounding.  Calls that share a workspace must not
 * overlap.
 */
PA_API int pa_attn_fwd_lse_ws(const void* q, const void* k, const void* v, void* out, float* lse,
                       int dtype, int B, int H, int Sq, int Skv, int D,
                       const int64_t q_strides[3], const int64_t k_strides[3],
                       const int64_t v_strides[3], const int64_t out_strides[3],
                       float scale, const int32_t* kv_len, int is_causal, void* workspace,
                       size_t workspace_bytes, void* stream);

/* kinds of attention mask taken by pa_attn_fwd_masked */
#define PA_MASK_BOOL 1 /* bytes; 0 = the key is dropped for that query */
#define PA_MASK_F32 2  /* fp32 bias added to the scaled score */
#define PA_MASK_ACT 3  /* bias in the activation type (bf16 / f16) */

/*
 * Dense attention forward with an attention mask: the attn_mask argument of
 * para_attn.ops.attention_forward_with_lse / attention_forward
 * (src/para_attn/ops/__init__.py:78-87: attn_bias of the efficient backend,
 * :215-223: F.scaled_dot_product_attention), boolean or additive, broadcastable
 * to [B,H,Sq,Skv].  mask_strides = {batch, head, query, key} in elements, 0 on
 * a broadcast dimension.  A query row that keeps no key yields out = 0 and
 * lse = -inf.  Not causal (torch refuses a mask together with is_causal).
 *
 * A boolean mask that only selects keys (head and query strides 0: the text
 * padding masks of src/para_attn/ops/__init__.py:248-299) is scanned on the
 * device; where it keeps a prefix of the keys in every batch element the fast
 * dense kernels run with the counts as kv_len (long launches whose prefixes
 * keep at least 7/8 of the keys everywhere: the kernel with resident
 * workgroups, which plain dense calls use).  Where it has holes (the mask of
 * the reference's sequence-parallel HunyuanVideo adapter, whose text padding
 * lies inside the gathered sequence:
 * context_parallel/diffusers_adapters/hunyuan_video.py:86-100) and the call
 * is one of 3e11 flop or more, the kept K and V rows are gathered into dense
 * copies in the workspace, as the reference's attention_forward_sparse_kv
 * does with index_select (ops/__init__.py:276-296), and the same kernels run
 * on the copies.  Smaller calls with such a mask, and every other mask, run a
 * kernel that reads the mask per score.  The choice is made on the device:
 * nothing is read back, so the call can be captured in a HIP graph.
 * workspace: pa_attn_fwd_masked_workspace_bytes() bytes (16-byte aligned, any
 * contents; from 3e11 flop on it includes the copies of K and V); null or
 * short is not an error: the per-score kernel runs where there is no room.
 */
PA_API int pa_attn_fwd_masked(const void* q, const void* k, const void* v, void* out, float* lse,
                       int dtype, int B, int H, int Sq, int Skv, int D,
                       const int64_t q_strides[3], const int64_t k_strides[3],
                       const int64_t v_strides[3], const int64_t out_strides[3], float scale,
                       const void* mask, int mask_kind, const int64_t mask_strides[4],
                       void* workspace, size_t workspace_bytes, void* stream);

PA_API size_t pa_attn_fwd_masked_workspace_bytes(int B, int H, int Sq, int Skv, int D,
                                          const int64_t k_strides[3], const int64_t v_strides[3]);

/*
 * pa_attn_fwd_lse_ws for callers that cannot allocate device memory or bring
 * a workspace: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference (whose aten
 * kernels take scratch from torch's allocator).  The workspace is a buffer of
 * PA_NOALLOC_SCRATCH_BYTES inside the library's device image, one copy per GPU,
 * held until the process ends; the call allocates and frees nothing.  Same
 * arguments, kernels and results as pa_attn_fwd_lse_ws with a workspace of
 * pa_attn_fwd_workspace_bytes() bytes, except that large problems (see the knob
 * "stream_dyn") keep one tail range per workgroup, the plan pa_attn_fwd_lse_ws
 * itself falls back to when its workspace is too small for drawn ranges; there
 * the two entry points agree to rounding, not bit for bit.  A problem whose
 * launch plan needs more scratch than the buffer holds even so is refused with
 * PA_ERR_WORKSPACE (it is not run unsplit behind the caller's back).  Nothing in the buffer has to survive
 * between calls and nothing has to be cleared; but all calls on one GPU share
 * it, so calls that overlap on one GPU (two streams, two threads) race.
 */
#define PA_NOALLOC_SCRATCH_BYTES (80u << 20)
PA_API int pa_attn_fwd_lse_noalloc(const void* q, const void* k, const void* v, void* out, float* lse,
                            int dtype, int B, int H, int Sq, int Skv, int D,
                            const int64_t q_strides[3], const int64_t k_strides[3],
                            const int64_t v_strides[3], const int64_t out_strides[3],
                            float scale, const int32_t* kv_len, int is_causal, void* stream);

/*
 * One step of a same-GPU ring sweep in one launch: attention of q against one
 * key/value block, folded into the running pair (acc_out, acc_lse) by the
 * log-sum-exp merge of pa_merge_lse inside the attention kernel's epilogue.
 * Replaces, per step of torch's _templated_ring_attention loop as the reference
 * drives it (src/para_attn/para_attn_interface.py:164-197), the attention op
 * (src/para_attn/ops/__init__.py:112-157) plus _SDPAMerger.step: the block's
 * own 16-bit output and the merge pass over it never exist.
 *
 * acc_out: fp32 [B,H,Sq,D] contiguous; acc_lse: fp32 [B,H,Sq]; both updated in
 * place.  first != 0: the pair holds nothing yet and is not read (no need to
 * initialise it).  out == NULL: acc_out receives the folded output.  out != NULL
 * (the last step): the folded output is written to out in `dtype` with
 * out_strides, acc_out is left as it was, acc_lse is the final LSE.
 * workspace: as for pa_attn_fwd_lse_ws (may be NULL).  head_dim 128 with K and
 * V below 4 GiB per (batch, head) only; otherwise PA_ERR_UNSUPPORTED (run
 * pa_attn_fwd_lse and pa_merge_lse instead).
 */
PA_API int pa_attn_fwd_accumulate(const void* q, const void* k, const void* v, float* acc_out,
                           float* acc_lse, void* out, int dtype, int B, int H, int Sq, int Skv,
                           int D, const int64_t q_strides[3], const int64_t k_strides[3],
                           const int64_t v_strides[3], const int64_t out_strides[3], float scale,
                           const int32_t* kv_len, int first, void* workspace,
                           size_t workspace_bytes, void* stream);

/*
 * A whole same-GPU ring sweep in one launch: attention of q against the
 * concatenation of n_blocks key/value blocks that lie at separate addresses
 * (the blocks a ring pass visits, src/para_attn/para_attn_interface.py:164-197:
 * one attention call and one _SDPAMerger.step per block in torch's
 * _templated_ring_attention).  The kernel walks the blocks as one key sequence
 * and carries the softmax state (running maximum, sum, output) across them in
 * registers, so neither the per-block outputs nor the fp32 running pair of
 * pa_attn_fwd_accumulate exist.  Result: out and lse of attention over all
 * n_blocks * block_len keys.
 *
 * k_blocks, v_blocks: host arrays of n_blocks (1..16) device pointers to
 * [B,H,block_len,D] tensors that share k_strides / v_strides; head_dim 128,
 * each block below 4 GiB per (batch, head).  Otherwise PA_ERR_UNSUPPORTED (run
 * pa_attn_fwd_accumulate per block instead).  workspace: as for
 * pa_attn_fwd_lse_ws, of pa_attn_fwd_sweep_workspace_bytes() bytes; may be NULL.
 */
PA_API int pa_attn_fwd_sweep(const void* q, const void* const* k_blocks, const void* const* v_blocks, int n_blocks,
                      int block_len, void* out, float* lse, int dtype, int B, int H, int Sq, int D,
                      const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                      const int64_t out_strides[3], float scale, void* workspace, size_t workspace_bytes,
                      void* stream);

PA_API size_t pa_attn_fwd_sweep_workspace_bytes(int B, int H, int Sq, int n_blocks, int block_len, int D,
                                         const int64_t k_strides[3], const int64_t v_strides[3]);

/*
 * Bytes of workspace pa_attn_fwd_lse_ws and pa_attn_fwd_accumulate can use for this problem on the current
 * device (0: neither partial results nor a score bound would be used): the larger of what a call with and a
 * call without per-batch key counts / is_causal would take.  Depends on the device's CU count; at most about
 * 68 MB on 256 compute units for a call without them (two fp32 partial results of 256 rows per compute unit).
 */
PA_API size_t pa_attn_fwd_workspace_bytes(int B, int H, int Sq, int Skv, int D,
                                   const int64_t k_strides[3], const int64_t v_strides[3]);

/*
 * The same for one particular call: has_kv_len != 0 if it passes per-batch key counts, is_causal as in the
 * call.  An is_causal launch never cuts its keys (its workgroups differ in length) and asks only for the few
 * KB of the score bound; pa_attn_fwd_workspace_bytes() reports the largest of the three plans because it does
 * not see these arguments.  No counterpart in the reference (aten sizes its own scratch).
 */
PA_API size_t pa_attn_fwd_call_workspace_bytes(int B, int H, int Sq, int Skv, int D, const int64_t k_strides[3],
                                        const int64_t v_strides[3], int has_kv_len, int is_causal);

/*
 * Block-sparse attention forward: query block i (of q_block rows, counted from
 * q_lo) attends key block j (of kv_block rows, counted from kv_lo) iff
 * block_mask[hm,i,j] != 0; query rows outside [q_lo, q_lo + nQ*q_block) attend
 * every key, and keys outside [kv_lo, kv_lo + nK*kv_block) are attended by every
 * query.  Equals dense attention with -inf on the dropped tiles.  Replaces the
 * Python loop of para_attn.sparse_attn.StructuredSparseAttnFunc.forward
 * (src/para_attn/sparse_attn.py:74-278: one SDPA launch per run of kept blocks
 * plus one merge each).  Unlike the reference it also returns the LSE.
 *
 * block_mask: uint8 [Hm,nQ,nK] contiguous, Hm == 1 (shared by all heads, the
 * reference's 2-D mask, sparse_attn.py:107) or Hm == H.
 * runs_ws: int32 workspace of at least pa_blocksparse_workspace_bytes() bytes;
 * it receives, per (hm, query segment), the list of key ranges the kernel
 * walks (the mask's runs of kept blocks, merged, exactly as
 * sparse_attn.py:215-234 scans them), and behind the lists the order in which
 * the query blocks of a head are started (the block that keeps most key blocks
 * first; up to 2048 blocks).
 * A query block that keeps no key at all yields out = 0 and lse = -inf.
 */
PA_API int pa_attn_fwd_blocksparse(const void* q, const void* k, const void* v, void* out, float* lse,
                            int dtype, int B, int H, int Sq, int Skv, int D,
                            const int64_t q_strides[3], const int64_t k_strides[3],
                            const int64_t v_strides[3], const int64_t out_strides[3],
                            float scale, const uint8_t* block_mask, int Hm, int nQ, int nK,
                            int q_lo, int q_block, int kv_lo, int kv_block,
                            int32_t* runs_ws, size_t runs_ws_bytes, void* stream);

/* Bytes of runs_ws needed by pa_attn_fwd_blocksparse for a [Hm,nQ,nK] mask. */
PA_API size_t pa_blocksparse_workspace_bytes(int Hm, int nQ, int nK);

/*
 * Only the run extraction of pa_attn_fwd_blocksparse (for tests and for callers
 * that reuse one mask over many calls).  Layout of runs_ws, with
 * nSeg = nQ + 2 (segment 0 = rows left of q_lo, 1..nQ = mask rows, nQ+1 = rows
 * right of the sparse range) and cap = nK/2 + 3:
 *   int32 count[Hm*nSeg], then int32 range[Hm*nSeg][cap][2] as {begin,end} key
 *   indices in ascending order.
 */
PA_API int pa_blocksparse_build_runs(const uint8_t* block_mask, int Hm, int nQ, int nK, int Skv,
                              int kv_lo, int kv_block, int32_t* runs_ws, size_t runs_ws_bytes,
                              void* stream);

/*
 * pa_attn_fwd_blocksparse for a mask that serves many calls (every layer and
 * step of a pipeline under the reference's StructSparseAttnMode,
 * src/para_attn/sparse_attn.py:643-677, uses one mask): `runs` is what
 * pa_blocksparse_build_runs wrote for the same Hm, nQ, nK, Skv, kv_lo and
 * kv_block, and is only read here, so the run extraction (about 9 us at a
 * [24,256,256] mask) is paid once.  The kernels cut every range at Skv and
 * end a walk at the first range beyond it, so a buffer built for a longer
 * key sequence cannot lead them past the tensors; ranges must be ascending
 * and non-negative, as pa_blocksparse_build_runs writes them.
 */
PA_API int pa_attn_fwd_blocksparse_runs(const void* q, const void* k, const void* v, void* out, float* lse,
                                 int dtype, int B, int H, int Sq, int Skv, int D,
                                 const int64_t q_strides[3], const int64_t k_strides[3],
                                 const int64_t v_strides[3], const int64_t out_strides[3],
                                 float scale, int Hm, int nQ, int nK, int q_lo, int q_block,
                                 const int32_t* runs, size_t runs_bytes, void* stream);

/*
 * One step of the ring-attention partial-result merge, fused into one pass:
 *   w       = sigmoid(blk_lse - acc_lse)
 *   out     = acc_out - w * (acc_out - blk_out)
 *   lse_out = acc_lse - logsigmoid(acc_lse - blk_lse)
 * i.e. torch's _SDPAMerger._merge_one (torch/distributed/tensor/experimental/
 * _context_parallel/_attention.py:150-203, the arithmetic the reference drives
 * from src/para_attn/para_attn_interface.py:182-193 and
 * src/para_attn/sparse_attn.py:174-259), computed in fp32.
 *
 * acc_out [rows,D] (acc_dtype), blk_out [rows,D] (blk_dtype), out [rows,D]
 * (out_dtype), all contiguous; acc_lse, blk_lse, lse_out fp32 [rows].  out may
 * alias acc_out when the dtypes match and lse_out may alias acc_lse (in-place
 * step).  Choosing acc_dtype = bf16 folds the merger's first-step cast
 * (_attention.py:209-211) into the step, out_dtype = bf16 folds results()'s
 * final cast (_attention.py:215-223).  D must be a multiple of 8.
 */
PA_API int pa_merge_lse(const void* acc_out, int acc_dtype, const float* acc_lse,
                 const void* blk_out, int blk_dtype, const float* blk_lse,
                 void* out, int out_dtype, float* lse_out,
                 int64_t rows, int D, void* stream);

/*
 * First Block Cache residual-difference reduction:
 *   mean_diff = mean(|prev - cur|), mean_prev = mean(|prev|), ratio = mean_diff / mean_prev
 * with torch's rounding chain for the activation dtype: the difference is
 * rounded to the dtype per element, both means are rounded to the dtype once,
 * and the quotient is rounded to the dtype.  Stands in for the seven torch ops
 * of are_two_tensors_similar (src/para_attn/first_block_cache/utils.py:228-233);
 * the caller keeps `.item() < threshold` (utils.py:234).
 *
 * prev, cur: [n_rows, row_len] views; *_row_stride and *_col_stride in
 * elements (col stride > 1 covers the [..., ::downsample_factor] slice of
 * utils.py:276-278).  ratio_out: one element of `dtype`.  stats_out: NULL or
 * fp32[2] receiving {mean_diff, mean_prev} after rounding to dtype.
 * workspace: at least pa_fbcache_workspace_bytes() bytes, any contents.
 */
PA_API int pa_fbcache_absdiff_ratio(const void* prev, const void* cur, int dtype,
                             int64_t n_rows, int64_t row_len,
                             int64_t prev_row_stride, int64_t prev_col_stride,
                             int64_t cur_row_stride, int64_t cur_col_stride,
                             void* ratio_out, float* stats_out,
                             void* workspace, size_t workspace_bytes, void* stream);

PA_API size_t pa_fbcache_workspace_bytes(void);

/*
 * Fused first-block residual + reduction (neighbours of the reduction in
 * CachedTransformerBlocks.forward, src/para_attn/first_block_cache/utils.py:359-366):
 *   resid = hidden - hidden0      (rounded to dtype, written to resid_out)
 *   ratio as above with cur = resid
 * All tensors contiguous with n elements.  prev may be NULL (first step: only
 * the residual is written, ratio_out is left untouched).
 */
PA_API int pa_fbcache_residual_ratio(const void* hidden, const void* hidden0, const void* prev,
                              void* resid_out, int dtype, int64_t n,
                              void* ratio_out, float* stats_out,
                              void* workspace, size_t workspace_bytes, void* stream);

/*
 * Cache-hit path: out = resid + hidden (src/para_attn/first_block_cache/utils.py:237-259),
 * contiguous, n elements, rounded to dtype.  out may alias hidden.
 */
PA_API int pa_fbcache_apply_residual(const void* resid, const void* hidden, void* out, int dtype,
                              int64_t n, void* stream);

/*
 * TaylorSeer finite differences (src/para_attn/first_block_cache/taylorseer.py:29-38,
 * approximate_derivative): with x_0 = y, for i < n
 *     cur[i] = (x_i - prev[i]) / window,   x_{i+1} = cur[i]
 * in one pass, with torch's eager rounding for 16-bit tensors (the difference
 * and the quotient are each rounded to `dtype`; true division).  prev and cur
 * are host arrays of n device pointers (n <= 4) to contiguous tensors of numel
 * elements, 16-byte aligned; cur[i] must not alias y or prev[j].
 */
PA_API int pa_taylorseer_update(const void* y, const void* const* prev, void* const* cur, int n,
                         int dtype, int64_t numel, float window, void* stream);

/*
 * TaylorSeer extrapolation (taylorseer.py:40-48, approximate_value):
 *     out = 0;  out += coef[i] * deriv[i] * pw[i]   for i < m
 * with coef[i] = (float)(1 / i!) and pw[i] = (float)(elapsed ** i) supplied by
 * the caller (host arrays of m floats, m <= 5), every product and sum rounded
 * to `dtype` as torch's eager ops round them.  hidden != NULL additionally
 * gives out = hidden + value: the cache-hit path of
 * src/para_attn/first_block_cache/utils.py:239-243 in the same pass.  deriv is
 * a host array of m device pointers.  out may alias hidden.
 */
PA_API int pa_taylorseer_value(const void* const* deriv, int m, const float* coef, const float* pw,
                        const void* hidden, void* out, int dtype, int64_t numel, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PARAATTN_HIP_H */
