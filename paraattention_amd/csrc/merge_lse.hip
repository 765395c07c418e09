// Fused ring-attention merge step: one HBM pass instead of the ~10 elementwise
// launches of torch's _SDPAMerger._merge_one
// (torch/distributed/tensor/experimental/_context_parallel/_attention.py:182-183),
// which the reference drives from src/para_attn/para_attn_interface.py:182-193
// and src/para_attn/sparse_attn.py:174-259.
//
// Bandwidth bound: per element 4 B (fp32 acc read) + 2 B (16-bit block read)
// + 4 B (fp32 acc write); per row three fp32 LSE values.

#include "pa_common.h"

namespace pa {

constexpr int MERGE_THREADS = 512;

template <int DT>
struct Elem8;  // 8 consecutive elements of a row

template <>
struct Elem8<PA_DTYPE_F32> {
  static __device__ __forceinline__ void load(const void* base, int64_t idx8, float (&x)[8]) {
    // streaming (non-temporal) loads: every element is read once (+1.5 % against plain loads on operands
    // that come from HBM; no loss on operands the memory-side cache still holds)
    const floatx4* p = (const floatx4*)base + idx8 * 2;
    floatx4 a = __builtin_nontemporal_load(p);
    floatx4 b = __builtin_nontemporal_load(p + 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[i] = a[i];
      x[4 + i] = b[i];
    }
  }
  static __device__ __forceinline__ void store(void* base, int64_t idx8, const float (&x)[8]) {
    floatx4* p = (floatx4*)base + idx8 * 2;
    floatx4 a = {x[0], x[1], x[2], x[3]};
    floatx4 b = {x[4], x[5], x[6], x[7]};
    __builtin_nontemporal_store(a, p);
    __builtin_nontemporal_store(b, p + 1);
  }
};

template <>
struct Elem8<PA_DTYPE_BF16> {
  static __device__ __forceinline__ void load(const void* base, int64_t idx8, float (&x)[8]) {
    u32x4 w = __builtin_nontemporal_load((const u32x4*)base + idx8);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = BF16::lo(w[i]);
      x[2 * i + 1] = BF16::hi(w[i]);
    }
  }
  static __device__ __forceinline__ void store(void* base, int64_t idx8, const float (&x)[8]) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = BF16::pack2(x[2 * i], x[2 * i + 1]);
    __builtin_nontemporal_store(w, (u32x4*)base + idx8);
  }
};

template <>
struct Elem8<PA_DTYPE_F16> {
  static __device__ __forceinline__ void load(const void* base, int64_t idx8, float (&x)[8]) {
    u32x4 w = __builtin_nontemporal_load((const u32x4*)base + idx8);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = F16::lo(w[i]);
      x[2 * i + 1] = F16::hi(w[i]);
    }
  }
  static __device__ __forceinline__ void store(void* base, int64_t idx8, const float (&x)[8]) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = F16::pack2(x[2 * i], x[2 * i + 1]);
    __builtin_nontemporal_store(w, (u32x4*)base + idx8);
  }
};

// The arithmetic of one step for one 8-element chunk (a, b in; r out) and the row's new LSE.
__device__ __forceinline__ void merge_weights(float la, float lb, float& w, float& ln) {
  // w = sigmoid(lb - la); new_lse = la - logsigmoid(la - lb)
  if (la == -INFINITY) {  // nothing accumulated yet for this row: take the block
    w = 1.f;
    ln = lb;
  } else {
    const float x = la - lb;  // may be +inf when the block is empty
    w = 1.f / (1.f + expf(x));
    // logsigmoid(x) = min(x,0) - log1p(exp(-|x|))
    const float ls = fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
    ln = la - ls;
  }
}

// One thread = 8 consecutive elements of one row.  chunks = D / 8 per row.
// Consecutive threads take consecutive chunks of the flat [rows * chunks] list.  An in-place step
// (lse_out == acc_lse) is only safe with this mapping when a row's threads sit in one wavefront
// (chunks divides 64): there the row's loads are all issued before its chunk-0 lane stores the new
// LSE.  The host sends every other in-place step to merge_lse_rows_kernel.
template <int ACC_DT, int BLK_DT, int OUT_DT>
__global__ __launch_bounds__(MERGE_THREADS) void merge_lse_kernel(const void* acc_out,
                                                        const float* acc_lse,
                                                        const void* __restrict__ blk_out,
                                                        const float* __restrict__ blk_lse,
                                                        void* out, float* lse_out, int64_t total8,
                                                        int chunks) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int64_t row = i / chunks;
  const int chunk = (int)(i - row * chunks);
  float a[8], b[8];
  Elem8<ACC_DT>::load(acc_out, i, a);
  Elem8<BLK_DT>::load(blk_out, i, b);
  float w, ln;
  merge_weights(acc_lse[row], blk_lse[row], w, ln);
  float r[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = a[j] - w * (a[j] - b[j]);
  Elem8<OUT_DT>::store(out, i, r);
  if (chunk == 0) lse_out[row] = ln;
}

// The same step for rows whose chunk count does not divide 64 (head_dim 48, 72, 80 ...): a
// workgroup owns rows_per_block whole rows and a barrier stands between every load and every
// store of the workgroup, so no thread of a row can read the LSE its chunk-0 thread has already
// replaced.  Threads beyond rows_per_block * chunks idle.
template <int ACC_DT, int BLK_DT, int OUT_DT>
__global__ __launch_bounds__(MERGE_THREADS) void merge_lse_rows_kernel(const void* acc_out,
                                                             const float* acc_lse,
                                                             const void* blk_out,
                                                             const float* blk_lse, void* out,
                                                             float* lse_out, int64_t rows,
                                                             int chunks, int rows_per_block) {
  const int local_row = (int)threadIdx.x / chunks;
  const int chunk = (int)threadIdx.x - local_row * chunks;
  const int64_t row = (int64_t)blockIdx.x * rows_per_block + local_row;
  const bool active = local_row < rows_per_block && row < rows;
  const int64_t i = row * chunks + chunk;
  float a[8], b[8], w = 0.f, ln = 0.f;
  if (active) {
    Elem8<ACC_DT>::load(acc_out, i, a);
    Elem8<BLK_DT>::load(blk_out, i, b);
    merge_weights(acc_lse[row], blk_lse[row], w, ln);
  }
  __syncthreads();  // every load of the workgroup's rows has returned (w and ln depend on them)
  if (active) {
    float r[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = a[j] - w * (a[j] - b[j]);
    Elem8<OUT_DT>::store(out, i, r);
    if (chunk == 0) lse_out[row] = ln;
  }
}

}  // namespace pa

using namespace pa;

struct MergeShape {
  int64_t rows;
  int chunks;
  bool by_rows;  // whole rows per workgroup with a barrier between loads and stores
};

template <int A, int B_, int O>
static void launch_merge(const void* acc_out, const float* acc_lse, const void* blk_out,
                         const float* blk_lse, void* out, float* lse_out, const MergeShape& sh,
                         hipStream_t stream) {
  // one 8-element chunk per thread, no grid-stride loop: measured fastest (more workgroups in
  // flight beat a capped loop for this read+write stream); the host has checked that the grid fits
  if (sh.by_rows) {
    const int rpb = MERGE_THREADS / sh.chunks;
    const int64_t blocks = (sh.rows + rpb - 1) / rpb;
    hipLaunchKernelGGL((merge_lse_rows_kernel<A, B_, O>), dim3((unsigned)blocks), dim3(MERGE_THREADS), 0, stream,
                       acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh.rows, sh.chunks, rpb);
  } else {
    const int64_t total8 = sh.rows * sh.chunks;
    const int64_t blocks = (total8 + MERGE_THREADS - 1) / MERGE_THREADS;
    hipLaunchKernelGGL((merge_lse_kernel<A, B_, O>), dim3((unsigned)blocks), dim3(MERGE_THREADS), 0, stream,
                       acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, sh.chunks);
  }
}

template <int A, int B_>
static int merge_out(int out_dtype, const void* acc_out, const float* acc_lse, const void* blk_out,
                     const float* blk_lse, void* out, float* lse_out, const MergeShape& sh,
                     hipStream_t s) {
  switch (out_dtype) {
    case PA_DTYPE_F32: launch_merge<A, B_, PA_DTYPE_F32>(acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s); return PA_OK;
    case PA_DTYPE_BF16: launch_merge<A, B_, PA_DTYPE_BF16>(acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s); return PA_OK;
    case PA_DTYPE_F16: launch_merge<A, B_, PA_DTYPE_F16>(acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s); return PA_OK;
  }
  PA_FAIL(PA_ERR_UNSUPPORTED, "merge: bad out dtype %d", out_dtype);
}

template <int A>
static int merge_blk(int blk_dtype, int out_dtype, const void* acc_out, const float* acc_lse,
                     const void* blk_out, const float* blk_lse, void* out, float* lse_out,
                     const MergeShape& sh, hipStream_t s) {
  switch (blk_dtype) {
    case PA_DTYPE_F32: return merge_out<A, PA_DTYPE_F32>(out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s);
    case PA_DTYPE_BF16: return merge_out<A, PA_DTYPE_BF16>(out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s);
    case PA_DTYPE_F16: return merge_out<A, PA_DTYPE_F16>(out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s);
  }
  PA_FAIL(PA_ERR_UNSUPPORTED, "merge: bad block dtype %d", blk_dtype);
}

extern "C" int pa_merge_lse(const void* acc_out, int acc_dtype, const float* acc_lse,
                            const void* blk_out, int blk_dtype, const float* blk_lse, void* out,
                            int out_dtype, float* lse_out, int64_t rows, int D, void* stream) {
  if (!acc_out || !acc_lse || !blk_out || !blk_lse || !out || !lse_out)
    PA_FAIL(PA_ERR_INVALID, "merge: null pointer argument");
  if (rows < 0 || D <= 0) PA_FAIL(PA_ERR_INVALID, "merge: bad sizes rows=%lld D=%d", (long long)rows, D);
  if (D % 8) PA_FAIL(PA_ERR_UNSUPPORTED, "merge: head_dim %d not a multiple of 8", D);
  const void* ptrs[3] = {acc_out, blk_out, out};
  for (int i = 0; i < 3; ++i)
    if (((uintptr_t)ptrs[i]) % 16) PA_FAIL(PA_ERR_UNSUPPORTED, "merge: tensor pointer not 16-byte aligned");
  if (out == acc_out && out_dtype != acc_dtype)
    PA_FAIL(PA_ERR_INVALID, "merge: in-place step needs out dtype == acc dtype");
  if (rows == 0) return PA_OK;
  const int chunks = D / 8;
  if (chunks > MERGE_THREADS) PA_FAIL(PA_ERR_UNSUPPORTED, "merge: head_dim %d too large (at most %d)", D, 8 * MERGE_THREADS);
  // An in-place step whose rows straddle wavefronts takes the kernel that keeps a row inside one
  // workgroup behind a barrier; everything else the flat one-chunk-per-thread kernel.
  const bool aliased = (const void*)lse_out == (const void*)acc_lse || out == acc_out;
  MergeShape sh = {rows, chunks, aliased && (64 % chunks) != 0};
  const int64_t blocks = sh.by_rows ? (rows + MERGE_THREADS / chunks - 1) / (MERGE_THREADS / chunks)
                                    : (rows * chunks + MERGE_THREADS - 1) / MERGE_THREADS;
  if (blocks > 0x7fffffffLL) PA_FAIL(PA_ERR_UNSUPPORTED, "merge: %lld rows of head_dim %d exceed the grid", (long long)rows, D);
  hipStream_t s = (hipStream_t)stream;
  int rc;
  switch (acc_dtype) {
    case PA_DTYPE_F32: rc = merge_blk<PA_DTYPE_F32>(blk_dtype, out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s); break;
    case PA_DTYPE_BF16: rc = merge_blk<PA_DTYPE_BF16>(blk_dtype, out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s); break;
    case PA_DTYPE_F16: rc = merge_blk<PA_DTYPE_F16>(blk_dtype, out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, sh, s); break;
    default: PA_FAIL(PA_ERR_UNSUPPORTED, "merge: bad acc dtype %d", acc_dtype);
  }
  if (rc) return rc;
  PA_CHECK_LAUNCH("merge_lse_kernel");
  return PA_OK;
}
