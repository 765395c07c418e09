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
    const floatx4* p = (const floatx4*)base + idx8 * 2;
    floatx4 a = p[0];
    floatx4 b = p[1];
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
    u32x4 w = ((const u32x4*)base)[idx8];
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
    u32x4 w = ((const u32x4*)base)[idx8];
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

// One thread = 8 consecutive elements of one row.  chunks = D / 8 per row.
template <int ACC_DT, int BLK_DT, int OUT_DT>
__global__ __launch_bounds__(MERGE_THREADS) void merge_lse_kernel(const void* acc_out,
                                                        const float* acc_lse,
                                                        const void* __restrict__ blk_out,
                                                        const float* __restrict__ blk_lse,
                                                        void* out, float* lse_out, int64_t total8,
                                                        int chunks) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total8; i += stride) {
    const int64_t row = i / chunks;
    const int chunk = (int)(i - row * chunks);
    float a[8], b[8];
    Elem8<ACC_DT>::load(acc_out, i, a);
    Elem8<BLK_DT>::load(blk_out, i, b);
    const float la = acc_lse[row];
    const float lb = blk_lse[row];
    // w = sigmoid(lb - la); new_lse = la - logsigmoid(la - lb)
    float w, ln;
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
    float r[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = a[j] - w * (a[j] - b[j]);
    Elem8<OUT_DT>::store(out, i, r);
    if (chunk == 0) lse_out[row] = ln;
  }
}

}  // namespace pa

using namespace pa;

template <int A, int B_, int O>
static void launch_merge(const void* acc_out, const float* acc_lse, const void* blk_out,
                         const float* blk_lse, void* out, float* lse_out, int64_t total8, int chunks,
                         hipStream_t stream) {
  // one 8-element chunk per thread, no grid cap: measured fastest (more workgroups in flight
  // beat a capped grid-stride loop for this read+write stream)
  int64_t blocks = (total8 + MERGE_THREADS - 1) / MERGE_THREADS;
  if (blocks > 0x7fffffffLL) blocks = 0x7fffffffLL;
  hipLaunchKernelGGL((merge_lse_kernel<A, B_, O>), dim3((unsigned)blocks), dim3(MERGE_THREADS), 0, stream,
                     acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks);
}

template <int A, int B_>
static int merge_out(int out_dtype, const void* acc_out, const float* acc_lse, const void* blk_out,
                     const float* blk_lse, void* out, float* lse_out, int64_t total8, int chunks,
                     hipStream_t s) {
  switch (out_dtype) {
    case PA_DTYPE_F32: launch_merge<A, B_, PA_DTYPE_F32>(acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s); return PA_OK;
    case PA_DTYPE_BF16: launch_merge<A, B_, PA_DTYPE_BF16>(acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s); return PA_OK;
    case PA_DTYPE_F16: launch_merge<A, B_, PA_DTYPE_F16>(acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s); return PA_OK;
  }
  PA_FAIL(PA_ERR_UNSUPPORTED, "merge: bad out dtype %d", out_dtype);
}

template <int A>
static int merge_blk(int blk_dtype, int out_dtype, const void* acc_out, const float* acc_lse,
                     const void* blk_out, const float* blk_lse, void* out, float* lse_out,
                     int64_t total8, int chunks, hipStream_t s) {
  switch (blk_dtype) {
    case PA_DTYPE_F32: return merge_out<A, PA_DTYPE_F32>(out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s);
    case PA_DTYPE_BF16: return merge_out<A, PA_DTYPE_BF16>(out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s);
    case PA_DTYPE_F16: return merge_out<A, PA_DTYPE_F16>(out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s);
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
  const int64_t total8 = rows * chunks;
  hipStream_t s = (hipStream_t)stream;
  int rc;
  switch (acc_dtype) {
    case PA_DTYPE_F32: rc = merge_blk<PA_DTYPE_F32>(blk_dtype, out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s); break;
    case PA_DTYPE_BF16: rc = merge_blk<PA_DTYPE_BF16>(blk_dtype, out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s); break;
    case PA_DTYPE_F16: rc = merge_blk<PA_DTYPE_F16>(blk_dtype, out_dtype, acc_out, acc_lse, blk_out, blk_lse, out, lse_out, total8, chunks, s); break;
    default: PA_FAIL(PA_ERR_UNSUPPORTED, "merge: bad acc dtype %d", acc_dtype);
  }
  if (rc) return rc;
  PA_CHECK_LAUNCH("merge_lse_kernel");
  return PA_OK;
}
