// First Block Cache residual-difference reduction in one HBM pass.
//
// Replaces the seven torch launches of are_two_tensors_similar
// (src/para_attn/first_block_cache/utils.py:228-233):
//   mean_diff = (t1 - t2).abs().mean(); mean_t1 = t1.abs().mean(); mean_diff / mean_t1
// and keeps torch's rounding chain for 16-bit activations: t1 - t2 is rounded
// to the activation type per element, each mean is accumulated wide and rounded
// once, the quotient is rounded once.
//
// Bandwidth bound: 2 reads of 2 B per element, nothing written but one scalar.
// Every thread keeps fp32 partial sums over a few hundred elements, a
// workgroup folds them in fp64, and the last workgroup to finish (ticket
// counter in the workspace) adds the per-workgroup partials in a fixed order,
// so the result does not depend on scheduling.

#include "pa_common.h"

namespace pa {

constexpr int FB_THREADS = 256;
constexpr int FB_MAX_BLOCKS = 4096;

struct FbWorkspace {
  unsigned int ticket;  // zero between calls
  unsigned int pad[3];
  double part[FB_MAX_BLOCKS][2];
};

template <int DT>
struct Act;
template <>
struct Act<PA_DTYPE_BF16> {
  static constexpr int VEC = 8;  // elements per 16-byte load
  // |round(a - b)| and |a| for a packed pair
  static __device__ __forceinline__ void pair(uint32_t wa, uint32_t wb, float& sd, float& sa) {
    const float a0 = BF16::lo(wa), a1 = BF16::hi(wa);
    const float d0 = a0 - BF16::lo(wb), d1 = a1 - BF16::hi(wb);
    const uint32_t r = BF16::pack2(d0, d1) & 0x7fff7fffu;
    sd += BF16::lo(r) + BF16::hi(r);
    sa += fabsf(a0) + fabsf(a1);
  }
  static __device__ __forceinline__ float load1(const void* p, int64_t i) {
    return __uint_as_float((uint32_t)((const uint16_t*)p)[i] << 16);
  }
  static __device__ __forceinline__ float round1(float x) { return BF16::lo(BF16::pack2(x, 0.f)); }
  static __device__ __forceinline__ void store1(void* p, float x) {
    *(uint16_t*)p = (uint16_t)(BF16::pack2(x, 0.f) & 0xffffu);
  }
};
template <>
struct Act<PA_DTYPE_F16> {
  static constexpr int VEC = 8;
  static __device__ __forceinline__ void pair(uint32_t wa, uint32_t wb, float& sd, float& sa) {
    const float a0 = F16::lo(wa), a1 = F16::hi(wa);
    const float d0 = a0 - F16::lo(wb), d1 = a1 - F16::hi(wb);
    const uint32_t r = F16::pack2(d0, d1) & 0x7fff7fffu;
    sd += F16::lo(r) + F16::hi(r);
    sa += fabsf(a0) + fabsf(a1);
  }
  static __device__ __forceinline__ float load1(const void* p, int64_t i) {
    return (float)((const _Float16*)p)[i];
  }
  static __device__ __forceinline__ float round1(float x) { return (float)(_Float16)x; }
  static __device__ __forceinline__ void store1(void* p, float x) { *(_Float16*)p = (_Float16)x; }
};
template <>
struct Act<PA_DTYPE_F32> {
  static constexpr int VEC = 4;
  static __device__ __forceinline__ float load1(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ float round1(float x) { return x; }
  static __device__ __forceinline__ void store1(void* p, float x) { *(float*)p = x; }
};

// accumulate one 16-byte vector of each operand
template <int DT>
__device__ __forceinline__ void accum_vec(const u32x4& a, const u32x4& b, float& sd, float& sa) {
  if constexpr (DT == PA_DTYPE_F32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float x = __uint_as_float(a[i]);
      sd += fabsf(x - __uint_as_float(b[i]));
      sa += fabsf(x);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) Act<DT>::pair(a[i], b[i], sd, sa);
  }
}

// Folds the workgroup's sums, publishes them, and lets the last workgroup finish.
template <int DT>
__device__ __forceinline__ void finish(float sd, float sa, double count, FbWorkspace* ws,
                                       void* ratio_out, float* stats_out) {
  __shared__ double red[2][FB_THREADS / 64];
  __shared__ bool is_last;
  double dd = (double)sd, da = (double)sa;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    dd += __shfl_down(dd, off);
    da += __shfl_down(da, off);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    red[0][wave] = dd;
    red[1][wave] = da;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double td = 0, ta = 0;
#pragma unroll
    for (int w = 0; w < FB_THREADS / 64; ++w) {
      td += red[0][w];
      ta += red[1][w];
    }
    __hip_atomic_store(&ws->part[blockIdx.x][0], td, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&ws->part[blockIdx.x][1], ta, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned t = __hip_atomic_fetch_add(&ws->ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    is_last = (t == gridDim.x - 1);
  }
  __syncthreads();
  if (!is_last) return;
  // last workgroup: fixed-order sum of all partials
  double pd = 0, pa_ = 0;
  for (unsigned i = threadIdx.x; i < gridDim.x; i += FB_THREADS) {
    pd += __hip_atomic_load(&ws->part[i][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    pa_ += __hip_atomic_load(&ws->part[i][1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    pd += __shfl_down(pd, off);
    pa_ += __shfl_down(pa_, off);
  }
  __syncthreads();
  if (lane == 0) {
    red[0][wave] = pd;
    red[1][wave] = pa_;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double td = 0, ta = 0;
#pragma unroll
    for (int w = 0; w < FB_THREADS / 64; ++w) {
      td += red[0][w];
      ta += red[1][w];
    }
    // mean -> fp32 -> activation type, as torch's mean does
    const float mean_d = Act<DT>::round1((float)(td / count));
    const float mean_a = Act<DT>::round1((float)(ta / count));
    const float ratio = mean_d / mean_a;
    Act<DT>::store1(ratio_out, ratio);
    if (stats_out) {
      stats_out[0] = mean_d;
      stats_out[1] = mean_a;
    }
    __hip_atomic_store(&ws->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Contiguous operands, 16-byte aligned: n_vec full vectors + scalar tail.
template <int DT>
__global__ __launch_bounds__(FB_THREADS) void fbcache_flat_kernel(const void* __restrict__ prev,
                                                                 const void* __restrict__ cur,
                                                                 int64_t n, FbWorkspace* ws,
                                                                 void* ratio_out, float* stats_out) {
  constexpr int VEC = Act<DT>::VEC;
  constexpr int UNROLL = 4;
  const u32x4* pv = (const u32x4*)prev;
  const u32x4* cv = (const u32x4*)cur;
  const int64_t n_vec = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * FB_THREADS;
  int64_t i = (int64_t)blockIdx.x * FB_THREADS + threadIdx.x;
  float sd = 0.f, sa = 0.f;
  for (; i + (UNROLL - 1) * stride < n_vec; i += UNROLL * stride) {
    u32x4 a[UNROLL], b[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      a[u] = __builtin_nontemporal_load(pv + i + u * stride);
      b[u] = __builtin_nontemporal_load(cv + i + u * stride);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) accum_vec<DT>(a[u], b[u], sd, sa);
  }
  for (; i < n_vec; i += stride) {
    u32x4 a = __builtin_nontemporal_load(pv + i);
    u32x4 b = __builtin_nontemporal_load(cv + i);
    accum_vec<DT>(a, b, sd, sa);
  }
  // scalar tail (< VEC elements), first workgroup only
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - n_vec * VEC)) {
    const int64_t j = n_vec * VEC + threadIdx.x;
    const float x = Act<DT>::load1(prev, j);
    sd += fabsf(Act<DT>::round1(x - Act<DT>::load1(cur, j)));
    sa += fabsf(x);
  }
  finish<DT>(sd, sa, (double)n, ws, ratio_out, stats_out);
}

// Any row/column strides (e.g. the [..., ::k] view): one element per step.
template <int DT>
__global__ __launch_bounds__(FB_THREADS) void fbcache_strided_kernel(
    const void* __restrict__ prev, const void* __restrict__ cur, int64_t n_rows, int64_t row_len,
    int64_t prs, int64_t pcs, int64_t crs, int64_t ccs, FbWorkspace* ws, void* ratio_out,
    float* stats_out) {
  const int64_t n = n_rows * row_len;
  const int64_t stride = (int64_t)gridDim.x * FB_THREADS;
  float sd = 0.f, sa = 0.f;
  for (int64_t i = (int64_t)blockIdx.x * FB_THREADS + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / row_len;
    const int64_t col = i - r * row_len;
    const float x = Act<DT>::load1(prev, r * prs + col * pcs);
    const float y = Act<DT>::load1(cur, r * crs + col * ccs);
    sd += fabsf(Act<DT>::round1(x - y));
    sa += fabsf(x);
  }
  finish<DT>(sd, sa, (double)n, ws, ratio_out, stats_out);
}

// resid = hidden - hidden0 (rounded, stored); reduction against prev if given.
template <int DT, bool HAVE_PREV>
__global__ __launch_bounds__(FB_THREADS) void fbcache_residual_kernel(
    const void* __restrict__ hidden, const void* __restrict__ hidden0,
    const void* __restrict__ prev, void* __restrict__ resid, int64_t n, FbWorkspace* ws,
    void* ratio_out, float* stats_out) {
  constexpr int VEC = Act<DT>::VEC;
  const u32x4* hv = (const u32x4*)hidden;
  const u32x4* h0v = (const u32x4*)hidden0;
  const u32x4* pv = (const u32x4*)prev;
  u32x4* rv = (u32x4*)resid;
  const int64_t n_vec = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * FB_THREADS;
  float sd = 0.f, sa = 0.f;
  for (int64_t i = (int64_t)blockIdx.x * FB_THREADS + threadIdx.x; i < n_vec; i += stride) {
    const u32x4 h = __builtin_nontemporal_load(hv + i);
    const u32x4 h0 = __builtin_nontemporal_load(h0v + i);
    u32x4 r;
    if constexpr (DT == PA_DTYPE_F32) {
#pragma unroll
      for (int k = 0; k < 4; ++k) r[k] = __float_as_uint(__uint_as_float(h[k]) - __uint_as_float(h0[k]));
    } else if constexpr (DT == PA_DTYPE_BF16) {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        r[k] = BF16::pack2(BF16::lo(h[k]) - BF16::lo(h0[k]), BF16::hi(h[k]) - BF16::hi(h0[k]));
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        r[k] = F16::pack2(F16::lo(h[k]) - F16::lo(h0[k]), F16::hi(h[k]) - F16::hi(h0[k]));
    }
    rv[i] = r;  // re-read by the next step: keep it cacheable
    if constexpr (HAVE_PREV) {
      const u32x4 pr = __builtin_nontemporal_load(pv + i);
      accum_vec<DT>(pr, r, sd, sa);
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - n_vec * VEC)) {
    const int64_t j = n_vec * VEC + threadIdx.x;
    const float r = Act<DT>::round1(Act<DT>::load1(hidden, j) - Act<DT>::load1(hidden0, j));
    if constexpr (DT == PA_DTYPE_F32) ((float*)resid)[j] = r;
    else Act<DT>::store1((uint16_t*)resid + j, r);
    if constexpr (HAVE_PREV) {
      const float x = Act<DT>::load1(prev, j);
      sd += fabsf(Act<DT>::round1(x - r));
      sa += fabsf(x);
    }
  }
  if constexpr (HAVE_PREV) finish<DT>(sd, sa, (double)n, ws, ratio_out, stats_out);
}

template <int DT>
__global__ __launch_bounds__(FB_THREADS) void fbcache_apply_kernel(const void* resid, const void* hidden,
                                                                  void* out, int64_t n) {
  constexpr int VEC = Act<DT>::VEC;
  const u32x4* rv = (const u32x4*)resid;
  const u32x4* hv = (const u32x4*)hidden;
  u32x4* ov = (u32x4*)out;
  const int64_t n_vec = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * FB_THREADS;
  for (int64_t i = (int64_t)blockIdx.x * FB_THREADS + threadIdx.x; i < n_vec; i += stride) {
    const u32x4 r = __builtin_nontemporal_load(rv + i);
    const u32x4 h = __builtin_nontemporal_load(hv + i);
    u32x4 o;
    if constexpr (DT == PA_DTYPE_F32) {
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = __float_as_uint(__uint_as_float(r[k]) + __uint_as_float(h[k]));
    } else if constexpr (DT == PA_DTYPE_BF16) {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        o[k] = BF16::pack2(BF16::lo(r[k]) + BF16::lo(h[k]), BF16::hi(r[k]) + BF16::hi(h[k]));
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        o[k] = F16::pack2(F16::lo(r[k]) + F16::lo(h[k]), F16::hi(r[k]) + F16::hi(h[k]));
    }
    ov[i] = o;
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - n_vec * VEC)) {
    const int64_t j = n_vec * VEC + threadIdx.x;
    const float s = Act<DT>::round1(Act<DT>::load1(resid, j) + Act<DT>::load1(hidden, j));
    if constexpr (DT == PA_DTYPE_F32) ((float*)out)[j] = s;
    else Act<DT>::store1((uint16_t*)out + j, s);
  }
}

// Grid-stride kernels here run fastest with ONE workgroup per CU (measured: 256 workgroups
// 6.2 TB/s, 2048 workgroups 3.3 TB/s on the 671 MB reduction), each thread keeping
// 2 x 4 16-byte loads in flight.
static inline int fb_grid(int64_t work_items, int per_cu = 1) {
  int64_t blocks = (work_items + FB_THREADS - 1) / FB_THREADS;
  if (blocks < 1) blocks = 1;
  int n_cu = device_cus();
  if (n_cu <= 0) n_cu = 256;
  const int64_t cap = (int64_t)n_cu * per_cu;
  return (int)(blocks < cap ? blocks : cap);
}

static inline size_t elem_size(int dtype) { return dtype == PA_DTYPE_F32 ? 4 : 2; }

}  // namespace pa

using namespace pa;

extern "C" size_t pa_fbcache_workspace_bytes(void) { return sizeof(FbWorkspace); }

#define FB_DISPATCH(dtype, CALL)                                             \
  switch (dtype) {                                                           \
    case PA_DTYPE_BF16: { constexpr int DT = PA_DTYPE_BF16; CALL; } break;   \
    case PA_DTYPE_F16: { constexpr int DT = PA_DTYPE_F16; CALL; } break;     \
    case PA_DTYPE_F32: { constexpr int DT = PA_DTYPE_F32; CALL; } break;     \
    default: PA_FAIL(PA_ERR_UNSUPPORTED, "fbcache: bad dtype %d", dtype);    \
  }

extern "C" int pa_fbcache_absdiff_ratio(const void* prev, const void* cur, int dtype, int64_t n_rows,
                                        int64_t row_len, int64_t prev_row_stride,
                                        int64_t prev_col_stride, int64_t cur_row_stride,
                                        int64_t cur_col_stride, void* ratio_out, float* stats_out,
                                        void* workspace, size_t workspace_bytes, void* stream) {
  if (!prev || !cur || !ratio_out || !workspace) PA_FAIL(PA_ERR_INVALID, "fbcache: null pointer argument");
  if (n_rows <= 0 || row_len <= 0) PA_FAIL(PA_ERR_INVALID, "fbcache: empty tensor (mean undefined)");
  if (workspace_bytes < sizeof(FbWorkspace)) PA_FAIL(PA_ERR_WORKSPACE, "fbcache: workspace too small");
  if (((uintptr_t)workspace) % 16) PA_FAIL(PA_ERR_INVALID, "fbcache: workspace not 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  FbWorkspace* ws = (FbWorkspace*)workspace;
  const int64_t n = n_rows * row_len;
  const bool flat = prev_col_stride == 1 && cur_col_stride == 1 &&
                    (n_rows == 1 || (prev_row_stride == row_len && cur_row_stride == row_len)) &&
                    ((uintptr_t)prev % 16 == 0) && ((uintptr_t)cur % 16 == 0);
  if (flat) {
    FB_DISPATCH(dtype, {
      const int grid = fb_grid(n / Act<DT>::VEC / 4);
      hipLaunchKernelGGL(fbcache_flat_kernel<DT>, dim3(grid), dim3(FB_THREADS), 0, s, prev, cur, n, ws,
                         ratio_out, stats_out);
    });
  } else {
    FB_DISPATCH(dtype, {
      const int grid = fb_grid(n / 8);
      hipLaunchKernelGGL(fbcache_strided_kernel<DT>, dim3(grid), dim3(FB_THREADS), 0, s, prev, cur,
                         n_rows, row_len, prev_row_stride, prev_col_stride, cur_row_stride,
                         cur_col_stride, ws, ratio_out, stats_out);
    });
  }
  PA_CHECK_LAUNCH("fbcache kernel");
  return PA_OK;
}

extern "C" int pa_fbcache_residual_ratio(const void* hidden, const void* hidden0, const void* prev,
                                         void* resid_out, int dtype, int64_t n, void* ratio_out,
                                         float* stats_out, void* workspace, size_t workspace_bytes,
                                         void* stream) {
  if (!hidden || !hidden0 || !resid_out) PA_FAIL(PA_ERR_INVALID, "fbcache: null pointer argument");
  if (n <= 0) PA_FAIL(PA_ERR_INVALID, "fbcache: empty tensor");
  if (prev && (!ratio_out || !workspace)) PA_FAIL(PA_ERR_INVALID, "fbcache: ratio_out/workspace missing");
  if (prev && workspace_bytes < sizeof(FbWorkspace)) PA_FAIL(PA_ERR_WORKSPACE, "fbcache: workspace too small");
  const void* ptrs[4] = {hidden, hidden0, resid_out, prev};
  for (int i = 0; i < 4; ++i)
    if (((uintptr_t)ptrs[i]) % 16) PA_FAIL(PA_ERR_UNSUPPORTED, "fbcache: tensor pointer not 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  FbWorkspace* ws = (FbWorkspace*)workspace;
  if (prev) {
    FB_DISPATCH(dtype, {
      const int grid = fb_grid(n / Act<DT>::VEC / 2);
      hipLaunchKernelGGL((fbcache_residual_kernel<DT, true>), dim3(grid), dim3(FB_THREADS), 0, s, hidden,
                         hidden0, prev, resid_out, n, ws, ratio_out, stats_out);
    });
  } else {
    FB_DISPATCH(dtype, {
      const int grid = fb_grid(n / Act<DT>::VEC / 2);
      hipLaunchKernelGGL((fbcache_residual_kernel<DT, false>), dim3(grid), dim3(FB_THREADS), 0, s, hidden,
                         hidden0, prev, resid_out, n, ws, ratio_out, stats_out);
    });
  }
  PA_CHECK_LAUNCH("fbcache residual kernel");
  return PA_OK;
}

extern "C" int pa_fbcache_apply_residual(const void* resid, const void* hidden, void* out, int dtype,
                                         int64_t n, void* stream) {
  if (!resid || !hidden || !out) PA_FAIL(PA_ERR_INVALID, "fbcache: null pointer argument");
  if (n < 0) PA_FAIL(PA_ERR_INVALID, "fbcache: negative size");
  if (n == 0) return PA_OK;
  const void* ptrs[3] = {resid, hidden, out};
  for (int i = 0; i < 3; ++i)
    if (((uintptr_t)ptrs[i]) % 16) PA_FAIL(PA_ERR_UNSUPPORTED, "fbcache: tensor pointer not 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  FB_DISPATCH(dtype, {
    const int grid = fb_grid(n / Act<DT>::VEC / 2);
    hipLaunchKernelGGL(fbcache_apply_kernel<DT>, dim3(grid), dim3(FB_THREADS), 0, s, resid, hidden, out, n);
  });
  PA_CHECK_LAUNCH("fbcache apply kernel");
  return PA_OK;
}
