// TaylorSeer finite differences and extrapolation as single passes over memory.
//
// The reference keeps, per cached residual, a list of finite-difference "derivatives" and
// rebuilds / evaluates it with one torch elementwise launch per arithmetic operation
// (src/para_attn/first_block_cache/taylorseer.py:29-48):
//   update:       dY[0] = Y;  dY[i+1] = (dY[i] - dY_prev[i]) / window
//   extrapolate:  out = 0;    out += (1 / i!) * dY[i] * elapsed**i   for every stored order
// and, on a cache hit, adds the extrapolated residual to the hidden states
// (src/para_attn/first_block_cache/utils.py:239-243).  Each chain is one kernel here: every
// operand is read once and every result written once (update of n orders: 1 + 2n tensor passes
// instead of 5n; extrapolation of m orders plus the add: m + 2 instead of 5m).
//
// Rounding follows torch's eager chain exactly for 16-bit activations: every operation is
// carried out in fp32 and its result rounded to the activation type before the next one;
// Python scalars enter as fp32; the division is a true division.
//
// Bandwidth bound.  One thread = one 16-byte vector of every operand, 512-thread workgroups, no
// grid cap, plain loads and streaming stores (the layout the merge kernel measured fastest).

#include "pa_common.h"

namespace pa {

constexpr int TS_THREADS = 512;
constexpr int TS_MAX_ORDER = 5;  // stored orders: value + up to 4 differences

struct TsUpdateParams {
  const void* y;
  const void* prev[TS_MAX_ORDER - 1];
  void* cur[TS_MAX_ORDER - 1];  // cur[i] = order i+1
  int n;
  float window;
  int64_t numel;
};

struct TsValueParams {
  const void* d[TS_MAX_ORDER];
  float coef[TS_MAX_ORDER];  // (float)(1 / i!)
  float pw[TS_MAX_ORDER];    // (float)(elapsed ** i)
  int m;
  const void* hidden;  // optional: out = hidden + value
  void* out;
  int64_t numel;
};

// 16 bytes of activations as floats, and back with the type's rounding
template <int DT>
struct TsVec;
template <>
struct TsVec<PA_DTYPE_BF16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const void* p, int64_t v, float* x) {
    const u32x4 w = *((const u32x4*)p + v);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = BF16::lo(w[i]);
      x[2 * i + 1] = BF16::hi(w[i]);
    }
  }
  static __device__ __forceinline__ float round(float x) { return BF16::lo(BF16::pack2(x, 0.f)); }
  static __device__ __forceinline__ void store(void* p, int64_t v, const float* x) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = BF16::pack2(x[2 * i], x[2 * i + 1]);
    __builtin_nontemporal_store(w, (u32x4*)p + v);
  }
  static __device__ __forceinline__ float load1(const void* p, int64_t i) {
    return __uint_as_float((uint32_t)((const uint16_t*)p)[i] << 16);
  }
  static __device__ __forceinline__ void store1(void* p, int64_t i, float x) {
    ((uint16_t*)p)[i] = (uint16_t)(BF16::pack2(x, 0.f) & 0xffffu);
  }
};
template <>
struct TsVec<PA_DTYPE_F16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const void* p, int64_t v, float* x) {
    const u32x4 w = *((const u32x4*)p + v);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = F16::lo(w[i]);
      x[2 * i + 1] = F16::hi(w[i]);
    }
  }
  // torch rounds the fp32 result of every operation to fp16.  Left alone, the compiler folds a
  // multiply and this conversion into one mixed-precision instruction that rounds the exact
  // product once, which differs on ties of the fp32 value; the empty asm keeps the fp32 value.
  static __device__ __forceinline__ float round(float x) {
    asm volatile("" : "+v"(x));
    return (float)(_Float16)x;
  }
  static __device__ __forceinline__ void store(void* p, int64_t v, const float* x) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = F16::pack2(x[2 * i], x[2 * i + 1]);
    __builtin_nontemporal_store(w, (u32x4*)p + v);
  }
  static __device__ __forceinline__ float load1(const void* p, int64_t i) { return (float)((const _Float16*)p)[i]; }
  static __device__ __forceinline__ void store1(void* p, int64_t i, float x) { ((_Float16*)p)[i] = (_Float16)x; }
};
template <>
struct TsVec<PA_DTYPE_F32> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const void* p, int64_t v, float* x) {
    const u32x4 w = *((const u32x4*)p + v);
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = __uint_as_float(w[i]);
  }
  static __device__ __forceinline__ float round(float x) { return x; }
  static __device__ __forceinline__ void store(void* p, int64_t v, const float* x) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = __float_as_uint(x[i]);
    __builtin_nontemporal_store(w, (u32x4*)p + v);
  }
  static __device__ __forceinline__ float load1(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ void store1(void* p, int64_t i, float x) { ((float*)p)[i] = x; }
};

// one element of the difference chain: x_{i+1} = round(round(x_i - prev_i) / window)
template <int DT>
__device__ __forceinline__ float ts_diff(float x, float prev, float window) {
#pragma clang fp contract(off)
  return TsVec<DT>::round(TsVec<DT>::round(x - prev) / window);
}

// one term of the extrapolation folded into the running sum:
// out = round(out + round(round(coef * d) * pw))
template <int DT>
__device__ __forceinline__ float ts_term(float out, float d, float coef, float pw) {
#pragma clang fp contract(off)  // fp32 activations: torch multiplies and adds in separate roundings
  return TsVec<DT>::round(out + TsVec<DT>::round(TsVec<DT>::round(coef * d) * pw));
}

template <int DT>
__global__ __launch_bounds__(TS_THREADS) void taylor_update_kernel(const TsUpdateParams p) {
  constexpr int N = TsVec<DT>::N;
  const int64_t v = (int64_t)blockIdx.x * TS_THREADS + threadIdx.x;
  const int64_t n_vec = p.numel / N;
  if (v < n_vec) {
    float x[N], q[N];
    TsVec<DT>::load(p.y, v, x);
    for (int i = 0; i < p.n; ++i) {
      TsVec<DT>::load(p.prev[i], v, q);
#pragma unroll
      for (int e = 0; e < N; ++e) x[e] = ts_diff<DT>(x[e], q[e], p.window);
      TsVec<DT>::store(p.cur[i], v, x);
    }
  } else if (v < n_vec + (p.numel - n_vec * N)) {  // ragged end, one element per thread
    const int64_t j = n_vec * N + (v - n_vec);
    float x = TsVec<DT>::load1(p.y, j);
    for (int i = 0; i < p.n; ++i) {
      x = ts_diff<DT>(x, TsVec<DT>::load1(p.prev[i], j), p.window);
      TsVec<DT>::store1(p.cur[i], j, x);
    }
  }
}

template <int DT>
__global__ __launch_bounds__(TS_THREADS) void taylor_value_kernel(const TsValueParams p) {
  constexpr int N = TsVec<DT>::N;
  const int64_t v = (int64_t)blockIdx.x * TS_THREADS + threadIdx.x;
  const int64_t n_vec = p.numel / N;
  if (v < n_vec) {
    float out[N], d[N];
    TsVec<DT>::load(p.d[0], v, out);
#pragma unroll
    for (int e = 0; e < N; ++e) out[e] = ts_term<DT>(0.f, out[e], p.coef[0], p.pw[0]);  // 0 + (1/0!) * d0 * elapsed**0
    for (int i = 1; i < p.m; ++i) {
      TsVec<DT>::load(p.d[i], v, d);
#pragma unroll
      for (int e = 0; e < N; ++e) out[e] = ts_term<DT>(out[e], d[e], p.coef[i], p.pw[i]);
    }
    if (p.hidden != nullptr) {
      TsVec<DT>::load(p.hidden, v, d);
#pragma unroll
      for (int e = 0; e < N; ++e) out[e] = TsVec<DT>::round(out[e] + d[e]);
    }
    TsVec<DT>::store(p.out, v, out);
  } else if (v < n_vec + (p.numel - n_vec * N)) {
    const int64_t j = n_vec * N + (v - n_vec);
    float out = ts_term<DT>(0.f, TsVec<DT>::load1(p.d[0], j), p.coef[0], p.pw[0]);
    for (int i = 1; i < p.m; ++i) out = ts_term<DT>(out, TsVec<DT>::load1(p.d[i], j), p.coef[i], p.pw[i]);
    if (p.hidden != nullptr) out = TsVec<DT>::round(out + TsVec<DT>::load1(p.hidden, j));
    TsVec<DT>::store1(p.out, j, out);
  }
}

static inline int64_t ts_grid(int dtype, int64_t numel) {
  const int N = dtype == PA_DTYPE_F32 ? 4 : 8;
  const int64_t threads = numel / N + numel % N;
  return (threads + TS_THREADS - 1) / TS_THREADS;
}

}  // namespace pa

using namespace pa;

#define TS_DISPATCH(dtype, CALL)                                             \
  switch (dtype) {                                                           \
    case PA_DTYPE_BF16: { constexpr int DT = PA_DTYPE_BF16; CALL; } break;   \
    case PA_DTYPE_F16: { constexpr int DT = PA_DTYPE_F16; CALL; } break;     \
    case PA_DTYPE_F32: { constexpr int DT = PA_DTYPE_F32; CALL; } break;     \
    default: PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: bad dtype %d", dtype); \
  }

extern "C" int pa_taylorseer_update(const void* y, const void* const* prev, void* const* cur, int n,
                                    int dtype, int64_t numel, float window, void* stream) {
  if (n < 0 || n > TS_MAX_ORDER - 1)
    PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: %d difference orders (at most %d)", n, TS_MAX_ORDER - 1);
  if (numel < 0) PA_FAIL(PA_ERR_INVALID, "taylorseer: negative size");
  if (n == 0 || numel == 0) return PA_OK;
  if (!y || !prev || !cur) PA_FAIL(PA_ERR_INVALID, "taylorseer: null pointer argument");
  if (!(window != 0.f)) PA_FAIL(PA_ERR_INVALID, "taylorseer: window must not be zero");
  TsUpdateParams p;
  p.y = y; p.n = n; p.window = window; p.numel = numel;
  if (((uintptr_t)y) % 16) PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: tensor pointer not 16-byte aligned");
  for (int i = 0; i < TS_MAX_ORDER - 1; ++i) {
    p.prev[i] = i < n ? prev[i] : nullptr;
    p.cur[i] = i < n ? cur[i] : nullptr;
    if (i < n) {
      if (!prev[i] || !cur[i]) PA_FAIL(PA_ERR_INVALID, "taylorseer: null pointer argument");
      if (((uintptr_t)prev[i]) % 16 || ((uintptr_t)cur[i]) % 16)
        PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: tensor pointer not 16-byte aligned");
    }
  }
  const int64_t grid = ts_grid(dtype, numel);
  if (grid > 0x7fffffffLL) PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: tensor too large");
  hipStream_t s = (hipStream_t)stream;
  TS_DISPATCH(dtype, hipLaunchKernelGGL(taylor_update_kernel<DT>, dim3((unsigned)grid), dim3(TS_THREADS), 0, s, p));
  PA_CHECK_LAUNCH("taylorseer update kernel");
  return PA_OK;
}

extern "C" int pa_taylorseer_value(const void* const* deriv, int m, const float* coef, const float* pw,
                                   const void* hidden, void* out, int dtype, int64_t numel, void* stream) {
  if (m < 1 || m > TS_MAX_ORDER) PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: %d stored orders (1 to %d)", m, TS_MAX_ORDER);
  if (numel < 0) PA_FAIL(PA_ERR_INVALID, "taylorseer: negative size");
  if (!deriv || !coef || !pw || !out) PA_FAIL(PA_ERR_INVALID, "taylorseer: null pointer argument");
  if (numel == 0) return PA_OK;
  TsValueParams p;
  p.m = m; p.hidden = hidden; p.out = out; p.numel = numel;
  if (((uintptr_t)out) % 16 || ((uintptr_t)hidden) % 16)
    PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: tensor pointer not 16-byte aligned");
  for (int i = 0; i < TS_MAX_ORDER; ++i) {
    p.d[i] = i < m ? deriv[i] : nullptr;
    p.coef[i] = i < m ? coef[i] : 0.f;
    p.pw[i] = i < m ? pw[i] : 0.f;
    if (i < m) {
      if (!deriv[i]) PA_FAIL(PA_ERR_INVALID, "taylorseer: null pointer argument");
      if (((uintptr_t)deriv[i]) % 16) PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: tensor pointer not 16-byte aligned");
    }
  }
  const int64_t grid = ts_grid(dtype, numel);
  if (grid > 0x7fffffffLL) PA_FAIL(PA_ERR_UNSUPPORTED, "taylorseer: tensor too large");
  hipStream_t s = (hipStream_t)stream;
  TS_DISPATCH(dtype, hipLaunchKernelGGL(taylor_value_kernel<DT>, dim3((unsigned)grid), dim3(TS_THREADS), 0, s, p));
  PA_CHECK_LAUNCH("taylorseer value kernel");
  return PA_OK;
}
