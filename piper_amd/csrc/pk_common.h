// Shared device/host helpers for the gfx950 kernels of libpiper_amd.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/piper_amd.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

#define PK_WAVE 64
#define PK_MAX_DEVICES 64

// Per-source set-up behind pk_init (current device).
int pk_init_grouped_gemm();

#define PK_RETURN_IF_LAUNCH_FAILED()        \
  do {                                      \
    hipError_t pk_e_ = hipGetLastError();   \
    if (pk_e_ != hipSuccess) return (int)pk_e_; \
  } while (0)

static inline bool pk_aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }
static inline int64_t pk_ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t pk_dtype_size(int dtype) { return dtype == PK_BF16 ? 2 : 4; }
static inline bool pk_dtype_ok(int dtype) { return dtype == PK_F32 || dtype == PK_BF16; }

// ---------------------------------------------------------------- optional kernel timing
namespace pk_timing {
enum KernelId {
  K_GATE_LOGITS = 0, K_ROUTE_TOPK, K_ROUTE_TOPK_BWD, K_GATE_LOGITS_BWD, K_SORT_HIST, K_SORT_SCAN,
  K_SORT_SCATTER, K_COUNTS_TO_STARTS, K_PERMUTE_FWD, K_GATHER_REDUCE, K_COMBINE_BWD,
  K_SWIGLU_GATE_UP, K_SWIGLU_DOWN, K_SWIGLU_DGRAD_DH, K_SWIGLU_DGRAD_DX, K_SWIGLU_WGRAD,
  K_SIMT_GEMM, K_SWIGLU_ELEMENTWISE, K_BUCKET_PACK, K_BUCKET_UNPACK, K_BUCKET_ZERO, K_ADAMW,
  K_RMSNORM_FWD, K_RMSNORM_BWD, K_MISC, K_SWIGLU_WGRAD_W2, K_SWIGLU_WGRAD_W13, K_COUNT
};
// Brackets one kernel launch with two event records on `s` when timing is enabled
// (pk_timing_enable); otherwise does nothing.
class Scope {
 public:
  Scope(int id, hipStream_t s);
  ~Scope();
 private:
  hipStream_t stream_;
  int slot_;
};
}  // namespace pk_timing

// Launch a kernel under a timing scope (the caller checks hipGetLastError afterwards).
#define PK_LAUNCH_NOCHECK(id, stream, ...)          \
  do {                                              \
    pk_timing::Scope pk_scope_((id), (stream));     \
    hipLaunchKernelGGL(__VA_ARGS__);                \
  } while (0)

// ---------------------------------------------------------------- device helpers
template <typename T>
__device__ __forceinline__ float pk_to_float(T v);
template <>
__device__ __forceinline__ float pk_to_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ float pk_to_float<bf16_t>(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T pk_from_float(float v);
template <>
__device__ __forceinline__ float pk_from_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t pk_from_float<bf16_t>(float v) { return (bf16_t)v; }  // RNE

// Wave-wide (64 lanes) butterfly reductions; every lane ends with the result.
__device__ __forceinline__ float pk_wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, PK_WAVE);
  return v;
}
__device__ __forceinline__ float pk_wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, PK_WAVE));
  return v;
}
__device__ __forceinline__ unsigned long long pk_wave_max_u64(unsigned long long v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    unsigned int lo = __shfl_xor((unsigned int)(v & 0xffffffffull), off, PK_WAVE);
    unsigned int hi = __shfl_xor((unsigned int)(v >> 32), off, PK_WAVE);
    unsigned long long o = ((unsigned long long)hi << 32) | lo;
    v = o > v ? o : v;
  }
  return v;
}

// Block-wide sum for blockDim.x a multiple of 64 and <= 1024; result valid on every thread.
__device__ __forceinline__ float pk_block_sum(float v, float* lds /* >= 16 floats */) {
  v = pk_wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[wave] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += lds[i];
  return r;
}

// 16-byte vector of elements of type T.
template <typename T>
struct PkVec16;
template <>
struct PkVec16<float> {
  static constexpr int N = 4;
  floatx4_t v;
  __device__ __forceinline__ float get(int i) const { return v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = f; }
};
template <>
struct PkVec16<bf16_t> {
  static constexpr int N = 8;
  bf16x8_t v;
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
  __device__ __forceinline__ void set(int i, float f) { v[i] = (bf16_t)f; }
};
