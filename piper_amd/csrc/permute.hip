// Row movers of the expert region: permute (gather by expert-sorted order), its backward
// (K-way gather-reduce), the fused unpermute+combine and its backward.  One block per row;
// 16 bytes per lane per access, rows are contiguous so every access is fully coalesced.
#include "pk_common.h"
#include <initializer_list>

namespace {

constexpr int kRowThreads = 256;

// VEC = true: 16-byte accesses (needs H % N == 0 and 16-byte aligned bases); false: scalar.
template <typename T, bool VEC>
struct RowIO {
  static constexpr int N = VEC ? PkVec16<T>::N : 1;
  __device__ static __forceinline__ void load(const T* row, int64_t v, float (&f)[PkVec16<T>::N]) {
    if (VEC) {
      PkVec16<T> x;
      x.v = *reinterpret_cast<const decltype(x.v)*>(row + v * N);
#pragma unroll
      for (int i = 0; i < N; ++i) f[i] = x.get(i);
    } else {
      f[0] = pk_to_float<T>(row[v]);
    }
  }
  __device__ static __forceinline__ void store(T* row, int64_t v, const float (&f)[PkVec16<T>::N]) {
    if (VEC) {
      PkVec16<T> x;
#pragma unroll
      for (int i = 0; i < N; ++i) x.set(i, f[i]);
      *reinterpret_cast<decltype(x.v)*>(row + v * N) = x.v;
    } else {
      row[v] = pk_from_float<T>(f[0]);
    }
  }
};

template <typename T, bool VEC>
__global__ __launch_bounds__(kRowThreads) void permute_fwd_kernel(
    const T* __restrict__ x, const int32_t* __restrict__ perm, T* __restrict__ routed, int64_t H,
    int K) {
  using IO = RowIO<T, VEC>;
  const int64_t p = blockIdx.x;
  const int64_t t = perm[p] / K;
  const T* src = x + t * H;
  T* dst = routed + p * H;
  const int64_t nv = H / IO::N;
  for (int64_t v = threadIdx.x; v < nv; v += kRowThreads) {
    if (VEC) {
      using V = decltype(PkVec16<T>::v);
      reinterpret_cast<V*>(dst)[v] = reinterpret_cast<const V*>(src)[v];
    } else {
      dst[v] = src[v];
    }
  }
}

// out[t,:] = sum_k w[t,k] * rows[inv_perm[t*K+k], :] (+ addend[t,:]);  w == nullptr -> 1
template <typename T, bool VEC>
__global__ __launch_bounds__(kRowThreads) void gather_reduce_kernel(
    const T* __restrict__ rows, const int32_t* __restrict__ inv_perm,
    const float* __restrict__ weights, const float* __restrict__ addend, T* __restrict__ out,
    int64_t H, int K) {
  using IO = RowIO<T, VEC>;
  constexpr int N = PkVec16<T>::N;
  const int64_t t = blockIdx.x;
  const int64_t nv = H / IO::N;
  for (int64_t v = threadIdx.x; v < nv; v += kRowThreads) {
    float acc[N];
#pragma unroll
    for (int i = 0; i < N; ++i) acc[i] = 0.f;
    for (int k = 0; k < K; ++k) {
      const int64_t p = inv_perm[t * K + k];
      const float w = weights ? weights[t * K + k] : 1.f;
      float f[N];
      IO::load(rows + p * H, v, f);
#pragma unroll
      for (int i = 0; i < IO::N; ++i) acc[i] = fmaf(w, f[i], acc[i]);
    }
    if (addend) {
#pragma unroll
      for (int i = 0; i < IO::N; ++i) acc[i] += addend[t * H + v * IO::N + i];
    }
    IO::store(out + t * H, v, acc);
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kRowThreads) void combine_bwd_kernel(
    const T* __restrict__ d_out, const T* __restrict__ y, const int32_t* __restrict__ perm,
    const float* __restrict__ scores, T* __restrict__ d_y, float* __restrict__ d_scores,
    int64_t H, int K) {
  using IO = RowIO<T, VEC>;
  constexpr int N = PkVec16<T>::N;
  __shared__ float red[16];
  const int64_t p = blockIdx.x;
  const int64_t slot = perm[p];
  const int64_t t = slot / K;
  const float s = scores[slot];
  const int64_t nv = H / IO::N;
  float dot = 0.f;
  for (int64_t v = threadIdx.x; v < nv; v += kRowThreads) {
    float d[N], yy[N], o[N];
    IO::load(d_out + t * H, v, d);
    IO::load(y + p * H, v, yy);
#pragma unroll
    for (int i = 0; i < IO::N; ++i) {
      o[i] = s * d[i];
      dot = fmaf(d[i], yy[i], dot);
    }
    IO::store(d_y + p * H, v, o);
  }
  dot = pk_block_sum(dot, red);
  if (threadIdx.x == 0) d_scores[slot] = dot;
}

bool vec_ok(int dtype, int64_t H, std::initializer_list<const void*> ptrs) {
  const int n = dtype == PK_BF16 ? 8 : 4;
  if (H % n != 0) return false;
  for (const void* p : ptrs)
    if (p && !pk_aligned16(p)) return false;
  return true;
}

}  // namespace

extern "C" {

int pk_permute_fwd(const void* x, int dtype, const int32_t* perm, void* routed, int64_t A,
                   int64_t H, int64_t K, pk_stream_t stream) {
  if (A < 0 || H <= 0 || K <= 0 || !pk_dtype_ok(dtype)) return PK_ERR_ARG;
  if (A == 0) return PK_OK;
  if (!x || !perm || !routed) return PK_ERR_ARG;
  if (A > 0x7fffffffll) return PK_ERR_SHAPE;
  const bool vec = vec_ok(dtype, H, {x, routed});
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)A);
  if (dtype == PK_BF16) {
    if (vec) PK_LAUNCH_NOCHECK(pk_timing::K_PERMUTE_FWD, s, (permute_fwd_kernel<bf16_t, true>), grid, dim3(kRowThreads), 0, s, (const bf16_t*)x, perm, (bf16_t*)routed, H, (int)K);
    else PK_LAUNCH_NOCHECK(pk_timing::K_PERMUTE_FWD, s, (permute_fwd_kernel<bf16_t, false>), grid, dim3(kRowThreads), 0, s, (const bf16_t*)x, perm, (bf16_t*)routed, H, (int)K);
  } else {
    if (vec) PK_LAUNCH_NOCHECK(pk_timing::K_PERMUTE_FWD, s, (permute_fwd_kernel<float, true>), grid, dim3(kRowThreads), 0, s, (const float*)x, perm, (float*)routed, H, (int)K);
    else PK_LAUNCH_NOCHECK(pk_timing::K_PERMUTE_FWD, s, (permute_fwd_kernel<float, false>), grid, dim3(kRowThreads), 0, s, (const float*)x, perm, (float*)routed, H, (int)K);
  }
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

static int gather_reduce(const void* rows, int dtype, const int32_t* inv_perm, const float* weights,
                         const float* addend, void* out, int64_t T, int64_t H, int64_t K,
                         pk_stream_t stream) {
  if (T < 0 || H <= 0 || K <= 0 || !pk_dtype_ok(dtype)) return PK_ERR_ARG;
  if (T == 0) return PK_OK;
  if (!rows || !inv_perm || !out) return PK_ERR_ARG;
  if (T > 0x7fffffffll) return PK_ERR_SHAPE;
  const bool vec = vec_ok(dtype, H, {rows, out});
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)T);
  if (dtype == PK_BF16) {
    if (vec) PK_LAUNCH_NOCHECK(pk_timing::K_GATHER_REDUCE, s, (gather_reduce_kernel<bf16_t, true>), grid, dim3(kRowThreads), 0, s, (const bf16_t*)rows, inv_perm, weights, addend, (bf16_t*)out, H, (int)K);
    else PK_LAUNCH_NOCHECK(pk_timing::K_GATHER_REDUCE, s, (gather_reduce_kernel<bf16_t, false>), grid, dim3(kRowThreads), 0, s, (const bf16_t*)rows, inv_perm, weights, addend, (bf16_t*)out, H, (int)K);
  } else {
    if (vec) PK_LAUNCH_NOCHECK(pk_timing::K_GATHER_REDUCE, s, (gather_reduce_kernel<float, true>), grid, dim3(kRowThreads), 0, s, (const float*)rows, inv_perm, weights, addend, (float*)out, H, (int)K);
    else PK_LAUNCH_NOCHECK(pk_timing::K_GATHER_REDUCE, s, (gather_reduce_kernel<float, false>), grid, dim3(kRowThreads), 0, s, (const float*)rows, inv_perm, weights, addend, (float*)out, H, (int)K);
  }
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int pk_permute_bwd(const void* d_routed, int dtype, const int32_t* inv_perm,
                   const float* addend_f32, void* d_x, int64_t T, int64_t H, int64_t K,
                   pk_stream_t stream) {
  return gather_reduce(d_routed, dtype, inv_perm, nullptr, addend_f32, d_x, T, H, K, stream);
}

int pk_combine_fwd(const void* y_sorted, int dtype, const int32_t* inv_perm,
                   const float* top_scores, void* out, int64_t T, int64_t H, int64_t K,
                   pk_stream_t stream) {
  if (!top_scores && T > 0) return PK_ERR_ARG;
  return gather_reduce(y_sorted, dtype, inv_perm, top_scores, nullptr, out, T, H, K, stream);
}

int pk_combine_bwd(const void* d_out, const void* y_sorted, int dtype, const int32_t* perm,
                   const float* top_scores, void* d_y_sorted, float* d_top_scores, int64_t A,
                   int64_t H, int64_t K, pk_stream_t stream) {
  if (A < 0 || H <= 0 || K <= 0 || !pk_dtype_ok(dtype)) return PK_ERR_ARG;
  if (A == 0) return PK_OK;
  if (!d_out || !y_sorted || !perm || !top_scores || !d_y_sorted || !d_top_scores) return PK_ERR_ARG;
  if (A > 0x7fffffffll) return PK_ERR_SHAPE;
  const bool vec = vec_ok(dtype, H, {d_out, y_sorted, d_y_sorted});
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)A);
  if (dtype == PK_BF16) {
    if (vec) PK_LAUNCH_NOCHECK(pk_timing::K_COMBINE_BWD, s, (combine_bwd_kernel<bf16_t, true>), grid, dim3(kRowThreads), 0, s, (const bf16_t*)d_out, (const bf16_t*)y_sorted, perm, top_scores, (bf16_t*)d_y_sorted, d_top_scores, H, (int)K);
    else PK_LAUNCH_NOCHECK(pk_timing::K_COMBINE_BWD, s, (combine_bwd_kernel<bf16_t, false>), grid, dim3(kRowThreads), 0, s, (const bf16_t*)d_out, (const bf16_t*)y_sorted, perm, top_scores, (bf16_t*)d_y_sorted, d_top_scores, H, (int)K);
  } else {
    if (vec) PK_LAUNCH_NOCHECK(pk_timing::K_COMBINE_BWD, s, (combine_bwd_kernel<float, true>), grid, dim3(kRowThreads), 0, s, (const float*)d_out, (const float*)y_sorted, perm, top_scores, (float*)d_y_sorted, d_top_scores, H, (int)K);
    else PK_LAUNCH_NOCHECK(pk_timing::K_COMBINE_BWD, s, (combine_bwd_kernel<float, false>), grid, dim3(kRowThreads), 0, s, (const float*)d_out, (const float*)y_sorted, perm, top_scores, (float*)d_y_sorted, d_top_scores, H, (int)K);
  }
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

}  // extern "C"
