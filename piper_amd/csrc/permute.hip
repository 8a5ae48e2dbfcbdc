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
  // the same load for rows that are read once and are too many to stay in a cache: a streaming
  // (nontemporal) load keeps them from pushing out what other kernels left there (measured on
  // 537 MB of gathered rows: 5.0 -> 5.5 TB/s; on 134 MB, which the memory-side cache holds, the
  // ordinary load is the faster one, 6.5 against 6.0 TB/s)
  __device__ static __forceinline__ void load_once(const T* row, int64_t v, float (&f)[PkVec16<T>::N]) {
    if (VEC) {
      PkVec16<T> x;
      x.v = __builtin_nontemporal_load(reinterpret_cast<const decltype(x.v)*>(row + v * N));
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

// out[t,:] = sum_k w[t,k] * rows[inv_perm[t*K+k], :] (+ addend[t,:]) (+ residual[t,:]);  w == nullptr -> 1
// The K rows of a token lie anywhere in the expert-sorted array, so every term is a round trip to
// memory behind the load of its index.  Indices and weights of up to KB terms are fetched first
// (wave-uniform addresses), then the KB row loads are issued together and summed in k order (the
// same sum, term by term, as one load at a time).
template <typename T, bool VEC, bool STREAM>
__global__ __launch_bounds__(kRowThreads) void gather_reduce_kernel(
    const T* __restrict__ rows, const int32_t* __restrict__ inv_perm,
    const float* __restrict__ weights, const float* __restrict__ addend, const T* __restrict__ residual,
    T* __restrict__ out, int64_t H, int K) {
  using IO = RowIO<T, VEC>;
  constexpr int N = PkVec16<T>::N;
  constexpr int KB = 8;
  const int64_t t = blockIdx.x;
  const int64_t nv = H / IO::N;
  for (int64_t v = threadIdx.x; v < nv; v += kRowThreads) {
    float acc[N];
#pragma unroll
    for (int i = 0; i < N; ++i) acc[i] = 0.f;
    for (int k0 = 0; k0 < K; k0 += KB) {
      int64_t p[KB];
      float w[KB];
#pragma unroll
      for (int j = 0; j < KB; ++j) {
        const int k = min(k0 + j, K - 1);       // past the end: the last term again, not added
        p[j] = inv_perm[t * K + k];
        w[j] = weights ? weights[t * K + k] : 1.f;
      }
      float f[KB][N];
#pragma unroll
      for (int j = 0; j < KB; ++j) {
        if (STREAM) IO::load_once(rows + p[j] * H, v, f[j]);
        else IO::load(rows + p[j] * H, v, f[j]);
      }
#pragma unroll
      for (int j = 0; j < KB; ++j) {
        if (k0 + j < K) {
#pragma unroll
          for (int i = 0; i < IO::N; ++i) acc[i] = fmaf(w[j], f[j][i], acc[i]);
        }
      }
    }
    if (addend) {
#pragma unroll
      for (int i = 0; i < IO::N; ++i) acc[i] += addend[t * H + v * IO::N + i];
    }
    if (residual) {   // the sum is rounded to T first, like a separate add of two T tensors
      float r[N];
      IO::load(residual + t * H, v, r);
#pragma unroll
      for (int i = 0; i < IO::N; ++i) acc[i] = pk_to_float<T>(pk_from_float<T>(acc[i])) + r[i];
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

// ---- RMSNorm over rows: y = x * rsqrt(mean(x^2) + eps) * w, computed in fp32 and rounded once.
// One block per row; the row is read twice (the second read hits the cache).
template <typename T, bool VEC>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_fwd_kernel(
    const T* __restrict__ x, const T* __restrict__ w, float eps, T* __restrict__ y,
    float* __restrict__ rstd, int64_t H) {
  using IO = RowIO<T, VEC>;
  constexpr int N = PkVec16<T>::N;
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const T* row = x + t * H;
  const int64_t nv = H / IO::N;
  float ss = 0.f;
  for (int64_t v = threadIdx.x; v < nv; v += kRowThreads) {
    float f[N];
    IO::load(row, v, f);
#pragma unroll
    for (int i = 0; i < IO::N; ++i) ss = fmaf(f[i], f[i], ss);
  }
  ss = pk_block_sum(ss, red);
  const float rs = rsqrtf(ss / (float)H + eps);
  if (threadIdx.x == 0 && rstd) rstd[t] = rs;
  for (int64_t v = threadIdx.x; v < nv; v += kRowThreads) {
    float f[N], g[N];
    IO::load(row, v, f);
    IO::load(w, v, g);
#pragma unroll
    for (int i = 0; i < IO::N; ++i) f[i] = (f[i] * rs) * g[i];
    IO::store(y + t * H, v, f);
  }
}

// Backward: with xh = x * rstd and s = d_y * w,
//   d_x = rstd * (s - xh * mean(s * xh)) (+ addend),   d_w[h] = sum_t d_y[t,h] * xh[t,h].
// Block b walks rows b, b + gridDim.x, ...; every thread keeps the d_w partial sums of the
// columns it touches in registers and writes them to partial[b, :] at the end, so the column
// sums are reduced in a fixed order by a second kernel.  CPT = column vectors per thread.
template <typename T, bool VEC, int CPT>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_bwd_kernel(
    const T* __restrict__ d_y, const T* __restrict__ x, const T* __restrict__ w,
    const float* __restrict__ rstd, const T* __restrict__ addend, T* __restrict__ d_x,
    float* __restrict__ partial, int64_t rows, int64_t H) {
  using IO = RowIO<T, VEC>;
  constexpr int N = PkVec16<T>::N;
  __shared__ float red[16];
  const int64_t nv = H / IO::N;
  float dw[CPT][N];
  float wv[CPT][N];
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    const int64_t v = threadIdx.x + (int64_t)c * kRowThreads;
#pragma unroll
    for (int i = 0; i < N; ++i) { dw[c][i] = 0.f; wv[c][i] = 0.f; }
    if (v < nv) IO::load(w, v, wv[c]);
  }
  for (int64_t t = blockIdx.x; t < rows; t += gridDim.x) {
    const float rs = rstd[t];
    float s[CPT][N], xh[CPT][N];
    float dot = 0.f;
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
      const int64_t v = threadIdx.x + (int64_t)c * kRowThreads;
#pragma unroll
      for (int i = 0; i < N; ++i) { s[c][i] = 0.f; xh[c][i] = 0.f; }
      if (v < nv) {
        float dy[N];
        IO::load(d_y + t * H, v, dy);
        IO::load(x + t * H, v, xh[c]);
#pragma unroll
        for (int i = 0; i < IO::N; ++i) {
          xh[c][i] *= rs;
          s[c][i] = dy[i] * wv[c][i];
          dw[c][i] = fmaf(dy[i], xh[c][i], dw[c][i]);
          dot = fmaf(s[c][i], xh[c][i], dot);
        }
      }
    }
    dot = pk_block_sum(dot, red) / (float)H;
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
      const int64_t v = threadIdx.x + (int64_t)c * kRowThreads;
      if (v < nv) {
        float o[N];
#pragma unroll
        for (int i = 0; i < IO::N; ++i) o[i] = rs * (s[c][i] - xh[c][i] * dot);
        if (addend) {   // both terms are T tensors in the unfused formulation: round, then add
          float a[N];
          IO::load(addend + t * H, v, a);
#pragma unroll
          for (int i = 0; i < IO::N; ++i) o[i] = pk_to_float<T>(pk_from_float<T>(o[i])) + a[i];
        }
        IO::store(d_x + t * H, v, o);
      }
    }
  }
  if (partial) {
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
      const int64_t v = threadIdx.x + (int64_t)c * kRowThreads;
      if (v < nv) {
#pragma unroll
        for (int i = 0; i < IO::N; ++i) partial[(int64_t)blockIdx.x * H + v * IO::N + i] = dw[c][i];
      }
    }
  }
}

// d_w[h] = (accumulate ? d_w[h] : 0) + sum_b partial[b, h], b ascending
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, int nb,
                                                                 T* __restrict__ d_w, int64_t H, int accumulate) {
  const int64_t h = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (h >= H) return;
  float s = 0.f;
  for (int b = 0; b < nb; ++b) s += partial[(int64_t)b * H + h];
  if (accumulate) s += pk_to_float<T>(d_w[h]);
  d_w[h] = pk_from_float<T>(s);
}

// Rows too long for the register-resident kernel (or not vectorisable): d_x with strided loops,
// one block per row, and d_w as plain column sums (one thread per column, rows in order).
template <typename T>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_bwd_dx_generic_kernel(
    const T* __restrict__ d_y, const T* __restrict__ x, const T* __restrict__ w,
    const float* __restrict__ rstd, const T* __restrict__ addend, T* __restrict__ d_x, int64_t H) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float rs = rstd[t];
  float dot = 0.f;
  for (int64_t h = threadIdx.x; h < H; h += kRowThreads)
    dot = fmaf(pk_to_float<T>(d_y[t * H + h]) * pk_to_float<T>(w[h]), pk_to_float<T>(x[t * H + h]) * rs, dot);
  dot = pk_block_sum(dot, red) / (float)H;
  for (int64_t h = threadIdx.x; h < H; h += kRowThreads) {
    const float xh = pk_to_float<T>(x[t * H + h]) * rs;
    float o = rs * (pk_to_float<T>(d_y[t * H + h]) * pk_to_float<T>(w[h]) - xh * dot);
    if (addend) o = pk_to_float<T>(pk_from_float<T>(o)) + pk_to_float<T>(addend[t * H + h]);
    d_x[t * H + h] = pk_from_float<T>(o);
  }
}
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_dw_generic_kernel(const T* __restrict__ d_y, const T* __restrict__ x,
                                                                  const float* __restrict__ rstd, T* __restrict__ d_w,
                                                                  int64_t rows, int64_t H, int accumulate) {
  const int64_t h = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (h >= H) return;
  float s = 0.f;
  for (int64_t t = 0; t < rows; ++t) s = fmaf(pk_to_float<T>(d_y[t * H + h]), pk_to_float<T>(x[t * H + h]) * rstd[t], s);
  if (accumulate) s += pk_to_float<T>(d_w[h]);
  d_w[h] = pk_from_float<T>(s);
}

constexpr int kNormBwdBlocks = 512;
constexpr int kNormBwdMaxCpt = 4;   // column vectors per thread

bool vec_ok(int dtype, int64_t H, std::initializer_list<const void*> ptrs) {
  const int n = dtype == PK_BF16 ? 8 : 4;
  if (H % n != 0) return false;
  for (const void* p : ptrs)
    if (p && !pk_aligned16(p)) return false;
  return true;
}


template <typename T, bool VEC>
int rmsnorm_bwd_launch(const void* d_y, const void* x, const void* weight, const float* rstd,
                       const void* addend, void* d_x, float* partial, int64_t rows, int64_t H,
                       int nb, hipStream_t s) {
  const int64_t nv = H / (VEC ? PkVec16<T>::N : 1);
  const int64_t cpt = pk_ceil_div(nv, kRowThreads);
  const dim3 grid((unsigned)nb);
#define PK_NORM_BWD(C)                                                                                       \
  PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_BWD, s, (rmsnorm_bwd_kernel<T, VEC, C>), grid, dim3(kRowThreads), 0, s, \
                    (const T*)d_y, (const T*)x, (const T*)weight, rstd, (const T*)addend, (T*)d_x, partial, rows, H)
  if (cpt <= 1) { PK_NORM_BWD(1); }
  else if (cpt <= 2) { PK_NORM_BWD(2); }
  else if (cpt <= kNormBwdMaxCpt) { PK_NORM_BWD(4); }
  else return PK_ERR_UNSUPPORTED;   // the caller takes the generic kernels
#undef PK_NORM_BWD
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

// buf[r, :] = 0 for r in [*first_row, rows): the rows of an expert-sorted buffer that no expert
// owns.  The first row is read on the device, so the grid is fixed and the blocks stride the rows.
__global__ __launch_bounds__(kRowThreads) void zero_rows_from_kernel(char* __restrict__ buf, const int32_t* __restrict__ first_row,
                                                                     int64_t rows, int64_t row_bytes) {
  for (int64_t r = (int64_t)*first_row + blockIdx.x; r < rows; r += gridDim.x) {
    char* row = buf + r * row_bytes;
    if ((row_bytes & 15) == 0 && (((uintptr_t)buf) & 15) == 0) {
      const u32x4_t z = {0u, 0u, 0u, 0u};
      for (int64_t v = threadIdx.x; v < row_bytes / 16; v += kRowThreads) reinterpret_cast<u32x4_t*>(row)[v] = z;
    } else {
      for (int64_t v = threadIdx.x; v < row_bytes; v += kRowThreads) row[v] = 0;
    }
  }
}

}  // namespace

extern "C" {

int pk_zero_rows_from(void* buf, int dtype, const int32_t* first_row, int64_t rows, int64_t width, pk_stream_t stream) {
  if (rows < 0 || width <= 0 || !pk_dtype_ok(dtype)) return PK_ERR_ARG;
  if (rows == 0) return PK_OK;
  if (!buf || !first_row) return PK_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const unsigned grid = (unsigned)(rows < 512 ? rows : 512);
  PK_LAUNCH_NOCHECK(pk_timing::K_MISC, s, zero_rows_from_kernel, dim3(grid), dim3(kRowThreads), 0, s, (char*)buf, first_row,
                    rows, width * (int64_t)pk_dtype_size(dtype));
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

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
                         const float* addend, const void* residual, void* out, int64_t T, int64_t H,
                         int64_t K, pk_stream_t stream) {
  if (T < 0 || H <= 0 || K <= 0 || !pk_dtype_ok(dtype)) return PK_ERR_ARG;
  if (T == 0) return PK_OK;
  if (!rows || !inv_perm || !out) return PK_ERR_ARG;
  if (T > 0x7fffffffll) return PK_ERR_SHAPE;
  const bool vec = vec_ok(dtype, H, {rows, out, residual});
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)T);
  // rows that do not fit the memory-side cache (256 MB) are streamed
  const bool stream_rows = T * K * H * (int64_t)pk_dtype_size(dtype) > (int64_t)192 * 1024 * 1024;
#define PK_GATHER_REDUCE(TYPE, VECF, STREAMF)                                                                          \
  PK_LAUNCH_NOCHECK(pk_timing::K_GATHER_REDUCE, s, (gather_reduce_kernel<TYPE, VECF, STREAMF>), grid, dim3(kRowThreads), 0, s, \
                    (const TYPE*)rows, inv_perm, weights, addend, (const TYPE*)residual, (TYPE*)out, H, (int)K)
  if (dtype == PK_BF16) {
    if (vec && stream_rows) PK_GATHER_REDUCE(bf16_t, true, true);
    else if (vec) PK_GATHER_REDUCE(bf16_t, true, false);
    else PK_GATHER_REDUCE(bf16_t, false, false);
  } else {
    if (vec && stream_rows) PK_GATHER_REDUCE(float, true, true);
    else if (vec) PK_GATHER_REDUCE(float, true, false);
    else PK_GATHER_REDUCE(float, false, false);
  }
#undef PK_GATHER_REDUCE
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int pk_permute_bwd(const void* d_routed, int dtype, const int32_t* inv_perm,
                   const float* addend_f32, void* d_x, int64_t T, int64_t H, int64_t K,
                   pk_stream_t stream) {
  return gather_reduce(d_routed, dtype, inv_perm, nullptr, addend_f32, nullptr, d_x, T, H, K, stream);
}

int pk_combine_fwd(const void* y_sorted, int dtype, const int32_t* inv_perm,
                   const float* top_scores, const void* residual, void* out, int64_t T, int64_t H,
                   int64_t K, pk_stream_t stream) {
  if (!top_scores && T > 0) return PK_ERR_ARG;
  return gather_reduce(y_sorted, dtype, inv_perm, top_scores, nullptr, residual, out, T, H, K, stream);
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

int pk_rmsnorm_fwd(const void* x, int dtype, const void* weight, float eps, void* y, float* rstd,
                   int64_t T, int64_t H, pk_stream_t stream) {
  if (T < 0 || H <= 0 || !pk_dtype_ok(dtype) || !(eps >= 0.f)) return PK_ERR_ARG;
  if (T == 0) return PK_OK;
  if (!x || !weight || !y) return PK_ERR_ARG;
  if (T > 0x7fffffffll) return PK_ERR_SHAPE;
  const bool vec = vec_ok(dtype, H, {x, weight, y});
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)T);
  if (dtype == PK_BF16) {
    if (vec) PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_FWD, s, (rmsnorm_fwd_kernel<bf16_t, true>), grid, dim3(kRowThreads), 0, s, (const bf16_t*)x, (const bf16_t*)weight, eps, (bf16_t*)y, rstd, H);
    else PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_FWD, s, (rmsnorm_fwd_kernel<bf16_t, false>), grid, dim3(kRowThreads), 0, s, (const bf16_t*)x, (const bf16_t*)weight, eps, (bf16_t*)y, rstd, H);
  } else {
    if (vec) PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_FWD, s, (rmsnorm_fwd_kernel<float, true>), grid, dim3(kRowThreads), 0, s, (const float*)x, (const float*)weight, eps, (float*)y, rstd, H);
    else PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_FWD, s, (rmsnorm_fwd_kernel<float, false>), grid, dim3(kRowThreads), 0, s, (const float*)x, (const float*)weight, eps, (float*)y, rstd, H);
  }
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int64_t pk_rmsnorm_bwd_workspace_bytes(int64_t T, int64_t H) {
  if (T < 0 || H <= 0) return PK_ERR_ARG;
  const int64_t nb = T < kNormBwdBlocks ? (T > 0 ? T : 1) : kNormBwdBlocks;
  return nb * H * (int64_t)sizeof(float);
}

int pk_rmsnorm_bwd(const void* d_y, const void* x, int dtype, const void* weight, const float* rstd,
                   const void* d_x_addend, void* d_x, void* d_weight, int accumulate, int64_t T,
                   int64_t H, void* workspace, int64_t workspace_bytes, pk_stream_t stream) {
  if (T < 0 || H <= 0 || !pk_dtype_ok(dtype)) return PK_ERR_ARG;
  if (T == 0) return PK_OK;
  if (!d_y || !x || !weight || !rstd || !d_x) return PK_ERR_ARG;
  if (T > 0x7fffffffll) return PK_ERR_SHAPE;
  const int nb = (int)(T < kNormBwdBlocks ? T : kNormBwdBlocks);
  float* partial = nullptr;
  if (d_weight) {
    if (!workspace || workspace_bytes < pk_rmsnorm_bwd_workspace_bytes(T, H)) return PK_ERR_WORKSPACE;
    partial = reinterpret_cast<float*>(workspace);
  }
  const bool vec = vec_ok(dtype, H, {d_y, x, weight, d_x, d_x_addend});
  hipStream_t s = (hipStream_t)stream;
  int rc;
  if (dtype == PK_BF16)
    rc = vec ? rmsnorm_bwd_launch<bf16_t, true>(d_y, x, weight, rstd, d_x_addend, d_x, partial, T, H, nb, s)
             : rmsnorm_bwd_launch<bf16_t, false>(d_y, x, weight, rstd, d_x_addend, d_x, partial, T, H, nb, s);
  else
    rc = vec ? rmsnorm_bwd_launch<float, true>(d_y, x, weight, rstd, d_x_addend, d_x, partial, T, H, nb, s)
             : rmsnorm_bwd_launch<float, false>(d_y, x, weight, rstd, d_x_addend, d_x, partial, T, H, nb, s);
  if (rc == PK_ERR_UNSUPPORTED) {
    const dim3 rows_grid((unsigned)T), cols_grid((unsigned)pk_ceil_div(H, 256));
    if (dtype == PK_BF16) {
      PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_BWD, s, (rmsnorm_bwd_dx_generic_kernel<bf16_t>), rows_grid, dim3(kRowThreads), 0, s, (const bf16_t*)d_y, (const bf16_t*)x, (const bf16_t*)weight, rstd, (const bf16_t*)d_x_addend, (bf16_t*)d_x, H);
      if (d_weight) PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_BWD, s, (rmsnorm_dw_generic_kernel<bf16_t>), cols_grid, dim3(256), 0, s, (const bf16_t*)d_y, (const bf16_t*)x, rstd, (bf16_t*)d_weight, T, H, accumulate ? 1 : 0);
    } else {
      PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_BWD, s, (rmsnorm_bwd_dx_generic_kernel<float>), rows_grid, dim3(kRowThreads), 0, s, (const float*)d_y, (const float*)x, (const float*)weight, rstd, (const float*)d_x_addend, (float*)d_x, H);
      if (d_weight) PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_BWD, s, (rmsnorm_dw_generic_kernel<float>), cols_grid, dim3(256), 0, s, (const float*)d_y, (const float*)x, rstd, (float*)d_weight, T, H, accumulate ? 1 : 0);
    }
    PK_RETURN_IF_LAUNCH_FAILED();
    return PK_OK;
  }
  if (rc != PK_OK) return rc;
  if (d_weight) {
    const dim3 grid((unsigned)pk_ceil_div(H, 256));
    if (dtype == PK_BF16)
      PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_BWD, s, (rmsnorm_dw_reduce_kernel<bf16_t>), grid, dim3(256), 0, s, partial, nb, (bf16_t*)d_weight, H, accumulate ? 1 : 0);
    else
      PK_LAUNCH_NOCHECK(pk_timing::K_RMSNORM_BWD, s, (rmsnorm_dw_reduce_kernel<float>), grid, dim3(256), 0, s, partial, nb, (float*)d_weight, H, accumulate ? 1 : 0);
    PK_RETURN_IF_LAUNCH_FAILED();
  }
  return PK_OK;
}

}  // extern "C"
