// Dense GEMM with exact fp32 products on v_mfma_f32_32x32x2_f32, for the router gate
// (logits, d_x, d_w_gate).  C[M,N] = sum_k A(m,k) * B(k,n), operands fp32 or bf16 (widened on
// load), arbitrary extents (edges are masked), optional split of the reduction dimension over
// blockIdx.z with partial results written to a workspace for a fixed-order second pass.
#pragma once
#include "pk_common.h"

namespace pk_f32mm {

constexpr int BK = 32;
constexpr int LDS_LD = BK + 1;  // +1 float: conflict-free fragment reads

struct Params {
  const void* A;
  const void* B;
  float* C;            // splits == 1: the result;  splits > 1: partials [splits][M][N]
  const float* bias;   // optional [N], added when splits == 1
  int64_t M, N, K;
  int64_t sam, sak;    // element strides of A(m,k)
  int64_t sbk, sbn;    // element strides of B(k,n)
  int32_t splits;
  int32_t accumulate;  // splits == 1: C += result
  int64_t plane_a, plane_b;   // elements between the bf16 planes of a pre-split operand (mfma_x3_gemm.h)
};

// Four consecutive elements of an operand as floats (16-byte / 8-byte load).
template <typename T>
__device__ __forceinline__ void load4(const T* p, float (&out)[4]);
template <>
__device__ __forceinline__ void load4<float>(const float* p, float (&out)[4]) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
}
template <>
__device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float (&out)[4]) {
  const bf16x4_t v = *reinterpret_cast<const bf16x4_t*>(p);
#pragma unroll
  for (int j = 0; j < 4; ++j) out[j] = (float)v[j];
}

// A_KC / B_KC: the operand's k index is the contiguous one in memory (coalesce along k),
// otherwise coalesce along m / n.  VEC: every thread fetches 4 consecutive elements of the
// contiguous index per load (the host checks extents, strides and alignment); without it
// loads are scalar and any extent works.
template <int WM, int WN, bool A_KC, bool B_KC, typename TA, typename TB, bool VEC>
__global__ __launch_bounds__(64 * WM * WN) void kernel(const Params p) {
  constexpr int BM = 32 * WM, BN = 32 * WN, THREADS = 64 * WM * WN;
  __shared__ float As[BM * LDS_LD];
  __shared__ float Bs[BN * LDS_LD];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave / WN, wn = wave % WN;
  const int64_t m0 = (int64_t)blockIdx.y * BM, n0 = (int64_t)blockIdx.x * BN;
  const int64_t kchunk = ((p.K + p.splits - 1) / p.splits + BK - 1) / BK * BK;
  const int64_t kbeg = (int64_t)blockIdx.z * kchunk;
  const int64_t kend = kbeg + kchunk < p.K ? kbeg + kchunk : p.K;

  const TA* A = reinterpret_cast<const TA*>(p.A);
  const TB* B = reinterpret_cast<const TB*>(p.B);

  floatx16_t acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;

  // register prefetch: the loads of tile k+1 are in flight while tile k is multiplied
  constexpr int W = VEC ? 4 : 1;
  constexpr int NA = BM * BK / (THREADS * W), NB = BN * BK / (THREADS * W);
  static_assert(NA >= 1 && NB >= 1, "tile too small for the thread count");
  float ra[NA][W], rb[NB][W];
  // element (row = m or n index in the tile, k) of the idx-th load of a tile with R rows
  auto slot = [](int idx, bool kc, int R, int& row, int& k) {
    if (kc) { k = (idx % (BK / W)) * W; row = idx / (BK / W); }
    else { row = (idx % (R / W)) * W; k = idx / (R / W); }
  };
  auto load_tile = [&](int64_t k0) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      int m, k;
      slot(tid + i * THREADS, A_KC, BM, m, k);
#pragma unroll
      for (int j = 0; j < W; ++j) ra[i][j] = 0.f;
      if (m0 + m < p.M && k0 + k < kend) {
        const TA* src = A + (m0 + m) * p.sam + (k0 + k) * p.sak;
        if (VEC) load4<TA>(src, reinterpret_cast<float(&)[4]>(ra[i]));
        else ra[i][0] = pk_to_float<TA>(*src);
      }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      int n, k;
      slot(tid + i * THREADS, B_KC, BN, n, k);
#pragma unroll
      for (int j = 0; j < W; ++j) rb[i][j] = 0.f;
      if (n0 + n < p.N && k0 + k < kend) {
        const TB* src = B + (k0 + k) * p.sbk + (n0 + n) * p.sbn;
        if (VEC) load4<TB>(src, reinterpret_cast<float(&)[4]>(rb[i]));
        else rb[i][0] = pk_to_float<TB>(*src);
      }
    }
  };
  if (kbeg < kend) load_tile(kbeg);
  for (int64_t k0 = kbeg; k0 < kend; k0 += BK) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      int m, k;
      slot(tid + i * THREADS, A_KC, BM, m, k);
#pragma unroll
      for (int j = 0; j < W; ++j) As[(A_KC ? m : m + j) * LDS_LD + (A_KC ? k + j : k)] = ra[i][j];
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      int n, k;
      slot(tid + i * THREADS, B_KC, BN, n, k);
#pragma unroll
      for (int j = 0; j < W; ++j) Bs[(B_KC ? n : n + j) * LDS_LD + (B_KC ? k + j : k)] = rb[i][j];
    }
    __syncthreads();
    if (k0 + BK < kend) load_tile(k0 + BK);
    const float* a = As + (wm * 32 + (lane & 31)) * LDS_LD + (lane >> 5);
    const float* b = Bs + (wn * 32 + (lane & 31)) * LDS_LD + (lane >> 5);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kk], b[kk], acc, 0, 0, 0);
    __syncthreads();
  }

  float* C = p.C + (p.splits > 1 ? (int64_t)blockIdx.z * p.M * p.N : 0);
  const int64_t n = n0 + wn * 32 + (lane & 31);
  if (n < p.N) {
    const float bias = (p.bias && p.splits == 1) ? p.bias[n] : 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int64_t m = m0 + wm * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      if (m < p.M) {
        float r = acc[v] + bias;
        if (p.accumulate && p.splits == 1) r += C[m * p.N + n];
        C[m * p.N + n] = r;
      }
    }
  }
}

// out[i] = (accumulate ? out[i] : 0) + sum_z partial[z][i], z ascending: a fixed summation order.
// bias (optional) has N entries and is added per column.
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ partial,
                                                              float* __restrict__ out, int64_t n,
                                                              int splits, int accumulate,
                                                              const float* __restrict__ bias, int N) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = accumulate ? out[i] : 0.f;
  for (int z = 0; z < splits; ++z) s += partial[(int64_t)z * n + i];
  if (bias) s += bias[i % N];
  out[i] = s;
}

// Whether every 4-element group along the contiguous index of an operand can be fetched with one
// aligned load: extent and the other stride multiples of 4, base aligned to 4 elements.
template <typename T>
inline bool vec4_ok(const void* base, int64_t contig_extent, int64_t other_stride) {
  return contig_extent % 4 == 0 && other_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(base) % (4 * sizeof(T))) == 0;
}

template <int WM, int WN, bool A_KC, bool B_KC, typename TA, typename TB>
inline int launch(const Params& p, int kernel_id, hipStream_t s) {
  if (p.M <= 0 || p.N <= 0) return PK_OK;
  dim3 grid((unsigned)pk_ceil_div(p.N, 32 * WN), (unsigned)pk_ceil_div(p.M, 32 * WM), (unsigned)p.splits);
  if (grid.y > 65535u || grid.z > 65535u) return PK_ERR_SHAPE;
  const bool vec = (A_KC ? (p.sak == 1 && vec4_ok<TA>(p.A, p.K, p.sam)) : (p.sam == 1 && vec4_ok<TA>(p.A, p.M, p.sak))) &&
                   (B_KC ? (p.sbk == 1 && vec4_ok<TB>(p.B, p.K, p.sbn)) : (p.sbn == 1 && vec4_ok<TB>(p.B, p.N, p.sbk)));
  if (vec)
    PK_LAUNCH_NOCHECK(kernel_id, s, (kernel<WM, WN, A_KC, B_KC, TA, TB, true>), grid, dim3(64 * WM * WN), 0, s, p);
  else
    PK_LAUNCH_NOCHECK(kernel_id, s, (kernel<WM, WN, A_KC, B_KC, TA, TB, false>), grid, dim3(64 * WM * WN), 0, s, p);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

}  // namespace pk_f32mm
