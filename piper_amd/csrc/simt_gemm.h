// Tiled fp32-FMA grouped GEMM for arbitrary strides, used where exact fp32 arithmetic is
// required (fp32 experts, router gate) and as the shape-unrestricted fallback.
//   C(m,n) = sum_k A(m,k) * B(k,n)  (+ C(m,n) when accumulate)
// One "group" per expert.  Either the M dimension or the K dimension is ragged: group g
// owns rows [starts[g], starts[g+1]) of the operand(s) indexed by that dimension.
#pragma once
#include "pk_common.h"

namespace pk_simt {

constexpr int TM = 64, TN = 64, TK = 16, THREADS = 256;

enum Ragged { RAGGED_NONE = 0, RAGGED_M = 1, RAGGED_K = 2 };

struct Params {
  const void* A;
  const void* B;
  void* C;
  const int32_t* starts;  // [G+1] row offsets of the ragged dimension (RAGGED_M / RAGGED_K)
  const int32_t* a_map;   // optional gather on A's ragged row index: row -> a_map[row] / map_div
  const int32_t* b_map;   // same for B (only meaningful for RAGGED_K)
  int32_t map_div;
  int32_t ragged;
  int32_t G;
  int32_t accumulate;
  int64_t M, N, K;        // fixed extents (the ragged one is ignored)
  int64_t sam, sak;       // A element strides
  int64_t sbk, sbn;       // B element strides
  int64_t scm, scn;       // C element strides
  int64_t gA, gB, gC;     // per-group base offsets in elements (0 when the operand is shared/ragged)
  int32_t total_m_tiles;  // RAGGED_M: upper bound of sum_g ceil(M_g / TM)
};

template <typename TA, typename TB, typename TC>
__global__ __launch_bounds__(THREADS) void gemm_kernel(const Params p) {
  __shared__ float As[TK][TM + 4];
  __shared__ float Bs[TK][TN + 4];
  __shared__ int s_group, s_mtile;

  int g, mt;
  if (p.ragged == RAGGED_M) {
    if (threadIdx.x == 0) {
      int acc = 0, found = -1, tile = 0;
      for (int e = 0; e < p.G; ++e) {
        const int cnt = p.starts[e + 1] - p.starts[e];
        const int nt = (cnt + TM - 1) / TM;
        if ((int)blockIdx.y < acc + nt) { found = e; tile = blockIdx.y - acc; break; }
        acc += nt;
      }
      s_group = found;
      s_mtile = tile;
    }
    __syncthreads();
    g = s_group;
    mt = s_mtile;
    if (g < 0) return;
  } else {
    g = blockIdx.z;
    mt = blockIdx.y;
  }
  const int nt = blockIdx.x;

  int64_t Mg = p.M, Kg = p.K;
  int64_t row0 = 0;  // offset of the ragged dimension
  if (p.ragged == RAGGED_M) { row0 = p.starts[g]; Mg = p.starts[g + 1] - row0; }
  if (p.ragged == RAGGED_K) { row0 = p.starts[g]; Kg = p.starts[g + 1] - row0; }

  const TA* A = reinterpret_cast<const TA*>(p.A) + (int64_t)g * p.gA;
  const TB* B = reinterpret_cast<const TB*>(p.B) + (int64_t)g * p.gB;
  TC* C = reinterpret_cast<TC*>(p.C) + (int64_t)g * p.gC;

  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;  // 16 x 16 threads, 4x4 outputs each
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const int64_t m0 = (int64_t)mt * TM, n0 = (int64_t)nt * TN;

  for (int64_t k0 = 0; k0 < Kg; k0 += TK) {
    // A tile: TM x TK, B tile: TK x TN; 1024 elements each, 4 per thread
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = threadIdx.x + i * THREADS;
      {
        const int m = idx % TM, k = idx / TM;
        float v = 0.f;
        const int64_t gm = m0 + m, gk = k0 + k;
        if (gm < Mg && gk < Kg) {
          int64_t rm = gm, rk = gk;
          if (p.ragged == RAGGED_M) { rm += row0; if (p.a_map) rm = p.a_map[rm] / p.map_div; }
          if (p.ragged == RAGGED_K) { rk += row0; if (p.a_map) rk = p.a_map[rk] / p.map_div; }
          v = pk_to_float<TA>(A[rm * p.sam + rk * p.sak]);
        }
        As[k][m] = v;
      }
      {
        const int n = idx % TN, k = idx / TN;
        float v = 0.f;
        const int64_t gn = n0 + n, gk = k0 + k;
        if (gn < p.N && gk < Kg) {
          int64_t rk = gk;
          if (p.ragged == RAGGED_K) { rk += row0; if (p.b_map) rk = p.b_map[rk] / p.map_div; }
          v = pk_to_float<TB>(B[rk * p.sbk + gn * p.sbn]);
        }
        Bs[k][n] = v;
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t gm = m0 + ty * 4 + i;
    if (gm >= Mg) continue;
    const int64_t rm = (p.ragged == RAGGED_M) ? gm + row0 : gm;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t gn = n0 + tx * 4 + j;
      if (gn >= p.N) continue;
      TC* c = C + rm * p.scm + gn * p.scn;
      float v = acc[i][j];
      if (p.accumulate) v += pk_to_float<TC>(*c);
      *c = pk_from_float<TC>(v);
    }
  }
}

template <typename TA, typename TB, typename TC>
inline int launch(Params p, hipStream_t s) {
  dim3 grid;
  grid.x = (unsigned)pk_ceil_div(p.N, TN);
  if (p.ragged == RAGGED_M) {
    grid.y = (unsigned)p.total_m_tiles;
    grid.z = 1;
  } else {
    grid.y = (unsigned)pk_ceil_div(p.M, TM);
    grid.z = (unsigned)(p.G > 0 ? p.G : 1);
  }
  if (grid.x == 0 || grid.y == 0) return PK_OK;
  if (grid.y > 65535u || grid.z > 65535u) return PK_ERR_SHAPE;
  PK_LAUNCH_NOCHECK(pk_timing::K_SIMT_GEMM, s, (gemm_kernel<TA, TB, TC>), grid, dim3(THREADS), 0, s, p);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

}  // namespace pk_simt
