// Dense GEMM C[M,N] = sum_k A(m,k) * B(k,n) with fp32-accurate products on the bf16 matrix
// cores: an fp32 operand is split exactly into three bf16 planes (v = hi + mid + lo, 8 mantissa
// bits each), a bf16 operand is its own single plane, and every pair of planes whose product is
// not below 2^-24 of the leading one is multiplied with v_mfma_f32_32x32x16_bf16 into one fp32
// accumulator (3 MFMAs for bf16 x fp32, 6 for fp32 x fp32).  Plane products are exact in fp32, so
// the result differs from an fp32 FMA chain only by summation order and the dropped 2^-24 terms.
// Against v_mfma_f32_32x32x2_f32 this is 5.3x (bf16 x fp32) / 2.7x (fp32 x fp32) fewer matrix-core
// cycles.  Same Params, tiling, split-K and epilogue as mfma_f32_gemm.h.  An operand whose k index
// is not the contiguous one is kept in LDS as [k][row] (8-byte stores of the 4 fetched elements)
// and turned into MFMA fragments by the transposing LDS read (ds_read_b64_tr_b16).
// An fp32 operand can also be handed over already split (split3_t: three bf16 planes in memory, made
// once by split_planes_kernel): every workgroup that loads a tile of an fp32 operand otherwise
// splits it again (about 20 vector instructions per MFMA with tiles this small).  The planes are
// 6 bytes per element where the fp32 value is 4, so this pays only where the split arithmetic is
// what the kernel waits for: measured, the gate weight gradient (a long reduction over the tokens,
// d_logits re-read by every column tile) gains a fifth, the forward and the d_x GEMM lose.
#pragma once
#include "mfma_f32_gemm.h"
#include <type_traits>

namespace pk_x3mm {

using pk_f32mm::Params;
constexpr int BK = 32;
constexpr int LDK = BK + 8;   // bf16 per LDS row: 80-byte rows keep 16-byte fragment reads aligned
constexpr int MN_PAD = 8;     // bf16 of padding per [k][row] LDS row

typedef short shortx4_t __attribute__((ext_vector_type(4)));
typedef short shortx8_t __attribute__((ext_vector_type(8)));

// MFMA operand fragment (lane -> row lane%32, k = kk + 8*(lane/32) + 0..7) of a [row][k] tile
__device__ __forceinline__ bf16x8_t frag_kc(const bf16_t* tile, int row0, int kk, int lane) {
  return *reinterpret_cast<const bf16x8_t*>(tile + (row0 + (lane & 31)) * LDK + kk + 8 * (lane >> 5));
}
// the same fragment out of a [k][row] tile with `ld` bf16 per k-row: within 16 lanes, lane i
// points at 4 consecutive rows of k-row i/4 and receives 4 consecutive k of row i
__device__ __forceinline__ bf16x8_t frag_mn(const bf16_t* tile, int ld, int row0, int kk, int lane) {
  const int i = lane & 15;
  const int krow = kk + 8 * (lane >> 5) + (i >> 2);
  const int row = row0 + 16 * ((lane >> 4) & 1) + 4 * (i & 3);
  const bf16_t* ptr = tile + krow * ld + row;
  const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4_t*)(ptr));
  const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4_t*)(ptr + 4 * ld));
  return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// operand element types: float (split on load), bf16_t (one plane), split3_t (three bf16 planes in
// memory: plane q of element i at base[q * plane_stride + i])
struct split3_t {};
template <typename T> struct Planes;
template <> struct Planes<float> { static constexpr int N = 3; };
template <> struct Planes<bf16_t> { static constexpr int N = 1; };
template <> struct Planes<split3_t> { static constexpr int N = 3; };
template <typename T> struct Mem { typedef T type; };
template <> struct Mem<split3_t> { typedef bf16_t type; };      // what the operand pointer points at

// fp32 [n] -> three bf16 planes [3][n]: hi = bf16(v), mid = bf16(v - hi), lo = bf16(v - hi - mid)
__global__ __launch_bounds__(256) void split_planes_kernel(const float* __restrict__ src, bf16_t* __restrict__ dst, int64_t n) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i + 4 <= n) {
    const float4 v = *reinterpret_cast<const float4*>(src + i);
    const float f[4] = {v.x, v.y, v.z, v.w};
    bf16x4_t pl[3];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bf16_t hi = (bf16_t)f[j];
      const float r1 = f[j] - (float)hi;
      const bf16_t mid = (bf16_t)r1;
      pl[0][j] = hi; pl[1][j] = mid; pl[2][j] = (bf16_t)(r1 - (float)mid);
    }
#pragma unroll
    for (int q = 0; q < 3; ++q) *reinterpret_cast<bf16x4_t*>(dst + q * n + i) = pl[q];
  } else {
    for (int64_t e = i; e < n; ++e) {
      const bf16_t hi = (bf16_t)src[e];
      const float r1 = src[e] - (float)hi;
      const bf16_t mid = (bf16_t)r1;
      dst[e] = hi; dst[n + e] = mid; dst[2 * n + e] = (bf16_t)(r1 - (float)mid);
    }
  }
}

template <int P>
__device__ __forceinline__ void split(float v, bf16_t (&out)[P]) {
  out[0] = (bf16_t)v;
  if (P > 1) {
    const float r1 = v - (float)out[0];
    out[1] = (bf16_t)r1;
    if (P > 2) out[2] = (bf16_t)(r1 - (float)out[1]);
  }
}
template <int P>
__device__ __forceinline__ void zero_planes(bf16x4_t (&out)[P]) {
  const bf16x4_t zero = {(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
#pragma unroll
  for (int q = 0; q < P; ++q) out[q] = zero;
}
// four consecutive elements of an operand as planes of four bf16
template <typename T>
__device__ __forceinline__ void fetch4(const typename Mem<T>::type* src, int64_t plane_stride, bf16x4_t (&out)[Planes<T>::N]) {
  constexpr int P = Planes<T>::N;
  if constexpr (std::is_same<T, float>::value) {
    float v[4];
    pk_f32mm::load4<float>(src, v);
    bf16_t pl[4][P];
#pragma unroll
    for (int j = 0; j < 4; ++j) split<P>(v[j], pl[j]);
#pragma unroll
    for (int q = 0; q < P; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) out[q][j] = pl[j][q];
  } else {
#pragma unroll
    for (int q = 0; q < P; ++q) out[q] = *reinterpret_cast<const bf16x4_t*>(src + q * plane_stride);
  }
}

template <int WM, int WN, bool A_KC, bool B_KC, typename TA, typename TB>
__global__ __launch_bounds__(64 * WM * WN) void kernel(const Params p) {
  constexpr int BM = 32 * WM, BN = 32 * WN, THREADS = 64 * WM * WN;
  constexpr int PA = Planes<TA>::N, PB = Planes<TB>::N;
  constexpr int LDA = BM + MN_PAD, LDB = BN + MN_PAD;     // [k][row] layouts
  __shared__ __attribute__((aligned(16))) bf16_t As[PA][A_KC ? BM * LDK : BK * LDA];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[PB][B_KC ? BN * LDK : BK * LDB];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave / WN, wn = wave % WN;
  const int64_t m0 = (int64_t)blockIdx.y * BM, n0 = (int64_t)blockIdx.x * BN;
  const int64_t kchunk = ((p.K + p.splits - 1) / p.splits + BK - 1) / BK * BK;
  const int64_t kbeg = (int64_t)blockIdx.z * kchunk;
  const int64_t kend = kbeg + kchunk < p.K ? kbeg + kchunk : p.K;

  typedef typename Mem<TA>::type MA;
  typedef typename Mem<TB>::type MB;
  const MA* A = reinterpret_cast<const MA*>(p.A);
  const MB* B = reinterpret_cast<const MB*>(p.B);

  floatx16_t acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;

  // every thread fetches 4 consecutive elements of the contiguous index per load (every plane of
  // them for a pre-split operand); the loads of tile k+1 are in flight while tile k is multiplied
  constexpr int NA = BM * BK / (THREADS * 4), NB = BN * BK / (THREADS * 4);
  static_assert(NA >= 1 && NB >= 1, "tile too small for the thread count");
  // four fetched elements as planes of four bf16 (an fp32 operand is split here, once per load)
  bf16x4_t ra[NA][PA], rb[NB][PB];
  auto slot = [](int idx, bool kc, int R, int& row, int& k) {
    if (kc) { k = (idx % (BK / 4)) * 4; row = idx / (BK / 4); }
    else { row = (idx % (R / 4)) * 4; k = idx / (R / 4); }
  };
  auto load_tile = [&](int64_t k0) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      int m, k;
      slot(tid + i * THREADS, A_KC, BM, m, k);
      zero_planes<PA>(ra[i]);
      if (m0 + m < p.M && k0 + k < kend) fetch4<TA>(A + (m0 + m) * p.sam + (k0 + k) * p.sak, p.plane_a, ra[i]);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      int n, k;
      slot(tid + i * THREADS, B_KC, BN, n, k);
      zero_planes<PB>(rb[i]);
      if (n0 + n < p.N && k0 + k < kend) fetch4<TB>(B + (k0 + k) * p.sbk + (n0 + n) * p.sbn, p.plane_b, rb[i]);
    }
  };
  // one 8-byte store per plane: along k of a [row][k] tile for a K-contiguous operand, along the
  // rows of a [k][row] tile otherwise
  auto store4 = [](auto& tiles, auto nplanes, bool kc, int ld_mn, int row, int k, const auto& v) {
    constexpr int P = decltype(nplanes)::value;
#pragma unroll
    for (int q = 0; q < P; ++q) *reinterpret_cast<bf16x4_t*>(&tiles[q][kc ? row * LDK + k : k * ld_mn + row]) = v[q];
  };
  if (kbeg < kend) load_tile(kbeg);
  for (int64_t k0 = kbeg; k0 < kend; k0 += BK) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      int m, k;
      slot(tid + i * THREADS, A_KC, BM, m, k);
      store4(As, std::integral_constant<int, PA>{}, A_KC, LDA, m, k, ra[i]);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      int n, k;
      slot(tid + i * THREADS, B_KC, BN, n, k);
      store4(Bs, std::integral_constant<int, PB>{}, B_KC, LDB, n, k, rb[i]);
    }
    __syncthreads();
    if (k0 + BK < kend) load_tile(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8_t a[PA], b[PB];
#pragma unroll
      for (int pl = 0; pl < PA; ++pl) a[pl] = A_KC ? frag_kc(As[pl], wm * 32, kk, lane) : frag_mn(As[pl], LDA, wm * 32, kk, lane);
#pragma unroll
      for (int pl = 0; pl < PB; ++pl) b[pl] = B_KC ? frag_kc(Bs[pl], wn * 32, kk, lane) : frag_mn(Bs[pl], LDB, wn * 32, kk, lane);
      // small terms first
#pragma unroll
      for (int s = PA + PB - 2; s >= 0; --s)
#pragma unroll
        for (int pa = 0; pa < PA; ++pa) {
          const int pb = s - pa;
          if (pb >= 0 && pb < PB && s <= 2) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[pa], b[pb], acc, 0, 0, 0);
        }
    }
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

// The operands must allow 4-element loads (pk_f32mm::vec4_ok); the caller falls back to
// pk_f32mm::launch otherwise.
template <int WM, int WN, bool A_KC, bool B_KC, typename TA, typename TB>
inline bool usable(const Params& p) {
  using pk_f32mm::vec4_ok;
  typedef typename Mem<TA>::type MA;
  typedef typename Mem<TB>::type MB;
  if (std::is_same<TA, split3_t>::value && p.plane_a % 4 != 0) return false;
  if (std::is_same<TB, split3_t>::value && p.plane_b % 4 != 0) return false;
  return (A_KC ? (p.sak == 1 && vec4_ok<MA>(p.A, p.K, p.sam)) : (p.sam == 1 && vec4_ok<MA>(p.A, p.M, p.sak))) &&
         (B_KC ? (p.sbk == 1 && vec4_ok<MB>(p.B, p.K, p.sbn)) : (p.sbn == 1 && vec4_ok<MB>(p.B, p.N, p.sbk)));
}

template <int WM, int WN, bool A_KC, bool B_KC, typename TA, typename TB>
inline int launch(const Params& p, int kernel_id, hipStream_t s) {
  if (!usable<WM, WN, A_KC, B_KC, TA, TB>(p)) {
    if constexpr (std::is_same<TA, split3_t>::value || std::is_same<TB, split3_t>::value) return PK_ERR_ALIGN;   // the caller splits only what this kernel can read
    else return pk_f32mm::launch<WM, WN, A_KC, B_KC, TA, TB>(p, kernel_id, s);
  }
  if (p.M <= 0 || p.N <= 0) return PK_OK;
  dim3 grid((unsigned)pk_ceil_div(p.N, 32 * WN), (unsigned)pk_ceil_div(p.M, 32 * WM), (unsigned)p.splits);
  if (grid.y > 65535u || grid.z > 65535u) return PK_ERR_SHAPE;
  PK_LAUNCH_NOCHECK(kernel_id, s, (kernel<WM, WN, A_KC, B_KC, TA, TB>), grid, dim3(64 * WM * WN), 0, s, p);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

}  // namespace pk_x3mm
