// Grouped SwiGLU expert GEMMs (forward, input gradient, weight gradient).
//   bf16: v_mfma_f32_32x32x16_bf16 tiles, 128x128x64 block tile, 4 waves (2x2), fused
//         SwiGLU / SwiGLU-backward epilogues, permute fused into the A-operand loader,
//         ragged row blocks located on the device from starts[] (no host sync, empty
//         experts launch nothing).
//   f32 : tiled FMA kernel (simt_gemm.h) + elementwise SwiGLU kernels; exact fp32 arithmetic.
#include "pk_common.h"
#include "simt_gemm.h"
#include <initializer_list>

namespace {

// ===================================================================== bf16 MFMA path
namespace mf {

constexpr int BM = 128, BN = 128, BK = 64, THREADS = 256;
constexpr int LDS_LD = BK + 8;  // bf16 elements per LDS row: 144 B keeps 16-B alignment and
                                // spreads 16 consecutive rows over all banks for b128 reads
constexpr int NXCD = 8;

enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_SWIGLU_BWD = 2 };

__device__ __forceinline__ floatx16_t mfma32(bf16x8_t a, bf16x8_t b, floatx16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous range of
// logical tiles so that tiles sharing operands hit the same L2.  gridDim.x is a multiple of 8.
__device__ __forceinline__ int logical_block() {
  const int per = gridDim.x / NXCD;
  return (blockIdx.x % NXCD) * per + blockIdx.x / NXCD;
}

// Ragged-M tile lookup, done redundantly by every wave (no LDS, no barrier).
// Expert e owns ceil(cnt_e/BM) * n_tiles units, laid out [n-tile][m-tile] so that neighbouring
// units share the weight tile.  Returns false when `unit` is past the last real tile.
__device__ __forceinline__ bool locate_ragged_m(const int32_t* __restrict__ starts, int E,
                                                int n_tiles, int unit, int& e_out, int& mt_out,
                                                int& nt_out) {
  const int lane = threadIdx.x & 63;
  const int epl = (E + 63) >> 6;
  const int e_lo = lane * epl;
  const int e_hi = min(E, e_lo + epl);
  int mine = 0;
  for (int e = e_lo; e < e_hi; ++e) mine += ((starts[e + 1] - starts[e] + BM - 1) / BM) * n_tiles;
  int incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int v = __shfl_up(incl, off, PK_WAVE);
    if (lane >= off) incl += v;
  }
  const int excl = incl - mine;
  const bool owner = unit >= excl && unit < incl;
  const unsigned long long bal = __ballot(owner);
  if (bal == 0ull) return false;
  const int src = __ffsll((long long)bal) - 1;
  int fe = 0, fmt = 0, fnt = 0;
  if (owner) {
    int u = unit - excl;
    for (int e = e_lo; e < e_hi; ++e) {
      const int tiles = (starts[e + 1] - starts[e] + BM - 1) / BM;
      const int units = tiles * n_tiles;
      if (u < units) { fe = e; fnt = u / tiles; fmt = u % tiles; break; }
      u -= units;
    }
  }
  e_out = __shfl(fe, src, PK_WAVE);
  mt_out = __shfl(fmt, src, PK_WAVE);
  nt_out = __shfl(fnt, src, PK_WAVE);
  return true;
}

// ---- operand tile loaders.  LDS tiles are always [row (M or N index)][k], k contiguous.

// K-contiguous operand: each thread moves 4 chunks of 8 bf16 (16 B); rows r = (tid>>3) + 32*i.
struct KContigRegs { u32x4_t v[4]; };

__device__ __forceinline__ void store_kcontig(const KContigRegs& r, bf16_t* lds) {
  const int row = threadIdx.x >> 3, kc = threadIdx.x & 7;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    *reinterpret_cast<u32x4_t*>(lds + (row + 32 * i) * LDS_LD + kc * 8) = r.v[i];
}

// MN-contiguous operand (global layout [k][mn]): each thread loads an 8(k) x 4(mn) block as
// eight 8-byte pieces, transposes it in registers and writes four 16-byte LDS rows.
struct MnContigRegs { u32x2_t v[8]; };

__device__ __forceinline__ void store_mncontig(const MnContigRegs& r, bf16_t* lds) {
  const int ng = threadIdx.x & 31, kg = threadIdx.x >> 5;
  u32x4_t out[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    // k = 2c (low half) and k = 2c+1 (high half)
    out[0][c] = __builtin_amdgcn_perm(r.v[2 * c + 1][0], r.v[2 * c][0], 0x05040100u);
    out[1][c] = __builtin_amdgcn_perm(r.v[2 * c + 1][0], r.v[2 * c][0], 0x07060302u);
    out[2][c] = __builtin_amdgcn_perm(r.v[2 * c + 1][1], r.v[2 * c][1], 0x05040100u);
    out[3][c] = __builtin_amdgcn_perm(r.v[2 * c + 1][1], r.v[2 * c][1], 0x07060302u);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j)
    *reinterpret_cast<u32x4_t*>(lds + (ng * 4 + j) * LDS_LD + kg * 8) = out[j];
}

// One 64-deep k-tile of MFMAs for this wave's 64x64 sub-tile.
__device__ __forceinline__ void mma_tile(const bf16_t* As, const bf16_t* Bs, int wm, int wn,
                                         floatx16_t (&acc)[2][2]) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, kq = (lane >> 5) * 8;
#pragma unroll
  for (int ks = 0; ks < BK / 16; ++ks) {
    bf16x8_t a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
      a[i] = *reinterpret_cast<const bf16x8_t*>(As + (wm * 64 + i * 32 + r) * LDS_LD + ks * 16 + kq);
#pragma unroll
    for (int j = 0; j < 2; ++j)
      b[j] = *reinterpret_cast<const bf16x8_t*>(Bs + (wn * 64 + j * 32 + r) * LDS_LD + ks * 16 + kq);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(a[i], b[j], acc[i][j]);
  }
}

// Accumulator element v of a 32x32 tile held by `lane`: row = 8*(v/4) + 4*(lane/32) + v%4,
// column = lane%32.
__device__ __forceinline__ int acc_row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }

struct RaggedMParams {
  const bf16_t* A0;      // A operand of k-segment 0, row-major [rows, lda]
  const bf16_t* A1;      // k-segment 1 (nseg == 2)
  int64_t lda;
  const int32_t* row_map;  // optional gather of A rows: src = row_map[row] / map_div
  int32_t map_div;
  const bf16_t* B0;      // weights of k-segment 0 (EPI_SWIGLU: gate matrix)
  const bf16_t* B1;      // weights of k-segment 1 (EPI_SWIGLU: up matrix)
  int64_t ldb;
  int64_t strideB;       // elements between experts
  const int32_t* starts;
  int32_t E;
  int32_t Kseg;          // k extent of one segment (multiple of BK)
  int32_t nseg;
  int32_t n_tiles;       // column tiles per expert
  const bf16_t* Gin;     // EPI_SWIGLU_BWD inputs [A, ldc]
  const bf16_t* Uin;
  bf16_t* O0;            // PLAIN: C;  SWIGLU: g;  SWIGLU_BWD: d_g
  bf16_t* O1;            //            SWIGLU: u;  SWIGLU_BWD: d_u
  bf16_t* O2;            //            SWIGLU: h
  int64_t ldc;
};

// C[rows_e, N] = A[rows_e, K] . op(B[e])   with B K-contiguous ([N,K], "NT") or
// MN-contiguous ([K,N], "NN").
template <bool B_KCONTIG, int EPI>
__global__ __launch_bounds__(THREADS) void ragged_m_kernel(const RaggedMParams p) {
  __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDS_LD];

  int e, mt, nt;
  if (!locate_ragged_m(p.starts, p.E, p.n_tiles, logical_block(), e, mt, nt)) return;
  const int row0 = p.starts[e] + mt * BM;
  const int rows = min(BM, p.starts[e + 1] - row0);

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- A loader: rows beyond the expert's range are clamped (their results are not stored)
  const int ld_r = tid >> 3, ld_kc = tid & 7;
  int64_t a_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int r = ld_r + 32 * i;
    r = r < rows ? r : rows - 1;
    int64_t src = row0 + r;
    if (p.row_map) src = p.row_map[src] / p.map_div;
    a_off[i] = src * p.lda + ld_kc * 8;
  }
  // ---- B loader
  const int64_t b_base = (int64_t)e * p.strideB;
  int64_t b_off[4];   // K-contiguous: per-row offsets
  int b_mat[4];
  if (B_KCONTIG) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = ld_r + 32 * i;
      int n;
      if (EPI == EPI_SWIGLU) {  // LDS rows: 32 gate | 32 up | 32 gate | 32 up
        b_mat[i] = (r >> 5) & 1;
        n = nt * 64 + (r >> 6) * 32 + (r & 31);
      } else {
        b_mat[i] = 0;
        n = nt * BN + r;
      }
      b_off[i] = b_base + (int64_t)n * p.ldb + ld_kc * 8;
    }
  }
  const int tn_g = tid & 31, tk_g = tid >> 5;  // MN-contiguous: 8(k) x 4(n) block per thread

  floatx16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int kt_per_seg = p.Kseg / BK;
  const int nkt = kt_per_seg * p.nseg;

  KContigRegs a_regs, bk_regs;
  MnContigRegs bm_regs;

  auto issue_loads = [&](int kt) {
    const int seg = kt >= kt_per_seg ? 1 : 0;
    const int k0 = (kt - seg * kt_per_seg) * BK;
    const bf16_t* A = seg ? p.A1 : p.A0;
#pragma unroll
    for (int i = 0; i < 4; ++i) a_regs.v[i] = *reinterpret_cast<const u32x4_t*>(A + a_off[i] + k0);
    if (B_KCONTIG) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bf16_t* B = (EPI == EPI_SWIGLU) ? (b_mat[i] ? p.B1 : p.B0) : (seg ? p.B1 : p.B0);
        bk_regs.v[i] = *reinterpret_cast<const u32x4_t*>(B + b_off[i] + k0);
      }
    } else {
      const bf16_t* B = (seg ? p.B1 : p.B0) + b_base + (int64_t)(k0 + tk_g * 8) * p.ldb +
                        (int64_t)nt * BN + tn_g * 4;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk)
        bm_regs.v[kk] = *reinterpret_cast<const u32x2_t*>(B + (int64_t)kk * p.ldb);
    }
  };

  issue_loads(0);
  for (int kt = 0; kt < nkt; ++kt) {
    store_kcontig(a_regs, As);
    if (B_KCONTIG) store_kcontig(bk_regs, Bs); else store_mncontig(bm_regs, Bs);
    __syncthreads();
    if (kt + 1 < nkt) issue_loads(kt + 1);
    mma_tile(As, Bs, wm, wn, acc);
    __syncthreads();
  }

  // ---- epilogue
  const int col_in_tile = lane & 31;
  if (EPI == EPI_SWIGLU) {
    const int64_t col = (int64_t)nt * 64 + wn * 32 + col_in_tile;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = wm * 64 + i * 32 + acc_row(v, lane);
        if (r < rows) {
          const bf16_t gb = (bf16_t)acc[i][0][v], ub = (bf16_t)acc[i][1][v];
          const float g = (float)gb, u = (float)ub;
          const float h = (g / (1.f + __expf(-g))) * u;
          const int64_t o = (int64_t)(row0 + r) * p.ldc + col;
          p.O0[o] = gb;
          p.O1[o] = ub;
          p.O2[o] = (bf16_t)h;
        }
      }
  } else {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int64_t col = (int64_t)nt * BN + wn * 64 + j * 32 + col_in_tile;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int r = wm * 64 + i * 32 + acc_row(v, lane);
          if (r < rows) {
            const int64_t o = (int64_t)(row0 + r) * p.ldc + col;
            if (EPI == EPI_PLAIN) {
              p.O0[o] = (bf16_t)acc[i][j][v];
            } else {  // SwiGLU backward: acc = d_h
              const float dh = (float)(bf16_t)acc[i][j][v];
              const float g = (float)p.Gin[o], u = (float)p.Uin[o];
              const float s = 1.f / (1.f + __expf(-g));
              const float silu = g * s;
              p.O0[o] = (bf16_t)(dh * u * (s * (1.f + g * (1.f - s))));
              p.O1[o] = (bf16_t)(dh * silu);
            }
          }
        }
      }
  }
}

// ---- weight gradient: C[e][M,N] (+)= A[rows_e, M]^T . B[rows_e, N], ragged reduction dim.
struct WgradProblem {
  const bf16_t* A; int64_t lda; const int32_t* a_map;
  const bf16_t* B; int64_t ldb; const int32_t* b_map;
  bf16_t* C;
  int32_t M, N;
};
struct WgradParams {
  WgradProblem prob[3];
  const int32_t* starts;
  int32_t E;
  int32_t map_div;
  int32_t accumulate;
  int32_t tiles_per_expert;  // (M/BM)*(N/BN), identical for the three problems
};

__device__ __forceinline__ void wgrad_load(MnContigRegs& r, const bf16_t* base, int64_t ld,
                                           const int32_t* map, int map_div, int row_begin,
                                           int row_end, int k0, int col0) {
  const int cg = threadIdx.x & 31, kg = threadIdx.x >> 5;
#pragma unroll
  for (int kk = 0; kk < 8; ++kk) {
    const int row = row_begin + k0 + kg * 8 + kk;
    u32x2_t v = {0u, 0u};
    if (row < row_end) {
      int64_t src = row;
      if (map) src = map[row] / map_div;
      v = *reinterpret_cast<const u32x2_t*>(base + src * ld + col0 + cg * 4);
    }
    r.v[kk] = v;
  }
}

__global__ __launch_bounds__(THREADS) void wgrad_kernel(const WgradParams p) {
  __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDS_LD];

  const WgradProblem& q = p.prob[blockIdx.y];
  const int L = logical_block();
  const int e = L / p.tiles_per_expert;
  if (e >= p.E) return;
  const int t = L % p.tiles_per_expert;
  const int n_tiles = q.N / BN;
  const int mt = t / n_tiles, nt = t % n_tiles;
  const int row_begin = p.starts[e], row_end = p.starts[e + 1];
  const int nkt = (row_end - row_begin + BK - 1) / BK;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;

  floatx16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  MnContigRegs a_regs, b_regs;
  if (nkt > 0) {
    wgrad_load(a_regs, q.A, q.lda, q.a_map, p.map_div, row_begin, row_end, 0, mt * BM);
    wgrad_load(b_regs, q.B, q.ldb, q.b_map, p.map_div, row_begin, row_end, 0, nt * BN);
  }
  for (int kt = 0; kt < nkt; ++kt) {
    store_mncontig(a_regs, As);
    store_mncontig(b_regs, Bs);
    __syncthreads();
    if (kt + 1 < nkt) {
      wgrad_load(a_regs, q.A, q.lda, q.a_map, p.map_div, row_begin, row_end, (kt + 1) * BK, mt * BM);
      wgrad_load(b_regs, q.B, q.ldb, q.b_map, p.map_div, row_begin, row_end, (kt + 1) * BK, nt * BN);
    }
    mma_tile(As, Bs, wm, wn, acc);
    __syncthreads();
  }

  bf16_t* C = q.C + (int64_t)e * q.M * q.N;
  const int col_in_tile = lane & 31;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t col = (int64_t)nt * BN + wn * 64 + j * 32 + col_in_tile;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t r = (int64_t)mt * BM + wm * 64 + i * 32 + acc_row(v, lane);
        const int64_t o = r * q.N + col;
        float val = acc[i][j][v];
        if (p.accumulate) val += (float)C[o];
        C[o] = (bf16_t)val;
      }
    }
}

inline int round_up_xcd(int64_t n) { return (int)(pk_ceil_div(n, NXCD) * NXCD); }

template <bool B_KCONTIG, int EPI>
int launch_ragged_m(RaggedMParams p, int64_t A_rows, int kernel_id, hipStream_t s) {
  const int64_t max_units = (pk_ceil_div(A_rows, BM) + p.E) * p.n_tiles;
  if (max_units > 0x7ffffff0ll) return PK_ERR_SHAPE;
  PK_LAUNCH_NOCHECK(kernel_id, s, (ragged_m_kernel<B_KCONTIG, EPI>), dim3(round_up_xcd(max_units)),
                     dim3(THREADS), 0, s, p);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

}  // namespace mf

// ===================================================================== fp32 path helpers
template <typename T>
__global__ void swiglu_fwd_kernel(const T* __restrict__ g, const T* __restrict__ u,
                                  T* __restrict__ h, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const float gv = pk_to_float<T>(g[i]), uv = pk_to_float<T>(u[i]);
    h[i] = pk_from_float<T>((gv / (1.f + expf(-gv))) * uv);
  }
}
template <typename T>
__global__ void swiglu_bwd_kernel(const T* dh, const T* __restrict__ g,
                                  const T* __restrict__ u, T* __restrict__ dg, T* du,
                                  int64_t n) {  // dh may alias du
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const float d = pk_to_float<T>(dh[i]), gv = pk_to_float<T>(g[i]), uv = pk_to_float<T>(u[i]);
    const float s = 1.f / (1.f + expf(-gv));
    dg[i] = pk_from_float<T>(d * uv * (s * (1.f + gv * (1.f - s))));
    du[i] = pk_from_float<T>(d * (gv * s));
  }
}

// Generic (any shape) ragged GEMMs on the FMA kernel.  T = element type of every operand.
template <typename T>
int simt_ragged_m(const void* A, int64_t lda, const int32_t* row_map, int64_t map_div,
                  const void* B, int64_t sbk, int64_t sbn, int64_t strideB, void* C, int64_t ldc,
                  const int32_t* starts, int64_t rows, int64_t N, int64_t K, int64_t E,
                  int accumulate, hipStream_t s) {
  pk_simt::Params p = {};
  p.A = A; p.B = B; p.C = C; p.starts = starts; p.a_map = row_map; p.map_div = (int32_t)map_div;
  p.ragged = pk_simt::RAGGED_M; p.G = (int32_t)E; p.accumulate = accumulate;
  p.M = 0; p.N = N; p.K = K;
  p.sam = lda; p.sak = 1; p.sbk = sbk; p.sbn = sbn; p.scm = ldc; p.scn = 1;
  p.gA = 0; p.gB = strideB; p.gC = 0;
  p.total_m_tiles = (int32_t)(pk_ceil_div(rows, pk_simt::TM) + E);
  return pk_simt::launch<T, T, T>(p, s);
}
template <typename T>
int simt_ragged_k(const void* A, int64_t lda, const int32_t* a_map, const void* B, int64_t ldb,
                  const int32_t* b_map, int64_t map_div, void* C, const int32_t* starts, int64_t M,
                  int64_t N, int64_t E, int accumulate, hipStream_t s) {
  pk_simt::Params p = {};
  p.A = A; p.B = B; p.C = C; p.starts = starts; p.a_map = a_map; p.b_map = b_map;
  p.map_div = (int32_t)map_div;
  p.ragged = pk_simt::RAGGED_K; p.G = (int32_t)E; p.accumulate = accumulate;
  p.M = M; p.N = N; p.K = 0;
  p.sam = 1; p.sak = lda;   // A(m,k) = A[k*lda + m]
  p.sbk = ldb; p.sbn = 1;   // B(k,n) = B[k*ldb + n]
  p.scm = N; p.scn = 1;
  p.gA = 0; p.gB = 0; p.gC = M * N;
  return pk_simt::launch<T, T, T>(p, s);
}

bool mfma_shape_ok(int64_t H, int64_t I) { return H % 128 == 0 && I % 128 == 0; }

bool all_aligned16(std::initializer_list<const void*> ptrs) {
  for (const void* p : ptrs)
    if (p && !pk_aligned16(p)) return false;
  return true;
}

int check_common(int64_t A, int64_t H, int64_t I, int64_t E, int dtype) {
  if (A < 0 || H <= 0 || I <= 0 || E <= 0 || !pk_dtype_ok(dtype)) return PK_ERR_ARG;
  if (E > PK_MAX_EXPERTS) return PK_ERR_SHAPE;
  if (A > 0x7fffffffll || E * I * H > 0x7fffffffffll) return PK_ERR_SHAPE;
  return PK_OK;
}

template <typename T>
int fwd_simt(const void* x, const int32_t* row_map, int64_t div, const void* w1, const void* w2,
             const void* w3, const int32_t* starts, void* g, void* u, void* h, void* y, int64_t A,
             int64_t H, int64_t I, int64_t E, hipStream_t s) {
  int rc = simt_ragged_m<T>(x, H, row_map, div, w1, 1, H, I * H, g, I, starts, A, I, H, E, 0, s);
  if (rc) return rc;
  rc = simt_ragged_m<T>(x, H, row_map, div, w3, 1, H, I * H, u, I, starts, A, I, H, E, 0, s);
  if (rc) return rc;
  const int64_t n = A * I;
  PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_ELEMENTWISE, s, (swiglu_fwd_kernel<T>), dim3((unsigned)pk_ceil_div(n, 256)), dim3(256), 0, s,
                     (const T*)g, (const T*)u, (T*)h, n);
  PK_RETURN_IF_LAUNCH_FAILED();
  return simt_ragged_m<T>(h, I, nullptr, 1, w2, 1, I, H * I, y, H, starts, A, H, I, E, 0, s);
}

template <typename T>
int dgrad_simt(const void* dy, const void* w1, const void* w2, const void* w3, const void* g,
               const void* u, const int32_t* starts, void* dg, void* du, void* dx, int64_t A,
               int64_t H, int64_t I, int64_t E, hipStream_t s) {
  // d_h = d_y . w2[e]  (w2[e] is [H, I]: B(k=h, n=i) = w2[h*I + i]); staged in d_u's buffer
  int rc = simt_ragged_m<T>(dy, H, nullptr, 1, w2, I, 1, H * I, du, I, starts, A, I, H, E, 0, s);
  if (rc) return rc;
  const int64_t n = A * I;
  PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_ELEMENTWISE, s, (swiglu_bwd_kernel<T>), dim3((unsigned)pk_ceil_div(n, 256)), dim3(256), 0, s,
                     (const T*)du, (const T*)g, (const T*)u, (T*)dg, (T*)du, n);
  PK_RETURN_IF_LAUNCH_FAILED();
  // d_x = d_g . w1[e] + d_u . w3[e]   (w[e] is [I, H]: B(k=i, n=h) = w[i*H + h])
  rc = simt_ragged_m<T>(dg, I, nullptr, 1, w1, H, 1, I * H, dx, H, starts, A, H, I, E, 0, s);
  if (rc) return rc;
  return simt_ragged_m<T>(du, I, nullptr, 1, w3, H, 1, I * H, dx, H, starts, A, H, I, E, 1, s);
}

template <typename T>
int wgrad_simt(const void* dy, const void* h, const void* dg, const void* du, const void* x,
               const int32_t* row_map, int64_t div, const int32_t* starts, void* dw1, void* dw2,
               void* dw3, int acc, int64_t H, int64_t I, int64_t E, hipStream_t s) {
  int rc = PK_OK;
  if (dw2) rc = simt_ragged_k<T>(dy, H, nullptr, h, I, nullptr, 1, dw2, starts, H, I, E, acc, s);
  if (rc) return rc;
  if (dw1) rc = simt_ragged_k<T>(dg, I, nullptr, x, H, row_map, div, dw1, starts, I, H, E, acc, s);
  if (rc) return rc;
  if (dw3) rc = simt_ragged_k<T>(du, I, nullptr, x, H, row_map, div, dw3, starts, I, H, E, acc, s);
  return rc;
}

}  // namespace

extern "C" {

int pk_grouped_swiglu_fwd(const void* x_rows, const int32_t* row_map, int64_t row_map_div,
                          const void* w1, const void* w2, const void* w3,
                          const int32_t* starts, void* g, void* u, void* h, void* y,
                          int64_t A, int64_t H, int64_t I, int64_t E, int dtype,
                          pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  if (A == 0) return PK_OK;
  if (!x_rows || !w1 || !w2 || !w3 || !starts || !g || !u || !h || !y) return PK_ERR_ARG;
  if (row_map && row_map_div <= 0) return PK_ERR_ARG;
  if (!row_map) row_map_div = 1;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PK_F32)
    return fwd_simt<float>(x_rows, row_map, row_map_div, w1, w2, w3, starts, g, u, h, y, A, H, I, E, s);
  if (!mfma_shape_ok(H, I) || !all_aligned16({x_rows, w1, w2, w3, g, u, h, y}))
    return fwd_simt<bf16_t>(x_rows, row_map, row_map_div, w1, w2, w3, starts, g, u, h, y, A, H, I, E, s);

  mf::RaggedMParams p = {};
  p.A0 = (const bf16_t*)x_rows; p.A1 = nullptr; p.lda = H;
  p.row_map = row_map; p.map_div = (int32_t)row_map_div;
  p.B0 = (const bf16_t*)w1; p.B1 = (const bf16_t*)w3; p.ldb = H; p.strideB = I * H;
  p.starts = starts; p.E = (int32_t)E; p.Kseg = (int32_t)H; p.nseg = 1;
  p.n_tiles = (int32_t)(I / 64);
  p.O0 = (bf16_t*)g; p.O1 = (bf16_t*)u; p.O2 = (bf16_t*)h; p.ldc = I;
  rc = mf::launch_ragged_m<true, mf::EPI_SWIGLU>(p, A, pk_timing::K_SWIGLU_GATE_UP, s);
  if (rc) return rc;

  mf::RaggedMParams q = {};
  q.A0 = (const bf16_t*)h; q.lda = I;
  q.B0 = (const bf16_t*)w2; q.B1 = nullptr; q.ldb = I; q.strideB = H * I;
  q.starts = starts; q.E = (int32_t)E; q.Kseg = (int32_t)I; q.nseg = 1;
  q.n_tiles = (int32_t)(H / mf::BN);
  q.O0 = (bf16_t*)y; q.ldc = H;
  return mf::launch_ragged_m<true, mf::EPI_PLAIN>(q, A, pk_timing::K_SWIGLU_DOWN, s);
}

int pk_grouped_swiglu_dgrad(const void* d_y, const void* w1, const void* w2, const void* w3,
                            const void* g, const void* u, const int32_t* starts, void* d_g,
                            void* d_u, void* d_x_sorted, int64_t A, int64_t H, int64_t I,
                            int64_t E, int dtype, pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  if (A == 0) return PK_OK;
  if (!d_y || !w1 || !w2 || !w3 || !g || !u || !starts || !d_g || !d_u || !d_x_sorted)
    return PK_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PK_F32)
    return dgrad_simt<float>(d_y, w1, w2, w3, g, u, starts, d_g, d_u, d_x_sorted, A, H, I, E, s);
  if (!mfma_shape_ok(H, I) || !all_aligned16({d_y, w1, w2, w3, g, u, d_g, d_u, d_x_sorted}))
    return dgrad_simt<bf16_t>(d_y, w1, w2, w3, g, u, starts, d_g, d_u, d_x_sorted, A, H, I, E, s);

  // d_h = d_y . w2[e]  ->  (d_g, d_u) in the epilogue
  mf::RaggedMParams p = {};
  p.A0 = (const bf16_t*)d_y; p.lda = H;
  p.B0 = (const bf16_t*)w2; p.ldb = I; p.strideB = H * I;
  p.starts = starts; p.E = (int32_t)E; p.Kseg = (int32_t)H; p.nseg = 1;
  p.n_tiles = (int32_t)(I / mf::BN);
  p.Gin = (const bf16_t*)g; p.Uin = (const bf16_t*)u;
  p.O0 = (bf16_t*)d_g; p.O1 = (bf16_t*)d_u; p.ldc = I;
  rc = mf::launch_ragged_m<false, mf::EPI_SWIGLU_BWD>(p, A, pk_timing::K_SWIGLU_DGRAD_DH, s);
  if (rc) return rc;

  // d_x = [d_g | d_u] . [w1[e] ; w3[e]]
  mf::RaggedMParams q = {};
  q.A0 = (const bf16_t*)d_g; q.A1 = (const bf16_t*)d_u; q.lda = I;
  q.B0 = (const bf16_t*)w1; q.B1 = (const bf16_t*)w3; q.ldb = H; q.strideB = I * H;
  q.starts = starts; q.E = (int32_t)E; q.Kseg = (int32_t)I; q.nseg = 2;
  q.n_tiles = (int32_t)(H / mf::BN);
  q.O0 = (bf16_t*)d_x_sorted; q.ldc = H;
  return mf::launch_ragged_m<false, mf::EPI_PLAIN>(q, A, pk_timing::K_SWIGLU_DGRAD_DX, s);
}

int pk_grouped_swiglu_wgrad(const void* d_y, const void* h, const void* d_g, const void* d_u,
                            const void* x_rows, const int32_t* row_map, int64_t row_map_div,
                            const int32_t* starts, void* d_w1, void* d_w2, void* d_w3,
                            int accumulate, int64_t A, int64_t H, int64_t I, int64_t E,
                            int dtype, pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  if (!starts) return PK_ERR_ARG;
  if (d_w2 && A > 0 && (!d_y || !h)) return PK_ERR_ARG;
  if (d_w1 && A > 0 && (!d_g || !x_rows)) return PK_ERR_ARG;
  if (d_w3 && A > 0 && (!d_u || !x_rows)) return PK_ERR_ARG;
  if (row_map && row_map_div <= 0) return PK_ERR_ARG;
  if (!row_map) row_map_div = 1;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PK_F32)
    return wgrad_simt<float>(d_y, h, d_g, d_u, x_rows, row_map, row_map_div, starts, d_w1, d_w2, d_w3, accumulate, H, I, E, s);
  if (!mfma_shape_ok(H, I) || !all_aligned16({d_y, h, d_g, d_u, x_rows, d_w1, d_w2, d_w3}))
    return wgrad_simt<bf16_t>(d_y, h, d_g, d_u, x_rows, row_map, row_map_div, starts, d_w1, d_w2, d_w3, accumulate, H, I, E, s);

  mf::WgradParams p = {};
  int n = 0;
  if (d_w2) {
    mf::WgradProblem& q = p.prob[n++];
    q.A = (const bf16_t*)d_y; q.lda = H; q.a_map = nullptr;
    q.B = (const bf16_t*)h; q.ldb = I; q.b_map = nullptr;
    q.C = (bf16_t*)d_w2; q.M = (int32_t)H; q.N = (int32_t)I;
  }
  if (d_w1) {
    mf::WgradProblem& q = p.prob[n++];
    q.A = (const bf16_t*)d_g; q.lda = I; q.a_map = nullptr;
    q.B = (const bf16_t*)x_rows; q.ldb = H; q.b_map = row_map;
    q.C = (bf16_t*)d_w1; q.M = (int32_t)I; q.N = (int32_t)H;
  }
  if (d_w3) {
    mf::WgradProblem& q = p.prob[n++];
    q.A = (const bf16_t*)d_u; q.lda = I; q.a_map = nullptr;
    q.B = (const bf16_t*)x_rows; q.ldb = H; q.b_map = row_map;
    q.C = (bf16_t*)d_w3; q.M = (int32_t)I; q.N = (int32_t)H;
  }
  if (n == 0) return PK_OK;
  p.starts = starts; p.E = (int32_t)E; p.map_div = (int32_t)row_map_div;
  p.accumulate = accumulate ? 1 : 0;
  p.tiles_per_expert = (int32_t)((H / mf::BM) * (I / mf::BN));
  const int64_t blocks = (int64_t)p.tiles_per_expert * E;
  if (blocks > 0x7ffffff0ll) return PK_ERR_SHAPE;
  PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_WGRAD, s, mf::wgrad_kernel, dim3(mf::round_up_xcd(blocks), n), dim3(mf::THREADS), 0, s, p);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

}  // extern "C"
