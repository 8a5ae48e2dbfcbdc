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

constexpr int NXCD = 8;

enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_SWIGLU_BWD = 2 };

typedef short shortx4_t __attribute__((ext_vector_type(4)));
// Read-only tables (row offsets, row maps) addressed wave-uniformly: going through the constant
// address space makes these scalar loads (lgkmcnt), which leaves vmcnt to the LDS ring.
typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
__device__ __forceinline__ const_i32_ptr as_const(const int32_t* p) { return (const_i32_ptr)(uintptr_t)p; }
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// 16 zero bytes: the source of operand rows past the end of a ragged reduction range.
__device__ __attribute__((aligned(16))) const uint32_t g_zero16[4] = {0u, 0u, 0u, 0u};

// Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous range of
// logical tiles so that tiles sharing operands hit the same L2.  gridDim.x is a multiple of 8.
__device__ __forceinline__ int logical_block() {
  const int per = gridDim.x / NXCD;
  return (blockIdx.x % NXCD) * per + blockIdx.x / NXCD;
}

// Direct global->LDS load of 16 bytes per lane: lane l's bytes land at lds_base + 16*l.
// Issued from inline asm so that the compiler does not serialise later LDS reads behind it;
// completion is tracked by hand with vmcnt (wait_dma) followed by a workgroup barrier.
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off"
               :: "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(gptr)
               : "memory");
}
template <int N>
__device__ __forceinline__ void wait_dma() {
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}
__device__ __forceinline__ void block_barrier() {
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)(lds_ptr_t)p;
}

// ---------------------------------------------------------------------------------------------
// LDS tile layouts (BK = 64 or 32 deep).  16-byte chunks are XOR-swizzled so that the fragment
// reads below touch every bank once.
//
// KC tile: [ROWS rows of the M or N index][BK k], k contiguous (2*BK bytes per row, BK/8 chunks).
//          chunk c of row r sits at position c ^ swz(r): (r >> 1) & 7 for BK 64, (r >> 2) & 3 for BK 32.
// MN tile: [BK k][COLS of the M or N index], the M/N index contiguous (COLS/8 chunks per row).
//          chunk c of row k sits at position c ^ ((k & 3) << 2).
//
// A wave-level dma16 fills 64 consecutive 16-byte slots; which global chunk a lane fetches is
// chosen so that the swizzled layout comes out.

// Global element offset (within the operand) of the chunk that lane `lane` of load `G`
// (G-th group of 64 slots of the tile) must fetch, for a KC tile: returns row and k offset.
template <int BK>
__device__ __forceinline__ int kc_swz(int row) { return BK == 64 ? ((row >> 1) & 7) : ((row >> 2) & 3); }
template <int BK>
__device__ __forceinline__ void kc_slot(int G, int lane, int& row, int& kofs) {
  constexpr int CPR = BK / 8;
  const int slot = G * 64 + lane;
  row = slot / CPR;
  kofs = ((slot % CPR) ^ kc_swz<BK>(row)) * 8;
}
template <int COLS>
__device__ __forceinline__ void mn_slot(int G, int lane, int& krow, int& cofs) {
  constexpr int CPR = COLS / 8;
  const int slot = G * 64 + lane;
  krow = slot / CPR;
  cofs = ((slot % CPR) ^ ((krow & 3) << 2)) * 8;
}

// MFMA operand fragment (8 bf16 per lane: row lane%32, k = 16*ks + 8*(lane/32) + 0..7).
template <int BK>
__device__ __forceinline__ bf16x8_t frag_kc(const char* tile, int row0, int ks, int lane) {
  const int r = row0 + (lane & 31);
  const int c = 2 * ks + (lane >> 5);
  return *reinterpret_cast<const bf16x8_t*>(tile + r * (2 * BK) + ((c ^ kc_swz<BK>(r)) << 4));
}
// Same fragment out of an MN tile through the transposing LDS read: within 16 lanes, lane i
// points at 4 consecutive columns of k-row i/4 and receives 4 consecutive k of column i.
template <int COLS>
__device__ __forceinline__ bf16x8_t frag_mn(const char* tile, int col0, int ks, int lane) {
  const int i = lane & 15;
  const int krow = ks * 16 + 8 * (lane >> 5) + (i >> 2);
  const int col = col0 + 16 * ((lane >> 4) & 1) + 4 * (i & 3);
  const int pos = (col >> 3) ^ ((i >> 2) << 2);
  const char* p = tile + krow * (COLS * 2) + pos * 16 + (col & 7) * 2;
  const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4_t*)(p));
  const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4_t*)(p + 4 * COLS * 2));
  typedef short shortx8_t __attribute__((ext_vector_type(8)));
  shortx8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8_t, v);
}

// Fragments of one 16-deep k-step for a wave tile of TM x TN MFMA tiles.
template <int TM, int TN>
struct Frags {
  bf16x8_t a[TM];
  bf16x8_t b[TN];
};
template <int BK, int TM, int TN, bool A_KC, bool B_KC, int ACOLS, int BCOLS>
__device__ __forceinline__ void load_frags(Frags<TM, TN>& f, const char* At, const char* Bt,
                                           int wrow0, int wcol0, int ks, int lane) {
#pragma unroll
  for (int i = 0; i < TM; ++i)
    f.a[i] = A_KC ? frag_kc<BK>(At, wrow0 + 32 * i, ks, lane) : frag_mn<ACOLS>(At, wrow0 + 32 * i, ks, lane);
#pragma unroll
  for (int j = 0; j < TN; ++j)
    f.b[j] = B_KC ? frag_kc<BK>(Bt, wcol0 + 32 * j, ks, lane) : frag_mn<BCOLS>(Bt, wcol0 + 32 * j, ks, lane);
}

// One 64-deep k-tile of MFMAs, software pipelined: the fragments of k-step s+1 are requested
// from LDS before / while the MFMAs of k-step s are issued, so the ~90-cycle LDS latency is
// covered.  LEAN keeps a single copy of the A fragments and refills each one right after its
// last use (fewer registers, for the 128x128 wave tiles).
// The operands are passed swapped (B first) so that each lane's accumulator holds 4
// CONSECUTIVE output columns of ONE output row:
//   acc[i][j][v] = C[row = 32*i + lane%32][col = 32*j + 8*(v/4) + 4*(lane/32) + v%4]
template <int BK, int TM, int TN, bool A_KC, bool B_KC, int ACOLS, int BCOLS, bool LEAN>
__device__ __forceinline__ void mma_tile(const char* At, const char* Bt, int wrow0, int wcol0,
                                         floatx16_t (&acc)[TM][TN]) {
  const int lane = threadIdx.x & 63;
  constexpr int KS = BK / 16;
  if (LEAN) {
    bf16x8_t a[TM], b[2][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
      a[i] = A_KC ? frag_kc<BK>(At, wrow0 + 32 * i, 0, lane) : frag_mn<ACOLS>(At, wrow0 + 32 * i, 0, lane);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      b[0][j] = B_KC ? frag_kc<BK>(Bt, wcol0 + 32 * j, 0, lane) : frag_mn<BCOLS>(Bt, wcol0 + 32 * j, 0, lane);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
          b[(ks + 1) & 1][j] = B_KC ? frag_kc<BK>(Bt, wcol0 + 32 * j, ks + 1, lane)
                                    : frag_mn<BCOLS>(Bt, wcol0 + 32 * j, ks + 1, lane);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[ks & 1][j], a[i], acc[i][j], 0, 0, 0);
        if (ks + 1 < KS)
          a[i] = A_KC ? frag_kc<BK>(At, wrow0 + 32 * i, ks + 1, lane) : frag_mn<ACOLS>(At, wrow0 + 32 * i, ks + 1, lane);
      }
    }
  } else {
    Frags<TM, TN> f[2];
    load_frags<BK, TM, TN, A_KC, B_KC, ACOLS, BCOLS>(f[0], At, Bt, wrow0, wcol0, 0, lane);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS)
        load_frags<BK, TM, TN, A_KC, B_KC, ACOLS, BCOLS>(f[(ks + 1) & 1], At, Bt, wrow0, wcol0, ks + 1, lane);
      // keep the LDS reads of the next k-step ahead of this k-step's MFMAs: without the fence
      // the scheduler sinks them behind the MFMAs to reuse the fragment registers, which
      // exposes the LDS latency once per k-step
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[ks & 1].b[j], f[ks & 1].a[i], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

__device__ __forceinline__ u32x2_t pack4(float a, float b, float c, float d) {
  bf16x4_t v;
  v[0] = (bf16_t)a; v[1] = (bf16_t)b; v[2] = (bf16_t)c; v[3] = (bf16_t)d;
  return __builtin_bit_cast(u32x2_t, v);
}
__device__ __forceinline__ void unpack4(u32x2_t p, float (&f)[4]) {
  bf16x4_t v = __builtin_bit_cast(bf16x4_t, p);
#pragma unroll
  for (int i = 0; i < 4; ++i) f[i] = (float)v[i];
}

// Wave-private staging of a [ROWS x COLS] bf16 tile through LDS so that global stores are 16
// bytes per lane and row-contiguous.  Row stride is COLS*2 + 16 bytes (keeps 16-B alignment).
template <int COLS>
struct Stage {
  static constexpr int LD = COLS * 2 + 16;
  // a lane deposits 4 consecutive columns of one row
  __device__ static __forceinline__ void put(char* buf, int row, int col, u32x2_t v) {
    *reinterpret_cast<u32x2_t*>(buf + row * LD + col * 2) = v;
  }
  // copy rows [0, nrows) x COLS of the staged tile to global memory (row stride ldc elements);
  // ACC adds the tile to what is already there (fp32 add, one rounding of the sum).
  template <int ROWS, bool ACC = false>
  __device__ static __forceinline__ void flush(const char* buf, bf16_t* dst, int64_t ldc, int nrows) {
    constexpr int LANES_PER_ROW = COLS / 8;        // 16 bytes per lane
    constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
    const int lane = threadIdx.x & 63;
    const int lr = lane / LANES_PER_ROW, lc = (lane % LANES_PER_ROW) * 8;
#pragma unroll 4
    for (int r0 = 0; r0 < ROWS; r0 += ROWS_PER_PASS) {
      const int r = r0 + lr;
      if (r < nrows) {
        u32x4_t v = *reinterpret_cast<const u32x4_t*>(buf + r * LD + lc * 2);
        u32x4_t* g = reinterpret_cast<u32x4_t*>(dst + (int64_t)r * ldc + lc);
        if (ACC) {
          const bf16x8_t a = __builtin_bit_cast(bf16x8_t, v);
          const bf16x8_t o = __builtin_bit_cast(bf16x8_t, *g);
          bf16x8_t sum;
#pragma unroll
          for (int t = 0; t < 8; ++t) sum[t] = (bf16_t)((float)a[t] + (float)o[t]);
          v = __builtin_bit_cast(u32x4_t, sum);
        }
        *g = v;
      }
    }
  }
};
// LDS traffic of one wave is ordered by the hardware; this only stops the compiler from
// moving the staged reads above the writes.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Ragged-M tile lookup, done redundantly by every wave (no LDS, no barrier).
// Expert e owns ceil(cnt_e/BM) * n_tiles units, laid out [n-tile][m-tile] so that neighbouring
// units share the weight tile.  Returns false when `unit` is past the last real tile.
template <int BM>
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
#ifdef PK_GEMM_DEBUG
  int32_t debug;         // 1: skip MFMAs, 2: skip loads, 4: skip stores
#endif
};

// C[rows_e, N] = A[rows_e, K] . op(B[e]) with B K-contiguous ([N,K]) or MN-contiguous ([K,N]).
// Block tile BM x BN, WMW x WNW waves, NS-stage LDS ring filled by direct-to-LDS loads.
// EPI_SWIGLU: the BN tile rows are [32 gate | 32 up | 32 gate | 32 up ...] of BN/2 output
// columns, so that a lane holds the gate and the up value of the same element.
template <int BM, int BN, int BK, int WMW, int WNW, int NS, int OCC, bool B_KC, int EPI>
__global__ __launch_bounds__(64 * WMW * WNW, OCC * WMW * WNW / 4) void ragged_m_kernel(const RaggedMParams p) {
  constexpr int NTHREADS = 64 * WMW * WNW;
  constexpr int WTM = BM / WMW, WTN = BN / WNW;          // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * BK * 2, STAGE = (BM + BN) * BK * 2;
  constexpr int LA = A_BYTES / (NTHREADS * 16), LB = (STAGE - A_BYTES) / (NTHREADS * 16);   // dma16 per thread per tile
  static_assert(LA >= 1 && LB >= 1 && TM >= 1 && TN >= 1, "tile too small for the wave grid");
  static_assert(EPI != EPI_SWIGLU || (WTN % 64 == 0), "gate/up pairs must stay inside a wave");
  // output columns a wave writes per output tensor, and its staging buffer
  constexpr int OUT_COLS = (EPI == EPI_SWIGLU) ? WTN / 2 : WTN;
  using St = Stage<OUT_COLS>;
  constexpr int STAGING = WTM * St::LD * (WMW * WNW);
  constexpr int SMEM = STAGING > NS * STAGE ? STAGING : NS * STAGE;
  __shared__ __attribute__((aligned(1024))) char smem[SMEM];

  int e, mt, nt;
  if (!locate_ragged_m<BM>(p.starts, p.E, p.n_tiles, logical_block(), e, mt, nt)) return;
  const int row0 = p.starts[e] + mt * BM;
  const int rows = min(BM, p.starts[e + 1] - row0);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave / WNW, wn = wave % WNW;
  const bool wave_has_rows = wm * WTM < rows;   // waves whose row slice is empty skip the math

  // ---- per-thread source pointers of the dma16 loads (k offset 0 of segment 0)
  int64_t a_off[LA];
#pragma unroll
  for (int i = 0; i < LA; ++i) {
    int r, kofs;
    kc_slot<BK>(wave * LA + i, lane, r, kofs);
    r = r < rows ? r : rows - 1;     // clamp: rows past the expert's range are never stored
    int64_t src = row0 + r;
    if (p.row_map) src = p.row_map[src] / p.map_div;
    a_off[i] = src * p.lda + kofs;
  }
  int64_t b_off[LB];
  int b_mat[LB];
  const int64_t b_base = (int64_t)e * p.strideB;
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    b_mat[i] = 0;
    if (B_KC) {
      int r, kofs;
      kc_slot<BK>(wave * LB + i, lane, r, kofs);
      int n;
      if (EPI == EPI_SWIGLU) {
        b_mat[i] = (r >> 5) & 1;
        n = nt * (BN / 2) + (r >> 6) * 32 + (r & 31);
      } else {
        n = nt * BN + r;
      }
      b_off[i] = b_base + (int64_t)n * p.ldb + kofs;
    } else {
      int krow, cofs;
      mn_slot<BN>(wave * LB + i, lane, krow, cofs);
      b_off[i] = b_base + (int64_t)krow * p.ldb + (int64_t)nt * BN + cofs;
    }
  }

  const int kt_per_seg = p.Kseg / BK;
  const int nkt = kt_per_seg * p.nseg;

  auto issue = [&](int kt, int stage) {
    char* st = smem + stage * STAGE;
    const int seg = kt >= kt_per_seg ? 1 : 0;
    const int k0 = (kt - seg * kt_per_seg) * BK;
    const bf16_t* A = seg ? p.A1 : p.A0;
    const uint32_t a_lds = lds_addr(st) + (wave * LA) * 1024;
    const uint32_t b_lds = lds_addr(st + A_BYTES) + (wave * LB) * 1024;
#pragma unroll
    for (int i = 0; i < LA; ++i) dma16(A + a_off[i] + k0, a_lds + i * 1024);
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      const bf16_t* B = (EPI == EPI_SWIGLU) ? (b_mat[i] ? p.B1 : p.B0) : (seg ? p.B1 : p.B0);
      dma16(B + b_off[i] + (B_KC ? (int64_t)k0 : (int64_t)k0 * p.ldb), b_lds + i * 1024);
    }
  };

  floatx16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

#pragma unroll
  for (int s = 0; s < NS - 1; ++s)
    if (s < nkt) issue(s, s);
  int cur = 0;            // stage of tile kt
  int nxt = NS - 1;       // stage of tile kt + NS - 1
  for (int kt = 0; kt < nkt; ++kt) {
    // tile kt has landed once at most the NS-2 younger tiles are still in flight
    if (kt + NS - 2 < nkt) wait_dma<(NS - 2) * (LA + LB)>(); else wait_dma<0>();
    block_barrier();   // everyone's part of tile kt is in LDS; everyone is done reading tile kt-1
#ifdef PK_GEMM_DEBUG
    if (!(p.debug & 2))
#endif
    if (kt + NS - 1 < nkt) issue(kt + NS - 1, nxt);
    const char* st = smem + cur * STAGE;
#ifdef PK_GEMM_DEBUG
    if (!(p.debug & 1))
#endif
    if (wave_has_rows)
      mma_tile<BK, TM, TN, true, B_KC, BM, BN, false>(st, st + A_BYTES, wm * WTM, wn * WTN, acc);
    cur = cur + 1 == NS ? 0 : cur + 1;
    nxt = nxt + 1 == NS ? 0 : nxt + 1;
  }
#ifdef PK_GEMM_DEBUG
  if (p.debug & 4) { if (acc[0][0][0] != 12345.678f) return; }
#endif

  // ---- epilogue: stage each wave's tile through LDS, then 16-byte row-contiguous stores
  block_barrier();   // the ring is free: every wave has finished its last fragment reads
  if (!wave_has_rows) return;
  char* sbuf = smem + wave * (WTM * St::LD);
  const int lrow = lane & 31, lq = 4 * (lane >> 5);
  const int wrows = min(WTM, rows - wm * WTM);          // valid rows of this wave's slice
  const int64_t grow0 = (int64_t)(row0 + wm * WTM) * p.ldc;
  if (EPI == EPI_SWIGLU) {
    const int64_t gcol0 = (int64_t)nt * (BN / 2) + wn * OUT_COLS;
#pragma unroll
    for (int which = 0; which < 3; ++which) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; j += 2)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const u32x2_t gp = pack4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
            const u32x2_t up = pack4(acc[i][j + 1][4 * q], acc[i][j + 1][4 * q + 1], acc[i][j + 1][4 * q + 2], acc[i][j + 1][4 * q + 3]);
            u32x2_t v = which == 0 ? gp : up;
            if (which == 2) {
              float g[4], u[4];
              unpack4(gp, g);
              unpack4(up, u);
              v = pack4((g[0] / (1.f + __expf(-g[0]))) * u[0], (g[1] / (1.f + __expf(-g[1]))) * u[1],
                        (g[2] / (1.f + __expf(-g[2]))) * u[2], (g[3] / (1.f + __expf(-g[3]))) * u[3]);
            }
            St::put(sbuf, 32 * i + lrow, 16 * j + 8 * q + lq, v);
          }
      wave_lds_fence();
      bf16_t* dst = (which == 0 ? p.O0 : which == 1 ? p.O1 : p.O2) + grow0 + gcol0;
      St::template flush<WTM>(sbuf, dst, p.ldc, wrows);
      wave_lds_fence();
    }
  } else {
    const int64_t gcol0 = (int64_t)nt * BN + wn * WTN;
#pragma unroll
    for (int which = 0; which < (EPI == EPI_PLAIN ? 1 : 2); ++which) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int r = 32 * i + lrow;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int c = 32 * j + 8 * q + lq;
            u32x2_t v = pack4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
            if (EPI == EPI_SWIGLU_BWD) {   // acc = d_h (rounded to bf16 like the reference's bmm output)
              float dh[4], g[4], u[4], o[4];
              unpack4(v, dh);
              const int rr = r < wrows ? r : wrows - 1;
              const int64_t off = grow0 + (int64_t)rr * p.ldc + gcol0 + c;
              unpack4(*reinterpret_cast<const u32x2_t*>(p.Gin + off), g);
              unpack4(*reinterpret_cast<const u32x2_t*>(p.Uin + off), u);
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                const float sg = 1.f / (1.f + __expf(-g[t]));
                o[t] = which == 0 ? dh[t] * u[t] * (sg * (1.f + g[t] * (1.f - sg))) : dh[t] * (g[t] * sg);
              }
              v = pack4(o[0], o[1], o[2], o[3]);
            }
            St::put(sbuf, r, c, v);
          }
      }
      wave_lds_fence();
      bf16_t* dst = (which == 0 ? p.O0 : p.O1) + grow0 + gcol0;
      St::template flush<WTM>(sbuf, dst, p.ldc, wrows);
      wave_lds_fence();
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
  const int32_t* order;      // optional [E]: experts by descending row count
  int32_t E;
  int32_t map_div;
  int32_t accumulate;
  int32_t tiles_per_expert;  // (M/BM)*(N/BN), identical for the three problems
#ifdef PK_GEMM_DEBUG
  int32_t debug;
#endif
};

template <int BM, int BN, int BK, int WMW, int WNW, int NS>
__global__ __launch_bounds__(64 * WMW * WNW) void wgrad_kernel(const WgradParams p) {
  constexpr int NTHREADS = 64 * WMW * WNW;
  constexpr int WTM = BM / WMW, WTN = BN / WNW;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * BK * 2, STAGE = (BM + BN) * BK * 2;
  constexpr int LA = A_BYTES / (NTHREADS * 16), LB = (STAGE - A_BYTES) / (NTHREADS * 16);
  using St = Stage<WTN>;
  constexpr int STAGING = WTM * St::LD * (WMW * WNW);
  constexpr int SMEM = STAGING > NS * STAGE ? STAGING : NS * STAGE;
  __shared__ __attribute__((aligned(1024))) char smem[SMEM];

  const WgradProblem& q = p.prob[blockIdx.y];
  // Workgroup b runs on XCD b % 8.  All tiles of one expert stay on one XCD, back to back, so its
  // rows are read from HBM once.  Experts are dealt to the XCDs in "snake" order (0..7, 7..0,
  // 0..7, ...) of p.order, the experts sorted by descending row count (pk_sort_by_expert), which
  // balances skewed routing; without an order they are dealt by index.
  const const_i32_ptr starts = as_const(p.starts);
  const int xcd = blockIdx.x % NXCD, pos = blockIdx.x / NXCD;
  const int jq = pos / p.tiles_per_expert;                       // position in this XCD's queue
  const int want = (jq & 1) ? jq * NXCD + (NXCD - 1 - xcd) : jq * NXCD + xcd;   // rank to serve
  if (want >= p.E) return;
  const int e = p.order ? as_const(p.order)[want] : want;
  const int t = pos % p.tiles_per_expert;
  const int n_tiles = q.N / BN;
  const int mt = t / n_tiles, nt = t % n_tiles;
  const int row_begin = starts[e], row_end = starts[e + 1];
  const int nkt = (row_end - row_begin + BK - 1) / BK;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WNW, wn = wave % WNW;

  // One dma16 covers 64 consecutive 16-byte slots = RPI rows of the tile; the row index (and the
  // optional gather through a row map) is wave-uniform per row, so it is resolved with scalar
  // loads, which do not disturb the vmcnt bookkeeping of the LDS ring.
  constexpr int A_CPR = BM / 8, B_CPR = BN / 8;
  constexpr int A_RPI = 64 / A_CPR, B_RPI = 64 / B_CPR;
  const const_i32_ptr a_map = as_const(q.a_map), b_map = as_const(q.b_map);
  const bf16_t* const Abase = q.A + (int64_t)mt * BM;
  const bf16_t* const Bbase = q.B + (int64_t)nt * BN;
  const int64_t lda = q.lda, ldb = q.ldb;
  const int map_div = p.map_div;

  auto issue = [&](int kt, int stage) {
    char* st = smem + stage * STAGE;
    const uint32_t a_lds = lds_addr(st) + (wave * LA) * 1024;
    const uint32_t b_lds = lds_addr(st + A_BYTES) + (wave * LB) * 1024;
    const int k0 = row_begin + kt * BK;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
      int krow, cofs;
      mn_slot<BM>(wave * LA + i, lane, krow, cofs);
      const void* src = g_zero16;
#pragma unroll
      for (int r = 0; r < A_RPI; ++r) {
        const int row = k0 + (wave * LA + i) * A_RPI + r;     // wave-uniform
        if (row < row_end) {
          int64_t rr = row;
          if (a_map) rr = a_map[row] / map_div;
          const bf16_t* cand = Abase + rr * lda;
          if (lane / A_CPR == r) src = cand + cofs;
        }
      }
      dma16(src, a_lds + i * 1024);
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      int krow, cofs;
      mn_slot<BN>(wave * LB + i, lane, krow, cofs);
      const void* src = g_zero16;
#pragma unroll
      for (int r = 0; r < B_RPI; ++r) {
        const int row = k0 + (wave * LB + i) * B_RPI + r;
        if (row < row_end) {
          int64_t rr = row;
          if (b_map) rr = b_map[row] / map_div;
          const bf16_t* cand = Bbase + rr * ldb;
          if (lane / B_CPR == r) src = cand + cofs;
        }
      }
      dma16(src, b_lds + i * 1024);
    }
  };

  floatx16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

#pragma unroll
  for (int s = 0; s < NS - 1; ++s)
    if (s < nkt) issue(s, s);
  int cur = 0, nxt = NS - 1;
  for (int kt = 0; kt < nkt; ++kt) {
    if (kt + NS - 2 < nkt) wait_dma<(NS - 2) * (LA + LB)>(); else wait_dma<0>();
    block_barrier();
#ifdef PK_GEMM_DEBUG
    if (!(p.debug & 2))
#endif
    if (kt + NS - 1 < nkt) issue(kt + NS - 1, nxt);
    const char* st = smem + cur * STAGE;
#ifdef PK_GEMM_DEBUG
    if (!(p.debug & 1))
#endif
    mma_tile<BK, TM, TN, false, false, BM, BN, (TM * TN >= 16)>(st, st + A_BYTES, wm * WTM, wn * WTN, acc);
    cur = cur + 1 == NS ? 0 : cur + 1;
    nxt = nxt + 1 == NS ? 0 : nxt + 1;
  }

#ifdef PK_GEMM_DEBUG
  if (p.debug & 4) { if (acc[0][0][0] != 12345.678f) return; }
#endif
  block_barrier();
  bf16_t* C = q.C + (int64_t)e * q.M * q.N + ((int64_t)mt * BM + wm * WTM) * q.N + (int64_t)nt * BN + wn * WTN;
  char* sbuf = smem + wave * (WTM * St::LD);
  const int lrow = lane & 31, lq = 4 * (lane >> 5);
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd)
        St::put(sbuf, 32 * i + lrow, 32 * j + 8 * qd + lq,
                pack4(acc[i][j][4 * qd], acc[i][j][4 * qd + 1], acc[i][j][4 * qd + 2], acc[i][j][4 * qd + 3]));
  wave_lds_fence();
  if (p.accumulate) St::template flush<WTM, true>(sbuf, C, q.N, WTM);
  else St::template flush<WTM, false>(sbuf, C, q.N, WTM);
}

inline int round_up_xcd(int64_t n) { return (int)(pk_ceil_div(n, NXCD) * NXCD); }

template <int BM, int BN, int BK, int WMW, int WNW, int NS, int OCC, bool B_KC, int EPI>
int launch_ragged_m(RaggedMParams p, int64_t A_rows, int kernel_id, hipStream_t s) {
#ifdef PK_GEMM_DEBUG
  { const char* d = getenv("PK_GEMM_DEBUG_MODE"); p.debug = d ? atoi(d) : 0; }
#endif
  const int64_t max_units = (pk_ceil_div(A_rows, BM) + p.E) * p.n_tiles;
  if (max_units > 0x7ffffff0ll) return PK_ERR_SHAPE;
  PK_LAUNCH_NOCHECK(kernel_id, s, (ragged_m_kernel<BM, BN, BK, WMW, WNW, NS, OCC, B_KC, EPI>),
                    dim3(round_up_xcd(max_units)), dim3(64 * WMW * WNW), 0, s, p);
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

// Tile configurations: BM, BN, waves along M, waves along N, LDS stages.  Measured on MI355X
// with random data and multinomial / Zipf row counts over {128,256}x{128,256} tiles, 4/8/16
// waves and 2/3 stages: 128x256 with 8 waves (64x64 wave tiles, 3-stage 144 KB ring) is fastest
// for the ragged-M kernels, 256x256 with 8 waves (128x64 wave tiles) for the weight gradient.
// (BM, BN, BK, waves M, waves N, stages, workgroups per CU)
#ifndef PK_RM_CFG
#define PK_RM_CFG 128, 256, 64, 2, 4, 3, 1
#define PK_RM_BN 256
#endif
#ifndef PK_WG_BIG
#define PK_WG_BIG 256, 256, 64, 2, 4, 2     /* 8 waves, 128x64 wave tiles, 128 KB ring */
#define PK_WG_BIG_THREADS 512
#endif
#define PK_WG_SMALL 128, 128, 64, 2, 2, 3
#define PK_WG_SMALL_THREADS 256

#define PK_RM_ALT 128, 128, 64, 2, 2, 3, 1      /* output widths that are a multiple of 128 but not of 256 */
bool mfma_shape_ok(int64_t H, int64_t I) { return H % 128 == 0 && I % 128 == 0; }

// Pick the tile width by the output width N of the GEMM (for the gate/up kernel a tile holds
// BN/2 gate and BN/2 up columns).
template <bool B_KC, int EPI>
int launch_rm(mf::RaggedMParams& p, int64_t A, int64_t N, int kernel_id, hipStream_t s) {
  const int64_t per_tile_big = (EPI == mf::EPI_SWIGLU) ? PK_RM_BN / 2 : PK_RM_BN;
  if (N % per_tile_big == 0) {
    p.n_tiles = (int32_t)(N / per_tile_big);
    return mf::launch_ragged_m<PK_RM_CFG, B_KC, EPI>(p, A, kernel_id, s);
  }
  const int64_t per_tile_alt = (EPI == mf::EPI_SWIGLU) ? 64 : 128;
  p.n_tiles = (int32_t)(N / per_tile_alt);
  return mf::launch_ragged_m<PK_RM_ALT, B_KC, EPI>(p, A, kernel_id, s);
}

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
  p.O0 = (bf16_t*)g; p.O1 = (bf16_t*)u; p.O2 = (bf16_t*)h; p.ldc = I;
  rc = launch_rm<true, mf::EPI_SWIGLU>(p, A, I, pk_timing::K_SWIGLU_GATE_UP, s);
  if (rc) return rc;

  mf::RaggedMParams q = {};
  q.A0 = (const bf16_t*)h; q.lda = I;
  q.B0 = (const bf16_t*)w2; q.B1 = nullptr; q.ldb = I; q.strideB = H * I;
  q.starts = starts; q.E = (int32_t)E; q.Kseg = (int32_t)I; q.nseg = 1;
  q.O0 = (bf16_t*)y; q.ldc = H;
  return launch_rm<true, mf::EPI_PLAIN>(q, A, H, pk_timing::K_SWIGLU_DOWN, s);
}

int pk_grouped_swiglu_dgrad_dh(const void* d_y, const void* w2, const void* g, const void* u,
                               const int32_t* starts, void* d_g, void* d_u, int64_t A, int64_t H,
                               int64_t I, int64_t E, int dtype, pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  if (A == 0) return PK_OK;
  if (!d_y || !w2 || !g || !u || !starts || !d_g || !d_u) return PK_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const bool simt = dtype == PK_F32 || !mfma_shape_ok(H, I) || !all_aligned16({d_y, w2, g, u, d_g, d_u});
  if (simt) {
    // d_h = d_y . w2[e]  (w2[e] is [H, I]: B(k=h, n=i) = w2[h*I + i]); staged in d_u's buffer
    const int64_t n = A * I;
    if (dtype == PK_F32) {
      rc = simt_ragged_m<float>(d_y, H, nullptr, 1, w2, I, 1, H * I, d_u, I, starts, A, I, H, E, 0, s);
      if (rc) return rc;
      PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_ELEMENTWISE, s, (swiglu_bwd_kernel<float>), dim3((unsigned)pk_ceil_div(n, 256)), dim3(256), 0, s,
                        (const float*)d_u, (const float*)g, (const float*)u, (float*)d_g, (float*)d_u, n);
    } else {
      rc = simt_ragged_m<bf16_t>(d_y, H, nullptr, 1, w2, I, 1, H * I, d_u, I, starts, A, I, H, E, 0, s);
      if (rc) return rc;
      PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_ELEMENTWISE, s, (swiglu_bwd_kernel<bf16_t>), dim3((unsigned)pk_ceil_div(n, 256)), dim3(256), 0, s,
                        (const bf16_t*)d_u, (const bf16_t*)g, (const bf16_t*)u, (bf16_t*)d_g, (bf16_t*)d_u, n);
    }
    PK_RETURN_IF_LAUNCH_FAILED();
    return PK_OK;
  }
  mf::RaggedMParams p = {};
  p.A0 = (const bf16_t*)d_y; p.lda = H;
  p.B0 = (const bf16_t*)w2; p.ldb = I; p.strideB = H * I;
  p.starts = starts; p.E = (int32_t)E; p.Kseg = (int32_t)H; p.nseg = 1;
  p.Gin = (const bf16_t*)g; p.Uin = (const bf16_t*)u;
  p.O0 = (bf16_t*)d_g; p.O1 = (bf16_t*)d_u; p.ldc = I;
  return launch_rm<false, mf::EPI_SWIGLU_BWD>(p, A, I, pk_timing::K_SWIGLU_DGRAD_DH, s);
}

int pk_grouped_swiglu_dgrad_dx(const void* d_g, const void* d_u, const void* w1, const void* w3,
                               const int32_t* starts, void* d_x_sorted, int64_t A, int64_t H,
                               int64_t I, int64_t E, int dtype, pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  if (A == 0) return PK_OK;
  if (!d_g || !d_u || !w1 || !w3 || !starts || !d_x_sorted) return PK_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const bool simt = dtype == PK_F32 || !mfma_shape_ok(H, I) || !all_aligned16({d_g, d_u, w1, w3, d_x_sorted});
  if (simt) {
    // d_x = d_g . w1[e] + d_u . w3[e]   (w[e] is [I, H]: B(k=i, n=h) = w[i*H + h])
    if (dtype == PK_F32) {
      rc = simt_ragged_m<float>(d_g, I, nullptr, 1, w1, H, 1, I * H, d_x_sorted, H, starts, A, H, I, E, 0, s);
      if (rc) return rc;
      return simt_ragged_m<float>(d_u, I, nullptr, 1, w3, H, 1, I * H, d_x_sorted, H, starts, A, H, I, E, 1, s);
    }
    rc = simt_ragged_m<bf16_t>(d_g, I, nullptr, 1, w1, H, 1, I * H, d_x_sorted, H, starts, A, H, I, E, 0, s);
    if (rc) return rc;
    return simt_ragged_m<bf16_t>(d_u, I, nullptr, 1, w3, H, 1, I * H, d_x_sorted, H, starts, A, H, I, E, 1, s);
  }
  // d_x = [d_g | d_u] . [w1[e] ; w3[e]]
  mf::RaggedMParams q = {};
  q.A0 = (const bf16_t*)d_g; q.A1 = (const bf16_t*)d_u; q.lda = I;
  q.B0 = (const bf16_t*)w1; q.B1 = (const bf16_t*)w3; q.ldb = H; q.strideB = I * H;
  q.starts = starts; q.E = (int32_t)E; q.Kseg = (int32_t)I; q.nseg = 2;
  q.O0 = (bf16_t*)d_x_sorted; q.ldc = H;
  return launch_rm<false, mf::EPI_PLAIN>(q, A, H, pk_timing::K_SWIGLU_DGRAD_DX, s);
}

int pk_grouped_swiglu_dgrad(const void* d_y, const void* w1, const void* w2, const void* w3,
                            const void* g, const void* u, const int32_t* starts, void* d_g,
                            void* d_u, void* d_x_sorted, int64_t A, int64_t H, int64_t I,
                            int64_t E, int dtype, pk_stream_t stream) {
  int rc = pk_grouped_swiglu_dgrad_dh(d_y, w2, g, u, starts, d_g, d_u, A, H, I, E, dtype, stream);
  if (rc) return rc;
  return pk_grouped_swiglu_dgrad_dx(d_g, d_u, w1, w3, starts, d_x_sorted, A, H, I, E, dtype, stream);
}

int pk_grouped_swiglu_wgrad(const void* d_y, const void* h, const void* d_g, const void* d_u,
                            const void* x_rows, const int32_t* row_map, int64_t row_map_div,
                            const int32_t* starts, const int32_t* expert_order, void* d_w1,
                            void* d_w2, void* d_w3,
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
  p.starts = starts; p.order = expert_order; p.E = (int32_t)E; p.map_div = (int32_t)row_map_div;
  p.accumulate = accumulate ? 1 : 0;
#ifdef PK_GEMM_DEBUG
  { const char* d = getenv("PK_GEMM_DEBUG_MODE"); p.debug = d ? atoi(d) : 0; }
#endif
  const bool big = (H % 256 == 0) && (I % 256 == 0);
  const int tile = big ? 256 : 128;
  p.tiles_per_expert = (int32_t)((H / tile) * (I / tile));
  const int64_t blocks = (int64_t)p.tiles_per_expert * pk_ceil_div(E, mf::NXCD) * mf::NXCD;
  if (blocks > 0x7ffffff0ll) return PK_ERR_SHAPE;
  if (big)
    PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_WGRAD, s, (mf::wgrad_kernel<PK_WG_BIG>), dim3((unsigned)blocks, n), dim3(PK_WG_BIG_THREADS), 0, s, p);
  else
    PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_WGRAD, s, (mf::wgrad_kernel<PK_WG_SMALL>), dim3((unsigned)blocks, n), dim3(PK_WG_SMALL_THREADS), 0, s, p);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

}  // extern "C"
