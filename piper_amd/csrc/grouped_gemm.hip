// Grouped SwiGLU expert GEMMs (forward, input gradient, weight gradient).
//   bf16: v_mfma_f32_32x32x16_bf16 tiles fed by a ring of direct-to-LDS loads.
//         Forward and input gradient (ragged_m_kernel): persistent workgroups (one per CU) that
//         take (expert, row tile, column tile) units from per-XCD counters, 256x256x32 or
//         128x256x64 block tiles with 8 waves, fused SwiGLU / SwiGLU-backward epilogues, permute
//         fused into the A-operand loader; ragged row tiles are located on the device from
//         starts[] (no host sync).  Weight gradient: wgrad_pp_kernel (persistent, 256x256x32, one
//         operand from the transposed copies the scaled SwiGLU backward writes) for the fused
//         region; wgrad_kernel (one workgroup per (expert, output tile), both operands through the
//         transposing LDS read) for the piecewise entry points.
//   f32 : tiled FMA kernel (simt_gemm.h) + elementwise SwiGLU kernels; exact fp32 arithmetic.
#include "pk_common.h"
#include "simt_gemm.h"
#include <functional>
#include <initializer_list>
#include <map>
#include <mutex>
#include <thread>
#include <tuple>
#include <type_traits>

namespace {

// ===================================================================== bf16 MFMA path
namespace mf {

constexpr int NXCD = 8;


// EPI_SWIGLU_BWD_SCALED: the A rows are rows of d_out gathered through the row map, the
// accumulator is the unscaled d_h; the epilogue multiplies by the row's combine score, also
// emits score * h and the per-row partial dot products <unscaled d_h, h> (the score gradient).
enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_SWIGLU_BWD = 2, EPI_SWIGLU_BWD_SCALED = 3 };

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
// The statement sets M0 and uses it at once.  M0 cannot be named as clobbered (the compiler
// treats it as reserved and rejects the promise to preserve it), and nothing else in these
// kernels keeps a value in it: on gfx9 ordinary LDS accesses do not read M0, and the kernels
// use no indirect register indexing, readlane with a register index excepted, which takes an
// SGPR operand and not M0.
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off"
               :: "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(gptr)
               : "memory");
}
// The same load with the address split into a wave-uniform 64-bit base (scalar registers) and a
// 32-bit byte offset per lane: a k-loop then advances one scalar pointer per operand and k-tile
// instead of forming a 64-bit address per lane and load.  The LDS destination is lds_base + IMM.
template <int IMM>
__device__ __forceinline__ void dma16_s(uint32_t voff, const void* sbase, uint32_t lds_base) {
  asm volatile("s_add_i32 m0, %0, %3\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_base), "v"(voff), "s"(sbase), "n"(IMM)
               : "memory", "scc");
}
// Four bytes per lane straight into LDS (lane l's dword lands at lds_base + 4*l), same address form.
__device__ __forceinline__ void dma4_s(uint32_t voff, const void* sbase, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2"
               :: "s"(lds_base), "v"(voff), "s"(sbase)
               : "memory");
}
// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{}) in order
template <int I0, int N, typename F>
__device__ __forceinline__ void static_for_impl(F&& f) {
  if constexpr (I0 < N) {
    f(std::integral_constant<int, I0>{});
    static_for_impl<I0 + 1, N>(f);
  }
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) { static_for_impl<0, N>(f); }
template <int N>
__device__ __forceinline__ void wait_dma() {
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}
__device__ __forceinline__ void block_barrier() {
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
// A wave-uniform 64-bit value that the compiler could not prove uniform: into scalar registers.
__device__ __forceinline__ int64_t uniform_i64(int64_t x) {
  const uint64_t v = (uint64_t)x;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ const char* uniform_ptr(const char* p) {
  return (const char*)(uintptr_t)uniform_i64((int64_t)(uintptr_t)p);
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

// 1 / (1 + e^-x) with the hardware exponential and reciprocal (each within 1 ulp of fp32; the
// results are rounded to bf16).  A full-precision division costs ten instructions per value.
__device__ __forceinline__ float sigmoid_fast(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }
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
        // streaming store: a weight gradient is not read again by this or the next kernels, and
        // without it the 1.2 GB of gradients push the activation rows, which every column tile
        // of an expert reads again, out of the L2 (measured: -3 % on the kernel, -2 % on the step)
        __builtin_nontemporal_store(v, g);
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

// Wait until at most `t` (0..MAXT) whole tiles of L loads each are still in flight.
template <int L, int MAXT>
__device__ __forceinline__ void wait_tiles(int t) {
  if (MAXT <= 0 || t <= 0) { wait_dma<0>(); return; }
  if (t >= MAXT) { wait_dma<(MAXT > 0 ? MAXT : 0) * L>(); return; }
  wait_tiles<L, (MAXT > 0 ? MAXT - 1 : 0)>(t);
}

// Wait until at most n (wave-uniform, rounded down to a multiple of 4, capped at 60) vector-memory
// operations are outstanding.  Loads, stores and atomics retire from the counter in issue
// order, so with n = a lower bound of the operations issued AFTER the ones of interest this
// waits for those without waiting for the younger ones (for example an epilogue's stores).
__device__ __forceinline__ void wait_vm_le(int n) {
  switch ((n < 60 ? n : 60) >> 2) {
    case 0: wait_dma<0>(); break;    case 1: wait_dma<4>(); break;    case 2: wait_dma<8>(); break;
    case 3: wait_dma<12>(); break;   case 4: wait_dma<16>(); break;   case 5: wait_dma<20>(); break;
    case 6: wait_dma<24>(); break;   case 7: wait_dma<28>(); break;   case 8: wait_dma<32>(); break;
    case 9: wait_dma<36>(); break;   case 10: wait_dma<40>(); break;  case 11: wait_dma<44>(); break;
    case 12: wait_dma<48>(); break;  case 13: wait_dma<52>(); break;  case 14: wait_dma<56>(); break;
    default: wait_dma<60>(); break;
  }
}

// Per-lane slice of the prefix sum of work units over experts: lane l covers experts
// [l*epl, (l+1)*epl).  Built once per wave with ordinary loads; locating a unit afterwards
// takes a ballot plus a short scalar walk, so it can run in the middle of the k-loop without
// touching the vector-memory counter that tracks the LDS ring.
struct UnitIndex {
  int excl, incl, total, epl;
};
template <int BM>
__device__ __forceinline__ UnitIndex build_unit_index(const int32_t* __restrict__ starts, int E, int n_tiles) {
  const int lane = threadIdx.x & 63;
  UnitIndex ui;
  ui.epl = (E + 63) >> 6;
  const int e_lo = lane * ui.epl, e_hi = min(E, e_lo + ui.epl);
  int mine = 0;
  for (int e = e_lo; e < e_hi; ++e) mine += ((starts[e + 1] - starts[e] + BM - 1) / BM) * n_tiles;
  int incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int v = __shfl_up(incl, off, PK_WAVE);
    if (lane >= off) incl += v;
  }
  ui.incl = incl;
  ui.excl = incl - mine;
  ui.total = __builtin_amdgcn_readlane(incl, 63);
  return ui;
}
// unit < ui.total.  Units of expert e are laid out [n-tile][m-tile], so neighbouring units share
// the weight tile.  Everything returned is wave-uniform.
template <int BM>
__device__ __forceinline__ void locate_unit(const UnitIndex& ui, const_i32_ptr starts, int E, int n_tiles,
                                            int unit, int& e_out, int& mt_out, int& nt_out) {
  const unsigned long long bal = __ballot(unit >= ui.excl && unit < ui.incl);
  const int src = __builtin_amdgcn_readfirstlane(__ffsll((long long)bal) - 1);
  int u = unit - __builtin_amdgcn_readlane(ui.excl, src);
  int e = src * ui.epl;
  const int e_hi = min(E, e + ui.epl);
  int tiles = 1;
  for (; e < e_hi; ++e) {
    tiles = (starts[e + 1] - starts[e] + BM - 1) / BM;
    const int units = tiles * n_tiles;
    if (u < units) break;
    u -= units;
  }
  tiles = tiles > 0 ? tiles : 1;
  e_out = e;
  nt_out = u / tiles;
  mt_out = u - nt_out * tiles;
}

// ---------------------------------------------------------------------------------------------
// Work distribution of the persistent kernels.  Units are grouped in chunks of SCHED_CHUNK
// consecutive units; chunk c belongs to XCD c % 8, whose workgroups take its units one at a
// time from a counter, so the workgroups of an XCD always run neighbouring units (shared
// operands stay in that XCD's L2) while uneven unit costs still balance.  A workgroup whose own
// XCD has run dry takes units from the other XCDs' counters.  Every launch uses one set of a
// pool of counter sets, chosen by its stream (sched_slot_for_launch); the last workgroup to finish
// zeroes the set again, so no memset precedes a launch and launches in flight on different
// streams do not share counters.
constexpr int SCHED_CHUNK = 32;
constexpr int SCHED_SLOTS = PK_SCHED_SETS;
struct SchedSlot {
  unsigned grabs[NXCD];
  unsigned finished;
  unsigned pad[7];
};
__device__ SchedSlot g_sched_pool[SCHED_SLOTS];

__device__ __forceinline__ int sched_unit_of(unsigned j, int x) {
  return (int)(((j / SCHED_CHUNK) * NXCD + x) * SCHED_CHUNK + j % SCHED_CHUNK);
}
// One lane: take the next grab index of XCD x.  The request and the wait for its answer are one
// statement, so the compiler never sees a register whose value is still on its way; the wait
// drains the whole vector-memory counter, so this goes where that counter is about to be
// drained anyway (after the last store of an epilogue).
// The first `base` grab indices of every XCD are not taken from the counter: a workgroup knows its
// own (its position among the XCD's workgroups, and that plus the XCD's workgroup count where
// two units are settled at the start), so a kernel starts without a round trip to the counter.
__device__ __forceinline__ unsigned sched_grab(SchedSlot* slot, int x, unsigned base) {
  unsigned ret;
  const unsigned one = 1u;
  asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)"
               : "=&v"(ret) : "v"(&slot->grabs[x]), "v"(one) : "memory");
  return ret + base;
}
// Publish a value in LDS for the other waves: the write must have landed before this wave
// arrives at the next barrier, also on paths that issue no further LDS traffic.
__device__ __forceinline__ void lds_publish(int* box, int v) {
  *box = v;
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}
// One lane: the next unit for a workgroup of XCD `xcd` (own counter first, then the others), or
// -1 when all units are taken.  `first` is an already fetched grab index of the own counter.
__device__ __forceinline__ int sched_resolve(SchedSlot* slot, int xcd, unsigned first, int total, unsigned base) {
  int unit = sched_unit_of(first, xcd);
  if (unit < total) return unit;
  for (int a = 1; a < NXCD; ++a) {
    const int x = (xcd + a) % NXCD;
    // skip counters that are visibly exhausted (plain read first keeps them from running away)
    if (sched_unit_of(__atomic_load_n(&slot->grabs[x], __ATOMIC_RELAXED) + base, x) >= total) continue;
    unit = sched_unit_of(atomicAdd(&slot->grabs[x], 1u) + base, x);
    if (unit < total) return unit;
  }
  return -1;
}
// One lane, after the workgroup's last unit: the last workgroup of the grid resets the slot.
__device__ __forceinline__ void sched_finish(SchedSlot* slot) {
  __threadfence();
  if (atomicAdd(&slot->finished, 1u) == gridDim.x - 1) {
#pragma unroll
    for (int i = 0; i < NXCD; ++i) slot->grabs[i] = 0u;
    slot->finished = 0u;
    __threadfence();
  }
}

// Transposed copies of an expert-sorted [rows][width] operand, for consumers that want the routed
// rows contiguous: the rows are placed on a padded row axis on which expert e starts at
// padded_start(e), a multiple of 64 computed from starts[e] alone, and owns
// [padded_start(e), padded_start(e+1)), which holds its rows rounded up to a multiple of 32
// (the range is a multiple of 64 and longer than the row count: round_down64(a + n) + 64 > n; an
// axis of round_up64(A) + 64 * E holds every expert).  The copy
// is stored in blocks of 32 padded rows, [axis / 32][width][32]: column c at padded row q sits at
// ((q / 32) * width + c) * 32 + q % 32.  A 32-row chunk of 64 columns that the producer stages is
// then 4 KB of consecutive memory, and a consumer's 32-deep k-tile of 256 columns 16 KB.
constexpr int kTransposedAlign = 64;
__host__ __device__ __forceinline__ int padded_start(int start, int e) {
  return (start & ~(kTransposedAlign - 1)) + kTransposedAlign * e;
}

// Division of a non-negative int32 by a divisor fixed per launch without the ~25 instructions of
// the general integer division: multiply-high by 2^(32-s) for d = 2^s, otherwise by
// floor(2^(31+s)/d)+1 followed by a shift by s-1 with s = ceil(log2 d) (exact for 0 <= n < 2^31).
struct FastDiv {
  uint32_t mul;    // 0: divisor is 1
  int32_t shift;
  int64_t d;       // the divisor itself (host side checks)
};
inline FastDiv make_fastdiv(int64_t d) {
  FastDiv f = {0u, 0, d < 1 ? 1 : d};
  if (d <= 1) return f;
  int s = 0;
  while (((int64_t)1 << s) < d) ++s;
  if (((int64_t)1 << s) == d) { f.mul = 1u << (32 - s); return f; }   // mulhi by 2^(32-s) is the shift by s
  f.mul = (uint32_t)((((uint64_t)1 << (31 + s)) / (uint64_t)d) + 1u);
  f.shift = s - 1;
  return f;
}
// No branch on the divisor's kind (it would sit between the MFMAs of the loops that divide per lane):
// the product is always formed and a mask picks n itself for a divisor of 1.
__device__ __forceinline__ int fastdiv(int n, const FastDiv f) {
  const uint32_t u = (uint32_t)n;
  const uint32_t q = __umulhi(u, f.mul) >> f.shift;
  const uint32_t keep = f.mul == 0u ? 0xffffffffu : 0u;
  return (int)((u & keep) | (q & ~keep));
}

struct RaggedMParams {
  const bf16_t* A0;      // A operand of k-segment 0, row-major [rows, lda]
  const bf16_t* A1;      // k-segment 1 (nseg == 2)
  int64_t lda;
  const int32_t* row_map;  // optional gather of A rows: src = row_map[row] / divisor of map_div
  FastDiv map_div;
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
  bf16_t* O2;            //            SWIGLU: h;  SWIGLU_BWD_SCALED: score * h
  int64_t ldc;
  const float* scores;   // SWIGLU_BWD_SCALED: score of sorted row r is scores[row_map[r]]
  float* ds_partial;     // SWIGLU_BWD_SCALED: [ldc / 64][total_rows] partial <unscaled d_h, h>
  int64_t total_rows;
  // SWIGLU_BWD_SCALED, optional: the three outputs once more, transposed in blocks of 32 padded rows
  // ([ldt / 32][ldc][32], see padded_start) for the weight-gradient kernels that want a K-contiguous
  // operand; the padded rows up to the next multiple of 32 after an expert's last row are zero.
  bf16_t* T0;            // d_g^T
  bf16_t* T1;            // d_u^T
  bf16_t* T2;            // (score * h)^T
  int64_t ldt;
  SchedSlot* sched;      // this launch's counters
};

// Wave-private staging of 32 rows x COLS bf16 of the output through LDS, so that global stores
// are 16 bytes per lane and row-contiguous.  Rows are unpadded (COLS*2 bytes); the 16-byte
// chunks of row r are XOR-swizzled with r so that a column of 8-byte deposits spreads over the banks.
template <int COLS>
struct Stage32 {
  static constexpr int ROWB = COLS * 2, CH = ROWB / 16, BYTES = 32 * ROWB;
  static_assert((CH & (CH - 1)) == 0 && CH >= 2, "power-of-two chunk count");
  // a lane deposits 4 consecutive columns (col % 4 == 0) of one row
  __device__ static __forceinline__ void put(char* buf, int row, int col, u32x2_t v) {
    *reinterpret_cast<u32x2_t*>(buf + row * ROWB + ((((col >> 3) ^ row) & (CH - 1)) << 4) + (col & 7) * 2) = v;
  }
  // rows [0, nrows) go to dst[r * ldc + 0..COLS); returns the number of store instructions
  // the wave issued (nrows is wave-uniform).  STREAM: nontemporal stores, for results that neither
  // this nor the next kernels read (weight gradients).
  // (lane: the caller's lane id; a caller that wants the per-lane addresses formed here, not hoisted
  // out of its loops into registers that stay live across them, passes a value the compiler cannot
  // see through)
  template <bool ACC, bool STREAM = false>
  __device__ static __forceinline__ int flush(const char* buf, bf16_t* dst, int64_t ldc, int nrows, int lane = threadIdx.x & 63) {
    constexpr int RPP = 64 / CH, NP = 32 / RPP;
    const int lr = lane / CH, lc = lane % CH;
    u32x4_t v[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) {     // all LDS reads first: one latency for the whole chunk
      const int r = q * RPP + lr;
      v[q] = *reinterpret_cast<const u32x4_t*>(buf + r * ROWB + (((lc ^ r) & (CH - 1)) << 4));
    }
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int r = q * RPP + lr;
      if (r < nrows) {
        u32x4_t* g = reinterpret_cast<u32x4_t*>(dst + (int64_t)r * ldc + lc * 8);
        if (ACC) {
          const bf16x8_t a = __builtin_bit_cast(bf16x8_t, v[q]);
          const bf16x8_t o = __builtin_bit_cast(bf16x8_t, *g);
          bf16x8_t sum;
#pragma unroll
          for (int t = 0; t < 8; ++t) sum[t] = (bf16_t)((float)a[t] + (float)o[t]);
          v[q] = __builtin_bit_cast(u32x4_t, sum);
        }
        if (STREAM) __builtin_nontemporal_store(v[q], g);
        else *g = v[q];
      }
    }
    return nrows >= 32 ? NP : nrows <= 0 ? 0 : (nrows + RPP - 1) / RPP;
  }
  // All 32 rows of the staged tile added to values fetched earlier (old[q]: what flush would read
  // at dst for pass q -- rows q * RPP + lane / CH, 16-byte piece lane % CH) and stored: fp32 add, one
  // rounding of the sum.  Returns the number of store instructions issued.
  template <bool STREAM>
  __device__ static __forceinline__ int flush_add(const char* buf, bf16_t* dst, int64_t ldc, const u32x4_t (&old)[32 / (64 / CH)],
                                                  int lane = threadIdx.x & 63) {
    constexpr int RPP = 64 / CH, NP = 32 / RPP;
    const int lr = lane / CH, lc = lane % CH;
    u32x4_t v[NP];
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int r = q * RPP + lr;
      v[q] = *reinterpret_cast<const u32x4_t*>(buf + r * ROWB + (((lc ^ r) & (CH - 1)) << 4));
    }
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int r = q * RPP + lr;
      const bf16x8_t a = __builtin_bit_cast(bf16x8_t, v[q]);
      const bf16x8_t o = __builtin_bit_cast(bf16x8_t, old[q]);
      bf16x8_t sum;
#pragma unroll
      for (int t = 0; t < 8; ++t) sum[t] = (bf16_t)((float)a[t] + (float)o[t]);
      u32x4_t* g = reinterpret_cast<u32x4_t*>(dst + (int64_t)r * ldc + lc * 8);
      if (STREAM) __builtin_nontemporal_store(__builtin_bit_cast(u32x4_t, sum), g);
      else *g = __builtin_bit_cast(u32x4_t, sum);
    }
    return NP;
  }
  // The staged tile transposed: element (r, c) goes to dstT[c * ldt + r] (ldt = 32 for the blocked
  // transposed copies), rows in groups of 8 (16 bytes per lane).  With nrows > 0 all 32 rows are
  // written: the caller stages zeros in rows nrows..31, and the consumer finds zeros up to the end
  // of the 32-row block.  dstT + multiples of ldt must be 16-byte aligned.  The transposing LDS read hands a lane 4
  // consecutive rows of one column: within 16 lanes, lane i points at row i/4, columns 4*(i%4)..+3
  // and receives rows 0..3 of column i.  One store instruction covers 16 columns x 32 rows: the
  // four 16-lane groups take the four 8-row groups, so each destination row receives 64
  // contiguous bytes per instruction.  Returns the number of store instructions issued.
  __device__ static __forceinline__ int flush_t(const char* buf, bf16_t* dstT, int64_t ldt, int nrows, int lane = threadIdx.x & 63) {
    static_assert(COLS % 16 == 0, "passes of 16 columns");
    constexpr int NQ = COLS / 16;
    const int i = lane & 15, grp = lane >> 4;
    const int r0 = 8 * grp + (i >> 2), r1 = r0 + 4;
    typedef short shortx8_t __attribute__((ext_vector_type(8)));
    u32x4_t v[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {                   // columns 16q .. 16q+15
      const int col = 16 * q + 4 * (i & 3);          // first of the 4 columns this lane points at
      const char* p0 = buf + r0 * ROWB + ((((col >> 3) ^ r0) & (CH - 1)) << 4) + (col & 7) * 2;
      const char* p1 = buf + r1 * ROWB + ((((col >> 3) ^ r1) & (CH - 1)) << 4) + (col & 7) * 2;
      const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4_t*)(p0));
      const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4_t*)(p1));
      v[q] = __builtin_bit_cast(u32x4_t, (shortx8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
    if (nrows > 0) {
#pragma unroll
      for (int q = 0; q < NQ; ++q)
        *reinterpret_cast<u32x4_t*>(dstT + (int64_t)(16 * q + i) * ldt + 8 * grp) = v[q];
    }
    return nrows > 0 ? NQ : 0;
  }
};

// MFMAs of one BK-deep k-tile for a wave tile of TM x TN MFMA tiles, with the L direct-to-LDS
// loads of a later tile spread evenly between them: a wave that issues its loads back to back
// blocks on the memory pipeline for many hundred cycles with its MFMAs queued behind them.
// Fragments are double buffered one 16-deep k-step ahead, and their LDS reads are spread between
// the MFMAs as well, which keeps the LDS queue short while the ring is being written.  Operands are passed to the MFMA
// swapped (B first) so that a lane's accumulator holds 4 CONSECUTIVE columns of ONE row:
//   acc[i][j][v] = C[row = 32*i + lane%32][col = 32*j + 8*(v/4) + 4*(lane/32) + v%4]
// There is no branch between the MFMAs: the L loads are issued for every k-tile (the caller
// points them at a block of zeros when no tile is left to fetch) and the first fragments of the
// "next tile" are always read (the caller passes any tile of the ring when there is none).
template <int BK, int TM, int TN, bool A_KC, bool B_KC, int ACOLS, int BCOLS, int L, typename F>
__device__ __forceinline__ void mma_ktile(const char* At, const char* Bt, const char* At_next, const char* Bt_next,
                                          int wrow0, int wcol0, Frags<TM, TN>& f0,
                                          floatx16_t (&acc)[TM][TN], F&& issue_one) {
  const int lane = threadIdx.x & 63;
  constexpr int KS = BK / 16, NM = KS * TM * TN;
  constexpr int EVERY = NM / L > 0 ? NM / L : 1;
  static_assert(L <= NM, "more loads than MFMAs in a k-tile");
  static_assert(TM + TN <= TM * TN, "one fragment read per MFMA slot");
  static_assert(KS % 2 == 0, "the fragments handed to the next k-tile live in buffer 0");
  // f0 holds the fragments of this tile's first k-step (read during the previous tile, or by
  // the caller for a unit's first tile); on return it holds those of the next tile, whose
  // operands the caller has made visible before this call
  Frags<TM, TN> f[2];
  f[0] = f0;
  // issue_one receives the load's index as a compile-time constant (std::integral_constant)
  static_for<NM>([&](auto idx_c) {
    constexpr int idx = decltype(idx_c)::value;
    constexpr int ks = idx / (TM * TN), m = idx % (TM * TN), i = m / TN, j = m % TN;
    constexpr bool last = ks + 1 == KS;
    constexpr int ksn = last ? 0 : ks + 1;
    const char* An = last ? At_next : At;
    const char* Bn = last ? Bt_next : Bt;
    if constexpr (m == 0) __builtin_amdgcn_sched_barrier(0);
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[ks & 1].b[j], f[ks & 1].a[i], acc[i][j], 0, 0, 0);
    // the sched barriers pin one fragment read of the next k-step (B first: the next
    // k-step starts with row 0) and at most one load behind each MFMA
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (m < TN)
      f[(ks + 1) & 1].b[m] = B_KC ? frag_kc<BK>(Bn, wcol0 + 32 * m, ksn, lane) : frag_mn<BCOLS>(Bn, wcol0 + 32 * m, ksn, lane);
    else if constexpr (m < TN + TM)
      f[(ks + 1) & 1].a[m - TN] = A_KC ? frag_kc<BK>(An, wrow0 + 32 * (m - TN), ksn, lane)
                                       : frag_mn<ACOLS>(An, wrow0 + 32 * (m - TN), ksn, lane);
    if constexpr (idx % EVERY == EVERY - 1 && idx / EVERY < L) issue_one(std::integral_constant<int, idx / EVERY>{});
    __builtin_amdgcn_sched_barrier(0);
  });
  f0 = f[0];
}

// C[rows_e, N] = A[rows_e, K] . op(B[e]) with B K-contiguous ([N,K]) or MN-contiguous ([K,N]).
// Persistent workgroups (one per CU): each walks a strided list of work units (expert, row tile,
// column tile), all units of one XCD being neighbours so that they share operands in its L2.
// Block tile BM x BN x BK, WMW x WNW waves, NS-stage LDS ring filled by direct-to-LDS loads;
// the ring is separate from the output staging, so the first NS-1 k-tiles of the next unit are
// requested before the epilogue of the current one, and the next unit's addresses (row map
// lookups included) are resolved with scalar loads during the current k-loop.
// EPI_SWIGLU: the BN tile rows are [32 gate | 32 up | 32 gate | 32 up ...] of BN/2 output
// columns, so that a lane holds the gate and the up value of the same element.
// A_T: the A operand comes from a transposed copy in blocks of 32 padded rows ([rows / 32][lda][32],
// see padded_start): a k-tile of it is one run of consecutive memory per 32-row block, it sits in LDS
// as [BK k][BM rows] and its fragments come out of the transposing LDS read.
template <int BM, int BN, int BK, int WMW, int WNW, int NS, bool B_KC, int EPI, bool A_T = false>
__global__ __launch_bounds__(64 * WMW * WNW) void ragged_m_kernel(const RaggedMParams p) {
  constexpr int NW = WMW * WNW, NTHREADS = 64 * NW;
  constexpr int WTM = BM / WMW, WTN = BN / WNW;          // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * BK * 2, STAGE = (BM + BN) * BK * 2;
  constexpr int LA = A_BYTES / (NTHREADS * 16), LB = (STAGE - A_BYTES) / (NTHREADS * 16), L = LA + LB;
  static_assert(LA >= 1 && LB >= 1 && TM >= 1 && TN >= 1, "tile too small for the wave grid");
  static_assert(EPI != EPI_SWIGLU || (WTN % 64 == 0), "gate/up pairs must stay inside a wave");
  static_assert(EPI != EPI_SWIGLU_BWD_SCALED || WTN == 64, "one score-gradient partial per 64 columns");
  constexpr bool BWD = EPI == EPI_SWIGLU_BWD || EPI == EPI_SWIGLU_BWD_SCALED;
  constexpr bool SCALED = EPI == EPI_SWIGLU_BWD_SCALED;
  constexpr bool PP = NW == 8;    // two waves per SIMD: the groups of the ping-pong k-loop
  constexpr int OUT_COLS = (EPI == EPI_SWIGLU) ? WTN / 2 : WTN;   // columns a wave writes per output tensor
  constexpr int BN_OUT = (EPI == EPI_SWIGLU) ? BN / 2 : BN;       // output columns per tile
  constexpr int RING = NS * STAGE;
  // The epilogue's staging area (32 rows x OUT_COLS per wave).  ALIAS: it is the ring stage that no
  // k-tile occupies between two units -- NS-1 stages hold the next unit's first k-tiles, the stage
  // of the last consumed tile is free until the next k-loop requests its tile NS-1, behind two
  // barriers that every wave reaches after its epilogue -- so the whole LDS can be ring.
  // Otherwise it lies behind the ring, 32 columns wide for the plain epilogue where the ring
  // leaves no room for all of them.
  constexpr bool ALIAS = PP && NW * 64 * OUT_COLS <= STAGE;
  constexpr int SW = ALIAS ? OUT_COLS : (EPI == EPI_PLAIN && RING + NW * 64 * OUT_COLS > 160 * 1024) ? 32 : OUT_COLS;
  using St = Stage32<SW>;
  constexpr int SMEM_BYTES = ALIAS ? RING : RING + NW * St::BYTES;
  // behind it, per wave: the row map entries of the A rows that the wave requests for the next unit
  constexpr int RM_BYTES = NW * 256;
  // and the two words through which one lane hands the next unit's index to the workgroup.  They
  // have a place of their own: inside the ring they would sit in a stage that the first memory
  // phase of the next k-loop may already be filling while a late wave still reads them.
  constexpr int BOX_BYTES = 16;
  static_assert(SMEM_BYTES + RM_BYTES + BOX_BYTES <= 160 * 1024, "LDS budget");
  __shared__ __attribute__((aligned(1024))) char smem[SMEM_BYTES + RM_BYTES + BOX_BYTES];
  constexpr int CPR = BK / 8, RPI = 64 / CPR;            // 16-byte chunks per A row, A rows per dma16
  static_assert(LA * RPI <= 64, "a wave's A rows of a tile: one entry per lane");
  static_assert(!A_T || BM % 32 == 0, "whole 32-row blocks of the transposed copy");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WNW, wn = wave % WNW;
  // staging area while `cur_stage` is the stage of the coming unit's k-tile 0
  auto staging_area = [&](int cur_stage) -> char* {
    return ALIAS ? smem + (cur_stage == 0 ? NS - 1 : cur_stage - 1) * STAGE : smem + RING;
  };
  const const_i32_ptr starts = as_const(p.starts);
  const const_i32_ptr row_map = as_const(p.row_map);

  // ---- first unit of this workgroup
  // the next unit, written by one lane, double buffered
  int* const sched_box = reinterpret_cast<int*>(smem + SMEM_BYTES + RM_BYTES);
  const UnitIndex ui = build_unit_index<BM>(p.starts, p.E, p.n_tiles);
  const int xcd = blockIdx.x % NXCD;
  unsigned grab = 0;                  // lane 0 of wave 0: grab index taken one unit ahead
  const unsigned sched_base = gridDim.x / NXCD;     // grab indices handed out without the counter
  if (tid == 0) sched_box[0] = sched_resolve(p.sched, xcd, blockIdx.x / NXCD, ui.total, sched_base);
  __syncthreads();
  int unit = __builtin_amdgcn_readfirstlane(sched_box[0]);
  if (unit < 0) {
    if (tid == 0) sched_finish(p.sched);
    return;
  }
  int par = 0;

  // ---- lane constants of the loaders: byte offsets of a lane's 16 bytes from a wave-uniform base
  uint32_t a_kofs[LA];
#pragma unroll
  for (int i = 0; i < LA; ++i) { int r, k; kc_slot<BK>(wave * LA + i, lane, r, k); a_kofs[i] = (uint32_t)k * 2u; }
  // EPI_SWIGLU: the rows of a wave's B pieces are 32 consecutive tile rows, i.e. 32 gate rows
  // (even waves) or 32 up rows (odd waves): a wave reads one of the two matrices only
  static_assert(EPI != EPI_SWIGLU || (B_KC && LB * RPI == 32), "a wave's B pieces are one 32-row group");
  uint32_t voffB[LB];
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    if (B_KC) {
      int r, kofs;
      kc_slot<BK>(wave * LB + i, lane, r, kofs);
      int n = r;
      if (EPI == EPI_SWIGLU) n = (r >> 6) * 32 + (r & 31);
      voffB[i] = (uint32_t)(n * (int)p.ldb + kofs) * 2u;
    } else {
      int krow, cofs;
      mn_slot<BN>(wave * LB + i, lane, krow, cofs);
      voffB[i] = (uint32_t)(krow * (int)p.ldb + cofs) * 2u;
    }
  }
  const int kt_per_seg = p.Kseg / BK;
  const int nkt = kt_per_seg * p.nseg;
  const uint32_t row_bytes = (uint32_t)p.lda * 2u;
  // bytes from one k-tile of A to the next: BK elements of a row, or BK columns of a 32-row block
  const uint32_t step_a = A_T ? BK * 64 : BK * 2, step_b = B_KC ? (uint32_t)(BK * 2) : (uint32_t)BK * (uint32_t)p.ldb * 2u;

  struct Unit {
    int row0, rows, nt;
    int tcol;            // column of row0 in the transposed outputs
    int64_t a_base;      // bytes from the A operand to the unit's first row (0 with a row map)
    int64_t b_base;      // bytes from the weights to the unit's tile
    uint32_t voff_a[LA]; // per lane: bytes from a_base to its row and 16-byte chunk
  };
  auto setup = [&](Unit& t, int un) {
    int e, mt, nt;
    locate_unit<BM>(ui, starts, p.E, p.n_tiles, un, e, mt, nt);
    const int s0 = starts[e], s1 = starts[e + 1];
    // (all wave-uniform; said again so that the pointers built from them stay in scalar registers)
    t.row0 = __builtin_amdgcn_readfirstlane(s0 + mt * BM);
    t.rows = __builtin_amdgcn_readfirstlane(min(BM, s1 - t.row0));
    t.nt = __builtin_amdgcn_readfirstlane(nt);
    t.tcol = __builtin_amdgcn_readfirstlane(padded_start(s0, e) + mt * BM);
    t.b_base = uniform_i64(((int64_t)e * p.strideB + (B_KC ? (int64_t)nt * BN_OUT * p.ldb : (int64_t)nt * BN)) * 2);
    if constexpr (A_T) {
      // the unit's first row sits at padded row tcol (a multiple of 64): block tcol / 32, and block b of
      // the copy starts at b * lda * 32 elements.  A lane's 16 bytes are 8 consecutive rows of one
      // column; blocks past the unit's last row are read from its last block instead (valid memory,
      // rows that are never stored).
      t.a_base = uniform_i64((int64_t)(t.tcol >> 5) * p.lda * 64);
#pragma unroll
      for (int i = 0; i < LA; ++i) {
        int krow, cofs;
        mn_slot<BM>(wave * LA + i, lane, krow, cofs);
        const int blk = min(cofs >> 5, (t.rows - 1) >> 5);
        t.voff_a[i] = (uint32_t)((blk * (int)p.lda + krow) * 32 + (cofs & 31)) * 2u;
      }
    } else {
      t.a_base = p.row_map ? (int64_t)0 : uniform_i64((int64_t)t.row0 * p.lda * 2);
      if (!p.row_map) {
#pragma unroll
        for (int i = 0; i < LA; ++i) {
          const int rbase = (wave * LA + i) * RPI;     // first tile row of this dma16 (wave-uniform)
          t.voff_a[i] = (uint32_t)min(rbase + lane / CPR, t.rows - 1) * row_bytes + a_kofs[i];   // rows past the range are never stored
        }
      }
    }
  };
  // With a row map the A rows are gathered: the entries of the wave's LA * RPI tile rows of unit t
  // go straight into LDS (one 4-byte load per lane, nothing waits for it), and the loader turns
  // them into lane offsets when it enters the unit, by which time they have landed: every
  // vector-memory operation of a wave retires in issue order, and the k-loop has by then waited
  // for tiles requested after them (rows_landed below).
  int* const rm_area = reinterpret_cast<int*>(smem + SMEM_BYTES) + wave * 64;
  auto request_rows = [&](const Unit& t) {
    const int r = wave * (LA * RPI) + lane % (LA * RPI);
    dma4_s((uint32_t)(t.row0 + min(r, t.rows - 1)) * 4u, p.row_map, lds_addr(rm_area));
  };

  // ---- the loader: requests k-tiles in the order the k-loops consume them, NS-1 tiles ahead.
  // Its position is two wave-uniform pointers (A rows and weights at the current k) that advance
  // by a constant per k-tile, plus the lanes' offsets of the unit it is in.  At the end of a unit
  // it moves on to the next unit if that is known by then (the k-loop then never waits for the
  // first tiles of a unit); otherwise it stays on a tile of the finished unit (requests that land
  // in free stages) until the epilogue points it at the next unit.
  const char* ld_a = nullptr;
  const char* ld_b = nullptr;
  int64_t ld_a_base = 0, ld_b_base = 0;
  uint32_t ld_voff_a[LA];
  int ld_rem = 0, ld_seg = 0;
  bool ld_on_next = false, ld_idle = false;
  auto ld_point = [&](int seg) {
    ld_a = uniform_ptr(reinterpret_cast<const char*>(seg ? p.A1 : p.A0) + ld_a_base);
    const bf16_t* B = (EPI == EPI_SWIGLU) ? ((wave & 1) ? p.B1 : p.B0) : (seg ? p.B1 : p.B0);
    ld_b = uniform_ptr(reinterpret_cast<const char*>(B) + ld_b_base);
    ld_seg = seg;
    ld_rem = kt_per_seg;
  };
  auto ld_take = [&](const Unit& t) {
    ld_a_base = t.a_base;
    ld_b_base = t.b_base;
    if (p.row_map) {
#pragma unroll
      for (int i = 0; i < LA; ++i)
        ld_voff_a[i] = (uint32_t)fastdiv(rm_area[i * RPI + lane / CPR], p.map_div) * row_bytes + a_kofs[i];
    } else {
#pragma unroll
      for (int i = 0; i < LA; ++i) ld_voff_a[i] = t.voff_a[i];
    }
    ld_idle = false;
    ld_point(0);
  };
  uint32_t ld_lds_a = 0, ld_lds_b = 0;     // LDS destinations of this wave's pieces in the stage being filled
  auto ld_target = [&](int stage) {
    ld_lds_a = lds_addr(smem) + stage * STAGE + wave * (LA * 1024);
    ld_lds_b = lds_addr(smem) + stage * STAGE + A_BYTES + wave * (LB * 1024);
  };
  auto issue_piece = [&](auto piece_c) {
    constexpr int P = decltype(piece_c)::value;
    if constexpr (P < LA) dma16_s<P * 1024>(ld_voff_a[P], ld_a, ld_lds_a);
    else dma16_s<(P - LA) * 1024>(voffB[P - LA], ld_b, ld_lds_b);
  };
  Unit cur_u, nxt_u;
  bool next_known = false;
  // after the L loads of a k-tile slot
  auto ld_advance = [&]() {
    ld_a += step_a;
    ld_b += step_b;
    if (--ld_rem == 0) {
      if (!ld_idle && ld_seg + 1 < p.nseg) {
        ld_point(ld_seg + 1);
      } else if (!ld_idle && next_known && !ld_on_next) {
        ld_on_next = true;
        ld_take(nxt_u);
      } else {           // nothing to request: the first tile of the same unit, again and again
        ld_idle = true;
        ld_point(0);
        ld_rem = 1;
      }
    }
  };
  // one k-tile slot outside the MFMA loop
  auto issue_slot = [&](int stage) {
    ld_target(stage);
    static_for<L>([&](auto pc) { issue_piece(pc); });
    ld_advance();
  };
  // the first k-tiles of the unit the loader points at, into the stages from `first` on
  auto issue_prologue = [&](int first) {
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) issue_slot(first + s >= NS ? first + s - NS : first + s);
  };

  int st_after = 0;     // stores this wave issued after its latest prefetch
  setup(cur_u, unit);
  nxt_u = cur_u;
  int cur = 0;          // ring stage of k-tile 0 of the current unit
  if (p.row_map) {
    request_rows(cur_u);
    wait_dma<0>();
  }
  ld_take(cur_u);
  issue_prologue(0);
  // the grab index of the second unit: its round trip runs next to the first tiles' (the wait in
  // it covers both)
  if (tid == 0) grab = sched_grab(p.sched, xcd, sched_base);
  // The loader may enter the next unit inside the k-loop only once that unit's row map entries
  // have landed.  They are requested before the k-loop; the wait at the end of k-tile NS-2 leaves
  // at most (NS-2)*L younger operations in flight, fewer than were issued after them by then; the
  // loader enters the next unit during k-tile nkt-NS.
  const bool rows_landed = !p.row_map || nkt - NS >= NS - 1;

  for (;;) {
    int unit_next = -1;
    next_known = false;
    ld_on_next = false;
    const bool wave_has_rows = wm * WTM < cur_u.rows;   // waves whose row slice is empty skip the math

    floatx16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // the unit after this one: one lane works it out from the ticket taken during the previous
    // unit and leaves it in LDS; everyone reads it behind the barrier below and resolves the
    // unit's addresses (row map lookups included) before the k-loop, which then holds no
    // bookkeeping besides the loader's
    if (tid == 0) lds_publish(&sched_box[par ^ 1], sched_resolve(p.sched, xcd, grab, ui.total, sched_base));
    // k-tile 0 has landed once only younger operations are in flight: the younger k-tiles and
    // the stores that the previous epilogue issued after its prefetch
    wait_vm_le((NS - 2) * L + st_after);
    block_barrier();
    unit_next = __builtin_amdgcn_readfirstlane(sched_box[par ^ 1]);
    if (unit_next >= 0) {
      setup(nxt_u, unit_next);
      if (p.row_map) {
        request_rows(nxt_u);
        st_after += 1;      // one more operation younger than this unit's first tiles
      }
    }
    next_known = unit_next >= 0 && rows_landed;
    if constexpr (PP) {
      // Two groups of four waves, one wave of each group on every SIMD, half a k-tile apart: while
      // one group multiplies a k-tile out of registers (16 MFMAs back to back, nothing else), the
      // other reads the fragments of its next k-tile from LDS, requests a later k-tile from memory
      // and does the loader's bookkeeping; a barrier, and they swap.  The matrix pipe of a SIMD
      // then always has one wave feeding it, and that wave neither waits for LDS nor shares the
      // instruction issue with its own address arithmetic.
      //   group 0:  M0 | C0 | M1 | C1 | ...        (M: memory phase, C: compute phase, | barrier)
      //   group 1:   . | M0 | C0 | M1 | ...
      // Tile t is read from LDS by group 0 in phase 2t and by group 1 in phase 2t+1; the loads of
      // tile t+NS-1 go into the stage of tile t-1, which both groups have finished reading when
      // either of them requests it (a memory phase ends with its LDS reads complete).  A wave's
      // own loads of tile t+1 have landed when the phase before 2t+2 ends: group 0 waits for them
      // at the end of C_t, group 1 at the end of M_t.
      constexpr int KS = BK / 16;
      Frags<TM, TN> fr[KS];
      const int grp = wave / (NW / 2);
      if (grp == 1) block_barrier();
      for (int kt = 0; kt < nkt; ++kt) {
        // ---- memory phase
        ld_target(cur + NS - 1 >= NS ? cur - 1 : cur + NS - 1);   // the stage of k-tile kt-1 takes k-tile kt+NS-1
        const char* st = smem + cur * STAGE;
        if (wave_has_rows) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            load_frags<BK, TM, TN, !A_T, B_KC, BM, BN>(fr[ks], st, st + A_BYTES, wm * WTM, wn * WTN, ks, lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        static_for<L>([&](auto pc) { issue_piece(pc); });
        ld_advance();
        cur = cur + 1 == NS ? 0 : cur + 1;
        // a wave's own part of tile kt+1 must have landed when the phase before its first read
        // ends: younger than it are the NS-2 tiles after it and, while tile kt+1 is one of those
        // requested before the previous epilogue's stores, these stores
        auto wait_next_tile = [&]() {
          if (kt <= NS - 3) wait_vm_le((NS - 2) * L + st_after);
          else wait_dma<(NS - 2) * L>();
        };
        if (grp == 1) wait_next_tile();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        block_barrier();
        // ---- compute phase
        if (wave_has_rows) {
          __builtin_amdgcn_s_setprio(1);
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
              for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[ks].b[j], fr[ks].a[i], acc[i][j], 0, 0, 0);
          __builtin_amdgcn_s_setprio(0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (grp == 0) wait_next_tile();
        block_barrier();
      }
      if (grp == 0) block_barrier();   // the whole ring is free: every fragment is in registers or used
    } else {
      Frags<TM, TN> f0;     // fragments of the first k-step of the coming k-tile, read one tile ahead
      if (wave_has_rows)
        load_frags<BK, TM, TN, !A_T, B_KC, BM, BN>(f0, smem + cur * STAGE, smem + cur * STAGE + A_BYTES, wm * WTM, wn * WTN, 0, lane);

      // k-tile kt+1 has to be in LDS before the MFMAs of k-tile kt: its first fragments are read
      // while they run, so that no wave waits for LDS behind the barrier of the next tile
      // (NS-1+kt tiles have been requested; all but the NS-3 youngest must be there)
      wait_vm_le((NS - 3) * L + st_after);
      block_barrier();
      for (int kt = 0;;) {
        ld_target(cur + NS - 1 >= NS ? cur - 1 : cur + NS - 1);   // the stage of k-tile kt-1 takes k-tile kt+NS-1
        const char* st = smem + cur * STAGE;
        const char* stn = smem + (cur + 1 == NS ? 0 : cur + 1) * STAGE;
        if (wave_has_rows) {
          mma_ktile<BK, TM, TN, !A_T, B_KC, BM, BN, L>(st, st + A_BYTES, stn, stn + A_BYTES, wm * WTM, wn * WTN, f0, acc,
                                                       [&](auto pc) {
                                                         issue_piece(pc);
                                                         if constexpr (decltype(pc)::value == L - 1) ld_advance();
                                                       });
        } else {
          static_for<L>([&](auto pc) { issue_piece(pc); });
          ld_advance();
        }
        cur = cur + 1 == NS ? 0 : cur + 1;
        if (++kt == nkt) break;
        wait_dma<(NS - 3) * L>();
        block_barrier();   // everyone's part of tile kt+1 is in LDS; everyone is done reading tile kt-1
      }
      block_barrier();   // every wave has finished its fragment reads: the whole ring is free
    }
    const bool chained = ld_on_next;   // the loader is NS-1 tiles into the next unit already
    const bool has_next = unit_next >= 0;
    // nothing is in flight here, so taking the ticket of the unit after the next one costs
    // one round trip on one wave, not a drain of stores
    if (has_next && tid == 0) grab = sched_grab(p.sched, xcd, sched_base);

    // the next unit's first k-tiles, unless the k-loop has requested them already (then every
    // store of this epilogue is younger than they are)
    if (chained) st_after = 0;
    auto prefetch_next = [&]() {
      if (chained) return;
      st_after = 0;
      if (has_next) {
        if (!rows_landed) wait_dma<0>();     // a k-loop too short to have covered the row map entries
        ld_on_next = true;
        ld_take(nxt_u);
        issue_prologue(cur);
      }
    };
    if (!BWD) prefetch_next();

    // ---- epilogue, 32 rows of the wave tile at a time through the wave's staging buffer
    char* const sbuf = staging_area(cur) + wave * St::BYTES;
    int lane_e = lane;      // opaque: the epilogue's per-lane addresses are formed per unit (see Stage32::flush)
    asm volatile("" : "+v"(lane_e));
    const int lrow = lane_e & 31, lq = 4 * (lane_e >> 5);
    const int64_t grow0 = (int64_t)(cur_u.row0 + wm * WTM) * p.ldc;
    const int64_t gcol0 = (int64_t)cur_u.nt * BN_OUT + wn * OUT_COLS;
    // SwiGLU backward: the epilogue reads g and u (and, scaled, the row's combine score through the
    // row map).  Each of these is a round trip to HBM, so they are requested in batches: all scores
    // first, then the vectors of JB column tiles of a 32-row chunk at once (a whole chunk where the
    // registers allow it).  One vector at a time, as the compiler orders the loop below on its
    // own, costs a wave about 2,000 cycles per vector: a quarter of a 128-row unit's time at 4,096
    // tokens.
    constexpr bool LEAN_BWD = BWD && TM > 2;
    constexpr int JB = !BWD ? 1 : (TM <= 2 || LEAN_BWD ? TN : 1);     // column tiles per batch
    u32x2_t graw[JB][4], uraw[JB][4];
    float sc_chunk[BWD ? TM : 1];
    auto load_gu = [&](int i, int j0) {
      const int crows = min(32, cur_u.rows - wm * WTM - 32 * i);
      if (crows <= 0) return;
      const int rr = lrow < crows ? lrow : crows - 1;
      const int64_t goff = grow0 + (int64_t)(32 * i) * p.ldc + gcol0 + (int64_t)rr * p.ldc + lq;
#pragma unroll
      for (int j = 0; j < JB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          graw[j][q] = *reinterpret_cast<const u32x2_t*>(p.Gin + goff + 32 * (j0 + j) + 8 * q);
          uraw[j][q] = *reinterpret_cast<const u32x2_t*>(p.Uin + goff + 32 * (j0 + j) + 8 * q);
        }
    };
    if constexpr (BWD) {
      if constexpr (SCALED) {
        int slot[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int crows = min(32, cur_u.rows - wm * WTM - 32 * i);
          const int rr = lrow < crows ? lrow : (crows > 0 ? crows - 1 : 0);
          slot[i] = crows > 0 ? p.row_map[cur_u.row0 + wm * WTM + 32 * i + rr] : 0;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) sc_chunk[i] = p.scores[slot[i]];
        // Every score counts as used here, also those of chunks past the unit's last row, which
        // nothing reads: a load still pending on some path at the end of the epilogue makes the
        // compiler wait for ALL vector memory operations where its register is next written, and
        // that is inside the next unit's k-loop, where such a wait drains the ring of operand loads.
#pragma unroll
        for (int i = 0; i < TM; ++i) asm volatile("" :: "v"(sc_chunk[i]));
      } else {
#pragma unroll
        for (int i = 0; i < TM; ++i) sc_chunk[i] = 1.f;
      }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int crows = min(32, cur_u.rows - wm * WTM - 32 * i);   // valid rows of this chunk
      const int64_t goff = grow0 + (int64_t)(32 * i) * p.ldc + gcol0;
      if (EPI == EPI_SWIGLU) {
#pragma unroll
        for (int which = 0; which < 3; ++which) {
          if (crows > 0) {
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
                  v = pack4((g[0] * sigmoid_fast(g[0])) * u[0], (g[1] * sigmoid_fast(g[1])) * u[1],
                            (g[2] * sigmoid_fast(g[2])) * u[2], (g[3] * sigmoid_fast(g[3])) * u[3]);
                }
                St::put(sbuf, lrow, 16 * j + 8 * q + lq, v);
              }
            wave_lds_fence();
            st_after += St::template flush<false>(sbuf, (which == 0 ? p.O0 : which == 1 ? p.O1 : p.O2) + goff, p.ldc, crows);
            wave_lds_fence();
          }
        }
      } else if (EPI == EPI_PLAIN) {
        if (crows > 0) {
          constexpr int JS = SW / 32;      // column tiles staged together
#pragma unroll
          for (int j0 = 0; j0 < TN; j0 += JS) {
#pragma unroll
            for (int j = j0; j < j0 + JS; ++j)
#pragma unroll
              for (int q = 0; q < 4; ++q)
                St::put(sbuf, lrow, 32 * (j - j0) + 8 * q + lq,
                        pack4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]));
            wave_lds_fence();
            st_after += St::template flush<false>(sbuf, p.O0 + goff + 32 * j0, p.ldc, crows);
            wave_lds_fence();
          }
        }
      } else if constexpr (LEAN_BWD) {
        // EPI_SWIGLU_BWD[_SCALED] with 128 accumulator registers: the packed outputs of 32 columns
        // at a time, d_g and d_u side by side in the staging buffer, score * h after them
        using S2 = Stage32<32>;
        static_assert(2 * S2::BYTES <= St::BYTES, "two 32-column areas in a wave's staging buffer");
        char* const sb0 = sbuf;
        char* const sb1 = sbuf + S2::BYTES;
        float ds = 0.f;
        if (crows > 0) {
          const float sc = sc_chunk[i];
          load_gu(i, 0);
          __builtin_amdgcn_sched_barrier(0);
          // the loads must have returned before the next unit's first tiles are requested: a load
          // behind those requests would wait for all of them
          const bool transposed = SCALED && p.T0 != nullptr;
          const bool live = lrow < crows;      // the transposed copies want zeros in the rows past the end
          const u32x2_t zero2 = {0u, 0u};
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            u32x2_t hsv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              float dh[4], g[4], u[4], og[4], ou[4], oh[4];
              unpack4(pack4(sc * acc[i][j][4 * q], sc * acc[i][j][4 * q + 1], sc * acc[i][j][4 * q + 2], sc * acc[i][j][4 * q + 3]), dh);
              unpack4(graw[j][q], g);
              unpack4(uraw[j][q], u);
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                const float sg = sigmoid_fast(g[t]);
                og[t] = dh[t] * u[t] * (sg * (1.f + g[t] * (1.f - sg)));
                ou[t] = dh[t] * (g[t] * sg);
                if (SCALED) {
                  const float hv = (g[t] * sg) * u[t];
                  ds += acc[i][j][4 * q + t] * hv;
                  oh[t] = sc * hv;
                }
              }
              const bool dead = transposed && !live;
              S2::put(sb0, lrow, 8 * q + lq, dead ? zero2 : pack4(og[0], og[1], og[2], og[3]));
              S2::put(sb1, lrow, 8 * q + lq, dead ? zero2 : pack4(ou[0], ou[1], ou[2], ou[3]));
              if (SCALED) hsv[q] = dead ? zero2 : pack4(oh[0], oh[1], oh[2], oh[3]);
            }
            if (j == TN - 1 && i == TM - 1) {
              __builtin_amdgcn_sched_barrier(0);
              prefetch_next();
            }
            const int64_t tofs = ((int64_t)((cur_u.tcol + wm * WTM + 32 * i) >> 5) * p.ldc + gcol0 + 32 * j) * 32;
            wave_lds_fence();
            st_after += S2::template flush<false>(sb0, p.O0 + goff + 32 * j, p.ldc, crows, lane_e);
            st_after += S2::template flush<false>(sb1, p.O1 + goff + 32 * j, p.ldc, crows, lane_e);
            if constexpr (SCALED) {
              if (transposed) {
                st_after += S2::flush_t(sb0, p.T0 + tofs, 32, crows, lane_e);
                st_after += S2::flush_t(sb1, p.T1 + tofs, 32, crows, lane_e);
              }
            }
            wave_lds_fence();
            if constexpr (SCALED) {
              if (p.O2 || transposed) {
#pragma unroll
                for (int q = 0; q < 4; ++q) S2::put(sb0, lrow, 8 * q + lq, hsv[q]);
                wave_lds_fence();
                if (p.O2) st_after += S2::template flush<false>(sb0, p.O2 + goff + 32 * j, p.ldc, crows, lane_e);
                if (transposed) st_after += S2::flush_t(sb0, p.T2 + tofs, 32, crows, lane_e);
                wave_lds_fence();
              }
            }
          }
          if (SCALED) {
            // lanes l and l+32 hold the two column halves of row l % 32
            ds += __shfl_xor(ds, 32);
            if (lane_e < 32 && lrow < crows)
              p.ds_partial[(int64_t)((cur_u.nt * BN + wn * WTN) >> 6) * p.total_rows + cur_u.row0 + wm * WTM + 32 * i + lrow] = ds;
            st_after += 1;
          }
        } else if (i == TM - 1) {
          prefetch_next();
        }
      } else {   // EPI_SWIGLU_BWD[_SCALED]: acc = d_h; d_g = d_h * u * silu'(g), d_u = d_h * silu(g)
        u32x2_t dg[TN][4], du[TN][4], hs[SCALED ? TN : 1][4];
        float ds = 0.f;
        if (crows > 0) {
          const float sc = sc_chunk[i];
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            if (j % JB == 0) {
              load_gu(i, j);
              __builtin_amdgcn_sched_barrier(0);    // keep the batch together, ahead of the arithmetic
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              float dh[4], g[4], u[4], og[4], ou[4], oh[4];
              // d_h is rounded to bf16 first, like the output of the reference's batched matmul
              unpack4(pack4(sc * acc[i][j][4 * q], sc * acc[i][j][4 * q + 1], sc * acc[i][j][4 * q + 2], sc * acc[i][j][4 * q + 3]), dh);
              unpack4(graw[j % JB][q], g);
              unpack4(uraw[j % JB][q], u);
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                const float sg = sigmoid_fast(g[t]);
                og[t] = dh[t] * u[t] * (sg * (1.f + g[t] * (1.f - sg)));
                ou[t] = dh[t] * (g[t] * sg);
                if (SCALED) {
                  const float hv = (g[t] * sg) * u[t];
                  ds += acc[i][j][4 * q + t] * hv;
                  oh[t] = sc * hv;
                }
              }
              dg[j][q] = pack4(og[0], og[1], og[2], og[3]);
              du[j][q] = pack4(ou[0], ou[1], ou[2], ou[3]);
              if (SCALED) hs[j][q] = pack4(oh[0], oh[1], oh[2], oh[3]);
            }
          }
        }
        // the loads above must have returned first: a load behind the prefetch waits for all of it
        __builtin_amdgcn_sched_barrier(0);
        if (i == TM - 1) prefetch_next();
        if (crows > 0) {
          if (SCALED) {
            // lanes l and l+32 hold the two column halves of row l % 32
            ds += __shfl_xor(ds, 32);
            if (lane < 32 && lrow < crows)
              p.ds_partial[(int64_t)((cur_u.nt * BN + wn * WTN) >> 6) * p.total_rows + cur_u.row0 + wm * WTM + 32 * i + lrow] = ds;
            st_after += 1;
          }
          const bool transposed = SCALED && p.T0 != nullptr;
          const bool live = lrow < crows;      // the transposed copies want zeros in the rows past the end
          const u32x2_t zero2 = {0u, 0u};
#pragma unroll
          for (int which = 0; which < (SCALED ? 3 : 2); ++which) {
            bf16_t* const out = which == 0 ? p.O0 : which == 1 ? p.O1 : p.O2;
            if (which == 2 && !out && !transposed) continue;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const u32x2_t v = which == 0 ? dg[j][q] : which == 1 ? du[j][q] : hs[SCALED ? j : 0][q];
                St::put(sbuf, lrow, 32 * j + 8 * q + lq, (transposed && !live) ? zero2 : v);
              }
            wave_lds_fence();
            if (out) st_after += St::template flush<false>(sbuf, out + goff, p.ldc, crows);
            if constexpr (SCALED) {
              if (transposed)
                st_after += St::flush_t(sbuf, (which == 0 ? p.T0 : which == 1 ? p.T1 : p.T2) +
                                                  ((int64_t)((cur_u.tcol + wm * WTM + 32 * i) >> 5) * p.ldc + gcol0) * 32,
                                        32, crows);
            }
            wave_lds_fence();
          }
        }
      }
    }
    if (!has_next) break;
    cur_u = nxt_u;
    unit = unit_next;
    par ^= 1;
  }
  wait_dma<0>();   // the zero loads of the last k-tiles must not land in LDS that a later workgroup owns
  if (tid == 0) sched_finish(p.sched);
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
  FastDiv map_div;
  int32_t accumulate;
  int32_t tiles_per_expert;  // (M/BM)*(N/BN), identical for the three problems
  int32_t nprob;
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

  const int nprob = p.nprob;
  // Workgroup b runs on XCD b % 8.  All tiles of one expert stay on one XCD, back to back, so its
  // rows are read from HBM once.  Experts are dealt to the XCDs in "snake" order (0..7, 7..0,
  // 0..7, ...) of p.order, the experts sorted by descending row count (pk_sort_by_expert), which
  // balances skewed routing; without an order they are dealt by index.
  const const_i32_ptr starts = as_const(p.starts);
  const int xcd = blockIdx.x % NXCD, pos = blockIdx.x / NXCD;
  // the problems of one expert follow each other on its XCD: d_w1 and d_w3 read the same x rows
  const int per_expert = p.tiles_per_expert * nprob;
  const int jq = pos / per_expert;                               // position in this XCD's queue
  const int rem = pos % per_expert;
  const WgradProblem& q = p.prob[rem / p.tiles_per_expert];
  const int t = rem % p.tiles_per_expert;
  const int want = (jq & 1) ? jq * NXCD + (NXCD - 1 - xcd) : jq * NXCD + xcd;   // rank to serve
  if (want >= p.E) return;
  const int e = p.order ? as_const(p.order)[want] : want;
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
  const FastDiv map_div = p.map_div;

  // Source rows of the k-tile that is issued next (wave-uniform, -1 past the expert's end).  They
  // are fetched one tile ahead, so the scalar loads of the row map run under the previous tile's
  // MFMAs instead of in front of the loads.
  constexpr int NA = LA * A_RPI, NB = LB * B_RPI;
  int arow[NA], brow[NB];
  auto fetch_rows = [&](int kt) {
    const int k0 = row_begin + kt * BK;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int row = k0 + wave * NA + i;     // piece i / A_RPI of this wave, row i % A_RPI of the piece
      int v = -1;
      if (row < row_end) v = a_map ? fastdiv(a_map[row], map_div) : row;
      arow[i] = v;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int row = k0 + wave * NB + i;
      int v = -1;
      if (row < row_end) v = b_map ? fastdiv(b_map[row], map_div) : row;
      brow[i] = v;
    }
  };
  uint32_t is_a = 0, is_b = 0;     // LDS destinations of this wave's pieces in the stage being filled
  bool is_real = true;             // false: no tile left, the pieces read zeros (rows are not looked up)
  auto issue_setup = [&](int stage) {
    char* st = smem + stage * STAGE;
    is_a = lds_addr(st) + (wave * LA) * 1024;
    is_b = lds_addr(st + A_BYTES) + (wave * LB) * 1024;
  };
  // piece 0..LA-1: A, LA..LA+LB-1: B (rows as fetched by fetch_rows)
  auto issue_piece = [&](int piece) {
    if (piece < LA) {
      const int i = piece;
      int krow, cofs;
      mn_slot<BM>(wave * LA + i, lane, krow, cofs);
      const void* src = g_zero16;
#pragma unroll
      for (int r = 0; r < A_RPI; ++r) {
        const int v = arow[i * A_RPI + r];
        if (is_real && v >= 0) {
          const bf16_t* cand = Abase + (int64_t)v * lda;
          if (lane / A_CPR == r) src = cand + cofs;
        }
      }
      dma16(src, is_a + i * 1024);
    } else {
      const int i = piece - LA;
      int krow, cofs;
      mn_slot<BN>(wave * LB + i, lane, krow, cofs);
      const void* src = g_zero16;
#pragma unroll
      for (int r = 0; r < B_RPI; ++r) {
        const int v = brow[i * B_RPI + r];
        if (is_real && v >= 0) {
          const bf16_t* cand = Bbase + (int64_t)v * ldb;
          if (lane / B_CPR == r) src = cand + cofs;
        }
      }
      dma16(src, is_b + i * 1024);
    }
  };
  auto issue = [&](int stage) {
    issue_setup(stage);
#pragma unroll
    for (int piece = 0; piece < LA + LB; ++piece) issue_piece(piece);
  };

  floatx16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  if constexpr (NS >= 3) {
    // every slot issues its loads (rows past the expert's end read a block of zeros), so the
    // number of loads in flight is the same at every k-tile
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) {
      is_real = s < nkt;
      if (is_real) fetch_rows(s);
      issue(s);
    }
    if (NS - 1 < nkt) fetch_rows(NS - 1);
  } else {
#pragma unroll
    for (int s = 0; s < NS - 1; ++s)
      if (s < nkt) {
        fetch_rows(s);
        issue(s);
      }
    if (NS - 1 < nkt) fetch_rows(NS - 1);
  }
  int cur = 0, nxt = NS - 1;
  if constexpr (NS >= 3) {
    // Rings of three or more stages: the loads of tile kt+NS-1 and the fragment reads of the
    // next k-step are spread between the MFMAs, and the first fragments of tile kt+1 are read
    // during tile kt (the barrier at the top of tile kt waits for tile kt+1).
    constexpr int L = LA + LB;
    wait_dma<(NS - 2) * L>();
    block_barrier();
    Frags<TM, TN> f0;
    load_frags<BK, TM, TN, false, false, BM, BN>(f0, smem, smem + A_BYTES, wm * WTM, wn * WTN, 0, lane);
    for (int kt = 0; kt < nkt; ++kt) {
      wait_dma<(NS - 3) * L>();
      block_barrier();
      issue_setup(nxt);
      is_real = kt + NS - 1 < nkt;
      const char* st = smem + cur * STAGE;
      const char* stn = smem + (cur + 1 == NS ? 0 : cur + 1) * STAGE;
      mma_ktile<BK, TM, TN, false, false, BM, BN, L>(st, st + A_BYTES, stn, stn + A_BYTES, wm * WTM, wn * WTN,
                                                     f0, acc, [&](int piece) { issue_piece(piece); });
      if (kt + NS < nkt) fetch_rows(kt + NS);
      cur = cur + 1 == NS ? 0 : cur + 1;
      nxt = nxt + 1 == NS ? 0 : nxt + 1;
    }
    wait_dma<0>();   // zero loads of the last k-tiles: the staging below reuses the ring
  } else {
    for (int kt = 0; kt < nkt; ++kt) {
      if (kt + NS - 2 < nkt) wait_dma<(NS - 2) * (LA + LB)>(); else wait_dma<0>();
      block_barrier();
      if (kt + NS - 1 < nkt) issue(nxt);
      if (kt + NS < nkt) fetch_rows(kt + NS);
      const char* st = smem + cur * STAGE;
      mma_tile<BK, TM, TN, false, false, BM, BN, (TM * TN >= 16)>(st, st + A_BYTES, wm * WTM, wn * WTN, acc);
      cur = cur + 1 == NS ? 0 : cur + 1;
      nxt = nxt + 1 == NS ? 0 : nxt + 1;
    }
  }

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

// ---- weight gradient with one K-contiguous operand, persistent workgroups.
// C[e][M,N] (+)= sum over the rows r of expert e of  m-side[r, m] * n-side[r, n], where one side comes
// from a transposed copy ("T": blocks of 32 padded rows, [ldt / 32][width][32], expert e at padded
// row padded_start(e), written by the scaled SwiGLU backward) and the other side from rows gathered
// through the row map ("R": x or d_out).  Against wgrad_kernel: the T operand is read with
// ds_read_b128 instead of the transposing read (the LDS read rate bounds a k-loop whose operands
// both need it) and the workgroups are persistent.  A_KC: T is the m side (d_w1 = d_g^T x,
// d_w3 = d_u^T x); otherwise T is the n side (d_w2 = d_out^T (score h)).  The wave grid puts the
// wider wave-tile side on T.
struct WgradKcProblem {
  const bf16_t* T;
  const bf16_t* R;
  bf16_t* C;
};
struct WgradKcParams {
  WgradKcProblem prob[2];
  int64_t ldt, ldr;
  const int32_t* row_map;    // sorted row -> flat slot; R row = slot / map_div
  FastDiv map_div;
  const int32_t* starts;
  const int32_t* order;      // optional [E]: experts by descending row count
  int32_t E, nprob;
  int32_t M, N;              // output per expert (multiples of the block tile)
  int32_t total_rows;        // A: entries of the row map
  int32_t accumulate;
  SchedSlot* sched;
};

// The kernel: 256x256x32 tiles, 8 waves, 4-stage ring, the ping-pong k-loop of ragged_m_kernel.
//  * The two waves of a SIMD belong to two groups half a k-tile apart: one reads the fragments of a
//    whole k-tile from LDS and requests a later k-tile while the other issues its MFMAs back to
//    back, with the loader's scalar bookkeeping in the issue slots between the first of them.
//  * The loader's position is scalar: a pointer into the transposed copy that advances by one
//    32-row block per k-tile (16 KB of consecutive memory per tile, no masking: the producer writes
//    zeros in an expert's rows up to the end of its last block), the base of the gathered operand,
//    and an index into the row map; a load is the scalar-base + 32-bit-lane-offset form.  The row
//    map entries of the slot after the one being requested are fetched with one 16-byte scalar
//    load per wave and picked up, per lane, one k-tile later.
//  * Rows of the gathered operand past the expert's end read whatever row the map holds next (a
//    valid, finite row): they meet the zeros of the transposed copy.
//  * One lane resolves the unit after the next one -- ticket, expert, row range -- behind its
//    epilogue's stores and hands it over through LDS at the top of the next unit, so no wave waits
//    for a chain of scalar loads between two k-loops.
//  * A workgroup requests the first k-tiles of its next unit before the epilogue of the current one
//    (or, when the next unit is known in time, as the last requests of the k-loop), and its
//    stores do not hold up the next unit's loads.
template <int WMW, int WNW, bool A_KC, bool DYNAMIC, bool ACCUMULATE>
__global__ __launch_bounds__(64 * WMW * WNW) void wgrad_pp_kernel(const WgradKcParams p) {
  constexpr int BM = 256, BN = 256, BK = 32, NS = 4;
  constexpr bool B_KC = !A_KC;
  constexpr int NW = WMW * WNW, NTHREADS = 64 * NW;
  static_assert(NW == 8, "two groups of four waves");
  constexpr int WTM = BM / WMW, WTN = BN / WNW, TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2, STAGE = A_BYTES + B_BYTES;
  constexpr int KC_ROWS = A_KC ? BM : BN, MN_COLS = A_KC ? BN : BM;
  constexpr int KC_OFF = A_KC ? 0 : A_BYTES, MN_OFF = A_KC ? A_BYTES : 0;
  constexpr int LKC = KC_ROWS * BK * 2 / (NTHREADS * 16), LMN = MN_COLS * BK * 2 / (NTHREADS * 16), L = LKC + LMN;
  constexpr int MN_CPR = MN_COLS / 8, MN_RPI = 64 / MN_CPR, NR = LMN * MN_RPI;
  static_assert(MN_RPI == 2, "a load of the gathered operand covers two rows, one per half wave");
  static_assert(WTN % 64 == 0, "the epilogue stages 64 columns at a time");
  using St = Stage32<64>;
  constexpr int RING = NS * STAGE;
  static_assert(RING + NW * St::BYTES <= 160 * 1024, "LDS budget");
  __shared__ __attribute__((aligned(1024))) char smem[RING + NW * St::BYTES];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WNW, wn = wave % WNW;
  char* const sbuf = smem + RING + wave * St::BYTES;
  const const_i32_ptr starts = as_const(p.starts);
  const const_i32_ptr row_map = as_const(p.row_map);
  const const_i32_ptr order = as_const(p.order);
  const int n_tiles = p.N / BN;
  const int tiles = (p.M / BM) * n_tiles;
  const int per_expert = tiles * p.nprob;
  const int total = p.E * per_expert;
  const int t_width = A_KC ? p.M : p.N;            // rows of a block of the transposed copy
  const uint32_t step_kc = (uint32_t)t_width * 64u;  // bytes from one 32-row block to the next
  const uint32_t ldr_bytes = (uint32_t)p.ldr * 2u;

  // ---- which units this workgroup runs: from the per-XCD counters (DYNAMIC; balances the very
  // uneven experts of skewed routing) or statically, round r giving XCD x the units
  // [(r*8 + x) * G8, +G8), one per workgroup of that XCD, experts in descending row count
  // (p.order), so the units of a round cost about the same.  Either way lane 0 works out the
  // description of a unit (UnitDesc) well before the unit starts and hands it over through LDS:
  // two boxes in the first bytes of wave 0's staging buffer, which is idle between the end of
  // that wave's epilogue and the end of the next k-loop.
  struct UnitDesc { int unit, e, q, mt, nt, s0, s1, pad; };
  UnitDesc* const box = reinterpret_cast<UnitDesc*>(smem + RING);
  const int xcd = blockIdx.x % NXCD, G8 = gridDim.x / NXCD;
  auto unit_at = [&](int r) {
    const int u = (r * NXCD + xcd) * G8 + (int)(blockIdx.x / NXCD);
    return u < total ? u : -1;
  };
  // lane 0: the unit after the current one (plain scalars: a struct would live in scratch memory)
  int nx_unit = -1, nx_e = 0, nx_q = 0, nx_mt = 0, nx_nt = 0, nx_s0 = 0, nx_s1 = 0;
  auto describe = [&](int un) __attribute__((always_inline)) {
    un = __builtin_amdgcn_readfirstlane(un);     // one lane runs this: scalar arithmetic and scalar loads
    nx_unit = un;
    if (un < 0) return;
    const int rank = un / per_expert;
    const int rem = un - rank * per_expert;
    nx_q = rem / tiles;
    const int tt = rem - nx_q * tiles;
    nx_mt = tt / n_tiles;
    nx_nt = tt - nx_mt * n_tiles;
    nx_e = p.order ? order[rank] : rank;
    nx_s0 = starts[nx_e];
    nx_s1 = starts[nx_e + 1];
  };
  auto publish = [&](int which) __attribute__((always_inline)) {
    int* const b = reinterpret_cast<int*>(&box[which]);
    b[0] = nx_unit; b[1] = nx_e; b[2] = nx_q; b[3] = nx_mt; b[4] = nx_nt; b[5] = nx_s0; b[6] = nx_s1;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };
  unsigned grab = 0;
  const unsigned sched_base = 2 * G8;      // two units per workgroup are settled without the counters
  int par = 0, round = 0;
  if (tid == 0) {
    int first, second = -1;
    if constexpr (DYNAMIC) {
      first = sched_resolve(p.sched, xcd, blockIdx.x / NXCD, total, sched_base);
      if (first >= 0) second = sched_resolve(p.sched, xcd, blockIdx.x / NXCD + G8, total, sched_base);
    } else {
      first = unit_at(0);
      if (first >= 0) second = unit_at(1);
    }
    describe(first);
    publish(0);
    describe(second);
  }
  __syncthreads();

  struct Unit {
    int e, q, mt, nt;
    int s0, rows, nkt;
    const char* t_ptr;   // the transposed copy at the expert's first block, first tile row
    const char* r_ptr;   // the gathered operand at the tile's first column
  };
  auto take_box = [&](Unit& t, int which) -> int {
    const int* const b = reinterpret_cast<const int*>(&box[which]);
    const int un = __builtin_amdgcn_readfirstlane(b[0]);
    if (un < 0) return un;
    t.e = __builtin_amdgcn_readfirstlane(b[1]);
    t.q = __builtin_amdgcn_readfirstlane(b[2]);
    t.mt = __builtin_amdgcn_readfirstlane(b[3]);
    t.nt = __builtin_amdgcn_readfirstlane(b[4]);
    t.s0 = __builtin_amdgcn_readfirstlane(b[5]);
    t.rows = __builtin_amdgcn_readfirstlane(b[6]) - t.s0;
    t.nkt = (t.rows + BK - 1) / BK;
    const WgradKcProblem& q = p.prob[t.q];
    t.t_ptr = uniform_ptr(reinterpret_cast<const char*>(
        q.T + ((int64_t)(padded_start(t.s0, t.e) >> 5) * t_width + (A_KC ? t.mt * BM : t.nt * BN)) * 32));
    t.r_ptr = uniform_ptr(reinterpret_cast<const char*>(q.R + (A_KC ? t.nt * BN : t.mt * BM)));
    return un;
  };
  Unit cur_u, nxt_u;
  if (take_box(cur_u, 0) < 0) {
    if constexpr (DYNAMIC) {
      if (tid == 0) sched_finish(p.sched);
    }
    return;
  }
  nxt_u = cur_u;

  // ---- lane constants of the loaders: byte offsets of a lane's 16 bytes
  uint32_t voff_kc[LKC];      // inside a 32-row block of the transposed copy: (row * 32 + k) * 2
#pragma unroll
  for (int i = 0; i < LKC; ++i) {
    int r, k;
    kc_slot<BK>(wave * LKC + i, lane, r, k);
    voff_kc[i] = (uint32_t)(r * 32 + k) * 2u;
  }
  uint32_t mn_cofs[LMN];      // inside a gathered row
#pragma unroll
  for (int i = 0; i < LMN; ++i) {
    int krow, cofs;
    mn_slot<MN_COLS>(wave * LMN + i, lane, krow, cofs);
    mn_cofs[i] = (uint32_t)cofs * 2u;
  }
  const bool upper = lane >= 32;     // the second of the two rows of a gathered load

  // ---- the loader: requests k-tiles in the order the k-loops consume them, NS-1 tiles ahead, and
  // moves on to the next unit at the end of one if that unit is known by then; otherwise it
  // stays on the first tile of the unit it is in (requests that land in stages nobody reads)
  // until the epilogue points it at the next unit.  rows_n holds the row map entries of the slot
  // the loader points at.
  const char* ld_kc = nullptr;
  const char* ld_kc0 = nullptr;
  const char* ld_r = nullptr;
  int ld_map = 0, ld_map0 = 0, ld_rem = 0;
  bool ld_on_next = false, ld_idle = false, next_known = false;
  int rows_n[NR];
  static_assert(NR == 4, "a wave's rows of a k-tile are one 16-byte scalar load");
  typedef int i32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
  auto fetch_rows = [&]() {
    const int idx = ld_map + wave * NR;
    if (idx + NR <= p.total_rows) {
      const i32x4_a4 v = *reinterpret_cast<const __attribute__((address_space(4))) i32x4_a4*>(row_map + idx);
      rows_n[0] = v[0]; rows_n[1] = v[1]; rows_n[2] = v[2]; rows_n[3] = v[3];
    } else {      // the last entries of the row map
#pragma unroll
      for (int i = 0; i < NR; ++i) rows_n[i] = row_map[min(idx + i, p.total_rows - 1)];
    }
  };
  auto ld_enter = [&](const Unit& t) {
    ld_kc0 = t.t_ptr;
    ld_map0 = t.s0;
    ld_r = t.r_ptr;
    ld_kc = ld_kc0;
    ld_map = ld_map0;
    ld_rem = t.nkt;
    ld_idle = false;
    if (ld_rem == 0) { ld_idle = true; ld_rem = 1; }    // an expert without rows: nothing to request
  };
  auto ld_advance = [&]() {
    ld_kc += step_kc;
    ld_map += BK;
    if (--ld_rem == 0) {
      if (!ld_idle && next_known && !ld_on_next) {
        ld_on_next = true;
        ld_enter(nxt_u);
      } else {
        ld_idle = true;
        ld_kc = ld_kc0;
        ld_map = ld_map0;
        ld_rem = 1;
      }
    }
  };
  uint32_t lds_kc = 0, lds_mn = 0;
  auto ld_target = [&](int stage) {
    lds_kc = lds_addr(smem) + stage * STAGE + KC_OFF + wave * (LKC * 1024);
    lds_mn = lds_addr(smem) + stage * STAGE + MN_OFF + wave * (LMN * 1024);
  };
  // One slot is requested in two steps.  slot_issue: the lane offsets of the gathered rows come out
  // of rows_n and the L loads go out to the stage that ld_target named (`between` runs before the
  // loads: the k-loop reads its fragments there).  slot_advance: the loader moves on and asks for
  // the next slot's row map entries -- scalar work that the k-loop does between its MFMAs.
  auto slot_issue = [&](auto&& between) __attribute__((always_inline)) {
    uint32_t voff_mn[LMN];
#pragma unroll
    for (int i = 0; i < LMN; ++i) {
      const int slot = upper ? rows_n[i * MN_RPI + 1] : rows_n[i * MN_RPI];
      voff_mn[i] = (uint32_t)fastdiv(slot, p.map_div) * ldr_bytes + mn_cofs[i];
    }
    between();
    static_for<L>([&](auto pc) {
      constexpr int P = decltype(pc)::value;
      if constexpr (P < LKC) dma16_s<P * 1024>(voff_kc[P], ld_kc, lds_kc);
      else dma16_s<(P - LKC) * 1024>(voff_mn[P - LKC], ld_r, lds_mn);
    });
  };
  auto slot_advance = [&]() __attribute__((always_inline)) {
    ld_advance();
    fetch_rows();
  };
  auto issue_prologue = [&](int first) __attribute__((always_inline)) {
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) {
      ld_target(first + s >= NS ? first + s - NS : first + s);
      slot_issue([] {});
      slot_advance();
    }
  };

  int st_after = 0;     // stores this wave issued after its latest prefetch
  int cur = 0;          // ring stage of k-tile 0 of the current unit
  ld_enter(cur_u);
  fetch_rows();
  issue_prologue(0);
  if constexpr (DYNAMIC) {
    // the grab index of the third unit: its round trip runs next to the first tiles'
    if (tid == 0 && nx_unit >= 0) grab = sched_grab(p.sched, xcd, sched_base);
  }

  for (;;) {
    next_known = false;
    ld_on_next = false;
    const int nkt = cur_u.nkt;
    floatx16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    if (tid == 0) publish(par ^ 1);
    // k-tile 0 has landed once only younger operations are in flight: the younger k-tiles and
    // the stores that the previous epilogue issued after its prefetch
    wait_vm_le((NS - 2) * L + st_after);
    block_barrier();
    const int unit_next = take_box(nxt_u, par ^ 1);
    next_known = unit_next >= 0;
    {
      // group 0:  M0 | C0 | M1 | C1 | ...        (M: memory phase, C: compute phase, | barrier)
      // group 1:   . | M0 | C0 | M1 | ...
      // Tile t is read from LDS by group 0 in phase 2t and by group 1 in phase 2t+1; the loads of
      // tile t+NS-1 go into the stage of tile t-1, which both groups have finished reading when
      // either of them requests it (a memory phase ends with its LDS reads complete).  A wave's
      // own loads of tile t+1 have landed when the phase before 2t+2 ends: group 0 waits for them
      // at the end of C_t, group 1 at the end of M_t.
      constexpr int KS = BK / 16;
      Frags<TM, TN> fr[KS];
      const int grp = wave / (NW / 2);
      if (grp == 1) block_barrier();
      ld_target(cur == 0 ? NS - 1 : cur - 1);     // the stage of k-tile kt-1 takes k-tile kt+NS-1
      for (int kt = 0; kt < nkt; ++kt) {
        // ---- memory phase
        const char* st = smem + cur * STAGE;
        slot_issue([&] {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            load_frags<BK, TM, TN, A_KC, B_KC, BM, BN>(fr[ks], st, st + A_BYTES, wm * WTM, wn * WTN, ks, lane);
          __builtin_amdgcn_sched_barrier(0);
        });
        const int filled = cur;     // free once both groups have read it: the next slot's target
        cur = cur + 1 == NS ? 0 : cur + 1;
        auto wait_next_tile = [&]() {
          if (kt <= NS - 3) wait_vm_le((NS - 2) * L + st_after);
          else wait_dma<(NS - 2) * L>();
        };
        if (grp == 1) wait_next_tile();
        // every fragment counts as used here: the compiler then waits for the LDS reads in this
        // phase, not in front of the MFMAs, where a wait would also cover the scalar loads that
        // the bookkeeping between the MFMAs has just issued (LDS and scalar loads share a counter)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
          for (int i = 0; i < TM; ++i) asm volatile("" :: "v"(fr[ks].a[i]));
#pragma unroll
          for (int j = 0; j < TN; ++j) asm volatile("" :: "v"(fr[ks].b[j]));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        block_barrier();
        // ---- compute phase: the MFMAs back to back, the loader's scalar bookkeeping for the next
        // slot in the issue slots between the first of them
        __builtin_amdgcn_s_setprio(1);
        static_for<KS * TM * TN>([&](auto idx_c) {
          constexpr int idx = decltype(idx_c)::value;
          constexpr int ks = idx / (TM * TN), i = (idx % (TM * TN)) / TN, j = idx % TN;
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[ks].b[j], fr[ks].a[i], acc[i][j], 0, 0, 0);
          if constexpr (idx == 0) {
            __builtin_amdgcn_sched_barrier(0);
            slot_advance();
            ld_target(filled);
            __builtin_amdgcn_sched_barrier(0);
          }
        });
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        if (grp == 0) wait_next_tile();
        block_barrier();
      }
      if (grp == 0) block_barrier();   // the whole ring is free: every fragment is in registers or used
    }
    const bool chained = ld_on_next;   // the loader is NS-1 tiles into the next unit already
    const bool has_next = unit_next >= 0;
    // lane 0: the unit after the next one.  Its expert and row range are scalar loads that return
    // while this lane's wave stores its tile; they are handed over at the top of the next unit.
    if (has_next && tid == 0) {
      int un2;
      if constexpr (DYNAMIC) {
        un2 = sched_resolve(p.sched, xcd, grab, total, sched_base);
        if (un2 >= 0) grab = sched_grab(p.sched, xcd, sched_base);
      } else {
        un2 = unit_at(round + 2);
      }
      describe(un2);
    }

    // the next unit's first k-tiles, unless the k-loop has requested them already (then every
    // store of this epilogue is younger than they are)
    auto prefetch_next = [&]() {
      st_after = 0;
      if (has_next && !chained) {
        ld_on_next = true;
        ld_enter(nxt_u);
        fetch_rows();
        issue_prologue(cur);
      }
    };
    // An accumulating epilogue (ACCUMULATE, a kernel of its own: the registers below would
    // otherwise be spilled around the k-loop of the plain one) adds to the gradients that are there.
    // Behind the requests for the next unit's first k-tiles a wave requests the old values of
    // OLD_BATCH of its 32 x 64 chunks at a time (the fragment registers are dead here) and only then
    // stages and stores them: the old values come back under one memory round trip per batch
    // instead of one per chunk.  They are younger than the next unit's first tiles, like the stores.
    constexpr int NCH = TM * (TN / 2), OLD_NP = 4, OLD_BATCH = 2;
    static_assert(St::CH == 8 && NCH % OLD_BATCH == 0, "a staged chunk is 32 rows of eight 16-byte pieces");
    const WgradKcProblem& q = p.prob[cur_u.q];
    bf16_t* const C = q.C + (int64_t)cur_u.e * p.M * p.N + (int64_t)(cur_u.mt * BM + wm * WTM) * p.N + cur_u.nt * BN + wn * WTN;
    const bool write_tile = !(ACCUMULATE && nkt == 0);      // nothing to add for an expert without rows
    prefetch_next();
    if (write_tile) {
      const int lrow = lane & 31, lq = 4 * (lane >> 5);
      const int lr = lane / St::CH, lc = lane % St::CH;
      auto chunk_dst = [&](int c) { return C + (int64_t)(32 * (c / (TN / 2))) * p.N + 64 * (c % (TN / 2)); };
#pragma unroll
      for (int c0 = 0; c0 < NCH; c0 += OLD_BATCH) {
        u32x4_t old[ACCUMULATE ? OLD_BATCH : 1][OLD_NP];
        if constexpr (ACCUMULATE) {
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int c = 0; c < OLD_BATCH; ++c)
#pragma unroll
            for (int qq = 0; qq < OLD_NP; ++qq)
              old[c][qq] = __builtin_nontemporal_load(
                  reinterpret_cast<const u32x4_t*>(chunk_dst(c0 + c) + (int64_t)(qq * 8 + lr) * p.N + lc * 8));
          st_after += OLD_BATCH * OLD_NP;
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int c = c0; c < c0 + OLD_BATCH; ++c) {
          const int i = c / (TN / 2), jh = 2 * (c % (TN / 2));
#pragma unroll
          for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd)
              St::put(sbuf, lrow, 32 * jj + 8 * qd + lq,
                      pack4(acc[i][jh + jj][4 * qd], acc[i][jh + jj][4 * qd + 1], acc[i][jh + jj][4 * qd + 2], acc[i][jh + jj][4 * qd + 3]));
          wave_lds_fence();
          if constexpr (ACCUMULATE) st_after += St::template flush_add<true>(sbuf, chunk_dst(c), p.N, old[c - c0]);
          else st_after += St::template flush<false, true>(sbuf, chunk_dst(c), p.N, 32);
          wave_lds_fence();
        }
      }
    }
    if (!has_next) break;
    cur_u = nxt_u;
    par ^= 1;
    ++round;
  }
  wait_dma<0>();   // the loads of the last slots must not land in LDS that a later workgroup owns
  if constexpr (DYNAMIC) {
    if (tid == 0) sched_finish(p.sched);
  }
}

inline int round_up_xcd(int64_t n) { return (int)(pk_ceil_div(n, NXCD) * NXCD); }

// One workgroup per CU (the ring takes most of the LDS), a multiple of 8 so that every XCD
// gets the same number of slots.
inline int persistent_grid() {
  static int cached = 0;
  if (cached == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    cached = cus / NXCD * NXCD;
    if (cached < NXCD) cached = NXCD;
  }
  return cached;
}

// Which counter set a launch uses.  Launches on one stream run one after the other and every
// launch leaves its set zeroed, so ONE set per stream is enough, and two launches share a set only
// if they cannot overlap.  The key of a set is (stream, capture sequence): a launch recorded into
// a HIP graph keeps its set for the life of the graph, which may replay next to eager work on the
// stream it was captured on, so a capture gets sets of its own (per stream of the capture: the
// streams of a forked capture run side by side inside the graph).  hipStreamPerThread is one
// handle for a different stream in every host thread, so there the thread is part of the key.
// When more keys than sets have been seen, sets are shared round-robin.
struct SchedKey {
  const void* stream;
  unsigned long long capture;
  size_t thread;
  bool operator<(const SchedKey& o) const {
    return std::tie(stream, capture, thread) < std::tie(o.stream, o.capture, o.thread);
  }
};
struct SchedDirectory {
  std::mutex mu;
  std::map<SchedKey, int> slot_of[PK_MAX_DEVICES];
  int next[PK_MAX_DEVICES] = {};
  SchedSlot* base[PK_MAX_DEVICES] = {};
};
SchedDirectory& sched_directory() {
  static SchedDirectory d;
  return d;
}
// Index of the set for a key on device `dev` (assigns the next set to a key seen for the first time).
int sched_slot_index(int dev, const void* stream, unsigned long long capture, size_t thread) {
  SchedDirectory& d = sched_directory();
  std::lock_guard<std::mutex> lock(d.mu);
  const SchedKey key{stream, capture, thread};
  auto it = d.slot_of[dev].find(key);
  if (it != d.slot_of[dev].end()) return it->second;
  const int slot = d.next[dev]++ % SCHED_SLOTS;
  d.slot_of[dev].emplace(key, slot);
  return slot;
}
// Device address of the pool on the current device, looked up once per device.
SchedSlot* sched_pool_base(int dev) {
  SchedDirectory& d = sched_directory();
  std::lock_guard<std::mutex> lock(d.mu);
  if (!d.base[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_sched_pool)) != hipSuccess || !ptr) return nullptr;
    d.base[dev] = (SchedSlot*)ptr;
  }
  return d.base[dev];
}
// Counter set for one launch on stream `s` of the current device (nullptr if the pool cannot be
// resolved).
inline SchedSlot* sched_slot_for_launch(hipStream_t s) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= PK_MAX_DEVICES) return nullptr;
  SchedSlot* const base = sched_pool_base(dev);
  if (!base) return nullptr;
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long capture = 0;
  if (hipStreamGetCaptureInfo(s, &status, &capture) != hipSuccess) {
    (void)hipGetLastError();
    status = hipStreamCaptureStatusNone;
  }
  if (status != hipStreamCaptureStatusActive) capture = 0;
  else capture += 1;      // 0 stands for "not capturing"
  const size_t thread = s == hipStreamPerThread ? std::hash<std::thread::id>{}(std::this_thread::get_id()) : 0;
  return base + sched_slot_index(dev, (const void*)s, capture, thread);
}

template <int BM, int BN, int BK, int WMW, int WNW, int NS, bool B_KC, int EPI, bool A_T = false>
int launch_ragged_m(RaggedMParams p, int64_t A_rows, int kernel_id, hipStream_t s) {
  const int64_t max_units = (pk_ceil_div(A_rows, BM) + p.E) * p.n_tiles;
  if (max_units > 0x7ffffff0ll || p.ldb * (int64_t)(BN > BK ? BN : BK) * 2 > 0x7fffffffll) return PK_ERR_SHAPE;
  // a lane addresses its A row by a 32-bit byte offset: from the unit's first row without a row
  // map, from the operand's first row with one (all the rows that the map can name: under 4 GiB)
  const int64_t a_span_rows = p.row_map ? pk_ceil_div(A_rows, p.map_div.d) : (int64_t)BM;
  if (p.lda * 2 > 0x7fffffffll || (a_span_rows + 1) * p.lda * 2 > 0xffffffffll) return PK_ERR_SHAPE;
  if (A_T && p.row_map) return PK_ERR_ARG;
  if ((int64_t)p.Kseg * p.nseg < 2 * BK) return PK_ERR_SHAPE;
  const int64_t grid = max_units < persistent_grid() ? round_up_xcd(max_units) : persistent_grid();
  p.sched = sched_slot_for_launch(s);
  if (!p.sched) return PK_ERR_UNSUPPORTED;
  PK_LAUNCH_NOCHECK(kernel_id, s, (ragged_m_kernel<BM, BN, BK, WMW, WNW, NS, B_KC, EPI, A_T>),
                    dim3((unsigned)grid), dim3(64 * WMW * WNW), 0, s, p);
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

// Sum the per-64-column partials of the score gradient and store them at the flat (token, k)
// slot of each sorted row.
__global__ void dscore_reduce_kernel(const float* __restrict__ part, int P, int64_t A,
                                     const int32_t* __restrict__ row_map, float* __restrict__ d_scores) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= A) return;
  float s = 0.f;
  for (int q = 0; q < P; ++q) s += part[(int64_t)q * A + r];
  d_scores[row_map[r]] = s;
}

// Generic second half of the scaled SwiGLU backward: one wave per sorted row.  dh holds the
// unscaled d_h = d_out[token] . w2 and may alias du.
template <typename T>
__global__ void swiglu_bwd_scaled_rows_kernel(const T* dh, const T* __restrict__ g, const T* __restrict__ u,
                                              const int32_t* __restrict__ row_map, const float* __restrict__ scores,
                                              T* __restrict__ dg, T* du, T* __restrict__ hs,
                                              float* __restrict__ d_scores, int64_t A, int64_t I) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (r >= A) return;
  const int slot = row_map[r];
  const float sc = scores[slot];
  float ds = 0.f;
  for (int64_t i = lane; i < I; i += 64) {
    const int64_t o = r * I + i;
    const float a = pk_to_float<T>(dh[o]), gv = pk_to_float<T>(g[o]), uv = pk_to_float<T>(u[o]);
    const float sg = 1.f / (1.f + expf(-gv));
    const float hv = (gv * sg) * uv;
    ds += a * hv;
    const float d = pk_to_float<T>(pk_from_float<T>(sc * a));
    dg[o] = pk_from_float<T>(d * uv * (sg * (1.f + gv * (1.f - sg))));
    du[o] = pk_from_float<T>(d * (gv * sg));
    hs[o] = pk_from_float<T>(sc * hv);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ds += __shfl_xor(ds, off);
  if (lane == 0) d_scores[slot] = ds;
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

// Tile configurations (BM, BN, BK, waves along M, waves along N, LDS ring stages), chosen by
// measurement on MI355X with random data and multinomial / Zipf row counts.
// Ragged-M kernels: 256x256x32 block tiles, 8 waves (128x64 wave tiles), 4-stage 128 KB ring (the
// epilogue stages its output in the stage that no k-tile occupies between two units).
#define PK_RM_CFG 256, 256, 32, 2, 4, 4
#define PK_RM_BN 256
// Same width with 128 rows, 64-deep k-tiles in a 3-stage ring (a weight row contributes 128
// contiguous bytes per k-tile).  For launches that would give a workgroup fewer than
// PK_RM_LOWM_UNITS of the 256-row units (the last round of units would run on a half-empty chip);
// for experts with fewer than PK_RM_SHORT_ROWS rows on average, where the weights dominate the
// traffic and are read from HBM by one or two row tiles each (measured at 256 rows per expert
// against the 256x256x32 tiles: gate/up -8 %, down -4 %, d_x -3 %; at 1,024 rows per expert +2 %
// to +8 %); and for the scaled SwiGLU backward at any size (against 32-deep k-tiles in a 5-stage
// ring: -9 % at 4,096 tokens, -8 % at 16,384).
#define PK_RM_SHORT 128, 256, 64, 2, 4, 3
#define PK_RM_LOWM_UNITS 3
#define PK_RM_SHORT_ROWS 512
// Output widths that are a multiple of 128 but not of 256.
#define PK_RM_ALT 128, 128, 64, 2, 2, 4
// Weight gradient of the piecewise entry points (wgrad_kernel; the fused region runs
// wgrad_pp_kernel, whose tile is fixed): 256x256x64 in a 2-stage ring; with fewer than
// PK_WG_SHORTK_ROWS rows per expert on average 32-deep tiles in a 4-stage ring with the loads spread
// between the MFMAs (measured against the 64-deep ring: -1.8 % at 256 rows per expert, +7 % at 1,024).
#define PK_WG_BIG 256, 256, 64, 2, 4, 2
#define PK_WG_BIG_THREADS 512
#define PK_WG_BIG_SHORTK 256, 256, 32, 2, 4, 4
#define PK_WG_SHORTK_ROWS 512
#define PK_WG_SMALL 128, 128, 64, 2, 2, 4
#define PK_WG_SMALL_THREADS 256

bool mfma_shape_ok(int64_t H, int64_t I) { return H % 128 == 0 && I % 128 == 0; }

// Pick the tile width by the output width N of the GEMM (for the gate/up kernel a tile holds
// BN/2 gate and BN/2 up columns).
template <bool B_KC, int EPI, bool A_T = false>
int launch_rm(mf::RaggedMParams& p, int64_t A, int64_t N, int kernel_id, hipStream_t s) {
  const int64_t per_tile_big = (EPI == mf::EPI_SWIGLU) ? PK_RM_BN / 2 : PK_RM_BN;
  if (N % per_tile_big == 0) {
    p.n_tiles = (int32_t)(N / per_tile_big);
    // 256-row tiles unless they would leave the persistent grid with only a few units per
    // workgroup (then the last round of units runs on a half-empty chip)
    const int64_t big_units = (A / 256 + p.E / 2) * p.n_tiles;
    const bool lowm = big_units < (int64_t)PK_RM_LOWM_UNITS * mf::persistent_grid();
    // the scaled SwiGLU backward stays on 128-row units: its time goes into the epilogue (loads of g
    // and u, the arithmetic, six stores per value), which 256-row units do not shorten, and with
    // 128 accumulator registers that epilogue spills (measured 14 % slower at 16,384 tokens even
    // with the packed outputs staged 32 columns at a time)
    if (EPI == mf::EPI_SWIGLU_BWD_SCALED || lowm || A < (int64_t)PK_RM_SHORT_ROWS * p.E)
      return mf::launch_ragged_m<PK_RM_SHORT, B_KC, EPI, A_T>(p, A, kernel_id, s);
    if constexpr (EPI != mf::EPI_SWIGLU_BWD_SCALED) return mf::launch_ragged_m<PK_RM_CFG, B_KC, EPI, A_T>(p, A, kernel_id, s);
  }
  if constexpr (A_T) return PK_ERR_SHAPE;      // the transposed copies exist for widths that are multiples of 256 only
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
int wgrad_simt(const void* dy, const int32_t* dy_map, const void* h, const void* dg, const void* du, const void* x,
               const int32_t* row_map, int64_t div, const int32_t* starts, void* dw1, void* dw2,
               void* dw3, int acc, int64_t H, int64_t I, int64_t E, hipStream_t s) {
  int rc = PK_OK;
  if (dw2) rc = simt_ragged_k<T>(dy, H, dy_map, h, I, nullptr, dy_map ? div : 1, dw2, starts, H, I, E, acc, s);
  if (rc) return rc;
  if (dw1) rc = simt_ragged_k<T>(dg, I, nullptr, x, H, row_map, div, dw1, starts, I, H, E, acc, s);
  if (rc) return rc;
  if (dw3) rc = simt_ragged_k<T>(du, I, nullptr, x, H, row_map, div, dw3, starts, I, H, E, acc, s);
  return rc;
}

}  // namespace

// Resolves, for the current device, what the grouped GEMMs otherwise look up on their first launch.
int pk_init_grouped_gemm() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= PK_MAX_DEVICES) return PK_ERR_UNSUPPORTED;
  (void)mf::persistent_grid();
  return mf::sched_pool_base(dev) ? PK_OK : PK_ERR_UNSUPPORTED;
}

extern "C" {

int pk_sched_slot_index(int device, uint64_t stream_handle, uint64_t capture_sequence, uint64_t thread_key) {
  if (device < 0 || device >= PK_MAX_DEVICES) return PK_ERR_ARG;
  return mf::sched_slot_index(device, (const void*)(uintptr_t)stream_handle, capture_sequence, (size_t)thread_key);
}

int pk_grouped_swiglu_fwd(const void* x_rows, const int32_t* row_map, int64_t row_map_div,
                          const void* w1, const void* w2, const void* w3,
                          const int32_t* starts, void* g, void* u, void* h, void* y,
                          int64_t A, int64_t H, int64_t I, int64_t E, int dtype,
                          pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  if (A == 0) return PK_OK;
  if (!x_rows || !w1 || !w2 || !w3 || !starts || !g || !u || !h || !y) return PK_ERR_ARG;
  if (row_map && (row_map_div <= 0 || row_map_div > 0x7fffffffll)) return PK_ERR_ARG;
  if (!row_map) row_map_div = 1;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PK_F32)
    return fwd_simt<float>(x_rows, row_map, row_map_div, w1, w2, w3, starts, g, u, h, y, A, H, I, E, s);
  if (!mfma_shape_ok(H, I) || !all_aligned16({x_rows, w1, w2, w3, g, u, h, y}))
    return fwd_simt<bf16_t>(x_rows, row_map, row_map_div, w1, w2, w3, starts, g, u, h, y, A, H, I, E, s);

  mf::RaggedMParams p = {};
  p.A0 = (const bf16_t*)x_rows; p.A1 = nullptr; p.lda = H;
  p.row_map = row_map; p.map_div = mf::make_fastdiv(row_map_div);
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

int64_t pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes(int64_t A, int64_t I) {
  if (A < 0 || I <= 0) return PK_ERR_ARG;
  return pk_ceil_div(I, 64) * A * (int64_t)sizeof(float);
}

int64_t pk_grouped_swiglu_transposed_ld(int64_t A, int64_t H, int64_t I, int64_t E, int dtype) {
  if (A < 0 || H <= 0 || I <= 0 || E <= 0) return PK_ERR_ARG;
  if (dtype != PK_BF16 || H % 256 != 0 || I % 256 != 0 || E > PK_MAX_EXPERTS || A + (int64_t)mf::kTransposedAlign * E > 0x7fffff00ll) return 0;
  // an odd multiple of 256 bytes: consecutive rows of a transposed copy then start in different
  // 256-byte phases of a 4 KiB period, so the 16 rows that one store (or the 256 rows that one
  // tile load) touches at the same column do not all map to the same memory channel
  int64_t units = ((A + mf::kTransposedAlign - 1) / mf::kTransposedAlign + E + 1) / 2;
  if (units % 2 == 0) ++units;
  return units * 2 * mf::kTransposedAlign;
}

// transposed outputs (d_gT, d_uT, hsT: [I][ldt]) are optional; with them hs itself may be NULL
static int dgrad_dh_scaled_impl(const void* d_out, const int32_t* row_map, int64_t row_map_div,
                                const float* scores, const void* w2, const void* g,
                                const void* u, const int32_t* starts, void* d_g, void* d_u,
                                void* hs, void* d_gT, void* d_uT, void* hsT, int64_t ldt, float* d_scores,
                                void* workspace, int64_t workspace_bytes, int64_t A, int64_t H, int64_t I,
                                int64_t E, int dtype, pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  if (A == 0) return PK_OK;
  const bool transposed = d_gT != nullptr;
  if (!d_out || !row_map || row_map_div <= 0 || row_map_div > 0x7fffffffll || !scores || !w2 || !g || !u || !starts || !d_scores)
    return PK_ERR_ARG;
  if ((!hs || !d_g || !d_u) && !transposed) return PK_ERR_ARG;      // the row-major outputs are optional beside the transposed ones
  if ((d_g == nullptr) != (d_u == nullptr)) return PK_ERR_ARG;
  if (transposed) {
    const int64_t need = pk_grouped_swiglu_transposed_ld(A, H, I, E, dtype);
    if (need <= 0) return PK_ERR_SHAPE;
    if (!d_uT || !hsT || ldt < need || ldt % 64 != 0) return PK_ERR_ARG;
    if (!all_aligned16({d_out, w2, g, u, d_g, d_u, hs, d_gT, d_uT, hsT})) return PK_ERR_ALIGN;
  }
  hipStream_t s = (hipStream_t)stream;
  const bool simt = dtype == PK_F32 || !mfma_shape_ok(H, I) || !all_aligned16({d_out, w2, g, u, d_g, d_u, hs});
  if (simt) {
    // unscaled d_h = d_out[token] . w2[e], staged in d_u's buffer; then one wave per row
    if (dtype == PK_F32) rc = simt_ragged_m<float>(d_out, H, row_map, row_map_div, w2, I, 1, H * I, d_u, I, starts, A, I, H, E, 0, s);
    else rc = simt_ragged_m<bf16_t>(d_out, H, row_map, row_map_div, w2, I, 1, H * I, d_u, I, starts, A, I, H, E, 0, s);
    if (rc) return rc;
    const dim3 grid((unsigned)pk_ceil_div(A, 4)), block(256);
    if (dtype == PK_F32)
      PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_ELEMENTWISE, s, (swiglu_bwd_scaled_rows_kernel<float>), grid, block, 0, s,
                        (const float*)d_u, (const float*)g, (const float*)u, row_map, scores, (float*)d_g, (float*)d_u, (float*)hs, d_scores, A, I);
    else
      PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_ELEMENTWISE, s, (swiglu_bwd_scaled_rows_kernel<bf16_t>), grid, block, 0, s,
                        (const bf16_t*)d_u, (const bf16_t*)g, (const bf16_t*)u, row_map, scores, (bf16_t*)d_g, (bf16_t*)d_u, (bf16_t*)hs, d_scores, A, I);
    PK_RETURN_IF_LAUNCH_FAILED();
    return PK_OK;
  }
  const int64_t need = pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes(A, I);
  if (!workspace || workspace_bytes < need) return PK_ERR_WORKSPACE;
  mf::RaggedMParams p = {};
  p.A0 = (const bf16_t*)d_out; p.lda = H;
  p.row_map = row_map; p.map_div = mf::make_fastdiv(row_map_div);
  p.B0 = (const bf16_t*)w2; p.ldb = I; p.strideB = H * I;
  p.starts = starts; p.E = (int32_t)E; p.Kseg = (int32_t)H; p.nseg = 1;
  p.Gin = (const bf16_t*)g; p.Uin = (const bf16_t*)u;
  p.O0 = (bf16_t*)d_g; p.O1 = (bf16_t*)d_u; p.O2 = (bf16_t*)hs; p.ldc = I;
  p.T0 = (bf16_t*)d_gT; p.T1 = (bf16_t*)d_uT; p.T2 = (bf16_t*)hsT; p.ldt = ldt;
  p.scores = scores; p.ds_partial = (float*)workspace; p.total_rows = A;
  rc = launch_rm<false, mf::EPI_SWIGLU_BWD_SCALED>(p, A, I, pk_timing::K_SWIGLU_DGRAD_DH, s);
  if (rc) return rc;
  PK_LAUNCH_NOCHECK(pk_timing::K_COMBINE_BWD, s, dscore_reduce_kernel, dim3((unsigned)pk_ceil_div(A, 256)), dim3(256), 0, s,
                    (const float*)workspace, (int)(I / 64), A, row_map, d_scores);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int pk_grouped_swiglu_dgrad_dh_scaled(const void* d_out, const int32_t* row_map, int64_t row_map_div,
                                      const float* scores, const void* w2, const void* g,
                                      const void* u, const int32_t* starts, void* d_g, void* d_u,
                                      void* hs, float* d_scores, void* workspace,
                                      int64_t workspace_bytes, int64_t A, int64_t H, int64_t I,
                                      int64_t E, int dtype, pk_stream_t stream) {
  if (A > 0 && !hs) return PK_ERR_ARG;
  return dgrad_dh_scaled_impl(d_out, row_map, row_map_div, scores, w2, g, u, starts, d_g, d_u, hs, nullptr, nullptr,
                              nullptr, 0, d_scores, workspace, workspace_bytes, A, H, I, E, dtype, stream);
}

int pk_grouped_swiglu_dgrad_dh_scaled_t(const void* d_out, const int32_t* row_map, int64_t row_map_div,
                                        const float* scores, const void* w2, const void* g,
                                        const void* u, const int32_t* starts, void* d_g, void* d_u,
                                        void* d_gT, void* d_uT, void* hsT, int64_t ldt, float* d_scores,
                                        void* workspace, int64_t workspace_bytes, int64_t A, int64_t H,
                                        int64_t I, int64_t E, int dtype, pk_stream_t stream) {
  if (A > 0 && (!d_gT || !d_uT || !hsT)) return PK_ERR_ARG;
  return dgrad_dh_scaled_impl(d_out, row_map, row_map_div, scores, w2, g, u, starts, d_g, d_u, nullptr, d_gT, d_uT, hsT,
                              ldt, d_scores, workspace, workspace_bytes, A, H, I, E, dtype, stream);
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

int pk_grouped_swiglu_dx_from_transposed_pays(int64_t A, int64_t H, int64_t I, int64_t E, int dtype) {
  if (pk_grouped_swiglu_transposed_ld(A, H, I, E, dtype) <= 0) return 0;
  // measured on MI355X (H 2048, I 768, 128 experts): with 1,024 rows per expert the SwiGLU backward is
  // 9 % and the d_x GEMM 4 % faster without the row-major copies (256-row units, the A tile arrives
  // as runs of 4 KB); with 256 rows per expert the d_x GEMM on 128-row units loses 6 %, more than
  // the SwiGLU backward gains
  return A >= (int64_t)PK_RM_SHORT_ROWS * E ? 1 : 0;
}

int pk_grouped_swiglu_dgrad_dx_t(const void* d_gT, const void* d_uT, int64_t ldt, const void* w1, const void* w3,
                                 const int32_t* starts, void* d_x_sorted, int64_t A, int64_t H, int64_t I,
                                 int64_t E, int dtype, pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  const int64_t need = pk_grouped_swiglu_transposed_ld(A, H, I, E, dtype);
  if (need <= 0) return PK_ERR_SHAPE;
  if (A == 0) return PK_OK;
  if (!d_gT || !d_uT || !w1 || !w3 || !starts || !d_x_sorted || ldt < need || ldt % 64 != 0) return PK_ERR_ARG;
  if (!all_aligned16({d_gT, d_uT, w1, w3, d_x_sorted})) return PK_ERR_ALIGN;
  // d_x = [d_g | d_u] . [w1[e] ; w3[e]] with the A operand read from the 32-row blocks
  mf::RaggedMParams q = {};
  q.A0 = (const bf16_t*)d_gT; q.A1 = (const bf16_t*)d_uT; q.lda = I;
  q.B0 = (const bf16_t*)w1; q.B1 = (const bf16_t*)w3; q.ldb = H; q.strideB = I * H;
  q.starts = starts; q.E = (int32_t)E; q.Kseg = (int32_t)I; q.nseg = 2;
  q.O0 = (bf16_t*)d_x_sorted; q.ldc = H;
  return launch_rm<false, mf::EPI_PLAIN, true>(q, A, H, pk_timing::K_SWIGLU_DGRAD_DX, (hipStream_t)stream);
}

int pk_grouped_swiglu_dgrad(const void* d_y, const void* w1, const void* w2, const void* w3,
                            const void* g, const void* u, const int32_t* starts, void* d_g,
                            void* d_u, void* d_x_sorted, int64_t A, int64_t H, int64_t I,
                            int64_t E, int dtype, pk_stream_t stream) {
  int rc = pk_grouped_swiglu_dgrad_dh(d_y, w2, g, u, starts, d_g, d_u, A, H, I, E, dtype, stream);
  if (rc) return rc;
  return pk_grouped_swiglu_dgrad_dx(d_g, d_u, w1, w3, starts, d_x_sorted, A, H, I, E, dtype, stream);
}

// d_y rows are addressed directly (dy_gathered == 0) or through the row map like x
static int wgrad_impl(const void* d_y, int dy_gathered, const void* h, const void* d_g, const void* d_u,
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
  if (row_map && (row_map_div <= 0 || row_map_div > 0x7fffffffll)) return PK_ERR_ARG;
  if (dy_gathered && !row_map) return PK_ERR_ARG;
  if (!row_map) row_map_div = 1;
  const int32_t* dy_map = dy_gathered ? row_map : nullptr;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == PK_F32)
    return wgrad_simt<float>(d_y, dy_map, h, d_g, d_u, x_rows, row_map, row_map_div, starts, d_w1, d_w2, d_w3, accumulate, H, I, E, s);
  if (!mfma_shape_ok(H, I) || !all_aligned16({d_y, h, d_g, d_u, x_rows, d_w1, d_w2, d_w3}))
    return wgrad_simt<bf16_t>(d_y, dy_map, h, d_g, d_u, x_rows, row_map, row_map_div, starts, d_w1, d_w2, d_w3, accumulate, H, I, E, s);

  mf::WgradParams p = {};
  int n = 0;
  if (d_w2) {
    mf::WgradProblem& q = p.prob[n++];
    q.A = (const bf16_t*)d_y; q.lda = H; q.a_map = dy_map;
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
  p.starts = starts; p.order = expert_order; p.E = (int32_t)E; p.map_div = mf::make_fastdiv(row_map_div);
  p.accumulate = accumulate ? 1 : 0;
  const bool big = (H % 256 == 0) && (I % 256 == 0);
  const int tile = big ? 256 : 128;
  p.tiles_per_expert = (int32_t)((H / tile) * (I / tile));
  p.nprob = n;
  const int64_t blocks = (int64_t)p.tiles_per_expert * n * pk_ceil_div(E, mf::NXCD) * mf::NXCD;
  const int gy = 1;
  if (blocks > 0x7ffffff0ll) return PK_ERR_SHAPE;
  if (big && A < (int64_t)PK_WG_SHORTK_ROWS * E)
    PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_WGRAD, s, (mf::wgrad_kernel<PK_WG_BIG_SHORTK>), dim3((unsigned)blocks, gy), dim3(PK_WG_BIG_THREADS), 0, s, p);
  else if (big)
    PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_WGRAD, s, (mf::wgrad_kernel<PK_WG_BIG>), dim3((unsigned)blocks, gy), dim3(PK_WG_BIG_THREADS), 0, s, p);
  else
    PK_LAUNCH_NOCHECK(pk_timing::K_SWIGLU_WGRAD, s, (mf::wgrad_kernel<PK_WG_SMALL>), dim3((unsigned)blocks, gy), dim3(PK_WG_SMALL_THREADS), 0, s, p);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int pk_grouped_swiglu_wgrad(const void* d_y, const void* h, const void* d_g, const void* d_u,
                            const void* x_rows, const int32_t* row_map, int64_t row_map_div,
                            const int32_t* starts, const int32_t* expert_order, void* d_w1,
                            void* d_w2, void* d_w3,
                            int accumulate, int64_t A, int64_t H, int64_t I, int64_t E,
                            int dtype, pk_stream_t stream) {
  return wgrad_impl(d_y, 0, h, d_g, d_u, x_rows, row_map, row_map_div, starts, expert_order, d_w1, d_w2, d_w3,
                    accumulate, A, H, I, E, dtype, stream);
}

int pk_grouped_swiglu_wgrad_scaled(const void* d_out, const void* hs, const void* d_g, const void* d_u,
                                   const void* x, const int32_t* row_map, int64_t row_map_div,
                                   const int32_t* starts, const int32_t* expert_order, void* d_w1,
                                   void* d_w2, void* d_w3,
                                   int accumulate, int64_t A, int64_t H, int64_t I, int64_t E,
                                   int dtype, pk_stream_t stream) {
  return wgrad_impl(d_out, 1, hs, d_g, d_u, x, row_map, row_map_div, starts, expert_order, d_w1, d_w2, d_w3,
                    accumulate, A, H, I, E, dtype, stream);
}

int pk_grouped_swiglu_wgrad_scaled_t(const void* d_out, const void* hsT, const void* d_gT, const void* d_uT,
                                     int64_t ldt, const void* x, const int32_t* row_map, int64_t row_map_div,
                                     const int32_t* starts, const int32_t* expert_order, void* d_w1,
                                     void* d_w2, void* d_w3, int accumulate, int64_t A, int64_t H,
                                     int64_t I, int64_t E, int dtype, pk_stream_t stream) {
  int rc = check_common(A, H, I, E, dtype);
  if (rc) return rc;
  const int64_t need = pk_grouped_swiglu_transposed_ld(A, H, I, E, dtype);
  if (need <= 0) return PK_ERR_SHAPE;
  // no routed rows: zero gradients (or nothing, when accumulating) from the kernel that needs no row map
  if (A == 0) return wgrad_impl(nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, 1, starts, expert_order, d_w1, d_w2, d_w3,
                                accumulate, A, H, I, E, dtype, stream);
  if (!starts || !row_map || row_map_div <= 0 || row_map_div > 0x7fffffffll || ldt < need || ldt % 64 != 0) return PK_ERR_ARG;
  if (d_w2 && (!d_out || !hsT)) return PK_ERR_ARG;
  if (d_w1 && (!d_gT || !x)) return PK_ERR_ARG;
  if (d_w3 && (!d_uT || !x)) return PK_ERR_ARG;
  if (!all_aligned16({d_out, hsT, d_gT, d_uT, x, d_w1, d_w2, d_w3})) return PK_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  mf::WgradKcParams base = {};
  base.ldt = ldt; base.ldr = H;
  base.row_map = row_map; base.map_div = mf::make_fastdiv(row_map_div);
  base.starts = starts; base.order = expert_order; base.E = (int32_t)E; base.total_rows = (int32_t)A;
  base.accumulate = accumulate ? 1 : 0;
  // skewed routing (experts of very different size) needs the dynamic hand-out of units; with a few
  // hundred rows per expert the static one is a few per cent faster
  const bool dynamic = A >= (int64_t)PK_WG_SHORTK_ROWS * E;
  // the kernels address the gathered operand with 32-bit byte offsets from its base
  if (((A + row_map_div - 1) / row_map_div) * H * 2 > 0xffffffffll) return PK_ERR_SHAPE;
  auto launch = [&](mf::WgradKcParams& p, bool a_kc) -> int {
    const int64_t units = (int64_t)E * p.nprob * (p.M / 256) * (p.N / 256);
    if (units > 0x7ffffff0ll) return PK_ERR_SHAPE;
    const dim3 grid((unsigned)(units < mf::persistent_grid() ? mf::round_up_xcd(units) : mf::persistent_grid())), block(512);
    if (dynamic) {
      p.sched = mf::sched_slot_for_launch(s);
      if (!p.sched) return PK_ERR_UNSUPPORTED;
    }
    const int id = a_kc ? pk_timing::K_SWIGLU_WGRAD_W13 : pk_timing::K_SWIGLU_WGRAD_W2;
#define PK_WGRAD_PP(WMW, WNW, AKC, DYN)                                                                         \
  do {                                                                                                          \
    if (p.accumulate) PK_LAUNCH_NOCHECK(id, s, (mf::wgrad_pp_kernel<WMW, WNW, AKC, DYN, true>), grid, block, 0, s, p);   \
    else PK_LAUNCH_NOCHECK(id, s, (mf::wgrad_pp_kernel<WMW, WNW, AKC, DYN, false>), grid, block, 0, s, p);               \
  } while (0)
    if (a_kc && dynamic) PK_WGRAD_PP(2, 4, true, true);
    else if (a_kc) PK_WGRAD_PP(2, 4, true, false);
    else if (dynamic) PK_WGRAD_PP(4, 2, false, true);
    else PK_WGRAD_PP(4, 2, false, false);
#undef PK_WGRAD_PP
    PK_RETURN_IF_LAUNCH_FAILED();
    return PK_OK;
  };
  if (d_w2) {   // d_w2[e][h][i] = sum_r d_out[token_r][h] * hs[r][i]: the transposed operand is the n side
    mf::WgradKcParams p = base;
    p.prob[0].T = (const bf16_t*)hsT; p.prob[0].R = (const bf16_t*)d_out; p.prob[0].C = (bf16_t*)d_w2;
    p.nprob = 1; p.M = (int32_t)H; p.N = (int32_t)I;
    rc = launch(p, false);
    if (rc) return rc;
  }
  if (d_w1 || d_w3) {   // d_w1[e][i][h] = sum_r d_g[r][i] * x[token_r][h]: the transposed operand is the m side
    mf::WgradKcParams p = base;
    int n = 0;
    if (d_w1) { p.prob[n].T = (const bf16_t*)d_gT; p.prob[n].R = (const bf16_t*)x; p.prob[n].C = (bf16_t*)d_w1; ++n; }
    if (d_w3) { p.prob[n].T = (const bf16_t*)d_uT; p.prob[n].R = (const bf16_t*)x; p.prob[n].C = (bf16_t*)d_w3; ++n; }
    p.nprob = n; p.M = (int32_t)I; p.N = (int32_t)H;
    rc = launch(p, true);
    if (rc) return rc;
  }
  return PK_OK;
}


}  // extern "C"
