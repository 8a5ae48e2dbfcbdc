// Routing: gate logits, wavefront softmax/top-k (+ backward), stable counting sort by expert.
#include "pk_common.h"
#include "mfma_x3_gemm.h"
#include <mutex>

namespace {

// ------------------------------------------------------------------ top-k
// Order-preserving map float -> uint32 (larger float -> larger uint).  -0.0 is folded into
// +0.0 and every NaN into the positive quiet NaN so that ties and NaNs behave like
// torch.sort(descending=True, stable=True).
__device__ __forceinline__ uint32_t orderable(float v) {
  v = v + 0.0f;
  uint32_t u = __float_as_uint(v);
  if (v != v) u = 0x7fc00000u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float from_orderable(uint32_t o) {
  const uint32_t u = (o & 0x80000000u) ? (o ^ 0x80000000u) : ~o;
  return __uint_as_float(u);
}

constexpr int kRouteThreads = 256;  // 4 waves, one token per wave

// One wave per token.  Lane l owns experts l, l+64, ... (EPL of them).
template <int EPL>
__global__ __launch_bounds__(kRouteThreads) void route_topk_kernel(
    const float* __restrict__ logits, int T, int E, int K, int route_norm, float route_scale,
    float* __restrict__ top_scores, int32_t* __restrict__ top_idx) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * (kRouteThreads / 64) + wave;
  if (t >= T) return;
  const float* row = logits + (int64_t)t * E;

  float val[EPL];
  unsigned long long key[EPL];
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane + 64 * j;
    if (e < E) {
      val[j] = row[e];
      key[j] = ((unsigned long long)orderable(val[j]) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)e);
    } else {
      val[j] = 0.f;
      key[j] = 0ull;  // never wins: every real key has a non-zero high word
    }
  }

  float vmax = 0.f;
  float my_v = 0.f;
  int my_e = 0;
  for (int k = 0; k < K; ++k) {
    unsigned long long best = 0ull;
#pragma unroll
    for (int j = 0; j < EPL; ++j) best = key[j] > best ? key[j] : best;
    best = pk_wave_max_u64(best);
    const uint32_t e_win = 0xffffffffu - (uint32_t)(best & 0xffffffffull);
    const float v_win = from_orderable((uint32_t)(best >> 32));
#pragma unroll
    for (int j = 0; j < EPL; ++j)
      if ((int)e_win == lane + 64 * j) key[j] = 0ull;
    if (k == 0) vmax = v_win;
    if (lane == k) { my_v = v_win; my_e = (int)e_win; }
  }

  float part = 0.f;
#pragma unroll
  for (int j = 0; j < EPL; ++j)
    if (lane + 64 * j < E) part += expf(val[j] - vmax);
  const float denom = pk_wave_sum(part);

  float s = (lane < K) ? expf(my_v - vmax) / denom : 0.f;
  if (route_norm) {
    const float S = pk_wave_sum(s);
    s = s / (S + 1e-20f);
  }
  s *= route_scale;
  if (lane < K) {
    top_scores[(int64_t)t * K + lane] = s;
    top_idx[(int64_t)t * K + lane] = my_e;
  }
}

template <int EPL>
__global__ __launch_bounds__(kRouteThreads) void route_topk_bwd_kernel(
    const float* __restrict__ logits, const int32_t* __restrict__ top_idx,
    const float* __restrict__ d_top_scores, int T, int E, int K, int route_norm,
    float route_scale, float* __restrict__ d_logits) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * (kRouteThreads / 64) + wave;
  if (t >= T) return;
  const float* row = logits + (int64_t)t * E;

  float val[EPL];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane + 64 * j;
    val[j] = (e < E) ? row[e] : -INFINITY;
    mx = fmaxf(mx, val[j]);
  }
  mx = pk_wave_max(mx);
  float p[EPL];
  float part = 0.f;
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    p[j] = (lane + 64 * j < E) ? expf(val[j] - mx) : 0.f;
    part += p[j];
  }
  const float denom = pk_wave_sum(part);
#pragma unroll
  for (int j = 0; j < EPL; ++j) p[j] = p[j] / denom;

  // lanes k < K: selected expert, its probability, incoming gradient
  int my_e = -1;
  float s = 0.f, dw = 0.f;
  if (lane < K) {
    my_e = top_idx[(int64_t)t * K + lane];
    s = expf(row[my_e] - mx) / denom;
    dw = d_top_scores[(int64_t)t * K + lane];
  }
  float ds;
  if (route_norm) {
    const float S = pk_wave_sum(s) + 1e-20f;
    const float dot = pk_wave_sum(dw * s);
    ds = route_scale * (dw / S - dot / (S * S));
  } else {
    ds = route_scale * dw;
  }
  if (lane >= K) ds = 0.f;
  const float D = pk_wave_sum(ds * s);  // sum_j dp_j p_j

  float dp[EPL];
#pragma unroll
  for (int j = 0; j < EPL; ++j) dp[j] = 0.f;
  for (int k = 0; k < K; ++k) {
    const int ek = __shfl(my_e, k, PK_WAVE);
    const float dsk = __shfl(ds, k, PK_WAVE);
#pragma unroll
    for (int j = 0; j < EPL; ++j)
      if (lane + 64 * j == ek) dp[j] = dsk;
  }
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane + 64 * j;
    if (e < E) d_logits[(int64_t)t * E + e] = p[j] * (dp[j] - D);
  }
}

// ------------------------------------------------------------------ counting sort
constexpr int kSortChunk = 512;  // flat slots per chunk; one wave walks a chunk in order

__global__ __launch_bounds__(64) void sort_hist_kernel(const int32_t* __restrict__ idx, int A,
                                                       int E, int32_t* __restrict__ chunk_hist) {
  extern __shared__ int32_t hist[];  // [E]
  for (int e = threadIdx.x; e < E; e += 64) hist[e] = 0;
  __syncthreads();
  const int base = blockIdx.x * kSortChunk;
  for (int i = threadIdx.x; i < kSortChunk; i += 64) {
    const int s = base + i;
    if (s < A) {
      const int e = idx[s];
      if ((unsigned)e < (unsigned)E) atomicAdd(&hist[e], 1);  // out-of-range ids are dropped
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 64) chunk_hist[(int64_t)blockIdx.x * E + e] = hist[e];
}

// Single block.  counts[e] = sum over chunks; starts = exclusive scan; chunk_hist[c][e] is
// replaced by the first output position of expert e's rows coming from chunk c.
__global__ __launch_bounds__(1024) void sort_scan_kernel(int32_t* __restrict__ chunk_hist,
                                                         int nchunks, int E,
                                                         int32_t* __restrict__ counts,
                                                         int32_t* __restrict__ starts,
                                                         int32_t* __restrict__ order) {
  // One block.  The 1024 threads form G = 1024 / Epad groups (Epad = E rounded up to a power of
  // two); group g of expert e walks chunks [g*cpg, (g+1)*cpg), so the two passes over the
  // chunk histograms are G times shorter than with one thread per expert.
  __shared__ int32_t part[1024];     // [g][e]: rows of expert e in the chunks of group g
  __shared__ int32_t scan[PK_MAX_EXPERTS];
  __shared__ int32_t cnts[PK_MAX_EXPERTS];
  int epad = 1;
  while (epad < E) epad <<= 1;
  const int G = 1024 / epad;
  const int e = threadIdx.x % epad, g = threadIdx.x / epad;
  const int cpg = (nchunks + G - 1) / G;
  const int c0 = g * cpg, c1 = min(nchunks, c0 + cpg);
  // (both walks over the chunks fetch eight values at a time: one round trip per eight chunks)
  constexpr int WALK = 8;
  int mine = 0;
  if (e < E)
    for (int c = c0; c < c1; c += WALK) {
      int v[WALK];
#pragma unroll
      for (int i = 0; i < WALK; ++i) v[i] = c + i < c1 ? chunk_hist[(int64_t)(c + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < WALK; ++i) mine += v[i];
    }
  part[threadIdx.x] = mine;
  __syncthreads();
  int total = 0, before = 0;      // rows of expert e in all chunks / in the chunks of earlier groups
  for (int k = 0; k < G; ++k) {
    const int v = part[k * epad + e];
    total += v;
    before += k < g ? v : 0;
  }
  if (threadIdx.x < 1024 && g == 0) {
    if (e < E && counts) counts[e] = total;
    scan[e] = (e < E) ? total : 0;
    cnts[e] = (e < E) ? total : -1;
  }
  __syncthreads();
  if (order && g == 0 && e < E) {
    // experts by descending row count, ties by index: order[rank] = e
    int rank = 0;
    for (int o = 0; o < E; ++o) {
      const int oc = cnts[o];
      rank += (oc > total || (oc == total && o < e)) ? 1 : 0;
    }
    order[rank] = e;
  }
  // Hillis-Steele inclusive scan over the Epad expert totals
  for (int off = 1; off < epad; off <<= 1) {
    int v = 0;
    if (g == 0 && e >= off) v = scan[e - off];
    __syncthreads();
    if (g == 0) scan[e] += v;
    __syncthreads();
  }
  const int start = scan[e] - total;  // exclusive
  if (e < E) {
    if (g == 0) {
      starts[e] = start;
      if (e == E - 1) starts[E] = scan[e];
    }
    int run = start + before;
    for (int c = c0; c < c1; c += WALK) {
      int v[WALK];
#pragma unroll
      for (int i = 0; i < WALK; ++i) v[i] = c + i < c1 ? chunk_hist[(int64_t)(c + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < WALK; ++i)
        if (c + i < c1) {
          chunk_hist[(int64_t)(c + i) * E + e] = run;
          run += v[i];
        }
    }
  }
}

__global__ __launch_bounds__(64) void sort_scatter_kernel(const int32_t* __restrict__ idx, int A,
                                                          int E, const int32_t* __restrict__ chunk_base,
                                                          int32_t* __restrict__ perm,
                                                          int32_t* __restrict__ inv_perm) {
  extern __shared__ int32_t base[];  // [E] next free position per expert
  const int lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) base[e] = chunk_base[(int64_t)blockIdx.x * E + e];
  __syncthreads();
  const int s0 = blockIdx.x * kSortChunk;
  const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int i = 0; i < kSortChunk; i += 64) {
    const int s = s0 + i + lane;
    int e = (s < A) ? idx[s] : -1;
    if ((unsigned)e >= (unsigned)E) e = -1;
    const bool active = e >= 0;
    // lanes holding the same expert id
    unsigned long long same = __ballot(active);
    for (int b = 0; b < 10; ++b) {
      const unsigned long long bal = __ballot((e >> b) & 1);
      same &= ((e >> b) & 1) ? bal : ~bal;
    }
    int pos = 0;
    if (active) {
      const int rank = __popcll(same & lt_mask);
      pos = base[e] + rank;
    }
    __syncthreads();
    if (active) {
      // the last lane of each group advances the expert's cursor
      const int top = 63 - __clzll(same);
      if (lane == top) base[e] += __popcll(same);
      perm[pos] = s;
      if (inv_perm) inv_perm[s] = pos;
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(1024) void counts_to_starts_kernel(const void* __restrict__ counts,
                                                                int is_i64, int E,
                                                                int32_t* __restrict__ starts) {
  __shared__ int32_t scan[PK_MAX_EXPERTS];
  const int e = threadIdx.x;
  int c = 0;
  if (e < E) c = is_i64 ? (int)reinterpret_cast<const int64_t*>(counts)[e]
                        : reinterpret_cast<const int32_t*>(counts)[e];
  scan[e] = c;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const int v = (e >= off) ? scan[e - off] : 0;
    __syncthreads();
    scan[e] += v;
    __syncthreads();
  }
  if (e < E) {
    starts[e] = scan[e] - c;
    if (e == E - 1) starts[E] = scan[e];
  }
}

// ------------------------------------------------------------------ small helpers
// d_bias[e] (+)= sum_t d_logits[t,e]; one block per expert
__global__ __launch_bounds__(256) void colsum_kernel(const float* __restrict__ d_logits, int64_t T,
                                                     int E, float* __restrict__ d_bias,
                                                     int accumulate) {
  __shared__ float red[16];
  const int e = blockIdx.x;
  float s = 0.f;
  for (int64_t t = threadIdx.x; t < T; t += blockDim.x) s += d_logits[t * E + e];
  s = pk_block_sum(s, red);
  if (threadIdx.x == 0) d_bias[e] = accumulate ? d_bias[e] + s : s;
}

// The same sum for long inputs in two steps with contiguous reads: block b adds up the rows
// [b * per, (b+1) * per) of d_logits (256 threads = RP rows x E/4 column groups of 16 bytes, a
// thread walks every RP-th row with eight rows in flight, the RP partial rows are added in order
// through LDS), then one thread per column adds the kColsumBlocks partial rows in block order.
// One block per expert reading a column touches every cache line of d_logits from every XCD.
constexpr int kColsumBlocks = 64;
__global__ __launch_bounds__(256) void colsum_partial_kernel(const float* __restrict__ d_logits, int64_t T,
                                                             int E, float* __restrict__ part) {
  __shared__ float red[1024];
  const int cols4 = E / 4, RP = 256 / cols4;
  const int r = threadIdx.x / cols4, c = threadIdx.x % cols4;
  const int64_t per = (T + gridDim.x - 1) / gridDim.x;
  const int64_t t0 = (int64_t)blockIdx.x * per, t1 = t0 + per < T ? t0 + per : T;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (r < RP) {
    const float4* src = reinterpret_cast<const float4*>(d_logits) + c;
    int64_t t = t0 + r;
    for (; t + 7 * RP < t1; t += 8 * RP) {
      float4 v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = src[(t + i * RP) * cols4];
#pragma unroll
      for (int i = 0; i < 8; ++i) { acc.x += v[i].x; acc.y += v[i].y; acc.z += v[i].z; acc.w += v[i].w; }
    }
    for (; t < t1; t += RP) {
      const float4 v = src[t * cols4];
      acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
    reinterpret_cast<float4*>(red)[r * cols4 + c] = acc;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256) {
    float s = 0.f;
    for (int q = 0; q < RP; ++q) s += red[q * E + e];
    part[(int64_t)blockIdx.x * E + e] = s;
  }
}
__global__ __launch_bounds__(256) void colsum_final_kernel(const float* __restrict__ part, int nblocks, int E,
                                                           float* __restrict__ d_bias, int accumulate) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= E) return;
  float v[kColsumBlocks];     // all loads first: one round trip, then the sum in block order
#pragma unroll
  for (int b = 0; b < kColsumBlocks; ++b) v[b] = b < nblocks ? part[(int64_t)b * E + e] : 0.f;
  float s = 0.f;
#pragma unroll
  for (int b = 0; b < kColsumBlocks; ++b) s += v[b];
  d_bias[e] = accumulate ? d_bias[e] + s : s;
}

// Scratch of pk_sort_by_expert_static: the per-chunk histograms of the counting sort.  Every GPU
// the library runs on holds its own copy of the array (PK_SORT_STATIC_WORDS * 4 bytes) until the
// process ends.  In host code the name `scratch` is only a handle for hipGetSymbolAddress: the
// address a kernel can use is looked up once per device, with that device current, and kept.
static __device__ __align__(256) int32_t scratch[PK_SORT_STATIC_WORDS];

int32_t* sort_scratch_for_current_device() {
  constexpr int MAX_DEV = PK_MAX_DEVICES;
  static int32_t* ptr[MAX_DEV] = {};
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
    ptr[dev] = static_cast<int32_t*>(p);
  }
  return ptr[dev];
}

}  // namespace

extern "C" {

int pk_version(void) { return 100; }

int pk_init(void) {
  if (!sort_scratch_for_current_device()) return PK_ERR_UNSUPPORTED;
  return pk_init_grouped_gemm();
}

const char* pk_status_string(int status) {
  switch (status) {
    case PK_OK: return "ok";
    case PK_ERR_ARG: return "invalid argument (null pointer, negative size or bad enum)";
    case PK_ERR_SHAPE: return "shape not supported by the kernels";
    case PK_ERR_ALIGN: return "pointer or leading dimension is not 16-byte aligned";
    case PK_ERR_WORKSPACE: return "workspace too small";
    case PK_ERR_UNSUPPORTED: return "dtype/option combination not supported";
    default: return status > 0 ? "HIP runtime error (status is the hipError_t value)" : "unknown status";
  }
}

static int gate_fwd_splits(int64_t H) {
  int64_t sp = H / 256;
  return (int)(sp < 1 ? 1 : (sp > 8 ? 8 : sp));
}

static int64_t align256(int64_t n) { return (n + 255) / 256 * 256; }
// bytes of the three bf16 planes of an fp32 array of n elements (0: cannot be pre-split)
static int64_t plane_bytes(int64_t n) { return n % 4 == 0 ? align256(3 * n * (int64_t)sizeof(bf16_t)) : 0; }
// fp32 [n] -> bf16 planes [3][n] at dst
static int split_planes(const float* src, bf16_t* dst, int64_t n, int kernel_id, hipStream_t s) {
  PK_LAUNCH_NOCHECK(kernel_id, s, pk_x3mm::split_planes_kernel, dim3((unsigned)pk_ceil_div(n, 1024)), dim3(256), 0, s, src, dst, n);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

static int64_t gate_fwd_partial_bytes(int64_t T, int64_t H, int64_t E) {
  const int sp = gate_fwd_splits(H);
  return sp > 1 ? (int64_t)sp * T * E * (int64_t)sizeof(float) : 0;
}

int64_t pk_gate_workspace_bytes(int64_t T, int64_t H, int64_t E) {
  if (T < 0 || H <= 0 || E <= 0) return PK_ERR_ARG;
  return gate_fwd_partial_bytes(T, H, E);
}

int pk_gate_logits(const void* x, int x_dtype, const float* w_gate, const float* gate_bias,
                   float* logits, int64_t T, int64_t H, int64_t E, void* workspace,
                   int64_t workspace_bytes, pk_stream_t stream) {
  if (T < 0 || H <= 0 || E <= 0 || !pk_dtype_ok(x_dtype)) return PK_ERR_ARG;
  if (T == 0) return PK_OK;
  if (!x || !w_gate || !logits) return PK_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  int sp = gate_fwd_splits(H);
  // the reduction is split only as far as it takes to give every CU two workgroups: each split
  // writes and re-reads a [T, E] fp32 partial result, which soon outweighs reading x
  const int64_t row_tiles = pk_ceil_div(T, 64);
  while (sp > 1 && row_tiles * (sp / 2) >= 512) sp /= 2;
  if (sp > 1 && (!workspace || workspace_bytes < gate_fwd_partial_bytes(T, H, E))) sp = 1;
  // (Handing this GEMM the weight already split into bf16 planes does not shorten it: the kernel
  // waits on its loads and barriers, not on the instructions of the split.)
  pk_f32mm::Params p = {};
  p.A = x; p.B = w_gate;
  p.C = sp > 1 ? reinterpret_cast<float*>(workspace) : logits;
  p.bias = sp > 1 ? nullptr : gate_bias;
  p.M = T; p.N = E; p.K = H;
  p.sam = H; p.sak = 1; p.sbk = 1; p.sbn = H;
  p.splits = sp; p.accumulate = 0;
  int rc;
  const bool xb = x_dtype == PK_BF16;
  if (E > 64)  // 64-token x 128-expert tiles, 8 waves
    rc = xb ? pk_x3mm::launch<2, 4, true, true, bf16_t, float>(p, pk_timing::K_GATE_LOGITS, s)
            : pk_x3mm::launch<2, 4, true, true, float, float>(p, pk_timing::K_GATE_LOGITS, s);
  else         // 64-token x 64-expert tiles, 4 waves
    rc = xb ? pk_x3mm::launch<2, 2, true, true, bf16_t, float>(p, pk_timing::K_GATE_LOGITS, s)
            : pk_x3mm::launch<2, 2, true, true, float, float>(p, pk_timing::K_GATE_LOGITS, s);
  if (rc != PK_OK) return rc;
  if (sp > 1) {
    const int64_t n = T * E;
    PK_LAUNCH_NOCHECK(pk_timing::K_GATE_LOGITS, s, pk_f32mm::reduce_partials_kernel,
                      dim3((unsigned)pk_ceil_div(n, 256)), dim3(256), 0, s,
                      reinterpret_cast<const float*>(workspace), logits, n, sp, 0, gate_bias, (int)E);
    PK_RETURN_IF_LAUNCH_FAILED();
  }
  return PK_OK;
}

static int gate_bwd_splits(int64_t T) {
  int64_t sp = T / 256;
  return (int)(sp < 1 ? 1 : (sp > 16 ? 16 : sp));
}

// workspace of the backward: [split-K partials of d_w_gate, reused for the bias partial sums]
// [d_logits as three bf16 planes, for the weight gradient]
static int64_t gate_bwd_partial_bytes(int64_t T, int64_t H, int64_t E) {
  const int sp = gate_bwd_splits(T);
  const int64_t part = sp > 1 ? (int64_t)sp * E * H * (int64_t)sizeof(float) : 0;
  const int64_t colsum = (int64_t)kColsumBlocks * E * (int64_t)sizeof(float);
  return align256(part > colsum ? part : colsum);
}

int64_t pk_gate_bwd_workspace_bytes(int64_t T, int64_t H, int64_t E) {
  if (T < 0 || H <= 0 || E <= 0) return PK_ERR_ARG;
  return gate_bwd_partial_bytes(T, H, E) + plane_bytes(T * E);
}

int pk_gate_logits_bwd(const float* d_logits, const void* x, int x_dtype, const float* w_gate,
                       float* d_x_f32, float* d_w_gate, float* d_gate_bias, int accumulate,
                       int64_t T, int64_t H, int64_t E, void* workspace, int64_t workspace_bytes,
                       pk_stream_t stream) {
  if (T < 0 || H <= 0 || E <= 0 || !pk_dtype_ok(x_dtype)) return PK_ERR_ARG;
  if (!d_logits && T > 0) return PK_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  using pk_x3mm::split3_t;
  const int64_t part_bytes = gate_bwd_partial_bytes(T, H, E);
  const bool have_ws = workspace && reinterpret_cast<uintptr_t>(workspace) % 16 == 0;
  const bool have_part = have_ws && workspace_bytes >= part_bytes;
  if (d_x_f32 && T > 0) {
    if (!w_gate) return PK_ERR_ARG;
    pk_f32mm::Params p = {};
    p.A = d_logits; p.B = w_gate; p.C = d_x_f32;
    p.M = T; p.N = H; p.K = E;
    p.sam = E; p.sak = 1; p.sbk = H; p.sbn = 1;
    p.splits = 1; p.accumulate = 0;
    int rc = pk_x3mm::launch<2, 2, true, false, float, float>(p, pk_timing::K_GATE_LOGITS_BWD, s);
    if (rc != PK_OK) return rc;
  }
  if (d_w_gate) {
    if (!x && T > 0) return PK_ERR_ARG;
    int sp = gate_bwd_splits(T);
    if (sp > 1 && !have_part) sp = 1;
    pk_f32mm::Params p = {};
    p.B = x;
    p.C = sp > 1 ? reinterpret_cast<float*>(workspace) : d_w_gate;
    p.M = E; p.N = H; p.K = T;
    p.sam = 1; p.sak = E; p.sbk = H; p.sbn = 1;
    p.splits = sp; p.accumulate = (sp == 1 && accumulate) ? 1 : 0;
    // d_logits, whose every tile is read by H / 64 workgroups, is split into its three bf16 planes
    // once when the workspace has room for them (this GEMM at 16,384 tokens: 74 -> 61 us, the split
    // included); the kernel splits the tiles it loads otherwise
    const int64_t pb = plane_bytes(T * E);
    const bool presplit = T > 0 && have_ws && pb > 0 && E % 4 == 0 && workspace_bytes >= part_bytes + pb &&
                          reinterpret_cast<uintptr_t>(d_logits) % 16 == 0;
    int rc = PK_ERR_ALIGN;
    if (presplit) {
      bf16_t* planes = reinterpret_cast<bf16_t*>(reinterpret_cast<char*>(workspace) + part_bytes);
      rc = split_planes(d_logits, planes, T * E, pk_timing::K_GATE_LOGITS_BWD, s);
      if (rc != PK_OK) return rc;
      p.A = planes; p.plane_a = T * E;
      rc = x_dtype == PK_BF16 ? pk_x3mm::launch<2, 2, false, false, split3_t, bf16_t>(p, pk_timing::K_GATE_LOGITS_BWD, s)
                              : pk_x3mm::launch<2, 2, false, false, split3_t, float>(p, pk_timing::K_GATE_LOGITS_BWD, s);
    }
    if (rc == PK_ERR_ALIGN) {  // no planes, or x cannot be read four elements at a time
      p.A = d_logits;
      rc = x_dtype == PK_BF16 ? pk_x3mm::launch<2, 2, false, false, float, bf16_t>(p, pk_timing::K_GATE_LOGITS_BWD, s)
                              : pk_x3mm::launch<2, 2, false, false, float, float>(p, pk_timing::K_GATE_LOGITS_BWD, s);
    }
    if (rc != PK_OK) return rc;
    if (sp > 1) {
      const int64_t n = E * H;
      PK_LAUNCH_NOCHECK(pk_timing::K_GATE_LOGITS_BWD, s, pk_f32mm::reduce_partials_kernel,
                        dim3((unsigned)pk_ceil_div(n, 256)), dim3(256), 0, s,
                        reinterpret_cast<const float*>(workspace), d_w_gate, n, sp, accumulate ? 1 : 0,
                        (const float*)nullptr, 1);
      PK_RETURN_IF_LAUNCH_FAILED();
    }
  }
  if (d_gate_bias) {
    // (the first part of the workspace is free again here: the reduction above has consumed the GEMM's partial results)
    const int64_t colsum_bytes = (int64_t)kColsumBlocks * E * (int64_t)sizeof(float);
    if (T >= 32 * kColsumBlocks && E % 4 == 0 && E <= 1024 && workspace && workspace_bytes >= colsum_bytes &&
        reinterpret_cast<uintptr_t>(d_logits) % 16 == 0) {
      float* part = reinterpret_cast<float*>(workspace);
      PK_LAUNCH_NOCHECK(pk_timing::K_MISC, s, colsum_partial_kernel, dim3(kColsumBlocks), dim3(256), 0, s, d_logits, T,
                        (int)E, part);
      PK_RETURN_IF_LAUNCH_FAILED();
      PK_LAUNCH_NOCHECK(pk_timing::K_MISC, s, colsum_final_kernel, dim3((unsigned)pk_ceil_div(E, 256)), dim3(256), 0, s,
                        (const float*)part, kColsumBlocks, (int)E, d_gate_bias, accumulate ? 1 : 0);
      PK_RETURN_IF_LAUNCH_FAILED();
    } else {
      PK_LAUNCH_NOCHECK(pk_timing::K_MISC, s, colsum_kernel, dim3((unsigned)E), dim3(256), 0, s, d_logits, T, (int)E,
                         d_gate_bias, accumulate ? 1 : 0);
      PK_RETURN_IF_LAUNCH_FAILED();
    }
  }
  return PK_OK;
}

#define PK_DISPATCH_EPL(E, LAUNCH)                 \
  do {                                             \
    if ((E) <= 64) { LAUNCH(1); }                  \
    else if ((E) <= 128) { LAUNCH(2); }            \
    else if ((E) <= 256) { LAUNCH(4); }            \
    else if ((E) <= 512) { LAUNCH(8); }            \
    else { LAUNCH(16); }                           \
  } while (0)

int pk_route_topk(const float* logits, int64_t T, int64_t E, int64_t K, int route_norm,
                  float route_scale, float* top_scores, int32_t* top_idx, pk_stream_t stream) {
  if (T < 0 || E <= 0 || K <= 0) return PK_ERR_ARG;
  if (E > PK_MAX_EXPERTS || K > PK_MAX_TOPK || K > E) return PK_ERR_SHAPE;
  if (T == 0) return PK_OK;
  if (!logits || !top_scores || !top_idx) return PK_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)pk_ceil_div(T, kRouteThreads / 64)), block(kRouteThreads);
#define PK_LAUNCH_TOPK(EPL)                                                                 \
  PK_LAUNCH_NOCHECK(pk_timing::K_ROUTE_TOPK, s, (route_topk_kernel<EPL>), grid, block, 0, s, logits, (int)T, (int)E,   \
                     (int)K, route_norm, route_scale, top_scores, top_idx)
  PK_DISPATCH_EPL(E, PK_LAUNCH_TOPK);
#undef PK_LAUNCH_TOPK
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int pk_route_topk_bwd(const float* logits, const int32_t* top_idx, const float* d_top_scores,
                      int64_t T, int64_t E, int64_t K, int route_norm, float route_scale,
                      float* d_logits, pk_stream_t stream) {
  if (T < 0 || E <= 0 || K <= 0) return PK_ERR_ARG;
  if (E > PK_MAX_EXPERTS || K > PK_MAX_TOPK || K > E) return PK_ERR_SHAPE;
  if (T == 0) return PK_OK;
  if (!logits || !top_idx || !d_top_scores || !d_logits) return PK_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)pk_ceil_div(T, kRouteThreads / 64)), block(kRouteThreads);
#define PK_LAUNCH_TOPK_BWD(EPL)                                                              \
  PK_LAUNCH_NOCHECK(pk_timing::K_ROUTE_TOPK_BWD, s, (route_topk_bwd_kernel<EPL>), grid, block, 0, s, logits, top_idx,       \
                     d_top_scores, (int)T, (int)E, (int)K, route_norm, route_scale, d_logits)
  PK_DISPATCH_EPL(E, PK_LAUNCH_TOPK_BWD);
#undef PK_LAUNCH_TOPK_BWD
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int64_t pk_sort_workspace_bytes(int64_t A, int64_t E) {
  if (A < 0 || E <= 0) return PK_ERR_ARG;
  const int64_t nchunks = pk_ceil_div(A > 0 ? A : 1, kSortChunk);
  return nchunks * E * (int64_t)sizeof(int32_t);
}

int pk_sort_by_expert(const int32_t* top_idx, int64_t A, int64_t E, int32_t* counts,
                      int32_t* starts, int32_t* perm, int32_t* inv_perm, int32_t* order,
                      void* workspace, int64_t workspace_bytes, pk_stream_t stream) {
  if (A < 0 || E <= 0) return PK_ERR_ARG;
  if (E > PK_MAX_EXPERTS || A > 0x7fffffffll) return PK_ERR_SHAPE;
  if (!starts || !workspace || (A > 0 && (!top_idx || !perm))) return PK_ERR_ARG;
  if (workspace_bytes < pk_sort_workspace_bytes(A, E)) return PK_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const int nchunks = (int)pk_ceil_div(A > 0 ? A : 1, kSortChunk);
  int32_t* chunk_hist = reinterpret_cast<int32_t*>(workspace);
  const size_t lds = (size_t)E * sizeof(int32_t);
  PK_LAUNCH_NOCHECK(pk_timing::K_SORT_HIST, s, sort_hist_kernel, dim3(nchunks), dim3(64), lds, s, top_idx, (int)A, (int)E,
                     chunk_hist);
  PK_RETURN_IF_LAUNCH_FAILED();
  PK_LAUNCH_NOCHECK(pk_timing::K_SORT_SCAN, s, sort_scan_kernel, dim3(1), dim3(1024), 0, s, chunk_hist, nchunks, (int)E,
                     counts, starts, order);
  PK_RETURN_IF_LAUNCH_FAILED();
  if (A > 0) {
    PK_LAUNCH_NOCHECK(pk_timing::K_SORT_SCATTER, s, sort_scatter_kernel, dim3(nchunks), dim3(64), lds, s, top_idx, (int)A,
                       (int)E, chunk_hist, perm, inv_perm);
    PK_RETURN_IF_LAUNCH_FAILED();
  }
  return PK_OK;
}

int pk_sort_by_expert_static(const int32_t* top_idx, int64_t A, int64_t E, int32_t* counts,
                             int32_t* starts, int32_t* perm, int32_t* inv_perm, int32_t* order,
                             pk_stream_t stream) {
  if (A < 0 || E <= 0) return PK_ERR_ARG;
  if (E > PK_MAX_EXPERTS || A > 0x7fffffffll) return PK_ERR_SHAPE;
  // the per-chunk histograms must fit the fixed scratch array
  const int64_t need = pk_sort_workspace_bytes(A, E);
  if (need > (int64_t)sizeof(int32_t) * PK_SORT_STATIC_WORDS) return PK_ERR_WORKSPACE;
  int32_t* ws = sort_scratch_for_current_device();
  if (!ws) return PK_ERR_UNSUPPORTED;
  return pk_sort_by_expert(top_idx, A, E, counts, starts, perm, inv_perm, order, ws, need, stream);
}

int pk_counts_to_starts(const void* counts, int counts_is_i64, int64_t E, int32_t* starts,
                        pk_stream_t stream) {
  if (E <= 0 || !counts || !starts) return PK_ERR_ARG;
  if (E > PK_MAX_EXPERTS) return PK_ERR_SHAPE;
  PK_LAUNCH_NOCHECK(pk_timing::K_COUNTS_TO_STARTS, (hipStream_t)stream, counts_to_starts_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, counts,
                     counts_is_i64, (int)E, starts);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

}  // extern "C"
