// ZeRO bucket path: multi-tensor pack/unpack, zero fill, fused AdamW over an fp32 bucket.
// All kernels are pure HBM streams: 16 bytes per lane per access, no LDS (the layout does
// not change, so staging through LDS would only add latency).
#include "pk_common.h"

namespace {

constexpr int kPackThreads = 256;
// One 16-byte source vector per lane and no loop: measured on MI355X (bf16 -> fp32, 170 M
// elements) 6.5 TB/s against 5.8 with two and 5.4 with four vectors per lane; the hardware hides
// latency better with many short-lived waves than with longer ones.
constexpr int kPackElemsPerThread = 8;
constexpr int kPackChunk = kPackThreads * kPackElemsPerThread;  // elements per block
constexpr int kPackTensorsPerLaunch = 120;                       // keeps kernargs < 4 KiB

struct PackArgs {
  const void* src[kPackTensorsPerLaunch];
  int64_t off[kPackTensorsPerLaunch];    // element offset into the flat bucket
  int64_t numel[kPackTensorsPerLaunch];
  int32_t blk_start[kPackTensorsPerLaunch + 1];  // first block of tensor i
  int32_t n;
};

template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&f)[8]);
template <>
__device__ __forceinline__ void load8<float>(const float* p, float (&f)[8]) {
  floatx4_t a = *reinterpret_cast<const floatx4_t*>(p);
  floatx4_t b = *reinterpret_cast<const floatx4_t*>(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) { f[i] = a[i]; f[4 + i] = b[i]; }
}
template <>
__device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float (&f)[8]) {
  bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = (float)a[i];
}
// The same for a source that is read once and not again (per-tensor gradients on their way into
// the bucket): a nontemporal load keeps it from displacing lines that are (+5 % on the pack).
template <typename T>
__device__ __forceinline__ void load8_stream(const T* p, float (&f)[8]);
template <>
__device__ __forceinline__ void load8_stream<float>(const float* p, float (&f)[8]) {
  floatx4_t a = __builtin_nontemporal_load(reinterpret_cast<const floatx4_t*>(p));
  floatx4_t b = __builtin_nontemporal_load(reinterpret_cast<const floatx4_t*>(p + 4));
#pragma unroll
  for (int i = 0; i < 4; ++i) { f[i] = a[i]; f[4 + i] = b[i]; }
}
template <>
__device__ __forceinline__ void load8_stream<bf16_t>(const bf16_t* p, float (&f)[8]) {
  bf16x8_t a = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(p));
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = (float)a[i];
}
template <typename T>
__device__ __forceinline__ void store8(T* p, const float (&f)[8]);
template <>
__device__ __forceinline__ void store8<float>(float* p, const float (&f)[8]) {
  floatx4_t a, b;
#pragma unroll
  for (int i = 0; i < 4; ++i) { a[i] = f[i]; b[i] = f[4 + i]; }
  *reinterpret_cast<floatx4_t*>(p) = a;
  *reinterpret_cast<floatx4_t*>(p + 4) = b;
}
template <>
__device__ __forceinline__ void store8<bf16_t>(bf16_t* p, const float (&f)[8]) {
  bf16x8_t a;
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = (bf16_t)f[i];
  *reinterpret_cast<bf16x8_t*>(p) = a;
}

// One block moves one kPackChunk-element chunk of one tensor.
// TO_FLAT: src[i] -> flat (+ accumulate); otherwise flat -> tensor i.
template <typename TS, typename TD, bool ACC, bool TO_FLAT>
__global__ __launch_bounds__(kPackThreads) void pack_kernel(const PackArgs args, void* flat_) {
  // uniform binary search: which tensor owns this block
  int lo = 0, hi = args.n;  // blk_start[lo] <= blockIdx.x < blk_start[hi]
  const int b = blockIdx.x;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (args.blk_start[mid] <= b) lo = mid; else hi = mid;
  }
  const int ti = lo;
  const int64_t numel = args.numel[ti];
  const int64_t base = (int64_t)(b - args.blk_start[ti]) * kPackChunk;
  const int64_t cnt = (numel - base) < (int64_t)kPackChunk ? (numel - base) : (int64_t)kPackChunk;

  const TS* src;
  TD* dst;
  if (TO_FLAT) {
    src = reinterpret_cast<const TS*>(args.src[ti]) + base;
    dst = reinterpret_cast<TD*>(flat_) + args.off[ti] + base;
  } else {
    src = reinterpret_cast<const TS*>(flat_) + args.off[ti] + base;
    dst = reinterpret_cast<TD*>(const_cast<void*>(args.src[ti])) + base;
  }
  const bool vec_ok = ((((uintptr_t)src) | ((uintptr_t)dst)) & 15u) == 0;
  if (vec_ok) {
    const int64_t nvec = cnt >> 3;
#pragma unroll
    for (int j = 0; j < kPackElemsPerThread / 8; ++j) {
      const int64_t v = (int64_t)threadIdx.x + (int64_t)j * kPackThreads;
      if (v < nvec) {
        float f[8];
        if (TO_FLAT) load8_stream<TS>(src + v * 8, f);
        else load8<TS>(src + v * 8, f);
        if (ACC) {
          float d[8];
          load8<TD>(dst + v * 8, d);
#pragma unroll
          for (int i = 0; i < 8; ++i) f[i] = d[i] + f[i];
        }
        store8<TD>(dst + v * 8, f);
      }
    }
    for (int64_t i = (nvec << 3) + threadIdx.x; i < cnt; i += kPackThreads) {
      float f = pk_to_float<TS>(src[i]);
      if (ACC) f = pk_to_float<TD>(dst[i]) + f;
      dst[i] = pk_from_float<TD>(f);
    }
  } else {
    for (int64_t i = threadIdx.x; i < cnt; i += kPackThreads) {
      float f = pk_to_float<TS>(src[i]);
      if (ACC) f = pk_to_float<TD>(dst[i]) + f;
      dst[i] = pk_from_float<TD>(f);
    }
  }
}

template <typename TS, typename TD, bool ACC, bool TO_FLAT>
int launch_pack(const PackArgs& a, int nblocks, void* flat, hipStream_t s) {
  PK_LAUNCH_NOCHECK(TO_FLAT ? pk_timing::K_BUCKET_PACK : pk_timing::K_BUCKET_UNPACK, s, (pack_kernel<TS, TD, ACC, TO_FLAT>), dim3(nblocks), dim3(kPackThreads), 0, s,
                     a, flat);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

template <bool TO_FLAT>
int dispatch_pack(const PackArgs& a, int nblocks, void* flat, int sd, int dd, int acc,
                  hipStream_t s) {
  // sd = dtype of the reading side, dd = dtype of the writing side
  if (sd == PK_BF16 && dd == PK_F32)
    return acc ? launch_pack<bf16_t, float, true, TO_FLAT>(a, nblocks, flat, s)
               : launch_pack<bf16_t, float, false, TO_FLAT>(a, nblocks, flat, s);
  if (sd == PK_F32 && dd == PK_F32)
    return acc ? launch_pack<float, float, true, TO_FLAT>(a, nblocks, flat, s)
               : launch_pack<float, float, false, TO_FLAT>(a, nblocks, flat, s);
  if (sd == PK_BF16 && dd == PK_BF16)
    return acc ? launch_pack<bf16_t, bf16_t, true, TO_FLAT>(a, nblocks, flat, s)
               : launch_pack<bf16_t, bf16_t, false, TO_FLAT>(a, nblocks, flat, s);
  if (sd == PK_F32 && dd == PK_BF16)
    return acc ? launch_pack<float, bf16_t, true, TO_FLAT>(a, nblocks, flat, s)
               : launch_pack<float, bf16_t, false, TO_FLAT>(a, nblocks, flat, s);
  return PK_ERR_UNSUPPORTED;
}

int pack_or_unpack(const void* const* ptrs, const int64_t* offsets, const int64_t* numels,
                   int64_t n, int tensor_dtype, void* flat, int flat_dtype, int accumulate,
                   bool to_flat, hipStream_t s) {
  if (n < 0 || (n > 0 && (!ptrs || !offsets || !numels)) || !pk_dtype_ok(tensor_dtype) ||
      !pk_dtype_ok(flat_dtype))
    return PK_ERR_ARG;
  if (n > 0 && !flat) return PK_ERR_ARG;
  for (int64_t i = 0; i < n; ++i)
    if (numels[i] < 0 || offsets[i] < 0) return PK_ERR_ARG;
  int64_t i = 0;
  while (i < n) {
    PackArgs a;
    a.n = 0;
    int64_t blocks = 0;
    while (i < n && a.n < kPackTensorsPerLaunch) {
      if (ptrs[i] != nullptr && numels[i] > 0) {
        const int64_t nb = pk_ceil_div(numels[i], kPackChunk);
        if (blocks + nb > 0x7fffffff) break;  // next launch
        a.src[a.n] = ptrs[i];
        a.off[a.n] = offsets[i];
        a.numel[a.n] = numels[i];
        a.blk_start[a.n] = (int32_t)blocks;
        blocks += nb;
        ++a.n;
      }
      ++i;
    }
    if (a.n == 0) {
      if (i < n) return PK_ERR_SHAPE;  // a single tensor larger than 2^31 blocks
      break;
    }
    a.blk_start[a.n] = (int32_t)blocks;
    int rc = to_flat ? dispatch_pack<true>(a, (int)blocks, flat, tensor_dtype, flat_dtype, accumulate, s)
                     : dispatch_pack<false>(a, (int)blocks, flat, flat_dtype, tensor_dtype, 0, s);
    if (rc != PK_OK) return rc;
  }
  return PK_OK;
}

// ------------------------------------------------------------------ zero fill
constexpr int kStreamThreads = 256;

__global__ __launch_bounds__(kStreamThreads) void zero_kernel(float* p, int64_t n) {
  const int64_t nvec = n >> 2;
  const int64_t stride = (int64_t)gridDim.x * kStreamThreads;
  floatx4_t z = {0.f, 0.f, 0.f, 0.f};
  for (int64_t v = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x; v < nvec; v += stride)
    reinterpret_cast<floatx4_t*>(p)[v] = z;
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) p[(nvec << 2) + threadIdx.x] = 0.f;
}

// ------------------------------------------------------------------ fused AdamW
struct AdamArgs {
  float decay;        // 1 - lr*wd
  float one_m_b1;     // 1 - beta1
  float beta2;
  float one_m_b2;     // 1 - beta2
  float step_size;    // lr / (1 - beta1^step)
  float bc2_sqrt;     // sqrt(1 - beta2^step); torch divides by it, so does the kernel
  float eps;
  float grad_scale;
};

__device__ __forceinline__ void adam_update(float& p, float& m, float& v, float g,
                                            const AdamArgs& a) {
  g *= a.grad_scale;
  p = p * a.decay;
  m = m + (g - m) * a.one_m_b1;
  v = v * a.beta2 + (a.one_m_b2 * g) * g;
  const float denom = sqrtf(v) / a.bc2_sqrt + a.eps;
  p = p - a.step_size * (m / denom);
}

template <typename TSH, bool SHADOW, bool ZERO>
__global__ __launch_bounds__(kStreamThreads) void adamw_kernel(
    float* __restrict__ master, float* __restrict__ exp_avg, float* __restrict__ exp_avg_sq,
    float* __restrict__ grad, TSH* __restrict__ shadow, int64_t n, const AdamArgs a) {
  // One float4 per lane per stream and no grid-stride loop: measured fastest on MI355X
  // (5.8 TB/s vs 4.5 TB/s for a 4096-block grid-stride loop); nontemporal on every stream.
  const int64_t nvec = n >> 2;
  const int64_t i = (int64_t)blockIdx.x * kStreamThreads + threadIdx.x;
  if (i < nvec) {
    floatx4_t p = __builtin_nontemporal_load(reinterpret_cast<floatx4_t*>(master) + i);
    floatx4_t m = __builtin_nontemporal_load(reinterpret_cast<floatx4_t*>(exp_avg) + i);
    floatx4_t v = __builtin_nontemporal_load(reinterpret_cast<floatx4_t*>(exp_avg_sq) + i);
    floatx4_t g = __builtin_nontemporal_load(reinterpret_cast<floatx4_t*>(grad) + i);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float pj = p[j], mj = m[j], vj = v[j];
      adam_update(pj, mj, vj, g[j], a);
      p[j] = pj; m[j] = mj; v[j] = vj;
    }
    __builtin_nontemporal_store(p, reinterpret_cast<floatx4_t*>(master) + i);
    __builtin_nontemporal_store(m, reinterpret_cast<floatx4_t*>(exp_avg) + i);
    __builtin_nontemporal_store(v, reinterpret_cast<floatx4_t*>(exp_avg_sq) + i);
    if (SHADOW) {
      if (sizeof(TSH) == 2) {
        bf16x4_t s;
#pragma unroll
        for (int j = 0; j < 4; ++j) s[j] = (bf16_t)p[j];
        __builtin_nontemporal_store(s, reinterpret_cast<bf16x4_t*>(shadow) + i);
      } else {
        __builtin_nontemporal_store(p, reinterpret_cast<floatx4_t*>(shadow) + i);
      }
    }
    if (ZERO) {
      floatx4_t z = {0.f, 0.f, 0.f, 0.f};
      __builtin_nontemporal_store(z, reinterpret_cast<floatx4_t*>(grad) + i);
    }
  }
  // scalar tail (n % 4 elements), handled by the first block
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
    const int64_t i = (nvec << 2) + threadIdx.x;
    float pj = master[i], mj = exp_avg[i], vj = exp_avg_sq[i];
    adam_update(pj, mj, vj, grad[i], a);
    master[i] = pj; exp_avg[i] = mj; exp_avg_sq[i] = vj;
    if (SHADOW) shadow[i] = pk_from_float<TSH>(pj);
    if (ZERO) grad[i] = 0.f;
  }
}

// AdamW with the last gradient pack folded in: the gradient of an element is what the fp32 bucket
// holds (earlier microbatches; optional) plus the per-tensor gradient of the last microbatch, read
// in its own dtype straight from the tensor.  One block updates kAdamPackChunk elements of one
// tensor (four per lane: one 16-byte vector per fp32 stream, as in adamw_kernel); bucket elements
// that belong to no tensor (alignment padding) are not touched.
constexpr int kAdamPackChunk = kStreamThreads * 4;

template <typename TG, typename TSH, bool SHADOW, bool FLAT, bool ZERO>
__global__ __launch_bounds__(kStreamThreads) void adamw_packed_kernel(
    const PackArgs args, float* __restrict__ master, float* __restrict__ exp_avg, float* __restrict__ exp_avg_sq,
    float* __restrict__ flat_grad, TSH* __restrict__ shadow, const AdamArgs a) {
  int lo = 0, hi = args.n;  // blk_start[lo] <= blockIdx.x < blk_start[hi]
  const int b = blockIdx.x;
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (args.blk_start[mid] <= b) lo = mid; else hi = mid;
  }
  const int ti = lo;
  const int64_t numel = args.numel[ti];
  const int64_t base = (int64_t)(b - args.blk_start[ti]) * kAdamPackChunk;
  const int64_t cnt = (numel - base) < (int64_t)kAdamPackChunk ? (numel - base) : (int64_t)kAdamPackChunk;
  const TG* src = args.src[ti] ? reinterpret_cast<const TG*>(args.src[ti]) + base : nullptr;
  const int64_t o = args.off[ti] + base;
  const bool src_vec = ((uintptr_t)src & (sizeof(TG) * 4 - 1)) == 0;
  const int64_t e = (int64_t)threadIdx.x * 4;
  if (e + 4 <= cnt && ((o & 3) == 0)) {
    floatx4_t p = __builtin_nontemporal_load(reinterpret_cast<floatx4_t*>(master + o + e));
    floatx4_t m = __builtin_nontemporal_load(reinterpret_cast<floatx4_t*>(exp_avg + o + e));
    floatx4_t v = __builtin_nontemporal_load(reinterpret_cast<floatx4_t*>(exp_avg_sq + o + e));
    floatx4_t g = {0.f, 0.f, 0.f, 0.f};
    if (FLAT) g = __builtin_nontemporal_load(reinterpret_cast<floatx4_t*>(flat_grad + o + e));
    if (src) {
      float t[4];
      if (src_vec) {
        if (sizeof(TG) == 2) {
          const bf16x4_t r = __builtin_nontemporal_load(reinterpret_cast<const bf16x4_t*>(src + e));
#pragma unroll
          for (int j = 0; j < 4; ++j) t[j] = (float)r[j];
        } else {
          const floatx4_t r = __builtin_nontemporal_load(reinterpret_cast<const floatx4_t*>(src + e));
#pragma unroll
          for (int j = 0; j < 4; ++j) t[j] = r[j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) t[j] = pk_to_float<TG>(src[e + j]);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) g[j] = g[j] + t[j];      // bucket + tensor: the sum the pack kernel stores
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float pj = p[j], mj = m[j], vj = v[j];
      adam_update(pj, mj, vj, g[j], a);
      p[j] = pj; m[j] = mj; v[j] = vj;
    }
    __builtin_nontemporal_store(p, reinterpret_cast<floatx4_t*>(master + o + e));
    __builtin_nontemporal_store(m, reinterpret_cast<floatx4_t*>(exp_avg + o + e));
    __builtin_nontemporal_store(v, reinterpret_cast<floatx4_t*>(exp_avg_sq + o + e));
    if (SHADOW) {
      if (sizeof(TSH) == 2) {
        bf16x4_t sh;
#pragma unroll
        for (int j = 0; j < 4; ++j) sh[j] = (bf16_t)p[j];
        __builtin_nontemporal_store(sh, reinterpret_cast<bf16x4_t*>(shadow + o + e));
      } else {
        __builtin_nontemporal_store(p, reinterpret_cast<floatx4_t*>(shadow + o + e));
      }
    }
    if (FLAT && ZERO) {
      floatx4_t z = {0.f, 0.f, 0.f, 0.f};
      __builtin_nontemporal_store(z, reinterpret_cast<floatx4_t*>(flat_grad + o + e));
    }
  } else {
    for (int64_t i = e; i < cnt && i < e + 4; ++i) {     // a tensor's last elements, unaligned offsets
      float pj = master[o + i], mj = exp_avg[o + i], vj = exp_avg_sq[o + i];
      float gj = FLAT ? flat_grad[o + i] : 0.f;
      if (src) gj = gj + pk_to_float<TG>(src[i]);
      adam_update(pj, mj, vj, gj, a);
      master[o + i] = pj; exp_avg[o + i] = mj; exp_avg_sq[o + i] = vj;
      if (SHADOW) shadow[o + i] = pk_from_float<TSH>(pj);
      if (FLAT && ZERO) flat_grad[o + i] = 0.f;
    }
  }
}

AdamArgs make_adam_args(float lr, float beta1, float beta2, float eps, float weight_decay, int64_t step, float grad_scale) {
  // scalar prologue in double, as torch does on the host (python floats)
  const double bc1 = 1.0 - pow((double)beta1, (double)step);
  const double bc2 = 1.0 - pow((double)beta2, (double)step);
  AdamArgs a;
  a.decay = (float)(1.0 - (double)lr * (double)weight_decay);
  a.one_m_b1 = (float)(1.0 - (double)beta1);
  a.beta2 = beta2;
  a.one_m_b2 = (float)(1.0 - (double)beta2);
  a.step_size = (float)((double)lr / bc1);
  a.bc2_sqrt = (float)sqrt(bc2);
  a.eps = eps;
  a.grad_scale = grad_scale;
  return a;
}

int stream_grid(int64_t nvec) {
  // enough blocks to keep every CU busy with several waves, capped so that the grid-stride
  // loop amortises the launch
  int64_t blocks = pk_ceil_div(nvec, kStreamThreads);
  const int64_t cap = 256 * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

}  // namespace

extern "C" {

int64_t pk_bucket_plan(const int64_t* numels, int64_t n, int64_t elem_size, int64_t align_bytes,
                       int64_t* offsets) {
  if (n < 0 || elem_size <= 0 || align_bytes <= 0 || (n > 0 && (!numels || !offsets)))
    return PK_ERR_ARG;
  if ((align_bytes & (align_bytes - 1)) != 0) return PK_ERR_ARG;
  int64_t align_elems = 1;
  if (align_bytes > elem_size) {
    if (align_bytes % elem_size != 0) return PK_ERR_ARG;
    align_elems = align_bytes / elem_size;
  }
  int64_t cur = 0;
  for (int64_t i = 0; i < n; ++i) {
    if (numels[i] < 0) return PK_ERR_ARG;
    cur = pk_ceil_div(cur, align_elems) * align_elems;
    offsets[i] = cur;
    cur += numels[i];
  }
  return pk_ceil_div(cur, align_elems) * align_elems;
}

int pk_bucket_pack(const void* const* srcs, const int64_t* offsets, const int64_t* numels,
                   int64_t n, int src_dtype, void* flat, int dst_dtype, int accumulate,
                   pk_stream_t stream) {
  return pack_or_unpack(srcs, offsets, numels, n, src_dtype, flat, dst_dtype, accumulate, true,
                        (hipStream_t)stream);
}

int pk_bucket_unpack(const void* flat, int flat_dtype, void* const* dsts, const int64_t* offsets,
                     const int64_t* numels, int64_t n, int dst_dtype, pk_stream_t stream) {
  return pack_or_unpack(const_cast<const void* const*>(dsts), offsets, numels, n, dst_dtype,
                        const_cast<void*>(flat), flat_dtype, 0, false, (hipStream_t)stream);
}

int pk_bucket_zero(float* flat, int64_t n, pk_stream_t stream) {
  if (n < 0 || (n > 0 && !flat)) return PK_ERR_ARG;
  if (n == 0) return PK_OK;
  if (!pk_aligned16(flat)) return PK_ERR_ALIGN;
  PK_LAUNCH_NOCHECK(pk_timing::K_BUCKET_ZERO, (hipStream_t)stream, zero_kernel, dim3(stream_grid(n >> 2)), dim3(kStreamThreads), 0,
                     (hipStream_t)stream, flat, n);
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int pk_adamw_fused(float* master, float* exp_avg, float* exp_avg_sq, float* grad, void* shadow,
                   int shadow_dtype, int64_t n, float lr, float beta1, float beta2, float eps,
                   float weight_decay, int64_t step, float grad_scale, int zero_grad,
                   pk_stream_t stream) {
  if (n < 0 || step < 1) return PK_ERR_ARG;
  if (n == 0) return PK_OK;
  if (!master || !exp_avg || !exp_avg_sq || !grad) return PK_ERR_ARG;
  if (shadow && !pk_dtype_ok(shadow_dtype)) return PK_ERR_ARG;
  if (!pk_aligned16(master) || !pk_aligned16(exp_avg) || !pk_aligned16(exp_avg_sq) ||
      !pk_aligned16(grad) || (shadow && !pk_aligned16(shadow)))
    return PK_ERR_ALIGN;
  const AdamArgs a = make_adam_args(lr, beta1, beta2, eps, weight_decay, step, grad_scale);
  hipStream_t s = (hipStream_t)stream;
  const int64_t nblocks = pk_ceil_div((n >> 2) > 0 ? (n >> 2) : 1, kStreamThreads);
  if (nblocks > 0x7fffffffll) return PK_ERR_SHAPE;
  const dim3 grid((unsigned)nblocks), block(kStreamThreads);
#define PK_ADAM_LAUNCH(TSH, SH, ZE)                                                          \
  PK_LAUNCH_NOCHECK(pk_timing::K_ADAMW, s, (adamw_kernel<TSH, SH, ZE>), grid, block, 0, s, master, exp_avg,        \
                     exp_avg_sq, grad, reinterpret_cast<TSH*>(shadow), n, a)
  if (!shadow) {
    if (zero_grad) PK_ADAM_LAUNCH(float, false, true); else PK_ADAM_LAUNCH(float, false, false);
  } else if (shadow_dtype == PK_BF16) {
    if (zero_grad) PK_ADAM_LAUNCH(bf16_t, true, true); else PK_ADAM_LAUNCH(bf16_t, true, false);
  } else {
    if (zero_grad) PK_ADAM_LAUNCH(float, true, true); else PK_ADAM_LAUNCH(float, true, false);
  }
#undef PK_ADAM_LAUNCH
  PK_RETURN_IF_LAUNCH_FAILED();
  return PK_OK;
}

int pk_adamw_fused_packed(float* master, float* exp_avg, float* exp_avg_sq, float* flat_grad,
                          const void* const* grads, const int64_t* offsets, const int64_t* numels, int64_t n,
                          int grad_dtype, void* shadow, int shadow_dtype, float lr, float beta1, float beta2,
                          float eps, float weight_decay, int64_t step, float grad_scale, int zero_grad,
                          pk_stream_t stream) {
  if (n < 0 || step < 1 || !pk_dtype_ok(grad_dtype)) return PK_ERR_ARG;
  if (n == 0) return PK_OK;
  if (!master || !exp_avg || !exp_avg_sq || !grads || !offsets || !numels) return PK_ERR_ARG;
  if (shadow && shadow_dtype != PK_BF16) return PK_ERR_UNSUPPORTED;
  if (!pk_aligned16(master) || !pk_aligned16(exp_avg) || !pk_aligned16(exp_avg_sq) ||
      (flat_grad && !pk_aligned16(flat_grad)) || (shadow && !pk_aligned16(shadow)))
    return PK_ERR_ALIGN;
  for (int64_t i = 0; i < n; ++i)
    if (numels[i] < 0 || offsets[i] < 0) return PK_ERR_ARG;
  const AdamArgs a = make_adam_args(lr, beta1, beta2, eps, weight_decay, step, grad_scale);
  hipStream_t s = (hipStream_t)stream;
  int64_t i = 0;
  while (i < n) {
    PackArgs pa;
    pa.n = 0;
    int64_t blocks = 0;
    while (i < n && pa.n < kPackTensorsPerLaunch) {
      if (numels[i] > 0) {      // a tensor without a gradient of its own is still stepped (decay, moments)
        const int64_t nb = pk_ceil_div(numels[i], kAdamPackChunk);
        if (blocks + nb > 0x7fffffff) break;
        pa.src[pa.n] = grads[i];
        pa.off[pa.n] = offsets[i];
        pa.numel[pa.n] = numels[i];
        pa.blk_start[pa.n] = (int32_t)blocks;
        blocks += nb;
        ++pa.n;
      }
      ++i;
    }
    if (pa.n == 0) {
      if (i < n) return PK_ERR_SHAPE;
      break;
    }
    pa.blk_start[pa.n] = (int32_t)blocks;
    const dim3 grid((unsigned)blocks), block(kStreamThreads);
#define PK_ADAMP(TG, SH, FL, ZE)                                                                               \
  PK_LAUNCH_NOCHECK(pk_timing::K_ADAMW, s, (adamw_packed_kernel<TG, bf16_t, SH, FL, ZE>), grid, block, 0, s, pa, master, \
                    exp_avg, exp_avg_sq, flat_grad, reinterpret_cast<bf16_t*>(shadow), a)
#define PK_ADAMP_G(TG)                                                                       \
  do {                                                                                       \
    if (shadow) {                                                                            \
      if (!flat_grad) PK_ADAMP(TG, true, false, false);                                      \
      else if (zero_grad) PK_ADAMP(TG, true, true, true);                                    \
      else PK_ADAMP(TG, true, true, false);                                                  \
    } else {                                                                                 \
      if (!flat_grad) PK_ADAMP(TG, false, false, false);                                     \
      else if (zero_grad) PK_ADAMP(TG, false, true, true);                                   \
      else PK_ADAMP(TG, false, true, false);                                                 \
    }                                                                                        \
  } while (0)
    if (grad_dtype == PK_BF16) PK_ADAMP_G(bf16_t);
    else PK_ADAMP_G(float);
#undef PK_ADAMP_G
#undef PK_ADAMP
    PK_RETURN_IF_LAUNCH_FAILED();
  }
  return PK_OK;
}

}  // extern "C"
