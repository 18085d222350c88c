// Optimizer-step kernels over flat fp32 buffers: fused AdamW, fp64 sum of squares, scaling and
// the low-precision -> fp32 gradient reduce.  All are single-pass HBM streams: 16-byte loads and
// stores, several independent vectors in flight per lane, no LDS.
#include "common.hpp"

namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;  // float4 vectors per lane per block tile

struct AdamArgs {
  float lr, beta1, beta2, eps, weight_decay;
  float step_size;   // lr / (1 - beta1^t)
  float bc2_sqrt;    // sqrt(1 - beta2^t)
  float grad_scale;
  float max_norm;
  const double* sq_norm;
};

__device__ __forceinline__ float clip_coef(const AdamArgs& a) {
  float c = a.grad_scale;
  if (a.sq_norm != nullptr) {
    // clip_coef = max_norm / (norm + 1e-6), evaluated in fp64 as the reference's Python floats are.
    double coef = static_cast<double>(a.max_norm) / (sqrt(*a.sq_norm) + 1e-6);
    if (coef < 1.0) c *= static_cast<float>(coef);
  }
  return c;
}

__device__ __forceinline__ void adam_update(float& p, float g, float& m, float& v, const AdamArgs& a, float c) {
  // rounded product, never contracted into the arithmetic below: clipping inside this kernel then gives the very bits of
  // a separate scaling pass over the gradients followed by an unclipped step, whichever way a caller clips
  g *= c;
  asm volatile("" : "+v"(g));
  p -= a.lr * a.weight_decay * p;
  m = m + (1.0f - a.beta1) * (g - m);
  v = a.beta2 * v + (1.0f - a.beta2) * g * g;
  float denom = sqrtf(v) / a.bc2_sqrt + a.eps;
  p -= a.step_size * m / denom;
}

template <bool LOWP>
__global__ __launch_bounds__(kThreads) void adamw_vec_kernel(float* __restrict__ p, const float* __restrict__ g,
                                                             float* __restrict__ m, float* __restrict__ v,
                                                             bf16_t* __restrict__ plow, int64_t nvec, AdamArgs a) {
  const float c = clip_coef(a);
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
  f32x4 pp[kUnroll], gg[kUnroll], mm[kUnroll], vv[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    int64_t i = base + static_cast<int64_t>(u) * kThreads;
    if (i < nvec) {
      pp[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p) + i);
      gg[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(g) + i);
      mm[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(m) + i);
      vv[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(v) + i);
    }
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    int64_t i = base + static_cast<int64_t>(u) * kThreads;
    if (i < nvec) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float pj = pp[u][j], mj = mm[u][j], vj = vv[u][j];
        adam_update(pj, gg[u][j], mj, vj, a, c);
        pp[u][j] = pj;
        mm[u][j] = mj;
        vv[u][j] = vj;
      }
      __builtin_nontemporal_store(pp[u], reinterpret_cast<f32x4*>(p) + i);
      __builtin_nontemporal_store(mm[u], reinterpret_cast<f32x4*>(m) + i);
      __builtin_nontemporal_store(vv[u], reinterpret_cast<f32x4*>(v) + i);
      if (LOWP) {
        bf16x4 lo;
#pragma unroll
        for (int j = 0; j < 4; ++j) lo[j] = static_cast<bf16_t>(pp[u][j]);
        __builtin_nontemporal_store(lo, reinterpret_cast<bf16x4*>(plow) + i);
      }
    }
  }
}

// Scalar form for the unaligned head/tail of a buffer (at most a few elements) or unaligned views.
template <bool LOWP>
__global__ __launch_bounds__(kThreads) void adamw_scalar_kernel(float* p, const float* g, float* m, float* v,
                                                                bf16_t* plow, int64_t n, AdamArgs a) {
  const float c = clip_coef(a);
  int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  float pj = p[i], mj = m[i], vj = v[i];
  adam_update(pj, g[i], mj, vj, a, c);
  p[i] = pj;
  m[i] = mj;
  v[i] = vj;
  if (LOWP) plow[i] = static_cast<bf16_t>(pj);
}

// ---- sum of squares, fp64 accumulate, two deterministic stages ---------------------------
constexpr int kSqBlocks = 1024;  // partials; 8 KiB of the workspace

__device__ __forceinline__ void block_sum_f64_store(double acc, double* out) {
  __shared__ double part[kThreads / MLTS_WAVE];
  acc = wave_sum_f64(acc);
  if ((threadIdx.x & (MLTS_WAVE - 1)) == 0) part[threadIdx.x / MLTS_WAVE] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double s = 0.0;
#pragma unroll
    for (int w = 0; w < kThreads / MLTS_WAVE; ++w) s += part[w];
    *out = s;
  }
}

__global__ __launch_bounds__(kThreads) void sq_norm_stage1(const float* __restrict__ x, int64_t n, double* partial) {
  // x is 16-byte aligned here; the vector body covers n/4 vectors, lane 0 of block 0 the tail.
  const int64_t nvec = n >> 2;
  double acc = 0.0;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < nvec; i += stride) {
    f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(x) + i);
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = fma(static_cast<double>(t[j]), static_cast<double>(t[j]), acc);
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    for (int64_t i = nvec << 2; i < n; ++i) acc += static_cast<double>(x[i]) * static_cast<double>(x[i]);
  }
  block_sum_f64_store(acc, partial + blockIdx.x);
}

__global__ __launch_bounds__(kThreads) void sq_norm_scalar_stage1(const float* __restrict__ x, int64_t n,
                                                                  double* partial) {
  double acc = 0.0;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
    double t = static_cast<double>(x[i]);
    acc += t * t;
  }
  block_sum_f64_store(acc, partial + blockIdx.x);
}

__global__ __launch_bounds__(kThreads) void sq_norm_stage2(const double* partial, int count, double* out) {
  double acc = 0.0;
  for (int i = threadIdx.x; i < count; i += kThreads) acc += partial[i];
  block_sum_f64_store(acc, out);
}

__global__ __launch_bounds__(kThreads) void scale_kernel(float* x, float s, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) x[i] *= s;
}

__global__ __launch_bounds__(kThreads) void scale_vec_kernel(float* x, float s, int64_t nvec) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < nvec; i += stride) {
    f32x4 t = reinterpret_cast<f32x4*>(x)[i];
    t *= s;
    reinterpret_cast<f32x4*>(x)[i] = t;
  }
}

// dst (=|+=) float(src), optional fp64 sum of squares of the result.  8 elements per lane step.
template <typename T, bool ACC, bool SQ>
__global__ __launch_bounds__(kThreads) void grad_to_f32_kernel(float* __restrict__ dst, const T* __restrict__ src,
                                                               int64_t n, double* partial) {
  double acc = 0.0;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
    float t = to_f32<T>(src[i]);
    if (ACC) t += dst[i];
    dst[i] = t;
    if (SQ) acc += static_cast<double>(t) * static_cast<double>(t);
  }
  if (SQ) block_sum_f64_store(acc, partial + blockIdx.x);
}

template <bool ACC, bool SQ>
__global__ __launch_bounds__(kThreads) void grad_bf16_to_f32_vec_kernel(float* __restrict__ dst,
                                                                        const bf16_t* __restrict__ src,
                                                                        int64_t nvec8, double* partial) {
  double acc = 0.0;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < nvec8; i += stride) {
    bf16x8 s = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(src) + i);
    f32x4 lo, hi;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo[j] = static_cast<float>(s[j]);
      hi[j] = static_cast<float>(s[4 + j]);
    }
    if (ACC) {
      lo += reinterpret_cast<const f32x4*>(dst)[2 * i];
      hi += reinterpret_cast<const f32x4*>(dst)[2 * i + 1];
    }
    reinterpret_cast<f32x4*>(dst)[2 * i] = lo;
    reinterpret_cast<f32x4*>(dst)[2 * i + 1] = hi;
    if (SQ) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc = fma(static_cast<double>(lo[j]), static_cast<double>(lo[j]), acc);
        acc = fma(static_cast<double>(hi[j]), static_cast<double>(hi[j]), acc);
      }
    }
  }
  if (SQ) block_sum_f64_store(acc, partial + blockIdx.x);
}

int grid_for(int64_t work_items, int max_blocks) {
  int64_t b = (work_items + kThreads - 1) / kThreads;
  if (b < 1) b = 1;
  if (b > max_blocks) b = max_blocks;
  return static_cast<int>(b);
}

}  // namespace

extern "C" int mlts_adamw_step(float* p, const float* g, float* m, float* v, void* p_lowp, int64_t n, float lr,
                               float beta1, float beta2, float eps, float weight_decay, int64_t step,
                               float grad_scale, const double* sq_norm, float max_norm, mlts_stream_t stream) {
  MLTS_REQUIRE(n >= 0, "mlts_adamw_step: n must be >= 0, got %lld", (long long)n);
  if (n == 0) return MLTS_OK;
  MLTS_REQUIRE(p && g && m && v, "mlts_adamw_step: p, g, m, v must be non-null");
  MLTS_REQUIRE(step >= 1, "mlts_adamw_step: step is the 1-based step count, got %lld", (long long)step);
  MLTS_REQUIRE(beta1 >= 0.f && beta1 < 1.f && beta2 >= 0.f && beta2 < 1.f, "mlts_adamw_step: betas must be in [0, 1)");
  hipStream_t st = static_cast<hipStream_t>(stream);
  AdamArgs a;
  a.lr = lr;
  a.beta1 = beta1;
  a.beta2 = beta2;
  a.eps = eps;
  a.weight_decay = weight_decay;
  const double bc1 = 1.0 - pow(static_cast<double>(beta1), static_cast<double>(step));
  const double bc2 = 1.0 - pow(static_cast<double>(beta2), static_cast<double>(step));
  a.step_size = static_cast<float>(static_cast<double>(lr) / bc1);
  a.bc2_sqrt = static_cast<float>(sqrt(bc2));
  a.grad_scale = grad_scale;
  a.max_norm = max_norm;
  a.sq_norm = sq_norm;
  bf16_t* plow = static_cast<bf16_t*>(p_lowp);

  const bool vec_ok = mlts_aligned16(p) && mlts_aligned16(g) && mlts_aligned16(m) && mlts_aligned16(v) &&
                      (plow == nullptr || (reinterpret_cast<uintptr_t>(plow) & 7u) == 0);
  int64_t done = 0;
  MltsKernelTimer timer("adamw", st);
  if (vec_ok && n >= 4) {
    const int64_t nvec = n >> 2;
    const int64_t per_block = static_cast<int64_t>(kThreads) * kUnroll;
    const int64_t blocks = (nvec + per_block - 1) / per_block;
    MLTS_REQUIRE(blocks <= 0x7fffffffLL, "mlts_adamw_step: n too large");
    if (plow)
      hipLaunchKernelGGL(adamw_vec_kernel<true>, dim3((unsigned)blocks), dim3(kThreads), 0, st, p, g, m, v, plow, nvec, a);
    else
      hipLaunchKernelGGL(adamw_vec_kernel<false>, dim3((unsigned)blocks), dim3(kThreads), 0, st, p, g, m, v, plow, nvec, a);
    done = nvec << 2;
  }
  if (done < n) {
    const int64_t rem = n - done;
    const int64_t blocks = (rem + kThreads - 1) / kThreads;
    MLTS_REQUIRE(blocks <= 0x7fffffffLL, "mlts_adamw_step: n too large");
    bf16_t* pl = plow ? plow + done : nullptr;
    if (plow)
      hipLaunchKernelGGL(adamw_scalar_kernel<true>, dim3((unsigned)blocks), dim3(kThreads), 0, st, p + done, g + done,
                         m + done, v + done, pl, rem, a);
    else
      hipLaunchKernelGGL(adamw_scalar_kernel<false>, dim3((unsigned)blocks), dim3(kThreads), 0, st, p + done, g + done,
                         m + done, v + done, pl, rem, a);
  }
  return mlts_check_launch("mlts_adamw_step");
}

extern "C" int mlts_sq_norm(const float* x, int64_t n, double* sq_out, void* workspace, mlts_stream_t stream) {
  MLTS_REQUIRE(n >= 0, "mlts_sq_norm: n must be >= 0");
  MLTS_REQUIRE(sq_out && workspace, "mlts_sq_norm: sq_out and workspace must be non-null");
  MLTS_REQUIRE(n == 0 || x, "mlts_sq_norm: x must be non-null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  double* partial = static_cast<double*>(workspace);
  int blocks;
  if (mlts_aligned16(x)) {
    blocks = grid_for(n >> 2, kSqBlocks);
    hipLaunchKernelGGL(sq_norm_stage1, dim3(blocks), dim3(kThreads), 0, st, x, n, partial);
  } else {
    blocks = grid_for(n, kSqBlocks);
    hipLaunchKernelGGL(sq_norm_scalar_stage1, dim3(blocks), dim3(kThreads), 0, st, x, n, partial);
  }
  hipLaunchKernelGGL(sq_norm_stage2, dim3(1), dim3(kThreads), 0, st, partial, blocks, sq_out);
  return mlts_check_launch("mlts_sq_norm");
}

extern "C" int mlts_scale(float* x, float scale, int64_t n, mlts_stream_t stream) {
  MLTS_REQUIRE(n >= 0, "mlts_scale: n must be >= 0");
  if (n == 0) return MLTS_OK;
  MLTS_REQUIRE(x, "mlts_scale: x must be non-null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (mlts_aligned16(x) && (n & 3) == 0) {
    hipLaunchKernelGGL(scale_vec_kernel, dim3(grid_for(n >> 2, 8192)), dim3(kThreads), 0, st, x, scale, n >> 2);
  } else {
    hipLaunchKernelGGL(scale_kernel, dim3(grid_for(n, 8192)), dim3(kThreads), 0, st, x, scale, n);
  }
  return mlts_check_launch("mlts_scale");
}

namespace {
template <typename T>
void launch_grad_to_f32(bool acc, bool sq, int blocks, hipStream_t st, float* dst, const T* src, int64_t n,
                        double* partial) {
  if (acc && sq)
    hipLaunchKernelGGL((grad_to_f32_kernel<T, true, true>), dim3(blocks), dim3(kThreads), 0, st, dst, src, n, partial);
  else if (acc)
    hipLaunchKernelGGL((grad_to_f32_kernel<T, true, false>), dim3(blocks), dim3(kThreads), 0, st, dst, src, n, partial);
  else if (sq)
    hipLaunchKernelGGL((grad_to_f32_kernel<T, false, true>), dim3(blocks), dim3(kThreads), 0, st, dst, src, n, partial);
  else
    hipLaunchKernelGGL((grad_to_f32_kernel<T, false, false>), dim3(blocks), dim3(kThreads), 0, st, dst, src, n, partial);
}
void launch_grad_bf16_vec(bool acc, bool sq, int blocks, hipStream_t st, float* dst, const bf16_t* src, int64_t nvec8,
                          double* partial) {
  if (acc && sq)
    hipLaunchKernelGGL((grad_bf16_to_f32_vec_kernel<true, true>), dim3(blocks), dim3(kThreads), 0, st, dst, src, nvec8, partial);
  else if (acc)
    hipLaunchKernelGGL((grad_bf16_to_f32_vec_kernel<true, false>), dim3(blocks), dim3(kThreads), 0, st, dst, src, nvec8, partial);
  else if (sq)
    hipLaunchKernelGGL((grad_bf16_to_f32_vec_kernel<false, true>), dim3(blocks), dim3(kThreads), 0, st, dst, src, nvec8, partial);
  else
    hipLaunchKernelGGL((grad_bf16_to_f32_vec_kernel<false, false>), dim3(blocks), dim3(kThreads), 0, st, dst, src, nvec8, partial);
}
// out[i] = T((ACC ? float(out[i]) : 0) + sum_s float(parts[s * n + i])): the row-slice partial products of a weight
// gradient added in fp32 and rounded once, optionally onto the gradient already in the buffer.
template <typename T, bool ACC>
__global__ __launch_bounds__(kThreads) void grad_sum_slices_vec_kernel(T* __restrict__ out, const T* __restrict__ parts, int slices,
                                                                       int64_t nvec) {
  using V = Vec16<T>;
  constexpr int U = 8;  // slice loads in flight per lane: the buffers are small, so latency, not bandwidth, is the limit
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  const V* pv = reinterpret_cast<const V*>(parts);
  V* ov = reinterpret_cast<V*>(out);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < nvec; i += stride) {
    float acc[V::N];
    V o;
    if (ACC) o = ov[i];
#pragma unroll
    for (int j = 0; j < V::N; ++j) acc[j] = 0.f;
    int s = 0;
    for (; s + U <= slices; s += U) {
      V p[U];
#pragma unroll
      for (int u = 0; u < U; ++u) p[u] = pv[static_cast<int64_t>(s + u) * nvec + i];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int j = 0; j < V::N; ++j) acc[j] += p[u].get(j);
    }
    for (; s < slices; ++s) {
      const V p = pv[static_cast<int64_t>(s) * nvec + i];
#pragma unroll
      for (int j = 0; j < V::N; ++j) acc[j] += p.get(j);
    }
    V r;
#pragma unroll
    for (int j = 0; j < V::N; ++j) r.set(j, ACC ? acc[j] + o.get(j) : acc[j]);
    ov[i] = r;
  }
}

template <typename T, bool ACC>
__global__ __launch_bounds__(kThreads) void grad_sum_slices_kernel(T* __restrict__ out, const T* __restrict__ parts, int slices, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
    float acc = ACC ? to_f32<T>(out[i]) : 0.f;
    for (int s = 0; s < slices; ++s) acc += to_f32<T>(parts[static_cast<int64_t>(s) * n + i]);
    out[i] = from_f32<T>(acc);
  }
}

template <typename T>
void launch_grad_sum_slices(void* out, const void* parts, int slices, int64_t n, bool acc, hipStream_t st) {
  constexpr int N = Vec16<T>::N;
  T* o = static_cast<T*>(out);
  const T* p = static_cast<const T*>(parts);
  if (n % N == 0 && mlts_aligned16(out) && mlts_aligned16(parts)) {
    const int64_t nvec = n / N;
    const int blocks = grid_for(nvec, 8192);
    if (acc)
      hipLaunchKernelGGL((grad_sum_slices_vec_kernel<T, true>), dim3(blocks), dim3(kThreads), 0, st, o, p, slices, nvec);
    else
      hipLaunchKernelGGL((grad_sum_slices_vec_kernel<T, false>), dim3(blocks), dim3(kThreads), 0, st, o, p, slices, nvec);
  } else {
    const int blocks = grid_for(n, 4096);
    if (acc)
      hipLaunchKernelGGL((grad_sum_slices_kernel<T, true>), dim3(blocks), dim3(kThreads), 0, st, o, p, slices, n);
    else
      hipLaunchKernelGGL((grad_sum_slices_kernel<T, false>), dim3(blocks), dim3(kThreads), 0, st, o, p, slices, n);
  }
}
}  // namespace

extern "C" int mlts_grad_sum_slices(void* out, const void* parts, int32_t dtype, int32_t slices, int64_t n, int accumulate,
                                   mlts_stream_t stream) {
  MLTS_REQUIRE(dtype == MLTS_F32 || dtype == MLTS_BF16, "mlts_grad_sum_slices: unknown dtype %d", dtype);
  MLTS_REQUIRE(n >= 0 && slices >= 1, "mlts_grad_sum_slices: n must be >= 0 and slices >= 1");
  if (n == 0) return MLTS_OK;
  MLTS_REQUIRE(out && parts, "mlts_grad_sum_slices: out and parts must be non-null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  MltsKernelTimer timer("grad_sum_slices", st);
  if (dtype == MLTS_BF16)
    launch_grad_sum_slices<bf16_t>(out, parts, slices, n, accumulate != 0, st);
  else
    launch_grad_sum_slices<float>(out, parts, slices, n, accumulate != 0, st);
  return mlts_check_launch("mlts_grad_sum_slices");
}

extern "C" int mlts_grad_to_f32(float* dst, const void* src, int32_t src_dtype, int64_t n, int accumulate,
                                double* sq_out, void* workspace, mlts_stream_t stream) {
  MLTS_REQUIRE(n >= 0, "mlts_grad_to_f32: n must be >= 0");
  MLTS_REQUIRE(src_dtype == MLTS_F32 || src_dtype == MLTS_BF16, "mlts_grad_to_f32: unknown dtype %d", src_dtype);
  MLTS_REQUIRE(n == 0 || (dst && src), "mlts_grad_to_f32: dst and src must be non-null");
  const bool sq = sq_out != nullptr;
  const bool acc = accumulate != 0;
  MLTS_REQUIRE(!sq || workspace, "mlts_grad_to_f32: workspace is required with sq_out");
  hipStream_t st = static_cast<hipStream_t>(stream);
  double* partial = static_cast<double*>(workspace);
  int blocks;
  MltsKernelTimer timer("grad_to_f32", st);
  if (src_dtype == MLTS_BF16 && mlts_aligned16(dst) && mlts_aligned16(src) && (n & 7) == 0 && n > 0) {
    blocks = grid_for(n >> 3, kSqBlocks);
    launch_grad_bf16_vec(acc, sq, blocks, st, dst, static_cast<const bf16_t*>(src), n >> 3, partial);
  } else if (src_dtype == MLTS_BF16) {
    blocks = grid_for(n, kSqBlocks);
    launch_grad_to_f32<bf16_t>(acc, sq, blocks, st, dst, static_cast<const bf16_t*>(src), n, partial);
  } else {
    blocks = grid_for(n, kSqBlocks);
    launch_grad_to_f32<float>(acc, sq, blocks, st, dst, static_cast<const float*>(src), n, partial);
  }
  if (sq) hipLaunchKernelGGL(sq_norm_stage2, dim3(1), dim3(kThreads), 0, st, partial, blocks, sq_out);
  return mlts_check_launch("mlts_grad_to_f32");
}
