// Causal cross-entropy: loss and d(logits) from ONE read of the logits.  A block owns one row,
// stages it in LDS (a 32000-entry bf16 row is 62.5 KiB of the CU's 160 KiB), reduces max and
// sum-exp with 64-lane shuffles, then streams the gradient out.  Rows whose label is the ignore
// index are never read: their gradient is zero.
#include "common.hpp"

namespace {

constexpr int kCeThreads = 512;
constexpr int kCeWaves = kCeThreads / MLTS_WAVE;
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float block_max(float x, float* red) {
  x = wave_max(x);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < kCeWaves; ++w) r = fmaxf(r, red[w]);
  __syncthreads();
  return r;
}
__device__ __forceinline__ float block_sum(float x, float* red) {
  x = wave_sum(x);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
  __syncthreads();
  float r = 0.f;
#pragma unroll
  for (int w = 0; w < kCeWaves; ++w) r += red[w];
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(1024) void ce_count_kernel(const int64_t* __restrict__ labels, int64_t rows,
                                                        int64_t ignore_index, int32_t* __restrict__ count_out) {
  __shared__ int part[16];
  int c = 0;
  for (int64_t i = threadIdx.x; i < rows; i += 1024) c += labels[i] != ignore_index ? 1 : 0;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, MLTS_WAVE);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int w = 0; w < 16; ++w) s += part[w];
    *count_out = s;
  }
}

// STAGED: the row lives in dynamic LDS between the passes; otherwise it is re-read from global
// memory (L2) -- used only when a row does not fit.
template <typename T, bool STAGED, bool VEC>
__global__ __launch_bounds__(kCeThreads) void ce_row_kernel(const T* logits,  // may be dlogits (gradient in place)
                                                            const int64_t* __restrict__ labels, T* dlogits,
                                                            float* __restrict__ row_loss,
                                                            const int32_t* __restrict__ count, int vocab,
                                                            int64_t ignore_index) {
  constexpr int N = Vec16<T>::N;
  extern __shared__ __attribute__((aligned(16))) unsigned char ce_smem[];
  __shared__ float red[kCeWaves];
  T* srow = reinterpret_cast<T*>(ce_smem);
  const int64_t row = blockIdx.x;
  const int64_t label = labels[row];
  const T* zr = logits + row * vocab;
  T* dr = dlogits + row * vocab;
  const int nvec = VEC ? vocab / N : 0;

  if (label == ignore_index) {
    if (threadIdx.x == 0) row_loss[row] = 0.f;
    if (VEC) {
      Vec16<T> z;
#pragma unroll
      for (int j = 0; j < N; ++j) z.set(j, 0.f);
      for (int c = threadIdx.x; c < nvec; c += kCeThreads) reinterpret_cast<Vec16<T>*>(dr)[c] = z;
    } else {
      for (int c = threadIdx.x; c < vocab; c += kCeThreads) dr[c] = from_f32<T>(0.f);
    }
    return;
  }
  const bool label_ok = label >= 0 && label < vocab;

  // pass 1: load (and stage), running max
  float mx = -INFINITY;
  if (VEC) {
    for (int c = threadIdx.x; c < nvec; c += kCeThreads) {
      Vec16<T> t;
      t.v = __builtin_nontemporal_load(reinterpret_cast<const decltype(t.v)*>(zr) + c);
      if (STAGED) reinterpret_cast<Vec16<T>*>(srow)[c] = t;
#pragma unroll
      for (int j = 0; j < N; ++j) mx = fmaxf(mx, t.get(j));
    }
  } else {
    for (int c = threadIdx.x; c < vocab; c += kCeThreads) {
      T t = zr[c];
      if (STAGED) srow[c] = t;
      mx = fmaxf(mx, to_f32<T>(t));
    }
  }
  mx = block_max(mx, red);  // the barrier inside also publishes the staged row
  const T* src = STAGED ? srow : zr;

  // pass 2: sum exp
  const float mxs = mx * kLog2e;
  float se = 0.f;
  if (VEC) {
    for (int c = threadIdx.x; c < nvec; c += kCeThreads) {
      Vec16<T> t = reinterpret_cast<const Vec16<T>*>(src)[c];
#pragma unroll
      for (int j = 0; j < N; ++j) se += exp2f(t.get(j) * kLog2e - mxs);
    }
  } else {
    for (int c = threadIdx.x; c < vocab; c += kCeThreads) se += exp2f(to_f32<T>(src[c]) * kLog2e - mxs);
  }
  // read before the barrier inside block_sum: behind it other threads may already be storing gradients over the row
  float label_logit = 0.f;
  if (threadIdx.x == 0 && label_ok) label_logit = to_f32<T>(src[label]);
  se = block_sum(se, red);
  const float lse = mx + logf(se);
  if (threadIdx.x == 0) {
    row_loss[row] = label_ok ? lse - label_logit : NAN;
  }

  // pass 3: gradient
  const int cnt = *count;
  const float inv = 1.0f / static_cast<float>(cnt > 0 ? cnt : 1);
  const float lses = lse * kLog2e;
  if (VEC) {
    const int lvec = label_ok ? static_cast<int>(label / N) : -1;
    const int lsub = label_ok ? static_cast<int>(label % N) : 0;
    for (int c = threadIdx.x; c < nvec; c += kCeThreads) {
      Vec16<T> t = reinterpret_cast<const Vec16<T>*>(src)[c];
      Vec16<T> o;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        float p = exp2f(t.get(j) * kLog2e - lses);
        if (c == lvec && j == lsub) p -= 1.0f;
        o.set(j, p * inv);
      }
      __builtin_nontemporal_store(o.v, reinterpret_cast<decltype(o.v)*>(dr) + c);
    }
  } else {
    for (int c = threadIdx.x; c < vocab; c += kCeThreads) {
      float p = exp2f(to_f32<T>(src[c]) * kLog2e - lses);
      if (c == label) p -= 1.0f;
      dr[c] = from_f32<T>(p * inv);
    }
  }
}

// Row kept in registers: NV 16-byte vectors per lane (a 32000-entry bf16 row is 8 per lane of a 512-lane block), all
// loads of a row issued before the first use.  No LDS beyond the reduction scratch, so four or more rows are in
// flight per CU instead of the two that fit when rows are staged in LDS (six wavefronts per SIMD = three blocks per CU
// is the register budget that still compiles without spills for eight vectors per lane).
template <typename T, int NV>
__global__ __launch_bounds__(kCeThreads, 6) void ce_row_reg_kernel(const T* logits,  // may be dlogits (gradient in place)
                                                                const int64_t* __restrict__ labels, T* dlogits,
                                                                float* __restrict__ row_loss,
                                                                const int32_t* __restrict__ count, int vocab,
                                                                int64_t ignore_index) {
  constexpr int N = Vec16<T>::N;
  __shared__ float red[kCeWaves];
  const int64_t row = blockIdx.x;
  const int64_t label = labels[row];
  const T* zr = logits + row * vocab;
  T* dr = dlogits + row * vocab;
  const int nvec = vocab / N;
  if (label == ignore_index) {
    if (threadIdx.x == 0) row_loss[row] = 0.f;
    Vec16<T> z;
#pragma unroll
    for (int j = 0; j < N; ++j) z.set(j, 0.f);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * kCeThreads;
      if (c < nvec) __builtin_nontemporal_store(z.v, reinterpret_cast<decltype(z.v)*>(dr) + c);
    }
    return;
  }
  const bool label_ok = label >= 0 && label < vocab;
  Vec16<T> t[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kCeThreads;
    if (c < nvec) t[i].v = __builtin_nontemporal_load(reinterpret_cast<const decltype(t[i].v)*>(zr) + c);
  }
  float label_logit = 0.f;
  if (threadIdx.x == 0 && label_ok) label_logit = to_f32<T>(zr[label]);
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (threadIdx.x + i * kCeThreads < nvec) {
#pragma unroll
      for (int j = 0; j < N; ++j) mx = fmaxf(mx, t[i].get(j));
    }
  }
  mx = block_max(mx, red);
  const float mxs = mx * kLog2e;
  float se = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (threadIdx.x + i * kCeThreads < nvec) {
#pragma unroll
      for (int j = 0; j < N; ++j) se += exp2f(t[i].get(j) * kLog2e - mxs);
    }
  }
  se = block_sum(se, red);
  const float lse = mx + logf(se);
  if (threadIdx.x == 0) row_loss[row] = label_ok ? lse - label_logit : NAN;
  const int cnt = *count;
  const float inv = 1.0f / static_cast<float>(cnt > 0 ? cnt : 1);
  const float lses = lse * kLog2e;
  const int lvec = label_ok ? static_cast<int>(label / N) : -1;
  const int lsub = label_ok ? static_cast<int>(label % N) : 0;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kCeThreads;
    if (c < nvec) {
      Vec16<T> o;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        float p = exp2f(t[i].get(j) * kLog2e - lses);
        if (c == lvec && j == lsub) p -= 1.0f;
        o.set(j, p * inv);
      }
      __builtin_nontemporal_store(o.v, reinterpret_cast<decltype(o.v)*>(dr) + c);
    }
  }
}

__global__ __launch_bounds__(kCeThreads) void ce_loss_reduce_kernel(const float* __restrict__ row_loss, int64_t rows,
                                                                    const int32_t* __restrict__ count,
                                                                    float* __restrict__ loss_out) {
  __shared__ double part[kCeWaves];
  double acc = 0.0;
  for (int64_t i = threadIdx.x; i < rows; i += kCeThreads) acc += static_cast<double>(row_loss[i]);
  acc = wave_sum_f64(acc);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double s = 0.0;
    for (int w = 0; w < kCeWaves; ++w) s += part[w];
    const int c = *count;
    *loss_out = static_cast<float>(s / static_cast<double>(c > 0 ? c : 1));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void scale_by_scalar_kernel(T* x, const float* scale, int64_t n) {
  const float s = *scale;
  if (s == 1.0f) return;  // the usual case: loss is the root of the graph
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride)
    x[i] = from_f32<T>(to_f32<T>(x[i]) * s);
}

// 16-byte form for an aligned buffer: n_vec whole vectors, the tail (< one vector) by the first lanes of block 0.
template <typename T>
__global__ __launch_bounds__(256) void scale_by_scalar_vec_kernel(T* x, const float* scale, int64_t n_vec, int64_t n) {
  using V = Vec16<T>;
  const float s = *scale;
  if (s == 1.0f) return;
  V* xv = reinterpret_cast<V*>(x);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n_vec; i += stride) {
    V v = xv[i];
#pragma unroll
    for (int j = 0; j < V::N; ++j) v.set(j, v.get(j) * s);
    xv[i] = v;
  }
  const int64_t tail = n_vec * V::N + static_cast<int64_t>(threadIdx.x);
  if (blockIdx.x == 0 && tail < n) x[tail] = from_f32<T>(to_f32<T>(x[tail]) * s);
}

constexpr int64_t kMaxStagedBytes = 128 * 1024;

template <typename T>
int ce_launch(const void* logits, const int64_t* labels, void* dlogits, float* row_loss, const int32_t* count,
              int64_t rows, int vocab, int64_t ignore_index, hipStream_t st) {
  constexpr int N = Vec16<T>::N;
  const bool vec = (vocab % N == 0) && mlts_aligned16(logits) && mlts_aligned16(dlogits);
  const int64_t row_bytes = static_cast<int64_t>(vocab) * static_cast<int64_t>(sizeof(T));
  const bool staged = row_bytes <= kMaxStagedBytes;
  const size_t smem = staged ? static_cast<size_t>((row_bytes + 15) & ~15LL) : 0;
  const T* lg = static_cast<const T*>(logits);
  T* dl = static_cast<T*>(dlogits);
  if (vec && vocab / N <= 8 * kCeThreads) {  // the row fits the registers of one block
    const int per_lane = (vocab / N + kCeThreads - 1) / kCeThreads;
#define MLTS_CE_REG(NV)                                                                                              \
  hipLaunchKernelGGL((ce_row_reg_kernel<T, NV>), dim3((unsigned)rows), dim3(kCeThreads), 0, st, lg, labels, dl, row_loss, \
                     count, vocab, ignore_index)
    if (per_lane <= 1) MLTS_CE_REG(1);
    else if (per_lane <= 2) MLTS_CE_REG(2);
    else if (per_lane <= 4) MLTS_CE_REG(4);
    else MLTS_CE_REG(8);
#undef MLTS_CE_REG
    return MLTS_OK;
  }
#define MLTS_CE_LAUNCH(ST, VC)                                                                                      \
  do {                                                                                                              \
    auto kern = ce_row_kernel<T, ST, VC>;                                                                           \
    if (smem > 48 * 1024) {                                                                                         \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                       \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));       \
      if (e != hipSuccess) {                                                                                        \
        mlts_set_error("mlts_ce_fwd_bwd: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));         \
        return MLTS_ERR_LAUNCH;                                                                                     \
      }                                                                                                             \
    }                                                                                                               \
    hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(kCeThreads), smem, st, lg, labels, dl, row_loss, count,     \
                       vocab, ignore_index);                                                                        \
  } while (0)
  if (staged && vec) MLTS_CE_LAUNCH(true, true);
  else if (staged) MLTS_CE_LAUNCH(true, false);
  else if (vec) MLTS_CE_LAUNCH(false, true);
  else MLTS_CE_LAUNCH(false, false);
#undef MLTS_CE_LAUNCH
  return MLTS_OK;
}

}  // namespace

extern "C" int64_t mlts_ce_workspace_bytes(int64_t rows) { return (rows < 0 ? 0 : rows) * 4 + 64; }

extern "C" int mlts_ce_fwd_bwd(const void* logits, const int64_t* labels, void* dlogits, float* loss_out,
                               int32_t* count_out, void* workspace, int64_t workspace_bytes, int64_t rows,
                               int32_t vocab, int64_t ignore_index, int32_t dtype, mlts_stream_t stream) {
  MLTS_REQUIRE(dtype == MLTS_BF16 || dtype == MLTS_F32, "mlts_ce_fwd_bwd: unknown dtype %d", dtype);
  MLTS_REQUIRE(rows >= 0 && vocab > 0, "mlts_ce_fwd_bwd: bad shape rows=%lld vocab=%d", (long long)rows, vocab);
  MLTS_REQUIRE(rows <= 0x7fffffffLL, "mlts_ce_fwd_bwd: too many rows");
  MLTS_REQUIRE(loss_out && count_out && workspace, "mlts_ce_fwd_bwd: null output pointer");
  MLTS_REQUIRE(workspace_bytes >= mlts_ce_workspace_bytes(rows), "mlts_ce_fwd_bwd: workspace too small");
  MLTS_REQUIRE(rows == 0 || (logits && labels && dlogits), "mlts_ce_fwd_bwd: null input pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* row_loss = static_cast<float*>(workspace);
  hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(1024), 0, st, labels, rows, ignore_index, count_out);
  if (rows > 0) {
    MltsKernelTimer timer("ce", st);
    int rc = dtype == MLTS_BF16
                 ? ce_launch<bf16_t>(logits, labels, dlogits, row_loss, count_out, rows, vocab, ignore_index, st)
                 : ce_launch<float>(logits, labels, dlogits, row_loss, count_out, rows, vocab, ignore_index, st);
    if (rc != MLTS_OK) return rc;
  }
  hipLaunchKernelGGL(ce_loss_reduce_kernel, dim3(1), dim3(kCeThreads), 0, st, row_loss, rows, count_out, loss_out);
  return mlts_check_launch("mlts_ce_fwd_bwd");
}

extern "C" int mlts_scale_by_device_scalar(void* x, const float* scale, int64_t n, int32_t dtype,
                                           mlts_stream_t stream) {
  MLTS_REQUIRE(dtype == MLTS_BF16 || dtype == MLTS_F32, "mlts_scale_by_device_scalar: unknown dtype %d", dtype);
  MLTS_REQUIRE(n >= 0, "mlts_scale_by_device_scalar: n must be >= 0");
  if (n == 0) return MLTS_OK;
  MLTS_REQUIRE(x && scale, "mlts_scale_by_device_scalar: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (mlts_aligned16(x)) {
    const int64_t per = dtype == MLTS_BF16 ? 8 : 4;
    const int64_t n_vec = n / per;
    int64_t blocks = (n_vec + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > 8192 ? 8192 : blocks);
    if (dtype == MLTS_BF16)
      hipLaunchKernelGGL(scale_by_scalar_vec_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<bf16_t*>(x), scale, n_vec, n);
    else
      hipLaunchKernelGGL(scale_by_scalar_vec_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<float*>(x), scale, n_vec, n);
    return mlts_check_launch("mlts_scale_by_device_scalar");
  }
  int64_t blocks = (n + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  if (dtype == MLTS_BF16)
    hipLaunchKernelGGL(scale_by_scalar_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<bf16_t*>(x), scale, n);
  else
    hipLaunchKernelGGL(scale_by_scalar_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<float*>(x), scale, n);
  return mlts_check_launch("mlts_scale_by_device_scalar");
}
