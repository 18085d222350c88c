// HBM-bound layer kernels: RMSNorm, interleaved RoPE, SwiGLU.  Each is one coalesced pass with
// 16-byte accesses; row statistics use 64-lane shuffle reductions.  Where the reference's eager ops
// materialise an intermediate in bf16 the same rounding is reproduced here, so the forward results
// are the reference's values and not merely close to them.
#include "common.hpp"

#include <initializer_list>

// The kernels below reproduce the reference's per-op bf16 roundings.  With contraction enabled the
// compiler narrows "round(a * b)" to a bf16 multiply and then fuses it into the following add as an
// fp32 FMA, which silently drops that rounding; contraction stays off for this whole file.
#pragma clang fp contract(off)

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / MLTS_WAVE;

// ============================== RMSNorm ==================================================
// One wavefront per row; a row is walked in chunks of 64 lanes x 16 bytes.
// ADD: the normalised row is h = x + res, rounded to T as the eager residual add rounds it; h is stored to `sum_out`
// (which the second pass reads back: a lane reads only what it wrote itself) and is the row the statistics are of.
template <typename T, bool ADD>
__global__ __launch_bounds__(kThreads) void rmsnorm_fwd_kernel(const T* __restrict__ x, const T* __restrict__ res,
                                                               T* __restrict__ sum_out, const T* __restrict__ w,
                                                               T* __restrict__ y, float* __restrict__ rstd_out,
                                                               int64_t rows, int hidden, float eps) {
  constexpr int N = Vec16<T>::N;
  const int lane = threadIdx.x & (MLTS_WAVE - 1);
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + (threadIdx.x / MLTS_WAVE);
  if (row >= rows) return;
  const T* xr = ADD ? sum_out + row * hidden : x + row * hidden;
  T* yr = y + row * hidden;
  const int nvec = hidden / N;
  float ss = 0.f;
  for (int c = lane; c < nvec; c += MLTS_WAVE) {
    Vec16<T> t;
    if (ADD) {
      const Vec16<T> a = reinterpret_cast<const Vec16<T>*>(x + row * hidden)[c];
      const Vec16<T> b = reinterpret_cast<const Vec16<T>*>(res + row * hidden)[c];
#pragma unroll
      for (int j = 0; j < N; ++j) t.set(j, a.get(j) + b.get(j));
      reinterpret_cast<Vec16<T>*>(sum_out + row * hidden)[c] = t;
    } else {
      t = reinterpret_cast<const Vec16<T>*>(xr)[c];
    }
#pragma unroll
    for (int j = 0; j < N; ++j) {
      float f = t.get(j);
      ss += f * f;
    }
  }
  ss = wave_sum(ss);
  const float r = rsqrtf(ss / static_cast<float>(hidden) + eps);
  if (lane == 0 && rstd_out) rstd_out[row] = r;
  for (int c = lane; c < nvec; c += MLTS_WAVE) {
    Vec16<T> t = reinterpret_cast<const Vec16<T>*>(xr)[c];
    Vec16<T> wv = reinterpret_cast<const Vec16<T>*>(w)[c];
    Vec16<T> o;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      float n = round_to<T>(t.get(j) * r);  // (x * rsqrt(var + eps)).to(x.dtype)
      o.set(j, wv.get(j) * n);              // weight * normed, rounded by set()
    }
    reinterpret_cast<Vec16<T>*>(yr)[c] = o;
  }
}

// dx = r * (g - xhat * mean(g * xhat)), g = dy * w, xhat = x * r; per-block partial of
// dw = sum_rows dy * xhat is written to dw_partial[block][hidden].
// Each wave walks rows block*rows_per_block + wave, + kWaves, ...; lanes own fixed columns, so dw
// partials live in registers (hidden <= 64 * N * kMaxChunks).
constexpr int kMaxChunks = 8;

// CH = 16-byte chunks per lane and row (1, 2, 4 or 8); R rows of a wavefront are in flight at once and their vectors
// stay in registers between the two passes (one row at a time leaves the memory latency of every row exposed); NW
// wavefronts per block.  A wavefront loads, then computes, then stores, so memory and arithmetic overlap only across
// wavefronts: narrow rows (CH <= 2) run 16 wavefronts per block, four per SIMD, with correspondingly fewer rows each.
// dres (may be null): gradient that reaches the same row by the residual path; dx = round(dx_norm) + dres, the two
// roundings of autograd's own sum of the two paths.
template <typename T, int CH, bool RES, int R, int NW>
__global__ __launch_bounds__(NW * MLTS_WAVE) void rmsnorm_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                               const T* __restrict__ w, const float* __restrict__ rstd,
                                                               const T* __restrict__ dres,
                                                               T* __restrict__ dx, float* __restrict__ dw_partial,
                                                               int64_t rows, int hidden, int rows_per_block) {
  constexpr int N = Vec16<T>::N;
  constexpr int kWaves = NW;       // shadows the file-wide block shape
  constexpr int kThreads = NW * MLTS_WAVE;
  extern __shared__ float smem[];  // [kWaves][hidden]
  const int lane = threadIdx.x & (MLTS_WAVE - 1);
  const int wave = threadIdx.x / MLTS_WAVE;
  const int nvec = hidden / N;
  constexpr int chunks = CH;
  float dwacc[CH][N];
  Vec16<T> wv[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) {
#pragma unroll
    for (int j = 0; j < N; ++j) dwacc[c][j] = 0.f;
    const int col = lane + c * MLTS_WAVE;
    if (col < nvec) wv[c] = reinterpret_cast<const Vec16<T>*>(w)[col];
  }

  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * rows_per_block;
  int64_t row_end = row0 + rows_per_block;
  if (row_end > rows) row_end = rows;
  const float inv_h = 1.0f / static_cast<float>(hidden);
  for (int64_t row = row0 + wave; row < row_end; row += kWaves * R) {
    Vec16<T> xv[R][CH], dv[R][CH], rv[RES ? R : 1][CH];
    float rr[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      int64_t ri = row + static_cast<int64_t>(i) * kWaves;
      if (ri >= row_end) ri = row;  // loaded again, not used
      rr[i] = rstd[ri];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int col = lane + c * MLTS_WAVE;
        if (col < nvec) {
          xv[i][c] = reinterpret_cast<const Vec16<T>*>(x + ri * hidden)[col];
          dv[i][c] = reinterpret_cast<const Vec16<T>*>(dy + ri * hidden)[col];
          if (RES) rv[RES ? i : 0][c] = reinterpret_cast<const Vec16<T>*>(dres + ri * hidden)[col];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int64_t ri = row + static_cast<int64_t>(i) * kWaves;
      if (ri < row_end) {
        const float r = rr[i];
        float dot = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          const int col = lane + c * MLTS_WAVE;
          if (col < nvec) {
#pragma unroll
            for (int j = 0; j < N; ++j) {
              float xh = xv[i][c].get(j) * r;
              float d = dv[i][c].get(j);
              dwacc[c][j] += d * xh;
              dot += d * wv[c].get(j) * xh;
            }
          }
        }
        dot = wave_sum(dot) * inv_h;
        T* dxr = dx + ri * hidden;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          const int col = lane + c * MLTS_WAVE;
          if (col < nvec) {
            Vec16<T> o;
#pragma unroll
            for (int j = 0; j < N; ++j) {
              float xh = xv[i][c].get(j) * r;
              const float g = r * (dv[i][c].get(j) * wv[c].get(j) - xh * dot);
              o.set(j, RES ? round_to<T>(g) + rv[RES ? i : 0][c].get(j) : g);
            }
            reinterpret_cast<Vec16<T>*>(dxr)[col] = o;
          }
        }
      }
    }
  }
  // reduce the four waves' dw partials through LDS
#pragma unroll
  for (int c = 0; c < chunks; ++c) {
    const int col = lane + c * MLTS_WAVE;
    if (col < nvec) {
#pragma unroll
      for (int j = 0; j < N; ++j) smem[wave * hidden + col * N + j] = dwacc[c][j];
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    float s = 0.f;
#pragma unroll
    for (int wi = 0; wi < kWaves; ++wi) s += smem[wi * hidden + i];
    dw_partial[static_cast<int64_t>(blockIdx.x) * hidden + i] = s;
  }
}

// dw[col] = sum over the per-block partial rows, in a fixed order: a block owns 32 columns, its 8 groups of 32
// lanes each add every 8th partial row (four loads in flight), then the 8 group sums are added through LDS.
template <typename T>
__global__ __launch_bounds__(kThreads) void rmsnorm_dw_reduce_kernel(const float* __restrict__ dw_partial, int nblocks,
                                                                     int hidden, T* __restrict__ dw) {
  __shared__ float part[8][32];
  const int c = threadIdx.x & 31, r = threadIdx.x >> 5;
  const int col = blockIdx.x * 32 + c;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (col < hidden) {
    int b = r;
    for (; b + 24 < nblocks; b += 32) {
      s0 += dw_partial[static_cast<int64_t>(b) * hidden + col];
      s1 += dw_partial[static_cast<int64_t>(b + 8) * hidden + col];
      s2 += dw_partial[static_cast<int64_t>(b + 16) * hidden + col];
      s3 += dw_partial[static_cast<int64_t>(b + 24) * hidden + col];
    }
    for (; b < nblocks; b += 8) s0 += dw_partial[static_cast<int64_t>(b) * hidden + col];
  }
  part[r][c] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (r == 0 && col < hidden) {
    float s = part[0][c];
#pragma unroll
    for (int i = 1; i < 8; ++i) s += part[i][c];
    dw[col] = from_f32<T>(s);
  }
}

int rmsnorm_bwd_blocks(int64_t rows) {
  int64_t b = (rows + 31) / 32;  // >= 32 rows per block keeps the partial buffer small
  if (b > 256) b = 256;          // one block per CU: more blocks only lengthen the reduction of their dw partials
  if (b < 1) b = 1;
  return static_cast<int>(b);
}

// ============================== RoPE =====================================================
// One lane rotates the pairs inside one 16-byte vector of a [b, h, s, :] row.
// IDX is the type the flat element index is taken apart in: 32-bit whenever the tensor has fewer than 2^31 vectors
// (three 64-bit divisions per lane cost several hundred instructions, more than the rotation itself).
// y may be x (rotation in place: a lane reads only the vector it writes), so the two carry no __restrict__.
template <typename T, bool INVERSE, typename IDX>
__device__ __forceinline__ void rope_rows(const int64_t idx64, const T* x, int64_t xsb, int64_t xsh, int64_t xss,
                                          T* y, int64_t ysb, int64_t ysh, int64_t yss,
                                          const T* __restrict__ cos_tab, const T* __restrict__ sin_tab, int max_pos,
                                          const int32_t* __restrict__ positions, int position_offset, int B, int H, int S,
                                          int D) {
  constexpr int N = Vec16<T>::N;
  const int vec_per_row = D / N;
  const int64_t total = static_cast<int64_t>(B) * S * H * vec_per_row;
  if (idx64 >= total) return;
  // order (b, s, h, vec): neighbouring lanes touch neighbouring memory for [B, S, H, D] storage
  const IDX idx = static_cast<IDX>(idx64);
  const int vc = static_cast<int>(idx % static_cast<IDX>(vec_per_row));
  IDX rest = idx / static_cast<IDX>(vec_per_row);
  const int h = static_cast<int>(rest % static_cast<IDX>(H));
  rest /= static_cast<IDX>(H);
  const int s = static_cast<int>(rest % static_cast<IDX>(S));
  const int b = static_cast<int>(rest / static_cast<IDX>(S));
  int pos = positions ? positions[static_cast<int64_t>(b) * S + s] : position_offset + s;
  pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);  // host validated; keeps reads in bounds
  const T* xp = x + b * xsb + h * xsh + s * xss + vc * N;
  T* yp = y + b * ysb + h * ysh + s * yss + vc * N;
  Vec16<T> xv = *reinterpret_cast<const Vec16<T>*>(xp);
  // the N / 2 table entries of this vector are 8 bytes (4 bf16 or 2 fp32), 8-byte aligned: one load each
  struct alignas(8) Half8 { T v[N / 2]; };
  const Half8 cv = *reinterpret_cast<const Half8*>(cos_tab + static_cast<int64_t>(pos) * (D / 2) + vc * (N / 2));
  const Half8 sv = *reinterpret_cast<const Half8*>(sin_tab + static_cast<int64_t>(pos) * (D / 2) + vc * (N / 2));
  Vec16<T> o;
#pragma unroll
  for (int j = 0; j < N / 2; ++j) {
    const float c = to_f32<T>(cv.v[j]);
    float sn = to_f32<T>(sv.v[j]);
    const float xe = xv.get(2 * j), xo = xv.get(2 * j + 1);
    float oe, oo;
    if (!INVERSE) {
      oe = round_to<T>(xe * c) - round_to<T>(xo * sn);  // x_even * cos - x_odd * sin
      oo = round_to<T>(xe * sn) + round_to<T>(xo * c);  // x_even * sin + x_odd * cos
    } else {
      oe = round_to<T>(xe * c) + round_to<T>(xo * sn);  // d_even * cos + d_odd * sin
      oo = round_to<T>(xo * c) - round_to<T>(xe * sn);  // d_odd * cos - d_even * sin
    }
    o.set(2 * j, oe);
    o.set(2 * j + 1, oo);
  }
  *reinterpret_cast<Vec16<T>*>(yp) = o;
}

template <typename T, bool INVERSE, typename IDX>
__global__ __launch_bounds__(kThreads) void rope_kernel(const T* x, int64_t xsb, int64_t xsh, int64_t xss,
                                                        T* y, int64_t ysb, int64_t ysh, int64_t yss,
                                                        const T* __restrict__ cos_tab, const T* __restrict__ sin_tab,
                                                        int max_pos, const int32_t* __restrict__ positions,
                                                        int position_offset, int B, int H, int S, int D) {
  rope_rows<T, INVERSE, IDX>(static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x, x, xsb, xsh, xss, y, ysb, ysh, yss,
                             cos_tab, sin_tab, max_pos, positions, position_offset, B, H, S, D);
}

// Two tensors of one layer (the query and the key projections) in one launch: blocks [0, first_blocks) rotate the
// first, the rest the second.  Same arithmetic as rope_kernel; a launch of this size costs more than it computes.
struct RopeOperand {
  const void* x;
  void* y;
  int64_t xs[3], ys[3];
  int H;
};
template <typename T, bool INVERSE>
__global__ __launch_bounds__(kThreads) void rope_pair_kernel(const RopeOperand a, const RopeOperand b, unsigned first_blocks,
                                                             const T* __restrict__ cos_tab, const T* __restrict__ sin_tab,
                                                             int max_pos, const int32_t* __restrict__ positions,
                                                             int position_offset, int B, int S, int D) {
  const bool second = blockIdx.x >= first_blocks;
  const RopeOperand& t = second ? b : a;
  const int64_t idx = static_cast<int64_t>(blockIdx.x - (second ? first_blocks : 0u)) * kThreads + threadIdx.x;
  rope_rows<T, INVERSE, uint32_t>(idx, static_cast<const T*>(t.x), t.xs[0], t.xs[1], t.xs[2], static_cast<T*>(t.y), t.ys[0],
                                  t.ys[1], t.ys[2], cos_tab, sin_tab, max_pos, positions, position_offset, B, t.H, S, D);
}

// ============================== SwiGLU ===================================================
__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.0f + expf(-x)); }  // the form ATen evaluates

template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_fwd_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                              T* __restrict__ h, int64_t nvec) {
  constexpr int N = Vec16<T>::N;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < nvec; i += stride) {
    Vec16<T> g = reinterpret_cast<const Vec16<T>*>(gate)[i];
    Vec16<T> u = reinterpret_cast<const Vec16<T>*>(up)[i];
    Vec16<T> o;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float gj = g.get(j);
      const float act = round_to<T>(siluf_(gj));  // F.silu materialised in T
      o.set(j, act * u.get(j));
    }
    reinterpret_cast<Vec16<T>*>(h)[i] = o;
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_bwd_kernel(const T* __restrict__ dh, const T* __restrict__ gate,
                                                              const T* __restrict__ up, T* __restrict__ dgate,
                                                              T* __restrict__ dup, int64_t nvec) {
  constexpr int N = Vec16<T>::N;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < nvec; i += stride) {
    Vec16<T> d = reinterpret_cast<const Vec16<T>*>(dh)[i];
    Vec16<T> g = reinterpret_cast<const Vec16<T>*>(gate)[i];
    Vec16<T> u = reinterpret_cast<const Vec16<T>*>(up)[i];
    Vec16<T> og, ou;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float gj = g.get(j), dj = d.get(j);
      const float sg = sigmoidf_(gj);
      ou.set(j, dj * (gj * sg));
      og.set(j, dj * u.get(j) * (sg * (1.0f + gj * (1.0f - sg))));
    }
    reinterpret_cast<Vec16<T>*>(dgate)[i] = og;
    reinterpret_cast<Vec16<T>*>(dup)[i] = ou;
  }
}

// The same two kernels over [rows, cols] matrices with row strides (in elements, multiples of the vector width): gate
// and up are the two column halves of one projection output, dgate and dup those of one gradient buffer.
template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_fwd_rows_kernel(const T* __restrict__ gate, const T* __restrict__ up, int64_t ld_in,
                                                                   T* __restrict__ h, int64_t ld_h, uint32_t vec_per_row, uint32_t nvec) {
  constexpr int N = Vec16<T>::N;
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < nvec; i += stride) {
    const uint32_t row = i / vec_per_row, c = i - row * vec_per_row;
    const int64_t in = static_cast<int64_t>(row) * ld_in + c * N;
    Vec16<T> g = *reinterpret_cast<const Vec16<T>*>(gate + in);
    Vec16<T> u = *reinterpret_cast<const Vec16<T>*>(up + in);
    Vec16<T> o;
#pragma unroll
    for (int j = 0; j < N; ++j) o.set(j, round_to<T>(siluf_(g.get(j))) * u.get(j));
    *reinterpret_cast<Vec16<T>*>(h + static_cast<int64_t>(row) * ld_h + c * N) = o;
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_bwd_rows_kernel(const T* __restrict__ dh, int64_t ld_dh, const T* __restrict__ gate,
                                                                   const T* __restrict__ up, int64_t ld_in, T* __restrict__ dgate,
                                                                   T* __restrict__ dup, int64_t ld_out, uint32_t vec_per_row,
                                                                   uint32_t nvec) {
  constexpr int N = Vec16<T>::N;
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < nvec; i += stride) {
    const uint32_t row = i / vec_per_row, c = i - row * vec_per_row;
    const int64_t in = static_cast<int64_t>(row) * ld_in + c * N, out = static_cast<int64_t>(row) * ld_out + c * N;
    Vec16<T> d = *reinterpret_cast<const Vec16<T>*>(dh + static_cast<int64_t>(row) * ld_dh + c * N);
    Vec16<T> g = *reinterpret_cast<const Vec16<T>*>(gate + in);
    Vec16<T> u = *reinterpret_cast<const Vec16<T>*>(up + in);
    Vec16<T> og, ou;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float gj = g.get(j), dj = d.get(j);
      const float sg = sigmoidf_(gj);
      ou.set(j, dj * (gj * sg));
      og.set(j, dj * u.get(j) * (sg * (1.0f + gj * (1.0f - sg))));
    }
    *reinterpret_cast<Vec16<T>*>(dgate + out) = og;
    *reinterpret_cast<Vec16<T>*>(dup + out) = ou;
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_fwd_tail(const T* gate, const T* up, T* h, int64_t start, int64_t n) {
  int64_t i = start + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const float gj = to_f32<T>(gate[i]);
  const float act = round_to<T>(siluf_(gj));
  h[i] = from_f32<T>(act * to_f32<T>(up[i]));
}
template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_bwd_tail(const T* dh, const T* gate, const T* up, T* dgate, T* dup,
                                                            int64_t start, int64_t n) {
  int64_t i = start + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const float gj = to_f32<T>(gate[i]), dj = to_f32<T>(dh[i]);
  const float sg = sigmoidf_(gj);
  dup[i] = from_f32<T>(dj * (gj * sg));
  dgate[i] = from_f32<T>(dj * to_f32<T>(up[i]) * (sg * (1.0f + gj * (1.0f - sg))));
}

int stream_grid(int64_t nvec) {
  int64_t b = (nvec + kThreads - 1) / kThreads;
  if (b > 16384) b = 16384;
  if (b < 1) b = 1;
  return static_cast<int>(b);
}

template <typename T>
int rmsnorm_fwd_t(const void* x, const void* res, void* sum_out, const void* w, void* y, float* rstd, int64_t rows,
                  int hidden, float eps, hipStream_t st) {
  const int64_t blocks = (rows + kWaves - 1) / kWaves;
  MltsKernelTimer timer("rmsnorm_fwd", st);
  if (res)
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<T, true>), dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const T*>(x),
                       static_cast<const T*>(res), static_cast<T*>(sum_out), static_cast<const T*>(w), static_cast<T*>(y),
                       rstd, rows, hidden, eps);
  else
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<T, false>), dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const T*>(x),
                       static_cast<const T*>(nullptr), static_cast<T*>(nullptr), static_cast<const T*>(w),
                       static_cast<T*>(y), rstd, rows, hidden, eps);
  return mlts_check_launch("mlts_rmsnorm_fwd");
}

template <typename T, int CH, int R, int NW>
void rmsnorm_bwd_launch(const void* dy, const void* x, const void* w, const float* rstd, const void* dres, void* dx,
                        float* partial, int64_t rows, int hidden, int blocks, int rows_per_block, hipStream_t st) {
  const size_t smem = static_cast<size_t>(NW) * hidden * sizeof(float);
  if (dres)
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, CH, true, R, NW>), dim3(blocks), dim3(NW * MLTS_WAVE), smem, st,
                       static_cast<const T*>(dy), static_cast<const T*>(x), static_cast<const T*>(w), rstd,
                       static_cast<const T*>(dres), static_cast<T*>(dx), partial, rows, hidden, rows_per_block);
  else
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, CH, false, R, NW>), dim3(blocks), dim3(NW * MLTS_WAVE), smem, st,
                       static_cast<const T*>(dy), static_cast<const T*>(x), static_cast<const T*>(w), rstd,
                       static_cast<const T*>(nullptr), static_cast<T*>(dx), partial, rows, hidden, rows_per_block);
}

template <typename T>
int rmsnorm_bwd_t(const void* dy, const void* x, const void* w, const float* rstd, const void* dres, void* dx, void* dw,
                  float* partial, int64_t rows, int hidden, hipStream_t st) {
  const int blocks = rmsnorm_bwd_blocks(rows);
  const int rows_per_block = static_cast<int>((rows + blocks - 1) / blocks);
  MltsKernelTimer timer("rmsnorm_bwd", st);
  const int chunks = (hidden / Vec16<T>::N + MLTS_WAVE - 1) / MLTS_WAVE;  // <= kMaxChunks, checked by the caller
#define MLTS_RMS_BWD(CH, R, NW) \
  rmsnorm_bwd_launch<T, CH, R, NW>(dy, x, w, rstd, dres, dx, partial, rows, hidden, blocks, rows_per_block, st)
  if (chunks <= 2) {
    // rows of one wavefront (of 16 per block) per pass: as many as it has, up to 8 vectors per operand and lane
    const int per_wave = (rows_per_block + 15) / 16;
    if (chunks <= 1) {
      if (per_wave >= 8) MLTS_RMS_BWD(1, 8, 16);
      else if (per_wave >= 4) MLTS_RMS_BWD(1, 4, 16);
      else if (per_wave >= 2) MLTS_RMS_BWD(1, 2, 16);
      else MLTS_RMS_BWD(1, 1, 16);
    } else {
      if (per_wave >= 4) MLTS_RMS_BWD(2, 4, 16);
      else if (per_wave >= 2) MLTS_RMS_BWD(2, 2, 16);
      else MLTS_RMS_BWD(2, 1, 16);
    }
  } else if (chunks <= 4) {
    MLTS_RMS_BWD(4, 2, 4);
  } else {
    MLTS_RMS_BWD(8, 1, 4);
  }
#undef MLTS_RMS_BWD
  hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel<T>, dim3((hidden + 31) / 32), dim3(kThreads), 0, st,
                     partial, blocks, hidden, static_cast<T*>(dw));
  return mlts_check_launch("mlts_rmsnorm_bwd");
}

template <typename T>
int rope_t(const void* x, const int64_t* xs, void* y, const int64_t* ys, const void* ct, const void* sn, int max_pos,
           const int32_t* positions, int off, int B, int H, int S, int D, int inverse, hipStream_t st) {
  MltsKernelTimer timer("rope", st);
  constexpr int N = Vec16<T>::N;
  const int64_t total = static_cast<int64_t>(B) * S * H * (D / N);
  const int64_t blocks = (total + kThreads - 1) / kThreads;
  if (blocks == 0) return MLTS_OK;
#define MLTS_ROPE(INV, IDX)                                                                                         \
  hipLaunchKernelGGL((rope_kernel<T, INV, IDX>), dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const T*>(x), \
                     xs[0], xs[1], xs[2], static_cast<T*>(y), ys[0], ys[1], ys[2], static_cast<const T*>(ct),         \
                     static_cast<const T*>(sn), max_pos, positions, off, B, H, S, D)
  const bool narrow = total < (1LL << 31);
  if (inverse) {
    if (narrow) MLTS_ROPE(true, uint32_t);
    else MLTS_ROPE(true, int64_t);
  } else {
    if (narrow) MLTS_ROPE(false, uint32_t);
    else MLTS_ROPE(false, int64_t);
  }
#undef MLTS_ROPE
  return mlts_check_launch("mlts_rope");
}

template <typename T>
int swiglu_fwd_t(const void* g, const void* u, void* h, int64_t n, bool vec, hipStream_t st) {
  MltsKernelTimer timer("swiglu_fwd", st);
  constexpr int N = Vec16<T>::N;
  int64_t done = 0;
  if (vec && n >= N) {
    const int64_t nvec = n / N;
    hipLaunchKernelGGL(swiglu_fwd_kernel<T>, dim3(stream_grid(nvec)), dim3(kThreads), 0, st, static_cast<const T*>(g),
                       static_cast<const T*>(u), static_cast<T*>(h), nvec);
    done = nvec * N;
  }
  if (done < n) {
    const int64_t rem = n - done;
    hipLaunchKernelGGL(swiglu_fwd_tail<T>, dim3((unsigned)((rem + kThreads - 1) / kThreads)), dim3(kThreads), 0, st,
                       static_cast<const T*>(g), static_cast<const T*>(u), static_cast<T*>(h), done, n);
  }
  return mlts_check_launch("mlts_swiglu_fwd");
}

template <typename T>
int swiglu_bwd_t(const void* dh, const void* g, const void* u, void* dg, void* du, int64_t n, bool vec,
                 hipStream_t st) {
  MltsKernelTimer timer("swiglu_bwd", st);
  constexpr int N = Vec16<T>::N;
  int64_t done = 0;
  if (vec && n >= N) {
    const int64_t nvec = n / N;
    hipLaunchKernelGGL(swiglu_bwd_kernel<T>, dim3(stream_grid(nvec)), dim3(kThreads), 0, st, static_cast<const T*>(dh),
                       static_cast<const T*>(g), static_cast<const T*>(u), static_cast<T*>(dg), static_cast<T*>(du),
                       nvec);
    done = nvec * N;
  }
  if (done < n) {
    const int64_t rem = n - done;
    hipLaunchKernelGGL(swiglu_bwd_tail<T>, dim3((unsigned)((rem + kThreads - 1) / kThreads)), dim3(kThreads), 0, st,
                       static_cast<const T*>(dh), static_cast<const T*>(g), static_cast<const T*>(u),
                       static_cast<T*>(dg), static_cast<T*>(du), done, n);
  }
  return mlts_check_launch("mlts_swiglu_bwd");
}

inline int elem_per_vec(int dtype) { return dtype == MLTS_BF16 ? 8 : 4; }
inline bool known_dtype(int dtype) { return dtype == MLTS_BF16 || dtype == MLTS_F32; }

}  // namespace

namespace {
int rmsnorm_fwd_checked(const char* who, const void* x, const void* res, void* sum_out, const void* w, void* y,
                        float* rstd_out, int64_t rows, int32_t hidden, float eps, int32_t dtype, mlts_stream_t stream) {
  MLTS_REQUIRE(known_dtype(dtype), "%s: unknown dtype %d", who, dtype);
  MLTS_REQUIRE(rows >= 0 && hidden > 0, "%s: bad shape rows=%lld hidden=%d", who, (long long)rows, hidden);
  MLTS_REQUIRE(hidden % elem_per_vec(dtype) == 0, "%s: hidden=%d must be a multiple of %d", who, hidden, elem_per_vec(dtype));
  if (rows == 0) return MLTS_OK;
  MLTS_REQUIRE(x && w && y, "%s: null pointer", who);
  MLTS_REQUIRE(mlts_aligned16(x) && mlts_aligned16(w) && mlts_aligned16(y), "%s: pointers must be 16-byte aligned", who);
  if (res) {
    MLTS_REQUIRE(sum_out, "%s: null pointer", who);
    MLTS_REQUIRE(mlts_aligned16(res) && mlts_aligned16(sum_out), "%s: pointers must be 16-byte aligned", who);
    MLTS_REQUIRE(sum_out != y, "%s: sum_out and y must be different buffers", who);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == MLTS_BF16 ? rmsnorm_fwd_t<bf16_t>(x, res, sum_out, w, y, rstd_out, rows, hidden, eps, st)
                            : rmsnorm_fwd_t<float>(x, res, sum_out, w, y, rstd_out, rows, hidden, eps, st);
}
}  // namespace

extern "C" int mlts_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd_out, int64_t rows, int32_t hidden,
                                float eps, int32_t dtype, mlts_stream_t stream) {
  return rmsnorm_fwd_checked("mlts_rmsnorm_fwd", x, nullptr, nullptr, w, y, rstd_out, rows, hidden, eps, dtype, stream);
}

extern "C" int mlts_add_rmsnorm_fwd(const void* x, const void* res, void* sum_out, const void* w, void* y, float* rstd_out,
                                    int64_t rows, int32_t hidden, float eps, int32_t dtype, mlts_stream_t stream) {
  MLTS_REQUIRE(rows == 0 || res, "mlts_add_rmsnorm_fwd: null pointer");
  return rmsnorm_fwd_checked("mlts_add_rmsnorm_fwd", x, res, sum_out, w, y, rstd_out, rows, hidden, eps, dtype, stream);
}

extern "C" int64_t mlts_rmsnorm_bwd_workspace_bytes(int64_t rows, int32_t hidden) {
  return static_cast<int64_t>(rmsnorm_bwd_blocks(rows)) * hidden * static_cast<int64_t>(sizeof(float));
}

namespace {
int rmsnorm_bwd_checked(const char* who, const void* dy, const void* x, const void* w, const float* rstd, const void* dres,
                        void* dx, void* dw, void* workspace, int64_t workspace_bytes, int64_t rows, int32_t hidden,
                        int32_t dtype, mlts_stream_t stream) {
  MLTS_REQUIRE(known_dtype(dtype), "%s: unknown dtype %d", who, dtype);
  MLTS_REQUIRE(rows > 0 && hidden > 0, "%s: bad shape rows=%lld hidden=%d", who, (long long)rows, hidden);
  const int n = elem_per_vec(dtype);
  MLTS_REQUIRE(hidden % n == 0, "%s: hidden=%d must be a multiple of %d", who, hidden, n);
  MLTS_REQUIRE(hidden <= MLTS_WAVE * n * kMaxChunks, "%s: hidden=%d exceeds the supported maximum %d", who, hidden,
               MLTS_WAVE * n * kMaxChunks);
  MLTS_REQUIRE(dy && x && w && rstd && dx && dw && workspace, "%s: null pointer", who);
  MLTS_REQUIRE(mlts_aligned16(dy) && mlts_aligned16(x) && mlts_aligned16(w) && mlts_aligned16(dx) && mlts_aligned16(dres),
               "%s: pointers must be 16-byte aligned", who);
  MLTS_REQUIRE(workspace_bytes >= mlts_rmsnorm_bwd_workspace_bytes(rows, hidden), "%s: workspace too small (%lld < %lld)",
               who, (long long)workspace_bytes, (long long)mlts_rmsnorm_bwd_workspace_bytes(rows, hidden));
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* partial = static_cast<float*>(workspace);
  return dtype == MLTS_BF16 ? rmsnorm_bwd_t<bf16_t>(dy, x, w, rstd, dres, dx, dw, partial, rows, hidden, st)
                            : rmsnorm_bwd_t<float>(dy, x, w, rstd, dres, dx, dw, partial, rows, hidden, st);
}
}  // namespace

extern "C" int mlts_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, void* dx, void* dw,
                                void* workspace, int64_t workspace_bytes, int64_t rows, int32_t hidden, int32_t dtype,
                                mlts_stream_t stream) {
  return rmsnorm_bwd_checked("mlts_rmsnorm_bwd", dy, x, w, rstd, nullptr, dx, dw, workspace, workspace_bytes, rows, hidden,
                             dtype, stream);
}

extern "C" int mlts_add_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, const void* dres,
                                    void* dx, void* dw, void* workspace, int64_t workspace_bytes, int64_t rows,
                                    int32_t hidden, int32_t dtype, mlts_stream_t stream) {
  MLTS_REQUIRE(dres, "mlts_add_rmsnorm_bwd: null pointer");
  return rmsnorm_bwd_checked("mlts_add_rmsnorm_bwd", dy, x, w, rstd, dres, dx, dw, workspace, workspace_bytes, rows,
                             hidden, dtype, stream);
}

// validation shared by mlts_rope and mlts_rope_pair
static int rope_check(const char* who, const void* x, const int64_t* x_stride, const void* y, const int64_t* y_stride,
                      const void* cos_tab, const void* sin_tab, int32_t max_pos, const int32_t* positions,
                      int32_t position_offset, int32_t B, int32_t H, int32_t S, int32_t D, int32_t dtype) {
  MLTS_REQUIRE(known_dtype(dtype), "%s: unknown dtype %d", who, dtype);
  MLTS_REQUIRE(B >= 0 && H >= 0 && S >= 0 && D > 0, "%s: bad shape", who);
  const int n = elem_per_vec(dtype);
  const int esz = dtype == MLTS_BF16 ? 2 : 4;
  MLTS_REQUIRE(D % n == 0, "%s: head_dim=%d must be a multiple of %d", who, D, n);
  if (B == 0 || H == 0 || S == 0) return MLTS_OK;
  MLTS_REQUIRE(x && y && cos_tab && sin_tab && x_stride && y_stride, "%s: null pointer", who);
  MLTS_REQUIRE(max_pos > 0, "%s: max_pos must be positive", who);
  MLTS_REQUIRE(positions != nullptr || (position_offset >= 0 && position_offset + S <= max_pos),
               "%s: positions [%d, %d) exceed the table (%d rows)", who, position_offset, position_offset + S, max_pos);
  MLTS_REQUIRE(mlts_aligned16(x) && mlts_aligned16(y), "%s: x and y must be 16-byte aligned", who);
  MLTS_REQUIRE((reinterpret_cast<uintptr_t>(cos_tab) & 7u) == 0 && (reinterpret_cast<uintptr_t>(sin_tab) & 7u) == 0,
               "%s: the cos / sin tables must be 8-byte aligned", who);
  for (int i = 0; i < 3; ++i)
    MLTS_REQUIRE((x_stride[i] * esz) % 16 == 0 && (y_stride[i] * esz) % 16 == 0,
                 "%s: strides must keep rows 16-byte aligned", who);
  return MLTS_OK;
}

extern "C" int mlts_rope(const void* x, const int64_t x_stride[3], void* y, const int64_t y_stride[3],
                         const void* cos_tab, const void* sin_tab, int32_t max_pos, const int32_t* positions,
                         int32_t position_offset, int32_t B, int32_t H, int32_t S, int32_t D, int32_t dtype,
                         int32_t inverse, mlts_stream_t stream) {
  if (int rc = rope_check("mlts_rope", x, x_stride, y, y_stride, cos_tab, sin_tab, max_pos, positions, position_offset, B,
                          H, S, D, dtype); rc != MLTS_OK)
    return rc;
  if (B == 0 || H == 0 || S == 0) return MLTS_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == MLTS_BF16 ? rope_t<bf16_t>(x, x_stride, y, y_stride, cos_tab, sin_tab, max_pos, positions,
                                             position_offset, B, H, S, D, inverse, st)
                            : rope_t<float>(x, x_stride, y, y_stride, cos_tab, sin_tab, max_pos, positions,
                                            position_offset, B, H, S, D, inverse, st);
}

template <typename T>
static int rope_pair_t(const RopeOperand& a, const RopeOperand& b, const void* ct, const void* sn, int max_pos,
                       const int32_t* positions, int off, int B, int S, int D, int inverse, hipStream_t st) {
  MltsKernelTimer timer("rope", st);
  constexpr int N = Vec16<T>::N;
  const int64_t per_head = static_cast<int64_t>(B) * S * (D / N);
  const int64_t blocks_a = (per_head * a.H + kThreads - 1) / kThreads, blocks_b = (per_head * b.H + kThreads - 1) / kThreads;
  if (inverse)
    hipLaunchKernelGGL((rope_pair_kernel<T, true>), dim3((unsigned)(blocks_a + blocks_b)), dim3(kThreads), 0, st, a, b,
                       (unsigned)blocks_a, static_cast<const T*>(ct), static_cast<const T*>(sn), max_pos, positions, off, B, S, D);
  else
    hipLaunchKernelGGL((rope_pair_kernel<T, false>), dim3((unsigned)(blocks_a + blocks_b)), dim3(kThreads), 0, st, a, b,
                       (unsigned)blocks_a, static_cast<const T*>(ct), static_cast<const T*>(sn), max_pos, positions, off, B, S, D);
  return mlts_check_launch("mlts_rope_pair");
}

extern "C" int mlts_rope_pair(const void* xa, const int64_t xa_stride[3], void* ya, const int64_t ya_stride[3], int32_t Ha,
                              const void* xb, const int64_t xb_stride[3], void* yb, const int64_t yb_stride[3], int32_t Hb,
                              const void* cos_tab, const void* sin_tab, int32_t max_pos, const int32_t* positions,
                              int32_t position_offset, int32_t B, int32_t S, int32_t D, int32_t dtype, int32_t inverse,
                              mlts_stream_t stream) {
  if (int rc = rope_check("mlts_rope_pair", xa, xa_stride, ya, ya_stride, cos_tab, sin_tab, max_pos, positions,
                          position_offset, B, Ha, S, D, dtype); rc != MLTS_OK)
    return rc;
  if (int rc = rope_check("mlts_rope_pair", xb, xb_stride, yb, yb_stride, cos_tab, sin_tab, max_pos, positions,
                          position_offset, B, Hb, S, D, dtype); rc != MLTS_OK)
    return rc;
  if (B == 0 || S == 0 || (Ha == 0 && Hb == 0)) return MLTS_OK;
  const int n = elem_per_vec(dtype);
  MLTS_REQUIRE(static_cast<int64_t>(B) * S * (Ha > Hb ? Ha : Hb) * (D / n) < (1LL << 31),
               "mlts_rope_pair: tensors of 2^31 or more 16-byte vectors go through mlts_rope");
  RopeOperand a{xa, ya, {xa_stride[0], xa_stride[1], xa_stride[2]}, {ya_stride[0], ya_stride[1], ya_stride[2]}, Ha};
  RopeOperand b{xb, yb, {xb_stride[0], xb_stride[1], xb_stride[2]}, {yb_stride[0], yb_stride[1], yb_stride[2]}, Hb};
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == MLTS_BF16 ? rope_pair_t<bf16_t>(a, b, cos_tab, sin_tab, max_pos, positions, position_offset, B, S, D, inverse, st)
                            : rope_pair_t<float>(a, b, cos_tab, sin_tab, max_pos, positions, position_offset, B, S, D, inverse, st);
}

extern "C" int mlts_swiglu_fwd(const void* gate, const void* up, void* h, int64_t n, int32_t dtype,
                               mlts_stream_t stream) {
  MLTS_REQUIRE(known_dtype(dtype), "mlts_swiglu_fwd: unknown dtype %d", dtype);
  MLTS_REQUIRE(n >= 0, "mlts_swiglu_fwd: n must be >= 0");
  if (n == 0) return MLTS_OK;
  MLTS_REQUIRE(gate && up && h, "mlts_swiglu_fwd: null pointer");
  const bool vec = mlts_aligned16(gate) && mlts_aligned16(up) && mlts_aligned16(h);
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == MLTS_BF16 ? swiglu_fwd_t<bf16_t>(gate, up, h, n, vec, st) : swiglu_fwd_t<float>(gate, up, h, n, vec, st);
}

extern "C" int mlts_swiglu_bwd(const void* dh, const void* gate, const void* up, void* dgate, void* dup, int64_t n,
                               int32_t dtype, mlts_stream_t stream) {
  MLTS_REQUIRE(known_dtype(dtype), "mlts_swiglu_bwd: unknown dtype %d", dtype);
  MLTS_REQUIRE(n >= 0, "mlts_swiglu_bwd: n must be >= 0");
  if (n == 0) return MLTS_OK;
  MLTS_REQUIRE(dh && gate && up && dgate && dup, "mlts_swiglu_bwd: null pointer");
  const bool vec = mlts_aligned16(dh) && mlts_aligned16(gate) && mlts_aligned16(up) && mlts_aligned16(dgate) &&
                   mlts_aligned16(dup);
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == MLTS_BF16 ? swiglu_bwd_t<bf16_t>(dh, gate, up, dgate, dup, n, vec, st)
                            : swiglu_bwd_t<float>(dh, gate, up, dgate, dup, n, vec, st);
}

namespace {
int swiglu_rows_check(const char* who, int64_t rows, int64_t cols, int32_t dtype, std::initializer_list<const void*> ptrs,
                      std::initializer_list<int64_t> lds) {
  MLTS_REQUIRE(known_dtype(dtype), "%s: unknown dtype %d", who, dtype);
  const int n = elem_per_vec(dtype);
  MLTS_REQUIRE(rows >= 0 && cols >= 0 && cols % n == 0, "%s: cols=%lld must be a multiple of %d", who, (long long)cols, n);
  MLTS_REQUIRE(rows * (cols / n) < (int64_t{1} << 31), "%s: rows * cols too large", who);
  for (const void* q : ptrs) MLTS_REQUIRE(rows * cols == 0 || (q && mlts_aligned16(q)), "%s: null or unaligned pointer", who);
  for (int64_t ld : lds) MLTS_REQUIRE(ld >= cols && ld % n == 0, "%s: row strides must be >= cols and multiples of %d", who, n);
  return MLTS_OK;
}
}  // namespace

extern "C" int mlts_swiglu_fwd_rows(const void* gate, const void* up, int64_t ld_in, void* h, int64_t ld_h, int64_t rows,
                                    int64_t cols, int32_t dtype, mlts_stream_t stream) {
  if (int rc = swiglu_rows_check("mlts_swiglu_fwd_rows", rows, cols, dtype, {gate, up, h}, {ld_in, ld_h}); rc != MLTS_OK) return rc;
  if (rows * cols == 0) return MLTS_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  MltsKernelTimer timer("swiglu_fwd", st);
  const uint32_t vpr = static_cast<uint32_t>(cols / elem_per_vec(dtype)), nvec = static_cast<uint32_t>(rows) * vpr;
  if (dtype == MLTS_BF16)
    hipLaunchKernelGGL(swiglu_fwd_rows_kernel<bf16_t>, dim3(stream_grid(nvec)), dim3(kThreads), 0, st, static_cast<const bf16_t*>(gate),
                       static_cast<const bf16_t*>(up), ld_in, static_cast<bf16_t*>(h), ld_h, vpr, nvec);
  else
    hipLaunchKernelGGL(swiglu_fwd_rows_kernel<float>, dim3(stream_grid(nvec)), dim3(kThreads), 0, st, static_cast<const float*>(gate),
                       static_cast<const float*>(up), ld_in, static_cast<float*>(h), ld_h, vpr, nvec);
  return mlts_check_launch("mlts_swiglu_fwd_rows");
}

extern "C" int mlts_swiglu_bwd_rows(const void* dh, int64_t ld_dh, const void* gate, const void* up, int64_t ld_in, void* dgate,
                                    void* dup, int64_t ld_out, int64_t rows, int64_t cols, int32_t dtype, mlts_stream_t stream) {
  if (int rc = swiglu_rows_check("mlts_swiglu_bwd_rows", rows, cols, dtype, {dh, gate, up, dgate, dup}, {ld_dh, ld_in, ld_out});
      rc != MLTS_OK)
    return rc;
  if (rows * cols == 0) return MLTS_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  MltsKernelTimer timer("swiglu_bwd", st);
  const uint32_t vpr = static_cast<uint32_t>(cols / elem_per_vec(dtype)), nvec = static_cast<uint32_t>(rows) * vpr;
  if (dtype == MLTS_BF16)
    hipLaunchKernelGGL(swiglu_bwd_rows_kernel<bf16_t>, dim3(stream_grid(nvec)), dim3(kThreads), 0, st, static_cast<const bf16_t*>(dh),
                       ld_dh, static_cast<const bf16_t*>(gate), static_cast<const bf16_t*>(up), ld_in, static_cast<bf16_t*>(dgate),
                       static_cast<bf16_t*>(dup), ld_out, vpr, nvec);
  else
    hipLaunchKernelGGL(swiglu_bwd_rows_kernel<float>, dim3(stream_grid(nvec)), dim3(kThreads), 0, st, static_cast<const float*>(dh), ld_dh,
                       static_cast<const float*>(gate), static_cast<const float*>(up), ld_in, static_cast<float*>(dgate),
                       static_cast<float*>(dup), ld_out, vpr, nvec);
  return mlts_check_launch("mlts_swiglu_bwd_rows");
}
