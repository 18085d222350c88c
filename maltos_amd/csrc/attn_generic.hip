// Generic attention kernels: any head_dim <= 192, fp32 or bf16 storage, fp32 arithmetic on the
// vector ALU (no MFMA).  They serve the fp32 configurations (1e-4 parity with the fp32 reference)
// and head dims the MFMA kernels do not cover.  Structure: a workgroup owns 16 query rows (forward,
// dQ) or 16 key rows (dK/dV) and walks the other side in tiles of 64 staged in LDS; in the score
// phase a lane owns one column of the tile so that row reductions are 64-lane shuffles; in the
// accumulate phase lanes own head-dim columns so that global accesses are coalesced.
#include "attn_common.hpp"

namespace {

constexpr int GT = 256;        // threads
constexpr int GROWS = 16;      // owned rows per workgroup (4 per wavefront)
constexpr int GTILE = 64;      // tile of the walked side
constexpr int GMAXDD = 4;      // head_dim <= 64 * GMAXDD

template <typename T>
__device__ __forceinline__ void load_tile(float* dst, int dstride, const T* src, int64_t row_stride, int row0, int nrows,
                                          int row_limit, int D) {
  // dst[r][d] = src[(row0 + r)][d] for r < nrows, zero beyond row_limit
  for (int idx = threadIdx.x; idx < nrows * D; idx += GT) {
    const int r = idx / D, d = idx - r * D;
    const int row = row0 + r;
    dst[r * dstride + d] = row < row_limit ? to_f32<T>(src[static_cast<int64_t>(row) * row_stride + d]) : 0.f;
  }
}

template <int MODE>
__device__ __forceinline__ bool visible(const AttnParams& p, int b, int qi, int kj) {
  if (qi >= p.Sq || kj >= p.Sk) return false;
  if (MODE == MLTS_MASK_CAUSAL) return kj <= qi + p.causal_off;
  if (MODE == MLTS_MASK_DOC) {
    const int qp = p.q_pos[static_cast<int64_t>(b) * p.Sq + qi], qs = p.q_seq[static_cast<int64_t>(b) * p.Sq + qi];
    const int kp = p.k_pos[static_cast<int64_t>(b) * p.Sk + kj], ks = p.k_seq[static_cast<int64_t>(b) * p.Sk + kj];
    return kp <= qp && ks == qs && qs >= 0;
  }
  return true;
}

// LDS carve-up (floats): own[GROWS][D], own2[GROWS][D], ta[GTILE][D+1], tb[GTILE][D+1], pa[GROWS][GTILE], pb[GROWS][GTILE]
__host__ __device__ inline size_t generic_lds_floats(int D) {
  return static_cast<size_t>(2 * GROWS * D + 2 * GTILE * (D + 1) + 2 * GROWS * GTILE);
}

template <typename T, int MODE>
__global__ __launch_bounds__(GT) void attn_generic_fwd(const AttnParams p, int D) {
  extern __shared__ float lds[];
  float* sQ = lds;
  float* sK = lds + 2 * GROWS * D;
  float* sV = sK + GTILE * (D + 1);
  float* sP = sV + GTILE * (D + 1);
  const int TS = D + 1;
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int q0 = blockIdx.x * GROWS;
  const int bh = blockIdx.y, b = bh / p.Hq, hq = bh % p.Hq, hkv = hq / (p.Hq / p.Hkv);
  const T* Q = static_cast<const T*>(p.q) + b * p.qs[0] + hq * p.qs[1];
  const T* K = static_cast<const T*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const T* V = static_cast<const T*>(p.v) + b * p.vs[0] + hkv * p.vs[1];
  T* O = static_cast<T*>(p.o) + b * p.os[0] + hq * p.os[1];

  load_tile<T>(sQ, D, Q, p.qs[2], q0, GROWS, p.Sq, D);
  float m[4], l[4], o[4][GMAXDD];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int dd = 0; dd < GMAXDD; ++dd) o[r][dd] = 0.f;
  }
  int kend = p.Sk;
  if (MODE == MLTS_MASK_CAUSAL) kend = max(0, min(p.Sk, min(q0 + GROWS, p.Sq) + p.causal_off));
  for (int k0 = 0; k0 < kend; k0 += GTILE) {
    __syncthreads();
    load_tile<T>(sK, TS, K, p.ks[2], k0, GTILE, p.Sk, D);
    load_tile<T>(sV, TS, V, p.vs[2], k0, GTILE, p.Sk, D);
    __syncthreads();
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    for (int d = 0; d < D; ++d) {
      const float kv = sK[lane * TS + d];
#pragma unroll
      for (int r = 0; r < 4; ++r) s[r] += sQ[(4 * g + r) * D + d] * kv;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const bool vis = visible<MODE>(p, b, q0 + 4 * g + r, k0 + lane);
      const float sc = vis ? s[r] * p.scale : -INFINITY;
      const float mx = wave_max(sc);
      const float m_new = fmaxf(m[r], mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = expf(m[r] - m_use);
      const float pv = expf(sc - m_use);
      l[r] = l[r] * alpha + wave_sum(pv);
      m[r] = m_new;
      sP[(4 * g + r) * GTILE + lane] = pv;
#pragma unroll
      for (int dd = 0; dd < GMAXDD; ++dd) o[r][dd] *= alpha;
    }
    // sP rows of this wavefront were written by this wavefront only
    for (int jj = 0; jj < GTILE; ++jj) {
#pragma unroll
      for (int dd = 0; dd < GMAXDD; ++dd) {
        const int d = lane + 64 * dd;
        if (d < D) {
          const float vv = sV[jj * TS + d];
#pragma unroll
          for (int r = 0; r < 4; ++r) o[r][dd] += sP[(4 * g + r) * GTILE + jj] * vv;
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = q0 + 4 * g + r;
    if (row >= p.Sq) continue;
    const float inv = l[r] > 0.f ? 1.0f / l[r] : 0.f;
#pragma unroll
    for (int dd = 0; dd < GMAXDD; ++dd) {
      const int d = lane + 64 * dd;
      if (d < D) O[static_cast<int64_t>(row) * p.os[2] + d] = from_f32<T>(o[r][dd] * inv);
    }
    if (lane == 0)
      p.lse[(static_cast<int64_t>(b) * p.Hq + hq) * p.Sq + row] = l[r] > 0.f ? m[r] + logf(l[r]) : -INFINITY;
  }
}

// dQ for 16 query rows: dq = scale * sum_j ds_ij k_j, ds = p (dp - delta), p = exp(scale s - lse).
// bp.dq_f32: dq is fp32 and added to (1) or overwritten (2); 0: dq has the input dtype.
template <typename T, int MODE>
__global__ __launch_bounds__(GT) void attn_generic_bwd_dq(const AttnBwdParams bp, int D) {
  const AttnParams& p = bp.a;
  extern __shared__ float lds[];
  float* sQ = lds;
  float* sdO = lds + GROWS * D;
  float* sK = lds + 2 * GROWS * D;
  float* sV = sK + GTILE * (D + 1);
  float* sP = sV + GTILE * (D + 1);
  const int TS = D + 1;
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int q0 = blockIdx.x * GROWS;
  const int bh = blockIdx.y, b = bh / p.Hq, hq = bh % p.Hq, hkv = hq / (p.Hq / p.Hkv);
  const T* Q = static_cast<const T*>(p.q) + b * p.qs[0] + hq * p.qs[1];
  const T* K = static_cast<const T*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const T* V = static_cast<const T*>(p.v) + b * p.vs[0] + hkv * p.vs[1];
  const T* dO = static_cast<const T*>(bp.dout) + b * bp.dos[0] + hq * bp.dos[1];

  load_tile<T>(sQ, D, Q, p.qs[2], q0, GROWS, p.Sq, D);
  load_tile<T>(sdO, D, dO, bp.dos[2], q0, GROWS, p.Sq, D);
  float lse_r[4], dl_r[4], dq[4][GMAXDD];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = q0 + 4 * g + r;
    const int64_t off = (static_cast<int64_t>(b) * p.Hq + hq) * p.Sq + row;
    lse_r[r] = row < p.Sq ? p.lse[off] : 0.f;
    dl_r[r] = row < p.Sq ? bp.delta[off] : 0.f;
#pragma unroll
    for (int dd = 0; dd < GMAXDD; ++dd) dq[r][dd] = 0.f;
  }
  int kend = p.Sk;
  if (MODE == MLTS_MASK_CAUSAL) kend = max(0, min(p.Sk, min(q0 + GROWS, p.Sq) + p.causal_off));
  for (int k0 = 0; k0 < kend; k0 += GTILE) {
    __syncthreads();
    load_tile<T>(sK, TS, K, p.ks[2], k0, GTILE, p.Sk, D);
    load_tile<T>(sV, TS, V, p.vs[2], k0, GTILE, p.Sk, D);
    __syncthreads();
    float s[4] = {0.f, 0.f, 0.f, 0.f}, dp[4] = {0.f, 0.f, 0.f, 0.f};
    for (int d = 0; d < D; ++d) {
      const float kv = sK[lane * TS + d], vv = sV[lane * TS + d];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[r] += sQ[(4 * g + r) * D + d] * kv;
        dp[r] += sdO[(4 * g + r) * D + d] * vv;
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const bool vis = visible<MODE>(p, b, q0 + 4 * g + r, k0 + lane) && lse_r[r] != -INFINITY;
      const float pv = vis ? expf(s[r] * p.scale - lse_r[r]) : 0.f;
      sP[(4 * g + r) * GTILE + lane] = pv * (dp[r] - dl_r[r]);
    }
    for (int jj = 0; jj < GTILE; ++jj) {
#pragma unroll
      for (int dd = 0; dd < GMAXDD; ++dd) {
        const int d = lane + 64 * dd;
        if (d < D) {
          const float kk = sK[jj * TS + d];
#pragma unroll
          for (int r = 0; r < 4; ++r) dq[r][dd] += sP[(4 * g + r) * GTILE + jj] * kk;
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = q0 + 4 * g + r;
    if (row >= p.Sq) continue;
#pragma unroll
    for (int dd = 0; dd < GMAXDD; ++dd) {
      const int d = lane + 64 * dd;
      if (d >= D) continue;
      const int64_t off = b * bp.dqs[0] + hq * bp.dqs[1] + static_cast<int64_t>(row) * bp.dqs[2] + d;
      if (bp.dq_f32 == 1) bp.dq_acc[off] += dq[r][dd] * p.scale;
      else if (bp.dq_f32 == 2) bp.dq_acc[off] = dq[r][dd] * p.scale;
      else reinterpret_cast<T*>(bp.dq_acc)[off] = from_f32<T>(dq[r][dd] * p.scale);
    }
  }
}

// dK, dV for 16 key rows of one KV head, summed over the query heads of its group.
template <typename T, int MODE, bool F32_ACC>
__global__ __launch_bounds__(GT) void attn_generic_bwd_dkv(const AttnBwdParams bp, int D) {
  const AttnParams& p = bp.a;
  extern __shared__ float lds[];
  float* sKk = lds;
  float* sVk = lds + GROWS * D;
  float* sQ = lds + 2 * GROWS * D;
  float* sdO = sQ + GTILE * (D + 1);
  float* sP = sdO + GTILE * (D + 1);
  float* sdS = sP + GROWS * GTILE;
  const int TS = D + 1;
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int k0 = blockIdx.x * GROWS;
  const int bh = blockIdx.y, b = bh / p.Hkv, hkv = bh % p.Hkv;
  const int group = p.Hq / p.Hkv;
  const T* K = static_cast<const T*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const T* V = static_cast<const T*>(p.v) + b * p.vs[0] + hkv * p.vs[1];
  load_tile<T>(sKk, D, K, p.ks[2], k0, GROWS, p.Sk, D);
  load_tile<T>(sVk, D, V, p.vs[2], k0, GROWS, p.Sk, D);
  float dk[4][GMAXDD], dv[4][GMAXDD];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int dd = 0; dd < GMAXDD; ++dd) dk[r][dd] = dv[r][dd] = 0.f;

  int qstart = 0;
  if (MODE == MLTS_MASK_CAUSAL) qstart = max(0, k0 - p.causal_off) / GTILE * GTILE;  // first query that can see key k0
  for (int hg = 0; hg < group; ++hg) {
    const int hq = hkv * group + hg;
    const T* Q = static_cast<const T*>(p.q) + b * p.qs[0] + hq * p.qs[1];
    const T* dO = static_cast<const T*>(bp.dout) + b * bp.dos[0] + hq * bp.dos[1];
    for (int q0 = qstart; q0 < p.Sq; q0 += GTILE) {
      __syncthreads();
      load_tile<T>(sQ, TS, Q, p.qs[2], q0, GTILE, p.Sq, D);
      load_tile<T>(sdO, TS, dO, bp.dos[2], q0, GTILE, p.Sq, D);
      __syncthreads();
      const int qi = q0 + lane;
      const int64_t off = (static_cast<int64_t>(b) * p.Hq + hq) * p.Sq + qi;
      const float lse_q = qi < p.Sq ? p.lse[off] : -INFINITY;
      const float dl_q = qi < p.Sq ? bp.delta[off] : 0.f;
      float s[4] = {0.f, 0.f, 0.f, 0.f}, dp[4] = {0.f, 0.f, 0.f, 0.f};
      for (int d = 0; d < D; ++d) {
        const float qv = sQ[lane * TS + d], dov = sdO[lane * TS + d];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          s[r] += sKk[(4 * g + r) * D + d] * qv;
          dp[r] += sVk[(4 * g + r) * D + d] * dov;
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool vis = visible<MODE>(p, b, qi, k0 + 4 * g + r) && lse_q != -INFINITY;
        const float pv = vis ? expf(s[r] * p.scale - lse_q) : 0.f;
        sP[(4 * g + r) * GTILE + lane] = pv;
        sdS[(4 * g + r) * GTILE + lane] = pv * (dp[r] - dl_q);
      }
      for (int qq = 0; qq < GTILE; ++qq) {
#pragma unroll
        for (int dd = 0; dd < GMAXDD; ++dd) {
          const int d = lane + 64 * dd;
          if (d < D) {
            const float dov = sdO[qq * TS + d], qv = sQ[qq * TS + d];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              dv[r][dd] += sP[(4 * g + r) * GTILE + qq] * dov;
              dk[r][dd] += sdS[(4 * g + r) * GTILE + qq] * qv;
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = k0 + 4 * g + r;
    if (row >= p.Sk) continue;
#pragma unroll
    for (int dd = 0; dd < GMAXDD; ++dd) {
      const int d = lane + 64 * dd;
      if (d >= D) continue;
      const int64_t ok = b * bp.dks[0] + hkv * bp.dks[1] + static_cast<int64_t>(row) * bp.dks[2] + d;
      const int64_t ov = b * bp.dvs[0] + hkv * bp.dvs[1] + static_cast<int64_t>(row) * bp.dvs[2] + d;
      if (F32_ACC) {
        static_cast<float*>(bp.dk)[ok] += dk[r][dd] * p.scale;
        static_cast<float*>(bp.dv)[ov] += dv[r][dd];
      } else {
        static_cast<T*>(bp.dk)[ok] = from_f32<T>(dk[r][dd] * p.scale);
        static_cast<T*>(bp.dv)[ov] = from_f32<T>(dv[r][dd]);
      }
    }
  }
}

// delta[b, h, q] = sum_d dO * O: one wavefront per row.
template <typename T>
__global__ __launch_bounds__(GT) void attn_delta_kernel(const T* __restrict__ dout, int64_t ds0, int64_t ds1, int64_t ds2,
                                                        const T* __restrict__ o, int64_t os0, int64_t os1, int64_t os2,
                                                        float* __restrict__ delta, int B, int H, int S, int D) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (GT / 64) + (threadIdx.x >> 6);
  const int64_t total = static_cast<int64_t>(B) * H * S;
  if (row >= total) return;
  const int s = static_cast<int>(row % S);
  const int h = static_cast<int>((row / S) % H);
  const int b = static_cast<int>(row / (static_cast<int64_t>(S) * H));
  const T* dp = dout + b * ds0 + h * ds1 + static_cast<int64_t>(s) * ds2;
  const T* op = o + b * os0 + h * os1 + static_cast<int64_t>(s) * os2;
  float acc = 0.f;
  for (int d = lane; d < D; d += 64) acc += to_f32<T>(dp[d]) * to_f32<T>(op[d]);
  acc = wave_sum(acc);
  if (lane == 0) delta[row] = acc;
}

// bf16, head_dim a multiple of 8, 16-byte aligned rows: D / 8 lanes share a row (one 16-byte load of dO and of O per
// lane), four rows per lane group in flight.  The plain kernel above reads two bytes per lane and reaches 3 TB/s.
// IDX: type the row index is split in (32-bit below 2^31 rows: 64-bit divisions would dominate the kernel).
template <int LPR, typename IDX>  // lanes per row, a power of two <= 32
__global__ __launch_bounds__(256) void attn_delta_vec_kernel(const bf16_t* __restrict__ dout, int64_t ds0, int64_t ds1, int64_t ds2,
                                                              const bf16_t* __restrict__ o, int64_t os0, int64_t os1, int64_t os2,
                                                              float* __restrict__ delta, int H, int S, int64_t total, int D) {
  constexpr int RPB = 256 / LPR;  // rows per block and pass
  constexpr int UNROLL = 4;
  const int sub = threadIdx.x % LPR;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * (RPB * UNROLL) + threadIdx.x / LPR;
  typedef int v4i32 __attribute__((ext_vector_type(4)));
  v4i32 a[UNROLL], c[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const IDX row = static_cast<IDX>(min(row0 + u * RPB, total - 1));
    const IDX bh = row / static_cast<IDX>(S);
    const int s = static_cast<int>(row - bh * static_cast<IDX>(S));
    const int64_t b = static_cast<int64_t>(bh / static_cast<IDX>(H));
    const int h = static_cast<int>(bh - static_cast<IDX>(b) * static_cast<IDX>(H));
    a[u] = v4i32{0, 0, 0, 0};
    c[u] = v4i32{0, 0, 0, 0};
    if (sub * 8 < D) {
      a[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i32*>(dout + b * ds0 + h * ds1 + static_cast<int64_t>(s) * ds2 + sub * 8));
      c[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i32*>(o + b * os0 + h * os1 + static_cast<int64_t>(s) * os2 + sub * 8));
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // two bf16 per 32-bit word: low half = even element
      acc += __builtin_bit_cast(float, a[u][i] << 16) * __builtin_bit_cast(float, c[u][i] << 16);
      acc += __builtin_bit_cast(float, a[u][i] & static_cast<int>(0xffff0000u)) * __builtin_bit_cast(float, c[u][i] & static_cast<int>(0xffff0000u));
    }
#pragma unroll
    for (int m = LPR / 2; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
    const int64_t row = row0 + u * RPB;
    if (sub == 0 && row < total) delta[row] = acc;
  }
}

template <typename KERN>
int set_lds(KERN kern, size_t bytes, const char* what) {
  if (bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(bytes));
    if (e != hipSuccess) {
      mlts_set_error("%s: cannot reserve %zu bytes of LDS: %s", what, bytes, hipGetErrorString(e));
      return MLTS_ERR_LAUNCH;
    }
  }
  return MLTS_OK;
}

template <typename T, int MODE>
int generic_fwd_t(const AttnParams& p, int D, hipStream_t st) {
  const size_t lds = generic_lds_floats(D) * sizeof(float);
  auto kern = attn_generic_fwd<T, MODE>;
  if (int rc = set_lds(kern, lds, "mlts_attn_fwd")) return rc;
  dim3 grid((p.Sq + GROWS - 1) / GROWS, p.B * p.Hq);
  hipLaunchKernelGGL(kern, grid, dim3(GT), lds, st, p, D);
  return mlts_check_launch("mlts_attn_fwd");
}

template <typename T, int MODE>
int generic_bwd_t(const AttnBwdParams& bp, int D, hipStream_t st) {
  const AttnParams& p = bp.a;
  const size_t lds = generic_lds_floats(D) * sizeof(float);
  dim3 gq((p.Sq + GROWS - 1) / GROWS, p.B * p.Hq);
  dim3 gk((p.Sk + GROWS - 1) / GROWS, p.B * p.Hkv);
  auto kq = attn_generic_bwd_dq<T, MODE>;
  if (int rc = set_lds(kq, lds, "mlts_attn_bwd")) return rc;
  hipLaunchKernelGGL(kq, gq, dim3(GT), lds, st, bp, D);
  if (bp.accumulate_f32) {
    auto kk = attn_generic_bwd_dkv<T, MODE, true>;
    if (int rc = set_lds(kk, lds, "mlts_attn_bwd")) return rc;
    hipLaunchKernelGGL(kk, gk, dim3(GT), lds, st, bp, D);
  } else {
    auto kk = attn_generic_bwd_dkv<T, MODE, false>;
    if (int rc = set_lds(kk, lds, "mlts_attn_bwd")) return rc;
    hipLaunchKernelGGL(kk, gk, dim3(GT), lds, st, bp, D);
  }
  return mlts_check_launch("mlts_attn_bwd");
}

}  // namespace

int mlts_attn_generic_fwd(const AttnParams& p, int D, int dtype, int mode, hipStream_t st) {
#define MLTS_GF(T)                                                         \
  do {                                                                     \
    if (mode == MLTS_MASK_NONE) return generic_fwd_t<T, MLTS_MASK_NONE>(p, D, st);     \
    if (mode == MLTS_MASK_CAUSAL) return generic_fwd_t<T, MLTS_MASK_CAUSAL>(p, D, st); \
    return generic_fwd_t<T, MLTS_MASK_DOC>(p, D, st);                      \
  } while (0)
  if (dtype == MLTS_BF16) MLTS_GF(bf16_t);
  MLTS_GF(float);
#undef MLTS_GF
}

int mlts_attn_generic_bwd(const AttnBwdParams& bp, int D, int dtype, int mode, hipStream_t st) {
#define MLTS_GB(T)                                                         \
  do {                                                                     \
    if (mode == MLTS_MASK_NONE) return generic_bwd_t<T, MLTS_MASK_NONE>(bp, D, st);     \
    if (mode == MLTS_MASK_CAUSAL) return generic_bwd_t<T, MLTS_MASK_CAUSAL>(bp, D, st); \
    return generic_bwd_t<T, MLTS_MASK_DOC>(bp, D, st);                     \
  } while (0)
  if (dtype == MLTS_BF16) MLTS_GB(bf16_t);
  MLTS_GB(float);
#undef MLTS_GB
}

int mlts_attn_delta(const void* dout, const int64_t* dos, const void* o, const int64_t* os, float* delta, int B, int H,
                    int S, int D, int dtype, hipStream_t st) {
  const int64_t rows = static_cast<int64_t>(B) * H * S;
  if (rows == 0) return MLTS_OK;
  MltsKernelTimer timer("attn_delta", st);
  const bool vec = dtype == MLTS_BF16 && D % 8 == 0 && D <= 256 && ((dos[0] | dos[1] | dos[2] | os[0] | os[1] | os[2]) & 7) == 0 &&
                   mlts_aligned16(dout) && mlts_aligned16(o);
  if (vec) {
    const int lpr = D <= 64 ? 8 : D <= 128 ? 16 : 32;
    const int64_t rows_per_block = (256 / lpr) * 4;
    const unsigned nb = static_cast<unsigned>((rows + rows_per_block - 1) / rows_per_block);
    const bf16_t* dp = static_cast<const bf16_t*>(dout);
    const bf16_t* op = static_cast<const bf16_t*>(o);
#define MLTS_DELTA_IDX(LPR, IDX) \
  hipLaunchKernelGGL((attn_delta_vec_kernel<LPR, IDX>), dim3(nb), dim3(256), 0, st, dp, dos[0], dos[1], dos[2], op, os[0], os[1], os[2], delta, H, S, rows, D)
#define MLTS_DELTA(LPR)                                  \
  do {                                                   \
    if (rows < (1LL << 31)) MLTS_DELTA_IDX(LPR, uint32_t); \
    else MLTS_DELTA_IDX(LPR, int64_t);                   \
  } while (0)
    if (lpr == 8) MLTS_DELTA(8);
    else if (lpr == 16) MLTS_DELTA(16);
    else MLTS_DELTA(32);
#undef MLTS_DELTA
#undef MLTS_DELTA_IDX
    return mlts_check_launch("mlts_attn_delta");
  }
  const int64_t blocks = (rows + (GT / 64) - 1) / (GT / 64);
  if (dtype == MLTS_BF16)
    hipLaunchKernelGGL(attn_delta_kernel<bf16_t>, dim3((unsigned)blocks), dim3(GT), 0, st, static_cast<const bf16_t*>(dout),
                       dos[0], dos[1], dos[2], static_cast<const bf16_t*>(o), os[0], os[1], os[2], delta, B, H, S, D);
  else
    hipLaunchKernelGGL(attn_delta_kernel<float>, dim3((unsigned)blocks), dim3(GT), 0, st, static_cast<const float*>(dout),
                       dos[0], dos[1], dos[2], static_cast<const float*>(o), os[0], os[1], os[2], delta, B, H, S, D);
  return mlts_check_launch("mlts_attn_delta");
}
