// Attention backward for gfx950 (bf16, head_dim 64/128), part 1 of 2: dK and dV by recompute from
// (Q, K, V, LSE, delta, dO) with v_mfma_f32_32x32x16_bf16.  (dQ is part 2, attn_bwd_dq.hip; splitting the
// backward pass costs two extra GEMMs of recompute but needs no atomics and no dS round trip.)
//
// A workgroup (4 wavefronts) owns 128 keys of one (batch, kv head) and walks the 64-row query
// tiles that can see them, for every query head of the GQA group, so dK/dV are accumulated in
// registers and written exactly once (native GQA, deterministic).  Per tile and wavefront (32 keys):
//     S  = Q K^T        A = Q  (LDS, row major)      B = K  (registers, loaded once)
//     dP = dO V^T       A = dO (LDS, row major)      B = V  (registers, loaded once)
//     P  = exp2(S c - LSE), dS = P (dP - delta)       in registers, lane = key, in-lane = query
//     dV += P^T dO      A = P^T  (registers as is)   B = dO^T (LDS, transposed while staging)
//     dK += dS^T Q      A = dS^T (registers as is)   B = Q^T  (LDS, transposed while staging)
// The accumulator layout of S is the A-operand layout of the dV/dK products, so P and dS never leave
// registers.  Q/dO tiles are double buffered in LDS: one barrier per tile.
#include "attn_common.hpp"
#include <type_traits>

namespace {

constexpr int BKV = 128;
constexpr int BQ = 64;
constexpr int WAVES = 4;
constexpr int THREADS = 256;

template <int D>
struct BwdLds {
  static constexpr int RSTR = D + 8;
  static constexpr int ROW_ELEMS = BQ * RSTR;     // row-major tile
  static constexpr int T_ELEMS = D * BQ;          // transposed tile
  static constexpr int OFF_Q = 0;
  static constexpr int OFF_DO = OFF_Q + ROW_ELEMS;
  static constexpr int OFF_QT = OFF_DO + ROW_ELEMS;
  static constexpr int OFF_DOT = OFF_QT + T_ELEMS;
  static constexpr int OFF_STAT = OFF_DOT + T_ELEMS;  // lse[64], delta[64] as floats
  static constexpr int STAGE = OFF_STAT + 4 * BQ;     // in bf16 elements (the two float arrays take 4 * BQ)
  static constexpr int BYTES = 2 * STAGE * 2;
};

__device__ __forceinline__ int t_swz(int d) { return ((d >> 1) ^ (d >> 4)) & 7; }
__device__ __forceinline__ int t_slot(int r) {
  const int kb = r >> 5, t = (r >> 4) & 1, grp = (r >> 2) & 3;
  return (((kb * 2 + t) * 2 + (grp & 1)) << 3) + ((grp >> 1) << 2) + (r & 3);
}

template <int D, int MODE>
__global__ __launch_bounds__(THREADS, 1) void attn_bwd_kernel(const AttnBwdParams bp) {
  const AttnParams& p = bp.a;
  using L = BwdLds<D>;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int VEC = D / 16;        // elements per thread per staged row
  constexpr int VW = VEC / 2;        // dwords

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* smem = reinterpret_cast<bf16_t*>(smem_raw);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;

  const int nbh = p.B * p.Hkv;
  const int bid = blockIdx.x;
  const int kt = bid / nbh;  // key tile; low tiles see the most queries under a causal mask and go first
  const int bh = bid % nbh;
  const int b = bh / p.Hkv, hkv = bh % p.Hkv;
  const int group = p.Hq / p.Hkv;
  const int kv0 = kt * BKV;
  const int wkv0 = kv0 + wave * 32;

  const bf16_t* K = static_cast<const bf16_t*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + b * p.vs[0] + hkv * p.vs[1];

  // ---- K, V fragments (B operands), loaded once -----------------------------------------
  bf16x8 kf[KS], vf[KS];
  {
    const int row = wkv0 + l32;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (row < p.Sk) {
        kf[ks] = *reinterpret_cast<const bf16x8*>(K + static_cast<int64_t>(row) * p.ks[2] + ks * 16 + hh * 8);
        vf[ks] = *reinterpret_cast<const bf16x8*>(V + static_cast<int64_t>(row) * p.vs[2] + ks * 16 + hh * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          kf[ks][i] = static_cast<bf16_t>(0.f);
          vf[ks][i] = static_cast<bf16_t>(0.f);
        }
      }
    }
  }
  // ---- query-tile range -------------------------------------------------------------------
  const int nqt = (p.Sq + BQ - 1) / BQ;
  int qt_begin = 0;
  if (MODE == MLTS_MASK_CAUSAL) {
    const int first_q = kv0 - p.causal_off;  // first query that sees key kv0
    qt_begin = first_q <= 0 ? 0 : first_q / BQ;
  }
  const int span = qt_begin < nqt ? nqt - qt_begin : 0;
  const int total_it = span * group;

  int4 kstats[2];
  if (MODE == MLTS_MASK_DOC) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int t = (kv0 >> 6) + i;
      kstats[i] = t < p.nk_stats ? p.k_stats[static_cast<int64_t>(b) * p.nk_stats + t] : make_int4(0x7fffffff, 0, 0, -2);
    }
  }
  const int4 wk_stats = MODE == MLTS_MASK_DOC ? ((wave >> 1) ? kstats[1] : kstats[0]) : make_int4(0, 0, 0, 0);
  int kpos = 0, kseq = -2;
  if (MODE == MLTS_MASK_DOC) {
    const int kj = wkv0 + l32;
    if (kj < p.Sk) {
      kpos = p.k_pos[static_cast<int64_t>(b) * p.Sk + kj];
      kseq = p.k_seq[static_cast<int64_t>(b) * p.Sk + kj];
    }
  }

  auto block_needs = [&](int it) -> bool {
    if (MODE != MLTS_MASK_DOC) return true;
    const int qt = qt_begin + it % span;
    const int4 qs4 = p.q_stats[static_cast<int64_t>(b) * p.nq_stats + qt];
    return classify_doc_tile(qs4, kstats[0]) != TILE_SKIP || classify_doc_tile(qs4, kstats[1]) != TILE_SKIP;
  };
  auto next_it = [&](int it) -> int {
    while (it < total_it && !block_needs(it)) ++it;
    return it;
  };

  // ---- staging ----------------------------------------------------------------------------
  uint32_t qreg[4][VW], doreg[4][VW];
  float stat_reg = 0.f;  // lanes 0..63: lse, 64..127: delta
  const int s_grp = tid >> 4, s_d0 = (tid & 15) * VEC;

  auto gload = [&](int it) {
    const int hq = hkv * group + it / span;
    const int q0 = (qt_begin + it % span) * BQ;
    const bf16_t* Q = static_cast<const bf16_t*>(p.q) + b * p.qs[0] + hq * p.qs[1];
    const bf16_t* dO = static_cast<const bf16_t*>(bp.dout) + b * bp.dos[0] + hq * bp.dos[1];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = q0 + s_grp * 4 + i;
      if (r < p.Sq) {
        const uint32_t* qsrc = reinterpret_cast<const uint32_t*>(Q + static_cast<int64_t>(r) * p.qs[2] + s_d0);
        const uint32_t* dsrc = reinterpret_cast<const uint32_t*>(dO + static_cast<int64_t>(r) * bp.dos[2] + s_d0);
        if (VW == 4) {
          const u32x4 a = *reinterpret_cast<const u32x4*>(qsrc);
          const u32x4 c = *reinterpret_cast<const u32x4*>(dsrc);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            qreg[i][e] = a[e];
            doreg[i][e] = c[e];
          }
        } else {
          const u32x2 a = *reinterpret_cast<const u32x2*>(qsrc);
          const u32x2 c = *reinterpret_cast<const u32x2*>(dsrc);
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            qreg[i][e] = a[e];
            doreg[i][e] = c[e];
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < VW; ++e) {
          qreg[i][e] = 0u;
          doreg[i][e] = 0u;
        }
      }
    }
    if (tid < 2 * BQ) {
      const int r = q0 + (tid & (BQ - 1));
      const int64_t off = (static_cast<int64_t>(b) * p.Hq + hq) * p.Sq + r;
      if (tid < BQ) {
        // stored as lse * log2(e); +inf for rows that saw no key (or lie beyond Sq) makes exp2(s - lse2) = 0
        const float l = r < p.Sq ? p.lse[off] : -INFINITY;
        stat_reg = l == -INFINITY ? INFINITY : l * kLog2e;
      } else {
        stat_reg = r < p.Sq ? bp.delta[off] : 0.f;
      }
    }
  };

  auto lds_store = [&](int stage) {
    bf16_t* base = smem + stage * L::STAGE;
    bf16_t* sQ = base + L::OFF_Q;
    bf16_t* sdO = base + L::OFF_DO;
    uint16_t* sQt = reinterpret_cast<uint16_t*>(base + L::OFF_QT);
    uint16_t* sdOt = reinterpret_cast<uint16_t*>(base + L::OFF_DOT);
    float* sLse = reinterpret_cast<float*>(base + L::OFF_STAT);
    float* sDelta = sLse + BQ;
    const int slot0 = t_slot(s_grp * 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = s_grp * 4 + i;
      uint32_t* dq_ = reinterpret_cast<uint32_t*>(sQ + r * L::RSTR + s_d0);
      uint32_t* dd_ = reinterpret_cast<uint32_t*>(sdO + r * L::RSTR + s_d0);
      if (VW == 4) {
        u32x4 a, c;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[e] = qreg[i][e];
          c[e] = doreg[i][e];
        }
        *reinterpret_cast<u32x4*>(dq_) = a;
        *reinterpret_cast<u32x4*>(dd_) = c;
      } else {
        u32x2 a, c;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          a[e] = qreg[i][e];
          c[e] = doreg[i][e];
        }
        *reinterpret_cast<u32x2*>(dq_) = a;
        *reinterpret_cast<u32x2*>(dd_) = c;
      }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const int d = s_d0 + e;
      const int chunk = (slot0 >> 3) ^ t_swz(d);
      const int sh = (e & 1) * 16;
      const int w = e >> 1;
      u32x2 a, c;
      a[0] = ((qreg[0][w] >> sh) & 0xffffu) | (((qreg[1][w] >> sh) & 0xffffu) << 16);
      a[1] = ((qreg[2][w] >> sh) & 0xffffu) | (((qreg[3][w] >> sh) & 0xffffu) << 16);
      c[0] = ((doreg[0][w] >> sh) & 0xffffu) | (((doreg[1][w] >> sh) & 0xffffu) << 16);
      c[1] = ((doreg[2][w] >> sh) & 0xffffu) | (((doreg[3][w] >> sh) & 0xffffu) << 16);
      *reinterpret_cast<u32x2*>(sQt + d * BQ + (chunk << 3) + (slot0 & 7)) = a;
      *reinterpret_cast<u32x2*>(sdOt + d * BQ + (chunk << 3) + (slot0 & 7)) = c;
    }
    if (tid < BQ) sLse[tid] = stat_reg;
    else if (tid < 2 * BQ) sDelta[tid - BQ] = stat_reg;
  };

  // ---- accumulators -----------------------------------------------------------------------
  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      dkacc[db][e] = 0.f;
      dvacc[db][e] = 0.f;
    }

  int it = next_it(0);
  if (it < total_it) gload(it);
  int stage = 0;
  while (it < total_it) {
    const int qt = qt_begin + it % span;
    const int q0 = qt * BQ;
    lds_store(stage);
    __syncthreads();
    const bf16_t* base = smem + stage * L::STAGE;
    const bf16_t* sQ = base + L::OFF_Q;
    const bf16_t* sdO = base + L::OFF_DO;
    const uint16_t* sQt = reinterpret_cast<const uint16_t*>(base + L::OFF_QT);
    const uint16_t* sdOt = reinterpret_cast<const uint16_t*>(base + L::OFF_DOT);
    const float* sLse = reinterpret_cast<const float*>(base + L::OFF_STAT);
    const float* sDelta = sLse + BQ;
    const int itn = next_it(it + 1);
    if (itn < total_it) gload(itn);

    int cls = TILE_FULL;
    if (MODE == MLTS_MASK_CAUSAL) {
      const int last_q = min(q0 + BQ, p.Sq) - 1;
      if (wkv0 > last_q + p.causal_off) cls = TILE_SKIP;
      else if (wkv0 + 31 > q0 + p.causal_off) cls = TILE_MASKED;
    } else if (MODE == MLTS_MASK_DOC) {
      cls = classify_doc_tile(p.q_stats[static_cast<int64_t>(b) * p.nq_stats + qt], wk_stats);
    }
    if (cls == TILE_FULL && (wkv0 + 32 > p.Sk || q0 + BQ > p.Sq)) cls = TILE_MASKED;
    if (wkv0 >= p.Sk) cls = TILE_SKIP;

    if (cls != TILE_SKIP) {
      // P and dS in registers; lane = key (wkv0 + l32), register e <-> query 32 qb + 8 (e/4) + 4 hh + e%4
      bf16x8 pfr[2][2], dsfr[2][2];
      const int kj = wkv0 + l32;
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        f32x16 sacc, dpacc;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          sacc[e] = 0.f;
          dpacc[e] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 qa = *reinterpret_cast<const bf16x8*>(sQ + (qb * 32 + l32) * L::RSTR + ks * 16 + hh * 8);
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[ks], sacc, 0, 0, 0);
          const bf16x8 da = *reinterpret_cast<const bf16x8*>(sdO + (qb * 32 + l32) * L::RSTR + ks * 16 + hh * 8);
          dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da, vf[ks], dpacc, 0, 0, 0);
        }
        auto softmax_bwd = [&](auto masked_tag) {
          constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int qrow = qb * 32 + g * 8 + hh * 4;
            const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sLse + qrow);  // already lse * log2(e)
            const f32x4 dl4 = *reinterpret_cast<const f32x4*>(sDelta + qrow);
            int qp4[4], qs4[4];
            if (MASKED && MODE == MLTS_MASK_DOC) {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int qi = q0 + qrow + r;
                const bool ok = qi < p.Sq;
                qp4[r] = ok ? p.q_pos[static_cast<int64_t>(b) * p.Sq + qi] : -0x7fffffff;
                qs4[r] = ok ? p.q_seq[static_cast<int64_t>(b) * p.Sq + qi] : -1;
              }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int e = g * 4 + r;
              float pv = __builtin_amdgcn_exp2f(sacc[e] * p.scale_log2 - lse4[r]);
              if (MASKED) {
                const int qi = q0 + qrow + r;
                bool vis = kj < p.Sk && qi < p.Sq;
                if (MODE == MLTS_MASK_CAUSAL) vis = vis && (kj <= qi + p.causal_off);
                if (MODE == MLTS_MASK_DOC) vis = vis && (kpos <= qp4[r]) && (kseq == qs4[r]) && (qs4[r] >= 0);
                if (!vis) pv = 0.f;
              }
              const float dsv = pv * (dpacc[e] - dl4[r]);
              pfr[qb][e >> 3][e & 7] = static_cast<bf16_t>(pv);
              dsfr[qb][e >> 3][e & 7] = static_cast<bf16_t>(dsv);
            }
          }
        };
        if (cls == TILE_MASKED) softmax_bwd(std::true_type{});
        else softmax_bwd(std::false_type{});
      }

      // dV += P^T dO, dK += dS^T Q
#pragma unroll
      for (int c = 0; c < 4; ++c) {  // c = qb * 2 + t: 16 queries per k-step
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int d = db * 32 + l32;
          const int chunk = (c * 2 + hh) ^ t_swz(d);
          const bf16x8 dob = *reinterpret_cast<const bf16x8*>(sdOt + d * BQ + (chunk << 3));
          dvacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pfr[c >> 1][c & 1], dob, dvacc[db], 0, 0, 0);
          const bf16x8 qb_ = *reinterpret_cast<const bf16x8*>(sQt + d * BQ + (chunk << 3));
          dkacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsfr[c >> 1][c & 1], qb_, dkacc[db], 0, 0, 0);
        }
      }
    }
    it = itn;
    stage ^= 1;
  }

  // ---- write dK, dV: register e <-> key wkv0 + 8 (e/4) + 4 hh + e%4, lane -> head-dim column ----
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    const int d = db * 32 + l32;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int row = wkv0 + (e >> 2) * 8 + hh * 4 + (e & 3);
      if (row < p.Sk) {
        const int64_t ok = b * bp.dks[0] + hkv * bp.dks[1] + static_cast<int64_t>(row) * bp.dks[2] + d;
        const int64_t ov = b * bp.dvs[0] + hkv * bp.dvs[1] + static_cast<int64_t>(row) * bp.dvs[2] + d;
        if (bp.accumulate_f32) {
          static_cast<float*>(bp.dk)[ok] += dkacc[db][e] * p.scale;
          static_cast<float*>(bp.dv)[ov] += dvacc[db][e];
        } else {
          static_cast<bf16_t*>(bp.dk)[ok] = static_cast<bf16_t>(dkacc[db][e] * p.scale);
          static_cast<bf16_t*>(bp.dv)[ov] = static_cast<bf16_t>(dvacc[db][e]);
        }
      }
    }
  }
}

template <int D, int MODE>
int launch_bwd(const AttnBwdParams& bp, hipStream_t st) {
  auto kern = attn_bwd_kernel<D, MODE>;
  constexpr int smem = BwdLds<D>::BYTES;
  static bool configured = false;
  if (!configured && smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) {
      mlts_set_error("mlts_attn_bwd: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
      return MLTS_ERR_LAUNCH;
    }
    configured = true;
  }
  const int64_t blocks = static_cast<int64_t>(bp.nkt) * bp.a.B * bp.a.Hkv;
  if (blocks > 0) {
    MltsKernelTimer timer("attn_bwd_dkdv", st);
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(THREADS), smem, st, bp);
  }
  return mlts_check_launch("mlts_attn_bwd");
}

}  // namespace

int mlts_attn_bwd_dq_bf16(const AttnBwdParams& bp, int D, int mode, hipStream_t st);

int64_t mlts_attn_bwd_dkdv_split_workspace(int64_t B, int64_t Hq, int64_t Sq);                           // attn_bwd_split.hip

int mlts_attn_bwd_dkdv_bf16_split(AttnBwdParams bp, int D, int mode, void* workspace, hipStream_t st);  // attn_bwd_split.hip
int mlts_attn_bwd_dq_bf16_tr(const AttnBwdParams& bp, int D, int mode, hipStream_t st);                    // attn_bwd_dq_tr.hip
int64_t mlts_attn_bwd_ds_bytes(int64_t B, int64_t Hq, int64_t Sq, int64_t Sk);                              // attn_bwd_dq_ds.hip
int mlts_attn_bwd_dq_bf16_ds(const AttnBwdParams& bp, int D, int mode, hipStream_t st);                    // attn_bwd_dq_ds.hip

namespace {
// Two-role dK/dV kernel and transpose-read dQ kernel by default; tuning aid MLTS_BWD_VARIANT=staged selects the
// register-staged kernels of this file and attn_bwd_dq.hip (also the fallback for very large row strides).
bool use_staged_bwd() {
  static const bool staged = [] {
    const char* e = getenv("MLTS_BWD_VARIANT");
    return e && e[0] == 's';
  }();
  return staged;
}
}  // namespace

// The dK/dV kernel can hand -dS (bf16, 2 bytes per (query, key) pair of the score matrix) over to a dQ kernel that
// then does one matrix product instead of recomputing the scores (three).  Used without a document mask when the
// hand-over fits the budget: MLTS_BWD_DS_MAX_MB megabytes (default 4096; 0 turns it off).
static int64_t ds_handover_bytes(int B, int Hq, int Sq, int Sk, int D, int mode, int accumulate_f32) {
  static const int64_t max_bytes = [] {
    const char* e = getenv("MLTS_BWD_DS_MAX_MB");
    return (e ? static_cast<int64_t>(atoll(e)) : int64_t{4096}) << 20;
  }();
  // head_dim 64 has half the matrix work per pair and the same hand-over bytes: recomputing is faster there.  Block
  // gradients that are accumulated in fp32 (ring steps) keep the recomputed, once-rounded dS.
  if (use_staged_bwd() || mode == MLTS_MASK_DOC || D != 128 || accumulate_f32 || Sq == 0 || Sk == 0) return 0;
  const int64_t n = mlts_attn_bwd_ds_bytes(B, Hq, Sq, Sk);
  return n <= max_bytes ? n : 0;
}

int64_t mlts_attn_bwd_bf16_workspace(const mlts_attn_shape* s, int accumulate_f32) {
  // lse2 (B*Hq*Sq + 1 floats), then the -dS hand-over
  return mlts_attn_bwd_dkdv_split_workspace(s->B, s->Hq, s->Sq) + ds_handover_bytes(s->B, s->Hq, s->Sq, s->Sk, s->D, s->mask_mode, accumulate_f32);
}

int mlts_attn_bwd_bf16(AttnBwdParams bp, int D, int mode, void* workspace, hipStream_t st) {
  const AttnParams& p = bp.a;
  bp.nkt = (p.Sk + BKV - 1) / BKV;
  int rc;
  // the newer kernels address rows of a tile with 32-bit element offsets
  const int64_t lim = int64_t{1} << 24;
  const bool staged = use_staged_bwd() || p.qs[2] >= lim || p.ks[2] >= lim || p.vs[2] >= lim || bp.dos[2] >= lim;
  const int64_t ds_bytes = staged ? 0 : ds_handover_bytes(p.B, p.Hq, p.Sq, p.Sk, D, mode, bp.accumulate_f32);
  if (ds_bytes > 0) {
    bp.ds_ws = static_cast<char*>(workspace) + mlts_attn_bwd_dkdv_split_workspace(p.B, p.Hq, p.Sq);
    bp.ds_nkb = (p.Sk + 31) / 32;
    bp.ds_nqt = (p.Sq + 63) / 64;
  }
  if (!staged) {
    rc = mlts_attn_bwd_dkdv_bf16_split(bp, D, mode, workspace, st);
  } else if (D == 128) {
    if (mode == MLTS_MASK_NONE) rc = launch_bwd<128, MLTS_MASK_NONE>(bp, st);
    else if (mode == MLTS_MASK_CAUSAL) rc = launch_bwd<128, MLTS_MASK_CAUSAL>(bp, st);
    else rc = launch_bwd<128, MLTS_MASK_DOC>(bp, st);
  } else {
    if (mode == MLTS_MASK_NONE) rc = launch_bwd<64, MLTS_MASK_NONE>(bp, st);
    else if (mode == MLTS_MASK_CAUSAL) rc = launch_bwd<64, MLTS_MASK_CAUSAL>(bp, st);
    else rc = launch_bwd<64, MLTS_MASK_DOC>(bp, st);
  }
  if (rc != MLTS_OK) return rc;
  if (ds_bytes > 0) return mlts_attn_bwd_dq_bf16_ds(bp, D, mode, st);
  if (!staged) return mlts_attn_bwd_dq_bf16_tr(bp, D, mode, st);
  return mlts_attn_bwd_dq_bf16(bp, D, mode, st);
}
