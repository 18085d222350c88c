// Attention backward for gfx950 (bf16, head_dim 64/128), part 2 of 2: dQ.
//
// Query-stationary, shaped like the forward kernel: a workgroup of 8 wavefronts owns 256 query rows of
// one (batch, head), each wavefront 32 of them, and walks the visible keys in tiles of 64.  Scores are
// recomputed TRANSPOSED so that a lane owns one query (LSE and delta are per-lane scalars):
//     S^T  = K Q^T        A = K  (LDS, row major)   B = Q  (registers, loaded once)
//     dP^T = V dO^T       A = V  (LDS, row major)   B = dO (registers, loaded once)
//     P = exp2(S c - LSE), dS = P (dP - delta)       registers; layout = B operand of the next product
//     dQ^T += K^T dS^T    A = K^T (LDS, transposed while staging, swizzled)   B = dS^T (registers)
// dQ rows belong to exactly one workgroup: plain stores (or fp32 read-add-write in accumulate mode),
// no atomics.  Two wavefronts per SIMD (<= 256 registers) let the hardware overlap one wavefront's
// exp2/VALU work with the other's MFMAs.
#include "attn_common.hpp"
#include <type_traits>

namespace {

constexpr int BN = 64;
constexpr int WAVES = 8;
constexpr int THREADS = WAVES * 64;
constexpr int BM = WAVES * 32;

template <int D>
struct DqLds {
  static constexpr int RSTR = D + 8;
  static constexpr int ROW_ELEMS = BN * RSTR;
  static constexpr int T_ELEMS = D * BN;
  static constexpr int OFF_K = 0;
  static constexpr int OFF_V = ROW_ELEMS;
  static constexpr int OFF_KT = 2 * ROW_ELEMS;
  static constexpr int STAGE = 2 * ROW_ELEMS + T_ELEMS;
  static constexpr int BYTES = 2 * STAGE * 2;
};

__device__ __forceinline__ int q_swz(int d) { return ((d >> 1) ^ (d >> 4)) & 7; }
__device__ __forceinline__ int q_slot(int r) {
  const int kb = r >> 5, t = (r >> 4) & 1, grp = (r >> 2) & 3;
  return (((kb * 2 + t) * 2 + (grp & 1)) << 3) + ((grp >> 1) << 2) + (r & 3);
}

template <int D, int MODE>
__global__ __launch_bounds__(THREADS) void attn_bwd_dq_kernel(const AttnBwdParams bp) {
  const AttnParams& p = bp.a;
  using L = DqLds<D>;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int KLD = D / 32;   // 16-byte vectors per thread for the row-major V tile (256 staging threads)
  constexpr int TPR = D / 8;
  constexpr int VEC = D / 16;   // K elements per thread per row (4 rows per thread, 256 staging threads)
  constexpr int VW = VEC / 2;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* smem = reinterpret_cast<bf16_t*>(smem_raw);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const int nbh = p.B * p.Hq;
  const int bid = blockIdx.x;
  const int qt = p.nqt - 1 - bid / nbh;
  const int bh = bid % nbh;
  const int b = bh / p.Hq, hq = bh % p.Hq;
  const int hkv = hq / (p.Hq / p.Hkv);
  const int q0 = qt * BM;
  const int wq0 = q0 + wave * 32;
  const int qrow = wq0 + l32;

  const bf16_t* Q = static_cast<const bf16_t*>(p.q) + b * p.qs[0] + hq * p.qs[1];
  const bf16_t* dO = static_cast<const bf16_t*>(bp.dout) + b * bp.dos[0] + hq * bp.dos[1];
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + b * p.vs[0] + hkv * p.vs[1];

  bf16x8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (qrow < p.Sq) {
      qf[ks] = *reinterpret_cast<const bf16x8*>(Q + static_cast<int64_t>(qrow) * p.qs[2] + ks * 16 + hh * 8);
      dof[ks] = *reinterpret_cast<const bf16x8*>(dO + static_cast<int64_t>(qrow) * bp.dos[2] + ks * 16 + hh * 8);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        qf[ks][i] = static_cast<bf16_t>(0.f);
        dof[ks][i] = static_cast<bf16_t>(0.f);
      }
    }
  }
  float lse2 = INFINITY, delta = 0.f;  // +inf makes exp2(s - lse2) = 0 for rows that saw no key
  if (qrow < p.Sq) {
    const int64_t off = (static_cast<int64_t>(b) * p.Hq + hq) * p.Sq + qrow;
    const float l = p.lse[off];
    lse2 = l == -INFINITY ? INFINITY : l * kLog2e;
    delta = bp.delta[off];
  }
  int qpos = 0, qseq = -1;
  int4 wq_stats = make_int4(0, -1, 0, -1);
  int4 bq_stats[BM / 64];
  if (MODE == MLTS_MASK_DOC) {
    if (qrow < p.Sq) {
      qpos = p.q_pos[static_cast<int64_t>(b) * p.Sq + qrow];
      qseq = p.q_seq[static_cast<int64_t>(b) * p.Sq + qrow];
    }
#pragma unroll
    for (int w = 0; w < BM / 64; ++w) {
      const int t = (q0 >> 6) + w;
      bq_stats[w] = t < p.nq_stats ? p.q_stats[static_cast<int64_t>(b) * p.nq_stats + t] : make_int4(0, -1, 0, -1);
    }
    const int t = wq0 >> 6;
    if (t < p.nq_stats) wq_stats = p.q_stats[static_cast<int64_t>(b) * p.nq_stats + t];
  }

  const int nkt = (p.Sk + BN - 1) / BN;
  int j_end = nkt;
  if (MODE == MLTS_MASK_CAUSAL) {
    const int lim = min(q0 + BM, p.Sq) - 1 + p.causal_off;
    j_end = lim < 0 ? 0 : min(nkt, lim / BN + 1);
  }
  const int wave_last_q = min(wq0 + 31, p.Sq - 1);

  auto block_needs = [&](int j) -> bool {
    if (MODE != MLTS_MASK_DOC) return true;
    const int4 ks4 = p.k_stats[static_cast<int64_t>(b) * p.nk_stats + j];
    bool need = false;
#pragma unroll
    for (int w = 0; w < BM / 64; ++w) need |= classify_doc_tile(bq_stats[w], ks4) != TILE_SKIP;
    return need;
  };
  auto next_tile = [&](int j) -> int {
    while (j < j_end && !block_needs(j)) ++j;
    return j;
  };

  // staging: threads 0..255 load K (4 rows x VEC columns each, written row major AND transposed),
  // threads 256..511 load V (row major)
  const int stid = tid & 255;
  const bool do_k = tid < 256;
  const int s_grp = stid >> 4, s_d0 = (stid & 15) * VEC;
  const int v_row0 = stid / TPR, v_col = (stid % TPR) * 8;
  uint32_t st[D / 8];  // one staging buffer for both roles: K rows [4][VW] words, or V vectors [KLD][4] words

  auto gload = [&](int j) {
    const int kv0 = j * BN;
    if (do_k) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = kv0 + s_grp * 4 + i;
        if (r < p.Sk) {
          const uint32_t* src = reinterpret_cast<const uint32_t*>(K + static_cast<int64_t>(r) * p.ks[2] + s_d0);
          if (VW == 4) {
            const u32x4 a = *reinterpret_cast<const u32x4*>(src);
#pragma unroll
            for (int e = 0; e < 4; ++e) st[i * VW + e] = a[e];
          } else {
            const u32x2 a = *reinterpret_cast<const u32x2*>(src);
#pragma unroll
            for (int e = 0; e < 2; ++e) st[i * VW + e] = a[e];
          }
        } else {
#pragma unroll
          for (int e = 0; e < VW; ++e) st[i * VW + e] = 0u;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < KLD; ++i) {
        const int r = kv0 + v_row0 + i * (256 / TPR);
        u32x4 a = {0u, 0u, 0u, 0u};
        if (r < p.Sk) a = *reinterpret_cast<const u32x4*>(V + static_cast<int64_t>(r) * p.vs[2] + v_col);
#pragma unroll
        for (int e = 0; e < 4; ++e) st[i * 4 + e] = a[e];
      }
    }
  };

  auto lds_store = [&](int stage) {
    bf16_t* base = smem + stage * L::STAGE;
    if (do_k) {
      bf16_t* sK = base + L::OFF_K;
      uint16_t* sKt = reinterpret_cast<uint16_t*>(base + L::OFF_KT);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t* dst = reinterpret_cast<uint32_t*>(sK + (s_grp * 4 + i) * L::RSTR + s_d0);
        if (VW == 4) {
          u32x4 a;
#pragma unroll
          for (int e = 0; e < 4; ++e) a[e] = st[i * VW + e];
          *reinterpret_cast<u32x4*>(dst) = a;
        } else {
          u32x2 a;
#pragma unroll
          for (int e = 0; e < 2; ++e) a[e] = st[i * VW + e];
          *reinterpret_cast<u32x2*>(dst) = a;
        }
      }
      const int slot0 = q_slot(s_grp * 4);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const int d = s_d0 + e;
        const int chunk = (slot0 >> 3) ^ q_swz(d);
        const int sh = (e & 1) * 16, w = e >> 1;
        u32x2 a;
        a[0] = ((st[0 * VW + w] >> sh) & 0xffffu) | (((st[1 * VW + w] >> sh) & 0xffffu) << 16);
        a[1] = ((st[2 * VW + w] >> sh) & 0xffffu) | (((st[3 * VW + w] >> sh) & 0xffffu) << 16);
        *reinterpret_cast<u32x2*>(sKt + d * BN + (chunk << 3) + (slot0 & 7)) = a;
      }
    } else {
      bf16_t* sV = base + L::OFF_V;
#pragma unroll
      for (int i = 0; i < KLD; ++i) {
        const int r = v_row0 + i * (256 / TPR);
        u32x4 a;
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] = st[i * 4 + e];
        *reinterpret_cast<u32x4*>(sV + r * L::RSTR + v_col) = a;
      }
    }
  };

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) dqacc[db][e] = 0.f;

  int j = next_tile(0);
  if (j < j_end) gload(j);
  int stage = 0;
  while (j < j_end) {
    lds_store(stage);
    __syncthreads();
    const int jn = next_tile(j + 1);
    if (jn < j_end) gload(jn);

    const int kv0 = j * BN;
    int cls = TILE_FULL;
    if (MODE == MLTS_MASK_CAUSAL) {
      if (kv0 > wave_last_q + p.causal_off) cls = TILE_SKIP;
      else if (kv0 + BN - 1 > wq0 + p.causal_off) cls = TILE_MASKED;
    } else if (MODE == MLTS_MASK_DOC) {
      cls = classify_doc_tile(wq_stats, p.k_stats[static_cast<int64_t>(b) * p.nk_stats + j]);
    }
    if (cls == TILE_FULL && kv0 + BN > p.Sk) cls = TILE_MASKED;
    if (wq0 >= p.Sq) cls = TILE_SKIP;

    if (cls != TILE_SKIP) {
      const bf16_t* base = smem + stage * L::STAGE;
      const bf16_t* sK = base + L::OFF_K;
      const bf16_t* sV = base + L::OFF_V;
      const bf16_t* sKt = base + L::OFF_KT;
      bf16x8 dsf[4];
      // one 32-key block at a time keeps only one S and one dP accumulator live
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        f32x16 sacc, dpacc;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          sacc[e] = 0.f;
          dpacc[e] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 ka = *reinterpret_cast<const bf16x8*>(sK + (kb * 32 + l32) * L::RSTR + ks * 16 + hh * 8);
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[ks], sacc, 0, 0, 0);
          const bf16x8 va = *reinterpret_cast<const bf16x8*>(sV + (kb * 32 + l32) * L::RSTR + ks * 16 + hh * 8);
          dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, dof[ks], dpacc, 0, 0, 0);
        }
        auto softmax_bwd = [&](auto masked_tag) {
          constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int kbase = kv0 + kb * 32 + g * 8 + hh * 4;
            int kp[4], ksq[4];
            if (MASKED && MODE == MLTS_MASK_DOC) {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int kj = kbase + r;
                const bool ok = kj < p.Sk;
                kp[r] = ok ? p.k_pos[static_cast<int64_t>(b) * p.Sk + kj] : 0x7fffffff;
                ksq[r] = ok ? p.k_seq[static_cast<int64_t>(b) * p.Sk + kj] : -2;
              }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int e = g * 4 + r;
              float pv = __builtin_amdgcn_exp2f(sacc[e] * p.scale_log2 - lse2);
              if (MASKED) {
                const int kj = kbase + r;
                bool vis = kj < p.Sk;
                if (MODE == MLTS_MASK_CAUSAL) vis = vis && (kj <= qrow + p.causal_off);
                if (MODE == MLTS_MASK_DOC) vis = vis && (kp[r] <= qpos) && (ksq[r] == qseq) && (qseq >= 0);
                if (!vis) pv = 0.f;
              }
              dsf[kb * 2 + (e >> 3)][e & 7] = static_cast<bf16_t>(pv * (dpacc[e] - delta));
            }
          }
        };
        if (cls == TILE_MASKED) softmax_bwd(std::true_type{});
        else softmax_bwd(std::false_type{});
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int d = db * 32 + l32;
          const int chunk = (c * 2 + hh) ^ q_swz(d);
          const bf16x8 kt = *reinterpret_cast<const bf16x8*>(sKt + d * BN + (chunk << 3));
          dqacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kt, dsf[c], dqacc[db], 0, 0, 0);
        }
      }
    }
    j = jn;
    stage ^= 1;
  }

  // dQ^T accumulator: register e <-> head-dim 32 db + 8 (e/4) + 4 hh + e%4, lane -> query row
  if (qrow < p.Sq) {
    const int64_t rowoff = b * bp.dqs[0] + hq * bp.dqs[1] + static_cast<int64_t>(qrow) * bp.dqs[2];
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = db * 32 + g * 8 + hh * 4;
        if (bp.accumulate_f32) {
          f32x4* dst = reinterpret_cast<f32x4*>(bp.dq_acc + rowoff + d);
          f32x4 cur = *dst;
#pragma unroll
          for (int r = 0; r < 4; ++r) cur[r] += dqacc[db][g * 4 + r] * p.scale;
          *dst = cur;
        } else {
          bf16x4 w;
#pragma unroll
          for (int r = 0; r < 4; ++r) w[r] = static_cast<bf16_t>(dqacc[db][g * 4 + r] * p.scale);
          *reinterpret_cast<bf16x4*>(reinterpret_cast<bf16_t*>(bp.dq_acc) + rowoff + d) = w;
        }
      }
    }
  }
}

template <int D, int MODE>
int launch_dq(AttnBwdParams bp, hipStream_t st) {
  auto kern = attn_bwd_dq_kernel<D, MODE>;
  constexpr int smem = DqLds<D>::BYTES;
  static bool configured = false;
  if (!configured && smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) {
      mlts_set_error("mlts_attn_bwd: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
      return MLTS_ERR_LAUNCH;
    }
    configured = true;
  }
  bp.a.nqt = (bp.a.Sq + BM - 1) / BM;
  const int64_t blocks = static_cast<int64_t>(bp.a.nqt) * bp.a.B * bp.a.Hq;
  if (blocks > 0) {
    MltsKernelTimer timer("attn_bwd_dq", st);
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(THREADS), smem, st, bp);
  }
  return mlts_check_launch("mlts_attn_bwd");
}

}  // namespace

int mlts_attn_bwd_dq_bf16(const AttnBwdParams& bp, int D, int mode, hipStream_t st) {
  if (D == 128) {
    if (mode == MLTS_MASK_NONE) return launch_dq<128, MLTS_MASK_NONE>(bp, st);
    if (mode == MLTS_MASK_CAUSAL) return launch_dq<128, MLTS_MASK_CAUSAL>(bp, st);
    return launch_dq<128, MLTS_MASK_DOC>(bp, st);
  }
  if (mode == MLTS_MASK_NONE) return launch_dq<64, MLTS_MASK_NONE>(bp, st);
  if (mode == MLTS_MASK_CAUSAL) return launch_dq<64, MLTS_MASK_CAUSAL>(bp, st);
  return launch_dq<64, MLTS_MASK_DOC>(bp, st);
}
