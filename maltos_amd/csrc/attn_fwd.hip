// Attention forward for gfx950: O = softmax(scale * Q K^T + mask) V and LSE, bf16 in, fp32 accumulate.
//
// Work decomposition (one workgroup = 4 wavefronts = 256 query rows of one (batch, head)):
//   * every wavefront owns 64 query rows as two 32-row MFMA column blocks and walks the keys in
//     tiles of 64; K and V tiles are staged once per workgroup in LDS (double buffered) and each
//     LDS fragment read feeds two MFMAs (one per query block), which keeps LDS traffic at half of
//     what the matrix pipe could consume;
//   * scores are produced TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16: a lane then holds
//     32 scores of ONE query, so the online-softmax row max / row sum are in-lane reductions plus a
//     single exchange with lane^32, and the rescale factor of O^T is a per-lane scalar;
//   * the S^T accumulator layout is, register for register, the B-operand layout of the second
//     product O^T = V^T P^T, so P never leaves registers; V is transposed on its way into LDS
//     (4x8 register transposes, 8-byte LDS writes, XOR-swizzled 16-byte chunks) so that V^T
//     fragments are single conflict-free ds_read_b128.
//   * masks: causal tiles above the diagonal are never visited; document masks use per-tile
//     (min/max position, min/max sequence id) statistics to skip or fast-path whole tiles and fall
//     back to the element predicate only on tiles that straddle a boundary.
#include "attn_common.hpp"
#include <stdlib.h>

namespace {

constexpr int BN = 64;          // keys per tile

template <int D>
struct FwdLds {
  static constexpr int KSTR = D + 8;         // K row stride in elements (16-byte pad: conflict-free b128 reads)
  static constexpr int K_ELEMS = BN * KSTR;
  static constexpr int V_ELEMS = D * BN;     // Vt[d][slot], 128-byte rows, swizzled chunks
  static constexpr int STAGE = K_ELEMS + V_ELEMS;
  static constexpr int BYTES = 2 * STAGE * 2;
};

// 16-byte chunk swizzle of a Vt row.  Chosen by measurement on gfx950: ds_read_b128 of 32 consecutive
// rows runs at the conflict-free rate (~225 B/clk/CU) with this function, while the look-alike
// (d >> 1) ^ (d >> 3) halves it; the 8-byte transposed staging writes (rows 8 apart) cost the same either way.
__device__ __forceinline__ int vt_swz(int d) { return ((d >> 1) ^ (d >> 4)) & 7; }

// slot of key row r (0..63) inside a Vt row: slot order is the order in which the S^T accumulator
// registers of a lane enumerate the keys, so a P fragment and a Vt fragment agree on k.
__device__ __forceinline__ int vt_slot(int r) {
  const int kb = r >> 5, t = (r >> 4) & 1, grp = (r >> 2) & 3;
  const int hh = grp & 1, ihi = grp >> 1;
  return (((kb * 2 + t) * 2 + hh) << 3) + (ihi << 2) + (r & 3);
}

// WAVES x QB: 4 x 2 (one wavefront per SIMD, 64 query rows each, up to 512 registers) or
// 8 x 1 (two wavefronts per SIMD, 32 query rows each, <= 256 registers: the hardware overlaps one
// wavefront's softmax VALU work with the other's MFMAs).  Both cover 256 query rows per workgroup.
template <int D, int MODE, int WAVES, int QB>
__global__ __launch_bounds__(WAVES * 64) void attn_fwd_kernel(const AttnParams p) {
  using L = FwdLds<D>;
  constexpr int THREADS = WAVES * 64;
  constexpr int BM = WAVES * QB * 32;
  constexpr int WROWS = QB * 32;     // query rows per wavefront
  constexpr int KS = D / 16;    // k-steps of the score product
  constexpr int DB = D / 32;    // 32-row blocks of O^T
  constexpr int KLD = D / 32;   // 16-byte K vectors staged per thread (256 staging threads)
  constexpr int TPR = D / 8;    // threads per K row
  constexpr int VEC = D / 16;   // V elements per thread per row (4 rows per thread, 256 staging threads)
  // with 8 wavefronts, threads 0..255 stage V (transposing) and threads 256..511 stage K
  constexpr bool SPLIT = WAVES == 8;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* smem = reinterpret_cast<bf16_t*>(smem_raw);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;

  const int nbh = p.B * p.Hq;
  const int bid = blockIdx.x;
  const int qt = p.nqt - 1 - bid / nbh;  // heaviest causal tiles are dispatched first
  const int bh = bid % nbh;
  const int b = bh / p.Hq, hq = bh % p.Hq;
  const int hkv = hq / (p.Hq / p.Hkv);
  const int q0 = qt * BM;
  const int wq0 = q0 + wave * WROWS;

  const bf16_t* Q = static_cast<const bf16_t*>(p.q) + b * p.qs[0] + hq * p.qs[1];
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + b * p.vs[0] + hkv * p.vs[1];
  bf16_t* O = static_cast<bf16_t*>(p.o) + b * p.os[0] + hq * p.os[1];

  // ---- Q fragments (B operand: column = query, k = head-dim slice) -----------------------
  bf16x8 qf[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int row = wq0 + qb * 32 + l32;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (row < p.Sq) {
        qf[qb][ks] = *reinterpret_cast<const bf16x8*>(Q + static_cast<int64_t>(row) * p.qs[2] + ks * 16 + hh * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[qb][ks][i] = static_cast<bf16_t>(0.f);
      }
    }
  }

  // per-lane query metadata for the document mask
  int qpos[QB], qseq[QB];
  int4 wq_stats = make_int4(0, -1, 0, -1);
  int4 bq_stats[BM / 64];
  if (MODE == MLTS_MASK_DOC) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int row = wq0 + qb * 32 + l32;
      const bool ok = row < p.Sq;
      qpos[qb] = ok ? p.q_pos[static_cast<int64_t>(b) * p.Sq + row] : 0;
      qseq[qb] = ok ? p.q_seq[static_cast<int64_t>(b) * p.Sq + row] : -1;
    }
#pragma unroll
    for (int w = 0; w < BM / 64; ++w) {
      const int t = (q0 >> 6) + w;
      bq_stats[w] = t < p.nq_stats ? p.q_stats[static_cast<int64_t>(b) * p.nq_stats + t] : make_int4(0, -1, 0, -1);
    }
    {
      const int t = wq0 >> 6;  // statistics are per 64 query rows; a 32-row wavefront uses its parent's
      if (t < p.nq_stats) wq_stats = p.q_stats[static_cast<int64_t>(b) * p.nq_stats + t];
    }
  }

  // ---- key-tile range -------------------------------------------------------------------
  const int nkt = (p.Sk + BN - 1) / BN;
  int j_end = nkt;
  if (MODE == MLTS_MASK_CAUSAL) {
    const int last_q = min(q0 + BM, p.Sq) - 1;
    const int lim = last_q + p.causal_off;  // last visible key index for the block
    j_end = lim < 0 ? 0 : min(nkt, lim / BN + 1);
  }
  const int wave_last_q = min(wq0 + WROWS - 1, p.Sq - 1);

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

  // ---- staging registers and helpers ------------------------------------------------------
  bf16x8 kreg[KLD];
  uint16_t vreg[4][VEC];
  const int stid = tid & 255;  // index among the 256 threads that share a staging role
  const bool do_k = !SPLIT || tid >= 256, do_v = !SPLIT || tid < 256;
  const int k_row0 = stid / TPR, k_col = (stid % TPR) * 8;
  const int v_grp = stid >> 4, v_d0 = (stid & 15) * VEC;

  auto gload = [&](int j) {
    const int kv0 = j * BN;
    if (do_k) {
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int r = kv0 + k_row0 + i * (256 / TPR);
      if (r < p.Sk) {
        kreg[i] = *reinterpret_cast<const bf16x8*>(K + static_cast<int64_t>(r) * p.ks[2] + k_col);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) kreg[i][e] = static_cast<bf16_t>(0.f);
      }
    }
    }
    if (do_v) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = kv0 + v_grp * 4 + i;
      if (r < p.Sk) {
        const uint16_t* src = reinterpret_cast<const uint16_t*>(V + static_cast<int64_t>(r) * p.vs[2] + v_d0);
        if (VEC == 8) {
          const u32x4 t = *reinterpret_cast<const u32x4*>(src);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            vreg[i][2 * e] = static_cast<uint16_t>(t[e] & 0xffffu);
            vreg[i][2 * e + 1] = static_cast<uint16_t>(t[e] >> 16);
          }
        } else {
          const u32x2 t = *reinterpret_cast<const u32x2*>(src);
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            vreg[i][2 * e] = static_cast<uint16_t>(t[e] & 0xffffu);
            vreg[i][2 * e + 1] = static_cast<uint16_t>(t[e] >> 16);
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) vreg[i][e] = 0;
      }
    }
    }
  };

  auto lds_store = [&](int stage) {
    bf16_t* sK = smem + stage * L::STAGE;
    uint16_t* sV = reinterpret_cast<uint16_t*>(smem + stage * L::STAGE + L::K_ELEMS);
    if (do_k) {
#pragma unroll
      for (int i = 0; i < KLD; ++i) {
        const int r = k_row0 + i * (256 / TPR);
        *reinterpret_cast<bf16x8*>(sK + r * L::KSTR + k_col) = kreg[i];
      }
    }
    const int slot0 = vt_slot(v_grp * 4);  // 4 consecutive rows -> 4 consecutive slots
    if (do_v)
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const int d = v_d0 + e;
      const int chunk = (slot0 >> 3) ^ vt_swz(d);
      u32x2 w;
      w[0] = static_cast<uint32_t>(vreg[0][e]) | (static_cast<uint32_t>(vreg[1][e]) << 16);
      w[1] = static_cast<uint32_t>(vreg[2][e]) | (static_cast<uint32_t>(vreg[3][e]) << 16);
      *reinterpret_cast<u32x2*>(sV + d * BN + (chunk << 3) + (slot0 & 7)) = w;
    }
  };

  // ---- running state ----------------------------------------------------------------------
  f32x16 oacc[QB][DB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) oacc[qb][db][e] = 0.f;
  float m_run[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
  }

  int j = next_tile(0);
  if (j < j_end) gload(j);
  int stage = 0;
  while (j < j_end) {
    lds_store(stage);
    __syncthreads();
    const int jn = next_tile(j + 1);
    if (jn < j_end) gload(jn);

    // ---- does this wavefront need the tile, and with which mask? ----
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
      const bf16_t* sK = smem + stage * L::STAGE;
      const bf16_t* sV = smem + stage * L::STAGE + L::K_ELEMS;

      // S^T[key][query] for two key blocks x two query blocks
      f32x16 sacc[QB][2];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 16; ++e) sacc[qb][kb][e] = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(sK + (kb * 32 + l32) * L::KSTR + ks * 16 + hh * 8);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
            sacc[qb][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][ks], sacc[qb][kb], 0, 0, 0);
        }
      }

      if (cls == TILE_MASKED) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int kbase = kv0 + kb * 32 + g * 8 + hh * 4;  // 4 consecutive keys
            int kp[4], ksq[4];
            if (MODE == MLTS_MASK_DOC) {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int kj = kbase + r;
                const bool ok = kj < p.Sk;
                kp[r] = ok ? p.k_pos[static_cast<int64_t>(b) * p.Sk + kj] : 0x7fffffff;
                ksq[r] = ok ? p.k_seq[static_cast<int64_t>(b) * p.Sk + kj] : -2;
              }
            }
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
              const int qi = wq0 + qb * 32 + l32;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int kj = kbase + r;
                bool vis = kj < p.Sk;
                if (MODE == MLTS_MASK_CAUSAL) vis = vis && (kj <= qi + p.causal_off);
                if (MODE == MLTS_MASK_DOC) vis = vis && (kp[r] <= qpos[qb]) && (ksq[r] == qseq[qb]) && (qseq[qb] >= 0);
                if (!vis) sacc[qb][kb][g * 4 + r] = -INFINITY;
              }
            }
          }
        }
      }

      // online softmax per query block; P packed to bf16 in the B-operand order of the PV product
      bf16x8 pf[QB][4];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        float mx = sacc[qb][0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sacc[qb][kb][e]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run[qb], mx * p.scale_log2);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - m_use);
        m_run[qb] = m_new;
        float ls = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
          for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              const float pv = __builtin_amdgcn_exp2f(sacc[qb][kb][t * 8 + i] * p.scale_log2 - m_use);
              ls += pv;
              pf[qb][kb * 2 + t][i] = static_cast<bf16_t>(pv);
            }
          }
        }
        l_run[qb] = l_run[qb] * alpha + ls;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int e = 0; e < 16; ++e) oacc[qb][db][e] *= alpha;
      }

      // O^T += V^T P^T
#pragma unroll
      for (int c = 0; c < 4; ++c) {  // c = kb * 2 + t: 16 keys per step
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int d = db * 32 + l32;
          const int chunk = (c * 2 + hh) ^ vt_swz(d);
          const bf16x8 vf = *reinterpret_cast<const bf16x8*>(sV + d * BN + (chunk << 3));
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
            oacc[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[qb][c], oacc[qb][db], 0, 0, 0);
        }
      }
    }
    j = jn;
    stage ^= 1;
  }

  // ---- epilogue: normalise, store O and LSE ------------------------------------------------
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int row = wq0 + qb * 32 + l32;
    const float l_tot = l_run[qb] + __shfl_xor(l_run[qb], 32, 64);
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    if (row < p.Sq) {
      if (hh == 0) {
        p.lse[(static_cast<int64_t>(b) * p.Hq + hq) * p.Sq + row] =
            l_tot > 0.f ? (m_run[qb] + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
      }
      bf16_t* orow = O + static_cast<int64_t>(row) * p.os[2];
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          bf16x4 w;
#pragma unroll
          for (int r = 0; r < 4; ++r) w[r] = static_cast<bf16_t>(oacc[qb][db][g * 4 + r] * inv);
          *reinterpret_cast<bf16x4*>(orow + db * 32 + g * 8 + hh * 4) = w;
        }
      }
    }
  }
}

// ---- tile statistics ------------------------------------------------------------------------
__global__ __launch_bounds__(64) void tile_stats_kernel(const int32_t* __restrict__ pos, const int32_t* __restrict__ seq,
                                                        int S, int ntiles, int4* __restrict__ out) {
  const int t = blockIdx.x % ntiles, b = blockIdx.x / ntiles;
  const int i = t * kAttnTile + threadIdx.x;
  int pmin = 0x7fffffff, pmax = -0x7fffffff - 1, smin = 0x7fffffff, smax = -0x7fffffff - 1;
  if (i < S) {
    const int pp = pos[static_cast<int64_t>(b) * S + i], ss = seq[static_cast<int64_t>(b) * S + i];
    pmin = pmax = pp;
    smin = smax = ss;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    pmin = min(pmin, __shfl_xor(pmin, o, 64));
    pmax = max(pmax, __shfl_xor(pmax, o, 64));
    smin = min(smin, __shfl_xor(smin, o, 64));
    smax = max(smax, __shfl_xor(smax, o, 64));
  }
  if (threadIdx.x == 0) out[static_cast<int64_t>(b) * ntiles + t] = make_int4(pmin, pmax, smin, smax);
}

template <int D, int MODE, int WAVES, int QB>
int launch_fwd(const AttnParams& p, hipStream_t st) {
  constexpr int THREADS = WAVES * 64;
  auto kern = attn_fwd_kernel<D, MODE, WAVES, QB>;
  constexpr int smem = FwdLds<D>::BYTES;
  static bool configured = false;  // per template instance; the attribute is sticky per function
  if (!configured && smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) {
      mlts_set_error("mlts_attn_fwd: cannot reserve %d bytes of LDS: %s", smem, hipGetErrorString(e));
      return MLTS_ERR_LAUNCH;
    }
    configured = true;
  }
  const int64_t blocks = static_cast<int64_t>(p.nqt) * p.B * p.Hq;
  {
    MltsKernelTimer timer("attn_fwd", st);
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(THREADS), smem, st, p);
  }
  return mlts_check_launch("mlts_attn_fwd");
}

}  // namespace

void mlts_launch_tile_stats(const int32_t* pos, const int32_t* seq, int B, int S, int4* out, hipStream_t st) {
  const int ntiles = (S + kAttnTile - 1) / kAttnTile;
  if (B * ntiles == 0) return;
  hipLaunchKernelGGL(tile_stats_kernel, dim3(B * ntiles), dim3(64), 0, st, pos, seq, S, ntiles, out);
}

namespace {
template <int WAVES, int QB>
int dispatch_fwd(AttnParams p, int D, int mode, hipStream_t st) {
  p.nqt = (p.Sq + WAVES * QB * 32 - 1) / (WAVES * QB * 32);
  if (D == 128) {
    if (mode == MLTS_MASK_NONE) return launch_fwd<128, MLTS_MASK_NONE, WAVES, QB>(p, st);
    if (mode == MLTS_MASK_CAUSAL) return launch_fwd<128, MLTS_MASK_CAUSAL, WAVES, QB>(p, st);
    return launch_fwd<128, MLTS_MASK_DOC, WAVES, QB>(p, st);
  }
  if (mode == MLTS_MASK_NONE) return launch_fwd<64, MLTS_MASK_NONE, WAVES, QB>(p, st);
  if (mode == MLTS_MASK_CAUSAL) return launch_fwd<64, MLTS_MASK_CAUSAL, WAVES, QB>(p, st);
  return launch_fwd<64, MLTS_MASK_DOC, WAVES, QB>(p, st);
}
}  // namespace

int mlts_attn_fwd_bf16_dma(const AttnParams& p, int D, int mode, hipStream_t st);  // attn_fwd_dma.hip

int mlts_attn_fwd_bf16(AttnParams p, int D, int mode, hipStream_t st) {
  // tuning aid: MLTS_FWD_VARIANT = "4x2" (one wavefront per SIMD) or "8x1" (register-staged tiles) selects the
  // older forms; the default is the LDS-DMA pipeline
  static const int variant = [] {
    const char* e = getenv("MLTS_FWD_VARIANT");
    if (e && e[0] == '4') return 4;
    if (e && e[0] == '8') return 8;
    return 0;
  }();
  if (variant == 4) return dispatch_fwd<4, 2>(p, D, mode, st);
  if (variant == 0) return mlts_attn_fwd_bf16_dma(p, D, mode, st);
  return dispatch_fwd<8, 1>(p, D, mode, st);
}
