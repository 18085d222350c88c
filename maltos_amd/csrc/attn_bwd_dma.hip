// Attention backward, dK and dV, head_dim 128, bf16: the gfx950 memory pipeline version of attn_bwd.hip.
//
// Same decomposition (a workgroup of 4 wavefronts owns 128 keys of one (batch, kv head), K and V fragments stay
// in registers, it walks the 64-row query tiles that can see them and keeps dK/dV in accumulators), but
//   * Q and dO tiles travel global -> LDS with 16-byte LDS-DMA loads into a three-stage ring (issued two tiles
//     ahead; no staging registers, no VALU transposes, no ds_write), together with the per-row statistics;
//   * each tile is stored once, row major with the chunk swizzle of attn_fwd_dma.hip; the transposed operands
//     of dV += P^T dO and dK += dS^T Q come from ds_read_b64_tr_b16;
//   * LDS reads are issued through inline assembly with counted waits (see attn_fwd_dma.hip for why);
//   * delta is folded into the matrix pipeline: the dP accumulator starts at delta and V is negated once, so it
//     ends as delta - dO V^T and -dS = P * that needs one multiply; dK is negated again with the softmax scale
//     when it is written;
//   * LSE arrives premultiplied by log2(e), with +inf for rows that saw no key (lse2, made by a one-pass kernel).
#include "attn_common.hpp"
#include <type_traits>

namespace {

constexpr int D = 128;
constexpr int BKV = 128;
constexpr int BQ = 64;
constexpr int WAVES = 4;
constexpr int THREADS = WAVES * 64;
constexpr int KS = D / 16;
constexpr int DB = D / 32;
constexpr int TILE_BYTES = BQ * D * 2;          // 16 KiB
constexpr int STAT_OFF = 2 * TILE_BYTES;        // lse2[64] then delta[64], fp32
constexpr int STAGE_BYTES = STAT_OFF + 2 * BQ * 4;
constexpr int STAGES = 3;
constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
constexpr int LOADS_PER_TILE = 2 * TILE_BYTES / (WAVES * 1024) + 1;  // DMA instructions per wavefront per tile (9)

typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef int v2i32 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int swz4(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

#define MLTS_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define MLTS_GLB(p) ((const __attribute__((address_space(1))) void*)(p))

template <int N>
__device__ __forceinline__ void wait_vm_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}
template <int OFF>
__device__ __forceinline__ v4i32 lds_read_b128(uint32_t addr) {
  v4i32 r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
template <int OFF>
__device__ __forceinline__ v2i32 lds_read_tr16_b64(uint32_t addr) {
  v2i32 r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
// wait_lgkm<N>(regs): only used when N or more LGKM operations of this code were issued after the reads into regs
template <int N>
__device__ __forceinline__ void wait_lgkm(v4i32 (&x)[4]) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_lgkm(v4i32 (&x)[8]) {
  asm volatile("s_waitcnt lgkmcnt(%8)"
               : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7])
               : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_lgkm(v2i32 (&x)[8]) {
  asm volatile("s_waitcnt lgkmcnt(%8)"
               : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7])
               : "n"(N));
}
__device__ __forceinline__ bf16x8 as_frag(v4i32 x) { return __builtin_bit_cast(bf16x8, x); }
__device__ __forceinline__ bf16x8 as_frag(v2i32 lo, v2i32 hi) {
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3));
}

// lse2[i] = lse[i] * log2(e), +inf where the row saw no key; lse2[n] = +inf is the entry that query rows beyond
// the end of the sequence are pointed at, so that their probabilities come out as exp2(s - inf) = 0 without a mask
__global__ __launch_bounds__(256) void lse2_kernel(const float* __restrict__ lse, float* __restrict__ lse2, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) {
    const float l = lse[i];
    lse2[i] = l == -INFINITY ? INFINITY : l * kLog2e;
  } else if (i == n) {
    lse2[i] = INFINITY;
  }
}

template <int MODE>
__global__ __launch_bounds__(THREADS, 1) void attn_bwd_dkdv_dma_kernel(const AttnBwdParams bp, const float* __restrict__ lse2) {
  const AttnParams& p = bp.a;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5, l16 = lane & 15;

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

  // ---- K and -V fragments (B operands), loaded once ----
  bf16x8 kf[KS], nvf[KS];
  {
    const int row = wkv0 + l32;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      v4i32 kk = {0, 0, 0, 0}, vv = {0, 0, 0, 0};
      if (row < p.Sk) {
        kk = *reinterpret_cast<const v4i32*>(K + static_cast<int64_t>(row) * p.ks[2] + ks * 16 + hh * 8);
        vv = *reinterpret_cast<const v4i32*>(V + static_cast<int64_t>(row) * p.vs[2] + ks * 16 + hh * 8);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) vv[i] ^= static_cast<int>(0x80008000u);
      kf[ks] = as_frag(kk);
      nvf[ks] = as_frag(vv);
    }
  }

  // ---- query-tile range ----
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

  // ---- DMA loader: this wavefront moves 1 KiB pieces 4w .. 4w+3 of the Q tile and of the dO tile, plus one row
  // of 64 statistics (even wavefronts lse2, odd ones delta; two wavefronts write each, identically) ----
  int ld_row[4], ld_col[4];
#pragma unroll
  for (int n = 0; n < 4; ++n) {
    const int row = (wave * 4 + n) * 4 + (lane >> 4);
    ld_row[n] = row;
    ld_col[n] = ((lane & 15) ^ swz4(row & 15)) * 8;
  }
  const int64_t lse2_inf = static_cast<int64_t>(p.B) * p.Hq * p.Sq;  // index of the +inf entry
  auto issue_tile = [&](int it, int stage) {
    const int hq = hkv * group + it / span;
    const int q0 = (qt_begin + it % span) * BQ;
    const bf16_t* Q = static_cast<const bf16_t*>(p.q) + b * p.qs[0] + hq * p.qs[1];
    const bf16_t* dO = static_cast<const bf16_t*>(bp.dout) + b * bp.dos[0] + hq * bp.dos[1];
    unsigned char* sbase = smem + stage * STAGE_BYTES;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int r = min(q0 + ld_row[n], p.Sq - 1);  // rows past the end repeat the last query; such tiles take the masked path
      const bf16_t* qsrc = Q + static_cast<int64_t>(r) * p.qs[2] + ld_col[n];
      const bf16_t* dsrc = dO + static_cast<int64_t>(r) * bp.dos[2] + ld_col[n];
      __builtin_amdgcn_global_load_lds(MLTS_GLB(qsrc), MLTS_LDS(sbase + (wave * 4 + n) * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(MLTS_GLB(dsrc), MLTS_LDS(sbase + TILE_BYTES + (wave * 4 + n) * 1024), 16, 0, 0);
    }
    const int64_t srow = (static_cast<int64_t>(b) * p.Hq + hq) * p.Sq;
    const float* ssrc = (wave & 1) ? bp.delta + srow + min(q0 + lane, p.Sq - 1)
                                   : lse2 + (q0 + lane < p.Sq ? srow + q0 + lane : lse2_inf);
    __builtin_amdgcn_global_load_lds(MLTS_GLB(ssrc), MLTS_LDS(sbase + STAT_OFF + (wave & 1) * (BQ * 4)), 4, 0, 0);
  };

  // ---- per-lane LDS read offsets (tile invariant) ----
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(MLTS_LDS(smem)));
  int roff[KS];  // row-major fragment (A operand): row l32 (+32 qb), chunk 2 ks + hh
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) roff[ks] = l32 * 256 + (((ks * 2 + hh) ^ swz4(l32 & 15)) << 4);
  int toff[2][DB];  // transposed fragment halves: query row 16 c + 8 part + 4 hh + l16/4, columns 32 db + 16 (l32/16) + 4 (l16%4)
#pragma unroll
  for (int part = 0; part < 2; ++part) {
    const int rlow = part * 8 + hh * 4 + (l16 >> 2);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int col = db * 32 + (l32 >> 4) * 16 + (l16 & 3) * 4;
      toff[part][db] = rlow * 256 + (((col >> 3) ^ swz4(rlow)) << 4) + ((col >> 2) & 1) * 8;
    }
  }
  const int soff_lane = STAT_OFF + hh * 16;  // statistics of rows 32 qb + 8 g + 4 hh .. +3

  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      dkacc[db][e] = 0.f;
      dvacc[db][e] = 0.f;
    }

  // ---- tile pipeline: sync number k = "needed tile k has landed everywhere"; tile k + 2 is issued right behind
  // it into stage (k + 2) % 3, which held tile k - 1: every wavefront finished reading it before this barrier ----
  int inflight = 0, istage = 0;
  int ji = next_it(0);
  auto issue_next = [&]() {
    if (ji < total_it) {
      issue_tile(ji, istage);
      istage = istage == STAGES - 1 ? 0 : istage + 1;
      ji = next_it(ji + 1);
      ++inflight;
    }
  };
  issue_next();
  issue_next();

  const int kj = wkv0 + l32;

  // One (128-key, 64-query) tile for this wavefront's 32 keys, straight-line code (the masked and the unmasked form
  // are separate instances so that nothing branches inside).  The matrix work is cut into sixteen groups of four
  // MFMAs; the softmax arithmetic of query block 0 is written between the S/dP groups of query block 1, and that of
  // block 1 between the first dV/dK groups, so that the one wavefront per SIMD has VALU work to issue while the
  // matrix pipe is busy.  P and -dS stay in registers: lane = key (wkv0 + l32), accumulator register e <-> query
  // 32 qb + 8 (e/4) + 4 hh + e%4, which is the A-operand layout of the dV/dK products.
  auto process_tile = [&](auto masked_tag, const int q0, const int stage) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const uint32_t sb = lds0 + stage * STAGE_BYTES;
    uint32_t ra[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ra[ks] = sb + roff[ks];
    const uint32_t sa = sb + soff_lane;
    uint32_t ta[2][DB];
#pragma unroll
    for (int part = 0; part < 2; ++part)
#pragma unroll
      for (int db = 0; db < DB; ++db) ta[part][db] = sb + toff[part][db];

    bf16x8 pfr[2][2], dsfr[2][2];
    f32x16 sacc[2], dpacc[2];  // matrix-pipe accumulators (AGPRs in this kernel)
    f32x16 sv[2], dv_[2];      // their copies in VGPRs for the softmax arithmetic
    f32x4 lse4[2][4];
    const int causal_t = kj - p.causal_off - q0 - hh * 4;

    auto softmax_chunk = [&](auto qb_tag, auto g_tag) {  // four queries: rows 32 qb + 8 g + 4 hh .. +3
      constexpr int qb = decltype(qb_tag)::value;
      constexpr int g = decltype(g_tag)::value;
      const int qrow = qb * 32 + g * 8 + hh * 4;
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
      float pv[4], nds[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int e = g * 4 + r;
        pv[r] = __builtin_amdgcn_exp2f(sv[qb][e] * p.scale_log2 - lse4[qb][g][r]);
        if (MASKED) {
          bool vis;
          if (MODE == MLTS_MASK_CAUSAL) {
            vis = causal_t <= qb * 32 + g * 8 + r;  // key <= query + causal_off; rows past Sq already give p = 0
          } else {
            const int qi = q0 + qrow + r;
            vis = kj < p.Sk && qi < p.Sq && (kpos <= qp4[r]) && (kseq == qs4[r]) && (qs4[r] >= 0);
          }
          if (!vis) pv[r] = 0.f;
        }
        nds[r] = pv[r] * dv_[qb][e];  // -dS
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pfr[qb][g >> 1][(g & 1) * 4 + r] = static_cast<bf16_t>(pv[r]);
        dsfr[qb][g >> 1][(g & 1) * 4 + r] = static_cast<bf16_t>(nds[r]);
      }
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;

#define MLTS_RREAD4(dst, QB, KS0)                                                  \
  dst[0] = lds_read_b128<(QB) * 8192>(ra[(KS0)]);                                  \
  dst[1] = lds_read_b128<(QB) * 8192>(ra[(KS0) + 1]);                              \
  dst[2] = lds_read_b128<TILE_BYTES + (QB) * 8192>(ra[(KS0)]);                     \
  dst[3] = lds_read_b128<TILE_BYTES + (QB) * 8192>(ra[(KS0) + 1]);
#define MLTS_SMFMA4(src, QB, KS0)                                                                                  \
  sacc[QB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[0]), kf[(KS0)], sacc[QB], 0, 0, 0);                \
  dpacc[QB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[2]), nvf[(KS0)], dpacc[QB], 0, 0, 0);             \
  sacc[QB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[1]), kf[(KS0) + 1], sacc[QB], 0, 0, 0);            \
  dpacc[QB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[3]), nvf[(KS0) + 1], dpacc[QB], 0, 0, 0);
#define MLTS_STAT_READ(st, QB)                                                    \
  _Pragma("unroll") for (int g = 0; g < 4; ++g) {                                 \
    st[g] = lds_read_b128<(QB) * 128>(sa + g * 32);                               \
    st[4 + g] = lds_read_b128<BQ * 4 + (QB) * 128>(sa + g * 32);                  \
  }
    // whole-vector casts below: casting a single element of an asm result is miscompiled (element 0 is broadcast)
#define MLTS_STAT_USE(st, QB)                                                     \
  _Pragma("unroll") for (int g = 0; g < 4; ++g) {                                 \
    lse4[QB][g] = __builtin_bit_cast(f32x4, st[g]);                               \
    const f32x4 dl = __builtin_bit_cast(f32x4, st[4 + g]);                        \
    _Pragma("unroll") for (int r = 0; r < 4; ++r) {                               \
      sacc[QB][g * 4 + r] = 0.f;                                                  \
      dpacc[QB][g * 4 + r] = dl[r];                                               \
    }                                                                             \
  }
#define MLTS_TREAD8(dst, C, H)                                                                   \
  _Pragma("unroll") for (int u = 0; u < 2; ++u) {                                                \
    dst[4 * u + 0] = lds_read_tr16_b64<TILE_BYTES + (C) * 4096>(ta[0][2 * (H) + u]);             \
    dst[4 * u + 1] = lds_read_tr16_b64<TILE_BYTES + (C) * 4096>(ta[1][2 * (H) + u]);             \
    dst[4 * u + 2] = lds_read_tr16_b64<(C) * 4096>(ta[0][2 * (H) + u]);                          \
    dst[4 * u + 3] = lds_read_tr16_b64<(C) * 4096>(ta[1][2 * (H) + u]);                          \
  }
#define MLTS_TMFMA4(src, C, H)                                                                                        \
  _Pragma("unroll") for (int u = 0; u < 2; ++u) {                                                                     \
    dvacc[2 * (H) + u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pfr[(C) >> 1][(C) & 1], as_frag(src[4 * u], src[4 * u + 1]), \
                                                                 dvacc[2 * (H) + u], 0, 0, 0);                        \
    dkacc[2 * (H) + u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsfr[(C) >> 1][(C) & 1], as_frag(src[4 * u + 2], src[4 * u + 3]), \
                                                                 dkacc[2 * (H) + u], 0, 0, 0);                        \
  }
    // the accumulators of one query block are copied out in one go, which frees their AGPRs for the next block
#define MLTS_TO_VGPR(QB)                                         \
  sv[QB] = sacc[QB];                                             \
  dv_[QB] = dpacc[QB];                                           \
  asm volatile("" : "+v"(sv[QB]), "+v"(dv_[QB]));
    v4i32 st[8], g0[4], g1[4];
    v2i32 h0[8], h1[8];
    // phase A: S and delta - dO V^T of query block 0
    MLTS_STAT_READ(st, 0)
    MLTS_RREAD4(g0, 0, 0)
    MLTS_RREAD4(g1, 0, 2)
    wait_lgkm<8>(st);
    MLTS_STAT_USE(st, 0)
    wait_lgkm<4>(g0);
    MLTS_SMFMA4(g0, 0, 0)
    MLTS_RREAD4(g0, 0, 4)
    wait_lgkm<4>(g1);
    MLTS_SMFMA4(g1, 0, 2)
    MLTS_RREAD4(g1, 0, 6)
    wait_lgkm<4>(g0);
    MLTS_SMFMA4(g0, 0, 4)
    MLTS_STAT_READ(st, 1)
    MLTS_RREAD4(g0, 1, 0)
    wait_lgkm<12>(g1);
    MLTS_SMFMA4(g1, 0, 6)
    MLTS_RREAD4(g1, 1, 2)
    MLTS_TO_VGPR(0)
    // phase B: the same for query block 1, with the softmax of block 0 in between
    wait_lgkm<8>(st);
    MLTS_STAT_USE(st, 1)
    wait_lgkm<4>(g0);
    MLTS_SMFMA4(g0, 1, 0)
    MLTS_RREAD4(g0, 1, 4)
    softmax_chunk(I0{}, I0{});
    wait_lgkm<4>(g1);
    MLTS_SMFMA4(g1, 1, 2)
    MLTS_RREAD4(g1, 1, 6)
    softmax_chunk(I0{}, I1{});
    wait_lgkm<4>(g0);
    MLTS_SMFMA4(g0, 1, 4)
    MLTS_TREAD8(h0, 0, 0)
    softmax_chunk(I0{}, I2{});
    wait_lgkm<8>(g1);
    MLTS_SMFMA4(g1, 1, 6)
    MLTS_TREAD8(h1, 0, 1)
    softmax_chunk(I0{}, I3{});
    MLTS_TO_VGPR(1)
    // phase C: dV += P^T dO, -dK += (-dS)^T Q for the queries of block 0, with the softmax of block 1 in between
    wait_lgkm<8>(h0);
    MLTS_TMFMA4(h0, 0, 0)
    MLTS_TREAD8(h0, 1, 0)
    softmax_chunk(I1{}, I0{});
    wait_lgkm<8>(h1);
    MLTS_TMFMA4(h1, 0, 1)
    MLTS_TREAD8(h1, 1, 1)
    softmax_chunk(I1{}, I1{});
    wait_lgkm<8>(h0);
    MLTS_TMFMA4(h0, 1, 0)
    MLTS_TREAD8(h0, 2, 0)
    softmax_chunk(I1{}, I2{});
    wait_lgkm<8>(h1);
    MLTS_TMFMA4(h1, 1, 1)
    MLTS_TREAD8(h1, 2, 1)
    softmax_chunk(I1{}, I3{});
    // phase D: the queries of block 1
    wait_lgkm<8>(h0);
    MLTS_TMFMA4(h0, 2, 0)
    MLTS_TREAD8(h0, 3, 0)
    wait_lgkm<8>(h1);
    MLTS_TMFMA4(h1, 2, 1)
    MLTS_TREAD8(h1, 3, 1)
    wait_lgkm<8>(h0);
    MLTS_TMFMA4(h0, 3, 0)
    wait_lgkm<0>(h1);
    MLTS_TMFMA4(h1, 3, 1)
#undef MLTS_RREAD4
#undef MLTS_SMFMA4
#undef MLTS_STAT_READ
#undef MLTS_STAT_USE
#undef MLTS_TREAD8
#undef MLTS_TMFMA4
#undef MLTS_TO_VGPR
  };

  int it = next_it(0);
  int stage = 0;
  while (it < total_it) {
    const int qt = qt_begin + it % span;
    const int q0 = qt * BQ;
    if (inflight >= 2) wait_vm_and_barrier<LOADS_PER_TILE>();
    else wait_vm_and_barrier<0>();
    --inflight;
    issue_next();

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

    // one instance of the tile body per mask mode where possible (two instances in one loop make the register
    // allocator move the accumulators at every block boundary): without a mask nothing needs masking (keys past Sk
    // are never stored, queries past Sq have lse2 = +inf), the causal comparison is cheap enough to be always on
    if (MODE == MLTS_MASK_NONE) {
      if (cls != TILE_SKIP) process_tile(std::false_type{}, q0, stage);
    } else if (MODE == MLTS_MASK_CAUSAL) {
      if (cls != TILE_SKIP) process_tile(std::true_type{}, q0, stage);
    } else {
      if (cls == TILE_FULL) process_tile(std::false_type{}, q0, stage);
      else if (cls == TILE_MASKED) process_tile(std::true_type{}, q0, stage);
    }
    it = next_it(it + 1);
    stage = stage == STAGES - 1 ? 0 : stage + 1;
  }

  // ---- write dK, dV: register e <-> key wkv0 + 8 (e/4) + 4 hh + e%4, lane -> head-dim column ----
  const float kscale = -p.scale;  // the accumulator holds -dS^T Q
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
          static_cast<float*>(bp.dk)[ok] += dkacc[db][e] * kscale;
          static_cast<float*>(bp.dv)[ov] += dvacc[db][e];
        } else {
          static_cast<bf16_t*>(bp.dk)[ok] = static_cast<bf16_t>(dkacc[db][e] * kscale);
          static_cast<bf16_t*>(bp.dv)[ov] = static_cast<bf16_t>(dvacc[db][e]);
        }
      }
    }
  }
}

template <int MODE>
int launch(const AttnBwdParams& bp, const float* lse2, hipStream_t st) {
  auto kern = attn_bwd_dkdv_dma_kernel<MODE>;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) {
      mlts_set_error("mlts_attn_bwd: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(e));
      return MLTS_ERR_LAUNCH;
    }
    configured = true;
  }
  const int64_t blocks = static_cast<int64_t>(bp.nkt) * bp.a.B * bp.a.Hkv;
  if (blocks > 0) {
    MltsKernelTimer timer("attn_bwd_dkdv", st);
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(THREADS), LDS_BYTES, st, bp, lse2);
  }
  return mlts_check_launch("mlts_attn_bwd");
}

}  // namespace

int64_t mlts_attn_bwd_dkdv_dma_workspace(int64_t B, int64_t Hq, int64_t Sq) { return (((B * Hq * Sq + 1) * 4 + 255) / 256) * 256; }

// head_dim 128, 16-byte aligned rows (checked by the caller); workspace holds B*Hq*Sq + 1 floats.
int mlts_attn_bwd_dkdv_bf16_dma(AttnBwdParams bp, int mode, void* workspace, hipStream_t st) {
  const AttnParams& p = bp.a;
  bp.nkt = (p.Sk + BKV - 1) / BKV;
  float* lse2 = static_cast<float*>(workspace);
  const int64_t n = static_cast<int64_t>(p.B) * p.Hq * p.Sq;
  hipLaunchKernelGGL(lse2_kernel, dim3(static_cast<unsigned>((n + 256) / 256)), dim3(256), 0, st, p.lse, lse2, n);
  if (mode == MLTS_MASK_NONE) return launch<MLTS_MASK_NONE>(bp, lse2, st);
  if (mode == MLTS_MASK_CAUSAL) return launch<MLTS_MASK_CAUSAL>(bp, lse2, st);
  return launch<MLTS_MASK_DOC>(bp, lse2, st);
}
