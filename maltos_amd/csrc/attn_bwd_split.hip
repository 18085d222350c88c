// Attention backward, dK and dV, head_dim 64 and 128, bf16: two-role workgroup.
//
// A workgroup owns 128 keys of one (batch, kv head) and walks the 64-row query tiles that can see them (all
// query heads of the GQA group); its EIGHT wavefronts come in two roles per 32-key block kb = wave % 4:
//     role 0 (wave < 4):   S = Q K^T,  P = exp2(S c - lse2)  ->  dV += P^T dO      and hands P (bf16) over in LDS
//     role 1 (wave >= 4):  delta - dO V^T,  -dS = P (delta - dO V^T)  ->  -dK += (-dS)^T Q     one tile behind
//                          (per barrier interval: dS of tile k-1, dP of tile k, then the dK products of tile k-1)
// Each role keeps one operand (K or -V) and one accumulator (dV or dK) in registers, so a wavefront fits in
// 256 registers, two wavefronts share a SIMD, the matrix instructions take plain VGPR accumulators (no AGPR
// copies around the softmax arithmetic) and the hardware overlaps one wavefront's VALU work with the other's
// matrix work.  The two GEMMs of a role read different LDS operands, so the split costs no extra LDS traffic
// beyond the 4 KiB of P per tile and key block.
//
// Memory pipeline: Q/dO tiles and the per-row statistics (lse2 = lse log2 e, delta) are fetched into registers right
// behind the barrier of tile k and written to a three-stage LDS ring after the work on tile k (role 1 still reads
// tile k - 1), row major with the chunk swizzle of attn_fwd_dma.hip; transposed operands come from
// ds_read_b64_tr_b16; LDS accesses are issued through inline assembly with counted waits; delta is folded into
// the dP accumulator and V is negated.
#include "attn_common.hpp"
#include <type_traits>

namespace {

constexpr int BKV = 128;
constexpr int BQ = 64;
constexpr int WAVES = 8;
constexpr int THREADS = WAVES * 64;
constexpr int STAGES = 3;
constexpr int PBUF_BYTES = 4 * 64 * 16;  // P hand-over: [2 buffers][4 key blocks][4 fragments][64 lanes] x 16 B

template <int D>
struct SplitCfg {
  static constexpr int KS = D / 16;                  // k-steps of the S / dP products
  static constexpr int DB = D / 32;                  // 32-column blocks of dV / dK
  static constexpr int RB = D * 2;                   // bytes per tile row
  static constexpr int CPR = RB / 16;                // 16-byte chunks per row
  static constexpr int TILE_BYTES = BQ * RB;
  static constexpr int STAT_OFF = 2 * TILE_BYTES;    // lse2[64], delta[64] (fp32); the rest of the stage's last KiB is unused
  static constexpr int STAGE_BYTES = STAT_OFF + 4 * BQ * 4;
  static constexpr int PBUF_OFF = STAGES * STAGE_BYTES;
  static constexpr int LDS_BYTES = PBUF_OFF + 2 * 4 * PBUF_BYTES;
  static constexpr int NLD = BQ * CPR / THREADS;     // 16-byte chunks per thread and tile (2 or 1)
};

typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef int v2i32 __attribute__((ext_vector_type(2)));

// chunk swizzle of a tile row (depends on row & 15): chunk c of row r is stored at chunk c ^ swz(r).  256-byte rows:
// swap of the two 2-bit halves; 128-byte rows (two rows per 256 bytes of banks): row bits 1,3,2 -> chunk bits 2,1,0.
// Measured: ds_read_b128 of 32 consecutive rows ~215-250 B/clk/CU and the transpose reads ~155-160 B/clk/CU.
template <int D>
__device__ __forceinline__ int swz(int r) {
  if (D == 128) return ((r & 3) << 2) | ((r >> 2) & 3);
  return (((r >> 1) & 1) << 2) | (((r >> 3) & 1) << 1) | ((r >> 2) & 1);
}

#define MLTS_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define MLTS_GLB(p) ((const __attribute__((address_space(1))) void*)(p))

// every LDS access of this wavefront has completed, then the workgroup barrier
__device__ __forceinline__ void drain_and_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

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
template <int OFF>
__device__ __forceinline__ void lds_write_b128(uint32_t addr, v4i32 x) {
  asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(x), "n"(OFF));
}
// wait_lgkm<N>(regs): only used when N or more LGKM operations of this code were issued after the reads into regs
template <int N>
__device__ __forceinline__ void wait_lgkm(v4i32 (&x)[4]) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_lgkm(v4i32 (&x)[2]) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x[0]), "+v"(x[1]) : "n"(N));
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

template <int D, int MODE>
__global__ __launch_bounds__(THREADS) void attn_bwd_dkdv_split_kernel(const AttnBwdParams bp, const float* __restrict__ lse2) {
  using C = SplitCfg<D>;
  constexpr int KS = C::KS, DB = C::DB, RB = C::RB, CPR = C::CPR, TILE_BYTES = C::TILE_BYTES, STAT_OFF = C::STAT_OFF,
                STAGE_BYTES = C::STAGE_BYTES, PBUF_OFF = C::PBUF_OFF, NLD = C::NLD;
  const AttnParams& p = bp.a;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5, l16 = lane & 15;
  const int role = wave >> 2, kb = wave & 3;

  const int nbh = p.B * p.Hkv;
  const int bid = blockIdx.x;
  int kt = bid / nbh;  // key tile; low tiles see the most queries under a causal mask and go first
  const int bh = bid % nbh;
  int b = bh / p.Hkv;
  const int hkv = bh % p.Hkv;
  if constexpr (MODE == MLTS_MASK_DOC) {
    // document masks: the (key tile, batch row) pairs are walked in the order of their work, most first
    if (p.kblock_order) {
      const int e = p.kblock_order[kt * p.B + b];
      kt = e / p.B;
      b = e % p.B;
    }
  }
  const int group = p.Hq / p.Hkv;
  const int kv0 = kt * BKV;
  const int wkv0 = kv0 + kb * 32;
  const int kj = wkv0 + l32;

  // ---- this wavefront's stationary operand (B operand of its first GEMM): K for role 0, -V for role 1 ----
  // (loaded here, sign applied after the first tile's loads have been issued too: one memory latency, not two)
  v4i32 kvraw[KS];
  {
    const bf16_t* src = role == 0 ? static_cast<const bf16_t*>(p.k) + b * p.ks[0] + hkv * p.ks[1] + static_cast<int64_t>(kj) * p.ks[2]
                                  : static_cast<const bf16_t*>(p.v) + b * p.vs[0] + hkv * p.vs[1] + static_cast<int64_t>(kj) * p.vs[2];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kvraw[ks] = v4i32{0, 0, 0, 0};
      if (kj < p.Sk) kvraw[ks] = *reinterpret_cast<const v4i32*>(src + ks * 16 + hh * 8);
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

  int4 kstats[2];
  if (MODE == MLTS_MASK_DOC) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int t = (kv0 >> 6) + i;
      kstats[i] = t < p.nk_stats ? p.k_stats[static_cast<int64_t>(b) * p.nk_stats + t] : make_int4(0x7fffffff, 0, 0, -2);
    }
  }
  const int4 wk_stats = MODE == MLTS_MASK_DOC ? ((kb >> 1) ? kstats[1] : kstats[0]) : make_int4(0, 0, 0, 0);
  // document masks: the lane's key has one 64-bit word per query tile (bit i = query i of the tile sees the key),
  // formed by a pre-pass for the tiles that classify() calls masked; role 0 fetches it along with the tile
  const unsigned long long* vis_row = nullptr;
  unsigned long long vis_next = 0;
  if (MODE == MLTS_MASK_DOC)
    vis_row = p.doc_bits_k + (static_cast<int64_t>(b) * p.nk_stats + min(wkv0 >> 6, p.nk_stats - 1)) * p.nq_stats * 64 + (wkv0 & 32) + l32;
  // The walk over (query head of the group, query tile) is kept as two counters; a position past the end has
  // h == group.  (No division by the runtime tile count in the loop.)
  struct Pos {
    int qt, h;  // query tile relative to qt_begin, head within the GQA group
  };
  auto at_end = [&](const Pos& x) -> bool { return x.h >= group || span == 0; };
  auto step = [&](Pos& x) {
    if (++x.qt == span) {
      x.qt = 0;
      ++x.h;
    }
  };
  // document masks: the needed query tiles (the same for every head of the group) are found 64 tiles of statistics
  // at a time; scan positions are relative to qt_begin
  DocTileScan scan;
  const int4* q_stats_row = MODE == MLTS_MASK_DOC ? p.q_stats + static_cast<int64_t>(b) * p.nq_stats + qt_begin : nullptr;
  auto first_needed = [&](Pos x) -> Pos {  // x itself or the next position whose tile is needed
    if (MODE != MLTS_MASK_DOC) return x;
    while (!at_end(x)) {
      const int q = doc_scan_next<2, false>(scan, x.qt, span, span, q_stats_row, kstats, wk_stats, lane);
      if (q < span) {
        x.qt = q;
        return x;
      }
      x.qt = 0;
      ++x.h;
    }
    return x;
  };
  auto classify = [&](const Pos& x) -> int {  // for this wavefront's 32 keys; identical in both roles of a key block
    const int qt = qt_begin + x.qt;
    const int q0 = qt * BQ;
    int cls = TILE_FULL;
    if (MODE == MLTS_MASK_CAUSAL) {
      const int last_q = min(q0 + BQ, p.Sq) - 1;
      if (wkv0 > last_q + p.causal_off) cls = TILE_SKIP;
      else if (wkv0 + 31 > q0 + p.causal_off) cls = TILE_MASKED;
    } else if (MODE == MLTS_MASK_DOC) {
      cls = doc_scan_class(scan, x.qt);
    }
    // (with a document mask, queries past Sq need no mask: their lse2 is +inf)
    if (cls == TILE_FULL && (wkv0 + 32 > p.Sk || (MODE != MLTS_MASK_DOC && q0 + BQ > p.Sq))) cls = TILE_MASKED;
    if (wkv0 >= p.Sk) cls = TILE_SKIP;
    return cls;
  };

  // ---- tile loader.  Measured on gfx950: an LDS-DMA load keeps the LDS busy for about 27 cycles per KiB while its
  // data arrives (3-4 times a ds_write_b128 of the same data) and ds_read streams of the whole CU stall meanwhile, and
  // this kernel is bound by LDS time.  So the next tile is fetched into registers right behind the barrier (chunks
  // t (and t + 512 for head_dim 128) of the Q tile and of the dO tile, chunk c = row c / CPR, stored 16-byte slot
  // c % CPR, source slot (c % CPR) ^ swz(row)) and written to LDS with ds_write_b128 after this tile's work.  Threads 0..127 also
  // carry the 64 + 64 row statistics (lse2, delta). ----
  const int64_t lse2_inf = static_cast<int64_t>(p.B) * p.Hq * p.Sq;  // index of the +inf entry
  // addresses: a wave-uniform tile pointer plus a 32-bit per-thread byte offset that is the same for every tile
  // not cut by the end of the sequence (row strides below 2^24 elements, checked by the caller)
  int ld_row[NLD], ld_col[NLD];
  uint32_t ld_qoff[NLD], ld_doff[NLD];
#pragma unroll
  for (int n = 0; n < NLD; ++n) {
    const int c = tid + n * THREADS;
    ld_row[n] = c / CPR;
    ld_col[n] = ((c % CPR) ^ swz<D>((c / CPR) & 15)) * 8;
    ld_qoff[n] = (static_cast<uint32_t>(ld_row[n]) * static_cast<uint32_t>(p.qs[2]) + ld_col[n]) * 2;  // bytes
    ld_doff[n] = (static_cast<uint32_t>(ld_row[n]) * static_cast<uint32_t>(bp.dos[2]) + ld_col[n]) * 2;
  }
  v4i32 stg_q[NLD], stg_d[NLD];
  float stg_s = 0.f;
  const uint32_t lds0_ = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(MLTS_LDS(smem)));
  auto stage_load = [&](const Pos& x) {
    const int hq = hkv * group + x.h;
    const int q0 = (qt_begin + x.qt) * BQ;
    const bf16_t* Q = static_cast<const bf16_t*>(p.q) + b * p.qs[0] + hq * p.qs[1] + static_cast<int64_t>(q0) * p.qs[2];
    const bf16_t* dO = static_cast<const bf16_t*>(bp.dout) + b * bp.dos[0] + hq * bp.dos[1] + static_cast<int64_t>(q0) * bp.dos[2];
    const int last = p.Sq - 1 - q0;  // rows past the end repeat the last query; their lse2 is +inf
#pragma unroll
    for (int n = 0; n < NLD; ++n) {
      uint32_t qo = ld_qoff[n], dofs = ld_doff[n];
      if (last < BQ - 1) {
        const uint32_t r = static_cast<uint32_t>(min(ld_row[n], last));
        qo = (r * static_cast<uint32_t>(p.qs[2]) + ld_col[n]) * 2;
        dofs = (r * static_cast<uint32_t>(bp.dos[2]) + ld_col[n]) * 2;
      }
      stg_q[n] = *reinterpret_cast<const v4i32*>(reinterpret_cast<const char*>(Q) + qo);
      stg_d[n] = *reinterpret_cast<const v4i32*>(reinterpret_cast<const char*>(dO) + dofs);
    }
    if (tid < 2 * BQ) {
      const int64_t srow = (static_cast<int64_t>(b) * p.Hq + hq) * p.Sq;
      const int r = q0 + (tid & (BQ - 1));
      stg_s = tid < BQ ? lse2[r < p.Sq ? srow + r : lse2_inf] : bp.delta[srow + min(r, p.Sq - 1)];
    }
    if (MODE == MLTS_MASK_DOC && role == 0) vis_next = vis_row[static_cast<int64_t>(qt_begin + x.qt) * 64];
  };
  const uint32_t stg_lane = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(MLTS_LDS(smem))) + tid * 16;
  auto stage_store = [&](int stage) {
    const uint32_t a = stg_lane + stage * STAGE_BYTES;
    lds_write_b128<0>(a, stg_q[0]);
    lds_write_b128<TILE_BYTES>(a, stg_d[0]);
    if (NLD == 2) {
      lds_write_b128<THREADS * 16>(a, stg_q[NLD - 1]);
      lds_write_b128<TILE_BYTES + THREADS * 16>(a, stg_d[NLD - 1]);
    }
    if (tid < 2 * BQ)
      asm volatile("ds_write_b32 %0, %1 offset:%2" ::"v"(lds0_ + stage * STAGE_BYTES + tid * 4), "v"(stg_s), "n"(STAT_OFF));
  };

  const Pos it0 = first_needed(Pos{0, 0});
  if (!at_end(it0)) stage_load(it0);
  bf16x8 kvf[KS];
  {
    const int flip = role == 0 ? 0 : static_cast<int>(0x80008000u);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int i = 0; i < 4; ++i) kvraw[ks][i] ^= flip;
      kvf[ks] = as_frag(kvraw[ks]);
    }
  }

  // ---- per-lane LDS offsets (tile invariant) ----
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(MLTS_LDS(smem)));
  // Row-major fragment (A operand): row l32 (+32 qb), chunk 2 ks + hh; role 0 reads Q, role 1 dO.  Transposed fragment
  // halves: query row 16 c + 8 part + 4 hh + l16/4, columns 32 db + 16 (l32/16) + 4 (l16%4); role 0 reads dO^T, role 1
  // Q^T.  The chunk swizzle is an XOR, so chunk (2 ks + hh) ^ s is ((ks ^ s/2) * 2) | ((hh ^ s) & 1) and column chunk
  // (4 db + y) ^ s is ((db ^ s/4) * 4) | (y ^ s % 4): an offset is a per-lane base plus an XOR of a compile-time index
  // with a per-lane constant.  With a document mask the kernel needs the registers of the sixteen offsets (it
  // otherwise spills into the tile loop) and forms them per tile from the six values they derive from.
  constexpr bool OFFS_IN_REGS = MODE == MLTS_MASK_CAUSAL;
  const int roff_base = role * TILE_BYTES + l32 * RB + (((hh ^ swz<D>(l32 & 15)) & 1) << 4);
  const int roff_x = swz<D>(l32 & 15) >> 1;
  int toff_base[2], toff_x[2];
#pragma unroll
  for (int part = 0; part < 2; ++part) {
    const int rlow = part * 8 + hh * 4 + (l16 >> 2);
    const int col0 = (l32 >> 4) * 16 + (l16 & 3) * 4;  // column inside a 32-column block
    toff_base[part] = (1 - role) * TILE_BYTES + rlow * RB + ((((col0 >> 3) ^ swz<D>(rlow)) & 3) << 4) + ((col0 >> 2) & 1) * 8;
    toff_x[part] = swz<D>(rlow) >> 2;
  }
  int roff_reg[KS], toff_reg[2][DB];
  if (OFFS_IN_REGS) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) roff_reg[ks] = roff_base + ((ks ^ roff_x) << 5);
#pragma unroll
    for (int part = 0; part < 2; ++part)
#pragma unroll
      for (int db = 0; db < DB; ++db) toff_reg[part][db] = toff_base[part] + ((db ^ toff_x[part]) << 6);
  }
  auto roff = [&](const int ks) -> int { return OFFS_IN_REGS ? roff_reg[ks] : roff_base + ((ks ^ roff_x) << 5); };
  auto toff = [&](const int part, const int db) -> int {
    return OFFS_IN_REGS ? toff_reg[part][db] : toff_base[part] + ((db ^ toff_x[part]) << 6);
  };
  // statistics of rows 32 qb + 8 g + 4 hh .. +3: role 0 reads lse2, role 1 delta
  const int soff_lane = STAT_OFF + role * (BQ * 4) + hh * 16;
  const uint32_t pbuf_lane = lds0 + PBUF_OFF + kb * PBUF_BYTES + lane * 16;

  f32x16 acc[DB];  // dV (role 0) or -dK / scale (role 1): register e <-> key wkv0 + 8 (e/4) + 4 hh + e%4, lane -> column
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[db][e] = 0.f;

#define MLTS_RREAD4(dst, QB, KS0)                              \
  dst[0] = lds_read_b128<(QB) * 32 * RB>(ra[(KS0)]);           \
  dst[1] = lds_read_b128<(QB) * 32 * RB>(ra[(KS0) + 1]);       \
  dst[2] = lds_read_b128<(QB) * 32 * RB>(ra[(KS0) + 2]);       \
  dst[3] = lds_read_b128<(QB) * 32 * RB>(ra[(KS0) + 3]);
#define MLTS_RMFMA4(src, ACC, KS0)                                                                    \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) ACC =                                                 \
      __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[i]), kvf[(KS0) + i], ACC, 0, 0, 0);
  // a transposed group = eight reads / four MFMAs: one 16-query step c (head_dim 128, four column blocks) or the
  // two steps c, c + 1 (head_dim 64, two column blocks each)
#define MLTS_TREAD8(dst, CS)                                                          \
  dst[0] = lds_read_tr16_b64<((CS) + 0 / DB) * 16 * RB>(ta[0][0 % DB]);               \
  dst[1] = lds_read_tr16_b64<((CS) + 0 / DB) * 16 * RB>(ta[1][0 % DB]);               \
  dst[2] = lds_read_tr16_b64<((CS) + 1 / DB) * 16 * RB>(ta[0][1 % DB]);               \
  dst[3] = lds_read_tr16_b64<((CS) + 1 / DB) * 16 * RB>(ta[1][1 % DB]);               \
  dst[4] = lds_read_tr16_b64<((CS) + 2 / DB) * 16 * RB>(ta[0][2 % DB]);               \
  dst[5] = lds_read_tr16_b64<((CS) + 2 / DB) * 16 * RB>(ta[1][2 % DB]);               \
  dst[6] = lds_read_tr16_b64<((CS) + 3 / DB) * 16 * RB>(ta[0][3 % DB]);               \
  dst[7] = lds_read_tr16_b64<((CS) + 3 / DB) * 16 * RB>(ta[1][3 % DB]);
#define MLTS_TMFMA4(src, AFRAG0, AFRAG1)                                                               \
  _Pragma("unroll") for (int u = 0; u < 4; ++u) acc[u % DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16( \
      (u / DB) ? AFRAG1 : AFRAG0, as_frag(src[2 * u], src[2 * u + 1]), acc[u % DB], 0, 0, 0);

  // ---- role 0: one tile.  lane = key, accumulator register e <-> query 32 qb + 8 (e/4) + 4 hh + e%4 ----
  auto role0_tile = [&](const bool masked, const int q0, const int stage, const int pbuf, const unsigned long long vis) {
    const uint32_t sb = lds0 + stage * STAGE_BYTES;
    uint32_t ra[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ra[ks] = sb + roff(ks);
    const uint32_t sa = sb + soff_lane;
    uint32_t ta[2][DB];
#pragma unroll
    for (int part = 0; part < 2; ++part)
#pragma unroll
      for (int db = 0; db < DB; ++db) ta[part][db] = sb + toff(part, db);
    const int causal_t = kj - p.causal_off - q0 - hh * 4;

    bf16x8 pfr[2][2];
    // masked tiles only (a wave-uniform branch around VALU work, no matrix instruction inside): hidden scores -> -inf
    auto apply_mask = [&](auto qb_tag, f32x16& s) {
      constexpr int qb = decltype(qb_tag)::value;
      // the comparisons below belong to masked tiles only: an opaque copy of their operand keeps the compiler from
      // hoisting all of them in front of the wave-uniform branch, where every tile would pay for them
      if constexpr (MODE == MLTS_MASK_DOC) {
        // bit 32 qb + 8 g + 4 hh + r of the key's word; the scores are handled as one integer vector (a cast of a
        // single element of a matrix result is miscompiled)
        typedef int i32x16 __attribute__((ext_vector_type(16)));
        const unsigned long long wsh = vis >> (hh * 4);
        const int wbits = static_cast<int>(qb ? (wsh >> 32) : wsh);
        i32x16 si = __builtin_bit_cast(i32x16, s);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int keep = __builtin_amdgcn_sbfe(wbits, (e >> 2) * 8 + (e & 3), 1);  // 0 or -1
          si[e] = (keep & si[e]) | (~keep & static_cast<int>(0xff800000u));
        }
        s = __builtin_bit_cast(f32x16, si);
      } else {
        int causal_here = causal_t;
        asm volatile("" : "+v"(causal_here));
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            // key <= query + causal_off; rows past Sq already give p = 0
            if (!(causal_here <= qb * 32 + g * 8 + r)) s[g * 4 + r] = -INFINITY;
          }
        }
      }
    };
    // one P fragment (8 of the 16 scores of a query block): exp2, packed conversion
    auto softmax_half = [&](auto qb_tag, auto t_tag, const f32x16& s, const f32x4 (&lse4)[4]) {
      constexpr int qb = decltype(qb_tag)::value;
      constexpr int t = decltype(t_tag)::value;
      v4i32 w;
#pragma unroll
      for (int j = 0; j < 4; ++j) {  // elements 8 t + 2 j, + 1 -> one packed conversion
        const int e = t * 8 + 2 * j;
        f32x2 pv;
        pv[0] = __builtin_amdgcn_exp2f(s[e] * p.scale_log2 - lse4[e >> 2][e & 3]);
        pv[1] = __builtin_amdgcn_exp2f(s[e + 1] * p.scale_log2 - lse4[(e + 1) >> 2][(e + 1) & 3]);
        w[j] = __builtin_bit_cast(int, __builtin_convertvector(pv, bf16x2));
      }
      pfr[qb][t] = __builtin_bit_cast(bf16x8, w);
    };
    // A wavefront can issue one MFMA per 32 cycles and VALU work in between: the four MFMAs of a group are spread
    // through the ~20 VALU instructions of half a softmax instead of being issued back to back.
#define MLTS_INTERLEAVE_4MFMA(NV)                                   \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
  __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);               \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
  __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);               \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
  __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);               \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
  __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);               \
  __builtin_amdgcn_sched_barrier(0);
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;

    v4i32 st0[4], st1[4], g0[4], g1[4];
    v2i32 h0[8], h1[8];
    f32x16 s0, s1;
    f32x4 lse4[4];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      s0[e] = 0.f;
      s1[e] = 0.f;
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) st0[g] = lds_read_b128<0>(sa + g * 32);
    // (whole-vector casts below: casting a single element of an asm result is miscompiled, element 0 is broadcast)
    if constexpr (D == 128) {
      MLTS_RREAD4(g0, 0, 0)
      MLTS_RREAD4(g1, 0, 4)
      wait_lgkm<8>(st0);
      wait_lgkm<4>(g0);
      MLTS_RMFMA4(g0, s0, 0)
#pragma unroll
      for (int g = 0; g < 4; ++g) st1[g] = lds_read_b128<128>(sa + g * 32);
      MLTS_RREAD4(g0, 1, 0)
      wait_lgkm<8>(g1);
      MLTS_RMFMA4(g1, s0, 4)
      MLTS_RREAD4(g1, 1, 4)
      wait_lgkm<8>(st1);
#pragma unroll
      for (int g = 0; g < 4; ++g) lse4[g] = __builtin_bit_cast(f32x4, st0[g]);
      if (masked) apply_mask(I0{}, s0);
      wait_lgkm<4>(g0);
      __builtin_amdgcn_sched_barrier(0);
      MLTS_RMFMA4(g0, s1, 0)
      softmax_half(I0{}, I0{}, s0, lse4);
      MLTS_INTERLEAVE_4MFMA(5)
      MLTS_TREAD8(h0, 0)
      wait_lgkm<8>(g1);
      __builtin_amdgcn_sched_barrier(0);
      MLTS_RMFMA4(g1, s1, 4)
      softmax_half(I0{}, I1{}, s0, lse4);
      MLTS_INTERLEAVE_4MFMA(5)
      MLTS_TREAD8(h1, 1)
      lds_write_b128<0>(pbuf_lane + pbuf, __builtin_bit_cast(v4i32, pfr[0][0]));
      lds_write_b128<1024>(pbuf_lane + pbuf, __builtin_bit_cast(v4i32, pfr[0][1]));
#pragma unroll
      for (int g = 0; g < 4; ++g) lse4[g] = __builtin_bit_cast(f32x4, st1[g]);
      if (masked) apply_mask(I1{}, s1);
      wait_lgkm<10>(h0);
      __builtin_amdgcn_sched_barrier(0);
      MLTS_TMFMA4(h0, pfr[0][0], pfr[0][0])
      softmax_half(I1{}, I0{}, s1, lse4);
      MLTS_INTERLEAVE_4MFMA(5)
      MLTS_TREAD8(h0, 2)
      wait_lgkm<8>(h1);
      __builtin_amdgcn_sched_barrier(0);
      MLTS_TMFMA4(h1, pfr[0][1], pfr[0][1])
      softmax_half(I1{}, I1{}, s1, lse4);
      MLTS_INTERLEAVE_4MFMA(5)
      MLTS_TREAD8(h1, 3)
      lds_write_b128<2048>(pbuf_lane + pbuf, __builtin_bit_cast(v4i32, pfr[1][0]));
      lds_write_b128<3072>(pbuf_lane + pbuf, __builtin_bit_cast(v4i32, pfr[1][1]));
      wait_lgkm<10>(h0);
      MLTS_TMFMA4(h0, pfr[1][0], pfr[1][0])
      wait_lgkm<0>(h1);
      MLTS_TMFMA4(h1, pfr[1][1], pfr[1][1])
    } else {
      // head_dim 64: one group of row reads per query block, one transposed group per two 16-query steps
#pragma unroll
      for (int g = 0; g < 4; ++g) st1[g] = lds_read_b128<128>(sa + g * 32);
      MLTS_RREAD4(g0, 0, 0)
      MLTS_RREAD4(g1, 1, 0)
      wait_lgkm<8>(st0);  // twelve reads follow: st0 and st1 have both arrived
      wait_lgkm<4>(g0);
      MLTS_RMFMA4(g0, s0, 0)
      MLTS_TREAD8(h0, 0)
#pragma unroll
      for (int g = 0; g < 4; ++g) lse4[g] = __builtin_bit_cast(f32x4, st0[g]);
      if (masked) apply_mask(I0{}, s0);
      wait_lgkm<8>(g1);
      __builtin_amdgcn_sched_barrier(0);
      MLTS_RMFMA4(g1, s1, 0)
      softmax_half(I0{}, I0{}, s0, lse4);
      softmax_half(I0{}, I1{}, s0, lse4);
      MLTS_INTERLEAVE_4MFMA(10)
      MLTS_TREAD8(h1, 2)
      lds_write_b128<0>(pbuf_lane + pbuf, __builtin_bit_cast(v4i32, pfr[0][0]));
      lds_write_b128<1024>(pbuf_lane + pbuf, __builtin_bit_cast(v4i32, pfr[0][1]));
#pragma unroll
      for (int g = 0; g < 4; ++g) lse4[g] = __builtin_bit_cast(f32x4, st1[g]);
      if (masked) apply_mask(I1{}, s1);
      wait_lgkm<10>(h0);
      __builtin_amdgcn_sched_barrier(0);
      MLTS_TMFMA4(h0, pfr[0][0], pfr[0][1])
      softmax_half(I1{}, I0{}, s1, lse4);
      softmax_half(I1{}, I1{}, s1, lse4);
      MLTS_INTERLEAVE_4MFMA(10)
      lds_write_b128<2048>(pbuf_lane + pbuf, __builtin_bit_cast(v4i32, pfr[1][0]));
      lds_write_b128<3072>(pbuf_lane + pbuf, __builtin_bit_cast(v4i32, pfr[1][1]));
      wait_lgkm<4>(h1);  // the four P writes follow it
      MLTS_TMFMA4(h1, pfr[1][0], pfr[1][1])
    }
#undef MLTS_INTERLEAVE_4MFMA
  };

  // ---- role 1, first half of a tile: dp = delta - dO V^T (kept in registers until P arrives) ----
  f32x16 dp0, dp1;
  auto role1_dp = [&](const int stage) {
    const uint32_t sb = lds0 + stage * STAGE_BYTES;
    uint32_t ra[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ra[ks] = sb + roff(ks);
    const uint32_t sa = sb + soff_lane;
    v4i32 st[8], g0[4], g1[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      st[g] = lds_read_b128<0>(sa + g * 32);
      st[4 + g] = lds_read_b128<128>(sa + g * 32);
    }
    MLTS_RREAD4(g0, 0, 0)
    if constexpr (D == 128) {
      MLTS_RREAD4(g1, 0, 4)
    } else {
      MLTS_RREAD4(g1, 1, 0)
    }
    wait_lgkm<8>(st);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 d0 = __builtin_bit_cast(f32x4, st[g]);
      const f32x4 d1 = __builtin_bit_cast(f32x4, st[4 + g]);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        dp0[g * 4 + r] = d0[r];
        dp1[g * 4 + r] = d1[r];
      }
    }
    if constexpr (D == 128) {
      wait_lgkm<4>(g0);
      MLTS_RMFMA4(g0, dp0, 0)
      MLTS_RREAD4(g0, 1, 0)
      wait_lgkm<4>(g1);
      MLTS_RMFMA4(g1, dp0, 4)
      MLTS_RREAD4(g1, 1, 4)
      wait_lgkm<4>(g0);
      MLTS_RMFMA4(g0, dp1, 0)
      wait_lgkm<0>(g1);
      MLTS_RMFMA4(g1, dp1, 4)
    } else {
      wait_lgkm<4>(g0);
      MLTS_RMFMA4(g0, dp0, 0)
      wait_lgkm<0>(g1);
      MLTS_RMFMA4(g1, dp1, 0)
    }
  };
  // ---- role 1, one barrier later: -dS = P dp as soon as P has arrived (frees dp for the next tile) ... ----
  bf16x8 dsfr[4];
  auto role1_ds = [&](const int pbuf) {
    v4i32 pp[4];
    pp[0] = lds_read_b128<0>(pbuf_lane + pbuf);
    pp[1] = lds_read_b128<1024>(pbuf_lane + pbuf);
    pp[2] = lds_read_b128<2048>(pbuf_lane + pbuf);
    pp[3] = lds_read_b128<3072>(pbuf_lane + pbuf);
    wait_lgkm<0>(pp);
#pragma unroll
    for (int f = 0; f < 4; ++f) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int pw = pp[f][w];  // two bf16 probabilities
        const float plo = __builtin_bit_cast(float, pw << 16);
        const float phi = __builtin_bit_cast(float, pw & static_cast<int>(0xffff0000u));
        const float dlo = (f >> 1) ? dp1[(f & 1) * 8 + 2 * w] : dp0[(f & 1) * 8 + 2 * w];
        const float dhi = (f >> 1) ? dp1[(f & 1) * 8 + 2 * w + 1] : dp0[(f & 1) * 8 + 2 * w + 1];
        dsfr[f][2 * w] = static_cast<bf16_t>(plo * dlo);
        dsfr[f][2 * w + 1] = static_cast<bf16_t>(phi * dhi);
      }
    }
  };
  // ---- ... and, after the dp of the next tile, -dK += (-dS)^T Q (transposed reads, while role 0 does its softmax) ----
  auto role1_dk = [&](const int stage) {
    const uint32_t sb = lds0 + stage * STAGE_BYTES;
    uint32_t ta[2][DB];
#pragma unroll
    for (int part = 0; part < 2; ++part)
#pragma unroll
      for (int db = 0; db < DB; ++db) ta[part][db] = sb + toff(part, db);
    v2i32 h0[8], h1[8];
    if constexpr (D == 128) {
      MLTS_TREAD8(h0, 0)
      MLTS_TREAD8(h1, 1)
      wait_lgkm<8>(h0);
      MLTS_TMFMA4(h0, dsfr[0], dsfr[0])
      MLTS_TREAD8(h0, 2)
      wait_lgkm<8>(h1);
      MLTS_TMFMA4(h1, dsfr[1], dsfr[1])
      MLTS_TREAD8(h1, 3)
      wait_lgkm<8>(h0);
      MLTS_TMFMA4(h0, dsfr[2], dsfr[2])
      wait_lgkm<0>(h1);
      MLTS_TMFMA4(h1, dsfr[3], dsfr[3])
    } else {
      MLTS_TREAD8(h0, 0)
      MLTS_TREAD8(h1, 2)
      wait_lgkm<8>(h0);
      MLTS_TMFMA4(h0, dsfr[0], dsfr[1])
      wait_lgkm<0>(h1);
      MLTS_TMFMA4(h1, dsfr[2], dsfr[3])
    }
  };
#undef MLTS_RREAD4
#undef MLTS_RMFMA4
#undef MLTS_TREAD8
#undef MLTS_TMFMA4

  // ---- tile loop, one instance per role (so that the state of one role is not live in the other's code).
  // Barrier k: tile k is in LDS and role 0 has handed over P of tile k - 1.  Tile k + 1 is fetched behind it and
  // stored into stage (k + 1) % 3, which held tile k - 2 (role 1 finished it before this barrier). ----
  int last_stage = 0;  // the only stage that role 1 still reads after the last barrier
  auto tile_loop = [&](auto role_tag) {
    constexpr int ROLE = decltype(role_tag)::value;
    Pos it = it0;  // its loads were issued in the prologue
    if (!at_end(it)) stage_store(0);
    int stage = 0, k = 0;
    bool prev_active = false;
    int prev_stage = 0;
    while (!at_end(it)) {
      const int cls = classify(it);  // before the scan of the needed tiles moves on
      const unsigned long long vis = vis_next;
      Pos itn = it;
      step(itn);
      itn = first_needed(itn);
      drain_and_barrier();
      if (!at_end(itn)) stage_load(itn);
      const int q0 = (qt_begin + it.qt) * BQ;
      const int pbuf = (k & 1) * (4 * PBUF_BYTES);
      if (ROLE == 0) {
        // one instance of the tile body (with several, the register allocator keeps the accumulators twice); the
        // mask is a branch around VALU work inside it.  Without a mask mode nothing needs masking: keys past Sk are
        // never stored and queries past Sq have lse2 = +inf.
        if (cls != TILE_SKIP) role0_tile(MODE != MLTS_MASK_NONE && cls == TILE_MASKED, q0, stage, pbuf, vis);
      } else {
        if (prev_active) role1_ds(pbuf ^ (4 * PBUF_BYTES));
        if (cls != TILE_SKIP) role1_dp(stage);
        if (prev_active) role1_dk(prev_stage);
      }
      if (!at_end(itn)) stage_store(stage == STAGES - 1 ? 0 : stage + 1);
      prev_active = cls != TILE_SKIP;
      prev_stage = stage;
      it = itn;
      stage = stage == STAGES - 1 ? 0 : stage + 1;
      ++k;
    }
    drain_and_barrier();
    if (ROLE == 1 && prev_active) {
      role1_ds(((k - 1) & 1) * (4 * PBUF_BYTES));
      role1_dk(prev_stage);
    }
    last_stage = prev_stage;
  };
  if (role == 0) {
    __builtin_amdgcn_s_setprio(1);  // role 0 has the longer chain per tile (softmax between its two products)
    tile_loop(std::integral_constant<int, 0>{});
    __builtin_amdgcn_s_setprio(0);
  } else {
    tile_loop(std::integral_constant<int, 1>{});
  }

  // ---- write dV (role 0) or dK (role 1) ----
  {
    const float oscale = role == 0 ? 1.0f : -p.scale;  // role 1 holds -dS^T Q
    void* optr = role == 0 ? bp.dv : bp.dk;
    const int64_t os[3] = {role == 0 ? bp.dvs[0] : bp.dks[0], role == 0 ? bp.dvs[1] : bp.dks[1], role == 0 ? bp.dvs[2] : bp.dks[2]};
    const bool rows16 = ((os[0] | os[1] | os[2]) & 7) == 0 && (reinterpret_cast<uintptr_t>(optr) & 15) == 0;
    if (!bp.accumulate_f32 && rows16) {
      // bf16 rows through LDS, so that global stores are 16 bytes per lane and cover whole rows: each wavefront owns
      // 32 rows x RB bytes of a stage that nobody reads any more (role 0: last_stage + 1, role 1: last_stage + 2);
      // chunk ^ (4 if row & 4) keeps the two half-wavefronts (rows 4 apart) on different banks
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      int es = last_stage + 1 + role;
      es = es >= STAGES ? es - STAGES : es;
      unsigned char* ebase = smem + es * STAGE_BYTES + kb * (32 * RB);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int col = db * 32 + l32;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = (e >> 2) * 8 + hh * 4 + (e & 3);
          const int chunk = (col >> 3) ^ (((row >> 2) & 1) << 2);
          *reinterpret_cast<bf16_t*>(ebase + row * RB + chunk * 16 + (col & 7) * 2) = static_cast<bf16_t>(acc[db][e] * oscale);
        }
      }
      bf16_t* obase = static_cast<bf16_t*>(optr) + b * os[0] + hkv * os[1];
#pragma unroll
      for (int i = 0; i < 32 * CPR / 64; ++i) {
        const int idx = i * 64 + lane;
        const int row = idx / CPR, chunk = idx % CPR;
        const v4i32 x = *reinterpret_cast<const v4i32*>(ebase + row * RB + ((chunk ^ (((row >> 2) & 1) << 2)) << 4));
        if (wkv0 + row < p.Sk) *reinterpret_cast<v4i32*>(obase + static_cast<int64_t>(wkv0 + row) * os[2] + chunk * 8) = x;
      }
    } else if (bp.accumulate_f32) {
      // fp32 gradients that are added to (ring steps): every load of the old values is issued before the first store,
      // so that the 64 read-modify-writes of a lane are one memory round trip and not 64 dependent ones (a store
      // between two loads through the same pointer keeps the compiler from moving the second load up)
      float* obase = static_cast<float*>(optr) + b * os[0] + hkv * os[1] + l32;
      float cur[DB][16];
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = wkv0 + (e >> 2) * 8 + hh * 4 + (e & 3);
          cur[db][e] = row < p.Sk ? obase[static_cast<int64_t>(row) * os[2] + db * 32] : 0.f;
        }
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = wkv0 + (e >> 2) * 8 + hh * 4 + (e & 3);
          if (row < p.Sk) obase[static_cast<int64_t>(row) * os[2] + db * 32] = cur[db][e] + acc[db][e] * oscale;
        }
    } else {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int d = db * 32 + l32;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = wkv0 + (e >> 2) * 8 + hh * 4 + (e & 3);
          if (row < p.Sk) {
            const int64_t o = b * os[0] + hkv * os[1] + static_cast<int64_t>(row) * os[2] + d;
            static_cast<bf16_t*>(optr)[o] = static_cast<bf16_t>(acc[db][e] * oscale);
          }
        }
      }
    }
  }
}

template <int D, int MODE>
int launch(const AttnBwdParams& bp, const float* lse2, hipStream_t st) {
  auto kern = attn_bwd_dkdv_split_kernel<D, MODE>;
  constexpr int lds_bytes = SplitCfg<D>::LDS_BYTES;
  static MltsLdsOptIn lds_opt_in;
  if (hipError_t e = lds_opt_in.reserve(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) {
    mlts_set_error("mlts_attn_bwd: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    return MLTS_ERR_LAUNCH;
  }
  const int64_t blocks = static_cast<int64_t>(bp.nkt) * bp.a.B * bp.a.Hkv;
  if (blocks > 0) {
    MltsKernelTimer timer("attn_bwd_dkdv", st);
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(THREADS), lds_bytes, st, bp, lse2);
  }
  return mlts_check_launch("mlts_attn_bwd");
}

template <int D>
int launch_mode(const AttnBwdParams& bp, int mode, const float* lse2, hipStream_t st) {
  if (mode == MLTS_MASK_NONE) return launch<D, MLTS_MASK_NONE>(bp, lse2, st);
  if (mode == MLTS_MASK_CAUSAL) return launch<D, MLTS_MASK_CAUSAL>(bp, lse2, st);
  return launch<D, MLTS_MASK_DOC>(bp, lse2, st);
}

}  // namespace

int64_t mlts_attn_bwd_dkdv_split_workspace(int64_t B, int64_t Hq, int64_t Sq) { return (((B * Hq * Sq + 1) * 4 + 255) / 256) * 256; }

// head_dim 64 or 128, 16-byte aligned rows (checked by the caller); workspace holds B*Hq*Sq + 1 floats.
// lse2_ready: the workspace already holds lse2 (written by the dQ kernel that ran before).
int mlts_attn_bwd_dkdv_bf16_split(AttnBwdParams bp, int D, int mode, void* workspace, bool lse2_ready, hipStream_t st) {
  const AttnParams& p = bp.a;
  bp.nkt = (p.Sk + BKV - 1) / BKV;
  float* lse2 = static_cast<float*>(workspace);
  const int64_t n = static_cast<int64_t>(p.B) * p.Hq * p.Sq;
  if (!lse2_ready)
    hipLaunchKernelGGL(lse2_kernel, dim3(static_cast<unsigned>((n + 256) / 256)), dim3(256), 0, st, p.lse, lse2, n);
  return D == 128 ? launch_mode<128>(bp, mode, lse2, st) : launch_mode<64>(bp, mode, lse2, st);
}
