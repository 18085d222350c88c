// Attention backward, dQ, head_dim 64 and 128, bf16: the version of attn_bwd_dq.hip with one LDS copy per tile.
//
// Same decomposition (a workgroup of 8 wavefronts owns 256 query rows of one (batch, head), each wavefront 32 of
// them, Q and dO stay in registers, it walks the visible keys in tiles of 64 and recomputes the scores transposed so
// that a lane owns one query and LSE / delta are per-lane scalars):
//     S^T  = K Q^T             A = K rows (LDS)              B = Q  (registers)
//     dlt - dP^T = dlt - V dO^T   A = V rows (LDS)              B = -dO (registers), accumulator starts at delta
//     P = exp2(S c - lse2),  -dS = P (delta - dP)               registers; layout = B operand of the next product
//     -dQ^T += K^T (-dS^T)     A = K^T (ds_read_b64_tr_b16 from the same K tile)
// K and V tiles are fetched into registers right behind the barrier and written once, row major with the chunk
// swizzle of attn_fwd_dma.hip, after the work on the current tile (two LDS stages); there is no transposed copy and
// no VALU transposition.  LDS reads go through inline assembly with counted waits (see attn_fwd_dma.hip).
#include "attn_common.hpp"
#include <type_traits>

namespace {

constexpr int BN = 64;
constexpr int WAVES = 8;
constexpr int THREADS = WAVES * 64;
constexpr int BM = WAVES * 32;
constexpr int STAGES = 2;

template <int D>
struct DqCfg {
  static constexpr int KS = D / 16;
  static constexpr int DB = D / 32;
  static constexpr int RB = D * 2;                     // bytes per tile row
  static constexpr int CPR = RB / 16;                  // 16-byte chunks per row
  static constexpr int TILE_BYTES = BN * RB;
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES;   // K then V
  static constexpr int PRO_BYTES = 2 * BM * RB;        // the prologue passes the Q and dO tiles through LDS
  static constexpr int DELTA_OFF = STAGES * STAGE_BYTES > PRO_BYTES ? STAGES * STAGE_BYTES : PRO_BYTES;  // delta[BM], fp32
  static constexpr int META_OFF = DELTA_OFF + BM * 4;  // document masks: per stage k_pos[64] then k_seq[64], int32
  static constexpr int META_BYTES = 2 * BN * 4;
  static constexpr int LDS_BYTES = META_OFF + STAGES * META_BYTES;
  static constexpr int NLD = BN * CPR / THREADS;       // 16-byte chunks per thread and tile (2 or 1)
};

typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef int v2i32 __attribute__((ext_vector_type(2)));

// chunk swizzle of a tile row (see attn_bwd_split.hip): 256-byte rows swap the 2-bit halves of row & 15, 128-byte rows
// send row bits 1,3,2 to chunk bits 2,1,0
template <int D>
__device__ __forceinline__ int swz(int r) {
  if (D == 128) return ((r & 3) << 2) | ((r >> 2) & 3);
  return (((r >> 1) & 1) << 2) | (((r >> 3) & 1) << 1) | ((r >> 2) & 1);
}

#define MLTS_LDS(p) ((__attribute__((address_space(3))) void*)(p))

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
__device__ __forceinline__ void wait_lgkm(v2i32 (&x)[8]) {
  asm volatile("s_waitcnt lgkmcnt(%8)"
               : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7])
               : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_lgkm(v4i32 (&x)[1]) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x[0]) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_lgkm(v4i32 (&x)[2]) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x[0]), "+v"(x[1]) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_lgkm(v2i32 (&x)[4]) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]) : "n"(N));
}
__device__ __forceinline__ bf16x8 as_frag(v4i32 x) { return __builtin_bit_cast(bf16x8, x); }
__device__ __forceinline__ bf16x8 as_frag(v2i32 lo, v2i32 hi) {
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3));
}

template <int D, int MODE>
__global__ __launch_bounds__(THREADS) void attn_bwd_dq_tr_kernel(const AttnBwdParams bp) {
  using C = DqCfg<D>;
  constexpr int KS = C::KS, DB = C::DB, RB = C::RB, CPR = C::CPR, TILE_BYTES = C::TILE_BYTES, STAGE_BYTES = C::STAGE_BYTES,
                NLD = C::NLD;
  const AttnParams& p = bp.a;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5, l16 = lane & 15;
  // Document masks with grouped-query heads: the workgroup's 256 rows are BM >> pack_shift rows of each of
  // 1 << pack_shift query heads of one KV head (the same rows: the same key tiles), and the (query block, batch row)
  // pairs are walked in the order of their work, most first (see AttnParams::head_pack_shift, qblock_order).
  const int pack_shift = MODE == MLTS_MASK_DOC ? p.head_pack_shift : 0;
  const int rows_per_head = BM >> pack_shift;
  const int hgroups = p.Hq >> pack_shift;
  const int nbh = p.B * hgroups;
  const int bid = blockIdx.x;
  int qt = p.nqt - 1 - bid / nbh;  // longest (last) q-tiles first under a causal mask
  const int bh = bid % nbh;
  int b = bh / hgroups;
  if constexpr (MODE == MLTS_MASK_DOC) {
    if (p.qblock_order) {
      const int e = p.qblock_order[(bid / nbh) * p.B + b];
      qt = e / p.B;
      b = e % p.B;
    }
  }
  const int hq0 = (bh % hgroups) << pack_shift;  // first head of the workgroup
  const int hq = MODE == MLTS_MASK_DOC ? hq0 + __builtin_amdgcn_readfirstlane((wave * 32) >> (8 - pack_shift)) : hq0;
  const int hkv = hq0 / (p.Hq / p.Hkv);
  const int q0 = qt * rows_per_head;
  const int wq0 = MODE == MLTS_MASK_DOC ? q0 + ((wave * 32) & (rows_per_head - 1)) : q0 + wave * 32;
  const int qrow = wq0 + l32;

  // (workgroup tile row -> head hq0 + (row >> (8 - pack_shift)), query q0 + (row & (rows_per_head - 1)))
  const bf16_t* Q = static_cast<const bf16_t*>(p.q) + b * p.qs[0] + hq0 * p.qs[1];
  const bf16_t* dO = static_cast<const bf16_t*>(bp.dout) + b * bp.dos[0] + hq0 * bp.dos[1];
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + b * p.vs[0] + hkv * p.vs[1];

  // Prologue loads, all issued before the first use of any of them.  The Q and dO tiles are fetched with whole-row
  // 16-byte loads (chunk c = tid + 512 n: row c / CPR, stored slot c % CPR, source slot (c % CPR) ^ swz(row), the tile
  // layout) and handed to the wavefronts through LDS: a fragment load straight from global memory touches 32 rows per
  // instruction and was measured at ~90 cycles per instruction, 8 us for the workgroup.  Rows past the end repeat
  // the last query (their lse2 is +inf, so they contribute nothing and are never stored).
  //
  // With bp.delta_out set, this kernel also produces the row statistics of the whole backward: it fetches the O rows
  // next to the dO rows, forms delta = rowsum(dO * O) from the chunks it holds (a row's CPR chunks sit in CPR
  // neighbouring lanes) and writes delta and lse2 for its rows; the dK/dV kernel, launched afterwards, reads them.
  constexpr int NPRO = BM * CPR / THREADS;
  const bool fold_stats = bp.delta_out != nullptr;
  const int64_t stat_off = (static_cast<int64_t>(b) * p.Hq + hq) * p.Sq + qrow;
  v4i32 pro_q[NPRO], pro_d[NPRO];
  float pro_dot[NPRO];
#pragma unroll
  for (int n = 0; n < NPRO; ++n) {
    const int c = tid + n * THREADS;
    const int row = c / CPR;
    const int col = ((c % CPR) ^ swz<D>(row & 15)) * 8;
    const int hrow = MODE == MLTS_MASK_DOC ? row >> (8 - pack_shift) : 0;
    const int64_t r = min(q0 + (MODE == MLTS_MASK_DOC ? row & (rows_per_head - 1) : row), p.Sq - 1);
    pro_q[n] = *reinterpret_cast<const v4i32*>(Q + hrow * p.qs[1] + r * p.qs[2] + col);
    pro_d[n] = *reinterpret_cast<const v4i32*>(dO + hrow * bp.dos[1] + r * bp.dos[2] + col);
  }
  if (fold_stats) {
    const bf16_t* O = static_cast<const bf16_t*>(p.o) + b * p.os[0] + hq0 * p.os[1];
    v4i32 pro_o[NPRO];
#pragma unroll
    for (int n = 0; n < NPRO; ++n) {
      const int c = tid + n * THREADS;
      const int row = c / CPR;
      const int col = ((c % CPR) ^ swz<D>(row & 15)) * 8;
      const int hrow = MODE == MLTS_MASK_DOC ? row >> (8 - pack_shift) : 0;
      const int64_t r = min(q0 + (MODE == MLTS_MASK_DOC ? row & (rows_per_head - 1) : row), p.Sq - 1);
      pro_o[n] = *reinterpret_cast<const v4i32*>(O + hrow * p.os[1] + r * p.os[2] + col);
    }
#pragma unroll
    for (int n = 0; n < NPRO; ++n) {
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {  // two bf16 per 32-bit word: low half = even element
        acc += __builtin_bit_cast(float, pro_d[n][i] << 16) * __builtin_bit_cast(float, pro_o[n][i] << 16);
        acc += __builtin_bit_cast(float, pro_d[n][i] & static_cast<int>(0xffff0000u)) *
               __builtin_bit_cast(float, pro_o[n][i] & static_cast<int>(0xffff0000u));
      }
#pragma unroll
      for (int m = CPR / 2; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
      pro_dot[n] = acc;
    }
  }
  float lse_raw = -INFINITY, delta = 0.f;
  if (qrow < p.Sq) {
    lse_raw = p.lse[stat_off];
    if (!fold_stats) delta = bp.delta[stat_off];
  }
  int4 wq_stats = make_int4(0, -1, 0, -1);
  int4 bq_stats[BM / 64];
  if (MODE == MLTS_MASK_DOC) {
#pragma unroll
    for (int w = 0; w < BM / 64; ++w) {
      const int t = (q0 >> 6) + w;
      bq_stats[w] = (w < (rows_per_head >> 6) && t < p.nq_stats) ? p.q_stats[static_cast<int64_t>(b) * p.nq_stats + t]
                                                                  : make_int4(0, -1, 0, -1);
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
  // needed tiles in increasing order (document masks: 64 tiles of statistics per step)
  DocTileScan scan;
  const int4* k_stats_row = MODE == MLTS_MASK_DOC ? p.k_stats + static_cast<int64_t>(b) * p.nk_stats : nullptr;
  auto next_tile = [&](int j) -> int {
    if (MODE != MLTS_MASK_DOC) return j < j_end ? j : j_end;
    return doc_scan_next<BM / 64, true>(scan, j, j_end, p.nk_stats, k_stats_row, bq_stats, wq_stats, lane);
  };

  // ---- tile loader: 64 bytes per thread, chunks t and t + 512 of the K tile and of the V tile (chunk c = row c/16,
  // stored 16-byte slot c%16, source slot (c%16) ^ swz(row)); registers now, ds_write_b128 after this tile's work ----
  // addresses: a wave-uniform tile pointer plus a 32-bit per-thread byte offset that is the same for every tile
  // not cut by the end of the sequence (a byte offset; row strides below 2^24 elements, checked by the caller)
  int ld_row[NLD], ld_col[NLD];
  uint32_t ld_koff[NLD], ld_voff[NLD];
#pragma unroll
  for (int n = 0; n < NLD; ++n) {
    const int c = tid + n * THREADS;
    ld_row[n] = c / CPR;
    ld_col[n] = ((c % CPR) ^ swz<D>((c / CPR) & 15)) * 8;
    ld_koff[n] = (static_cast<uint32_t>(ld_row[n]) * static_cast<uint32_t>(p.ks[2]) + ld_col[n]) * 2;  // bytes
    ld_voff[n] = (static_cast<uint32_t>(ld_row[n]) * static_cast<uint32_t>(p.vs[2]) + ld_col[n]) * 2;
  }
  v4i32 stg_k[NLD], stg_v[NLD];
  // document masks: this lane's query against the 64 keys of a tile, one bit per key (formed once per call by the pre-pass
  // for the pairs the kernels mask; other pairs' words are never looked at).  The word of the next tile is fetched with
  // that tile, always, so that no load of the loop stands under a branch.
  unsigned long long vis_next = 0;
  const unsigned long long* vis_row = nullptr;
  if (MODE == MLTS_MASK_DOC) {
    const int g = min(wq0 >> 6, p.nq_stats - 1);
    vis_row = p.doc_bits + (static_cast<int64_t>(b) * p.nq_stats + g) * p.nk_stats * 64 + ((wq0 >> 5) & 1) * 32 + l32;
  }
  auto stage_load = [&](int j) {
    const int kv0 = j * BN;
    if (MODE == MLTS_MASK_DOC) vis_next = vis_row[static_cast<int64_t>(j) * 64];
    const bf16_t* Kt = K + static_cast<int64_t>(kv0) * p.ks[2];
    const bf16_t* Vt = V + static_cast<int64_t>(kv0) * p.vs[2];
    const int last = p.Sk - 1 - kv0;  // rows past the end repeat the last key; their scores are masked
#pragma unroll
    for (int n = 0; n < NLD; ++n) {
      uint32_t ko = ld_koff[n], vo = ld_voff[n];
      if (last < BN - 1) {
        const uint32_t r = static_cast<uint32_t>(min(ld_row[n], last));
        ko = (r * static_cast<uint32_t>(p.ks[2]) + ld_col[n]) * 2;
        vo = (r * static_cast<uint32_t>(p.vs[2]) + ld_col[n]) * 2;
      }
      stg_k[n] = *reinterpret_cast<const v4i32*>(reinterpret_cast<const char*>(Kt) + ko);
      stg_v[n] = *reinterpret_cast<const v4i32*>(reinterpret_cast<const char*>(Vt) + vo);
    }
  };
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(MLTS_LDS(smem)));
  auto stage_store = [&](int stage) {
    const uint32_t a = lds0 + stage * STAGE_BYTES + tid * 16;
    lds_write_b128<0>(a, stg_k[0]);
    lds_write_b128<TILE_BYTES>(a, stg_v[0]);
    if (NLD == 2) {
      lds_write_b128<THREADS * 16>(a, stg_k[NLD - 1]);
      lds_write_b128<TILE_BYTES + THREADS * 16>(a, stg_v[NLD - 1]);
    }
  };

  const int j0 = next_tile(0);
  if (j0 < j_end) stage_load(j0);

  // ---- per-lane LDS read offsets (tile invariant) ----
  // (LDS addresses of stage 0; the stage, the key block and the tile are added as instruction offsets)
  // Row-major fragment (A operand): row l32 (+32 kb), chunk 2 ks + hh.  K^T fragment halves: key row 16 c + 8 part + 4 hh
  // + l16/4, columns 32 db + 16 (l32/16) + 4 (l16%4).  The chunk swizzle is an XOR, so chunk (2 ks + hh) ^ s is
  // ((ks ^ s/2) * 2) | ((hh ^ s) & 1) and column chunk (4 db + y) ^ s is ((db ^ s/4) * 4) | (y ^ s % 4): an address is a
  // per-lane base plus an XOR of a compile-time index with a per-lane constant.  Without a document mask the sixteen
  // addresses are kept in registers; with one the kernel needs those registers (it otherwise spills into the tile
  // loop) and forms each address where it is used, two instructions each.
  constexpr bool ADDR_IN_REGS = MODE != MLTS_MASK_DOC;
  const uint32_t ra_base = lds0 + l32 * RB + (((hh ^ swz<D>(l32 & 15)) & 1) << 4);
  const uint32_t ra_x = static_cast<uint32_t>(swz<D>(l32 & 15) >> 1);
  uint32_t ta_base[2], ta_x[2];
#pragma unroll
  for (int part = 0; part < 2; ++part) {
    const int rlow = part * 8 + hh * 4 + (l16 >> 2);
    const int col0 = (l32 >> 4) * 16 + (l16 & 3) * 4;  // column inside a 32-column block
    ta_base[part] = lds0 + rlow * RB + ((((col0 >> 3) ^ swz<D>(rlow)) & 3) << 4) + ((col0 >> 2) & 1) * 8;
    ta_x[part] = static_cast<uint32_t>(swz<D>(rlow) >> 2);
  }
  uint32_t ra_reg[KS], ta_reg[2][DB];
  if (ADDR_IN_REGS) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ra_reg[ks] = ra_base + ((static_cast<uint32_t>(ks) ^ ra_x) << 5);
#pragma unroll
    for (int part = 0; part < 2; ++part)
#pragma unroll
      for (int db = 0; db < DB; ++db) ta_reg[part][db] = ta_base[part] + ((static_cast<uint32_t>(db) ^ ta_x[part]) << 6);
  }
  auto ra = [&](const int ks) -> uint32_t {
    return ADDR_IN_REGS ? ra_reg[ks] : ra_base + ((static_cast<uint32_t>(ks) ^ ra_x) << 5);
  };
  auto ta = [&](const int part, const int db) -> uint32_t {
    return ADDR_IN_REGS ? ta_reg[part][db] : ta_base[part] + ((static_cast<uint32_t>(db) ^ ta_x[part]) << 6);
  };

  bf16x8 qf[KS], ndof[KS];  // Q and -dO fragments (B operands): row 32 wave + l32, the row-major fragment pattern
  {
    const uint32_t wbase = lds0 + tid * 16;
#pragma unroll
    for (int n = 0; n < NPRO; ++n) {
      lds_write_b128<0>(wbase + n * (THREADS * 16), pro_q[n]);
      lds_write_b128<0>(wbase + BM * RB + n * (THREADS * 16), pro_d[n]);
    }
    if (fold_stats && tid % CPR == 0) {
      float* sdelta = reinterpret_cast<float*>(smem + C::DELTA_OFF);
#pragma unroll
      for (int n = 0; n < NPRO; ++n) sdelta[tid / CPR + n * (THREADS / CPR)] = pro_dot[n];
    }
    drain_and_barrier();
    v4i32 fq[KS], fd[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      fq[ks] = lds_read_b128<0>(ra(ks) + wave * (32 * RB));
      fd[ks] = lds_read_b128<0>(ra(ks) + wave * (32 * RB) + BM * RB);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      // (the registers are operands of the wait, so that the compiler cannot touch them before it)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fq[ks]), "+v"(fd[ks])::"memory");
#pragma unroll
      for (int i = 0; i < 4; ++i) fd[ks][i] ^= static_cast<int>(0x80008000u);
      qf[ks] = as_frag(fq[ks]);
      ndof[ks] = as_frag(fd[ks]);
    }
    if (fold_stats) delta = reinterpret_cast<const float*>(smem + C::DELTA_OFF)[wave * 32 + l32];
    drain_and_barrier();  // the K/V tiles may overwrite the Q and dO tiles from here on
  }
  // +inf makes exp2(s - lse2) = 0 for rows that saw no key or lie past Sq
  const float lse2 = lse_raw == -INFINITY ? INFINITY : lse_raw * kLog2e;
  if (fold_stats) {
    if (qrow < p.Sq && hh == 0) {
      bp.delta_out[stat_off] = delta;
      bp.lse2_out[stat_off] = lse2;
    }
    if (bid == 0 && tid == 0) bp.lse2_out[static_cast<int64_t>(p.B) * p.Hq * p.Sq] = INFINITY;
  }

  f32x16 dqacc[DB];  // -dQ^T / scale: register e <-> head-dim 32 db + 8 (e/4) + 4 hh + e%4, lane -> query row
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) dqacc[db][e] = 0.f;

  // read groups are kept small (two 16-byte row reads, or four transpose reads) and two are in flight: the kernel
  // sits at the 256-register limit of two wavefronts per SIMD
#define MLTS_RREAD2(dst, KB, KS0)                                                  \
  dst[0] = lds_read_b128<(KB) * 32 * RB>(ra((KS0)) + so);                             \
  dst[1] = lds_read_b128<TILE_BYTES + (KB) * 32 * RB>(ra((KS0)) + so);
  // Two idle cycles behind every MFMA: a wavefront that streams MFMAs back to back keeps the SIMD's vector issue port,
  // and the other wavefront of the SIMD (all eight do the same work, the older one of a pair wins every arbitration: it
  // finishes a tile in 2800 cycles and waits 1500 at the barrier for the other's 4400) gets no vector instruction in.
  // With the pause the other wavefront's exponentials go in between (measured: 3 % at head_dim 128, 4.5 % at 64; the
  // same pause in the forward and dK/dV kernels, whose wavefronts run in different phases by construction, gave nothing).
#define MLTS_MFMA_PAUSE(acc) asm volatile("s_nop 1" : "+v"(acc));
#define MLTS_SMFMA2(src, KS0)                                                                            \
  s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[0]), qf[(KS0)], s, 0, 0, 0);                   \
  MLTS_MFMA_PAUSE(s)                                                                                     \
  dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[1]), ndof[(KS0)], dp, 0, 0, 0);               \
  MLTS_MFMA_PAUSE(dp)
#define MLTS_TREAD4(dst, C, H)                                                       \
  dst[0] = lds_read_tr16_b64<(C) * 16 * RB>(ta(0, 2 * (H)) + so);                       \
  dst[1] = lds_read_tr16_b64<(C) * 16 * RB>(ta(1, 2 * (H)) + so);                       \
  dst[2] = lds_read_tr16_b64<(C) * 16 * RB>(ta(0, 2 * (H) + 1) + so);                   \
  dst[3] = lds_read_tr16_b64<(C) * 16 * RB>(ta(1, 2 * (H) + 1) + so);
#define MLTS_TMFMA2(src, H, BFRAG)                                                                                        \
  dqacc[2 * (H)] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[0], src[1]), BFRAG, dqacc[2 * (H)], 0, 0, 0);       \
  MLTS_MFMA_PAUSE(dqacc[2 * (H)])                                                                                         \
  dqacc[2 * (H) + 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[2], src[3]), BFRAG, dqacc[2 * (H) + 1], 0, 0, 0); \
  MLTS_MFMA_PAUSE(dqacc[2 * (H) + 1])

  // one 64-key tile for this wavefront's 32 queries, one 32-key block after the other; lane = query, accumulator
  // register e <-> key 32 kb + 8 (e/4) + 4 hh + e%4
  auto process_tile = [&](const bool masked, const uint32_t so, const int kv0, const unsigned long long vis) {
    const int klim_t = min(qrow + (MODE == MLTS_MASK_CAUSAL ? p.causal_off : 0x3fffffff), p.Sk - 1) - kv0 - hh * 4;
    bf16x8 dsf[2];
    f32x16 s, dp;
    // masked tiles only (a wave-uniform branch around VALU work, no matrix instruction inside): hidden scores -> -inf
    auto apply_mask = [&](const int kb) {
      if constexpr (MODE == MLTS_MASK_DOC) {
        // register (g, r) <-> key kb * 32 + g * 8 + hh * 4 + r: after a shift by hh * 4 the bit positions are constants
        typedef int i32x16 __attribute__((ext_vector_type(16)));
        const unsigned long long wsh = vis >> (hh * 4);
        const int wbits = static_cast<int>(kb ? wsh >> 32 : wsh);
        // whole-vector casts: casting single elements of an MFMA result is miscompiled (element 0 is broadcast)
        i32x16 si = __builtin_bit_cast(i32x16, s);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int keep = __builtin_amdgcn_sbfe(wbits, (e >> 2) * 8 + (e & 3), 1);  // all ones if visible
          si[e] = (keep & si[e]) | (~keep & static_cast<int>(0xff800000u));
        }
        s = __builtin_bit_cast(f32x16, si);
      } else {
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            // key <= min(query + causal_off, Sk - 1), as one comparison against a per-lane, per-tile threshold
            if (!(kb * 32 + g * 8 + r <= klim_t)) s[g * 4 + r] = -INFINITY;
          }
      }
    };
    auto ds_block = [&](const int kb) {
      if (masked) apply_mask(kb);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        v4i32 w;
#pragma unroll
        for (int j = 0; j < 4; ++j) {  // elements 8 t + 2 j, + 1 -> one packed conversion of -dS
          const int e = t * 8 + 2 * j;
          f32x2 ds;
          ds[0] = __builtin_amdgcn_exp2f(s[e] * p.scale_log2 - lse2) * dp[e];
          ds[1] = __builtin_amdgcn_exp2f(s[e + 1] * p.scale_log2 - lse2) * dp[e + 1];
          w[j] = __builtin_bit_cast(int, __builtin_convertvector(ds, bf16x2));
        }
        dsf[t] = __builtin_bit_cast(bf16x8, w);
      }
    };
    auto acc_init = [&]() {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        s[e] = 0.f;
        dp[e] = delta;
      }
    };
    v4i32 g0[2], g1[2];
    v2i32 h0[4], h1[4];
#define MLTS_KEY_BLOCK_128(KB)                                                     \
    acc_init();                                                                    \
    MLTS_RREAD2(g0, KB, 0)                                                         \
    MLTS_RREAD2(g1, KB, 1)                                                         \
    wait_lgkm<2>(g0); MLTS_SMFMA2(g0, 0) MLTS_RREAD2(g0, KB, 2)                    \
    wait_lgkm<2>(g1); MLTS_SMFMA2(g1, 1) MLTS_RREAD2(g1, KB, 3)                    \
    wait_lgkm<2>(g0); MLTS_SMFMA2(g0, 2) MLTS_RREAD2(g0, KB, 4)                    \
    wait_lgkm<2>(g1); MLTS_SMFMA2(g1, 3) MLTS_RREAD2(g1, KB, 5)                    \
    wait_lgkm<2>(g0); MLTS_SMFMA2(g0, 4) MLTS_RREAD2(g0, KB, 6)                    \
    wait_lgkm<2>(g1); MLTS_SMFMA2(g1, 5) MLTS_RREAD2(g1, KB, 7)                    \
    wait_lgkm<2>(g0); MLTS_SMFMA2(g0, 6) MLTS_TREAD4(h0, 2 * (KB), 0)              \
    wait_lgkm<4>(g1); MLTS_SMFMA2(g1, 7) MLTS_TREAD4(h1, 2 * (KB), 1)              \
    ds_block(KB);                                                                  \
    wait_lgkm<4>(h0); MLTS_TMFMA2(h0, 0, dsf[0]) MLTS_TREAD4(h0, 2 * (KB) + 1, 0)  \
    wait_lgkm<4>(h1); MLTS_TMFMA2(h1, 1, dsf[0]) MLTS_TREAD4(h1, 2 * (KB) + 1, 1)  \
    wait_lgkm<4>(h0); MLTS_TMFMA2(h0, 0, dsf[1])                                   \
    wait_lgkm<0>(h1); MLTS_TMFMA2(h1, 1, dsf[1])
#define MLTS_KEY_BLOCK_64(KB)                                                      \
    acc_init();                                                                    \
    MLTS_RREAD2(g0, KB, 0)                                                         \
    MLTS_RREAD2(g1, KB, 1)                                                         \
    wait_lgkm<2>(g0); MLTS_SMFMA2(g0, 0) MLTS_RREAD2(g0, KB, 2)                    \
    wait_lgkm<2>(g1); MLTS_SMFMA2(g1, 1) MLTS_RREAD2(g1, KB, 3)                    \
    wait_lgkm<2>(g0); MLTS_SMFMA2(g0, 2) MLTS_TREAD4(h0, 2 * (KB), 0)              \
    wait_lgkm<4>(g1); MLTS_SMFMA2(g1, 3) MLTS_TREAD4(h1, 2 * (KB) + 1, 0)          \
    ds_block(KB);                                                                  \
    wait_lgkm<4>(h0); MLTS_TMFMA2(h0, 0, dsf[0])                                   \
    wait_lgkm<0>(h1); MLTS_TMFMA2(h1, 0, dsf[1])
    if constexpr (D == 128) {
      MLTS_KEY_BLOCK_128(0)
      MLTS_KEY_BLOCK_128(1)
    } else {
      MLTS_KEY_BLOCK_64(0)
      MLTS_KEY_BLOCK_64(1)
    }
#undef MLTS_KEY_BLOCK_128
#undef MLTS_KEY_BLOCK_64
  };
#undef MLTS_RREAD2
#undef MLTS_SMFMA2
#undef MLTS_TREAD4
#undef MLTS_TMFMA2
#undef MLTS_MFMA_PAUSE

  // ---- tile loop.  Barrier k: tile k is in LDS.  Tile k + 1 is fetched behind it into registers and stored into the
  // other stage (read last during tile k - 1) after the work on tile k.  There is one instance of the tile body
  // (with several, the register allocator keeps the dQ accumulators twice); masking is a branch inside it. ----
  {
    int j = j0;  // its loads were issued in the prologue
    if (j < j_end) stage_store(0);
    int stage = 0;
    while (j < j_end) {
      const int doc_cls = MODE == MLTS_MASK_DOC ? doc_scan_class(scan, j) : TILE_FULL;  // before the scan moves on
      const int jn = next_tile(j + 1);
      drain_and_barrier();
      const unsigned long long vis = vis_next;  // of tile j; stage_load fetches the next tile's
      if (jn < j_end) stage_load(jn);

      const int kv0 = j * BN;
      int cls = TILE_FULL;
      if (MODE == MLTS_MASK_CAUSAL) {
        if (kv0 > wave_last_q + p.causal_off) cls = TILE_SKIP;
        else if (kv0 + BN - 1 > wq0 + p.causal_off) cls = TILE_MASKED;
      } else if (MODE == MLTS_MASK_DOC) {
        cls = doc_cls;
      }
      if (cls == TILE_FULL && kv0 + BN > p.Sk) cls = TILE_MASKED;  // ragged last tile: key < Sk
      if (wq0 >= p.Sq) cls = TILE_SKIP;
      if (cls != TILE_SKIP) process_tile(cls == TILE_MASKED, stage * STAGE_BYTES, kv0, vis);

      if (jn < j_end) stage_store(stage ^ 1);
      j = jn;
      stage ^= 1;
    }
  }

  const float oscale = -p.scale;  // the accumulator holds K^T (-dS^T)
  const bool rows16 = ((bp.dqs[0] | bp.dqs[1] | bp.dqs[2]) & 7) == 0 && (reinterpret_cast<uintptr_t>(bp.dq_acc) & 15) == 0;
  if (!bp.dq_f32 && rows16) {
    // bf16 rows through LDS (each wavefront owns 32 rows x RB bytes, tile-row swizzle), so that global stores are
    // 16 bytes per lane and cover whole rows
    drain_and_barrier();  // every wavefront has finished reading the last K/V tile
    unsigned char* ebase = smem + wave * (32 * RB);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = static_cast<bf16_t>(dqacc[db][g * 4 + r] * oscale);
        *reinterpret_cast<bf16x4*>(ebase + l32 * RB + (((db * 4 + g) ^ swz<D>(l32 & 15)) << 4) + hh * 8) = w;
      }
    }
    bf16_t* obase = reinterpret_cast<bf16_t*>(bp.dq_acc) + b * bp.dqs[0] + hq * bp.dqs[1];
#pragma unroll
    for (int i = 0; i < 32 * CPR / 64; ++i) {
      const int idx = i * 64 + lane;
      const int row = idx / CPR, chunk = idx % CPR;
      const v4i32 x = *reinterpret_cast<const v4i32*>(ebase + row * RB + ((chunk ^ swz<D>(row & 15)) << 4));
      if (wq0 + row < p.Sq) *reinterpret_cast<v4i32*>(obase + static_cast<int64_t>(wq0 + row) * bp.dqs[2] + chunk * 8) = x;
    }
  } else if (qrow < p.Sq && bp.dq_f32) {
    // fp32 gradients that are added to (ring steps): all loads of the old values before the first store, one memory
    // round trip instead of sixteen dependent ones; the first block of an accumulation (dq_f32 == 2) stores only
    f32x4* dst = reinterpret_cast<f32x4*>(bp.dq_acc + b * bp.dqs[0] + hq * bp.dqs[1] + static_cast<int64_t>(qrow) * bp.dqs[2] + hh * 4);
    f32x4 cur[DB][4];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) cur[db][g] = bp.dq_f32 == 2 ? f32x4{0.f, 0.f, 0.f, 0.f} : dst[db * 8 + g * 2];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
#pragma unroll
        for (int r = 0; r < 4; ++r) cur[db][g][r] += dqacc[db][g * 4 + r] * oscale;
        dst[db * 8 + g * 2] = cur[db][g];
      }
  } else if (qrow < p.Sq) {
    const int64_t rowoff = b * bp.dqs[0] + hq * bp.dqs[1] + static_cast<int64_t>(qrow) * bp.dqs[2];
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = db * 32 + g * 8 + hh * 4;
        bf16x4 w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = static_cast<bf16_t>(dqacc[db][g * 4 + r] * oscale);
        *reinterpret_cast<bf16x4*>(reinterpret_cast<bf16_t*>(bp.dq_acc) + rowoff + d) = w;
      }
    }
  }
}

template <int D, int MODE>
int launch(AttnBwdParams bp, hipStream_t st) {
  auto kern = attn_bwd_dq_tr_kernel<D, MODE>;
  constexpr int lds_bytes = DqCfg<D>::LDS_BYTES;
  static MltsLdsOptIn lds_opt_in;
  if (hipError_t e = lds_opt_in.reserve(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) {
    mlts_set_error("mlts_attn_bwd: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    return MLTS_ERR_LAUNCH;
  }
  if (MODE != MLTS_MASK_DOC) bp.a.head_pack_shift = 0;  // (set with the block order by the caller's pre-pass otherwise)
  const int rows = BM >> bp.a.head_pack_shift;
  bp.a.nqt = (bp.a.Sq + rows - 1) / rows;
  const int64_t blocks = static_cast<int64_t>(bp.a.nqt) * bp.a.B * (bp.a.Hq >> bp.a.head_pack_shift);
  if (blocks > 0) {
    MltsKernelTimer timer("attn_bwd_dq", st);
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(THREADS), lds_bytes, st, bp);
  }
  return mlts_check_launch("mlts_attn_bwd");
}

template <int D>
int launch_mode(const AttnBwdParams& bp, int mode, hipStream_t st) {
  if (mode == MLTS_MASK_NONE) return launch<D, MLTS_MASK_NONE>(bp, st);
  if (mode == MLTS_MASK_CAUSAL) return launch<D, MLTS_MASK_CAUSAL>(bp, st);
  return launch<D, MLTS_MASK_DOC>(bp, st);
}

}  // namespace

// head_dim 64 or 128, 16-byte aligned rows (checked by the caller)
int mlts_attn_bwd_dq_bf16_tr(const AttnBwdParams& bp, int D, int mode, hipStream_t st) {
  return D == 128 ? launch_mode<128>(bp, mode, st) : launch_mode<64>(bp, mode, st);
}
