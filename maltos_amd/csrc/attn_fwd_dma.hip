// Attention forward, head_dim 64 and 128, bf16.
//
// S^T = K Q^T, P in registers, O^T = V^T P^T, eight wavefronts x 32 query rows; K and V tiles travel
// global -> LDS with the 16-byte LDS-DMA loads
// (global_load_lds_dwordx4: no staging registers, no ds_write, no VALU work) into a four-stage ring, so a
// tile's loads are issued two tiles ahead of its use.  Tiles are stored row major; V^T fragments come from
// ds_read_b64_tr_b16 (transpose-on-read), so nothing is transposed on the way in.
//
// LDS layout of a [64][128] bf16 tile: 256-byte rows of sixteen 16-byte chunks, chunk c of row r stored at
// chunk c ^ swz(r & 15), swz = swap of the two 2-bit halves.  The DMA writes LDS linearly in lane order, so
// the swizzle is applied on the GLOBAL side (lane L of a load fetches the chunk that belongs at position L).
// Measured on gfx950: ds_read_b128 over 32 consecutive rows ~220 B/clk/CU and the transpose reads
// ~150 B/clk/CU with this function (row & 15 alone gives 219 / 61).
#include "attn_common.hpp"

namespace {

constexpr int BN = 64;
constexpr int WAVES = 8;
constexpr int THREADS = WAVES * 64;
constexpr int BM = WAVES * 32;
constexpr int STAGES = 4;

template <int D>
struct FwdCfg {
  static constexpr int KS = D / 16;
  static constexpr int DB = D / 32;
  static constexpr int RB = D * 2;                     // bytes per tile row
  static constexpr int CPR = RB / 16;                  // 16-byte chunks per row
  static constexpr int TILE_BYTES = BN * RB;
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES;   // K then V
  static constexpr int META_OFF = STAGES * STAGE_BYTES;     // document masks: per stage and wavefront the visibility words
  static constexpr int META_BYTES = WAVES * 32 * 8;         // of its 32 queries against the stage's 64 keys
  static constexpr int LDS_BYTES = META_OFF + STAGES * META_BYTES;
  static constexpr int PPW = TILE_BYTES / (WAVES * 1024);  // 1 KiB pieces of each tile per wavefront (2 or 1)
  static constexpr int LOADS_PER_TILE = 2 * PPW;           // DMA instructions per wavefront per stage
};

// chunk swizzle of a tile row (depends on row & 15): 256-byte rows swap the two 2-bit halves; 128-byte rows (two rows
// per 256 bytes of banks) send row bits 1,3,2 to chunk bits 2,1,0
template <int D>
__device__ __forceinline__ int swz(int r) {
  if (D == 128) return ((r & 3) << 2) | ((r >> 2) & 3);
  return (((r >> 1) & 1) << 2) | (((r >> 3) & 1) << 1) | ((r >> 2) & 1);
}

#define MLTS_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define MLTS_GLB(p) ((const __attribute__((address_space(1))) void*)(p))

template <int N>
__device__ __forceinline__ void wait_vm_and_barrier() {
  // raw barrier: __syncthreads() would also wait for the DMA loads of the NEXT tiles (vmcnt(0))
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// LDS reads are issued through inline assembly with explicitly counted waits.  Reads the compiler knows about are
// made to wait for every outstanding LDS-DMA load (it cannot tell the ring stages apart), which would drain
// the prefetch of the next tiles in the middle of each tile.  The rule that keeps the counted waits safe whatever
// the compiler interleaves: wait_lgkm<N>(regs) is only used when N or more LGKM operations of this code
// were issued AFTER the reads that fill `regs`; LDS operations return in order, so those reads are done.
typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef int v2i32 __attribute__((ext_vector_type(2)));

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
template <int N>
__device__ __forceinline__ void wait_lgkm(v4i32& a, v4i32& b, v4i32& c, v4i32& d) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
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

// x of this lane and of lane ^ 32, without the LDS round trip of a bpermute: v_permlane32_swap exchanges the upper
// half of one register with the lower half of another
__device__ __forceinline__ void both_halves(float x, float& lo, float& hi) {
  asm("v_mov_b32 %0, %2\n\tv_mov_b32 %1, %2\n\ts_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "=&v"(lo), "=&v"(hi) : "v"(x));
}

template <int D, int MODE>
__global__ __launch_bounds__(THREADS) void attn_fwd_dma_kernel(const AttnParams p) {
  using C = FwdCfg<D>;
  constexpr int KS = C::KS, DB = C::DB, RB = C::RB, CPR = C::CPR, TILE_BYTES = C::TILE_BYTES, STAGE_BYTES = C::STAGE_BYTES,
                PPW = C::PPW, META_OFF = C::META_OFF, META_BYTES = C::META_BYTES;
  // DMA instructions per wavefront and tile; with document masks one more: 16 of the tile's 128 position / sequence ids
  constexpr int LOADS_PER_TILE = C::LOADS_PER_TILE + (MODE == MLTS_MASK_DOC ? 1 : 0);
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: everything derived from it stays scalar
  const int l32 = lane & 31, hh = lane >> 5, l16 = lane & 15;

  // Longest (last) q-tiles first across the whole grid: with causal masks the work per q-tile varies 16:1 and
  // this order keeps the tail short.  (Grouping a head's q-tiles on one XCD for L2 locality was measured: no gain
  // without a mask, 14% slower with the causal mask because of the longer tail.)
  // Document masks with grouped-query heads: the workgroup's eight wavefronts are split over 1 << pack_shift query heads
  // of one KV head, BM >> pack_shift rows of each (the same rows: the same key tiles).
  const int pack_shift = MODE == MLTS_MASK_DOC ? p.head_pack_shift : 0;
  const int rows_per_head = BM >> pack_shift;
  const int hgroups = p.Hq >> pack_shift;
  const int nbh = p.B * hgroups;
  const int bid = blockIdx.x;
  int qt = p.nqt - 1 - bid / nbh;
  const int bh = bid % nbh;
  int b = bh / hgroups;
  if constexpr (MODE == MLTS_MASK_DOC) {
    // document masks: the (query block, batch row) pairs are walked in the order of their work, most first
    if (p.qblock_order) {
      const int e = p.qblock_order[(bid / nbh) * p.B + b];
      qt = e / p.B;
      b = e % p.B;
    }
  }
  const int hq = ((bh % hgroups) << pack_shift) + ((wave * 32) >> (8 - pack_shift));
  const int hkv = hq / (p.Hq / p.Hkv);
  const int q0 = qt * rows_per_head;
  const int wq0 = q0 + ((wave * 32) & (rows_per_head - 1));
  const int qrow = wq0 + l32;

  const bf16_t* Q = static_cast<const bf16_t*>(p.q) + b * p.qs[0] + hq * p.qs[1];
  const bf16_t* K = static_cast<const bf16_t*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const bf16_t* V = static_cast<const bf16_t*>(p.v) + b * p.vs[0] + hkv * p.vs[1];
  bf16_t* O = static_cast<bf16_t*>(p.o) + b * p.os[0] + hq * p.os[1];

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
  // needed tiles in increasing order: one cursor for the loader (two tiles ahead), one for the consumer
  DocTileScan scan_load, scan_use;
  const int4* k_stats_row = MODE == MLTS_MASK_DOC ? p.k_stats + static_cast<int64_t>(b) * p.nk_stats : nullptr;
  auto next_tile = [&](DocTileScan& sc, int j) -> int {
    if (MODE != MLTS_MASK_DOC) return j < j_end ? j : j_end;
    return doc_scan_next<BM / 64, true>(sc, j, j_end, p.nk_stats, k_stats_row, bq_stats, wq_stats, lane);
  };

  // ---- DMA loader: this wavefront moves PPW 1 KiB pieces of the K tile and of the V tile; piece n holds rows
  // n * 64 / CPR ..; lane L -> row n * 64 / CPR + L / CPR, stored chunk L % CPR, source chunk (L % CPR) ^ swz(row) ----
  // Addresses are a wave-uniform tile base (scalar arithmetic) plus a tile-invariant lane offset, so a tile's loads cost
  // four instructions and almost no vector arithmetic; only a tile that reaches past Sk clamps its rows.
  int ld_row[PPW], ld_col[PPW];
  uint32_t ld_koff[PPW], ld_voff[PPW];
#pragma unroll
  for (int n = 0; n < PPW; ++n) {
    const int row = (wave * PPW + n) * (64 / CPR) + lane / CPR;
    ld_row[n] = row;
    ld_col[n] = ((lane % CPR) ^ swz<D>(row & 15)) * 8;
    ld_koff[n] = static_cast<uint32_t>(row * static_cast<int>(p.ks[2]) + ld_col[n]) * 2u;
    ld_voff[n] = static_cast<uint32_t>(row * static_cast<int>(p.vs[2]) + ld_col[n]) * 2u;
  }
  const unsigned char* Kb = reinterpret_cast<const unsigned char*>(K);
  const unsigned char* Vb = reinterpret_cast<const unsigned char*>(V);
  auto issue_tile = [&](int j, int stage) {
    const int kv0 = j * BN;
    unsigned char* sbase = smem + stage * STAGE_BYTES + wave * PPW * 1024;
    if (MODE == MLTS_MASK_DOC) {
      // the visibility words of this wavefront's 32 queries against the tile's keys (256 bytes; read only if the pair is
      // one whose words the pre-pass wrote, i.e. if the wavefront masks the tile)
      if (lane < 16) {
        const int g = min(wq0 >> 6, p.nq_stats - 1);
        const unsigned long long* src =
            p.doc_bits + ((static_cast<int64_t>(b) * p.nq_stats + g) * p.nk_stats + j) * 64 + (wq0 & 32) + lane * 2;
        __builtin_amdgcn_global_load_lds(MLTS_GLB(src), MLTS_LDS(smem + META_OFF + stage * META_BYTES + wave * 256), 16, 0, 0);
      }
    }
    if (kv0 + BN <= p.Sk) {
      const unsigned char* kt = Kb + static_cast<int64_t>(kv0) * p.ks[2] * 2;
      const unsigned char* vt = Vb + static_cast<int64_t>(kv0) * p.vs[2] * 2;
#pragma unroll
      for (int n = 0; n < PPW; ++n) {
        __builtin_amdgcn_global_load_lds(MLTS_GLB(kt + ld_koff[n]), MLTS_LDS(sbase + n * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(MLTS_GLB(vt + ld_voff[n]), MLTS_LDS(sbase + TILE_BYTES + n * 1024), 16, 0, 0);
      }
    } else {
#pragma unroll
      for (int n = 0; n < PPW; ++n) {
        const int r = min(kv0 + ld_row[n], p.Sk - 1);  // rows past the end repeat the last key; their scores are masked
        const bf16_t* ksrc = K + static_cast<int64_t>(r) * p.ks[2] + ld_col[n];
        const bf16_t* vsrc = V + static_cast<int64_t>(r) * p.vs[2] + ld_col[n];
        __builtin_amdgcn_global_load_lds(MLTS_GLB(ksrc), MLTS_LDS(sbase + n * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(MLTS_GLB(vsrc), MLTS_LDS(sbase + TILE_BYTES + n * 1024), 16, 0, 0);
      }
    }
  };

  // ---- per-lane LDS read offsets (tile invariant) ----
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(MLTS_LDS(smem)));
  int koff[KS];   // K fragment (A operand of S^T): row l32 (+32 kb), chunk 2 ks + hh
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff[ks] = l32 * RB + (((ks * 2 + hh) ^ swz<D>(l32 & 15)) << 4);
  int voff[2][DB];  // V^T fragment halves: key row 16 c + 8 part + 4 hh + l16/4, columns 32 db + 16 (l32/16) + 4 (l16%4)
#pragma unroll
  for (int part = 0; part < 2; ++part) {
    const int rlow = part * 8 + hh * 4 + (l16 >> 2);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int col = db * 32 + (l32 >> 4) * 16 + (l16 & 3) * 4;
      voff[part][db] = rlow * RB + (((col >> 3) ^ swz<D>(rlow)) << 4) + ((col >> 2) & 1) * 8;
    }
  }

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- tile pipeline ----
  // Per wavefront the phases of the tile stream are ... PV(t-1) QK(t) | SM(t) PV(t) QK(t+1) | SM(t+1) ...: one block
  // of MFMA work (PV of the previous tile, then QK of this one) and one block of VALU work (softmax).  A SIMD hosts
  // two wavefronts of the workgroup, w and w + 4; the workgroup barrier sits before the MFMA block in w < 4 and
  // before the VALU block in w >= 4, so that the two run half a tile apart and one does softmax while the other
  // keeps the matrix cores busy.  sync() number k (k = 0, 1, ...) means "the k-th needed tile has landed everywhere";
  // the load of tile k + 2 is issued right behind it into ring stage (k + 2) % 4, which held tile k - 2: the early
  // wavefronts finished it two syncs ago, the late ones read its V before their QK(k - 1), i.e. before this sync.
  const bool late = wave >= WAVES / 2;
  int inflight = 0, istage = 0;
  int ji = next_tile(scan_load, 0);
  auto issue_next = [&]() {
    if (ji < j_end) {
      issue_tile(ji, istage);
      istage = (istage + 1) & (STAGES - 1);
      ji = next_tile(scan_load, ji + 1);
      ++inflight;
    }
  };
  auto sync = [&]() {
    if (inflight >= 2) wait_vm_and_barrier<LOADS_PER_TILE>();  // oldest tile landed; the next may still be in flight
    else wait_vm_and_barrier<0>();
    --inflight;
    issue_next();
  };
  // ---- Q: this wavefront's 32 rows travel like a K tile (whole rows by LDS-DMA, same row layout and swizzle) into the
  // ring stages that the first two tiles do not use, and come back as B-operand fragments with one ds_read_b128 each.
  // (A fragment gathered straight from global memory touches 32 cache lines per instruction: eight such loads per
  // wavefront took most of the time before the first tile.)  Rows past the end repeat the last row; they are never
  // stored.  Every wavefront reads its fragments before its first sync(), whose barrier therefore also says that
  // stages 2 and 3 are free for tiles 2 and 3. ----
  bf16x8 qf[KS];
  {
    constexpr int QP = 32 * RB / 1024;  // 1 KiB pieces of this wavefront's rows
    unsigned char* qbase = smem + 2 * STAGE_BYTES + wave * (32 * RB);
#pragma unroll
    for (int n = 0; n < QP; ++n) {
      const int row = n * (64 / CPR) + lane / CPR;
      const int col = ((lane % CPR) ^ swz<D>(row & 15)) * 8;
      const int r = min(wq0 + row, p.Sq - 1);
      __builtin_amdgcn_global_load_lds(MLTS_GLB(Q + static_cast<int64_t>(r) * p.qs[2] + col), MLTS_LDS(qbase + n * 1024), 16, 0, 0);
    }
    issue_next();
    issue_next();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    v4i32 qraw[KS];
    const uint32_t qa = lds0 + 2 * STAGE_BYTES + wave * (32 * RB);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qraw[ks] = lds_read_b128<0>(qa + koff[ks]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      asm volatile("" : "+v"(qraw[ks]));  // the fragments are used only behind the wait above
      qf[ks] = as_frag(qraw[ks]);
    }
  }

  f32x16 sacc[2];
  bf16x8 pf[4];
  bool pv_pending = false;
  int pv_stage = 0;

  auto pv_phase = [&]() {
      {
        // V^T fragments of one 16-key step: eight transpose reads (4 head-dim blocks x 2 halves); two steps in flight
        const uint32_t sb = lds0 + pv_stage * STAGE_BYTES;
        uint32_t va[2][DB];
#pragma unroll
        for (int part = 0; part < 2; ++part)
#pragma unroll
          for (int db = 0; db < DB; ++db) va[part][db] = sb + voff[part][db];
        v2i32 h0[8], h1[8];
        // a group = eight transpose reads / four MFMAs: one 16-key step c (head_dim 128, four column blocks) or the
        // two steps c, c + 1 (head_dim 64, two column blocks each)
#define MLTS_VREAD8(dst, CS)                                                                   \
  dst[0] = lds_read_tr16_b64<TILE_BYTES + ((CS) + 0 / DB) * 16 * RB>(va[0][0 % DB]);           \
  dst[1] = lds_read_tr16_b64<TILE_BYTES + ((CS) + 0 / DB) * 16 * RB>(va[1][0 % DB]);           \
  dst[2] = lds_read_tr16_b64<TILE_BYTES + ((CS) + 1 / DB) * 16 * RB>(va[0][1 % DB]);           \
  dst[3] = lds_read_tr16_b64<TILE_BYTES + ((CS) + 1 / DB) * 16 * RB>(va[1][1 % DB]);           \
  dst[4] = lds_read_tr16_b64<TILE_BYTES + ((CS) + 2 / DB) * 16 * RB>(va[0][2 % DB]);           \
  dst[5] = lds_read_tr16_b64<TILE_BYTES + ((CS) + 2 / DB) * 16 * RB>(va[1][2 % DB]);           \
  dst[6] = lds_read_tr16_b64<TILE_BYTES + ((CS) + 3 / DB) * 16 * RB>(va[0][3 % DB]);           \
  dst[7] = lds_read_tr16_b64<TILE_BYTES + ((CS) + 3 / DB) * 16 * RB>(va[1][3 % DB]);
#define MLTS_VMFMA4(src, CS)                                                                                 \
  _Pragma("unroll") for (int u = 0; u < 4; ++u) oacc[u % DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(      \
      as_frag(src[2 * u], src[2 * u + 1]), pf[(CS) + u / DB], oacc[u % DB], 0, 0, 0);
        if constexpr (D == 128) {
          MLTS_VREAD8(h0, 0)
          MLTS_VREAD8(h1, 1)
          wait_lgkm<8>(h0);
          MLTS_VMFMA4(h0, 0)
          MLTS_VREAD8(h0, 2)
          wait_lgkm<8>(h1);
          MLTS_VMFMA4(h1, 1)
          MLTS_VREAD8(h1, 3)
          wait_lgkm<8>(h0);
          MLTS_VMFMA4(h0, 2)
          wait_lgkm<0>(h1);
          MLTS_VMFMA4(h1, 3)
        } else {
          MLTS_VREAD8(h0, 0)
          MLTS_VREAD8(h1, 2)
          wait_lgkm<8>(h0);
          MLTS_VMFMA4(h0, 0)
          wait_lgkm<0>(h1);
          MLTS_VMFMA4(h1, 2)
        }
#undef MLTS_VREAD8
#undef MLTS_VMFMA4
      }
  };

  int j = next_tile(scan_use, 0);
  int stage = 0;
  if (late && j < j_end) sync();
  while (j < j_end) {
    const int doc_cls = MODE == MLTS_MASK_DOC ? doc_scan_class(scan_use, j) : TILE_FULL;  // before the scan moves on
    const int jn = next_tile(scan_use, j + 1);
    if (!late) sync();
    __builtin_amdgcn_s_setprio(1);  // the matrix block of this wavefront goes ahead of the other wavefront's softmax
    if (pv_pending) pv_phase();

    const int kv0 = j * BN;
    int cls = TILE_FULL;
    if (MODE == MLTS_MASK_CAUSAL) {
      if (kv0 > wave_last_q + p.causal_off) cls = TILE_SKIP;
      else if (kv0 + BN - 1 > wq0 + p.causal_off) cls = TILE_MASKED;
    } else if (MODE == MLTS_MASK_DOC) {
      cls = doc_cls;
    }
    if (cls == TILE_FULL && kv0 + BN > p.Sk) cls = TILE_MASKED;
    if (wq0 >= p.Sq) cls = TILE_SKIP;

    if (cls != TILE_SKIP) {
      const uint32_t sb = lds0 + stage * STAGE_BYTES;
      uint32_t ka[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ka[ks] = sb + koff[ks];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) sacc[kb][e] = 0.f;
      {
        // sixteen K fragments in four groups of four, two groups in flight
        v4i32 g0[4], g1[4];
#define MLTS_KREAD4(dst, KB, KS0)                                   \
  dst[0] = lds_read_b128<(KB) * 32 * RB>(ka[(KS0) + 0]);               \
  dst[1] = lds_read_b128<(KB) * 32 * RB>(ka[(KS0) + 1]);               \
  dst[2] = lds_read_b128<(KB) * 32 * RB>(ka[(KS0) + 2]);               \
  dst[3] = lds_read_b128<(KB) * 32 * RB>(ka[(KS0) + 3]);
#define MLTS_KMFMA4(src, KB, KS0)                                                                              \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) sacc[KB] =                                                     \
      __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(src[i]), qf[(KS0) + i], sacc[KB], 0, 0, 0);
        if constexpr (D == 128) {
          MLTS_KREAD4(g0, 0, 0)
          MLTS_KREAD4(g1, 0, 4)
          wait_lgkm<4>(g0[0], g0[1], g0[2], g0[3]);
          MLTS_KMFMA4(g0, 0, 0)
          MLTS_KREAD4(g0, 1, 0)
          wait_lgkm<4>(g1[0], g1[1], g1[2], g1[3]);
          MLTS_KMFMA4(g1, 0, 4)
          MLTS_KREAD4(g1, 1, 4)
          wait_lgkm<4>(g0[0], g0[1], g0[2], g0[3]);
          MLTS_KMFMA4(g0, 1, 0)
          wait_lgkm<0>(g1[0], g1[1], g1[2], g1[3]);
          MLTS_KMFMA4(g1, 1, 4)
        } else {
          MLTS_KREAD4(g0, 0, 0)
          MLTS_KREAD4(g1, 1, 0)
          wait_lgkm<4>(g0[0], g0[1], g0[2], g0[3]);
          MLTS_KMFMA4(g0, 0, 0)
          wait_lgkm<0>(g1[0], g1[1], g1[2], g1[3]);
          MLTS_KMFMA4(g1, 1, 0)
        }
#undef MLTS_KREAD4
#undef MLTS_KMFMA4
      }

    }
    __builtin_amdgcn_s_setprio(0);
    if (late && jn < j_end) sync();
    if (cls != TILE_SKIP) {
      if (cls == TILE_MASKED) {
        if constexpr (MODE == MLTS_MASK_DOC) {
          // this query's visibility bits of the tile's 64 keys (formed once per call by the pre-pass): score register
          // (kb, g, r) <-> key kb * 32 + g * 8 + hh * 4 + r, so after a shift by hh * 4 the bit positions are constants
          v2i32 wraw;
          asm volatile("ds_read_b64 %0, %1" : "=v"(wraw) : "v"(lds0 + META_OFF + stage * META_BYTES + wave * 256 + l32 * 8));
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wraw));
          const unsigned long long wsh =
              ((static_cast<unsigned long long>(static_cast<unsigned>(wraw[1])) << 32) | static_cast<unsigned>(wraw[0])) >> (hh * 4);
          const int wlo = static_cast<int>(wsh), whi = static_cast<int>(wsh >> 32);
          typedef int i32x16 __attribute__((ext_vector_type(16)));
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) {
            // whole-vector casts: casting single elements of an MFMA result is miscompiled (element 0 is broadcast)
            i32x16 si = __builtin_bit_cast(i32x16, sacc[kb]);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const int bit = (e >> 2) * 8 + (e & 3);
              const int keep = __builtin_amdgcn_sbfe(kb ? whi : wlo, bit, 1);  // all ones if visible
              si[e] = (keep & si[e]) | (~keep & static_cast<int>(0xff800000u));
            }
            sacc[kb] = __builtin_bit_cast(f32x16, si);
          }
        } else {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const int kbase = kv0 + kb * 32 + g * 8 + hh * 4;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int kj = kbase + r;
                bool vis = kj < p.Sk;
                if (MODE == MLTS_MASK_CAUSAL) vis = vis && (kj <= qrow + p.causal_off);
                if (!vis) sacc[kb][g * 4 + r] = -INFINITY;
              }
            }
          }
        }
      }

      // online softmax; the running maximum is only raised when it grows by more than 2^8 (the result is
      // exact either way: l and O carry the same stale scale), so the O rescale is rare after the first tiles
      float mx = sacc[0][0];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sacc[kb][e]);
      {
        float mlo, mhi;
        both_halves(mx, mlo, mhi);
        mx = fmaxf(mlo, mhi) * p.scale_log2;
      }
      const bool raise = mx > m_run + 8.0f;  // also true for the first visible tile (m_run = -inf)
      if (__builtin_amdgcn_ballot_w64(raise) != 0) {
        const float m_new = raise ? mx : m_run;
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);  // 1 for lanes that do not raise; 0 from -inf
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int e = 0; e < 16; ++e) oacc[db][e] *= alpha;
      }
      const float m_use = m_run == -INFINITY ? 0.f : m_run;
      if constexpr (D == 64) {
        // probabilities in pairs: one packed conversion per pair.  The row sum is taken over the fp32 values, not over
        // the bf16 ones that enter the PV product: a dot product of each converted pair with (1, 1) is one instruction
        // less per pair, but a bf16 value is off by up to 2^-8 of itself, and in a row that a few keys dominate that
        // error goes straight into LSE (up to 4e-3, where the fp32 sum keeps it near 1e-6)
        float ls4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            v4i32 w;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              f32x2 pv;
              pv[0] = __builtin_amdgcn_exp2f(sacc[kb][t * 8 + 2 * i] * p.scale_log2 - m_use);
              pv[1] = __builtin_amdgcn_exp2f(sacc[kb][t * 8 + 2 * i + 1] * p.scale_log2 - m_use);
              const bf16x2 pb = __builtin_convertvector(pv, bf16x2);
              ls4[i] += pv[0] + pv[1];
              w[i] = __builtin_bit_cast(int, pb);
            }
            pf[kb * 2 + t] = __builtin_bit_cast(bf16x8, w);
          }
        l_run += (ls4[0] + ls4[1]) + (ls4[2] + ls4[3]);
      } else {
        float ls = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              const float pv = __builtin_amdgcn_exp2f(sacc[kb][t * 8 + i] * p.scale_log2 - m_use);
              ls += pv;
              pf[kb * 2 + t][i] = static_cast<bf16_t>(pv);
            }
        l_run += ls;
      }

    }
    pv_pending = cls != TILE_SKIP;
    pv_stage = stage;
    j = jn;
    stage = (stage + 1) & (STAGES - 1);
  }
  if (pv_pending) pv_phase();

  float l_lo, l_hi;
  both_halves(l_run, l_lo, l_hi);
  const float l_tot = l_lo + l_hi;
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (qrow < p.Sq && hh == 0) {
    p.lse[(static_cast<int64_t>(b) * p.Hq + hq) * p.Sq + qrow] =
        l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
  }
  const bool rows16 = ((p.os[0] | p.os[1] | p.os[2]) & 7) == 0 && (reinterpret_cast<uintptr_t>(p.o) & 15) == 0;
  if (rows16) {
    // rows through LDS (each wavefront owns 32 rows x RB bytes, tile-row swizzle), so that global stores are 16 bytes
    // per lane and cover whole rows
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // nobody reads a K/V tile any more
    unsigned char* ebase = smem + wave * (32 * RB);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = static_cast<bf16_t>(oacc[db][g * 4 + r] * inv);
        *reinterpret_cast<bf16x4*>(ebase + l32 * RB + (((db * 4 + g) ^ swz<D>(l32 & 15)) << 4) + hh * 8) = w;
      }
    }
#pragma unroll
    for (int i = 0; i < 32 * CPR / 64; ++i) {
      const int idx = i * 64 + lane;
      const int row = idx / CPR, chunk = idx % CPR;
      const v4i32 x = *reinterpret_cast<const v4i32*>(ebase + row * RB + ((chunk ^ swz<D>(row & 15)) << 4));
      if (wq0 + row < p.Sq) *reinterpret_cast<v4i32*>(O + static_cast<int64_t>(wq0 + row) * p.os[2] + chunk * 8) = x;
    }
  } else if (qrow < p.Sq) {
    bf16_t* orow = O + static_cast<int64_t>(qrow) * p.os[2];
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = static_cast<bf16_t>(oacc[db][g * 4 + r] * inv);
        *reinterpret_cast<bf16x4*>(orow + db * 32 + g * 8 + hh * 4) = w;
      }
    }
  }
}

template <int D, int MODE>
int launch(AttnParams p, hipStream_t st) {
  auto kern = attn_fwd_dma_kernel<D, MODE>;
  constexpr int lds_bytes = FwdCfg<D>::LDS_BYTES;
  static MltsLdsOptIn lds_opt_in;
  if (hipError_t e = lds_opt_in.reserve(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) {
    mlts_set_error("mlts_attn_fwd: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    return MLTS_ERR_LAUNCH;
  }
  if (MODE != MLTS_MASK_DOC) p.head_pack_shift = 0;  // (set with the block order by the caller's pre-pass otherwise)
  const int rows = BM >> p.head_pack_shift;
  p.nqt = (p.Sq + rows - 1) / rows;
  const int64_t blocks = static_cast<int64_t>(p.nqt) * p.B * (p.Hq >> p.head_pack_shift);
  {
    MltsKernelTimer timer("attn_fwd", st);
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(THREADS), lds_bytes, st, p);
  }
  return mlts_check_launch("mlts_attn_fwd");
}

template <int D>
int launch_mode(const AttnParams& p, int mode, hipStream_t st) {
  if (mode == MLTS_MASK_NONE) return launch<D, MLTS_MASK_NONE>(p, st);
  if (mode == MLTS_MASK_CAUSAL) return launch<D, MLTS_MASK_CAUSAL>(p, st);
  return launch<D, MLTS_MASK_DOC>(p, st);
}

}  // namespace

// Requires head_dim 64 or 128, Sk >= 1 and 16-byte aligned rows (checked by the caller).
int mlts_attn_fwd_bf16_dma(const AttnParams& p, int D, int mode, hipStream_t st) {
  return D == 128 ? launch_mode<128>(p, mode, st) : launch_mode<64>(p, mode, st);
}
