// Attention backward, dQ from the -dS blocks that the dK/dV kernel hands over, head_dim 128, bf16.
//
// The two-kernel backward computes the scores twice (once per kernel).  When the caller's workspace has room for
// -dS (bf16, one value per visible (query, key) pair), the dK/dV kernel stores it and this kernel only does
//     -dQ^T += K^T (-dS^T)          A = K^T and B = -dS^T, both by ds_read_b64_tr_b16 from row-major LDS tiles
// which is one matrix product instead of three; it is bound by the HBM read of -dS (about 2 bytes per visible pair),
// not by the matrix cores.  A workgroup of 8 wavefronts owns 256 query rows of one (batch, head), each wavefront 32
// of them, and walks the visible keys in tiles of 64.
//
// -dS arrives in 4 KiB blocks (32 keys x 64 queries, layout at AttnBwdParams::ds_ws): 16-byte units (fragment f,
// key, hh) that hold eight queries of one key.  A unit is written to LDS as it is, at row = key, 16-byte slot
// 8 (tile & 1) + 2 f + hh of a [64 keys][128 slots] sub-tile (two sub-tiles side by side cover the 256 queries), so a
// lane's column in LDS is a SLOT, not a query: slot s of a 64-query tile is query 16 (s / 16) + 8 ((s / 4) % 2) +
// 4 ((s / 8) % 2) + s % 4.  The permutation only matters where rows are named: in the epilogue.  Blocks that were
// not written (above the causal diagonal, past the end) are replaced by zeros.
//
// K tiles and -dS tiles are fetched into registers right behind the barrier and written to a two-stage LDS ring
// after the work on the current tile, as in attn_bwd_dq_tr.hip.
#include "attn_common.hpp"
#include <type_traits>

namespace {

constexpr int BN = 64;
constexpr int WAVES = 8;
constexpr int THREADS = WAVES * 64;
constexpr int BM = WAVES * 32;
constexpr int STAGES = 2;
constexpr int SUB_ROW = 256;                   // bytes per row of a -dS sub-tile (128 slots)
constexpr int SUB_BYTES = BN * SUB_ROW;        // 16 KiB
constexpr int DS_TILE_BYTES = 2 * SUB_BYTES;   // 64 keys x 256 slots
constexpr int NDS = DS_TILE_BYTES / 16 / THREADS;  // 16-byte units per thread and tile (4)

template <int D>
struct DsCfg {
  static constexpr int DB = D / 32;
  static constexpr int RB = D * 2;                     // bytes per K tile row
  static constexpr int CPR = RB / 16;
  static constexpr int K_TILE_BYTES = BN * RB;
  static constexpr int STAGE_BYTES = DS_TILE_BYTES + K_TILE_BYTES;   // -dS then K
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;             // >= 8 x 32 rows x RB of the epilogue
  static constexpr int NLD = BN * CPR / THREADS;       // 16-byte chunks of K per thread and tile (2 or 1)
};

typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef int v2i32 __attribute__((ext_vector_type(2)));

// chunk swizzle of a tile row (see attn_bwd_split.hip)
template <int D>
__device__ __forceinline__ int swz(int r) {
  if (D == 128) return ((r & 3) << 2) | ((r >> 2) & 3);
  return (((r >> 1) & 1) << 2) | (((r >> 3) & 1) << 1) | ((r >> 2) & 1);
}

#define MLTS_LDS(p) ((__attribute__((address_space(3))) void*)(p))

__device__ __forceinline__ void drain_and_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

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
// (the registers are operands of the wait, so that the compiler cannot touch them before it)
template <int N>
__device__ __forceinline__ void wait_lgkm(v2i32 (&x)[10]) {
  asm volatile("s_waitcnt lgkmcnt(%10)"
               : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]), "+v"(x[8]),
                 "+v"(x[9])
               : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_lgkm(v2i32 (&x)[6]) {
  asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]) : "n"(N));
}
__device__ __forceinline__ bf16x8 as_frag(v2i32 lo, v2i32 hi) {
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3));
}

// query (within its 64-row tile) of LDS slot s
__device__ __forceinline__ int slot_query(int s) { return (s & 48) + ((s >> 2) & 1) * 8 + ((s >> 3) & 1) * 4 + (s & 3); }

template <int D, bool CAUSAL>
__global__ __launch_bounds__(THREADS) void attn_bwd_dq_ds_kernel(const AttnBwdParams bp) {
  using C = DsCfg<D>;
  constexpr int DB = C::DB, RB = C::RB, CPR = C::CPR, STAGE_BYTES = C::STAGE_BYTES, NLD = C::NLD;
  const AttnParams& p = bp.a;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5, l16 = lane & 15;
  const int nbh = p.B * p.Hq;
  const int bid = blockIdx.x;
  const int qt = p.nqt - 1 - bid / nbh;  // longest (last) q-tiles first under a causal mask
  const int bh = bid % nbh;
  const int b = bh / p.Hq, hq = bh % p.Hq;
  const int hkv = hq / (p.Hq / p.Hkv);
  const int q0 = qt * BM;
  const int wq0 = q0 + wave * 32;

  const bf16_t* K = static_cast<const bf16_t*>(p.k) + b * p.ks[0] + hkv * p.ks[1];
  const unsigned char* ds_head = static_cast<const unsigned char*>(bp.ds_ws) + static_cast<int64_t>(bh) * bp.ds_nkb * bp.ds_nqt * 4096;

  const int nkt = (p.Sk + BN - 1) / BN;
  int j_end = nkt;
  if (CAUSAL) {
    const int lim = min(q0 + BM, p.Sq) - 1 + p.causal_off;
    j_end = lim < 0 ? 0 : min(nkt, lim / BN + 1);
  }
  const int wave_last_q = min(wq0 + 31, p.Sq - 1);

  // ---- tile loader.  K: chunks t (and t + 512) of the tile, chunk c = row c / CPR, stored slot c % CPR, source slot
  // (c % CPR) ^ swz(row); rows past the end are stored as zeros.  -dS: units u = t + 512 n; block u / 256 = 4 (32-key half) +
  // 64-query tile is the same for a whole wavefront, so "was it written" is a scalar branch ----
  int ld_row[NLD], ld_col[NLD];
  uint32_t ld_koff[NLD];
#pragma unroll
  for (int n = 0; n < NLD; ++n) {
    const int c = tid + n * THREADS;
    ld_row[n] = c / CPR;
    ld_col[n] = ((c % CPR) ^ swz<D>((c / CPR) & 15)) * 8;
    ld_koff[n] = (static_cast<uint32_t>(ld_row[n]) * static_cast<uint32_t>(p.ks[2]) + ld_col[n]) * 2;  // bytes
  }
  const int wave4 = __builtin_amdgcn_readfirstlane(wave >> 2);
  uint32_t ds_dst[NDS];  // LDS byte offset of unit n inside the -dS tile
#pragma unroll
  for (int n = 0; n < NDS; ++n) {
    const int u = tid + n * THREADS;
    const int blk = u >> 8, f = (u >> 6) & 3;
    const int row = (blk >> 2) * 32 + l32;
    const int chunk = (blk & 1) * 8 + 2 * f + hh;
    ds_dst[n] = ((blk >> 1) & 1) * SUB_BYTES + row * SUB_ROW + ((chunk ^ swz<128>(row & 15)) << 4);
  }
  // two register sets: the kernel is bound by the HBM read of -dS, so two tiles are kept in flight
  v4i32 ka[NLD], sa[NDS], kb[NLD], sb[NDS];
  // Loads are unconditional (clamped addresses) and what must read as zero is cleared at the store: with a load
  // inside a branch the compiler waits for every outstanding load, not only for the older tile's.
  auto stage_load = [&](int j, v4i32 (&stg_k)[NLD], v4i32 (&stg_s)[NDS]) {
    const int kv0 = j * BN;
    const unsigned char* Kt = reinterpret_cast<const unsigned char*>(K + static_cast<int64_t>(kv0) * p.ks[2]);
    const int last = p.Sk - 1 - kv0;
#pragma unroll
    for (int n = 0; n < NLD; ++n) {
      uint32_t ko = ld_koff[n];
      if (last < BN - 1) ko = (static_cast<uint32_t>(min(ld_row[n], last)) * static_cast<uint32_t>(p.ks[2]) + ld_col[n]) * 2;
      stg_k[n] = *reinterpret_cast<const v4i32*>(Kt + ko);
    }
#pragma unroll
    for (int n = 0; n < NDS; ++n) {
      const int blk = wave4 + 2 * n;  // = (tid + 512 n) / 256
      const int kb32 = min(2 * j + (blk >> 2), bp.ds_nkb - 1), qt64 = min(4 * qt + (blk & 3), bp.ds_nqt - 1);
      const unsigned char* src = ds_head + (static_cast<int64_t>(kb32) * bp.ds_nqt + qt64) * 4096;
      stg_s[n] = __builtin_nontemporal_load(reinterpret_cast<const v4i32*>(src + (tid & 255) * 16));  // read once
    }
  };
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(MLTS_LDS(smem)));
  auto stage_store = [&](int j, v4i32 (&stg_k)[NLD], v4i32 (&stg_s)[NDS]) {  // tile j into stage j % 2
    const uint32_t sb_ = lds0 + (j & 1) * STAGE_BYTES;
#pragma unroll
    for (int n = 0; n < NDS; ++n) {
      const int blk = wave4 + 2 * n;
      if (!mlts_ds_block_written(2 * j + (blk >> 2), 4 * qt + (blk & 3), p.Sq, p.Sk, p.causal_off, CAUSAL)) stg_s[n] = v4i32{0, 0, 0, 0};
      lds_write_b128<0>(sb_ + ds_dst[n], stg_s[n]);
    }
    const uint32_t a = sb_ + DS_TILE_BYTES + tid * 16;
#pragma unroll
    for (int n = 0; n < NLD; ++n) {
      if (j * BN + ld_row[n] >= p.Sk) stg_k[n] = v4i32{0, 0, 0, 0};  // keys past the end
      lds_write_b128<0>(a + n * (THREADS * 16), stg_k[n]);
    }
  };

  // ---- per-lane LDS read offsets (stage 0; the 16-key step is an instruction offset): transposed fragment halves,
  // key row 16 c + 8 part + 4 hh + l16/4, columns 32 blk + 16 (l32/16) + 4 (l16%4) ----
  uint32_t ta_s[2], ta_k[2][DB];
#pragma unroll
  for (int part = 0; part < 2; ++part) {
    const int rlow = part * 8 + hh * 4 + (l16 >> 2);
    const int cs = (wave & 3) * 32 + (l32 >> 4) * 16 + (l16 & 3) * 4;
    ta_s[part] = lds0 + (wave >> 2) * SUB_BYTES + rlow * SUB_ROW + (((cs >> 3) ^ swz<128>(rlow)) << 4) + ((cs >> 2) & 1) * 8;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int col = db * 32 + (l32 >> 4) * 16 + (l16 & 3) * 4;
      ta_k[part][db] = lds0 + DS_TILE_BYTES + rlow * RB + (((col >> 3) ^ swz<D>(rlow)) << 4) + ((col >> 2) & 1) * 8;
    }
  }

  f32x16 dqacc[DB];  // -dQ^T / scale: register e <-> head-dim 32 db + 8 (e/4) + 4 hh + e%4, lane -> slot 32 wave + l32
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) dqacc[db][e] = 0.f;

  constexpr int NR = 2 + 2 * DB;  // transposed reads of one 16-key step: -dS halves, then K^T halves per column block
#define MLTS_STEP_READ(dst, C)                                           \
  dst[0] = lds_read_tr16_b64<(C) * 16 * SUB_ROW>(ta_s[0] + so);          \
  dst[1] = lds_read_tr16_b64<(C) * 16 * SUB_ROW>(ta_s[1] + so);          \
  _Pragma("unroll") for (int db = 0; db < DB; ++db) {                    \
    dst[2 + 2 * db] = lds_read_tr16_b64<(C) * 16 * RB>(ta_k[0][db] + so);     \
    dst[3 + 2 * db] = lds_read_tr16_b64<(C) * 16 * RB>(ta_k[1][db] + so);     \
  }
#define MLTS_STEP_MFMA(src)                                                                                         \
  _Pragma("unroll") for (int db = 0; db < DB; ++db) dqacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(            \
      as_frag(src[2 + 2 * db], src[3 + 2 * db]), as_frag(src[0], src[1]), dqacc[db], 0, 0, 0);
  auto process_tile = [&](const uint32_t so) {
    v2i32 r0[NR], r1[NR];
    MLTS_STEP_READ(r0, 0)
    MLTS_STEP_READ(r1, 1)
    wait_lgkm<NR>(r0);
    MLTS_STEP_MFMA(r0)
    MLTS_STEP_READ(r0, 2)
    wait_lgkm<NR>(r1);
    MLTS_STEP_MFMA(r1)
    MLTS_STEP_READ(r1, 3)
    wait_lgkm<NR>(r0);
    MLTS_STEP_MFMA(r0)
    wait_lgkm<0>(r1);
    MLTS_STEP_MFMA(r1)
  };
#undef MLTS_STEP_READ
#undef MLTS_STEP_MFMA

  // ---- tile loop, two tiles per trip.  Barrier k: tile k is in LDS stage k % 2 and tile k + 1 is on its way into
  // one register set; tile k + 2 is fetched into the other set, then tile k is worked on, then tile k + 1 is written
  // to the other stage (read last during tile k - 1). ----
  {
    // keys past this wavefront's last query hold zeros only
    auto skip = [&](int j) { return wq0 >= p.Sq || (CAUSAL && j * BN > wave_last_q + p.causal_off); };
    // (loads past the last tile repeat it and are never stored: a load under a branch would make every wait of the
    // loop a wait for all outstanding loads)
    if (j_end > 0) {
      stage_load(0, ka, sa);
      stage_load(min(1, j_end - 1), kb, sb);
      stage_store(0, ka, sa);
    }
    int j = 0;
    while (j < j_end) {
      drain_and_barrier();
      stage_load(min(j + 2, j_end - 1), ka, sa);
      if (!skip(j)) process_tile(0);
      if (j + 1 < j_end) stage_store(j + 1, kb, sb);
      if (++j >= j_end) break;
      drain_and_barrier();
      stage_load(min(j + 2, j_end - 1), kb, sb);
      if (!skip(j)) process_tile(STAGE_BYTES);
      if (j + 1 < j_end) stage_store(j + 1, ka, sa);
      ++j;
    }
  }

  // ---- dQ rows: lane l32 of this wavefront holds slot 32 wave + l32 ----
  const float oscale = -p.scale;  // the accumulator holds K^T (-dS^T)
  const int tile_q0 = q0 + (wave >> 1) * 64;
  const bool rows16 = ((bp.dqs[0] | bp.dqs[1] | bp.dqs[2]) & 7) == 0 && (reinterpret_cast<uintptr_t>(bp.dq_acc) & 15) == 0;
  if (!bp.accumulate_f32 && rows16) {
    // bf16 rows through LDS (each wavefront owns 32 rows x RB bytes, tile-row swizzle), so that global stores are
    // 16 bytes per lane and cover whole rows
    drain_and_barrier();  // every wavefront has finished reading the last tile
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
      const int qrow = tile_q0 + slot_query((wave & 1) * 32 + row);
      const v4i32 x = *reinterpret_cast<const v4i32*>(ebase + row * RB + ((chunk ^ swz<D>(row & 15)) << 4));
      if (qrow < p.Sq) *reinterpret_cast<v4i32*>(obase + static_cast<int64_t>(qrow) * bp.dqs[2] + chunk * 8) = x;
    }
  } else {
    const int qrow = tile_q0 + slot_query((wave & 1) * 32 + l32);
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
            for (int r = 0; r < 4; ++r) cur[r] += dqacc[db][g * 4 + r] * oscale;
            *dst = cur;
          } else {
            bf16x4 w;
#pragma unroll
            for (int r = 0; r < 4; ++r) w[r] = static_cast<bf16_t>(dqacc[db][g * 4 + r] * oscale);
            *reinterpret_cast<bf16x4*>(reinterpret_cast<bf16_t*>(bp.dq_acc) + rowoff + d) = w;
          }
        }
      }
    }
  }
}

template <int D, bool CAUSAL>
int launch(AttnBwdParams bp, hipStream_t st) {
  auto kern = attn_bwd_dq_ds_kernel<D, CAUSAL>;
  constexpr int lds_bytes = DsCfg<D>::LDS_BYTES;
  static_assert(lds_bytes >= WAVES * 32 * DsCfg<D>::RB, "the epilogue needs 32 rows per wavefront");
  static MltsLdsOptIn lds_opt_in;
  if (hipError_t e = lds_opt_in.reserve(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) {
    mlts_set_error("mlts_attn_bwd: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    return MLTS_ERR_LAUNCH;
  }
  bp.a.nqt = (bp.a.Sq + BM - 1) / BM;
  const int64_t blocks = static_cast<int64_t>(bp.a.nqt) * bp.a.B * bp.a.Hq;
  if (blocks > 0) {
    MltsKernelTimer timer("attn_bwd_dq_ds", st);  // its own name: one matrix product, not three
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(THREADS), lds_bytes, st, bp);
  }
  return mlts_check_launch("mlts_attn_bwd");
}

}  // namespace

// bytes of the -dS hand-over for this shape (layout at AttnBwdParams::ds_ws)
int64_t mlts_attn_bwd_ds_bytes(int64_t B, int64_t Hq, int64_t Sq, int64_t Sk) {
  return B * Hq * ((Sk + 31) / 32) * ((Sq + 63) / 64) * 4096;
}

// head_dim 128 (at 64 the recomputing kernel is faster and the caller never hands dS over), MLTS_MASK_NONE or
// MLTS_MASK_CAUSAL, bp.ds_ws filled by the dK/dV kernel on the same stream
int mlts_attn_bwd_dq_bf16_ds(const AttnBwdParams& bp, int D, int mode, hipStream_t st) {
  if (D != 128 || mode == MLTS_MASK_DOC || !bp.ds_ws) {
    mlts_set_error("mlts_attn_bwd: the dS hand-over kernel needs head_dim 128, no document mask and a hand-over buffer");
    return MLTS_ERR_UNSUPPORTED;
  }
  return mode == MLTS_MASK_CAUSAL ? launch<128, true>(bp, st) : launch<128, false>(bp, st);
}
