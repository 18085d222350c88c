// Shared pieces of the attention kernels: kernel parameter block, mask predicate, per-tile
// position/sequence statistics used to skip or fast-path whole 64-key tiles.
#pragma once
#include "common.hpp"

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

constexpr int kAttnTile = 64;  // granularity of the tile statistics (queries per wave, keys per tile)

struct AttnParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;
  int64_t qs[3], ks[3], vs[3], os[3];
  int B, Hq, Hkv, Sq, Sk;
  float scale;        // softmax scale
  float scale_log2;   // scale * log2(e)
  int causal_off;     // Sk - Sq: key j visible to query i iff j <= i + causal_off
  const int32_t* q_pos;
  const int32_t* k_pos;
  const int32_t* q_seq;
  const int32_t* k_seq;
  const int4* q_stats;  // [B, ceil(Sq/64)] (min_pos, max_pos, min_seq, max_seq)
  const int4* k_stats;  // [B, ceil(Sk/64)]
  int nq_stats, nk_stats;
  // MLTS_MASK_DOC: for every (64-query group, 64-key tile) pair that classify_doc_tile calls mixed (and for fully visible
  // pairs of a ragged last key tile), 64 words [B][nq_stats][nk_stats][64]: bit i of word r = key i of the tile is
  // visible to query r of the group.  The mask is the same for every head and for forward and dQ, so it is evaluated
  // once per call by a pre-pass instead of per head inside the kernels.  Words of other pairs are not written.
  const unsigned long long* doc_bits;
  // The same bits for the mixed pairs, key-major, for the dK/dV kernel whose lanes are keys: [B][nk_stats][nq_stats][64],
  // bit i of word r = query i of the group sees key r of the tile.  Null in the forward pass.
  const unsigned long long* doc_bits_k;
  // Backward with MLTS_MASK_DOC: the (128-key block, batch row) pairs, index kt * B + b, sorted by the number of query
  // tiles they need, most first.  The dK/dV grid walks them in this order: a block's work ranges from one tile to all
  // tiles of two long documents, and in plain order a heavy block that starts late sets the kernel's duration.  Null:
  // plain order.
  const int* kblock_order;
  int nqt;              // query tiles per (batch, head) for the launched kernel
  // Forward with MLTS_MASK_DOC and grouped-query heads: log2 of the number of query heads of one KV head that share a
  // workgroup (0, 1 or 2).  The workgroup's 256 rows are then 256 >> shift rows of each of those heads: the heads need
  // the same key tiles, where 256 consecutive rows of one head need the union of the tiles of every document they touch.
  int head_pack_shift;
  // Forward with MLTS_MASK_DOC: the (query block of 256 >> head_pack_shift rows, batch row) pairs, index qt * B + b,
  // sorted by the number of key tiles they need, most first (as kblock_order for the dK/dV kernel).  Null: last blocks
  // first, the order of a causal mask.
  const int* qblock_order;
};

// Backward-only extras.
struct AttnBwdParams {
  AttnParams a;
  const void* dout;
  int64_t dos[3];
  const float* delta;  // [B, Hq, Sq] rowsum(dO * O)
  float* dq_acc;       // dQ [B, Hq, Sq, D] with caller strides: the input dtype, or fp32 (dq_f32 != 0)
  int64_t dqs[3];
  void* dk;
  void* dv;
  int64_t dks[3], dvs[3];
  int accumulate_f32;  // dk/dv are fp32 and added to (otherwise the input dtype, overwritten)
  int dq_f32;          // 0: dq has the input dtype and is overwritten; 1: fp32, added to; 2: fp32, overwritten
  int nkt;             // key tiles per (batch, kv head)
  // Optional outputs of the recomputing dQ kernel, which then runs first and takes the place of the separate row
  // statistics passes: delta_out[B, Hq, Sq] = rowsum(dO * O) (the kernel ignores `delta` and reads `a.o`), and
  // lse2_out[B * Hq * Sq + 1] = lse * log2(e) with +inf for rows that saw no key and in the last entry.
  float* delta_out;
  float* lse2_out;
};

enum TileClass { TILE_SKIP = 0, TILE_FULL = 1, TILE_MASKED = 2 };

// Classification of a (64-query group, 64-key tile) pair from the statistics, MLTS_MASK_DOC.
__device__ __forceinline__ int classify_doc_tile(const int4 qs, const int4 ks) {
  // nothing visible: every key is later than every query, or the sequence-id ranges are disjoint,
  // or every query is padding
  if (ks.x > qs.y || ks.w < qs.z || ks.z > qs.w || qs.w < 0) return TILE_SKIP;
  // everything visible: all keys precede all queries and a single non-padding sequence id
  if (ks.y <= qs.x && qs.z == qs.w && ks.z == ks.w && ks.z == qs.z && qs.z >= 0) return TILE_FULL;
  return TILE_MASKED;
}

// MLTS_MASK_DOC: which tiles of one batch row's tile statistics a workgroup needs and how one wavefront sees them,
// evaluated 64 tiles at a time (lane i looks at tile base + i, the answers travel as wave-uniform 64-bit masks).
// Walking the statistics one tile at a time costs a dependent global load per tile, needed or not, which is as long
// as the work on a needed tile.
struct DocTileScan {
  unsigned long long need = 0, skip = 0, full = 0;  // bit i <-> tile base + i
  int base = -64;                                   // no chunk loaded
};

// KEYS = true: the scanned tiles are key tiles, `grp` / `own` are query statistics (forward, dQ); false: the scanned
// tiles are query tiles and `grp` / `own` key statistics (dK/dV).  need: some group of `grp` sees the tile; skip / full:
// classification against `own`.
template <int NG, bool KEYS>
__device__ __forceinline__ void doc_scan_fill(DocTileScan& sc, int base, int n_tiles, const int4* __restrict__ row_stats,
                                              const int4 (&grp)[NG], const int4 own, int lane) {
  const int t = base + lane;
  bool need = false, skip = true, full = false;
  if (t < n_tiles) {
    const int4 ts = row_stats[t];
#pragma unroll
    for (int w = 0; w < NG; ++w) need |= (KEYS ? classify_doc_tile(grp[w], ts) : classify_doc_tile(ts, grp[w])) != TILE_SKIP;
    const int c = KEYS ? classify_doc_tile(own, ts) : classify_doc_tile(ts, own);
    skip = c == TILE_SKIP;
    full = c == TILE_FULL;
  }
  sc.need = __builtin_amdgcn_ballot_w64(need);
  sc.skip = __builtin_amdgcn_ballot_w64(skip);
  sc.full = __builtin_amdgcn_ballot_w64(full);
  sc.base = base;
}

// first needed tile in [j, end), or end; n_tiles = number of statistics entries of the row
template <int NG, bool KEYS>
__device__ __forceinline__ int doc_scan_next(DocTileScan& sc, int j, int end, int n_tiles, const int4* __restrict__ row_stats,
                                             const int4 (&grp)[NG], const int4 own, int lane) {
  while (j < end) {
    if (j < sc.base || j >= sc.base + 64) doc_scan_fill<NG, KEYS>(sc, j & ~63, n_tiles, row_stats, grp, own, lane);
    const unsigned long long m = sc.need >> (j - sc.base);
    if (m != 0) {
      const int t = j + __builtin_ctzll(m);
      return t < end ? t : end;
    }
    j = sc.base + 64;
  }
  return end;
}

// classification of tile j for the wavefront; j must lie in the chunk the scan holds (it does right after
// doc_scan_next returned it)
__device__ __forceinline__ int doc_scan_class(const DocTileScan& sc, int j) {
  const int bit = j - sc.base;
  if ((sc.skip >> bit) & 1ull) return TILE_SKIP;
  return ((sc.full >> bit) & 1ull) ? TILE_FULL : TILE_MASKED;
}

constexpr int kMaxOrderedBlocks = 8192;  // more blocks than this are walked in plain order
// log2 of the query heads per forward workgroup under a document mask (AttnParams::head_pack_shift)
inline int mlts_doc_head_pack_shift(int Hq, int Hkv) {
  const int group = Hq / Hkv;
  return group % 4 == 0 ? 2 : group % 2 == 0 ? 1 : 0;
}
