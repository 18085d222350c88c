// C-ABI entry points for attention: argument validation on the host, workspace carving, kernel
// selection (bf16 head_dim 64/128 -> MFMA kernels, everything else -> generic fp32-ALU kernels) and
// the log-sum-exp block merge.
#include <mutex>

#include "attn_common.hpp"

int mlts_attn_fwd_bf16_dma(const AttnParams& p, int D, int mode, hipStream_t st);                        // attn_fwd_dma.hip
int64_t mlts_attn_bwd_dkdv_split_workspace(int64_t B, int64_t Hq, int64_t Sq);                             // attn_bwd_split.hip
int mlts_attn_bwd_dkdv_bf16_split(AttnBwdParams bp, int D, int mode, void* workspace, bool lse2_ready, hipStream_t st);    // attn_bwd_split.hip
int mlts_attn_bwd_dq_bf16_tr(const AttnBwdParams& bp, int D, int mode, hipStream_t st);                    // attn_bwd_dq_tr.hip
int mlts_attn_generic_fwd(const AttnParams& p, int D, int dtype, int mode, hipStream_t st);
int mlts_attn_generic_bwd(const AttnBwdParams& bp, int D, int dtype, int mode, hipStream_t st);
int mlts_attn_delta(const void* dout, const int64_t* dos, const void* o, const int64_t* os, float* delta, int B, int H,
                    int S, int D, int dtype, hipStream_t st);

namespace {

inline int64_t align256(int64_t x) { return (x + 255) & ~255LL; }
constexpr int64_t kMaxRowStride = int64_t{1} << 24;  // the MFMA kernels address the rows of a tile with 32-bit element offsets

bool uses_mfma(const mlts_attn_shape* s) { return s->dtype == MLTS_BF16 && (s->D == 64 || s->D == 128); }

bool strides_aligned(const int64_t* st, int es) {
  for (int i = 0; i < 3; ++i)
    if ((st[i] * es) % 16 != 0) return false;
  return true;
}

const char* shape_problem(const mlts_attn_shape* s) {
  if (!s) return "shape is null";
  if (s->dtype != MLTS_BF16 && s->dtype != MLTS_F32) return "dtype must be MLTS_F32 or MLTS_BF16";
  if (s->B < 0 || s->Hq <= 0 || s->Hkv <= 0 || s->Sq < 0 || s->Sk < 0 || s->D <= 0) return "negative or zero dimension";
  if (s->Hq % s->Hkv != 0) return "Hq must be a multiple of Hkv";
  if (s->D > 192) return "head_dim > 192 is not supported";
  if (s->mask_mode < MLTS_MASK_NONE || s->mask_mode > MLTS_MASK_DOC) return "unknown mask_mode";
  if (!(s->scale > 0.f)) return "softmax scale must be positive";
  if (s->mask_mode == MLTS_MASK_DOC && !(s->q_pos && s->k_pos && s->q_seq && s->k_seq))
    return "MLTS_MASK_DOC needs q_pos, k_pos, q_seq and k_seq";
  if (uses_mfma(s)) {
    if (!strides_aligned(s->q_stride, 2) || !strides_aligned(s->k_stride, 2) || !strides_aligned(s->v_stride, 2) ||
        !strides_aligned(s->o_stride, 2))
      return "bf16 MFMA path needs strides that keep rows 16-byte aligned";
    if (s->q_stride[2] >= kMaxRowStride || s->k_stride[2] >= kMaxRowStride || s->v_stride[2] >= kMaxRowStride)
      return "bf16 MFMA path needs sequence strides below 2^24 elements";
    if (s->mask_mode == MLTS_MASK_DOC) {
      // the pre-pass launches one wavefront per (batch row, 64-query group, four 64-key tiles) and the kernels index the
      // visibility words of a (group, tile) pair densely; both counts are kept in 32 bits (the plan of such a call would
      // be B * Sq * Sk / 4 bytes = 2 TiB: far beyond the memory of one GPU)
      const int64_t nq = (static_cast<int64_t>(s->Sq) + kAttnTile - 1) / kAttnTile, nk = (static_cast<int64_t>(s->Sk) + kAttnTile - 1) / kAttnTile;
      if (static_cast<int64_t>(s->B) * nq * nk >= (int64_t{1} << 31))
        return "MLTS_MASK_DOC: B * ceil(Sq/64) * ceil(Sk/64) must stay below 2^31 tile pairs";
    }
  }
  return nullptr;
}

// bytes of the document-mask plan at the front of a call's workspace; none when the caller brings the plan
int64_t stats_bytes(const mlts_attn_shape* s, bool backward) {
  if (s->mask_mode != MLTS_MASK_DOC || !uses_mfma(s) || s->doc_plan) return 0;
  const int64_t nq = (s->Sq + kAttnTile - 1) / kAttnTile, nk = (s->Sk + kAttnTile - 1) / kAttnTile;
  // tile statistics of both sides, then the visibility bits of the mixed (query group, key tile) pairs (512 bytes per
  // pair, indexed densely: Sq * Sk / 8 bytes per batch row), query-major and, for the backward pass, key-major as well
  int64_t n = align256(s->B * nq * 16) + align256(s->B * nk * 16) + (backward ? 2 : 1) * align256(s->B * nq * nk * 512);
  n += 2 * align256(s->B * nq * 4);                                   // work count and order of the query blocks
  if (backward) n += 2 * align256(s->B * ((s->Sk + 127) / 128) * 4);  // ... and of the 128-key blocks
  return n;
}

void fill_params(AttnParams& p, const mlts_attn_shape* s, const void* q, const void* k, const void* v, void* o,
                 float* lse) {
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = o;
  p.lse = lse;
  for (int i = 0; i < 3; ++i) {
    p.qs[i] = s->q_stride[i];
    p.ks[i] = s->k_stride[i];
    p.vs[i] = s->v_stride[i];
    p.os[i] = s->o_stride[i];
  }
  p.B = s->B;
  p.Hq = s->Hq;
  p.Hkv = s->Hkv;
  p.Sq = s->Sq;
  p.Sk = s->Sk;
  p.scale = s->scale;
  p.scale_log2 = s->scale * kLog2e;
  p.causal_off = s->Sk - s->Sq;
  p.q_pos = s->q_pos;
  p.k_pos = s->k_pos;
  p.q_seq = s->q_seq;
  p.k_seq = s->k_seq;
  p.q_stats = nullptr;
  p.k_stats = nullptr;
  p.doc_bits = nullptr;
  p.doc_bits_k = nullptr;
  p.kblock_order = nullptr;
  p.qblock_order = nullptr;
  p.nq_stats = (s->Sq + kAttnTile - 1) / kAttnTile;
  p.nk_stats = (s->Sk + kAttnTile - 1) / kAttnTile;
  p.nqt = 0;
  p.head_pack_shift = 0;
}

char* setup_stats(AttnParams& p, const mlts_attn_shape* s, bool backward, char* ws, hipStream_t st);

// A row (D/4 vectors) is owned by G = 2^k <= 64 adjacent lanes of ONE wavefront, so the row's
// lse_acc is read by all of them before one of them rewrites it (program order inside a wave).
template <typename T>
__global__ __launch_bounds__(256) void merge_kernel(float* __restrict__ out_acc, float* __restrict__ lse_acc,
                                                    const T* __restrict__ o_blk, int64_t bs0, int64_t bs1, int64_t bs2,
                                                    const float* __restrict__ lse_blk, int H, int S, int D, int q_off,
                                                    int q_len, int64_t total_rows, int G, int blk_vec) {
  const int vec_per_row = D >> 2;
  const int rows_per_block = 256 / G;
  const int64_t rowi = static_cast<int64_t>(blockIdx.x) * rows_per_block + threadIdx.x / G;
  const int sub = threadIdx.x % G;
  if (rowi >= total_rows) return;
  // 32-bit divisions whenever they suffice (a wave-uniform choice): three 64-bit ones cost more than the merge itself
  int i, h, b;
  int64_t bh;
  if (total_rows < (1LL << 31)) {
    const uint32_t r = static_cast<uint32_t>(rowi), bh32 = r / static_cast<uint32_t>(q_len);
    i = static_cast<int>(r - bh32 * static_cast<uint32_t>(q_len));
    b = static_cast<int>(bh32 / static_cast<uint32_t>(H));
    h = static_cast<int>(bh32 - static_cast<uint32_t>(b) * static_cast<uint32_t>(H));
    bh = bh32;
  } else {
    i = static_cast<int>(rowi % q_len);
    bh = rowi / q_len;
    h = static_cast<int>(bh % H);
    b = static_cast<int>(bh / H);
  }
  const int64_t arow = bh * S + q_off + i;
  const float la = lse_acc[arow], lb = lse_blk[bh * q_len + i];
  const float mx = fmaxf(la, lb);
  float ln = -INFINITY, pa = 0.f, pb = 0.f;
  if (mx != -INFINITY) {
    ln = mx + log1pf(expf(-fabsf(la - lb)));  // logaddexp; -inf on one side returns the other side
    pa = isfinite(la) ? expf(la - ln) : 0.f;
    pb = isfinite(lb) ? expf(lb - ln) : 0.f;
  }
  const T* bp = o_blk + b * bs0 + h * bs1 + static_cast<int64_t>(i) * bs2;
  if ((D & 3) == 0) {
    for (int vc = sub; vc < vec_per_row; vc += G) {
      const f32x4 acc = reinterpret_cast<const f32x4*>(out_acc + arow * D)[vc];
      struct alignas(4 * sizeof(T)) Blk4 { T v[4]; };   // one 8- or 16-byte load where the block's layout allows it
      Blk4 blk4;
      if (blk_vec) {
        blk4 = *reinterpret_cast<const Blk4*>(bp + vc * 4);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) blk4.v[e] = bp[vc * 4 + e];
      }
      f32x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = acc[e] * pa + to_f32<T>(blk4.v[e]) * pb;
      reinterpret_cast<f32x4*>(out_acc + arow * D)[vc] = r;
    }
  } else {
    for (int d = sub; d < D; d += G) out_acc[arow * D + d] = out_acc[arow * D + d] * pa + to_f32<T>(bp[d]) * pb;
  }
  if (sub == 0) lse_acc[arow] = ln;
}


int64_t bwd_min_workspace(const mlts_attn_shape* s) {
  const int64_t delta = align256(static_cast<int64_t>(s->B) * s->Hq * s->Sq * 4);
  const int64_t lse2 = uses_mfma(s) ? mlts_attn_bwd_dkdv_split_workspace(s->B, s->Hq, s->Sq) : 0;
  return stats_bytes(s, true) + delta + lse2;
}

// The recomputing dQ kernel first, which (stats_in_dq) also writes the row statistics (delta, lse2) into the workspace,
// then the dK/dV kernel that reads them.
int attn_bwd_bf16(AttnBwdParams bp, int D, int mode, float* delta_ws, void* lse2_ws, bool stats_in_dq, hipStream_t st) {
  const AttnParams& p = bp.a;
  bp.nkt = (p.Sk + 127) / 128;
  if (stats_in_dq) {
    bp.delta_out = delta_ws;
    bp.lse2_out = static_cast<float*>(lse2_ws);
  }
  int rc = mlts_attn_bwd_dq_bf16_tr(bp, D, mode, st);
  if (rc != MLTS_OK) return rc;
  bp.delta_out = bp.lse2_out = nullptr;
  return mlts_attn_bwd_dkdv_bf16_split(bp, D, mode, lse2_ws, stats_in_dq, st);
}

int attn_bwd_impl(const char* who, const mlts_attn_shape* s, const void* dout, const int64_t do_stride[3], const void* q,
                  const void* k, const void* v, const void* o, const float* lse, void* dq, const int64_t dq_stride[3],
                  void* dk, const int64_t dk_stride[3], void* dv, const int64_t dv_stride[3], int accumulate_f32,
                  void* workspace, int64_t workspace_bytes, hipStream_t st) {
  MLTS_REQUIRE(dout && q && k && v && o && lse && dq && dk && dv, "%s: null tensor pointer", who);
  MLTS_REQUIRE(do_stride && dq_stride && dk_stride && dv_stride, "%s: null stride pointer", who);
  MLTS_REQUIRE(accumulate_f32 >= MLTS_BWD_OVERWRITE && accumulate_f32 <= MLTS_BWD_DQ_STORE, "%s: unknown accumulate_f32 mode %d", who,
               accumulate_f32);
  const int dq_f32 = accumulate_f32 == MLTS_BWD_OVERWRITE ? 0 : accumulate_f32 == MLTS_BWD_DQ_STORE ? 2 : 1;
  const int dkv_f32 = accumulate_f32 == MLTS_BWD_ACCUMULATE ? 1 : 0;
  const int64_t need = bwd_min_workspace(s);
  MLTS_REQUIRE(workspace && workspace_bytes >= need, "%s: workspace too small (%lld < %lld)", who,
               (long long)workspace_bytes, (long long)need);
  AttnBwdParams bp;
  fill_params(bp.a, s, q, k, v, const_cast<void*>(o), const_cast<float*>(lse));
  char* ws = setup_stats(bp.a, s, true, static_cast<char*>(workspace), st);
  float* delta = reinterpret_cast<float*>(ws);
  ws += align256(static_cast<int64_t>(s->B) * s->Hq * s->Sq * 4);
  bp.dout = dout;
  bp.delta = delta;
  bp.dq_acc = static_cast<float*>(dq);
  bp.dk = dk;
  bp.dv = dv;
  for (int i = 0; i < 3; ++i) {
    bp.dos[i] = do_stride[i];
    bp.dqs[i] = dq_stride[i];
    bp.dks[i] = dk_stride[i];
    bp.dvs[i] = dv_stride[i];
  }
  bp.accumulate_f32 = dkv_f32;
  bp.dq_f32 = dq_f32;
  bp.nkt = 0;
  bp.delta_out = bp.lse2_out = nullptr;
  if (uses_mfma(s)) {
    MLTS_REQUIRE(mlts_aligned16(dout) && mlts_aligned16(q) && mlts_aligned16(k) && mlts_aligned16(v) &&
                     mlts_aligned16(dq) && mlts_aligned16(dk) && mlts_aligned16(dv),
                 "%s: tensors must be 16-byte aligned", who);
    MLTS_REQUIRE(strides_aligned(do_stride, 2) && strides_aligned(dq_stride, dq_f32 ? 4 : 2) &&
                     strides_aligned(dk_stride, dkv_f32 ? 4 : 2) && strides_aligned(dv_stride, dkv_f32 ? 4 : 2),
                 "%s: strides must keep rows 16-byte aligned", who);
    MLTS_REQUIRE(do_stride[2] < kMaxRowStride, "%s: the sequence stride of dout must be below 2^24 elements", who);
  }
  void* lse2_ws = ws;
  // the recomputing dQ kernel forms delta itself from 16-byte chunks of the O rows
  const bool stats_in_dq = uses_mfma(s) && s->Sk > 0 && mlts_aligned16(o) && strides_aligned(s->o_stride, 2);
  if (s->Sq > 0 && !stats_in_dq) {
    int rc = mlts_attn_delta(dout, do_stride, o, s->o_stride, delta, s->B, s->Hq, s->Sq, s->D, s->dtype, st);
    if (rc != MLTS_OK) return rc;
  }
  if (!uses_mfma(s)) return mlts_attn_generic_bwd(bp, s->D, s->dtype, s->mask_mode, st);
  return attn_bwd_bf16(bp, s->D, s->mask_mode, delta, lse2_ws, stats_in_dq, st);
}

// ---- scratch of the entry point that allocates nothing --------------------------------------------------------
// Device memory that belongs to the library image: every GPU the library runs on holds its own copy at its own
// address until the process ends.  Host code never uses the array's name as an address; the per-device address is
// looked up once (hipGetSymbolAddress with that device current) and kept in g_scratch_addr.
constexpr int64_t kScratchBytes = MLTS_ATTN_BWD_NOALLOC_MAX_WORKSPACE;
__device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
void* g_scratch_addr[kMaxDevices] = {};
// the last use of a device's scratch: an event behind the kernels of the last call and the stream they ran on.  A call
// on another stream waits for that event first, so that calls on different streams of one GPU take turns.
hipEvent_t g_scratch_event[kMaxDevices] = {};
hipStream_t g_scratch_stream[kMaxDevices] = {};
bool g_scratch_used[kMaxDevices] = {};
std::mutex g_scratch_mutex;

bool stream_is_capturing(hipStream_t st) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

int scratch_for_current_device(void** out, int* dev_out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    mlts_set_error("mlts_attn_bwd_noalloc: cannot identify the current device (%s)", hipGetErrorString(e));
    return MLTS_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_addr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      mlts_set_error("mlts_attn_bwd_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return MLTS_ERR_LAUNCH;
    }
    g_scratch_addr[dev] = ptr;
    if (hipEventCreateWithFlags(&g_scratch_event[dev], hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      g_scratch_event[dev] = nullptr;  // calls still work; calls on different streams are then the caller's to order
    }
  }
  *out = g_scratch_addr[dev];
  *dev_out = dev;
  return MLTS_OK;
}

}  // namespace

// ---- document masks: the pre-pass ------------------------------------------------------------
// Three launches per call: (1) the per-64-token statistics of both sides, (2) the visibility bits of the mixed tile
// pairs and the work counts of the kernels' blocks, (3) the blocks ranked by work.  Each part is a device function over
// a virtual block index; a launch strings the parts' block ranges together (one wavefront per block).

// (position min, max, sequence id min, max) of tile t of row b
__device__ __forceinline__ void doc_tile_stats(const int32_t* __restrict__ pos, const int32_t* __restrict__ seq, int S,
                                               int ntiles, int blk, int lane, int4* __restrict__ out) {
  const int t = blk % ntiles, b = blk / ntiles;
  const int i = t * kAttnTile + lane;
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
  if (lane == 0) out[static_cast<int64_t>(b) * ntiles + t] = make_int4(pmin, pmax, smin, smax);
}

__global__ __launch_bounds__(64) void doc_stats_kernel(const AttnParams p, int q_blocks, int4* __restrict__ q_out,
                                                       int4* __restrict__ k_out) {
  const int blk = blockIdx.x;
  if (blk < q_blocks) doc_tile_stats(p.q_pos, p.q_seq, p.Sq, p.nq_stats, blk, threadIdx.x, q_out);
  else doc_tile_stats(p.k_pos, p.k_seq, p.Sk, p.nk_stats, blk - q_blocks, threadIdx.x, k_out);
}

// One wavefront per (batch row, 64-query group, kDocBitsChunk key tiles), lane = query of the group.  For each pair of
// the chunk whose mask the attention kernels evaluate (mixed pairs, and fully visible pairs of a ragged last key tile)
// the lanes load one key's ids each and the 64 keys are walked with lane reads: a pair costs one memory round trip
// and a few hundred instructions, and a query group that straddles a document boundary (every key tile of both
// documents is mixed for it) is spread over many wavefronts.  The ballot of one step is the key-major word of that key
// (which queries of the group see it); it goes into lane i of the key-major result.
constexpr int kDocBitsChunk = 4;

template <bool KEY_MAJOR>
__device__ __forceinline__ void doc_pair_bits(const AttnParams& p, int n_chunks, int blk, int r,
                                              unsigned long long* __restrict__ out, unsigned long long* __restrict__ out_k) {
  const int chunk = blk % n_chunks, bg = blk / n_chunks;
  const int g = bg % p.nq_stats, b = bg / p.nq_stats;
  const int4 qs = p.q_stats[static_cast<int64_t>(b) * p.nq_stats + g];
  const int t = chunk * kDocBitsChunk + r;  // lane r < kDocBitsChunk classifies key tile t
  bool mixed = false;
  if (r < kDocBitsChunk && t < p.nk_stats) {
    const int4 ks = p.k_stats[static_cast<int64_t>(b) * p.nk_stats + t];
    const int cls = classify_doc_tile(qs, ks);
    mixed = cls == TILE_MASKED || (cls == TILE_FULL && t * kAttnTile + kAttnTile > p.Sk);
  }
  unsigned long long todo = __builtin_amdgcn_ballot_w64(mixed);
  if (todo == 0) return;
  const int qi = g * kAttnTile + r;
  int qpos = 0, qseq = -1;
  if (qi < p.Sq) {
    qpos = p.q_pos[static_cast<int64_t>(b) * p.Sq + qi];
    qseq = p.q_seq[static_cast<int64_t>(b) * p.Sq + qi];
  }
  const int32_t* kpos = p.k_pos + static_cast<int64_t>(b) * p.Sk;
  const int32_t* kseq = p.k_seq + static_cast<int64_t>(b) * p.Sk;
  // the ids of every tile of the chunk are requested before the first pair is walked (one memory latency per wavefront)
  int kp[kDocBitsChunk], ksq[kDocBitsChunk];
#pragma unroll
  for (int c = 0; c < kDocBitsChunk; ++c) {
    const int kj = (chunk * kDocBitsChunk + c) * kAttnTile + r;
    kp[c] = 0;
    ksq[c] = -2;  // keys past the end: an id that no query has
    if (((todo >> c) & 1ull) && kj < p.Sk) {
      kp[c] = kpos[kj];
      ksq[c] = kseq[kj];
    }
  }
#pragma unroll
  for (int c = 0; c < kDocBitsChunk; ++c) {
    if (!((todo >> c) & 1ull)) continue;
    const int j = chunk * kDocBitsChunk + c;
    unsigned long long w = 0;
    int wk_lo = 0, wk_hi = 0;
#pragma unroll
    for (int i = 0; i < kAttnTile; ++i) {
      const int kpi = __builtin_amdgcn_readlane(kp[c], i), ksi = __builtin_amdgcn_readlane(ksq[c], i);
      const bool vis = kpi <= qpos && ksi == qseq && qseq >= 0;
      w |= static_cast<unsigned long long>(vis) << i;
      if (KEY_MAJOR) {
        const unsigned long long col = __builtin_amdgcn_ballot_w64(vis);
        asm("v_writelane_b32 %0, %1, %2" : "+v"(wk_lo) : "s"(static_cast<int>(col)), "n"(i));
        asm("v_writelane_b32 %0, %1, %2" : "+v"(wk_hi) : "s"(static_cast<int>(col >> 32)), "n"(i));
      }
    }
    out[((static_cast<int64_t>(b) * p.nq_stats + g) * p.nk_stats + j) * 64 + r] = w;
    if (KEY_MAJOR)
      out_k[((static_cast<int64_t>(b) * p.nk_stats + j) * p.nq_stats + g) * 64 + r] =
          (static_cast<unsigned long long>(static_cast<unsigned>(wk_hi)) << 32) | static_cast<unsigned>(wk_lo);
  }
}

// Number of key tiles that query block qt (`rows` rows: 64, 128 or 256) of batch row b needs (entry qt * B + b): the
// test of the forward and dQ kernels' scan of the key statistics.
__device__ __forceinline__ void doc_qblock_work(const AttnParams& p, int rows, int e, int lane, int* __restrict__ work) {
  const int b = e % p.B, qt = e / p.B;
  int4 qs[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = qt * (rows >> 6) + i;
    qs[i] = (i < (rows >> 6) && t < p.nq_stats) ? p.q_stats[static_cast<int64_t>(b) * p.nq_stats + t] : make_int4(0, -1, 0, -1);
  }
  int cnt = 0;
  for (int base = 0; base < p.nk_stats; base += 64) {
    bool need = false;
    if (base + lane < p.nk_stats) {
      const int4 ks = p.k_stats[static_cast<int64_t>(b) * p.nk_stats + base + lane];
#pragma unroll
      for (int i = 0; i < 4; ++i) need |= classify_doc_tile(qs[i], ks) != TILE_SKIP;
    }
    cnt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(need));
  }
  if (lane == 0) work[e] = cnt;
}

// Number of query tiles that 128-key block kt of batch row b needs (entry kt * B + b): the test of the dK/dV kernel's
// scan of the query statistics.
__device__ __forceinline__ void doc_kblock_work(const AttnParams& p, int e, int lane, int* __restrict__ work) {
  const int b = e % p.B, kt = e / p.B;
  int4 ks[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int t = kt * 2 + i;
    ks[i] = t < p.nk_stats ? p.k_stats[static_cast<int64_t>(b) * p.nk_stats + t] : make_int4(0x7fffffff, 0, 0, -2);
  }
  int cnt = 0;
  for (int base = 0; base < p.nq_stats; base += 64) {
    bool need = false;
    if (base + lane < p.nq_stats) {
      const int4 qs = p.q_stats[static_cast<int64_t>(b) * p.nq_stats + base + lane];
      need = classify_doc_tile(qs, ks[0]) != TILE_SKIP || classify_doc_tile(qs, ks[1]) != TILE_SKIP;
    }
    cnt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(need));
  }
  if (lane == 0) work[e] = cnt;
}

struct DocPairsArgs {
  int n_chunks, bits_blocks;  // blocks [0, bits_blocks): visibility bits
  int q_blocks, q_rows;       // then q_blocks query blocks of q_rows rows: work counts into q_work
  int k_blocks;               // then k_blocks 128-key blocks: work counts into k_work (backward only)
  unsigned long long *bits, *bits_k;
  int *q_work, *k_work;
};

template <bool BACKWARD>
__global__ __launch_bounds__(64) void doc_pairs_kernel(const AttnParams p, const DocPairsArgs a) {
  int blk = blockIdx.x;
  if (blk < a.bits_blocks) {
    doc_pair_bits<BACKWARD>(p, a.n_chunks, blk, threadIdx.x, a.bits, a.bits_k);
    return;
  }
  blk -= a.bits_blocks;
  if (blk < a.q_blocks) {
    doc_qblock_work(p, a.q_rows, blk, threadIdx.x, a.q_work);
    return;
  }
  if (BACKWARD) doc_kblock_work(p, blk - a.q_blocks, threadIdx.x, a.k_work);
}

// order[rank of i] = i, ranks by work descending (ties by index): every thread counts the entries in front of its own
__device__ __forceinline__ void doc_rank(const int* __restrict__ work, int n, int blk, int* __restrict__ order, int* chunk) {
  const int i = blk * 256 + threadIdx.x;
  const int wi = i < n ? work[i] : 0;
  int rank = 0;
  for (int base = 0; base < n; base += 256) {
    __syncthreads();
    const int at_t = base + static_cast<int>(threadIdx.x);
    chunk[threadIdx.x] = at_t < n ? work[at_t] : -1;
    __syncthreads();
    // (entries past n hold -1: never in front of an entry, whose count is >= 0)
    const int4* chunk4 = reinterpret_cast<const int4*>(chunk);
#pragma unroll 4
    for (int j = 0; j < 64; ++j) {
      const int4 w = chunk4[j];
      const int at = base + 4 * j;
      rank += (w.x > wi || (w.x == wi && at < i)) ? 1 : 0;
      rank += (w.y > wi || (w.y == wi && at + 1 < i)) ? 1 : 0;
      rank += (w.z > wi || (w.z == wi && at + 2 < i)) ? 1 : 0;
      rank += (w.w > wi || (w.w == wi && at + 3 < i)) ? 1 : 0;
    }
  }
  if (i < n) order[rank] = i;
}

// blocks [0, q_grid): the query blocks; then the key blocks (n_k may be 0)
__global__ __launch_bounds__(256) void doc_order_kernel(const int* __restrict__ q_work, int n_q, int* __restrict__ q_order,
                                                        int q_grid, const int* __restrict__ k_work, int n_k,
                                                        int* __restrict__ k_order) {
  __shared__ __attribute__((aligned(16))) int chunk[256];
  if (static_cast<int>(blockIdx.x) < q_grid) doc_rank(q_work, n_q, blockIdx.x, q_order, chunk);
  else doc_rank(k_work, n_k, blockIdx.x - q_grid, k_order, chunk);
}

namespace {
// The document-mask plan at the front of a call's workspace (layout: stats_bytes), or the one the caller brought
// (s->doc_plan, always in the backward's layout): sets the plan pointers of p; builds the plan unless it was brought.
char* setup_stats(AttnParams& p, const mlts_attn_shape* s, bool backward, char* ws, hipStream_t st) {
  if (s->mask_mode != MLTS_MASK_DOC || !uses_mfma(s)) return ws;
  const bool brought = s->doc_plan != nullptr;
  char* const ws_in = ws;
  if (brought) {
    ws = static_cast<char*>(const_cast<void*>(s->doc_plan));
    backward = true;
  }
  const int64_t B = s->B, nq = p.nq_stats, nk = p.nk_stats;
  int4* qst = reinterpret_cast<int4*>(ws);
  ws += align256(B * nq * 16);
  int4* kst = reinterpret_cast<int4*>(ws);
  ws += align256(B * nk * 16);
  DocPairsArgs a{};
  a.bits = reinterpret_cast<unsigned long long*>(ws);
  ws += align256(B * nq * nk * 512);
  if (backward) {
    a.bits_k = reinterpret_cast<unsigned long long*>(ws);
    ws += align256(B * nq * nk * 512);
  }
  a.q_work = reinterpret_cast<int*>(ws);
  ws += align256(B * nq * 4);
  int* q_order = reinterpret_cast<int*>(ws);
  ws += align256(B * nq * 4);
  int* k_order = nullptr;
  if (backward) {
    a.k_work = reinterpret_cast<int*>(ws);
    ws += align256(B * ((s->Sk + 127) / 128) * 4);
    k_order = reinterpret_cast<int*>(ws);
    ws += align256(B * ((s->Sk + 127) / 128) * 4);
  }
  char* const ws_out = brought ? ws_in : ws;
  p.q_stats = qst;
  p.k_stats = kst;
  p.doc_bits = a.bits;
  p.doc_bits_k = a.bits_k;
  p.head_pack_shift = mlts_doc_head_pack_shift(s->Hq, s->Hkv);
  a.q_rows = 256 >> p.head_pack_shift;
  // (B * nq * nk < 2^31 was checked with the shape, so these block counts and their sum fit 32 bits)
  a.n_chunks = static_cast<int>((nk + kDocBitsChunk - 1) / kDocBitsChunk);
  a.bits_blocks = static_cast<int>(B * nq * a.n_chunks);
  a.q_blocks = static_cast<int>(B * ((s->Sq + a.q_rows - 1) / a.q_rows));
  a.k_blocks = backward ? static_cast<int>(B * ((s->Sk + 127) / 128)) : 0;
  const bool pairs = B * nq > 0 && nk > 0;
  const bool order_q = pairs && a.q_blocks > 1 && a.q_blocks <= kMaxOrderedBlocks;
  const bool order_k = pairs && a.k_blocks > 1 && a.k_blocks <= kMaxOrderedBlocks;
  if (!order_q) a.q_blocks = 0;
  if (!order_k) a.k_blocks = 0;
  if (order_q) p.qblock_order = q_order;
  if (order_k) p.kblock_order = k_order;
  if (brought || B * (nq + nk) == 0) return ws_out;

  MltsKernelTimer timer("attn_doc_prepass", st);
  hipLaunchKernelGGL(doc_stats_kernel, dim3(static_cast<unsigned>(B * (nq + nk))), dim3(64), 0, st, p, static_cast<int>(B * nq),
                     qst, kst);
  if (!pairs) return ws_out;
  const unsigned pair_grid = static_cast<unsigned>(a.bits_blocks + a.q_blocks + a.k_blocks);
  if (backward) hipLaunchKernelGGL(doc_pairs_kernel<true>, dim3(pair_grid), dim3(64), 0, st, p, a);
  else hipLaunchKernelGGL(doc_pairs_kernel<false>, dim3(pair_grid), dim3(64), 0, st, p, a);
  if (order_q || order_k) {
    const int q_grid = (a.q_blocks + 255) / 256, k_grid = (a.k_blocks + 255) / 256;
    hipLaunchKernelGGL(doc_order_kernel, dim3(q_grid + k_grid), dim3(256), 0, st, a.q_work, a.q_blocks, q_order, q_grid, a.k_work,
                       a.k_blocks, k_order);
  }
  return ws_out;
}
}  // namespace

extern "C" int64_t mlts_attn_doc_plan_bytes(const mlts_attn_shape* s) {
  if (shape_problem(s)) return -1;
  mlts_attn_shape t = *s;
  t.doc_plan = nullptr;
  return stats_bytes(&t, true);
}

extern "C" int mlts_attn_doc_plan(const mlts_attn_shape* s, void* plan, int64_t plan_bytes, mlts_stream_t stream) {
  const char* why = shape_problem(s);
  MLTS_REQUIRE(why == nullptr, "mlts_attn_doc_plan: %s", why);
  MLTS_REQUIRE(s->mask_mode == MLTS_MASK_DOC, "mlts_attn_doc_plan: mask_mode must be MLTS_MASK_DOC");
  mlts_attn_shape t = *s;
  t.doc_plan = nullptr;
  const int64_t need = stats_bytes(&t, true);
  if (need == 0) return MLTS_OK;  // a shape the generic kernels serve: they evaluate the mask themselves
  MLTS_REQUIRE(plan && plan_bytes >= need, "mlts_attn_doc_plan: plan buffer too small (%lld < %lld)", (long long)plan_bytes,
               (long long)need);
  MLTS_REQUIRE(mlts_aligned16(plan), "mlts_attn_doc_plan: the plan buffer must be 16-byte aligned");
  AttnParams p;
  fill_params(p, &t, nullptr, nullptr, nullptr, nullptr, nullptr);
  setup_stats(p, &t, true, static_cast<char*>(plan), static_cast<hipStream_t>(stream));
  return mlts_check_launch("mlts_attn_doc_plan");
}

extern "C" const char* mlts_attn_supports(const mlts_attn_shape* s) { return shape_problem(s); }

extern "C" int64_t mlts_attn_fwd_workspace_bytes(const mlts_attn_shape* s) {
  if (shape_problem(s)) return -1;
  return stats_bytes(s, false);
}

extern "C" int64_t mlts_attn_bwd_workspace_bytes(const mlts_attn_shape* s, int accumulate_f32) {
  (void)accumulate_f32;
  if (shape_problem(s)) return -1;
  return bwd_min_workspace(s);
}

extern "C" int mlts_attn_fwd(const mlts_attn_shape* s, const void* q, const void* k, const void* v, void* o, float* lse,
                             void* workspace, int64_t workspace_bytes, mlts_stream_t stream) {
  const char* why = shape_problem(s);
  MLTS_REQUIRE(why == nullptr, "mlts_attn_fwd: %s", why);
  if (s->B == 0 || s->Sq == 0) return MLTS_OK;
  MLTS_REQUIRE(q && o && lse, "mlts_attn_fwd: q, o, lse must be non-null");
  MLTS_REQUIRE(s->Sk == 0 || (k && v), "mlts_attn_fwd: k, v must be non-null");
  const int64_t need = stats_bytes(s, false);
  MLTS_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), "mlts_attn_fwd: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)need);
  hipStream_t st = static_cast<hipStream_t>(stream);
  AttnParams p;
  fill_params(p, s, q, k, v, o, lse);
  if (uses_mfma(s)) {
    MLTS_REQUIRE(mlts_aligned16(q) && mlts_aligned16(k) && mlts_aligned16(v) && mlts_aligned16(o),
                 "mlts_attn_fwd: q, k, v, o must be 16-byte aligned");
    setup_stats(p, s, false, static_cast<char*>(workspace), st);
    return mlts_attn_fwd_bf16_dma(p, s->D, s->mask_mode, st);
  }
  return mlts_attn_generic_fwd(p, s->D, s->dtype, s->mask_mode, st);
}

extern "C" int mlts_attn_bwd(const mlts_attn_shape* s, const void* dout, const int64_t do_stride[3], const void* q,
                             const void* k, const void* v, const void* o, const float* lse, void* dq,
                             const int64_t dq_stride[3], void* dk, const int64_t dk_stride[3], void* dv,
                             const int64_t dv_stride[3], int accumulate_f32, void* workspace, int64_t workspace_bytes,
                             mlts_stream_t stream) {
  const char* why = shape_problem(s);
  MLTS_REQUIRE(why == nullptr, "mlts_attn_bwd: %s", why);
  if (s->B == 0 || (s->Sq == 0 && s->Sk == 0)) return MLTS_OK;
  return attn_bwd_impl("mlts_attn_bwd", s, dout, do_stride, q, k, v, o, lse, dq, dq_stride, dk, dk_stride, dv, dv_stride,
                       accumulate_f32, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int mlts_attn_bwd_noalloc(const mlts_attn_shape* s, const void* dout, const int64_t do_stride[3], const void* q,
                                     const void* k, const void* v, const void* o, const float* lse, void* dq,
                                     const int64_t dq_stride[3], void* dk, const int64_t dk_stride[3], void* dv,
                                     const int64_t dv_stride[3], int accumulate_f32, mlts_stream_t stream) {
  const char* why = shape_problem(s);
  MLTS_REQUIRE(why == nullptr, "mlts_attn_bwd_noalloc: %s", why);
  if (s->B == 0 || (s->Sq == 0 && s->Sk == 0)) return MLTS_OK;
  const int64_t need = bwd_min_workspace(s);
  MLTS_REQUIRE(need <= kScratchBytes,
               "mlts_attn_bwd_noalloc: this shape needs %lld bytes of workspace, the built-in scratch holds %lld "
               "(about B*Hq*Sq <= %lld query rows); use mlts_attn_bwd with a caller workspace",
               (long long)need, (long long)kScratchBytes, (long long)(kScratchBytes / 8 - 64));
  void* ws = nullptr;
  int dev = 0;
  int rc = scratch_for_current_device(&ws, &dev);
  if (rc != MLTS_OK) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Calls on different streams take turns on the scratch: this call waits for the event behind the last one.  Not
  // while a stream is being captured (an event recorded outside the capture cannot be waited for inside it): graphs
  // that hold this call and are replayed on different streams of one GPU must be ordered by the caller.
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  const bool ordered = g_scratch_event[dev] != nullptr && !stream_is_capturing(st);
  if (ordered && g_scratch_used[dev] && g_scratch_stream[dev] != st) {
    if (hipStreamWaitEvent(st, g_scratch_event[dev], 0) != hipSuccess) {
      mlts_set_error("mlts_attn_bwd_noalloc: cannot order this call behind the last user of the scratch: %s",
                     hipGetErrorString(hipGetLastError()));
      return MLTS_ERR_LAUNCH;
    }
  }
  rc = attn_bwd_impl("mlts_attn_bwd_noalloc", s, dout, do_stride, q, k, v, o, lse, dq, dq_stride, dk, dk_stride, dv,
                     dv_stride, accumulate_f32, ws, need, st);
  if (ordered) {
    if (hipEventRecord(g_scratch_event[dev], st) == hipSuccess) {
      g_scratch_stream[dev] = st;
      g_scratch_used[dev] = true;
    } else {
      (void)hipGetLastError();
    }
  }
  return rc;
}

extern "C" int mlts_attn_merge(float* out_acc, float* lse_acc, const void* o_blk, const int64_t o_blk_stride[3],
                               int32_t blk_dtype, const float* lse_blk, int32_t B, int32_t H, int32_t S, int32_t D,
                               int32_t q_off, int32_t q_len, mlts_stream_t stream) {
  MLTS_REQUIRE(blk_dtype == MLTS_BF16 || blk_dtype == MLTS_F32, "mlts_attn_merge: unknown dtype %d", blk_dtype);
  MLTS_REQUIRE(B >= 0 && H >= 0 && S >= 0 && D > 0 && q_off >= 0 && q_len >= 0 && q_off + q_len <= S,
               "mlts_attn_merge: rows [%d, %d) do not fit S=%d", q_off, q_off + q_len, S);
  if (B == 0 || H == 0 || q_len == 0) return MLTS_OK;
  MLTS_REQUIRE(out_acc && lse_acc && o_blk && lse_blk && o_blk_stride, "mlts_attn_merge: null pointer");
  MLTS_REQUIRE((D & 3) != 0 || mlts_aligned16(out_acc), "mlts_attn_merge: out_acc must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  MltsKernelTimer timer("attn_merge", st);
  const int64_t total_rows = static_cast<int64_t>(B) * H * q_len;
  int G = 1;
  while (G < (D + 3) / 4 && G < 64) G <<= 1;
  const int rows_per_block = 256 / G;
  const int64_t blocks = (total_rows + rows_per_block - 1) / rows_per_block;
  const uintptr_t blk_bytes4 = blk_dtype == MLTS_BF16 ? 8 : 16;  // four elements of the block
  const int blk_vec = (reinterpret_cast<uintptr_t>(o_blk) % blk_bytes4 == 0) &&
                      ((o_blk_stride[0] | o_blk_stride[1] | o_blk_stride[2]) & 3) == 0;
  if (blk_dtype == MLTS_BF16)
    hipLaunchKernelGGL(merge_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, st, out_acc, lse_acc,
                       static_cast<const bf16_t*>(o_blk), o_blk_stride[0], o_blk_stride[1], o_blk_stride[2], lse_blk, H, S,
                       D, q_off, q_len, total_rows, G, blk_vec);
  else
    hipLaunchKernelGGL(merge_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, out_acc, lse_acc,
                       static_cast<const float*>(o_blk), o_blk_stride[0], o_blk_stride[1], o_blk_stride[2], lse_blk, H, S,
                       D, q_off, q_len, total_rows, G, blk_vec);
  return mlts_check_launch("mlts_attn_merge");
}
