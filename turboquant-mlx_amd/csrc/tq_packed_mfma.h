// Matrix-core tile pass over PACKED keys and/or values (d = 128, 1 to 4 bits, n_rep <= 16).
// Included by tq_attn.hip after tq_decode_mfma.h, whose conventions it shares: a workgroup of 8
// waves owns 512 positions of one kv head, a wave 64 of them; partials go to the workspace and
// the merge pass finishes.  Three modes:
//
//   kFlash    packed K and packed V: scores from the pre-rotated query, online-softmax partials
//             (tq_flash_decode);
//   kScores   packed K only: the scores themselves are the output (tq_prerot_qk_scores);
//   kWeights  packed V only: the weights are given, positions below the threshold contribute
//             nothing (tq_sparse_v_matvec).
//
// Packed rows are 52 bytes at three bits, so the wave's 64 rows of K (and of V) are one contiguous
// 3328-byte block: 4 coalesced 16-byte loads per lane, copied into the wave's LDS area.  A lane then
// needs, per row, the 24 bits holding 8 consecutive elements: two words, one shift-or (the other
// widths divide the word: one shift).  For K the 8 elements are 4 ADJACENT pairs, i.e. four
// contiguous fields of 2 * bits bits, each of which indexes the centroid-pair table directly and
// yields one register of the A operand; for V two positions are interleaved first (see
// tq_decode_mfma.h).  Scores are (sum_e c_k[idx] q_rot[e]) * k_norm * (1/d) [* scale].
#pragma once

#include "tq_decode_mfma.h"

namespace tqm {

enum PackedMode { kFlash = 0, kScores = 1, kWeights = 2, kSoftWeights = 3, kSoftScores = 4 };
enum PackedTileShape { kTilesDefault = 0, kTilesOnePerCu = 1, kTilesFourWaves = 2 };

struct PackedArgs {
  const float* q_rot;         // kFlash / kScores: [n_seq, n_q, 128] f32, pre-rotated; or NULL with q_raw set
  const void* q_raw;          // the query itself, [n_seq, n_q, 128] of q_dtype: rotated inside the kernel
  const float* k_signs;       //   (q * k_signs, raw butterfly: the bits of tq_prerotate_query)
  int32_t q_dtype;
  const float* weights;       // kWeights: [n_seq * n_q, w_stride] f32 weights; kSoftWeights: scores in log2 units
  const float* stats;         // kSoftWeights: [n_seq * n_kv, n_tiles_max, n_rep, 2] (maximum, sum of 2^(s - maximum)) per tile
  int64_t w_stride;           // floats per row of `weights`
  int32_t stats_tile_pos;     // kSoftWeights: positions per entry of `stats`
  int32_t n_stats_max;        //               entries of `stats` per (sequence, kv head)
  const uint32_t* k_packed;
  const float* k_norms;
  const uint32_t* v_packed;
  const float* v_norms;
  const int32_t* seq_offsets;
  const int64_t* len_dev;     // optional (no seq_offsets): every sequence attends
  int64_t len_bias;           // min(max(*len_dev + len_bias, 0), seq_len) positions, read when the kernel runs
  const float* mask;
  float* scores;              // kScores: [n_q, T] f32; kSoftScores: [n_seq * n_q, w_stride] f32, log2 units
  float* stats_out;           // kSoftScores: [n_seq * n_kv, n_tiles_max, n_rep, 2] (maximum, sum of 2^(s - maximum)) per tile
  float* ws_S;
  float* ws_ml;
  int64_t seq_len;
  int64_t k_seq_stride, k_head_stride, kn_seq_stride, kn_head_stride;
  int64_t v_seq_stride, v_head_stride, vn_seq_stride, vn_head_stride;
  int64_t mask_seq_stride, mask_head_stride;
  int32_t n_kv, n_rep, n_tiles_max;
  float score_scale;          // (1/d) * attn_scale for kFlash, 1/d for kScores; times 1/key-table scale
  float v_unscale;            // 1 / the scale the value table was multiplied by on the host
  float threshold;            // kWeights
};

// copy one wave's 64 packed rows of PD words each (3328 bytes at three bits) from global memory into its LDS area:
// wave-wide 16-byte loads where the block is whole and aligned (three and a quarter of them at three bits), else
// PD 4-byte loads per lane with the index clamped into the tile
template <int PD>
struct PackedBlockT {
  static constexpr int kFull = (16 * PD) / 64;            // whole-wave 16-byte loads
  static constexpr int kTail = 16 * PD - 64 * kFull;      // pieces of the last, partial one (0 or 16)
  u4 q[kFull + (kTail ? 1 : 0)];
  uint32_t d[PD];
  bool wide;
};
using PackedBlock = PackedBlockT<kPdim>;

// STREAM: streaming loads (load_stream).  They pay in the passes that decode values (given weights: 11.9 -> 11.7 us at
// 32 768 positions) and cost where a pass only scores keys and writes as many bytes as it reads (65 536 positions:
// 10.7 -> 11.0 us), so the score-only passes keep the default policy.
template <bool STREAM, int PD>
__device__ __forceinline__ void load_block(PackedBlockT<PD>& b, const uint32_t* block, int lane, int wrow0, int rows_here) {
  constexpr int kFull = PackedBlockT<PD>::kFull, kTail = PackedBlockT<PD>::kTail;
  b.wide = (wrow0 + kWavePos <= rows_here) && ((reinterpret_cast<uintptr_t>(block) & 15) == 0);
  if (b.wide) {
    const u4* b4 = reinterpret_cast<const u4*>(block);
#pragma unroll
    for (int i = 0; i < kFull; ++i) b.q[i] = STREAM ? load_stream(b4 + i * 64 + lane) : b4[i * 64 + lane];
    if (kTail) b.q[kFull] = STREAM ? load_stream(b4 + kFull * 64 + (lane & (kTail - 1))) : b4[kFull * 64 + (lane & (kTail - 1))];
  } else {
    const int valid_words = max(0, rows_here - wrow0) * PD;
    const uint32_t* tile_base = block - (int64_t)wrow0 * PD;          // row 0 of the tile: always valid
#pragma unroll
    for (int i = 0; i < PD; ++i) {
      const int w = i * 64 + lane;
      b.d[i] = load_stream((w < valid_words) ? block + w : tile_base);
    }
  }
}

template <int PD>
__device__ __forceinline__ void stage_block(const PackedBlockT<PD>& b, uint32_t* stage, int lane) {
  constexpr int kFull = PackedBlockT<PD>::kFull, kTail = PackedBlockT<PD>::kTail;
  if (b.wide) {
    u4* st4 = reinterpret_cast<u4*>(stage);
#pragma unroll
    for (int i = 0; i < kFull; ++i) st4[i * 64 + lane] = b.q[i];
    if (kTail) { if (lane < kTail) st4[kFull * 64 + lane] = b.q[kFull]; }
  } else {
#pragma unroll
    for (int i = 0; i < PD; ++i) stage[i * 64 + lane] = b.d[i];
  }
}

// Query rows of one kv head, rotated in place of a separate pre-rotation launch: wave w takes rows w, w + N_WAVES, ...
// of the 16 (rows at or past n_rep are zeros), lane l the elements l and l + 64; q * signs, the raw butterfly of
// tq_prerotate_query (same stage order, hence the same bits), then the fp16 value and the fp16 remainder of that
// rounding into q_s / ql_s.  Runs while the key/value loads are in flight.
template <int N_WAVES>
__device__ __forceinline__ void rotate_query_rows(const void* q_raw, int q_dtype, const float* k_signs, int64_t q_row0,
                                                  int n_rep, int wave, int lane, uint32_t (*q_s)[kD / 2],
                                                  uint32_t (*ql_s)[kD / 2]) {
  const float s0 = k_signs[lane], s1 = k_signs[lane + 64];
#pragma unroll
  for (int it = 0; it < kHeadsMax / N_WAVES; ++it) {
    const int r = wave + it * N_WAVES;
    float v[2] = {0.0f, 0.0f};
    if (r < n_rep) {
      const int64_t base = (q_row0 + r) * kD;
      if (q_dtype == TQ_F32) {
        v[0] = reinterpret_cast<const float*>(q_raw)[base + lane];
        v[1] = reinterpret_cast<const float*>(q_raw)[base + lane + 64];
      } else if (q_dtype == TQ_F16) {
        v[0] = __half2float(reinterpret_cast<const __half*>(q_raw)[base + lane]);
        v[1] = __half2float(reinterpret_cast<const __half*>(q_raw)[base + lane + 64]);
      } else {
        v[0] = __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(q_raw)[base + lane] << 16);
        v[1] = __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(q_raw)[base + lane + 64] << 16);
      }
      v[0] *= s0;
      v[1] *= s1;
    }
    raw_butterfly<kD>(v, lane);
    __half* hi = reinterpret_cast<__half*>(&q_s[r][0]);
    __half* lo = reinterpret_cast<__half*>(&ql_s[r][0]);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const __half h = __float2half_rn(v[i]);
      hi[lane + 64 * i] = h;
      lo[lane + 64 * i] = __float2half_rn(v[i] - __half2float(h));
    }
  }
}

// A operand of a score product: the centroids of the 8 consecutive key elements in the low 8 * BITS bits of f,
// as two quad look-ups or four pair look-ups
template <int BITS, bool QUAD>
__device__ __forceinline__ u4 key_operand(uint32_t f, const uint2* quad_lut, const uint32_t* pair_lut) {
  using VF = VField<BITS>;
  u4 ka;
  if constexpr (QUAD) {
    const uint2 lo = VF::quad_lookup(quad_lut, f, 0), hi = VF::quad_lookup(quad_lut, f, 1);
    ka = u4{lo.x, lo.y, hi.x, hi.y};
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) ka[k] = pair_lut[VF::index(f, k)];
  }
  return ka;
}

// Table indices of the value products of 32 positions (kb2 = which 32 of the wave's 64): lane (n16, g) decodes
// elements 8 n16 .. 8 n16 + 7 (piece at word w0, shifts sh_lo / sh_hi of a row) of positions 16 t + 4 g + j,
// t = 2 kb2, 2 kb2 + 1, j = 0 .. 3 -- the eight contraction slots of this lane in the matrix instruction.
// Pairs: VI[qd] / VI[4 + qd] = even / odd elements of positions (2 jp, 2 jp + 1) of t, qd = 2 (t - 2 kb2) + jp.
// Quads: VI[4 th + w] = word w of interleave4_raw over the four positions of t = 2 kb2 + th.
template <int BITS, bool QUAD>
__device__ __forceinline__ void value_indices(const uint32_t* rows, int kb2, int g, int w0, int sh_lo, int sh_hi,
                                              uint32_t (&VI)[8]) {
  using VF = VField<BITS>;
  constexpr int kPd = VF::kPd;
  if constexpr (QUAD) {
#pragma unroll
    for (int th = 0; th < 2; ++th) {
      const uint32_t* r = rows + (16 * (2 * kb2 + th) + 4 * g) * kPd + w0;
      uint32_t Z[4];
      VF::interleave4_raw(VF::field_raw(r, sh_lo, sh_hi), VF::field_raw(r + kPd, sh_lo, sh_hi),
                          VF::field_raw(r + 2 * kPd, sh_lo, sh_hi), VF::field_raw(r + 3 * kPd, sh_lo, sh_hi), Z);
#pragma unroll
      for (int w = 0; w < 4; ++w) VI[4 * th + w] = Z[w];
    }
  } else {
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int t = 2 * kb2 + (qd >> 1), jp = qd & 1;
      const uint32_t* ra = rows + (16 * t + 4 * g + 2 * jp) * kPd + w0;
      VF::interleave_raw(VF::field_raw(ra, sh_lo, sh_hi), VF::field_raw(ra + kPd, sh_lo, sh_hi), VI[qd], VI[4 + qd]);
    }
  }
}

// Value products of 32 positions: accS[et] += A x B[et], B[et] = the centroids of element et of this lane's piece at
// its eight positions: two quad look-ups (four positions each) or four pair look-ups.
template <int BITS, bool QUAD>
__device__ __forceinline__ void value_products(const u4& A, const uint32_t (&VI)[8], const uint2* quad_lut,
                                               const uint32_t* pair_lut, f4 (&accS)[8]) {
  using VF = VField<BITS>;
#pragma unroll
  for (int et = 0; et < 8; ++et) {
    u4 B;
    if constexpr (QUAD) {
      const uint2 lo = VF::quad_lookup(quad_lut, VI[VF::z_word(et)], VF::z_quad(et));
      const uint2 hi = VF::quad_lookup(quad_lut, VI[4 + VF::z_word(et)], VF::z_quad(et));
      B = u4{lo.x, lo.y, hi.x, hi.y};
    } else {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) B[qd] = pair_lut[VF::index(VI[(et & 1) * 4 + qd], et >> 1)];
    }
    accS[et] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, A), __builtin_bit_cast(h8, B),
                                                      accS[et], 0, 0, 0);
  }
}

// grid = (n_tiles_max, n_kv, n_seq), NW * 64 threads, a tile of NW * 64 positions.  BITS: width of the packed keys and
// values (a cache has one width for both).  WPE = waves per SIMD the registers are budgeted for: 4 lets two eight-wave
// workgroups share a CU (the flash mode then spills some registers, which large grids repay); 3 is the flash mode
// without spills, for grids that give a CU one workgroup at most.  NW = 4 (flash mode, budget of two waves per SIMD)
// is for short caches whose eight-wave tiles would fill at most half of the CUs: twice the workgroups, each wave with
// its SIMD to itself.
// Centroids come from the pair tables here: a workgroup decodes 512 positions once, which does not repay building the
// 32 KB quad table (measured: scores over 65 536 positions 10.65 us with pairs, 10.95 us with quads).
template <int MODE, int BITS = 3, int WPE = 4, int NW = kWaves>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
void packed_tile_mfma_kernel(PackedArgs a, Codebook kcb, Codebook vcb) {
  static_assert(NW == kWaves || (NW == 4 && MODE == kFlash), "the four-wave shape exists for the flash mode");
  constexpr int kThr = NW * 64, kPos = NW * kWavePos;               // threads and positions of a workgroup
  using VF = VField<BITS>;
  constexpr int kVPd = VF::kPd;                                      // words per packed row
  constexpr bool GIVEN = MODE == kWeights || MODE == kSoftWeights;   // weights come from memory, no keys
  constexpr bool HAS_K = !GIVEN;
  constexpr bool HAS_V = MODE != kScores && MODE != kSoftScores;
  constexpr bool SOFT = MODE == kFlash || MODE == kSoftScores;        // scores carry attn_scale * log2 e and the mask
  constexpr bool KQUAD = false, VQUAD = false;
  __shared__ __align__(16) unsigned char big_s[NW * 4096];    // per-wave 4 KB areas, later S_all[NW][8][128]
  __shared__ uint32_t lutk_s[VF::kLut < 64 ? 64 : VF::kLut], lutv_s[VF::kLut < 64 ? 64 : VF::kLut];
  const uint2* quad_s = nullptr;
  __shared__ __align__(16) uint32_t q_s[kHeadsMax][kD / 2];      // rotated queries as half2: rounded value ...
  __shared__ __align__(16) uint32_t ql_s[kHeadsMax][kD / 2];     // ... and what the rounding lost
  __shared__ __align__(16) float kn_s[NW][kWavePos], vn_s[NW][kWavePos];
  __shared__ float m_s[NW][kHeadsMax], l_s[NW][kHeadsMax];
  __shared__ __align__(16) MergeLds<NW> mg_s;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
  const int n_rep = a.n_rep;
  const int n_q = a.n_kv * n_rep;
  const int64_t q_row0 = (int64_t)seq * n_q + (int64_t)kvh * n_rep;

  int64_t first = 0, len = a.seq_len;
  if (a.seq_offsets) {
    first = a.seq_offsets[seq];
    len = (int64_t)a.seq_offsets[seq + 1] - first;
  } else if (a.len_dev) {
    const int64_t want = *a.len_dev + a.len_bias;
    len = want < 0 ? 0 : (want < len ? want : len);
  }
  const int64_t tile_p0 = (int64_t)tile * kPos;
  if (tile_p0 >= len) return;
  const int rows_here = (int)min((int64_t)kPos, len - tile_p0);
  const int last_row = rows_here - 1;
  const int wrow0 = wave * kWavePos;
  int crow = wrow0 + lane;
  crow = crow < last_row ? crow : last_row;                           // clamped row of this lane

  // ---- loads ----------------------------------------------------------------------------------------
  constexpr int kQIt = kHeadsMax * (kD / 2) / kThr;
  float2 my_q[kQIt];
  if (HAS_K && !a.q_raw) {
#pragma unroll
    for (int i = 0; i < kQIt; ++i) {
      const int w = tid + i * kThr;                           // word = 2 consecutive elements
      my_q[i] = (w < n_rep * (kD / 2)) ? reinterpret_cast<const float2*>(a.q_rot + q_row0 * kD)[w]
                                       : make_float2(0.f, 0.f);
    }
  }
  float my_kn = 0.0f, my_vn = 0.0f;
  PackedBlockT<kVPd> kb_, vb_;
  if (HAS_V) {
    my_vn = load_stream(a.v_norms + (int64_t)seq * a.vn_seq_stride + (int64_t)kvh * a.vn_head_stride + first + tile_p0 + crow);
    load_block<true>(vb_, a.v_packed + ((int64_t)seq * a.v_seq_stride + (int64_t)kvh * a.v_head_stride + first +
                                  tile_p0 + wrow0) * kVPd, lane, wrow0, rows_here);
  }
  if (HAS_K) {
    my_kn = load_stream(a.k_norms + (int64_t)seq * a.kn_seq_stride + (int64_t)kvh * a.kn_head_stride + first + tile_p0 + crow);
    load_block<HAS_V>(kb_, a.k_packed + ((int64_t)seq * a.k_seq_stride + (int64_t)kvh * a.k_head_stride + first +
                                  tile_p0 + wrow0) * kVPd, lane, wrow0, rows_here);
  }
  // given weights: lane (head n16, group g) takes positions 16t + 4g + j
  float wgt[4][4];
  float2 st_ml[4];
  int st_tiles = 0;
  const float* st_base = nullptr;
  if (GIVEN) {
    // four consecutive positions per (lane, t): one 16-byte load where the row is aligned and inside the tile.
    // kSoftWeights: the rows hold scores s in log2 units (absent positions count as -inf).
    const bool vec_ok = ((a.w_stride & 3) == 0) && ((reinterpret_cast<uintptr_t>(a.weights) & 15) == 0);   // uniform
    const float absent = (MODE == kSoftWeights) ? -INFINITY : 0.0f;     // positions outside the tile / heads past n_rep
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int row0 = wrow0 + 16 * t + 4 * g;
      const float* src = a.weights + (q_row0 + n16) * a.w_stride + tile_p0 + row0;
#pragma unroll
      for (int j = 0; j < 4; ++j) wgt[t][j] = absent;
      if (n16 < n_rep) {
        if (vec_ok && row0 + 4 <= rows_here) {
          // the thresholded step's own scores are read once here (streaming load: 23.6 -> 23.0 us per step); weights handed
          // in by a caller are usually fresh in the caches and keep the default policy (a streaming load costs 0.4 us there)
          const f4 v = (MODE == kSoftWeights) ? __builtin_nontemporal_load(reinterpret_cast<const f4*>(src))
                                              : *reinterpret_cast<const f4*>(src);
          wgt[t][0] = v[0]; wgt[t][1] = v[1]; wgt[t][2] = v[2]; wgt[t][3] = v[3];
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (row0 + j < rows_here) wgt[t][j] = src[j];
        }
      }
    }
    // kSoftWeights: the per-tile statistics, up to four tiles per thread at once (thread = head tid % 16, tiles
    // tid / 16 + 32 u: 128 tiles per sweep).  Requested LAST and folded after the value rows have been prepared: they
    // come back later than the rows (every workgroup of a kv head asks for the same few lines), and a wait for an
    // earlier request would wait for them too.
    if (MODE == kSoftWeights) {
      st_tiles = (int)((len + a.stats_tile_pos - 1) / a.stats_tile_pos);
      st_base = a.stats + (((int64_t)seq * a.n_kv + kvh) * a.n_stats_max) * (int64_t)(n_rep * 2);
      const int h = tid & 15, part = tid >> 4;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = part + 32 * u;
        st_ml[u] = (h < n_rep && t < st_tiles) ? *reinterpret_cast<const float2*>(st_base + (int64_t)t * (n_rep * 2) + 2 * h)
                                               : make_float2(-INFINITY, 0.0f);
      }
    }
  }
  if (HAS_K) { if (tid >= 64 && tid < 128) VF::fill(lutk_s, kcb, tid - 64); }
  if (HAS_V) { if (tid < 64) VF::fill(lutv_s, vcb, tid); }
  if (HAS_K) {
    if (a.q_raw) {
      rotate_query_rows<NW>(a.q_raw, a.q_dtype, a.k_signs, q_row0, n_rep, wave, lane, q_s, ql_s);
    } else {
#pragma unroll
      for (int i = 0; i < kQIt; ++i) {
        const __half2 h = __floats2half2_rn(my_q[i].x, my_q[i].y);
        const float2 back = __half22float2(h);
        (&q_s[0][0])[tid + i * kThr] = *reinterpret_cast<const uint32_t*>(&h);
        (&ql_s[0][0])[tid + i * kThr] = pack_h2(my_q[i].x - back.x, my_q[i].y - back.y);
      }
    }
    // the score scale rides on the key norm: log2 units for the softmax, plain units for kScores
    kn_s[wave][lane] = my_kn * (SOFT ? a.score_scale * kLog2e : a.score_scale);
  }
  if (HAS_V) vn_s[wave][lane] = my_vn;
  __syncthreads();

  uint32_t* stage = reinterpret_cast<uint32_t*>(big_s) + wave * 1024;

  // ---- V: norms, table indices --------------------------------------------------------------------------
  float vn[4][4];
  float inv_tscale = 1.0f, kexp = 0.0f;
  uint32_t VI[2][8];
  if (HAS_V) {
    float nmax = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float4 n4 = *reinterpret_cast<const float4*>(&vn_s[wave][16 * t + 4 * g]);
      vn[t][0] = n4.x; vn[t][1] = n4.y; vn[t][2] = n4.z; vn[t][3] = n4.w;
      nmax = fmaxf(nmax, fmaxf(fmaxf(n4.x, n4.y), fmaxf(n4.z, n4.w)));
    }
    nmax = fmaxf(nmax, shfl_xor_f(nmax, 16));
    nmax = fmaxf(nmax, shfl_xor_f(nmax, 32));
    int ex = (int)((__float_as_uint(nmax) >> 23) & 0xFF);
    ex = ex < 27 ? (ex < 1 ? 127 : 27) : (ex > 227 ? 227 : ex);
    kexp = (float)(127 - ex);                            // weights carry 2^kexp: through the exponent (kFlash) ...
    inv_tscale = __uint_as_float((uint32_t)ex << 23);
    if (GIVEN) {                                         // ... or, for given weights, on the norms
      const float tscale = __uint_as_float((uint32_t)(254 - ex) << 23);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) vn[t][j] *= tscale;
    }

    stage_block(vb_, stage, lane);
    int w0, sh_lo, sh_hi;
    VF::pos(n16, w0, sh_lo, sh_hi);
#pragma unroll
    for (int kb2 = 0; kb2 < 2; ++kb2) value_indices<BITS, VQUAD>(stage, kb2, g, w0, sh_lo, sh_hi, VI[kb2]);
  }

  // ---- K: scores ----------------------------------------------------------------------------------------
  float s[4][4];
  const bool mask_vec = a.mask && ((reinterpret_cast<uintptr_t>(a.mask) & 15) == 0) && ((a.mask_seq_stride & 3) == 0) &&
                        ((a.mask_head_stride & 3) == 0);      // uniform
  if (HAS_K) {
    u4 qreg[4], qlow[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      qreg[kb] = *reinterpret_cast<const u4*>(&q_s[n16][(4 * kb + g) * 4]);
      qlow[kb] = *reinterpret_cast<const u4*>(&ql_s[n16][(4 * kb + g) * 4]);
    }
    stage_block(kb_, stage, lane);                       // the V image has been consumed
    int kw0[4], ksl[4], ksh[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) VF::pos(4 * kb + g, kw0[kb], ksl[kb], ksh[kb]);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      f4 acc = {0.f, 0.f, 0.f, 0.f};
      const uint32_t* krow = stage + (16 * t + n16) * kVPd;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const uint32_t f = VF::field_raw(krow + kw0[kb], ksl[kb], ksh[kb]);
        const u4 ka = key_operand<BITS, KQUAD>(f, quad_s, lutk_s);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qreg[kb]),
                                                     acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qlow[kb]),
                                                     acc, 0, 0, 0);
      }
      const float4 kn4 = *reinterpret_cast<const float4*>(&kn_s[wave][16 * t + 4 * g]);
      const float knv[4] = {kn4.x, kn4.y, kn4.z, kn4.w};
      float mk[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (SOFT && a.mask && n16 < n_rep)
        load_mask4(a.mask + (int64_t)seq * a.mask_seq_stride + ((int64_t)kvh * n_rep + n16) * a.mask_head_stride + tile_p0 +
                       wrow0 + 16 * t + 4 * g, wrow0 + 16 * t + 4 * g, rows_here, mask_vec, mk);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int row = wrow0 + 16 * t + 4 * g + j;
        const float v = SOFT ? __builtin_fmaf(mk[j], kLog2e, acc[j] * knv[j]) : acc[j] * knv[j];
        s[t][j] = (row < rows_here) ? v : -INFINITY;
      }
    }
    if (MODE == kScores || MODE == kSoftScores) {
      // kSoftScores: softmax statistics of head n16 over the wave's 64 positions, combined over the waves below
      if (MODE == kSoftScores) {
        float m = -INFINITY;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) m = fmaxf(m, s[t][j]);
        m = fmaxf(m, shfl_xor_f(m, 16));
        m = fmaxf(m, shfl_xor_f(m, 32));
        const float msafe = (m == -INFINITY) ? 0.0f : m;
        float l = 0.0f;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) l += __builtin_amdgcn_exp2f(s[t][j] - msafe);
        l += shfl_xor_f(l, 16);
        l += shfl_xor_f(l, 32);
        if (g == 0) {
          m_s[wave][n16] = m;
          l_s[wave][n16] = l;
        }
      }
      // The wave's 64 x n_rep scores leave through its LDS area (the key image has been consumed), so that a
      // store instruction writes whole 256-byte runs of a head's row instead of 64 separate floats: the
      // area is [16 heads][16 units of 4 positions], the unit index xor-ed with the head (conflict-free
      // 16-byte accesses both ways).
      f4* sc = reinterpret_cast<f4*>(stage);
#pragma unroll
      for (int t = 0; t < 4; ++t) sc[n16 * 16 + ((4 * t + g) ^ n16)] = f4{s[t][0], s[t][1], s[t][2], s[t][3]};
      const int64_t row_len = (MODE == kSoftScores) ? a.w_stride : len;
      const bool vec_ok = ((row_len & 3) == 0) && ((reinterpret_cast<uintptr_t>(a.scores) & 15) == 0);   // uniform
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int h = 4 * i + g, unit = n16;                          // lane -> head 4i + lane / 16, positions 4 * (lane % 16) ..
        if (h < n_rep) {
          const f4 v = sc[h * 16 + (unit ^ h)];
          const int row0 = wrow0 + 4 * unit;
          float* dst = a.scores + ((MODE == kSoftScores ? q_row0 : (int64_t)kvh * n_rep) + h) * row_len + tile_p0 + row0;
          if (vec_ok && row0 + 4 <= rows_here) {
            // streaming stores: 10.9 -> 10.3 us for scores handed to the caller at 65 536 positions; the scores of a
            // thresholded step are read back by its next pass, from the memory side in either case
            __builtin_nontemporal_store(v, reinterpret_cast<f4*>(dst));
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (row0 + j < rows_here) dst[j] = v[j];
          }
        }
      }
      if (MODE == kSoftScores) {
        __syncthreads();
        if (tid < n_rep) {
          float M = m_s[0][tid];
#pragma unroll
          for (int w = 1; w < NW; ++w) M = fmaxf(M, m_s[w][tid]);
          float L = 0.0f;
#pragma unroll
          for (int w = 0; w < NW; ++w) {
            const float mw = m_s[w][tid];
            L += (mw == -INFINITY) ? 0.0f : l_s[w][tid] * __builtin_amdgcn_exp2f(mw - M);
          }
          float* pst = a.stats_out + ((((int64_t)seq * a.n_kv + kvh) * a.n_tiles_max) + tile) * (int64_t)(n_rep * 2);
          pst[2 * tid] = M;
          pst[2 * tid + 1] = L;
        }
      }
      return;
    }
  }

  if (GIVEN) {
    // kSoftWeights: the weight is 2^(s - M) / L with (M, L) of the whole sequence, folded here from the per-tile
    // pairs the scores pass left (every workgroup folds them itself: a few KB from L2).  Rows that are masked
    // out entirely (L = 0) get weight 0.
    float Mh = 0.0f, iL = 1.0f;
    if (MODE == kSoftWeights) {
      const int h = tid & 15, part = tid >> 4;
      float M = -INFINITY, L = 0.0f;
      auto fold = [&](const float2 ml) {
        const float Mn = fmaxf(M, ml.x);
        if (Mn != -INFINITY) {
          L = L * __builtin_amdgcn_exp2f(M - Mn) + ml.y * __builtin_amdgcn_exp2f(ml.x - Mn);
          M = Mn;
        }
      };
#pragma unroll
      for (int u = 0; u < 4; ++u) fold(st_ml[u]);
      if (h < n_rep) {
        for (int t = part + 128; t < st_tiles; t += 32)
          fold(*reinterpret_cast<const float2*>(st_base + (int64_t)t * (n_rep * 2) + 2 * h));
      }
      // the four threads of a head in this wave (lanes h + 16 k), then the eight waves through LDS; every thread
      // folds the eight pairs of ITS head (n16 = h) itself: one barrier, no serial pass over all parts
#pragma unroll
      for (int d = 16; d <= 32; d <<= 1) {
        const float Mo = shfl_xor_f(M, d), Lo = shfl_xor_f(L, d);
        const float Mn = fmaxf(M, Mo);
        if (Mn != -INFINITY) L = L * __builtin_amdgcn_exp2f(M - Mn) + Lo * __builtin_amdgcn_exp2f(Mo - Mn);
        M = Mn;
      }
      if (lane < kHeadsMax) {
        m_s[wave][lane] = M;
        l_s[wave][lane] = L;
      }
      __syncthreads();
      float Mt = -INFINITY;
#pragma unroll
      for (int w = 0; w < NW; ++w) Mt = fmaxf(Mt, m_s[w][n16]);
      float Lt = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float pm = m_s[w][n16];
        Lt += (pm == -INFINITY) ? 0.0f : l_s[w][n16] * __builtin_amdgcn_exp2f(pm - Mt);
      }
      Mh = (Mt == -INFINITY) ? 0.0f : Mt;
      iL = (Lt > 0.0f) ? 1.0f / Lt : 0.0f;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float w = wgt[t][j];
        if (MODE == kSoftWeights) w = __builtin_amdgcn_exp2f(w - Mh) * iL;
        wgt[t][j] = (w < a.threshold) ? 0.0f : w;
      }
  }

  // ---- weights of the value product -------------------------------------------------------------------
  float m = 0.0f, l = 0.0f;
  uint32_t pa[2][4];
  if (MODE == kFlash) {
    m = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) m = fmaxf(m, s[t][j]);
    m = fmaxf(m, shfl_xor_f(m, 16));
    m = fmaxf(m, shfl_xor_f(m, 32));
  }
  const float bias = kexp - ((m == -INFINITY) ? 0.0f : m);
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    float p[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      p[j] = (MODE == kFlash) ? __builtin_amdgcn_exp2f(s[t][j] + bias) : wgt[t][j];   // kFlash: weight * 2^kexp
      l += p[j];
      p[j] *= vn[t][j];
    }
    pa[t >> 1][2 * (t & 1)] = pack_h2(p[0], p[1]);
    pa[t >> 1][2 * (t & 1) + 1] = pack_h2(p[2], p[3]);
  }
  l += shfl_xor_f(l, 16);
  l += shfl_xor_f(l, 32);
  if (MODE == kFlash) l *= inv_tscale;

  // ---- values ------------------------------------------------------------------------------------------
  f4 accS[8];
#pragma unroll
  for (int et = 0; et < 8; ++et) accS[et] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kb2 = 0; kb2 < 2; ++kb2) {
    const u4 A = {pa[kb2][0], pa[kb2][1], pa[kb2][2], pa[kb2][3]};
    value_products<BITS, VQUAD>(A, VI[kb2], quad_s, lutv_s, accS);
  }

  // ---- merge the eight waves (merge_waves, tq_decode_mfma.h) ------------------------------------------------
  const int64_t grp = (int64_t)seq * a.n_kv + kvh;
  float* pS = a.ws_S + (grp * a.n_tiles_max + tile) * (int64_t)(n_rep * kD);
  float* pml = a.ws_ml + (grp * a.n_tiles_max + tile) * (int64_t)(n_rep * 2);
  merge_waves<NW>(mg_s, big_s, 4096, accS, m, l, inv_tscale, a.v_unscale, n_rep, pS, pml);
}

// Streaming flash-decode pass (packed K and V, no mask): a workgroup of FOUR waves runs through
// n_steps consecutive 256-position steps of one (sequence, kv head), a wave 64 positions per step,
// with the online-softmax recurrence in registers, and writes one partial at the end.  Two such
// workgroups share a CU, so the set-up and the cross-wave merge of one overlap the arithmetic of
// the other; the packed rows and norms of step s+1 are fetched into registers before step s is
// computed.  The fixed work of a tile (query staging, tables, merge, partial store) is paid once
// per n_steps * 256 positions and the merge pass sees that many fewer partials.
//
// Loads: at three bits a wave's 64 rows of 52 bytes start at an arbitrary multiple of 4 bytes (ragged
// batches start a sequence at any row).  They are fetched as ALIGNED 16-byte pieces from the 16-byte
// boundary at or below the first row (at most 209 pieces) into the wave's LDS image, and rows are
// read from the image at the misalignment offset.  An aligned 16-byte piece never crosses a page,
// so a piece that holds at least one valid byte is readable in full; a piece with no valid byte
// (rows past the end of the sequence) is replaced by the last piece that has one, and such rows get
// -inf scores.  Rows of the other widths are 16, 32 or 64 bytes: every row of a 16-byte aligned
// tensor is aligned (the host sends other tensors to the tile pass), and a block is 64, 128 or 256 pieces.
constexpr int kSWaves = 4;
constexpr int kSThreads = kSWaves * 64;
constexpr int kSStepPos = kSWaves * kWavePos;     // 256 positions per workgroup step
constexpr int kSImageBytes = 4096;                // 209 pieces of 16 bytes, rounded up; 256 pieces at four bits

template <int BITS, bool VQ = true>
__global__ __launch_bounds__(kSThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
void packed_stream_kernel(PackedArgs a, Codebook kcb, Codebook vcb, int n_steps) {
  using VF = VField<BITS>;
  // A workgroup decodes up to 8 x 256 positions, which repays building the quad table (one for keys and values when
  // their codebooks are equal, VQ; else the values use their pair table).
  constexpr bool KQUAD = VF::kQuad, VQUAD = VF::kQuad && VQ;
  constexpr int kPd = VF::kPd;                                  // words per packed row
  constexpr int kPieces = BITS == 3 ? 209 : 16 * kPd;           // 16-byte pieces of a wave's 64 rows (three bits: + misalignment)
  constexpr int kWhole = kPieces / 64, kRest = kPieces % 64;    // whole-wave stores into the image, lanes of the last one
  constexpr int kLoads = kWhole + (kRest ? 1 : 0);
  __shared__ __align__(16) unsigned char big_s[kSWaves * 2 * kSImageBytes];   // per wave: K image, V image; later S_all[4][8][128]
  __shared__ uint32_t lutk_s[VF::kLut < 64 ? 64 : VF::kLut], lutv_s[VF::kLut < 64 ? 64 : VF::kLut];
  __shared__ __align__(16) uint2 quad_s[KQUAD ? VF::kQuadEntries : 1];
  __shared__ __align__(16) uint32_t q_s[kHeadsMax][kD / 2];
  __shared__ __align__(16) uint32_t ql_s[kHeadsMax][kD / 2];
  __shared__ __align__(16) float kn_s[kSWaves][kWavePos], vn_s[kSWaves][kWavePos];
  __shared__ __align__(16) float alpha_s[kSWaves][kHeadsMax];
  __shared__ __align__(16) MergeLds<kSWaves> mg_s;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int wg = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
  const int n_rep = a.n_rep;
  const int n_q = a.n_kv * n_rep;
  const int64_t q_row0 = (int64_t)seq * n_q + (int64_t)kvh * n_rep;

  int64_t first = 0, len = a.seq_len;
  if (a.seq_offsets) {
    first = a.seq_offsets[seq];
    len = (int64_t)a.seq_offsets[seq + 1] - first;
  } else if (a.len_dev) {
    const int64_t want = *a.len_dev + a.len_bias;
    len = want < 0 ? 0 : (want < len ? want : len);
  }
  const int64_t wg_p0 = (int64_t)wg * kSStepPos * n_steps;
  if (wg_p0 >= len) return;

  // ---- addresses: row 0 of the sequence for this kv head, misalignment of the wave's blocks
  const char* krow0 = reinterpret_cast<const char*>(
      a.k_packed + ((int64_t)seq * a.k_seq_stride + (int64_t)kvh * a.k_head_stride + first) * kPd);
  const char* vrow0 = reinterpret_cast<const char*>(
      a.v_packed + ((int64_t)seq * a.v_seq_stride + (int64_t)kvh * a.v_head_stride + first) * kPd);
  // every block of this workgroup starts a multiple of 64 rows = 208 pieces after row wg_p0: one misalignment
  const int kmis = BITS == 3 ? (int)((reinterpret_cast<uintptr_t>(krow0) + (uint64_t)wg_p0 * (kPd * 4)) & 15) : 0;
  const int vmis = BITS == 3 ? (int)((reinterpret_cast<uintptr_t>(vrow0) + (uint64_t)wg_p0 * (kPd * 4)) & 15) : 0;
  const float* knrow0 = a.k_norms + (int64_t)seq * a.kn_seq_stride + (int64_t)kvh * a.kn_head_stride + first;
  const float* vnrow0 = a.v_norms + (int64_t)seq * a.vn_seq_stride + (int64_t)kvh * a.vn_head_stride + first;

  auto rows_left_of = [&](int s) {
    const int64_t p0w = wg_p0 + (int64_t)s * kSStepPos + wave * kWavePos;
    const int64_t left = s < n_steps ? len - p0w : 0;      // steps past the workgroup's last have no rows
    return (int)(left < 0 ? 0 : (left > kWavePos ? kWavePos : left));
  };
  // Requests the rows of step s.  Every call issues the same loads whatever s is: a piece past the end of the sequence
  // is fetched from the last piece of the block that holds a valid byte, a norm past the end (and everything of a step
  // past the workgroup's last) from the first piece / row of the workgroup's range, which exists, so that no branch
  // surrounds a load -- the compiler can then count the requests in flight and wait for one buffer's rows while the
  // other buffer's are still on their way.  What comes back for a row that does not exist is real data of another row:
  // finite, and its score is set to -inf.
  // Addresses are a base that is the same for the whole workgroup (its first piece / first norm) plus a 32-bit
  // offset per lane: one register per load instead of a 64-bit pointer.
  const char* k_base = krow0 + wg_p0 * (kPd * 4) - kmis;
  const char* v_base = vrow0 + wg_p0 * (kPd * 4) - vmis;
  const float* kn_base = knrow0 + wg_p0;
  const float* vn_base = vnrow0 + wg_p0;
  auto issue = [&](int s, u4 (&kq)[kLoads], u4 (&vq)[kLoads], float& kn, float& vn) {
    const uint32_t row0 = (uint32_t)(s * kSStepPos + wave * kWavePos);   // first row of the wave's block, from wg_p0
    const int rows = rows_left_of(s);
    // offset of the last piece that holds a valid byte (pieces past it are fetched from there), first byte of the block
    const uint32_t klast = rows ? ((uint32_t)(kmis + rows * (kPd * 4) - 1) & ~15u) : 0u;
    const uint32_t vlast = rows ? ((uint32_t)(vmis + rows * (kPd * 4) - 1) & ~15u) : 0u;
    const uint32_t blk = rows ? row0 * (kPd * 4) : 0u;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const uint32_t off = (uint32_t)(i * 64 + lane) * 16;
      kq[i] = load_stream(k_base + (blk + min(off, klast)));
      vq[i] = load_stream(v_base + (blk + min(off, vlast)));
    }
    const uint32_t nrow = (lane < rows) ? row0 + lane : 0u;
    kn = load_stream(kn_base + nrow);
    vn = load_stream(vn_base + nrow);
  };

  float2 my_q[4];
  if (!a.q_raw) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int w = tid + i * kSThreads;                                  // word = 2 consecutive elements
      my_q[i] = (w < n_rep * (kD / 2)) ? reinterpret_cast<const float2*>(a.q_rot + q_row0 * kD)[w] : make_float2(0.f, 0.f);
    }
  }
  u4 kqA[kLoads], vqA[kLoads], kqB[kLoads], vqB[kLoads];
  float knA, vnA, knB = 0.0f, vnB = 0.0f;
  issue(0, kqA, vqA, knA, vnA);

  if (tid < 64) VF::fill(lutk_s, kcb, tid);
  else if (tid < 128) VF::fill(lutv_s, vcb, tid - 64);
  if (a.q_raw) {
    rotate_query_rows<kSWaves>(a.q_raw, a.q_dtype, a.k_signs, q_row0, n_rep, wave, lane, q_s, ql_s);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const __half2 h = __floats2half2_rn(my_q[i].x, my_q[i].y);
      const float2 back = __half22float2(h);
      (&q_s[0][0])[tid + i * kSThreads] = *reinterpret_cast<const uint32_t*>(&h);
      (&ql_s[0][0])[tid + i * kSThreads] = pack_h2(my_q[i].x - back.x, my_q[i].y - back.y);
    }
  }
  __syncthreads();
  if (KQUAD) {
    VF::fill_quad(quad_s, lutk_s, tid, kSThreads);
    __syncthreads();
  }

  u4 qreg[4], qlow[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    qreg[kb] = *reinterpret_cast<const u4*>(&q_s[n16][(4 * kb + g) * 4]);
    qlow[kb] = *reinterpret_cast<const u4*>(&ql_s[n16][(4 * kb + g) * 4]);
  }
  unsigned char* image = big_s + wave * (2 * kSImageBytes);
  const uint32_t* kimg = reinterpret_cast<const uint32_t*>(image + kmis);
  const uint32_t* vimg = reinterpret_cast<const uint32_t*>(image + kSImageBytes + vmis);
  int kw0[4], ksl[4], ksh[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) VF::pos(4 * kb + g, kw0[kb], ksl[kb], ksh[kb]);
  int vw0, vsl, vsh;
  VF::pos(n16, vw0, vsl, vsh);
  const float kscale = a.score_scale * kLog2e;           // scores in log2 units

  f4 accS[8];
#pragma unroll
  for (int et = 0; et < 8; ++et) accS[et] = f4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, R_run = -INFINITY, l_run = 0.0f, inv_tscale = 1.0f;

  // one step on the buffers (kq, vq, kn, vn); `next()` issues the loads of the following step
  auto step = [&](int sidx, u4 (&kq)[kLoads], u4 (&vq)[kLoads], float kn, float vn_, auto&& next) {
    const int rows = rows_left_of(sidx);                 // uniform over the wave, at least 1 (the caller checks)
    // ---- the request for the next step's rows goes out first (the other buffer is free): what separates the arrival
    // of one step's rows from the request for the next is on the critical path of a loop that a memory round trip bounds
    __builtin_amdgcn_sched_barrier(0);
    next();
    __builtin_amdgcn_sched_barrier(0);
    // ---- images and norms into the wave's LDS area
    {
      u4* k4 = reinterpret_cast<u4*>(image);
      u4* v4 = reinterpret_cast<u4*>(image + kSImageBytes);
#pragma unroll
      for (int i = 0; i < kWhole; ++i) { k4[i * 64 + lane] = kq[i]; v4[i * 64 + lane] = vq[i]; }
      if (kRest) { if (lane < kRest) { k4[kWhole * 64 + lane] = kq[kLoads - 1]; v4[kWhole * 64 + lane] = vq[kLoads - 1]; } }
      kn_s[wave][lane] = kn * kscale;
      vn_s[wave][lane] = vn_;
    }
    // ---- scores of the 64 rows (log2 units)
    float s[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      f4 acc = {0.f, 0.f, 0.f, 0.f};
      const uint32_t* krow = kimg + (16 * t + n16) * kPd;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const uint32_t f = VF::field_raw(krow + kw0[kb], ksl[kb], ksh[kb]);
        const u4 ka = key_operand<BITS, KQUAD>(f, quad_s, lutk_s);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qreg[kb]),
                                                     acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qlow[kb]),
                                                     acc, 0, 0, 0);
      }
      const float4 kn4 = *reinterpret_cast<const float4*>(&kn_s[wave][16 * t + 4 * g]);
      const float knv[4] = {kn4.x, kn4.y, kn4.z, kn4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) s[t][j] = acc[j] * knv[j];
    }
    if (rows < kWavePos) {                                 // only a sequence's last block has rows to mask
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) s[t][j] = (16 * t + 4 * g + j < rows) ? s[t][j] : -INFINITY;
    }
    // ---- value norms, their power-of-two scale
    float vn[4][4];
    float nmax = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float4 n4 = *reinterpret_cast<const float4*>(&vn_s[wave][16 * t + 4 * g]);
      vn[t][0] = n4.x; vn[t][1] = n4.y; vn[t][2] = n4.z; vn[t][3] = n4.w;
      nmax = fmaxf(nmax, fmaxf(fmaxf(n4.x, n4.y), fmaxf(n4.z, n4.w)));
    }
    nmax = max_over_rows(nmax);
    int ex = (int)((__float_as_uint(nmax) >> 23) & 0xFF);
    ex = ex < 27 ? (ex < 1 ? 127 : 27) : (ex > 227 ? 227 : ex);
    const float kexp = (float)(127 - ex);
    inv_tscale = __uint_as_float((uint32_t)ex << 23);
    // ---- online softmax: rows >= 1, so the maximum of the step is finite
    float mb = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) mb = fmaxf(mb, s[t][j]);
    mb = max_over_rows(mb);
    const float m_new = fmaxf(m_run, mb);
    const float R_new = m_new - kexp;
    const float factor = __builtin_amdgcn_exp2f(R_run - R_new);      // 0 on the wave's first step
    m_run = m_new;
    R_run = R_new;
    float lsum = 0.0f;
    uint32_t pa[2][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      float p[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        p[j] = __builtin_amdgcn_exp2f(s[t][j] - R_new);              // weight * 2^kexp
        lsum += p[j];
        p[j] *= vn[t][j];
      }
      pa[t >> 1][2 * (t & 1)] = pack_h2(p[0], p[1]);
      pa[t >> 1][2 * (t & 1) + 1] = pack_h2(p[2], p[3]);
    }
    l_run = l_run * factor + lsum;
    if (sidx > 0 && __any(factor != 1.0f)) {               // accumulator rows are heads 4g + j: factors through LDS
      if (g == 0) alpha_s[wave][n16] = factor;
      const float4 a4 = *reinterpret_cast<const float4*>(&alpha_s[wave][4 * g]);
      const float av[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
      for (int et = 0; et < 8; ++et)
#pragma unroll
        for (int j = 0; j < 4; ++j) accS[et][j] *= av[j];
    }
    // ---- values: packed V -> interleaved table indices -> centroids, 32 positions at a time
#pragma unroll
    for (int kb2 = 0; kb2 < 2; ++kb2) {
      uint32_t VI[8];
      value_indices<BITS, VQUAD>(vimg, kb2, g, vw0, vsl, vsh, VI);
      const u4 A = {pa[kb2][0], pa[kb2][1], pa[kb2][2], pa[kb2][3]};
      value_products<BITS, VQUAD>(A, VI, quad_s, lutv_s, accS);
    }
  };

  // Steps come in pairs so that the two register buffers keep their names; the rows of step s + 1 are requested as
  // the first thing step s does.  A wave stops at its first step without rows (steps only run out at the end of the
  // sequence).
  for (int sidx = 0; sidx < n_steps; sidx += 2) {
    if (rows_left_of(sidx) <= 0) break;
    step(sidx, kqA, vqA, knA, vnA, [&]() { issue(sidx + 1, kqB, vqB, knB, vnB); });
    if (sidx + 1 >= n_steps || rows_left_of(sidx + 1) <= 0) break;
    step(sidx + 1, kqB, vqB, knB, vnB, [&]() { issue(sidx + 2, kqA, vqA, knA, vnA); });
  }


  // ---- merge the four waves (merge_waves): a wave deposits into its own image area.  A wave that saw no valid
  // row has m = -inf, l = 0 and zero accumulators.
  float l = l_run;
  l += shfl_xor_f(l, 16);
  l += shfl_xor_f(l, 32);
  l *= inv_tscale;
  const int64_t grp = (int64_t)seq * a.n_kv + kvh;
  float* pS = a.ws_S + (grp * a.n_tiles_max + wg) * (int64_t)(n_rep * kD);
  float* pml = a.ws_ml + (grp * a.n_tiles_max + wg) * (int64_t)(n_rep * 2);
  static_assert(2 * kSImageBytes >= 8 * kD * 4 && (2 * kSImageBytes) % 16 == 0, "a wave's image area holds its eight deposit rows");
  merge_waves<kSWaves>(mg_s, big_s, 2 * kSImageBytes, accS, m_run, l, inv_tscale, a.v_unscale, n_rep, pS, pml);
}

// Scores pass of the thresholded flash step in the streaming form (packed K, no mask): the key half of
// packed_stream_kernel.  A workgroup of four waves runs through n_steps consecutive 256-position steps of one
// (sequence, kv head); a wave writes the scores of its 64 rows (log2 units) through its LDS area in 256-byte runs per
// head and keeps the running (maximum, sum of 2^(s - maximum)) of its rows; at the end the four waves are folded into
// ONE pair per head for the workgroup's range (a.stats_out, [n_seq * n_kv, n_tiles_max, n_rep, 2]), so the weights
// pass has n_steps * 256 positions per statistics entry.
template <int BITS>
__global__ __launch_bounds__(kSThreads) __attribute__((amdgpu_waves_per_eu(3, 3)))
void packed_stream_scores_kernel(PackedArgs a, Codebook kcb, int n_steps) {
  using VF = VField<BITS>;
  constexpr bool KQUAD = VF::kQuad;
  constexpr int kPd = VF::kPd;
  constexpr int kPieces = BITS == 3 ? 209 : 16 * kPd;
  constexpr int kWhole = kPieces / 64, kRest = kPieces % 64;
  constexpr int kLoads = kWhole + (kRest ? 1 : 0);
  __shared__ __align__(16) unsigned char big_s[kSWaves * kSImageBytes];   // per wave: K image, then its 64 x 16 scores
  __shared__ uint32_t lutk_s[VF::kLut < 64 ? 64 : VF::kLut];
  __shared__ __align__(16) uint2 quad_s[KQUAD ? VF::kQuadEntries : 1];
  // the rotated query (fp16 value and remainder, 8 KB) is staged in the image area: it is in registers before any image is written
  uint32_t (*q_s)[kD / 2] = reinterpret_cast<uint32_t (*)[kD / 2]>(big_s);
  uint32_t (*ql_s)[kD / 2] = reinterpret_cast<uint32_t (*)[kD / 2]>(big_s + kHeadsMax * (kD / 2) * 4);
  __shared__ __align__(16) float kn_s[kSWaves][kWavePos];
  __shared__ float m_s[kSWaves][kHeadsMax], l_s[kSWaves][kHeadsMax];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int wg = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
  const int n_rep = a.n_rep;
  const int n_q = a.n_kv * n_rep;
  const int64_t q_row0 = (int64_t)seq * n_q + (int64_t)kvh * n_rep;

  int64_t first = 0, len = a.seq_len;
  if (a.seq_offsets) {
    first = a.seq_offsets[seq];
    len = (int64_t)a.seq_offsets[seq + 1] - first;
  }
  const int64_t wg_p0 = (int64_t)wg * kSStepPos * n_steps;
  if (wg_p0 >= len) return;                              // the weights pass never reads this entry

  const char* krow0 = reinterpret_cast<const char*>(
      a.k_packed + ((int64_t)seq * a.k_seq_stride + (int64_t)kvh * a.k_head_stride + first) * kPd);
  const int kmis = BITS == 3 ? (int)((reinterpret_cast<uintptr_t>(krow0) + (uint64_t)wg_p0 * (kPd * 4)) & 15) : 0;
  const float* knrow0 = a.k_norms + (int64_t)seq * a.kn_seq_stride + (int64_t)kvh * a.kn_head_stride + first;
  auto rows_left_of = [&](int s) {
    const int64_t p0w = wg_p0 + (int64_t)s * kSStepPos + wave * kWavePos;
    const int64_t left = s < n_steps ? len - p0w : 0;
    return (int)(left < 0 ? 0 : (left > kWavePos ? kWavePos : left));
  };
  // requests as in packed_stream_kernel: the same loads whatever s is, no branch around a load
  const char* k_base = krow0 + wg_p0 * (kPd * 4) - kmis;
  const float* kn_base = knrow0 + wg_p0;
  auto issue = [&](int s, u4 (&kq)[kLoads], float& kn) {
    const uint32_t row0 = (uint32_t)(s * kSStepPos + wave * kWavePos);
    const int rows = rows_left_of(s);
    const uint32_t klast = rows ? ((uint32_t)(kmis + rows * (kPd * 4) - 1) & ~15u) : 0u;
    const uint32_t blk = rows ? row0 * (kPd * 4) : 0u;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const uint32_t off = (uint32_t)(i * 64 + lane) * 16;
      kq[i] = load_stream(k_base + (blk + min(off, klast)));
    }
    kn = load_stream(kn_base + ((lane < rows) ? row0 + lane : 0u));
  };

  float2 my_q[4];
  if (!a.q_raw) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int w = tid + i * kSThreads;
      my_q[i] = (w < n_rep * (kD / 2)) ? reinterpret_cast<const float2*>(a.q_rot + q_row0 * kD)[w] : make_float2(0.f, 0.f);
    }
  }
  u4 kqA[kLoads], kqB[kLoads];
  float knA, knB = 0.0f;
  issue(0, kqA, knA);

  if (tid < 64) VF::fill(lutk_s, kcb, tid);
  if (a.q_raw) {
    rotate_query_rows<kSWaves>(a.q_raw, a.q_dtype, a.k_signs, q_row0, n_rep, wave, lane, q_s, ql_s);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const __half2 h = __floats2half2_rn(my_q[i].x, my_q[i].y);
      const float2 back = __half22float2(h);
      (&q_s[0][0])[tid + i * kSThreads] = *reinterpret_cast<const uint32_t*>(&h);
      (&ql_s[0][0])[tid + i * kSThreads] = pack_h2(my_q[i].x - back.x, my_q[i].y - back.y);
    }
  }
  __syncthreads();
  u4 qreg[4], qlow[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    qreg[kb] = *reinterpret_cast<const u4*>(&q_s[n16][(4 * kb + g) * 4]);
    qlow[kb] = *reinterpret_cast<const u4*>(&ql_s[n16][(4 * kb + g) * 4]);
  }
  if (KQUAD) VF::fill_quad(quad_s, lutk_s, tid, kSThreads);
  __syncthreads();                                       // every wave has its query operands: the image area is free
  unsigned char* image = big_s + wave * kSImageBytes;
  const uint32_t* kimg = reinterpret_cast<const uint32_t*>(image + kmis);
  int kw0[4], ksl[4], ksh[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) VF::pos(4 * kb + g, kw0[kb], ksl[kb], ksh[kb]);
  const float kscale = a.score_scale * kLog2e;           // scores in log2 units
  const bool vec_ok = ((a.w_stride & 3) == 0) && ((reinterpret_cast<uintptr_t>(a.scores) & 15) == 0);   // uniform
  float m_run = -INFINITY, l_run = 0.0f;

  auto step = [&](int sidx, u4 (&kq)[kLoads], float kn, auto&& next) {
    const int rows = rows_left_of(sidx);                 // uniform over the wave, at least 1 (the caller checks)
    __builtin_amdgcn_sched_barrier(0);
    next();
    __builtin_amdgcn_sched_barrier(0);
    {
      u4* k4 = reinterpret_cast<u4*>(image);
#pragma unroll
      for (int i = 0; i < kWhole; ++i) k4[i * 64 + lane] = kq[i];
      if (kRest) { if (lane < kRest) k4[kWhole * 64 + lane] = kq[kLoads - 1]; }
      kn_s[wave][lane] = kn * kscale;
    }
    float s[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      f4 acc = {0.f, 0.f, 0.f, 0.f};
      const uint32_t* krow = kimg + (16 * t + n16) * kPd;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const uint32_t f = VF::field_raw(krow + kw0[kb], ksl[kb], ksh[kb]);
        const u4 ka = key_operand<BITS, KQUAD>(f, quad_s, lutk_s);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qreg[kb]),
                                                     acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qlow[kb]),
                                                     acc, 0, 0, 0);
      }
      const float4 kn4 = *reinterpret_cast<const float4*>(&kn_s[wave][16 * t + 4 * g]);
      const float knv[4] = {kn4.x, kn4.y, kn4.z, kn4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) s[t][j] = acc[j] * knv[j];
    }
    if (rows < kWavePos) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) s[t][j] = (16 * t + 4 * g + j < rows) ? s[t][j] : -INFINITY;
    }
    // ---- running statistics of head n16 (rows >= 1: the maximum of the step is finite)
    float mb = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) mb = fmaxf(mb, s[t][j]);
    mb = max_over_rows(mb);
    const float m_new = fmaxf(m_run, mb);
    float lsum = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) lsum += __builtin_amdgcn_exp2f(s[t][j] - m_new);
    l_run = l_run * __builtin_amdgcn_exp2f(m_run - m_new) + lsum;       // 2^(-inf) = 0 on the wave's first step
    m_run = m_new;
    // ---- the scores leave through the wave's LDS area (the key image has been consumed): [16 heads][16 units of
    // four positions], the unit index xor-ed with the head, so that a store instruction writes 256-byte runs
    f4* sc = reinterpret_cast<f4*>(image);
#pragma unroll
    for (int t = 0; t < 4; ++t) sc[n16 * 16 + ((4 * t + g) ^ n16)] = f4{s[t][0], s[t][1], s[t][2], s[t][3]};
    const int64_t p0w = wg_p0 + (int64_t)sidx * kSStepPos + wave * kWavePos;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int h = 4 * i + g, unit = n16;
      if (h < n_rep) {
        const f4 v = sc[h * 16 + (unit ^ h)];
        float* dst = a.scores + (q_row0 + h) * a.w_stride + p0w + 4 * unit;
        if (vec_ok && 4 * unit + 4 <= rows) {
          __builtin_nontemporal_store(v, reinterpret_cast<f4*>(dst));
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (4 * unit + j < rows) dst[j] = v[j];
        }
      }
    }
  };

  for (int sidx = 0; sidx < n_steps; sidx += 2) {
    if (rows_left_of(sidx) <= 0) break;
    step(sidx, kqA, knA, [&]() { issue(sidx + 1, kqB, knB); });
    if (sidx + 1 >= n_steps || rows_left_of(sidx + 1) <= 0) break;
    step(sidx + 1, kqB, knB, [&]() { issue(sidx + 2, kqA, knA); });
  }

  // ---- one (maximum, sum) pair per head for the workgroup's range; a wave without rows has (-inf, 0)
  float l = l_run;
  l += shfl_xor_f(l, 16);
  l += shfl_xor_f(l, 32);
  if (g == 0) {
    m_s[wave][n16] = m_run;
    l_s[wave][n16] = l;
  }
  __syncthreads();
  if (tid < n_rep) {
    float M = m_s[0][tid];
#pragma unroll
    for (int w = 1; w < kSWaves; ++w) M = fmaxf(M, m_s[w][tid]);
    float L = 0.0f;
#pragma unroll
    for (int w = 0; w < kSWaves; ++w) {
      const float mw = m_s[w][tid];
      L += (mw == -INFINITY) ? 0.0f : l_s[w][tid] * __builtin_amdgcn_exp2f(mw - M);
    }
    float* pst = a.stats_out + ((((int64_t)seq * a.n_kv + kvh) * a.n_tiles_max) + wg) * (int64_t)(n_rep * 2);
    pst[2 * tid] = M;
    pst[2 * tid + 1] = L;
  }
}

// Weights-and-values pass of the thresholded steps in the streaming form (packed V, scores and per-range statistics
// from a scores pass): the value half of packed_stream_kernel.  Every workgroup first folds the statistics of its
// (sequence, kv head) into (M, L) per head; a wave then forms w = 2^(s - M) / L for its 64 rows per step, drops
// w < threshold, and sums w * norm * centroids on the matrix cores.  No softmax recurrence: the weights are final.
// What does move from step to step is the power-of-two scale that keeps w * norm inside fp16 (taken from the largest
// value norm seen so far); the accumulators are rescaled when it grows.  The partial of a workgroup is a plain
// weighted sum (maximum 0), folded by the merge pass without normalisation.
template <int BITS>
__global__ __launch_bounds__(kSThreads) __attribute__((amdgpu_waves_per_eu(3, 3)))
void packed_stream_weights_kernel(PackedArgs a, Codebook vcb, int n_steps) {
  using VF = VField<BITS>;
  constexpr bool VQUAD = VF::kQuad;
  constexpr int kPd = VF::kPd;
  constexpr int kPieces = BITS == 3 ? 209 : 16 * kPd;
  constexpr int kWhole = kPieces / 64, kRest = kPieces % 64;
  constexpr int kLoads = kWhole + (kRest ? 1 : 0);
  __shared__ __align__(16) unsigned char big_s[kSWaves * kSImageBytes];   // per wave: V image; later its eight deposit rows
  __shared__ uint32_t lutv_s[VF::kLut < 64 ? 64 : VF::kLut];
  __shared__ __align__(16) uint2 quad_s[VQUAD ? VF::kQuadEntries : 1];
  __shared__ __align__(16) float vn_s[kSWaves][kWavePos];
  __shared__ float m_s[kSWaves][kHeadsMax], l_s[kSWaves][kHeadsMax];
  __shared__ __align__(16) MergeLds<kSWaves> mg_s;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int wg = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
  const int n_rep = a.n_rep;
  const int n_q = a.n_kv * n_rep;
  const int64_t q_row0 = (int64_t)seq * n_q + (int64_t)kvh * n_rep;

  int64_t first = 0, len = a.seq_len;
  if (a.seq_offsets) {
    first = a.seq_offsets[seq];
    len = (int64_t)a.seq_offsets[seq + 1] - first;
  }
  const int64_t wg_p0 = (int64_t)wg * kSStepPos * n_steps;
  if (wg_p0 >= len) return;

  const char* vrow0 = reinterpret_cast<const char*>(
      a.v_packed + ((int64_t)seq * a.v_seq_stride + (int64_t)kvh * a.v_head_stride + first) * kPd);
  const int vmis = BITS == 3 ? (int)((reinterpret_cast<uintptr_t>(vrow0) + (uint64_t)wg_p0 * (kPd * 4)) & 15) : 0;
  const float* vnrow0 = a.v_norms + (int64_t)seq * a.vn_seq_stride + (int64_t)kvh * a.vn_head_stride + first;
  auto rows_left_of = [&](int s) {
    const int64_t p0w = wg_p0 + (int64_t)s * kSStepPos + wave * kWavePos;
    const int64_t left = s < n_steps ? len - p0w : 0;
    return (int)(left < 0 ? 0 : (left > kWavePos ? kWavePos : left));
  };
  // Requests of a step: the same loads whatever s is, no branch around a load (see packed_stream_kernel).  The scores
  // of head n16 (heads past n_rep: head 0) at positions 16 t + 4 g .. + 3 of the wave's rows come as one 16-byte
  // piece per t (rows of `weights` are w_stride floats, a multiple of four, from a 16-byte aligned base; a row's
  // padding and the pieces of blocks past the end are read and then masked).
  const char* v_base = vrow0 + wg_p0 * (kPd * 4) - vmis;
  const float* vn_base = vnrow0 + wg_p0;
  const float* sc_base = a.weights + (q_row0 + (n16 < n_rep ? n16 : 0)) * a.w_stride + wg_p0;
  const bool vec_ok = ((a.w_stride & 3) == 0) && ((reinterpret_cast<uintptr_t>(a.weights) & 15) == 0);   // uniform
  auto issue = [&](int s, u4 (&vq)[kLoads], float& vn, f4 (&sc)[4]) {
    const uint32_t row0 = (uint32_t)(s * kSStepPos + wave * kWavePos);
    const int rows = rows_left_of(s);
    const uint32_t vlast = rows ? ((uint32_t)(vmis + rows * (kPd * 4) - 1) & ~15u) : 0u;
    const uint32_t blk = rows ? row0 * (kPd * 4) : 0u;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const uint32_t off = (uint32_t)(i * 64 + lane) * 16;
      vq[i] = load_stream(v_base + (blk + min(off, vlast)));
    }
    vn = load_stream(vn_base + ((lane < rows) ? row0 + lane : 0u));
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint32_t at = (16 * t + 4 * g < rows) ? row0 + 16 * t + 4 * g : 0u;   // a piece with no valid position: the range's first
      if (vec_ok) {
        sc[t] = __builtin_nontemporal_load(reinterpret_cast<const f4*>(sc_base + at));
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) sc[t][j] = sc_base[at + (16 * t + 4 * g + j < rows ? j : 0)];
      }
    }
  };

  // ---- statistics of this (sequence, kv head): thread = head tid % 16, entries tid / 16 + 16 u
  float2 st_ml[4];
  const int st_tiles = (int)((len + a.stats_tile_pos - 1) / a.stats_tile_pos);
  const float* st_base = a.stats + (((int64_t)seq * a.n_kv + kvh) * a.n_stats_max) * (int64_t)(n_rep * 2);
  {
    const int h = tid & 15, part = tid >> 4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int t = part + 16 * u;
      st_ml[u] = (h < n_rep && t < st_tiles) ? *reinterpret_cast<const float2*>(st_base + (int64_t)t * (n_rep * 2) + 2 * h)
                                             : make_float2(-INFINITY, 0.0f);
    }
  }
  u4 vqA[kLoads], vqB[kLoads];
  float vnA, vnB = 0.0f;
  f4 scA[4], scB[4];
  issue(0, vqA, vnA, scA);

  if (tid < 64) VF::fill(lutv_s, vcb, tid);
  float Mh, iL;
  {
    const int h = tid & 15, part = tid >> 4;
    float M = -INFINITY, L = 0.0f;
    auto fold = [&](const float2 ml) {
      const float Mn = fmaxf(M, ml.x);
      if (Mn != -INFINITY) {
        L = L * __builtin_amdgcn_exp2f(M - Mn) + ml.y * __builtin_amdgcn_exp2f(ml.x - Mn);
        M = Mn;
      }
    };
#pragma unroll
    for (int u = 0; u < 4; ++u) fold(st_ml[u]);
    if (h < n_rep) {
      for (int t = part + 64; t < st_tiles; t += 16)
        fold(*reinterpret_cast<const float2*>(st_base + (int64_t)t * (n_rep * 2) + 2 * h));
    }
#pragma unroll
    for (int d = 16; d <= 32; d <<= 1) {
      const float Mo = shfl_xor_f(M, d), Lo = shfl_xor_f(L, d);
      const float Mn = fmaxf(M, Mo);
      if (Mn != -INFINITY) L = L * __builtin_amdgcn_exp2f(M - Mn) + Lo * __builtin_amdgcn_exp2f(Mo - Mn);
      M = Mn;
    }
    if (lane < kHeadsMax) {
      m_s[wave][lane] = M;
      l_s[wave][lane] = L;
    }
  }
  __syncthreads();
  {
    float Mt = -INFINITY;
#pragma unroll
    for (int w = 0; w < kSWaves; ++w) Mt = fmaxf(Mt, m_s[w][n16]);
    float Lt = 0.0f;
#pragma unroll
    for (int w = 0; w < kSWaves; ++w) {
      const float pm = m_s[w][n16];
      Lt += (pm == -INFINITY) ? 0.0f : l_s[w][n16] * __builtin_amdgcn_exp2f(pm - Mt);
    }
    Mh = (Mt == -INFINITY) ? 0.0f : Mt;
    iL = (Lt > 0.0f) ? 1.0f / Lt : 0.0f;                  // rows that are masked out entirely: weight 0
  }
  if (VQUAD) {
    VF::fill_quad(quad_s, lutv_s, tid, kSThreads);
    __syncthreads();
  }

  unsigned char* image = big_s + wave * kSImageBytes;
  const uint32_t* vimg = reinterpret_cast<const uint32_t*>(image + vmis);
  int vw0, vsl, vsh;
  VF::pos(n16, vw0, vsl, vsh);
  const bool head_ok = n16 < n_rep;

  f4 accS[8];
#pragma unroll
  for (int et = 0; et < 8; ++et) accS[et] = f4{0.f, 0.f, 0.f, 0.f};
  int ex_run = 27;                                          // exponent of the scale of the value norms, only grows

  auto step = [&](int sidx, u4 (&vq)[kLoads], float vn_, f4 (&sc)[4], auto&& next) {
    const int rows = rows_left_of(sidx);                 // uniform over the wave, at least 1 (the caller checks)
    __builtin_amdgcn_sched_barrier(0);
    next();
    __builtin_amdgcn_sched_barrier(0);
    {
      u4* v4 = reinterpret_cast<u4*>(image);
#pragma unroll
      for (int i = 0; i < kWhole; ++i) v4[i * 64 + lane] = vq[i];
      if (kRest) { if (lane < kRest) v4[kWhole * 64 + lane] = vq[kLoads - 1]; }
      vn_s[wave][lane] = vn_;
    }
    // ---- value norms, their power-of-two scale (as the tile pass takes it, here a running maximum)
    float vn[4][4];
    float nmax = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float4 n4 = *reinterpret_cast<const float4*>(&vn_s[wave][16 * t + 4 * g]);
      vn[t][0] = n4.x; vn[t][1] = n4.y; vn[t][2] = n4.z; vn[t][3] = n4.w;
      nmax = fmaxf(nmax, fmaxf(fmaxf(n4.x, n4.y), fmaxf(n4.z, n4.w)));
    }
    nmax = max_over_rows(nmax);
    int ex = (int)((__float_as_uint(nmax) >> 23) & 0xFF);
    ex = ex < 27 ? (ex < 1 ? 127 : 27) : (ex > 227 ? 227 : ex);
    if (sidx == 0) ex_run = ex;
    if (ex > ex_run) {                                     // uniform: the scale grows, what has been summed shrinks
      const float shrink = (ex - ex_run < 127) ? __uint_as_float((uint32_t)(127 - (ex - ex_run)) << 23) : 0.0f;
#pragma unroll
      for (int et = 0; et < 8; ++et)
#pragma unroll
        for (int j = 0; j < 4; ++j) accS[et][j] *= shrink;
      ex_run = ex;
    }
    const float tscale = __uint_as_float((uint32_t)(254 - ex_run) << 23);
    // ---- weights
    uint32_t pa[2][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      float p[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float w = __builtin_amdgcn_exp2f(sc[t][j] - Mh) * iL;
        w = (w < a.threshold) ? 0.0f : w;
        w = (head_ok && 16 * t + 4 * g + j < rows) ? w : 0.0f;
        p[j] = w * (vn[t][j] * tscale);
      }
      pa[t >> 1][2 * (t & 1)] = pack_h2(p[0], p[1]);
      pa[t >> 1][2 * (t & 1) + 1] = pack_h2(p[2], p[3]);
    }
    // ---- values
#pragma unroll
    for (int kb2 = 0; kb2 < 2; ++kb2) {
      uint32_t VI[8];
      value_indices<BITS, VQUAD>(vimg, kb2, g, vw0, vsl, vsh, VI);
      const u4 A = {pa[kb2][0], pa[kb2][1], pa[kb2][2], pa[kb2][3]};
      value_products<BITS, VQUAD>(A, VI, quad_s, lutv_s, accS);
    }
  };

  for (int sidx = 0; sidx < n_steps; sidx += 2) {
    if (rows_left_of(sidx) <= 0) break;
    step(sidx, vqA, vnA, scA, [&]() { issue(sidx + 1, vqB, vnB, scB); });
    if (sidx + 1 >= n_steps || rows_left_of(sidx + 1) <= 0) break;
    step(sidx + 1, vqB, vnB, scB, [&]() { issue(sidx + 2, vqA, vnA, scA); });
  }

  // ---- merge the four waves: plain weighted sums (maximum 0 everywhere), each with its own scale
  const float inv_tscale = __uint_as_float((uint32_t)ex_run << 23);
  const int64_t grp = (int64_t)seq * a.n_kv + kvh;
  float* pS = a.ws_S + (grp * a.n_tiles_max + wg) * (int64_t)(n_rep * kD);
  float* pml = a.ws_ml + (grp * a.n_tiles_max + wg) * (int64_t)(n_rep * 2);
  static_assert(kSImageBytes >= 8 * kD * 4 && kSImageBytes % 16 == 0, "a wave's image area holds its eight deposit rows");
  merge_waves<kSWaves>(mg_s, big_s, kSImageBytes, accS, 0.0f, 0.0f, inv_tscale, a.v_unscale, n_rep, pS, pml);
}

// Launchers of the kernels above for one width.  Instantiated once per width: 3 beside the host code of the entry
// points, 1, 2 and 4 in translation units of their own (the widths compile in parallel).
//   launch_packed_tiles: the tile pass in `mode`; shape (flash mode): kTilesOnePerCu when the grid gives a CU one
//     workgroup at most, kTilesFourWaves for workgroups of four waves (tiles of 256 positions)
//   launch_packed_stream: the streaming flash pass (no mask); rows of widths other than 3 must be 16-byte aligned
template <int BITS>
void launch_packed_tiles(int mode, int shape, dim3 grid, const PackedArgs& a, const Codebook& kcb, const Codebook& vcb,
                         hipStream_t stream) {
  switch (mode) {
    case kFlash:
      if (shape == kTilesFourWaves) packed_tile_mfma_kernel<kFlash, BITS, 2, 4><<<grid, 256, 0, stream>>>(a, kcb, vcb);
      else if (shape == kTilesOnePerCu) packed_tile_mfma_kernel<kFlash, BITS, 3><<<grid, kMfmaThreads, 0, stream>>>(a, kcb, vcb);
      else packed_tile_mfma_kernel<kFlash, BITS><<<grid, kMfmaThreads, 0, stream>>>(a, kcb, vcb);
      break;
    case kScores: packed_tile_mfma_kernel<kScores, BITS><<<grid, kMfmaThreads, 0, stream>>>(a, kcb, vcb); break;
    case kSoftScores: packed_tile_mfma_kernel<kSoftScores, BITS><<<grid, kMfmaThreads, 0, stream>>>(a, kcb, vcb); break;
    case kWeights: packed_tile_mfma_kernel<kWeights, BITS><<<grid, kMfmaThreads, 0, stream>>>(a, kcb, vcb); break;
    default: packed_tile_mfma_kernel<kSoftWeights, BITS><<<grid, kMfmaThreads, 0, stream>>>(a, kcb, vcb); break;
  }
}

template <int BITS>
void launch_packed_stream(dim3 grid, const PackedArgs& a, const Codebook& kcb, const Codebook& vcb, int n_steps,
                          hipStream_t stream) {
  if constexpr (VField<BITS>::kQuad) {
    if (std::memcmp(kcb.c, vcb.c, sizeof(kcb.c)) != 0) {
      packed_stream_kernel<BITS, false><<<grid, kSThreads, 0, stream>>>(a, kcb, vcb, n_steps);
      return;
    }
  }
  packed_stream_kernel<BITS><<<grid, kSThreads, 0, stream>>>(a, kcb, vcb, n_steps);
}

template <int BITS>
void launch_packed_stream_scores(dim3 grid, const PackedArgs& a, const Codebook& kcb, int n_steps, hipStream_t stream) {
  packed_stream_scores_kernel<BITS><<<grid, kSThreads, 0, stream>>>(a, kcb, n_steps);
}

template <int BITS>
void launch_packed_stream_weights(dim3 grid, const PackedArgs& a, const Codebook& vcb, int n_steps, hipStream_t stream) {
  packed_stream_weights_kernel<BITS><<<grid, kSThreads, 0, stream>>>(a, vcb, n_steps);
}

#define TQ_PACKED_LAUNCHERS(KEYWORD, B_)                                                                               \
  KEYWORD template void launch_packed_tiles<B_>(int, int, dim3, const PackedArgs&, const Codebook&, const Codebook&,  \
                                                hipStream_t);                                                          \
  KEYWORD template void launch_packed_stream<B_>(dim3, const PackedArgs&, const Codebook&, const Codebook&, int, hipStream_t); \
  KEYWORD template void launch_packed_stream_scores<B_>(dim3, const PackedArgs&, const Codebook&, int, hipStream_t);          \
  KEYWORD template void launch_packed_stream_weights<B_>(dim3, const PackedArgs&, const Codebook&, int, hipStream_t);
#ifndef TQ_WIDTH_HERE
TQ_PACKED_LAUNCHERS(extern, 1)
TQ_PACKED_LAUNCHERS(extern, 2)
TQ_PACKED_LAUNCHERS(extern, 4)
#endif

}  // namespace tqm
