// Decode attention on the matrix cores for the common shape d = 128, 3-bit values, fp16 queries,
// n_rep <= 16 query heads per kv head.  Included by tq_attn.hip.
//
// Tile pass.  A workgroup of 8 wavefronts owns 512 consecutive KV positions of one kv head; a
// wavefront owns 64 of them and serves all n_rep query heads that share the kv head.  A CU can only
// start one wave-wide load instruction every ~24 clocks, so the pass is built to need few of them
// (Q, norm, 4 for V, 16 for K per wave), issued as early as the schedule below allows:
//
//   K rows   16 x 16-byte loads per lane, fully coalesced (an instruction reads 4 whole rows), then
//            turned into matrix-operand layout (one row per lane) through a 4 KB per-wave LDS buffer
//            with an XOR swizzle on the 16-byte piece index: writes and reads are conflict-free.
//   V words  the wave's 64 packed rows are one contiguous 3328-byte block: 4 coalesced 16-byte loads
//            per lane, copied into the same LDS buffer, from which each lane picks the two words
//            that hold its 8 three-bit fields of a position.
//   Q, norms one 4-byte load per thread each, shared through LDS.
//   scores   D[p][h] = sum_e K[p][e] * Q[h][e]: per 16 positions 4 x v_mfma_f32_16x16x32_f16
//            (A = K rows, B = Q columns, heads padded to 16).
//   softmax  over the wave's 64 positions per head, in registers plus two lane exchanges.
//   values   S[h][e] += sum_p P[h][p] * c[idx[p][e]]: A = P * v_norm, taken straight from the score
//            accumulators (the D layout of the first product is the A layout of the second);
//            B = centroid pairs looked up in a 64-entry LDS table indexed by two 3-bit fields --
//            the look-ups are done while K is still arriving.
//   output   the 8 waves combine (m, l, S) through LDS; one partial per workgroup goes to the
//            workspace.
//
// Merge pass.  One workgroup per query head folds the tile partials (running-maximum rescale),
// applies the ONE Walsh-Hadamard butterfly per output row, signs, 1/dim and 1/l.  As a dependent
// launch it costs a launch gap plus one memory round trip; merging inside the tile pass instead (last
// workgroup to arrive) was measured slower, because a single CU cannot pull the ~230 KB of partials
// of a kv head quickly and the counter/visibility round trips sit on the critical path.
//
// The contraction index of a matrix instruction may be permuted freely as long as A and B use the
// same permutation; that freedom is what lets K be read in 16-byte pieces and lets positions inside
// a 32-position block keep the order the score accumulators come in.
#pragma once

#include "tq_common.h"

namespace tqm {

using namespace tqd;

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));   // plain vector: stays in registers
// 16 bytes of K / V that this launch reads once: a streaming load (the "nt" hint).  Measured on the tile pass of the
// decode step (41 MB per launch over rotating buffers): 10.25 -> 9.35 us.  Operands that many workgroups share (the
// query rows, the per-tile partials) keep the default policy.
__device__ __forceinline__ u4 load_stream(const void* p) { return __builtin_nontemporal_load(reinterpret_cast<const u4*>(p)); }
__device__ __forceinline__ uint32_t load_stream(const uint32_t* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ float load_stream(const float* p) { return __builtin_nontemporal_load(p); }

constexpr int kD = 128;
constexpr int kPdim = 13;
constexpr int kWaves = 8;
constexpr int kWavePos = 64;
constexpr int kTilePos = kWaves * kWavePos;      // 512 positions per workgroup
constexpr int kMfmaThreads = kWaves * 64;
constexpr int kHeadsMax = 16;
constexpr float kLog2e = 1.44269504088896340736f;
constexpr int kMergeThreads = 256;

struct MfmaArgs {
  const __half* q;            // [n_seq, n_q, 128] fp16, or bf16 when q_bf16 is set (converted to fp16 on load: exact
                              // for values inside the fp16 range, which queries are)
  const __half* k;            // dense keys, rows of 128 halfs
  const uint32_t* v_packed;
  const float* v_norms;
  const int32_t* seq_offsets;
  const int64_t* len_dev;     // optional (tile + merge pass of the V-only step, no seq_offsets): every sequence attends
  int64_t len_bias;           // min(max(*len_dev + len_bias, 0), seq_len) positions, read when the kernel runs
  const float* mask;
  float* ws_S;                // [n_seq * n_kv, n_tiles_max, n_rep, 128]
  float* ws_ml;               // [n_seq * n_kv, n_tiles_max, n_rep, 2]
  int64_t seq_len;
  int64_t k_seq_stride, k_head_stride;
  int64_t v_seq_stride, v_head_stride, vn_seq_stride, vn_head_stride;
  int64_t mask_seq_stride, mask_head_stride;
  int32_t n_kv, n_rep, n_tiles_max;
  float attn_scale;
  float v_unscale;            // 1 / the scale the value table was multiplied by on the host
  int32_t q_bf16;
  float* scores;              // vonly_scores_kernel: [n_seq * n_q, scores_stride] f32, log2 units
  int64_t scores_stride;      // floats per score row (a multiple of 4)
};

// additive mask of four consecutive positions row0 .. row0 + 3 of one head: one 16-byte load where the row is
// aligned and the positions are inside the tile, else element by element; positions past the tile read as 0
__device__ __forceinline__ void load_mask4(const float* src, int row0, int rows_here, bool vec_ok, float (&m)[4]) {
  m[0] = m[1] = m[2] = m[3] = 0.0f;
  if (vec_ok && row0 + 4 <= rows_here) {
    const f4 v = *reinterpret_cast<const f4*>(src);
    m[0] = v[0]; m[1] = v[1]; m[2] = v[2]; m[3] = v[3];
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (row0 + j < rows_here) m[j] = src[j];
  }
}

// packed rows of one width: words per row, field extraction, centroid-pair table (tq_common.h)
template <int BITS>
using VField = PackedField<BITS>;

// Cross-wave merge of a workgroup's tile.  Every wave leaves, per head, the maximum m of its scores (log2 units)
// and its weight sum l, its power-of-two accumulator scale, and its RAW accumulator rows in an LDS area of its
// own (`area`, 4 KB: eight rows of 128 floats; nothing of another wave lives there, so no barrier is needed
// before the deposit).  After ONE barrier one thread per (head, four elements) folds the NW deposits with the
// factors 2^(m_w - M) * scale_w, which it derives itself: NW exponentials per thread instead of two more
// barriers around a shared table of factors.  The partial of the tile goes to pS / pml.
template <int NW>
struct MergeLds {
  float m[kHeadsMax][NW];
  float l[kHeadsMax][NW];
  float ts[NW];
};

template <int NW>
__device__ __forceinline__ void merge_waves(MergeLds<NW>& mg, unsigned char* areas, int area_stride, const f4 (&accS)[8],
                                            float m, float l, float inv_tscale, float v_unscale, int n_rep,
                                            float* __restrict__ pS, float* __restrict__ pml) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  if (g == 0) {
    mg.m[n16][wave] = m;
    mg.l[n16][wave] = l;
  }
  if (lane == 0) mg.ts[wave] = inv_tscale;
  float (*mine)[kD] = reinterpret_cast<float (*)[kD]>(areas + wave * area_stride);
  for (int h0 = 0; h0 < n_rep; h0 += 8) {
    if (h0) __syncthreads();                             // the previous eight heads have been summed
    if ((g >> 1) == (h0 >> 3)) {                         // lanes whose rows 4g+j are among these eight heads
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float4* dst = reinterpret_cast<float4*>(&mine[(4 * g + j) & 7][8 * n16]);
        dst[0] = make_float4(accS[0][j], accS[1][j], accS[2][j], accS[3][j]);
        dst[1] = make_float4(accS[4][j], accS[5][j], accS[6][j], accS[7][j]);
      }
    }
    __syncthreads();
    const int rows = min(8, n_rep - h0);
    if (tid < rows * (kD / 4)) {                         // one float4 of one head per thread
      const int hl = tid >> 5, e4 = tid & 31, h = h0 + hl;
      float mw[NW], fw[NW];
      float M = -INFINITY;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        mw[w] = mg.m[h][w];
        M = fmaxf(M, mw[w]);
      }
      float L = 0.0f;
      f4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float e = (mw[w] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(mw[w] - M);
        fw[w] = e * mg.ts[w];
        L += e * mg.l[h][w];
        const f4 x = *reinterpret_cast<const f4*>(areas + w * area_stride + (hl * kD + 4 * e4) * 4);
        sum = sum + x * fw[w];
      }
      sum = sum * v_unscale;
      *reinterpret_cast<f4*>(pS + h * kD + 4 * e4) = sum;
      if (e4 == 0) {
        pml[2 * h] = M;
        pml[2 * h + 1] = L;
      }
    }
  }
}

// grid = (n_tiles_max, n_kv, n_seq), NW * 64 threads: a workgroup of NW waves owns NW * 64 consecutive positions.
// NW = 8 (one workgroup per CU) is the faster shape when the tiles of a launch fill the CUs exactly once; NW = 4
// lets two or three workgroups share a CU, so a launch whose tile count is not a multiple of the CU count does
// not pay a second, nearly empty round of workgroups.
// PLAIN = no mask, no ragged offsets, seq_len a multiple of the tile, 16-byte aligned V rows (checked
// by the host): every tile is full, so the row clamps, the validity selects, the mask reads and the
// narrow V path drop out, and K / V addresses are a uniform base plus a lane-constant offset.
// QF32: the queries are float32 and enter as an fp16 value plus the fp16 remainder of that rounding (two
// matrix instructions per key operand), which keeps float32-query fidelity; otherwise fp16 (or bf16) queries.
template <bool PLAIN, bool QF32, int NW, int BITS>
__device__ __forceinline__ void vonly_tile_body(const MfmaArgs& a, const Codebook& vcb, const int64_t first,
                                                const int64_t len) {
  using VF = VField<BITS>;
  constexpr int kPd = VF::kPd;                         // words per packed value row
  constexpr int kTPos = NW * kWavePos;                 // positions per workgroup
  constexpr int kThr = NW * 64;
  // 4 KB per wave used three ways: per-wave staging first for the packed V block, then for K
  // tiles; finally the cross-wave merge buffer S_all[NW][8][128].
  __shared__ __align__(16) unsigned char big_s[NW * 4096];
  __shared__ uint32_t lut_s[NW][VF::kLut < 64 ? 64 : VF::kLut];   // per wave: half2(c[i & mask], c[i >> BITS])
  __shared__ __align__(16) float nrm_s[NW][kWavePos];
  __shared__ __align__(16) MergeLds<NW> mg_s;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
  const int n_rep = a.n_rep;
  const int n_q = a.n_kv * n_rep;
  const int64_t q_row0 = (int64_t)seq * n_q + (int64_t)kvh * n_rep;

  const int64_t tile_p0 = (int64_t)tile * kTPos;
  if (tile_p0 >= len) return;                          // the merge pass never reads this tile
  const int rows_here = PLAIN ? kTPos : (int)min((int64_t)kTPos, len - tile_p0);   // valid rows of this tile
  const int last_row = rows_here - 1;
  const int wrow0 = wave * kWavePos;                                  // wave's first row inside the tile

  // ---- issue every global load of this wave, small ones first -------------------------------------
  // Q operand of the score products, straight from global memory (the rows of a kv head are a few KB that
  // every workgroup of the head reads: cache hits): lane (n16, g) takes piece 4 kb + g of row n16 for kb = 0 .. 3,
  // 16 bytes of fp16 / bf16 or 32 bytes of float32.  Rows >= n_rep read row 0 and are zeroed.  Nothing here
  // goes through LDS, so no wave waits for another before the merge.
  const bool q_row_ok = n16 < n_rep;
  u4 qraw[QF32 ? 8 : 4];
  {
    const char* qrow = reinterpret_cast<const char*>(a.q) + (q_row0 + (q_row_ok ? n16 : 0)) * (int64_t)(kD * (QF32 ? 4 : 2));
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      if (QF32) {
        qraw[2 * kb] = *reinterpret_cast<const u4*>(qrow + (4 * kb + g) * 32);
        qraw[2 * kb + 1] = *reinterpret_cast<const u4*>(qrow + (4 * kb + g) * 32 + 16);
      } else {
        qraw[kb] = *reinterpret_cast<const u4*>(qrow + (4 * kb + g) * 16);
      }
    }
  }
  float my_norm;
  {
    const float* nb = a.v_norms + (int64_t)seq * a.vn_seq_stride + (int64_t)kvh * a.vn_head_stride + first + tile_p0;
    int row = wrow0 + lane;
    if (!PLAIN) row = row < last_row ? row : last_row;
    my_norm = load_stream(nb + (unsigned)row);
  }
  // packed V of the wave: 64 rows x 4 kPd bytes (52 at three bits), contiguous.  Full, 16-byte aligned blocks
  // take up to four 16-byte loads per lane; ragged or unaligned ones take kPd 4-byte loads with the index
  // clamped to the last valid word.  Either way the LDS image is the plain copy of the block.
  constexpr int kVFull = (16 * kPd) / 64;              // whole-wave 16-byte loads: 3 at three bits (then 16 more pieces)
  constexpr int kVTail = 16 * kPd - 64 * kVFull;       // pieces of the last, partial load (0 or 16)
  const uint32_t* vblock = a.v_packed +
      ((int64_t)seq * a.v_seq_stride + (int64_t)kvh * a.v_head_stride + first + tile_p0 + wrow0) * kPd;
  const bool v_wide = PLAIN || ((wrow0 + kWavePos <= rows_here) && ((reinterpret_cast<uintptr_t>(vblock) & 15) == 0));
  u4 vq[4];
  uint32_t vd[kPd];
  if (v_wide) {
    const char* vb = reinterpret_cast<const char*>(vblock);
#pragma unroll
    for (int i = 0; i < kVFull; ++i) vq[i] = load_stream(vb + i * 1024 + (uint32_t)(lane * 16));
    if (kVTail) vq[kVFull] = load_stream(vb + kVFull * 1024 + (uint32_t)((lane & (kVTail - 1)) * 16));   // lanes >= kVTail repeat
  } else {
    const int valid_words = max(0, rows_here - wrow0) * kPd;         // words of the block inside the sequence
    const uint32_t* tile_base = vblock - (int64_t)wrow0 * kPd;       // row 0 of the tile: always valid
#pragma unroll
    for (int i = 0; i < kPd; ++i) {
      const int w = i * 64 + lane;
      vd[i] = load_stream((w < valid_words) ? vblock + w : tile_base);
    }
  }
  // K: instruction i reads rows 4i .. 4i+3 of the wave; lane L takes 16-byte piece (L & 15) ^ (row & 7)
  // of row 4i + (L >> 4) -- any order of the 16 pieces covers the same 256 contiguous bytes.
  // A wave cannot run ahead of a load it is unable to issue, and the CU's memory pipeline is busy
  // for the whole pass, so the K loads are issued in three instalments with the V decode (pure
  // ALU / LDS work) placed between them; scheduling barriers keep the compiler from regrouping.
  const u4* kbase = reinterpret_cast<const u4*>(
      a.k + ((int64_t)seq * a.k_seq_stride + (int64_t)kvh * a.k_head_stride + first + tile_p0) * kD);
  // Every wave issues its V block (needed first) before any wave issues K: the CU's memory
  // pipeline takes requests in issue order, and without this the last wave's V block queues
  // behind the first waves' K loads and that wave reaches the merge a microsecond late.
  // A bare barrier: it orders the issue, it does not wait for any data.
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  u4 kreg[16];
  // byte offsets of this lane's piece for even / odd instruction numbers (r & 7 depends on i & 1 only)
  const uint32_t koff_even = (uint32_t)(((wrow0 + (lane >> 4)) * 16 + ((lane & 15) ^ ((lane >> 4) & 7))) * 16);
  const uint32_t koff_odd = (uint32_t)(((wrow0 + 4 + (lane >> 4)) * 16 + ((lane & 15) ^ ((4 + (lane >> 4)) & 7))) * 16);
  auto issue_k = [&](int i) {
    if (PLAIN) {
      const char* kb = reinterpret_cast<const char*>(kbase) + (i >> 1) * 2048;      // 8 rows of 256 bytes per pair
      kreg[i] = load_stream(kb + ((i & 1) ? koff_odd : koff_even));
    } else {
      const int r = 4 * i + (lane >> 4);
      const int piece = (lane & 15) ^ (r & 7);
      int row = wrow0 + r;
      row = row < last_row ? row : last_row;
      kreg[i] = load_stream(reinterpret_cast<const char*>(kbase) + (uint32_t)((row * 16 + piece) * 16));
    }
  };
  // (instalments of 4 + 8 + 4 instructions: the first is what the first score tile needs.  With streaming loads a
  // smaller first instalment lets the value block and the first keys arrive sooner: 9.44 -> 9.02 us against 8 + 4 + 4;
  // 2 + 10 + 4 gives 9.54, 0 + 12 + 4 9.97, 6 + 6 + 4 9.26, 12 or 16 up front 10.1)
  // The four-wave shape (short caches, two or three workgroups per CU) keeps 8 + 4 + 4: 10.7 against 11.1 us at 16 384;
  // the ten- and twelve-wave shapes are one workgroup per CU like the eight-wave one.
  constexpr int kFirstK = NW >= 8 ? 4 : 8;
#pragma unroll
  for (int i = 0; i < kFirstK; ++i) issue_k(i);
  __builtin_amdgcn_sched_barrier(0);
  VF::fill(lut_s[wave], vcb, lane);
  nrm_s[wave][lane] = my_norm;
  const uint32_t* lut_w = lut_s[wave];

  // ---- Q operand (converted now that every early load is in flight) and the V norms of this lane's 16 positions
  u4 qreg[4], qlow[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    if (QF32) {
      const f4 lo4 = __builtin_bit_cast(f4, qraw[2 * kb]), hi4 = __builtin_bit_cast(f4, qraw[2 * kb + 1]);
      const float f[8] = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const __half2 h = __floats2half2_rn(f[2 * i], f[2 * i + 1]);
        const float2 back = __half22float2(h);
        qreg[kb][i] = q_row_ok ? *reinterpret_cast<const uint32_t*>(&h) : 0u;
        qlow[kb][i] = q_row_ok ? pack_h2(f[2 * i] - back.x, f[2 * i + 1] - back.y) : 0u;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t w = qraw[kb][i];
        if (a.q_bf16) w = pack_h2(__uint_as_float(w << 16), __uint_as_float(w & 0xFFFF0000u));
        qreg[kb][i] = q_row_ok ? w : 0u;
      }
    }
  }
  float vn[4][4];
  float nmax = 0.0f;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const float4 n4 = *reinterpret_cast<const float4*>(&nrm_s[wave][16 * t + 4 * g]);
    vn[t][0] = n4.x; vn[t][1] = n4.y; vn[t][2] = n4.z; vn[t][3] = n4.w;
    nmax = fmaxf(nmax, fmaxf(fmaxf(n4.x, n4.y), fmaxf(n4.z, n4.w)));
  }
  nmax = fmaxf(nmax, shfl_xor_f(nmax, 16));
  nmax = fmaxf(nmax, shfl_xor_f(nmax, 32));
  // power-of-two scale 2^kexp, kexp = -floor(log2 nmax) (clamped to +-100): keeps P * norm inside half
  // range whatever the norms are.  It enters through the exponent of the weights (exact), not as
  // a multiplication of the norms.
  int ex = (int)((__float_as_uint(nmax) >> 23) & 0xFF);
  ex = ex < 27 ? (ex < 1 ? 127 : 27) : (ex > 227 ? 227 : ex);
  const float kexp = (float)(127 - ex);
  const float inv_tscale = __uint_as_float((uint32_t)ex << 23);

  // ---- packed V -> table indices (registers), then look-ups interleaved with the score tiles -----------
  uint32_t* stage = reinterpret_cast<uint32_t*>(big_s) + wave * 1024;   // this wave's 4 KB
  if (v_wide) {
    u4* st4 = reinterpret_cast<u4*>(stage);
#pragma unroll
    for (int i = 0; i < kVFull; ++i) st4[i * 64 + lane] = vq[i];
    if (kVTail) { if (lane < kVTail) st4[kVFull * 64 + lane] = vq[kVFull]; }
  } else {
#pragma unroll
    for (int i = 0; i < kPd; ++i) stage[i * 64 + lane] = vd[i];
  }
  // lane (n16, g) decodes elements 8*n16 .. 8*n16+7 of positions 16t + 4g + j: 8 * BITS bits that start in
  // word w0 (at three bits they may spill into word w0 + 1; lane 15 then reads words 11, 12 and takes
  // everything from the second).  X / Y interleave the even / odd fields of two positions into
  // table indices of 2 * BITS bits each; each index fetches a centroid pair.
  int w0, sh_lo, sh_hi;
  VF::pos(n16, w0, sh_lo, sh_hi);
  uint32_t X[2][4], Y[2][4];
#pragma unroll
  for (int kb2 = 0; kb2 < 2; ++kb2)
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int t = 2 * kb2 + (qd >> 1), jp = qd & 1;
      const uint32_t* ra = stage + (16 * t + 4 * g + 2 * jp) * kPd + w0;
      VF::interleave(VF::field(ra, sh_lo, sh_hi), VF::field(ra + kPd, sh_lo, sh_hi), X[kb2][qd], Y[kb2][qd]);
    }
  u4 breg[2][8];
  auto lookups = [&](int kb2) {
#pragma unroll
    for (int et = 0; et < 8; ++et)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const uint32_t src = (et & 1) ? Y[kb2][qd] : X[kb2][qd];
        breg[kb2][et][qd] = lut_w[VF::index(src, et >> 1)];
      }
  };
  // one 16-position score tile: K pieces through the wave's staging area, 4 matrix instructions
  float s[4][4];
  const float cs = a.attn_scale * kLog2e;                // scores are kept in log2 units: e^x = 2^(x log2 e)
  u4* kst = reinterpret_cast<u4*>(stage);                             // 256 pieces of 16 bytes
  const bool mask_vec = a.mask && ((reinterpret_cast<uintptr_t>(a.mask) & 15) == 0) && ((a.mask_seq_stride & 3) == 0) &&
                        ((a.mask_head_stride & 3) == 0);      // uniform
  auto qk_tile = [&](int t) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) kst[ii * 64 + lane] = kreg[4 * t + ii];
    f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const u4 ka = kst[n16 * 16 + ((4 * kb + g) ^ (n16 & 7))];       // piece 4kb+g of row n16
      if (QF32) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qlow[kb]),
                                                             acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qreg[kb]),
                                                   acc, 0, 0, 0);
    }
    float mk[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (!PLAIN && a.mask && n16 < n_rep)
      load_mask4(a.mask + (int64_t)seq * a.mask_seq_stride + ((int64_t)kvh * n_rep + n16) * a.mask_head_stride + tile_p0 +
                     wrow0 + 16 * t + 4 * g, wrow0 + 16 * t + 4 * g, rows_here, mask_vec, mk);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = wrow0 + 16 * t + 4 * g + j;                      // accumulator row 4g + j of tile t
      if (PLAIN) {
        s[t][j] = acc[j];                                              // raw: the scale joins the exponent's fma
      } else {
        const float v = __builtin_fmaf(mk[j], kLog2e, acc[j] * cs);    // log2 units
        s[t][j] = (row < rows_here) ? v : -INFINITY;
      }
    }
  };
  // schedule: look-ups (ALU + LDS) alternate with K instalments and score tiles, so the memory
  // pipeline, the LDS and the ALUs all stay busy while K streams in
  __builtin_amdgcn_sched_barrier(0);
  lookups(0);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = kFirstK; i < 12; ++i) issue_k(i);
  __builtin_amdgcn_sched_barrier(0);
  qk_tile(0);
  __builtin_amdgcn_sched_barrier(0);
  lookups(1);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 12; i < 16; ++i) issue_k(i);
  __builtin_amdgcn_sched_barrier(0);
  qk_tile(1);
  qk_tile(2);
  qk_tile(3);

  // ---- softmax statistics of head n16 over the wave's 64 positions ----------------------------------
  float m = -INFINITY;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) m = fmaxf(m, s[t][j]);
  m = fmaxf(m, shfl_xor_f(m, 16));
  m = fmaxf(m, shfl_xor_f(m, 32));
  // PLAIN: s is the raw product and attn_scale > 0 (host check), so the maximum commutes with the
  // scaling; weights = 2^(s * cs - m * cs + kexp) in one fma + v_exp_f32.
  const float arg_scale = PLAIN ? cs : 1.0f;
  m = m * arg_scale;                                     // log2 units from here on (-inf stays -inf)
  const float bias = kexp - ((m == -INFINITY) ? 0.0f : m);
  float l = 0.0f;
  uint32_t pa[2][4];                                     // A operands of the value product
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    float p[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][j], arg_scale, bias));   // weight * 2^kexp
      l += p[j];
      p[j] *= vn[t][j];
    }
    pa[t >> 1][2 * (t & 1)] = pack_h2(p[0], p[1]);
    pa[t >> 1][2 * (t & 1) + 1] = pack_h2(p[2], p[3]);
  }
  l += shfl_xor_f(l, 16);
  l += shfl_xor_f(l, 32);
  l *= inv_tscale;

  // ---- values ------------------------------------------------------------------------------------------
  f4 accS[8];
#pragma unroll
  for (int et = 0; et < 8; ++et) accS[et] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kb2 = 0; kb2 < 2; ++kb2) {
    const u4 A = {pa[kb2][0], pa[kb2][1], pa[kb2][2], pa[kb2][3]};
#pragma unroll
    for (int et = 0; et < 8; ++et)
      accS[et] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, A), __builtin_bit_cast(h8, breg[kb2][et]),
                                                        accS[et], 0, 0, 0);
  }

  // ---- merge the waves of the workgroup (merge_waves): one partial per workgroup goes to the workspace -----------
  const int64_t grp = (int64_t)seq * a.n_kv + kvh;
  float* pS = a.ws_S + (grp * a.n_tiles_max + tile) * (int64_t)(n_rep * kD);
  float* pml = a.ws_ml + (grp * a.n_tiles_max + tile) * (int64_t)(n_rep * 2);
  merge_waves<NW>(mg_s, big_s, 4096, accS, m, l, inv_tscale, a.v_unscale, n_rep, pS, pml);
}

template <bool PLAIN, bool QF32, int NW, int BITS = 3>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW == 8 ? 2 : 3, NW == 8 ? 2 : 3)))
void vonly_tile_mfma_kernel(MfmaArgs a, Codebook vcb) {
  int64_t first = 0, len = a.seq_len;
  if (!PLAIN && a.seq_offsets) {
    first = a.seq_offsets[blockIdx.z];
    len = (int64_t)a.seq_offsets[blockIdx.z + 1] - first;
  } else if (!PLAIN && a.len_dev) {
    const int64_t want = *a.len_dev + a.len_bias;
    len = want < 0 ? 0 : (want < len ? want : len);
  }
  vonly_tile_body<PLAIN, QF32, NW, BITS>(a, vcb, first, len);
}

// The same pass for unmasked caches of ANY length (host-checked: no mask, no ragged offsets, positive scale,
// 16-byte aligned value rows): a workgroup whose tile lies wholly inside the sequence runs the PLAIN body, the one
// tile that straddles the end runs the general body, tiles past the end leave at once.  The length may live in
// device memory (len_dev), which is what a step recorded in a HIP graph needs.
template <bool QF32, int NW, int BITS = 3>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW == 8 ? 2 : 3, NW == 8 ? 2 : 3)))
void vonly_tile_anylen_kernel(MfmaArgs a, Codebook vcb) {
  int64_t len = a.seq_len;
  if (a.len_dev) {
    const int64_t want = *a.len_dev + a.len_bias;
    len = want < 0 ? 0 : (want < len ? want : len);
  }
  const int64_t tile_end = ((int64_t)blockIdx.x + 1) * (NW * kWavePos);
  if (tile_end <= len) vonly_tile_body<true, QF32, NW, BITS>(a, vcb, 0, len);
  else vonly_tile_body<false, QF32, NW, BITS>(a, vcb, 0, len);
}

// Scores pass of the thresholded decode step (weights below a threshold are dropped, and the threshold
// applies to the FINAL softmax weights, so the scores of the whole sequence must exist before any value
// is summed).  Same tiling and K path as the kernel above, no V work: a workgroup writes the scaled
// (and masked) scores of its 512 positions in log2 units, s = (q . k) * attn_scale * log2 e + mask * log2 e,
// to a.scores and one (maximum, sum of 2^(s - maximum)) pair per query head to a.ws_ml, from which the
// second pass derives the softmax denominator of the sequence.
// grid = (n_tiles_max, n_kv, n_seq), 512 threads.
template <bool QF32, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void vonly_scores_kernel(MfmaArgs a) {
  constexpr int kPos = WAVES * kWavePos;             // positions per workgroup
  constexpr int kThr = WAVES * 64;
  __shared__ __align__(16) unsigned char big_s[WAVES * 4096]; // per-wave 4 KB: K tiles, then the score block
  __shared__ __align__(16) uint32_t q_s[kHeadsMax][kD / 2];
  __shared__ __align__(16) uint32_t ql_s[QF32 ? kHeadsMax : 1][kD / 2];
  __shared__ float m_s[WAVES][kHeadsMax], l_s[WAVES][kHeadsMax];

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
  }
  const int64_t tile_p0 = (int64_t)tile * kPos;
  if (tile_p0 >= len) return;                          // the second pass never reads this tile
  const int rows_here = (int)min((int64_t)kPos, len - tile_p0);
  const int last_row = rows_here - 1;
  const int wrow0 = wave * kWavePos;

  constexpr int kQIt = kHeadsMax * (kD / 2) / kThr;
  uint32_t my_q[kQIt], my_ql[kQIt];
#pragma unroll
  for (int i = 0; i < kQIt; ++i) {
    my_ql[i] = 0u;
    const int w = tid + i * kThr;
    if (QF32) {
      const float2 f = (w < n_rep * (kD / 2)) ? reinterpret_cast<const float2*>(reinterpret_cast<const float*>(a.q) + q_row0 * kD)[w]
                                              : make_float2(0.f, 0.f);
      const __half2 h = __floats2half2_rn(f.x, f.y);
      const float2 back = __half22float2(h);
      my_q[i] = *reinterpret_cast<const uint32_t*>(&h);
      my_ql[i] = pack_h2(f.x - back.x, f.y - back.y);
    } else {
      my_q[i] = (w < n_rep * (kD / 2)) ? reinterpret_cast<const uint32_t*>(a.q + q_row0 * kD)[w] : 0u;
    }
  }
  // K: instruction i reads rows 4i .. 4i+3 of the wave (1 KB contiguous); lane L takes 16-byte piece
  // (L & 15) ^ (row & 7) of row 4i + (L >> 4); rows past the end of the sequence repeat the last valid row
  const char* kbase = reinterpret_cast<const char*>(
      a.k + ((int64_t)seq * a.k_seq_stride + (int64_t)kvh * a.k_head_stride + first + tile_p0) * kD);
  u4 kreg[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = 4 * i + (lane >> 4);
    const int piece = (lane & 15) ^ (r & 7);
    int row = wrow0 + r;
    row = row < last_row ? row : last_row;
    kreg[i] = load_stream(kbase + (uint32_t)((row * 16 + piece) * 16));
  }
#pragma unroll
  for (int i = 0; i < kQIt; ++i) {
    // bf16 queries become fp16 here, after every load of the pass has been requested: converting where the word
    // is loaded would wait for it before anything else is in flight
    if (!QF32 && a.q_bf16) my_q[i] = pack_h2(__uint_as_float(my_q[i] << 16), __uint_as_float(my_q[i] & 0xFFFF0000u));
    (&q_s[0][0])[tid + i * kThr] = my_q[i];
    if (QF32) (&ql_s[0][0])[tid + i * kThr] = my_ql[i];
  }
  __syncthreads();

  u4 qreg[4], qlow[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    qreg[kb] = *reinterpret_cast<const u4*>(&q_s[n16][(4 * kb + g) * 4]);
    if (QF32) qlow[kb] = *reinterpret_cast<const u4*>(&ql_s[n16][(4 * kb + g) * 4]);
  }
  u4* kst = reinterpret_cast<u4*>(big_s) + wave * 256;          // this wave's 256 pieces of 16 bytes
  const float cs = a.attn_scale * kLog2e;
  const bool mask_vec = a.mask && ((reinterpret_cast<uintptr_t>(a.mask) & 15) == 0) && ((a.mask_seq_stride & 3) == 0) &&
                        ((a.mask_head_stride & 3) == 0);      // uniform
  float s[4][4];                                               // positions 16t + 4g + j of head n16
#pragma unroll
  for (int t = 0; t < 4; ++t) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) kst[ii * 64 + lane] = kreg[4 * t + ii];
    f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const u4 ka = kst[n16 * 16 + ((4 * kb + g) ^ (n16 & 7))];
      if (QF32) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qlow[kb]),
                                                             acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qreg[kb]),
                                                   acc, 0, 0, 0);
    }
    float mk[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (a.mask && n16 < n_rep)
      load_mask4(a.mask + (int64_t)seq * a.mask_seq_stride + ((int64_t)kvh * n_rep + n16) * a.mask_head_stride + tile_p0 +
                     wrow0 + 16 * t + 4 * g, wrow0 + 16 * t + 4 * g, rows_here, mask_vec, mk);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = wrow0 + 16 * t + 4 * g + j;
      const float v = __builtin_fmaf(mk[j], kLog2e, acc[j] * cs);
      s[t][j] = (row < rows_here) ? v : -INFINITY;
    }
  }
  // statistics of head n16 over the wave's 64 positions
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
  // The wave's 64 x n_rep scores leave through its LDS area (the last K tile has been consumed; LDS
  // operations of one wave complete in order): [16 heads][16 units of 4 positions], the unit index
  // xor-ed with the head, so that a store instruction writes 256-byte runs of a head's row.
#pragma unroll
  for (int t = 0; t < 4; ++t)
    kst[n16 * 16 + ((4 * t + g) ^ n16)] = __builtin_bit_cast(u4, f4{s[t][0], s[t][1], s[t][2], s[t][3]});
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int h = 4 * i + g;
    if (h < n_rep) {
      const f4 v = __builtin_bit_cast(f4, kst[h * 16 + (n16 ^ h)]);
      const int row0 = wrow0 + 4 * n16;
      float* dst = a.scores + (q_row0 + h) * a.scores_stride + tile_p0 + row0;
      if (row0 + 4 <= rows_here) {
        // rows are 16-byte aligned (host check).  Streaming stores: the next pass reads the scores from the memory side
        // whatever the policy, and without them the end of this pass waits for 3.7 MB of dirty lines (config 2 with a
        // threshold: 21.5 -> 20.8 us per step)
        __builtin_nontemporal_store(v, reinterpret_cast<f4*>(dst));
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (row0 + j < rows_here) dst[j] = v[j];
      }
    }
  }
  __syncthreads();
  if (tid < n_rep) {
    float M = m_s[0][tid];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) M = fmaxf(M, m_s[w][tid]);
    float L = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float mw = m_s[w][tid];
      L += (mw == -INFINITY) ? 0.0f : l_s[w][tid] * __builtin_amdgcn_exp2f(mw - M);
    }
    const int64_t grp = (int64_t)seq * a.n_kv + kvh;
    float* pml = a.ws_ml + (grp * a.n_tiles_max + tile) * (int64_t)(n_rep * 2);
    pml[2 * tid] = M;
    pml[2 * tid + 1] = L;
  }
}

// Streaming variant for unmasked caches: one workgroup of NW waves runs through n_blocks CONSECUTIVE
// blocks of NW * 64 positions; a wave walks its 64 rows of every block in STEPS of 32 positions with an
// online softmax in registers (the flash recurrence: running maximum, rescale of the accumulators
// when it moves).  Loads are double-buffered: the norm, packed-V and K loads of step s+1 are
// issued in three instalments between the phases of step s, so memory streams while the ALUs and
// matrix cores work, and the value product of the first 32 rows does not wait for the K rows of
// the last 32.  The fixed work of a tile (address set-up, Q / table staging, cross-wave merge,
// partial store) is paid once per workgroup.
// The partial of a workgroup is taken relative to R = m - kexp (running maximum in log2 units minus
// the exponent of the power-of-two norm scale of the step that set it): weights are
// 2^(s*cs - R), and moving from R_old to R_new multiplies accumulators and weight sum by 2^(R_old - R_new).
// grid = (ceil(seq_len / (NW * 64 * n_blocks)), n_kv, n_seq), NW * 64 threads.
// RAGGED = the length is not a multiple of a workgroup's range: the last workgroup of a (sequence, kv head) runs
// through fewer blocks, loads of rows past the end are redirected to valid rows (norms and K rows to the last
// valid row, packed-V pieces with no valid byte to the first piece of the last partly valid step; an aligned
// 16-byte piece that holds a valid byte never crosses a page) and the scores of those rows are set to -inf.
// RAGGED also serves ragged batches (seq_offsets): a sequence starts at any row, so its packed three-bit rows of
// 52 bytes start at any multiple of 4 bytes; every step's 32 rows are 104 pieces, hence ONE misalignment per
// sequence: pieces are fetched from the 16-byte boundary at or below the step's first row (105 of them) and the
// rows are read from the wave's LDS image at that offset.  Workgroups past a sequence's end leave at once.
constexpr int kStepPos = 32;

// MODE 0: every range is whole and starts 16-byte aligned (no offsets); 1: the general ragged body (per-row checks);
// 2: a whole range of a ragged launch (rows may start misaligned, no per-row checks).
// NW waves per workgroup (a block is NW * 64 positions): 8 where one round of workgroups covers the launch, 4
// where there are several, so that two workgroups share a CU and the set-up of one runs under the steps of the other.
template <bool QF32, int MODE, int BITS, int NW>
__device__ __forceinline__ void vonly_stream_body(const MfmaArgs& a, const Codebook& vcb, int n_blocks, int64_t first, int64_t len) {
  using VF = VField<BITS>;
  constexpr bool RAGGED = MODE == 1;                     // per-row checks
  constexpr bool MISALIGNED = MODE != 0 && BITS == 3;    // rows may start at any multiple of 4 bytes
  constexpr int kPd = VF::kPd;                           // words per packed value row
  constexpr int kBlk = NW * kWavePos;                    // positions of a block
  constexpr int kThr = NW * 64;
  constexpr int kPieces = 8 * kPd + (MISALIGNED ? 1 : 0);   // 16-byte pieces of a step's 32 packed rows: 104 at three bits (+ 1 misaligned)
  __shared__ __align__(16) unsigned char big_s[NW * 4096];
  __shared__ uint32_t lut_s[VF::kLut < 64 ? 64 : VF::kLut];
  __shared__ __align__(16) uint32_t q_s[kHeadsMax][kD / 2];
  __shared__ __align__(16) uint32_t ql_s[QF32 ? kHeadsMax : 1][kD / 2];
  __shared__ __align__(16) float nrm_s[NW][kStepPos];
  __shared__ __align__(16) float alpha_s[NW][kHeadsMax];
  __shared__ __align__(16) MergeLds<NW> mg_s;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
  const int n_rep = a.n_rep;
  const int n_q = a.n_kv * n_rep;
  const int64_t q_row0 = (int64_t)seq * n_q + (int64_t)kvh * n_rep;
  const int64_t tile_p0 = (int64_t)tile * kBlk * n_blocks;
  // positions of this workgroup's range that exist (RAGGED: the last workgroup has fewer)
  const int valid = RAGGED ? (int)min((int64_t)kBlk * n_blocks, len - tile_p0) : kBlk * n_blocks;
  const int n_steps = RAGGED ? 2 * ((valid + kBlk - 1) / kBlk) : 2 * n_blocks;
  const int last_valid = valid - 1;
  const int last_step_row = last_valid & ~(kStepPos - 1);               // first row of the last partly valid step

  // row of step s inside the workgroup's range: block s/2, this wave's 64 rows, half s%2
  auto step_row = [&](int s) { return (s >> 1) * kBlk + wave * kWavePos + (s & 1) * kStepPos; };
  const float* nbase = a.v_norms + (int64_t)seq * a.vn_seq_stride + (int64_t)kvh * a.vn_head_stride + first + tile_p0;
  const float* nbase_l = nbase + (lane & 31);
  const char* vrow0 = reinterpret_cast<const char*>(
      a.v_packed + ((int64_t)seq * a.v_seq_stride + (int64_t)kvh * a.v_head_stride + first + tile_p0) * kPd);
  // bytes between the 16-byte boundary below the range's first row and that row (uniform; 0 unless RAGGED at three bits)
  const int vmis = MISALIGNED ? (int)(reinterpret_cast<uintptr_t>(vrow0) & 15) : 0;
  const char* vbase = vrow0 - vmis;
  const char* kbase = reinterpret_cast<const char*>(
      a.k + ((int64_t)seq * a.k_seq_stride + (int64_t)kvh * a.k_head_stride + first + tile_p0) * kD);
  // pieces lane and 64 + lane of a step's block (the second load only where a block has more than 64 pieces);
  // lanes past the last piece repeat an earlier one
  const uint32_t voff0 = (uint32_t)((kPieces >= 64 ? lane : (lane & (kPieces - 1))) * 16);
  const uint32_t voff1 = (uint32_t)((64 + lane < kPieces ? 64 + lane : kPieces - 1) * 16);
  // the same for a full range: the extra piece of a misaligned step exists only where it holds a valid byte
  const uint32_t voff1_full = (MISALIGNED && voff1 >= (uint32_t)(8 * kPd * 16) && vmis == 0) ? 0u : voff1;
  const uint32_t koff_even = (uint32_t)(((lane >> 4) * 16 + ((lane & 15) ^ ((lane >> 4) & 7))) * 16);
  const uint32_t koff_odd = (uint32_t)(((4 + (lane >> 4)) * 16 + ((lane & 15) ^ ((4 + (lane >> 4)) & 7))) * 16);
  auto issue_nv = [&](int s, float& nrm, u4 (&vqx)[2]) {
    const int r = step_row(s);
    if (RAGGED) {
      nrm = load_stream(nbase + min(r + (lane & 31), last_valid));
      const int rc = min(r, last_step_row);                             // a step with no valid row re-reads the last one that has
      const uint32_t limit = (uint32_t)(vmis + (valid - rc) * (kPd * 4));   // bytes from the piece boundary to the end of the valid rows (> 0)
      const char* vb = vbase + (int64_t)rc * (kPd * 4);
      vqx[0] = load_stream(vb + (voff0 < limit ? voff0 : 0u));
      if (kPieces > 64) vqx[1] = load_stream(vb + (voff1 < limit ? voff1 : 0u));
    } else {
      nrm = load_stream(nbase_l + r);
      const char* vb = vbase + (int64_t)r * (kPd * 4);
      vqx[0] = load_stream(vb + voff0);
      if (kPieces > 64) vqx[1] = load_stream(vb + voff1_full);
    }
  };
  auto issue_k4 = [&](int s, u4 (&kx)[8], int part) {     // instructions 4*part .. 4*part+3: rows 16*part .. +15 of the step
    if (RAGGED) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int rin = 16 * part + 4 * i + (lane >> 4);                  // row inside the step
        const int piece = (lane & 15) ^ (rin & 7);
        const int row = min(step_row(s) + rin, last_valid);
        kx[4 * part + i] = load_stream(kbase + (int64_t)row * (kD * 2) + piece * 16);
      }
    } else {
      const char* kb = kbase + (int64_t)step_row(s) * (kD * 2) + part * 4096;
      kx[4 * part + 0] = load_stream(kb + koff_even);
      kx[4 * part + 1] = load_stream(kb + koff_odd);
      kx[4 * part + 2] = load_stream(kb + 2048 + koff_even);
      kx[4 * part + 3] = load_stream(kb + 2048 + koff_odd);
    }
  };

  constexpr int kQIt = kHeadsMax * (kD / 2) / kThr;      // words of the staged queries per thread
  uint32_t my_q[kQIt], my_ql[kQIt];
#pragma unroll
  for (int i = 0; i < kQIt; ++i) {
    my_ql[i] = 0u;
    const int w = tid + i * kThr;
    if (QF32) {
      const float2 f = (w < n_rep * (kD / 2)) ? reinterpret_cast<const float2*>(reinterpret_cast<const float*>(a.q) + q_row0 * kD)[w]
                                              : make_float2(0.f, 0.f);
      const __half2 h = __floats2half2_rn(f.x, f.y);
      const float2 back = __half22float2(h);
      my_q[i] = *reinterpret_cast<const uint32_t*>(&h);
      my_ql[i] = pack_h2(f.x - back.x, f.y - back.y);
    } else {
      my_q[i] = (w < n_rep * (kD / 2)) ? reinterpret_cast<const uint32_t*>(a.q + q_row0 * kD)[w] : 0u;
    }
  }
  float nrmA, nrmB = 0.0f;
  u4 vqA[2], vqB[2], kA[8], kB[8];
  issue_nv(0, nrmA, vqA);
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();                          // orders the issue: every wave's first V block ahead of all K
  __builtin_amdgcn_sched_barrier(0);
  issue_k4(0, kA, 0);
  issue_k4(0, kA, 1);
  __builtin_amdgcn_sched_barrier(0);

  if (tid < 64) VF::fill(lut_s, vcb, tid);
#pragma unroll
  for (int i = 0; i < kQIt; ++i) {
    // bf16 queries become fp16 here, after every load of the pass has been requested: converting where the word
    // is loaded would wait for it before anything else is in flight
    if (!QF32 && a.q_bf16) my_q[i] = pack_h2(__uint_as_float(my_q[i] << 16), __uint_as_float(my_q[i] & 0xFFFF0000u));
    (&q_s[0][0])[tid + i * kThr] = my_q[i];
    if (QF32) (&ql_s[0][0])[tid + i * kThr] = my_ql[i];
  }
  __syncthreads();

  u4 qreg[4], qlow[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    qreg[kb] = *reinterpret_cast<const u4*>(&q_s[n16][(4 * kb + g) * 4]);
    if (QF32) qlow[kb] = *reinterpret_cast<const u4*>(&ql_s[n16][(4 * kb + g) * 4]);
  }
  const float cs = a.attn_scale * kLog2e;
  uint32_t* stage = reinterpret_cast<uint32_t*>(big_s) + wave * 1024;   // this wave's 4 KB
  u4* kst = reinterpret_cast<u4*>(stage);
  int w0, sh_lo, sh_hi;
  VF::pos(n16, w0, sh_lo, sh_hi);

  f4 accS[8];
#pragma unroll
  for (int et = 0; et < 8; ++et) accS[et] = f4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, R_run = -INFINITY, l_run = 0.0f, inv_tscale = 1.0f;

  // one step on the buffers (nrm, vqx, kx); `next(i)` issues instalment i (0: norm + V, 1 and 2: K) of the following step
  auto step = [&](int sidx, float nrm, u4 (&vqx)[2], u4 (&kx)[8], auto&& next) {
    // ---- norms (wave-local through LDS), power-of-two scale
    if (lane < kStepPos) nrm_s[wave][lane] = nrm;
    float vn[2][4];
    float nmax = 0.0f;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const float4 n4 = *reinterpret_cast<const float4*>(&nrm_s[wave][16 * t + 4 * g]);
      vn[t][0] = n4.x; vn[t][1] = n4.y; vn[t][2] = n4.z; vn[t][3] = n4.w;
      nmax = fmaxf(nmax, fmaxf(fmaxf(n4.x, n4.y), fmaxf(n4.z, n4.w)));
    }
    nmax = fmaxf(nmax, shfl_xor_f(nmax, 16));
    nmax = fmaxf(nmax, shfl_xor_f(nmax, 32));
    int ex = (int)((__float_as_uint(nmax) >> 23) & 0xFF);
    ex = ex < 27 ? (ex < 1 ? 127 : 27) : (ex > 227 ? 227 : ex);
    const float kexp = (float)(127 - ex);
    inv_tscale = __uint_as_float((uint32_t)ex << 23);
    // ---- packed V -> table indices -> centroid pairs
    {
      u4* st4 = reinterpret_cast<u4*>(stage);
      if (kPieces >= 64 || lane < kPieces) st4[lane] = vqx[0];
      if (kPieces > 64) { if (64 + lane < kPieces) st4[64 + lane] = vqx[1]; }
    }
    __builtin_amdgcn_sched_barrier(0);
    next(0);
    __builtin_amdgcn_sched_barrier(0);
    uint32_t X[4], Y[4];
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int t = qd >> 1, jp = qd & 1;
      const uint32_t* ra = stage + (vmis >> 2) + (16 * t + 4 * g + 2 * jp) * kPd + w0;
      VF::interleave(VF::field(ra, sh_lo, sh_hi), VF::field(ra + kPd, sh_lo, sh_hi), X[qd], Y[qd]);
    }
    u4 breg[8];
#pragma unroll
    for (int et = 0; et < 8; ++et)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const uint32_t src = (et & 1) ? Y[qd] : X[qd];
        breg[et][qd] = lut_s[VF::index(src, et >> 1)];
      }
    __builtin_amdgcn_sched_barrier(0);
    next(1);
    __builtin_amdgcn_sched_barrier(0);
    // ---- scores of the 32 rows
    float s[2][4];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int ii = 0; ii < 4; ++ii) kst[ii * 64 + lane] = kx[4 * t + ii];
      f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const u4 ka = kst[n16 * 16 + ((4 * kb + g) ^ (n16 & 7))];
        if (QF32) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qlow[kb]),
                                                               acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, ka), __builtin_bit_cast(h8, qreg[kb]),
                                                     acc, 0, 0, 0);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s[t][j] = acc[j];
        if (RAGGED && step_row(sidx) + 16 * t + 4 * g + j > last_valid) s[t][j] = -INFINITY;
      }
      if (t == 0) {
        __builtin_amdgcn_sched_barrier(0);
        next(2);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- online softmax
    float mb = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                     fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
    mb = fmaxf(mb, shfl_xor_f(mb, 16));
    mb = fmaxf(mb, shfl_xor_f(mb, 32));
    const float m_new = fmaxf(m_run, mb * cs);            // log2 units; attn_scale > 0 (host check)
    // RAGGED: a wave whose rows so far all lie past the end has seen nothing yet (m_new = -inf): it keeps its
    // empty state (weights 2^-inf = 0, no rescale) instead of forming -inf - -inf
    const bool empty = RAGGED && m_new == -INFINITY;
    const float R_new = empty ? 0.0f : m_new - kexp;
    const float factor = empty ? 1.0f : __builtin_amdgcn_exp2f(R_run - R_new);      // 0 on the first step
    m_run = m_new;
    R_run = empty ? R_run : R_new;
    float lsum = 0.0f;
    uint32_t pa[4];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      float p[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][j], cs, -R_new));   // weight * 2^kexp
        lsum += p[j];
        p[j] *= vn[t][j];
      }
      pa[2 * t] = pack_h2(p[0], p[1]);
      pa[2 * t + 1] = pack_h2(p[2], p[3]);
    }
    l_run = l_run * factor + lsum;                         // per-lane part; the four lanes of a head share `factor`
    if (sidx > 0 && __any(factor != 1.0f)) {               // accumulator rows are heads 4g + j: factors through LDS
      if (g == 0) alpha_s[wave][n16] = factor;
      const float4 a4 = *reinterpret_cast<const float4*>(&alpha_s[wave][4 * g]);
      const float av[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
      for (int et = 0; et < 8; ++et)
#pragma unroll
        for (int j = 0; j < 4; ++j) accS[et][j] *= av[j];
    }
    const u4 A = {pa[0], pa[1], pa[2], pa[3]};
#pragma unroll
    for (int et = 0; et < 8; ++et)
      accS[et] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, A), __builtin_bit_cast(h8, breg[et]),
                                                        accS[et], 0, 0, 0);
  };

  for (int sidx = 0; sidx < n_steps; sidx += 2) {         // steps come in pairs: buffers A and B stay in fixed registers
    step(sidx, nrmA, vqA, kA, [&](int i) {
      if (i == 0) issue_nv(sidx + 1, nrmB, vqB); else issue_k4(sidx + 1, kB, i - 1);
    });
    const bool more = sidx + 2 < n_steps;                  // uniform
    step(sidx + 1, nrmB, vqB, kB, [&](int i) {
      if (more) { if (i == 0) issue_nv(sidx + 2, nrmA, vqA); else issue_k4(sidx + 2, kA, i - 1); }
    });
  }

  // ---- merge the eight waves (merge_waves): m is the running maximum, the weight sum and the accumulators carry
  // 2^kexp of the last step
  float l = l_run;
  l += shfl_xor_f(l, 16);
  l += shfl_xor_f(l, 32);
  l *= inv_tscale;
  const int64_t grp = (int64_t)seq * a.n_kv + kvh;
  float* pS = a.ws_S + (grp * a.n_tiles_max + tile) * (int64_t)(n_rep * kD);
  float* pml = a.ws_ml + (grp * a.n_tiles_max + tile) * (int64_t)(n_rep * 2);
  merge_waves<NW>(mg_s, big_s, 4096, accS, m_run, l, inv_tscale, a.v_unscale, n_rep, pS, pml);
}

template <bool QF32, bool RAGGED, int BITS = 3, int NW = 8>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void vonly_stream_kernel(MfmaArgs a, Codebook vcb, int n_blocks) {
  if (!RAGGED) {
    vonly_stream_body<QF32, 0, BITS, NW>(a, vcb, n_blocks, 0, a.seq_len);
    return;
  }
  int64_t first = 0, len = a.seq_len;
  if (a.seq_offsets) {
    first = a.seq_offsets[blockIdx.z];
    len = (int64_t)a.seq_offsets[blockIdx.z + 1] - first;
  }
  const int64_t range = (int64_t)(NW * kWavePos) * n_blocks;
  const int64_t tile_p0 = (int64_t)blockIdx.x * range;
  if (tile_p0 >= len) return;                             // uniform over the workgroup, ahead of every barrier
  if (tile_p0 + range <= len) vonly_stream_body<QF32, 2, BITS, NW>(a, vcb, n_blocks, first, len);
  else vonly_stream_body<QF32, 1, BITS, NW>(a, vcb, n_blocks, first, len);
}

// The token a decode step inserts, handled by the merge pass instead of a launch of its own ahead of the
// tile pass: an extra wavefront of every merge workgroup encodes the new value row (the arithmetic of the
// encoder, operation for operation: tree-ordered sum of squares, division by max(norm, 1e-8), signs, raw
// butterfly, strict threshold count), takes q . k of its head against the float16-rounded new key, and hands
// (score, 1, norm * c[idx]) to the fold as one more partial; the workgroup of the first query head of a kv
// head also stores the key row, the raw value row, the packed words and the norm.  The tile pass then covers
// the positions before the new one only.
struct FreshToken {
  const void* k_new;          // [n_seq, n_kv, 128], dtype k_dtype
  const void* v_new;          // [n_seq, n_kv, 128], dtype v_dtype
  const void* q;              // [n_seq, n_q, 128], dtype q_dtype
  __half* k_f16;              // storage, time index 0 of group 0; t_alloc positions per (sequence, kv head)
  void* v_raw;                // may be null
  uint32_t* v_packed;
  float* v_norms;
  const int64_t* pos_dev;     // insert position in device memory, or null: `pos`
  int64_t pos, t_alloc;
  float thr[15];              // decision thresholds in the domain of the raw butterfly output; +inf past the 2^bits - 1 real ones
  float cent[16];
  int32_t bits;               // width of the packed fields, 1-4 (keys, where packed, and values alike)
  float cs;                   // attn_scale * log2 e
  int32_t k_dtype, v_dtype, q_dtype;
  // Cache with packed keys (k_packed set; k_f16 / v_raw unused): the new key row is encoded as well (signs
  // k_signs, same thresholds and centroids), the query is rotated (raw butterfly of q * k_signs) and the
  // score is sum_e c[idx_k[e]] * q_rot[e] * k_norm / dim, as the packed tile pass takes it.
  const float* k_signs;
  uint32_t* k_packed;
  float* k_norms;
};

// Level of one butterfly output (count of thresholds it exceeds, strictly) and the centroid of that level, for a
// token inserted by the merge pass.  NB = thresholds looked at: 7 serves widths up to three bits (entries past the
// width are +inf), 15 the four-bit width; selects, not a dynamic index into kernel arguments.
template <int NB>
__device__ __forceinline__ void fresh_level(const FreshToken& f, float w, uint32_t& n, float& c) {
  n = 0;
#pragma unroll
  for (int b = 0; b < NB; ++b) n += (w > f.thr[b]) ? 1u : 0u;
  c = f.cent[0];
#pragma unroll
  for (int k = 1; k <= NB; ++k) c = (n == (uint32_t)k) ? f.cent[k] : c;
}

// Packed word `lane` of a row whose 128 indices sit two per lane (idx[0] = element lane, idx[1] = element
// lane + 64): elements VPW * lane .. VPW * lane + VPW - 1, fields of BITS bits, lowest first (packing.py:26-56).
template <int BITS>
__device__ __forceinline__ uint32_t fresh_word(const int (&idx)[2], int lane) {
  constexpr int VPW = BITS == 3 ? 10 : 32 / BITS;
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < VPW; ++i) {
    const int e = min(VPW * lane + i, kD - 1);
    const int lo = __shfl(idx[0], e & 63), hi = __shfl(idx[1], e & 63);
    const uint32_t fld = (uint32_t)((e >> 6) ? hi : lo);
    if (VPW * lane + i < kD) word |= fld << (BITS * i);
  }
  return word;
}

// An element of a tensor whose dtype is a run-time value, in two steps so that a wavefront can have the loads of
// several such tensors in flight together: the raw bits first (one uniform branch on the element size, no use of
// the value), the conversion (selects, no branch) once everything has been requested.
__device__ __forceinline__ uint32_t load_raw(const void* p, int dtype, int64_t at) {
  if (dtype == TQ_F32) return ((const uint32_t*)p)[at];
  return ((const uint16_t*)p)[at];
}
__device__ __forceinline__ float raw_to_float(uint32_t raw, int dtype) {
  const float f32 = __uint_as_float(raw);
  const float bf = __uint_as_float(raw << 16);
  const unsigned short hbits = (unsigned short)(raw & 0xFFFFu);
  const float f16 = __half2float(__ushort_as_half(hbits));
  return dtype == TQ_F32 ? f32 : (dtype == TQ_F16 ? f16 : bf);
}

// Merge pass: grid = (n_q, n_seq), 256 threads (320 with FRESH).  Lane group ph = tid / 32 folds tiles ph, ph + 8, ...
// (4 elements per lane) with a running maximum, U tiles per round with all loads of a round issued together (a
// round costs one memory round trip, so the host picks U to cover the tiles in one round where it can: 8, 16
// or 32); the 8 groups are then combined through LDS and wave 0 finishes the row.  NORM = false (given weights,
// all maxima zero) skips the division by l.
template <typename TO, bool NORM, int U, bool FRESH>
__device__ __forceinline__ void merge_rows_body(
    const float* __restrict__ ws_S, const float* __restrict__ ws_ml, const int32_t* __restrict__ seq_offsets,
    int64_t seq_len, int n_tiles_max, int n_kv, int n_rep, const float* __restrict__ signs, float inv_dim,
    TO* __restrict__ out, int tile_pos, const int64_t* __restrict__ len_dev, int64_t len_bias, const FreshToken* ft) {
  __shared__ __align__(16) float acc_s[FRESH ? 9 : 8][kD];
  __shared__ float ml_s[FRESH ? 9 : 8][2];
  const int tid = threadIdx.x, lane = tid & 63;
  const int eq = tid & 31, ph = tid >> 5;
  const int head = blockIdx.x, seq = blockIdx.y;
  const int kvh = head / n_rep, r = head - kvh * n_rep;
  int64_t len = seq_len;
  if (seq_offsets) {
    len = (int64_t)seq_offsets[seq + 1] - seq_offsets[seq];
  } else if (len_dev) {                                  // as the tile pass reads it
    const int64_t want = *len_dev + len_bias;
    len = want < 0 ? 0 : (want < len ? want : len);
  }
  const int n_tiles = (int)((len + tile_pos - 1) / tile_pos);
  const int64_t grp = (int64_t)seq * n_kv + kvh;
  const float* gS = ws_S + grp * n_tiles_max * (int64_t)(n_rep * kD) + r * kD + 4 * eq;
  const float* gml = ws_ml + grp * n_tiles_max * (int64_t)(n_rep * 2) + r * 2;
  // issued first: the signs are only needed at the very end, their latency hides behind everything else
  const float sign0 = signs[lane], sign1 = signs[lane + 64];
  bool fresh_wave = false;
  if constexpr (FRESH) fresh_wave = tid >= 256;
  // what the wavefront of the inserted token keeps for its stores, which wait until the fold is under way
  float x[2] = {0.f, 0.f}, kx[2] = {0.f, 0.f}, fresh_nrm = 0.0f, fresh_knrm = 0.0f;
  int idx[2] = {0, 0}, kidx[2] = {0, 0};
  int64_t fresh_row = -1;
  if constexpr (FRESH) { if (fresh_wave) {
    // ---- the inserted token (one wavefront) ------------------------------------------------------------
    const FreshToken& f = *ft;
    const int64_t pos = f.pos_dev ? *f.pos_dev : f.pos;
    const bool ok = pos >= 0 && pos < f.t_alloc;
    const int64_t src = grp * kD;
    float qx[2], sq[2];
    uint32_t rv[2], rk[2], rq[2];
    const int64_t qsrc = ((int64_t)seq * gridDim.x + head) * kD;
    rv[0] = load_raw(f.v_new, f.v_dtype, src + lane); rv[1] = load_raw(f.v_new, f.v_dtype, src + lane + 64);
    rk[0] = load_raw(f.k_new, f.k_dtype, src + lane); rk[1] = load_raw(f.k_new, f.k_dtype, src + lane + 64);
    rq[0] = load_raw(f.q, f.q_dtype, qsrc + lane); rq[1] = load_raw(f.q, f.q_dtype, qsrc + lane + 64);
    float ksg[2] = {0.f, 0.f};
    if (f.k_packed) { ksg[0] = f.k_signs[lane]; ksg[1] = f.k_signs[lane + 64]; }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      x[i] = raw_to_float(rv[i], f.v_dtype);
      kx[i] = raw_to_float(rk[i], f.k_dtype);
      if (!f.k_packed) kx[i] = __half2float(__float2half_rn(kx[i]));
      qx[i] = raw_to_float(rq[i], f.q_dtype);
      sq[i] = x[i] * x[i];
    }
    const float ss = tree_sum<kD>(sq);
    const float nrm = sqrtf(ss);
    const float safe = fmaxf(nrm, 1e-8f);
    float v[2] = {(x[0] / safe) * sign0, (x[1] / safe) * sign1};
    raw_butterfly<kD>(v, lane);
    fresh_nrm = nrm;
    if (ok && r == 0) fresh_row = grp * f.t_alloc + pos;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      uint32_t n;
      float c;
      if (f.bits <= 3) fresh_level<7>(f, v[i], n, c); else fresh_level<15>(f, v[i], n, c);      // uniform
      idx[i] = (int)n;
      acc_s[8][lane + 64 * i] = nrm * c;
    }
    float d;
    if (f.k_packed) {
      float ksq[2] = {kx[0] * kx[0], kx[1] * kx[1]};
      const float kss = tree_sum<kD>(ksq);
      const float knrm = sqrtf(kss);
      const float ksafe = fmaxf(knrm, 1e-8f);
      float kv[2] = {(kx[0] / ksafe) * ksg[0], (kx[1] / ksafe) * ksg[1]};
      raw_butterfly<kD>(kv, lane);
      float qr[2] = {qx[0] * ksg[0], qx[1] * ksg[1]};
      raw_butterfly<kD>(qr, lane);
      fresh_knrm = knrm;
      d = 0.0f;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        uint32_t n;
        float c;
        if (f.bits <= 3) fresh_level<7>(f, kv[i], n, c); else fresh_level<15>(f, kv[i], n, c);  // uniform
        kidx[i] = (int)n;
        d += c * qr[i];
      }
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) d += shfl_xor_f(d, m);
      d = (d * knrm) * inv_dim;
    } else {
      d = qx[0] * kx[0] + qx[1] * kx[1];
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) d += shfl_xor_f(d, m);
    }
    if (lane == 0) {
      ml_s[8][0] = ok ? d * f.cs : -INFINITY;
      ml_s[8][1] = 1.0f;
    }
  } }
  if (!fresh_wave) {
  float M = -INFINITY, L = 0.0f;
  f4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int t0 = ph; t0 < n_tiles; t0 += 8 * U) {         // U tiles per lane group and round
    f4 x[U];
    float2 ml[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = min(t0 + 8 * u, n_tiles - 1);
      x[u] = __builtin_nontemporal_load(reinterpret_cast<const f4*>(gS + (int64_t)t * (n_rep * kD)));
      ml[u] = *reinterpret_cast<const float2*>(gml + (int64_t)t * (n_rep * 2));
    }
    // maximum of the round first, then one independent 2^(m - M) per tile
    float Mr = M;
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (t0 + 8 * u < n_tiles) Mr = fmaxf(Mr, ml[u].x);
    if (Mr != -INFINITY) {
      const float fo = (M == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(M - Mr);
      acc = acc * fo;
      L = L * fo;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float fc = (t0 + 8 * u < n_tiles && ml[u].x != -INFINITY) ? __builtin_amdgcn_exp2f(ml[u].x - Mr) : 0.0f;
        acc = acc + x[u] * fc;
        L = L + ml[u].y * fc;
      }
      M = Mr;
    }
  }
  *reinterpret_cast<f4*>(&acc_s[ph][4 * eq]) = acc;
  if (eq == 0) { ml_s[ph][0] = M; ml_s[ph][1] = L; }
  }
  __syncthreads();
  if constexpr (FRESH) { if (fresh_wave) {
    // packed word `lane` holds elements vpw * lane .. vpw * lane + vpw - 1 (fields of `bits` bits, lowest first;
    // 10 per word at three bits, else 32 / bits)
    const FreshToken& f = *ft;
    const int bits = f.bits;                               // uniform
    const int pd = bits == 3 ? kPdim : 4 * bits;           // words per row: 4, 8, 13, 16
    uint32_t word, kword = 0;
    if (bits == 3) { word = fresh_word<3>(idx, lane); if (f.k_packed) kword = fresh_word<3>(kidx, lane); }
    else if (bits == 4) { word = fresh_word<4>(idx, lane); if (f.k_packed) kword = fresh_word<4>(kidx, lane); }
    else if (bits == 2) { word = fresh_word<2>(idx, lane); if (f.k_packed) kword = fresh_word<2>(kidx, lane); }
    else { word = fresh_word<1>(idx, lane); if (f.k_packed) kword = fresh_word<1>(kidx, lane); }
    if (fresh_row >= 0) {                                  // first query head of the kv head, position inside the storage
      const int64_t row = fresh_row;
      if (lane < pd) f.v_packed[row * pd + lane] = word;
      if (lane == 0) f.v_norms[row] = fresh_nrm;
      if (f.k_packed) {
        if (lane < pd) f.k_packed[row * pd + lane] = kword;
        if (lane == 0) f.k_norms[row] = fresh_knrm;
      } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int e = lane + 64 * i;
        f.k_f16[row * kD + e] = __float2half_rn(kx[i]);
        if (f.v_raw) {
          if (f.v_dtype == TQ_F32) ((float*)f.v_raw)[row * kD + e] = x[i];
          else if (f.v_dtype == TQ_F16) ((__half*)f.v_raw)[row * kD + e] = __float2half_rn(x[i]);
          else ((__hip_bfloat16*)f.v_raw)[row * kD + e] = __float2bfloat16(x[i]);
        }
      }
      }
    }
  } }
  if (tid >= 64) return;
  constexpr int NP = FRESH ? 9 : 8;
  float Mt = ml_s[0][0];
#pragma unroll
  for (int p = 1; p < NP; ++p) Mt = fmaxf(Mt, ml_s[p][0]);
  float Lt = 0.0f;
  float v[2] = {0.0f, 0.0f};
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const float f = (ml_s[p][0] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(ml_s[p][0] - Mt);
    Lt += f * ml_s[p][1];
    v[0] += f * acc_s[p][lane];
    v[1] += f * acc_s[p][lane + 64];
  }
  raw_butterfly<kD>(v, lane);
  TO* o = out + ((int64_t)seq * gridDim.x + head) * kD;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int e = lane + 64 * i;
    float val = (v[i] * (i ? sign1 : sign0)) * inv_dim;
    if (NORM) val = (Lt > 0.0f) ? val / Lt : 0.0f;
    store_from_float<TO>(o + e, val);
  }
}

template <typename TO, bool NORM, int U = 8>
__global__ __launch_bounds__(kMergeThreads) void decode_merge_rows_kernel(
    const float* __restrict__ ws_S, const float* __restrict__ ws_ml, const int32_t* __restrict__ seq_offsets,
    int64_t seq_len, int n_tiles_max, int n_kv, int n_rep, const float* __restrict__ signs, float inv_dim,
    TO* __restrict__ out, int tile_pos, const int64_t* __restrict__ len_dev = nullptr, int64_t len_bias = 0) {
  merge_rows_body<TO, NORM, U, false>(ws_S, ws_ml, seq_offsets, seq_len, n_tiles_max, n_kv, n_rep, signs, inv_dim, out,
                                      tile_pos, len_dev, len_bias, nullptr);
}

// The merge pass of a decode step that inserts its token here (see FreshToken): 320 threads.
template <typename TO, int U>
__global__ __launch_bounds__(kMergeThreads + 64) void decode_merge_fresh_kernel(
    const float* __restrict__ ws_S, const float* __restrict__ ws_ml, int64_t seq_len, int n_tiles_max, int n_kv,
    int n_rep, const float* __restrict__ signs, float inv_dim, TO* __restrict__ out, int tile_pos,
    const int64_t* __restrict__ len_dev, FreshToken ft) {
  merge_rows_body<TO, true, U, true>(ws_S, ws_ml, nullptr, seq_len, n_tiles_max, n_kv, n_rep, signs, inv_dim, out,
                                     tile_pos, len_dev, 0, &ft);
}

// Which tile kernel a launch uses (chosen by the host from the length, the mask / offsets and the alignment).
struct VonlyTileChoice {
  int nw;                     // waves per workgroup: 8 or 4; 10 or 12 (any-length kernel only) just above a full round of 8
  int n_blocks;               // > 1: streaming pass, that many blocks of nw * 64 positions per workgroup
  bool ragged_stream;         // the streaming pass with a ragged end and / or over a ragged batch
  bool plain;                 // full 512-position tiles, no mask, no offsets
  bool plain4;                // full 256-position tiles, no mask, no offsets
  bool plain_any;             // no mask, no offsets, any length
  bool q_f32;
};

// The tile pass for values of BITS bits.  Instantiated once per width: 3 beside the host code of the decode
// entry points, 1, 2 and 4 in translation units of their own (those define TQ_WIDTH_HERE).
template <int BITS>
void launch_vonly_tiles(dim3 grid, const VonlyTileChoice& c, const MfmaArgs& a, const Codebook& vcb, hipStream_t stream) {
#define TQ_LAUNCH_TILE(QF)                                                                                              \
  if (c.n_blocks > 1 && c.ragged_stream && c.nw == 4) vonly_stream_kernel<QF, true, BITS, 4><<<grid, 256, 0, stream>>>(a, vcb, c.n_blocks); \
  else if (c.n_blocks > 1 && c.ragged_stream) vonly_stream_kernel<QF, true, BITS, 8><<<grid, 512, 0, stream>>>(a, vcb, c.n_blocks); \
  else if (c.n_blocks > 1 && c.nw == 4) vonly_stream_kernel<QF, false, BITS, 4><<<grid, 256, 0, stream>>>(a, vcb, c.n_blocks);  \
  else if (c.n_blocks > 1) vonly_stream_kernel<QF, false, BITS, 8><<<grid, 512, 0, stream>>>(a, vcb, c.n_blocks);  \
  else if (c.nw == 12) vonly_tile_anylen_kernel<QF, 12, BITS><<<grid, 768, 0, stream>>>(a, vcb);                        \
  else if (c.nw == 10) vonly_tile_anylen_kernel<QF, 10, BITS><<<grid, 640, 0, stream>>>(a, vcb);                        \
  else if (c.nw == 8 && c.plain) vonly_tile_mfma_kernel<true, QF, 8, BITS><<<grid, 512, 0, stream>>>(a, vcb);           \
  else if (c.nw == 8 && c.plain_any) vonly_tile_anylen_kernel<QF, 8, BITS><<<grid, 512, 0, stream>>>(a, vcb);           \
  else if (c.nw == 8) vonly_tile_mfma_kernel<false, QF, 8, BITS><<<grid, 512, 0, stream>>>(a, vcb);                     \
  else if (c.plain4) vonly_tile_mfma_kernel<true, QF, 4, BITS><<<grid, 256, 0, stream>>>(a, vcb);                       \
  else if (c.plain_any) vonly_tile_anylen_kernel<QF, 4, BITS><<<grid, 256, 0, stream>>>(a, vcb);                        \
  else vonly_tile_mfma_kernel<false, QF, 4, BITS><<<grid, 256, 0, stream>>>(a, vcb)
  if (c.q_f32) { TQ_LAUNCH_TILE(true); } else { TQ_LAUNCH_TILE(false); }
#undef TQ_LAUNCH_TILE
}
#ifndef TQ_WIDTH_HERE
extern template void launch_vonly_tiles<1>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
extern template void launch_vonly_tiles<2>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
extern template void launch_vonly_tiles<4>(dim3, const VonlyTileChoice&, const MfmaArgs&, const Codebook&, hipStream_t);
#endif

}  // namespace tqm
