// Chunked-prefill attention over PACKED keys and values (d = 128, 1 to 4 bits) on the gfx950 matrix
// cores: a chunk of query rows (all q heads) against the packed cache up to the chunk's end,
// causal inside the chunk.  The reference has no kernel for this step: its prefill dequantises
// the whole cache to fp16 (cache.py:125-129, 209-210) and calls stock SDPA, i.e. it moves
// 256 B per cached vector where this path moves 56 B (at three bits) and never materialises K or V.
//
// Everything happens in the rotated domain, as in flash_attention.py:79-162:
//   q_rot = B(q * signs_K)                                  (one pass, rounded to fp16)
//   s[r, p] = <q_rot[r], c_K[idx_K[p]]> * norm_K[p] * attn_scale / d
//   O[r]    = sum_p softmax_p(s[r, .]) * norm_V[p] * c_V[idx_V[p]]
//   out[r]  = B(O[r]) * signs_V / d                         (one butterfly per output row)
// Three launches: pre-rotation, the tile kernel below (split over key positions), and a merge
// pass that combines the splits and does the final butterfly.
#include "tq_common.h"

#include <math.h>

namespace {

using namespace tqd;

typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int kD = 128;
constexpr int kBlkPos = 64;                     // key positions decoded into LDS per step
constexpr int kWaves = 8;
constexpr int kWaveRows = 32;                   // query rows per wavefront
constexpr int kRowTiles = kWaveRows / 16;
constexpr int kWgRows = kWaves * kWaveRows;     // 256 query rows per workgroup
constexpr int kThreads = kWaves * 64;
constexpr int kKStride = 136;                   // halfs per decoded key row in LDS (272 B: conflict-free b128 reads)
constexpr int kVStride = 72;                    // halfs per row of the transposed value block (144 B)
constexpr float kVnScale = 0.0625f;             // value norms enter the fp16 weights times 2^-4 (norms up to 1e6)
constexpr float kLog2e = 1.44269504088896340736f;
constexpr int kRowsPerWavePass = 16;            // four lanes per row in the pre-rotation and merge kernels

struct PrefillArgs {
  const __half* q_rot;          // [n_q, n_rows, 128] fp16, pre-rotated
  const __half* q_rot_lo;       // same shape: what rounding q_rot to fp16 lost, as fp16
  const uint32_t* k_packed;     // [n_kv, k_head_stride rows, words per packed row]
  const float* k_norms;
  const uint32_t* v_packed;
  const float* v_norms;
  float* ws_O;                  // [n_splits, n_q, n_rows, 128] unnormalised sums, rotated domain
  float* ws_ml;                 // [n_splits, n_q, n_rows, 2]   running maximum (log2 units), sum of weights
  int64_t n_rows, kv_len, q_pos0;
  int64_t k_head_stride, kn_head_stride, v_head_stride, vn_head_stride;
  int64_t split_len;            // multiple of kBlkPos
  int32_t n_q, n_rep, causal;
  float score_scale;            // attn_scale / d / key-table scale * log2(e)
};

// grid = (n_splits, ceil(n_rows / 256), n_q), 512 threads: two wavefronts per SIMD, so that one's
// matrix instructions overlap the other's LDS reads and softmax arithmetic.
// Wavefront w owns query rows 32w .. 32w+31 of the workgroup's 256.  Per block of 64 key
// positions: all threads decode the packed rows (BITS bits per field) through centroid-pair tables into LDS
//   Ks[p][e]   keys, row-major, fp16
//   Vt[e][s]   values, transposed; position p = 32b + 16h + 4g + j sits in slot s = 32b + 8g + 4h + j,
//              the order in which the weights come out of the score accumulators
// then every wavefront runs S^T = K Q^T (MFMA 16x16x32, the query as fp16 value + fp16 remainder:
// rounding q_rot to one fp16 costs up to 1e-2 of an output row when an outlier channel of V
// cancels in the average), the online softmax on its accumulators, and O += P V with the
// accumulator registers of S^T reused as the A operand.  The packed words of the next block are
// fetched while the current one is computed.
// QLO = false leaves the query remainder out (one matrix instruction per key operand instead of two): for callers
// that declare their data free of outlier channels.
template <int BITS, bool QLO = true>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
void prefill_tile_kernel(PrefillArgs a, Codebook kcb, Codebook vcb) {
  using PF = PackedField<BITS>;
  constexpr int kPdim = PF::kPd;                    // words per packed row
  constexpr int kStageWords = kBlkPos * kPdim;      // packed words per block and tensor (832 at three bits)
  constexpr int kLut = PF::kLut < 64 ? 64 : PF::kLut;
  __shared__ __align__(16) _Float16 Ks2[2][kBlkPos * kKStride];
  __shared__ __align__(16) _Float16 Vt2[2][kD * kVStride];
  __shared__ uint32_t stK2[2][kStageWords + 4], stV2[2][kStageWords + 4];
  __shared__ float stN2[2][2 * kBlkPos];                       // raw key norms, then raw value norms
  __shared__ __align__(16) float kn_s2[2][kBlkPos], vn_s2[2][kBlkPos];
  __shared__ uint32_t lutk_s[kLut], lutv_s[kLut];
  __shared__ __align__(16) float alpha_s[kWaves][kWaveRows];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n16 = lane & 15, g = lane >> 4;
  const int split = blockIdx.x, rb = blockIdx.y, head = blockIdx.z;
  const int kvh = head / a.n_rep;
  const int64_t row_base = (int64_t)rb * kWgRows;
  const int64_t wrow0 = row_base + (int64_t)wave * kWaveRows;

  // key positions of this workgroup: its split, cut at the last position any of its rows may see
  const int64_t p_lo = (int64_t)split * a.split_len;
  int64_t p_hi = min(a.kv_len, p_lo + a.split_len);
  if (a.causal) {
    const int64_t last_row = min(a.n_rows, row_base + kWgRows) - 1;
    p_hi = min(p_hi, a.q_pos0 + last_row + 1);
  }
  const int64_t part = ((int64_t)split * a.n_q + head) * a.n_rows;       // first row of this (split, head) in the workspace

  if (tid < 64) PF::fill(lutk_s, kcb, tid);
  else if (tid < 128) PF::fill(lutv_s, vcb, tid - 64);

  // ---- query operands: B[k = element][n = row], 8 consecutive elements per lane; value and remainder
  u4 qhi[kRowTiles][4], qlo[kRowTiles][4];
#pragma unroll
  for (int ct = 0; ct < kRowTiles; ++ct) {
    const int64_t r = wrow0 + 16 * ct + n16;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      u4 vh = {0u, 0u, 0u, 0u}, vl = {0u, 0u, 0u, 0u};
      if (r < a.n_rows) {
        const int64_t off = ((int64_t)head * a.n_rows + r) * kD + 32 * kb + 8 * g;
        vh = *reinterpret_cast<const u4*>(a.q_rot + off);
        if (QLO) vl = *reinterpret_cast<const u4*>(a.q_rot_lo + off);
      }
      qhi[ct][kb] = vh;
      qlo[ct][kb] = vl;
    }
  }

  f4 oacc[kRowTiles][8];
#pragma unroll
  for (int ct = 0; ct < kRowTiles; ++ct)
#pragma unroll
    for (int et = 0; et < 8; ++et) oacc[ct][et] = f4{0.f, 0.f, 0.f, 0.f};
  float m_run[kRowTiles], l_run[kRowTiles];
#pragma unroll
  for (int ct = 0; ct < kRowTiles; ++ct) { m_run[ct] = -INFINITY; l_run[ct] = 0.0f; }

  // decode roles: keys -- position tid/8, chunks 2*(tid%8) and +1; values -- position pair tid%32, chunk tid/32
  const int kpos = tid >> 3, kq = tid & 7;
  int kcw[2], kcl[2], kch[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) PF::pos(2 * kq + i, kcw[i], kcl[i], kch[i]);
  const int vpp = tid & 31, vc = tid >> 5;
  int vcw, vcl, vch;
  PF::pos(vc, vcw, vcl, vch);
  // slot of the even position 2*vpp: p = 32b + 16h + 4gg + j  ->  32b + 8gg + 4h + j
  const int vp = 2 * vpp;
  const int vslot = (vp & 32) + 8 * ((vp >> 2) & 3) + 4 * ((vp >> 4) & 1) + (vp & 3);

  const uint32_t* kbase = a.k_packed + (int64_t)kvh * a.k_head_stride * kPdim;
  const uint32_t* vbase = a.v_packed + (int64_t)kvh * a.v_head_stride * kPdim;
  const float* knbase = a.k_norms + (int64_t)kvh * a.kn_head_stride;
  const float* vnbase = a.v_norms + (int64_t)kvh * a.vn_head_stride;

  uint32_t pk[2], pv[2];
  float pn = 0.0f;
  auto prefetch = [&](int64_t pb) {
    const int64_t words_left = (a.kv_len - pb) * kPdim;               // rows past the end read as zeros
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = tid + kThreads * i;
      const bool ok = id < kStageWords && id < words_left;
      pk[i] = ok ? kbase[pb * kPdim + id] : 0u;
      pv[i] = ok ? vbase[pb * kPdim + id] : 0u;
    }
    if (tid < 64) pn = (pb + tid < a.kv_len) ? knbase[pb + tid] : 0.0f;
    else if (tid < 128) pn = (pb + tid - 64 < a.kv_len) ? vnbase[pb + tid - 64] : 0.0f;
  };

  // Pipeline over blocks with ONE barrier per block: block b+1 is decoded into the other LDS
  // buffer in the same stretch of code that computes block b, so decode arithmetic and LDS
  // traffic can be scheduled between the matrix instructions.
  auto stage = [&](int sb) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = tid + kThreads * i;
      if (id < kStageWords) { stK2[sb][id] = pk[i]; stV2[sb][id] = pv[i]; }
    }
    if (tid < 128) stN2[sb][tid] = pn;
  };
  auto decode = [&](int sb) {
    const uint32_t* stK = stK2[sb];
    const uint32_t* stV = stV2[sb];
    _Float16* Ks = Ks2[sb];
    _Float16* Vt = Vt2[sb];
    if (tid < 64) kn_s2[sb][tid] = stN2[sb][tid] * a.score_scale;
    else if (tid < 128) vn_s2[sb][tid - 64] = stN2[sb][tid] * kVnScale;
    // ---- decode keys: 16 elements of one position
    {
      const uint32_t* row = stK + kpos * kPdim;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint32_t f = PF::field(row + kcw[i], kcl[i], kch[i]);
        u4 w;
#pragma unroll
        for (int jp = 0; jp < 4; ++jp) w[jp] = lutk_s[PF::index(f, jp)];
        *reinterpret_cast<u4*>(&Ks[kpos * kKStride + 8 * (2 * kq + i)]) = w;
      }
    }
    // ---- decode values: two positions x 8 elements, written transposed
    {
      const uint32_t* ra = stV + vp * kPdim + vcw;
      uint32_t X, Y;                                                    // elements 8c + 0, 2, 4, 6 / 8c + 1, 3, 5, 7
      PF::interleave(PF::field(ra, vcl, vch), PF::field(ra + kPdim, vcl, vch), X, Y);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *reinterpret_cast<uint32_t*>(&Vt[(8 * vc + 2 * i) * kVStride + vslot]) = lutv_s[PF::index(X, i)];
        *reinterpret_cast<uint32_t*>(&Vt[(8 * vc + 2 * i + 1) * kVStride + vslot]) = lutv_s[PF::index(Y, i)];
      }
    }
  };
  auto compute = [&](int sb, int64_t pb) {
    const _Float16* Ks = Ks2[sb];
    const _Float16* Vt = Vt2[sb];
    const float* kn_s = kn_s2[sb];
    const float* vn_s = vn_s2[sb];
    // Two sub-blocks of 32 positions, each with its own online-softmax step, so that only 32
    // positions of scores are live at a time; the registers this frees hold operands that are
    // read from LDS two (keys) or three (values) matrix instructions ahead of their use.
    const int64_t first_lim = a.causal ? min(a.kv_len, a.q_pos0 + wrow0 + 1) : a.kv_len;
    const _Float16* kop = Ks + n16 * kKStride + 8 * g;               // + (16 pt) * kKStride + 32 kb
    const _Float16* vop = Vt + n16 * kVStride + 8 * g;               // + (16 et) * kVStride + 32 kb2
#pragma nounroll
    for (int h = 0; h < 2; ++h) {
      // ---- S^T = K Q^T : accumulator (t, ct) holds positions 32h + 16t + 4g + j of row 16ct + n16
      f4 sacc[2][kRowTiles];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ct = 0; ct < kRowTiles; ++ct) sacc[t][ct] = f4{0.f, 0.f, 0.f, 0.f};
      u4 kreg[3];
      kreg[0] = *reinterpret_cast<const u4*>(kop + (32 * h) * kKStride);
      kreg[1] = *reinterpret_cast<const u4*>(kop + (32 * h) * kKStride + 32);
#pragma unroll
      for (int i = 0; i < 8; ++i) {                                   // i = 4t + kb
        if (i + 2 < 8)
          kreg[(i + 2) % 3] = *reinterpret_cast<const u4*>(kop + (32 * h + 16 * ((i + 2) >> 2)) * kKStride +
                                                           32 * ((i + 2) & 3));
        const u4 A = kreg[i % 3];
#pragma unroll
        for (int ct = 0; ct < kRowTiles; ++ct) {
          if (QLO)
            sacc[i >> 2][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, A),
                                                                      __builtin_bit_cast(h8, qlo[ct][i & 3]),
                                                                      sacc[i >> 2][ct], 0, 0, 0);
          sacc[i >> 2][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, A),
                                                                    __builtin_bit_cast(h8, qhi[ct][i & 3]),
                                                                    sacc[i >> 2][ct], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      // first value operands: in flight during the softmax arithmetic
      u4 vreg[4];
#pragma unroll
      for (int i = 0; i < 3; ++i) vreg[i] = *reinterpret_cast<const u4*>(vop + (16 * i) * kVStride + 32 * h);
      __builtin_amdgcn_sched_barrier(0);

      // ---- scale by key norm (log2 units), mask
      const bool need_mask = pb + 32 * (h + 1) > first_lim;              // uniform over the wavefront
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const float4 kn4 = *reinterpret_cast<const float4*>(&kn_s[32 * h + 16 * t + 4 * g]);
        const float knv[4] = {kn4.x, kn4.y, kn4.z, kn4.w};
#pragma unroll
        for (int ct = 0; ct < kRowTiles; ++ct)
#pragma unroll
          for (int j = 0; j < 4; ++j) sacc[t][ct][j] *= knv[j];
      }
      if (need_mask) {
#pragma unroll
        for (int ct = 0; ct < kRowTiles; ++ct) {
          const int64_t r = wrow0 + 16 * ct + n16;
          const int64_t lim = a.causal ? min(a.kv_len, a.q_pos0 + r + 1) : a.kv_len;
          // own positions 32h + 16t + 4g + j are visible while 16t + j < rel
          const int rel = (int)min((int64_t)kBlkPos, max((int64_t)0, lim - pb)) - 4 * g - 32 * h;
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) sacc[t][ct][j] = (16 * t + j >= rel) ? -INFINITY : sacc[t][ct][j];
        }
      }
      // ---- online softmax per row (a row lives in the four lanes n16 + 16g)
      uint32_t pa[kRowTiles][4];
      bool rescale = false;
#pragma unroll
      for (int ct = 0; ct < kRowTiles; ++ct) {
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) mx = fmaxf(mx, sacc[t][ct][j]);
        mx = fmaxf(mx, shfl_xor_f(mx, 16));
        mx = fmaxf(mx, shfl_xor_f(mx, 32));
        const float m_new = fmaxf(m_run[ct], mx);
        const float msafe = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run[ct] - msafe);   // v_exp_f32: 2^-inf = 0, tiny results flush to 0
        rescale = rescale || (alpha != 1.0f);
        m_run[ct] = m_new;
        float lsum = 0.0f;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const float4 vn4 = *reinterpret_cast<const float4*>(&vn_s[32 * h + 16 * t + 4 * g]);
          float p[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            p[j] = __builtin_amdgcn_exp2f(sacc[t][ct][j] - msafe);
            lsum += p[j];
          }
          pa[ct][2 * t] = pack_h2(p[0] * vn4.x, p[1] * vn4.y);
          pa[ct][2 * t + 1] = pack_h2(p[2] * vn4.z, p[3] * vn4.w);
        }
        l_run[ct] = l_run[ct] * alpha + lsum;
        if (g == 0) alpha_s[wave][16 * ct + n16] = alpha;
      }
      // ---- rescale the output accumulators (rows 16ct + 4g + j) when some running maximum moved
      if (__any(rescale)) {
#pragma unroll
        for (int ct = 0; ct < kRowTiles; ++ct) {
          const float4 a4 = *reinterpret_cast<const float4*>(&alpha_s[wave][16 * ct + 4 * g]);
          const float av[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
          for (int et = 0; et < 8; ++et)
#pragma unroll
            for (int j = 0; j < 4; ++j) oacc[ct][et][j] *= av[j];
        }
      }
      // ---- O += P V over the 32 positions of this sub-block
#pragma unroll
      for (int et = 0; et < 8; ++et) {
        if (et + 3 < 8) vreg[(et + 3) & 3] = *reinterpret_cast<const u4*>(vop + (16 * (et + 3)) * kVStride + 32 * h);
        const u4 B = vreg[et & 3];
#pragma unroll
        for (int ct = 0; ct < kRowTiles; ++ct) {
          const u4 A = {pa[ct][0], pa[ct][1], pa[ct][2], pa[ct][3]};
          oacc[ct][et] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, A), __builtin_bit_cast(h8, B),
                                                                oacc[ct][et], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  if (p_lo < p_hi) {
    prefetch(p_lo);
    stage(0);
    __syncthreads();
    if (p_lo + kBlkPos < p_hi) prefetch(p_lo + kBlkPos);
    decode(0);
  }
  int sb = 0;
  for (int64_t pb = p_lo; pb < p_hi; pb += kBlkPos, sb ^= 1) {
    const bool more = pb + kBlkPos < p_hi;
    if (more) stage(sb ^ 1);               // words of block b+1 (fetched during block b-1)
    __syncthreads();                       // block b decoded by all; block b-1 computed by all; stage of b+1 visible
    if (pb + 2 * kBlkPos < p_hi) prefetch(pb + 2 * kBlkPos);
    if (more) decode(sb ^ 1);
    compute(sb, pb);
  }

  // ---- partial results of this split
#pragma unroll
  for (int ct = 0; ct < kRowTiles; ++ct) {
    float l = l_run[ct];
    l += shfl_xor_f(l, 16);
    l += shfl_xor_f(l, 32);
    const int64_t r = wrow0 + 16 * ct + n16;
    if (g == 0 && r < a.n_rows) {
      a.ws_ml[(part + r) * 2] = m_run[ct];
      a.ws_ml[(part + r) * 2 + 1] = l;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t ro = wrow0 + 16 * ct + 4 * g + j;
      if (ro < a.n_rows) {
        float* orow = a.ws_O + (part + ro) * kD;
#pragma unroll
        for (int et = 0; et < 8; ++et) orow[16 * et + n16] = oacc[ct][et][j];
      }
    }
  }
}

// Pre-rotation of the query chunk: q_rot = B(q * signs_K) rounded to fp16.  Four lanes per row.
template <typename T>
__global__ __launch_bounds__(256) void prefill_prerotate_kernel(const T* __restrict__ q,
                                                                const float* __restrict__ signs,
                                                                __half* __restrict__ q_rot,
                                                                __half* __restrict__ q_rot_lo, int64_t n) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int ls = lane & 3, v = lane >> 2;
  const int64_t row = ((int64_t)blockIdx.x * 4 + (tid >> 6)) * kRowsPerWavePass + v;
  const bool ok = row < n;
  const int64_t rr = ok ? row : 0;
  float xs[4][8];
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int e = 32 * k + 8 * ls + j;
      xs[k][j] = load_as_float<T>(q + rr * kD + e) * signs[e];
    }
  butterfly_4lane(xs, (ls & 1) ? 0x80000000u : 0u, (ls & 2) ? 0x80000000u : 0u);
  if (ok) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      u4 w, wl;
#pragma unroll
      for (int jp = 0; jp < 4; ++jp) {
        const __half2 h = __floats2half2_rn(xs[k][2 * jp], xs[k][2 * jp + 1]);
        const float2 back = __half22float2(h);
        w[jp] = *reinterpret_cast<const uint32_t*>(&h);
        wl[jp] = pack_h2(xs[k][2 * jp] - back.x, xs[k][2 * jp + 1] - back.y);
      }
      *reinterpret_cast<u4*>(q_rot + row * kD + 32 * k + 8 * ls) = w;
      *reinterpret_cast<u4*>(q_rot_lo + row * kD + 32 * k + 8 * ls) = wl;
    }
  }
}

// Merge of the splits and the final butterfly: out[r] = B(sum_s f_s O_s[r]) * signs_V * unscale / L,
// f_s = 2^(m_s - max m), L = sum_s f_s l_s.  Four lanes per row.
template <typename TO>
__global__ __launch_bounds__(256) void prefill_merge_kernel(const float* __restrict__ ws_O,
                                                            const float* __restrict__ ws_ml,
                                                            const float* __restrict__ signs, TO* __restrict__ out,
                                                            int64_t n /* n_q * n_rows */, int n_splits, float unscale) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int ls = lane & 3, v = lane >> 2;
  const int64_t row = ((int64_t)blockIdx.x * 4 + (tid >> 6)) * kRowsPerWavePass + v;
  const bool ok = row < n;
  const int64_t rr = ok ? row : 0;
  float M = -INFINITY;
  for (int s = 0; s < n_splits; ++s) M = fmaxf(M, ws_ml[((int64_t)s * n + rr) * 2]);
  float acc[4][8];
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[k][j] = 0.0f;
  float L = 0.0f;
  for (int s = 0; s < n_splits; ++s) {
    const float ms = ws_ml[((int64_t)s * n + rr) * 2];
    if (ms == -INFINITY) continue;                                       // this split saw no position of the row
    const float f = exp2f(ms - M);
    L += f * ws_ml[((int64_t)s * n + rr) * 2 + 1];
    const float* src = ws_O + ((int64_t)s * n + rr) * kD + 8 * ls;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float4 x0 = *reinterpret_cast<const float4*>(src + 32 * k);
      const float4 x1 = *reinterpret_cast<const float4*>(src + 32 * k + 4);
      acc[k][0] += f * x0.x; acc[k][1] += f * x0.y; acc[k][2] += f * x0.z; acc[k][3] += f * x0.w;
      acc[k][4] += f * x1.x; acc[k][5] += f * x1.y; acc[k][6] += f * x1.z; acc[k][7] += f * x1.w;
    }
  }
  butterfly_4lane(acc, (ls & 1) ? 0x80000000u : 0u, (ls & 2) ? 0x80000000u : 0u);
  const float scale = (L > 0.0f) ? unscale / L : 0.0f;
  if (ok) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int e = 32 * k + 8 * ls + j;
        store_from_float<TO>(out + row * kD + e, acc[k][j] * signs[e] * scale);
      }
  }
}

struct SplitPlan { int n_splits, cap; int64_t split_len; };

// Splits of the key positions: a workgroup fills a CU (LDS), so the launch runs in rounds of 256 workgroups and
// its duration goes as rounds * split length, i.e. as ceil(columns * n / 256) / n for n splits of
// columns = row blocks * query heads.  The smallest n within 3 % of the best such figure is taken (fewer splits =
// less merge traffic: 4 at benchmark configuration 5, one workgroup per CU), with at least 8 blocks of positions
// per split and at most 32 splits.  cap bounds n_splits for every shorter kv_len too (the causal launch may see
// fewer positions than the workspace was sized for).
SplitPlan plan_splits(int n_q, int64_t n_rows, int64_t kv_len) {
  const int64_t row_blocks = (n_rows + kWgRows - 1) / kWgRows;
  const int64_t blocks = (kv_len + kBlkPos - 1) / kBlkPos;
  const int64_t cols = row_blocks * n_q;
  int64_t most = blocks / 8 > 0 ? blocks / 8 : 1;
  if (most > 32) most = 32;
  int64_t want = 1;
  double best = 1e30;
  for (int64_t n = 1; n <= most; ++n) {
    const double cost = (double)((cols * n + 255) / 256) / (double)n;
    if (cost < best * 0.97) { best = cost; want = n; }
  }
  const int64_t per = (blocks + want - 1) / want;
  SplitPlan p;
  p.cap = (int)want;      // the scan is a prefix of itself for any shorter kv_len, so its choice there is <= want
  p.split_len = per * kBlkPos;
  p.n_splits = (int)((blocks + per - 1) / per);
  if (p.n_splits < 1) p.n_splits = 1;
  return p;
}

size_t align256(size_t v) { return (v + 255) / 256 * 256; }

}  // namespace

extern "C" size_t tq_prefill_workspace_bytes(int n_q_heads, int64_t n_rows, int64_t kv_len, int dim) {
  if (n_q_heads < 1 || n_rows < 1 || kv_len < 1 || dim != kD) return 0;
  const SplitPlan p = plan_splits(n_q_heads, n_rows, kv_len);
  const size_t rows = (size_t)n_q_heads * (size_t)n_rows;
  return 2 * align256(rows * kD * sizeof(__half)) + align256((size_t)p.cap * rows * kD * sizeof(float)) +
         align256((size_t)p.cap * rows * 2 * sizeof(float));
}

extern "C" int tq_prefill_attn(const void* q, int q_dtype, const uint32_t* k_packed, const float* k_norms,
                               const uint32_t* v_packed, const float* v_norms, const float* k_centroids,
                               const float* v_centroids, const float* k_signs, const float* v_signs, void* out,
                               int out_dtype, void* workspace, size_t workspace_bytes, int n_kv_heads, int n_rep,
                               int64_t n_rows, int64_t kv_len, int64_t q_pos0, int64_t k_head_stride,
                               int64_t kn_head_stride, int64_t v_head_stride, int64_t vn_head_stride, int dim,
                               int bits, float attn_scale, int flags, tq_stream_t stream_) {
  const char* who = "tq_prefill_attn";
  if (flags & ~(TQ_PREFILL_CAUSAL | TQ_PREFILL_FP16_QUERY))
    return tq::fail(TQ_ERR_ARG, "%s: unknown flag bits 0x%x", who, flags);
  const int causal = flags & TQ_PREFILL_CAUSAL;
  if (int rc = tq::check_dim_bits(dim, bits)) return rc;
  if (dim != kD)
    return tq::fail(TQ_ERR_UNSUPPORTED, "%s: only dim 128 has a kernel, got dim %d", who, dim);
  if (n_kv_heads < 1) return tq::fail(TQ_ERR_ARG, "%s: n_kv_heads must be >= 1, got %d", who, n_kv_heads);
  if (n_rep < 1) return tq::fail(TQ_ERR_NREP, "%s: n_rep must be >= 1, got %d", who, n_rep);
  if (tq::check_dtype(q_dtype) || tq::check_dtype(out_dtype)) return tq::fail(TQ_ERR_DTYPE, "%s: unknown dtype", who);
  if (n_rows < 0 || kv_len < 0 || q_pos0 < 0) return tq::fail(TQ_ERR_ARG, "%s: negative size", who);
  if (n_rows == 0) return TQ_OK;
  if (kv_len < 1) return tq::fail(TQ_ERR_ARG, "%s: kv_len must be >= 1", who);
  if (causal && q_pos0 + 1 > kv_len)
    return tq::fail(TQ_ERR_ARG, "%s: causal chunk starts at position %lld beyond the %lld cached positions", who,
                    (long long)q_pos0, (long long)kv_len);
  if (k_head_stride < kv_len || kn_head_stride < kv_len || v_head_stride < kv_len || vn_head_stride < kv_len)
    return tq::fail(TQ_ERR_ARG, "%s: a head stride is smaller than kv_len (%lld)", who, (long long)kv_len);
  if (!q || !k_packed || !k_norms || !v_packed || !v_norms || !k_centroids || !v_centroids || !k_signs ||
      !v_signs || !out || !workspace)
    return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (!tq::aligned(q, tq::dtype_size(q_dtype)) || !tq::aligned(out, tq::dtype_size(out_dtype)) ||
      !tq::aligned(k_packed, 4) || !tq::aligned(v_packed, 4) || !tq::aligned(workspace, 256))
    return tq::fail(TQ_ERR_ALIGN, "%s: misaligned pointer (workspace needs 256 bytes)", who);
  const int n_q = n_kv_heads * n_rep;
  // positions past the last row's own are never visible under the causal rule
  const int64_t kv_eff = causal ? (kv_len < q_pos0 + n_rows ? kv_len : q_pos0 + n_rows) : kv_len;
  const size_t need = tq_prefill_workspace_bytes(n_q, n_rows, kv_len, dim);
  if (workspace_bytes < need)
    return tq::fail(TQ_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
  const SplitPlan plan = plan_splits(n_q, n_rows, kv_eff);       // never more splits than the size above holds
  const size_t rows = (size_t)n_q * (size_t)n_rows;
  char* ws = (char*)workspace;
  __half* q_rot = (__half*)ws;
  __half* q_rot_lo = (__half*)(ws + align256(rows * kD * sizeof(__half)));
  float* ws_O = (float*)(ws + 2 * align256(rows * kD * sizeof(__half)));
  float* ws_ml = (float*)((char*)ws_O + align256((size_t)plan.n_splits * rows * kD * sizeof(float)));
  hipStream_t stream = (hipStream_t)stream_;

  const int rgrid = (int)((rows + 4 * kRowsPerWavePass - 1) / (4 * kRowsPerWavePass));
  if (q_dtype == TQ_F32)
    prefill_prerotate_kernel<float><<<rgrid, 256, 0, stream>>>((const float*)q, k_signs, q_rot, q_rot_lo, (int64_t)rows);
  else if (q_dtype == TQ_F16)
    prefill_prerotate_kernel<__half><<<rgrid, 256, 0, stream>>>((const __half*)q, k_signs, q_rot, q_rot_lo, (int64_t)rows);
  else
    prefill_prerotate_kernel<__hip_bfloat16><<<rgrid, 256, 0, stream>>>((const __hip_bfloat16*)q, k_signs, q_rot,
                                                                        q_rot_lo, (int64_t)rows);
  TQ_CHECK_LAUNCH("tq_prefill_attn pre-rotation");

  PrefillArgs a{};
  a.q_rot = q_rot; a.q_rot_lo = q_rot_lo; a.k_packed = k_packed; a.k_norms = k_norms; a.v_packed = v_packed; a.v_norms = v_norms;
  a.ws_O = ws_O; a.ws_ml = ws_ml;
  a.n_rows = n_rows; a.kv_len = kv_eff; a.q_pos0 = q_pos0;
  a.k_head_stride = k_head_stride; a.kn_head_stride = kn_head_stride;
  a.v_head_stride = v_head_stride; a.vn_head_stride = vn_head_stride;
  a.split_len = plan.split_len;
  a.n_q = n_q; a.n_rep = n_rep; a.causal = causal ? 1 : 0;
  Codebook kcb, vcb;
  const float k_unscale = tq::fill_codebook_fp16(kcb, k_centroids, bits);
  const float v_unscale = tq::fill_codebook_fp16(vcb, v_centroids, bits);
  a.score_scale = attn_scale / (float)dim * k_unscale * kLog2e;
  dim3 grid(plan.n_splits, (unsigned)((n_rows + kWgRows - 1) / kWgRows), n_q);
  if (flags & TQ_PREFILL_FP16_QUERY) {
    TQ_DISPATCH_BITS(bits, (prefill_tile_kernel<B_, false><<<grid, kThreads, 0, stream>>>(a, kcb, vcb)));
  } else {
    TQ_DISPATCH_BITS(bits, (prefill_tile_kernel<B_><<<grid, kThreads, 0, stream>>>(a, kcb, vcb)));
  }
  TQ_CHECK_LAUNCH("tq_prefill_attn tile pass");

  const float unscale = v_unscale / kVnScale / (float)dim;
  if (out_dtype == TQ_F32)
    prefill_merge_kernel<float><<<rgrid, 256, 0, stream>>>(ws_O, ws_ml, v_signs, (float*)out, (int64_t)rows,
                                                           plan.n_splits, unscale);
  else if (out_dtype == TQ_F16)
    prefill_merge_kernel<__half><<<rgrid, 256, 0, stream>>>(ws_O, ws_ml, v_signs, (__half*)out, (int64_t)rows,
                                                            plan.n_splits, unscale);
  else
    prefill_merge_kernel<__hip_bfloat16><<<rgrid, 256, 0, stream>>>(ws_O, ws_ml, v_signs, (__hip_bfloat16*)out,
                                                                    (int64_t)rows, plan.n_splits, unscale);
  TQ_CHECK_LAUNCH("tq_prefill_attn merge pass");
  return TQ_OK;
}
