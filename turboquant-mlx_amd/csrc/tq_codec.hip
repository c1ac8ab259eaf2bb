// PolarQuant codec kernels for gfx950: fused encode, dequantise, query pre-rotation and the
// per-row-butterfly QK scoring.  One wavefront owns one vector; the Walsh-Hadamard butterfly
// and the norm reduction run on lane exchanges, never through LDS barriers.
#include "tq_common.h"

#include <math.h>
#include <cmath>
#include <string.h>
#include <mutex>

namespace {

using namespace tqd;

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * TQ_WAVE;

struct Thresholds { float t[15]; };

struct RowMap {
  int64_t n_rows, rows_per_group, packed_group_stride, norms_group_stride, out_group_stride;
};

// Optional row copies done by the wavefront that encodes a row (the append of a cache that keeps
// float16 keys beside its packed values): key row `row` of k_src (dtype k_dtype) goes, converted to
// float16, to k_dst + (g * k_group_stride + r) * D, and the value row itself, unchanged, to
// v_dst + (g * v_group_stride + r) * D.  Null destinations switch a copy off.
// With pos_dev set, every destination row index (packed words, norms and the two copies) is
// shifted by the value pos_dev points to, read on the GPU when the kernel runs: a launch recorded
// once (HIP graph) then inserts at whatever position the device counter holds.  Rows that would
// land outside 0 .. pos_cap - 1 are not stored.
struct RowCopy {
  const void* k_src;
  __half* k_dst;
  void* v_dst;
  int64_t k_group_stride, v_group_stride;
  int k_dtype;
  const int64_t* pos_dev;
  int64_t pos_cap;
};

// ---------------------------------------------------------------- encode
// Per vector: sum of squares in stride-halving tree order, sqrt, divide by max(n, 1e-8), sign
// flip, raw butterfly, count of thresholds exceeded (strict >), pack.  `thr` holds the decision
// thresholds in the domain of the raw butterfly output (see encode_thresholds below).
template <int D, int BITS, typename T>
__global__ __launch_bounds__(kBlock) void encode_kernel(const T* __restrict__ x,
                                                        const float* __restrict__ signs,
                                                        Thresholds thr, uint32_t* __restrict__ packed,
                                                        float* __restrict__ norms, RowMap rm, RowCopy rc) {
  constexpr int EPL = Lay<D>::EPL;
  constexpr int VPW = Pk<BITS>::VPW;
  constexpr int PDIM = Pk<BITS>::pdim(D);
  constexpr int NB = (1 << BITS) - 1;
  __shared__ uint8_t idx_s[kWavesPerBlock][D >= 64 ? D : 64];

  const int lane = threadIdx.x & (TQ_WAVE - 1);
  const int wave = threadIdx.x >> 6;
  float sg[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    int e = lane + 64 * i;
    sg[i] = (e < D) ? signs[e] : 0.0f;
  }
  const int64_t rows_per_sweep = (int64_t)gridDim.x * kWavesPerBlock;
  const int64_t n_iter = (rm.n_rows + rows_per_sweep - 1) / rows_per_sweep;
  for (int64_t it = 0; it < n_iter; ++it) {
    const int64_t row = (it * gridDim.x + blockIdx.x) * kWavesPerBlock + wave;
    const bool valid = row < rm.n_rows;
    float xv[EPL], sq[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      int e = lane + 64 * i;
      xv[i] = (valid && e < D) ? load_as_float<T>(x + row * D + e) : 0.0f;
      sq[i] = xv[i] * xv[i];
    }
    const float ss = tree_sum<D>(sq);
    const float nrm = sqrtf(ss);
    const float safe = fmaxf(nrm, 1e-8f);
    float v[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) v[i] = (xv[i] / safe) * sg[i];
    raw_butterfly<D>(v, lane);
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      uint32_t idx = 0;
#pragma unroll
      for (int b = 0; b < NB; ++b) idx += (v[i] > thr.t[b]) ? 1u : 0u;
      int e = lane + 64 * i;
      if (e < D) idx_s[wave][e] = (uint8_t)idx;
    }
    __syncthreads();
    if (valid) {
      const int64_t g = row / rm.rows_per_group;
      int64_t r = row - g * rm.rows_per_group;
      bool store = true;
      if (rc.pos_dev) {
        r += *rc.pos_dev;
        store = r >= 0 && r < rc.pos_cap;
      }
      if (store) {
      if (lane < PDIM) {
        uint32_t word = 0;
#pragma unroll
        for (int i = 0; i < VPW; ++i) {
          int e = lane * VPW + i;
          if (e < D) word |= (uint32_t)idx_s[wave][e] << (i * BITS);
        }
        packed[(g * rm.packed_group_stride + r) * PDIM + lane] = word;
      }
      if (lane == 0) norms[g * rm.norms_group_stride + r] = nrm;
      if (rc.v_dst) {
        T* vd = (T*)rc.v_dst + (g * rc.v_group_stride + r) * D;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
          const int e = lane + 64 * i;
          if (e < D) vd[e] = x[row * D + e];
        }
      }
      if (rc.k_dst) {
        __half* kd = rc.k_dst + (g * rc.k_group_stride + r) * D;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
          const int e = lane + 64 * i;
          if (e < D) {
            const int64_t at = row * D + e;
            if (rc.k_dtype == TQ_F16) kd[e] = ((const __half*)rc.k_src)[at];
            else if (rc.k_dtype == TQ_F32) kd[e] = __float2half_rn(((const float*)rc.k_src)[at]);
            else kd[e] = __float2half_rn(__bfloat162float(((const __hip_bfloat16*)rc.k_src)[at]));
          }
        }
      }
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- encode, d = 128
// The streaming encoder for the cache's own head dimension (every width; the notes below describe three bits,
// the width-dependent parts are the level table and the word assembly at the end of a pass).  Four lanes own one vector, so a wavefront
// encodes 16 vectors per pass: lane ls = lane % 4 of a vector holds the four 8-element chunks
// c = ls + 4k (k = 0..3), element e = 32k + 8ls + j.  Each load instruction therefore reads 64
// contiguous bytes per vector; butterfly stages 1, 2, 4, 32 and 64 and five of the seven levels of
// the sum-of-squares tree stay inside a lane, and stages 8 and 16 are quad-permute lane exchanges
// folded into the add.  Results are bit-identical to encode_kernel:
//  * the sum of squares is added in the same stride-halving tree order;
//  * x / n is computed as q = x*r, q += r * fma(-n, q, x) with r = 1/n correctly rounded, which
//    yields the correctly rounded quotient (checked against IEEE division on 3e10 operand pairs
//    with |x| <= n), at 3 operations per element instead of a full division;
//  * the count of thresholds exceeded is g + (w > t[g]) where g is a guess that the host has verified to be
//    the count or one less for every w: v = fma(w, alpha, beta + 2^20 + 32) lies in [2^20, 2^21), where
//    floats are 1/8 apart, so bits 3..8 of v are 32 + floor(alpha*w + beta) (to within the rounding to
//    1/8) and, masked, are the byte offset into a 64-entry LDS table of (t[g], g) pairs whose entries
//    below / above the seven levels hold (+inf, 0) / (-inf, 6): no clamp, no float-to-int convert, no
//    address shift.  A NaN norm forces all indices of the vector to 0 (as comparisons with NaN do).
// Packed words leave through LDS so that a wavefront stores 208 contiguous words per pass.
// Mixed-precision FMA on one half of a packed fp16 pair (HI = 0: low half, 1: high half), so that fp16
// inputs need no separate widening instruction.  A product is taken as fma(a, b, -0): adding -0 changes
// no value, not even the sign of a zero, so it rounds exactly like the float32 multiply of the widened
// operands.
template <int HI>
__device__ __forceinline__ float mix_sq(uint32_t h2, float negzero) {           // widen(h) * widen(h)
  float d;
  if (HI) asm("v_fma_mix_f32 %0, %1, %1, %2 op_sel:[1,1,0] op_sel_hi:[1,1,0]" : "=v"(d) : "v"(h2), "v"(negzero));
  else    asm("v_fma_mix_f32 %0, %1, %1, %2 op_sel:[0,0,0] op_sel_hi:[1,1,0]" : "=v"(d) : "v"(h2), "v"(negzero));
  return d;
}
template <int HI>
__device__ __forceinline__ float mix_mul(uint32_t h2, float b, float negzero) { // widen(h) * b
  float d;
  if (HI) asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(d) : "v"(h2), "v"(b), "v"(negzero));
  else    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(d) : "v"(h2), "v"(b), "v"(negzero));
  return d;
}
template <int HI>
__device__ __forceinline__ float mix_fma_addend(float a, float b, uint32_t h2) { // fma(a, b, widen(h))
  float d;
  if (HI) asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "=v"(d) : "v"(a), "v"(b), "v"(h2));
  else    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[0,0,1]" : "=v"(d) : "v"(a), "v"(b), "v"(h2));
  return d;
}

// The 8 * BITS bits that hold elements 8c .. 8c+7 (chunk c) of a packed d = 128 row: word and shifts.  Three-bit
// rows hold ten fields per word, so a chunk may straddle two words (chunk 15 is all of word 12: taken as word
// 11 >> 30, which is 0, | word 12); the other widths divide the word.
template <int BITS>
struct Chunk {
  static constexpr int kPd = BITS == 3 ? 13 : 4 * BITS;       // words per row
  static constexpr uint32_t kPairMask = (1u << (2 * BITS)) - 1u;
  __device__ static __forceinline__ void pos(int c, int& w0, int& sh_lo, int& sh_hi) {
    if (BITS == 3) {
      w0 = (c == 15) ? 11 : (8 * c) / 10;
      const int s0 = (c == 15) ? 10 : (8 * c) % 10;
      sh_lo = 3 * s0;
      sh_hi = 30 - 3 * s0;
    } else {
      constexpr int kPerWord = 4 / BITS;
      w0 = c / kPerWord;
      sh_lo = (c % kPerWord) * 8 * BITS;
      sh_hi = 0;
    }
  }
  __device__ static __forceinline__ uint32_t field(const uint32_t* at_w0, int sh_lo, int sh_hi) {
    if (BITS == 3) return ((at_w0[0] >> sh_lo) | (at_w0[1] << sh_hi)) & 0xFFFFFFu;
    if (BITS == 4) return at_w0[0];
    return (at_w0[0] >> sh_lo) & ((1u << (8 * BITS)) - 1u);
  }
};

constexpr int kEncVecs = 16;      // vectors per wavefront pass
constexpr int kEncPasses = 4;     // passes per wavefront once there are rows enough to fill the chip

// alpha and beta of the level guess; beta0 = beta without the 2^20 + 32 that places the guess in the mantissa
struct EncodeGuess { float alpha, beta, beta0; };

// BITS = 3: every threshold j sits in cell j of the guess (level_guess_search), and the table is written down
// directly.  Other widths: any guess line under which no cell holds two thresholds (level_cells_search); cell
// c = floor(alpha * w + beta0) then knows the count g of thresholds below its lower edge and the one threshold it
// may hold (else +inf: nothing to compare with), both derived here from the thresholds themselves.
template <typename T, int BITS = 3>
__global__ __launch_bounds__(kBlock) void encode128x3_kernel(const T* __restrict__ x,
                                                             const float* __restrict__ signs, Thresholds thr,
                                                             EncodeGuess gs, uint32_t* __restrict__ packed,
                                                             float* __restrict__ norms, RowMap rm, int passes) {
  constexpr bool kHalfWidth = sizeof(T) == 2;
  constexpr int NM = kHalfWidth ? 4 : 8;                       // sign masks per chunk
  constexpr int NB = (1 << BITS) - 1;                          // thresholds
  constexpr int kPd = Chunk<BITS>::kPd;
  constexpr int kCells = BITS == 4 ? 128 : 64;                 // cells of the level guess (fifteen thresholds need finer ones)
  __shared__ __align__(8) uint2 lvl_s[kCells];                 // (threshold bits, guess) by kCells / 2 + floor(alpha*w + beta0)
  __shared__ __align__(16) float sg_s[128];
  __shared__ uint32_t chunk_s[kWavesPerBlock][kEncVecs * 16 + 4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ls = lane & 3, v = lane >> 2;
  if (tid < kCells) {
    const int gq = tid - kCells / 2;
    if (BITS == 3) {
      float t = gq < 0 ? INFINITY : -INFINITY;
#pragma unroll
      for (int i = 0; i < 7; ++i) t = (gq == i) ? thr.t[i] : t;
      lvl_s[tid] = make_uint2(__float_as_uint(t), (uint32_t)(gq < 0 ? 0 : (gq > 6 ? 6 : gq)));
    } else {
      int g = 0;                                               // thresholds below the cell's lower edge
#pragma unroll
      for (int i = 0; i < NB; ++i) g += (__fmaf_rn(thr.t[i], gs.alpha, gs.beta0) < (float)gq) ? 1 : 0;
      float t = INFINITY;                                      // threshold number g, if it lies inside the cell
#pragma unroll
      for (int i = 0; i < NB; ++i)
        t = (i == g && __fmaf_rn(thr.t[i], gs.alpha, gs.beta0) < (float)(gq + 1)) ? thr.t[i] : t;
      lvl_s[tid] = make_uint2(__float_as_uint(t), (uint32_t)g);
    }
  }
  if (tid < 128) sg_s[tid] = signs[tid];
  __syncthreads();

  // sign flips as xor masks on the raw input bits
  uint32_t sm[4][NM];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float4 a = *reinterpret_cast<const float4*>(&sg_s[32 * k + 8 * ls]);
    const float4 b = *reinterpret_cast<const float4*>(&sg_s[32 * k + 8 * ls + 4]);
    const float sv[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    if (kHalfWidth) {
#pragma unroll
      for (int jp = 0; jp < 4; ++jp)
        sm[k][jp] = ((__float_as_uint(sv[2 * jp]) >> 16) & 0x8000u) | (__float_as_uint(sv[2 * jp + 1]) & 0x80000000u);
    } else {
#pragma unroll
      for (int j = 0; j < NM; ++j) sm[k][j] = __float_as_uint(sv[j & 7]) & 0x80000000u;
    }
  }
  // lanes 1 and 2 of a vector take their inputs negated (folded into the sign masks): butterfly_4lane_neg12
  if (ls == 1 || ls == 2) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int j = 0; j < NM; ++j) sm[k][j] ^= kHalfWidth ? 0x80008000u : 0x80000000u;
  }
  const float m1 = (ls & 1) ? 1.0f : -1.0f, m2 = (ls & 2) ? 1.0f : -1.0f;
  uint32_t* chunks = chunk_s[wave];

  // first batch of 16 rows of this wavefront and its place in the (group, row) map
  const uint32_t batch0 = ((uint32_t)blockIdx.x * kWavesPerBlock + wave) * (uint32_t)passes;
  uint32_t row0 = batch0 * kEncVecs;
  uint32_t grp = row0 / (uint32_t)rm.rows_per_group;
  uint32_t rin = row0 - grp * (uint32_t)rm.rows_per_group;

  // 16-bit inputs: the rows of the next pass are fetched while the current one is computed
  uint4 nraw[4] = {};
  if (kHalfWidth && row0 < (uint32_t)rm.n_rows) {
    const T* xr = x + ((int64_t)row0 + v) * 128 + 8 * ls;
#pragma unroll
    for (int k = 0; k < 4; ++k) nraw[k] = *reinterpret_cast<const uint4*>(xr + 32 * k);
  }
  for (int pass = 0; pass < passes; ++pass) {
    if (row0 >= (uint32_t)rm.n_rows) break;                    // uniform over the wavefront
    // ---- load, flip signs, widen (fp16: the packed pairs stay as they are and are widened inside the
    // mixed-precision multiplies below)
    constexpr bool kMix = __is_same(T, __half);
    float xs[4][8];
    uint32_t hw[4][4];
    const T* xr = x + ((int64_t)row0 + v) * 128 + 8 * ls;
    if (kHalfWidth) {
      uint4 raw[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) raw[k] = nraw[k];
      if (pass + 1 < passes && row0 + kEncVecs < (uint32_t)rm.n_rows) {
#pragma unroll
        for (int k = 0; k < 4; ++k) nraw[k] = *reinterpret_cast<const uint4*>(xr + kEncVecs * 128 + 32 * k);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t w[4] = {raw[k].x ^ sm[k][0], raw[k].y ^ sm[k][1], raw[k].z ^ sm[k][2], raw[k].w ^ sm[k][3]};
#pragma unroll
        for (int jp = 0; jp < 4; ++jp) {
          hw[k][jp] = w[jp];
          if (!kMix) {
            xs[k][2 * jp] = __uint_as_float(w[jp] << 16);
            xs[k][2 * jp + 1] = __uint_as_float(w[jp] & 0xFFFF0000u);
          }
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint4 a = *reinterpret_cast<const uint4*>(xr + 32 * k);
        const uint4 b = *reinterpret_cast<const uint4*>(xr + 32 * k + 4);
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) xs[k][j] = __uint_as_float(w[j] ^ sm[k][j & (NM - 1)]);
      }
    }
    const float negzero = -0.0f;
    // ---- sum of squares: strides 64, 32 (k), 16, 8 (lanes), 4, 2, 1 (j)
    float t8[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float sq[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (kMix) sq[k] = (j & 1) ? mix_sq<1>(hw[k][j >> 1], negzero) : mix_sq<0>(hw[k][j >> 1], negzero);
        else sq[k] = xs[k][j] * xs[k][j];
      }
      t8[j] = (sq[0] + sq[2]) + (sq[1] + sq[3]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) t8[j] = t8[j] + quad_xor2(t8[j]);
#pragma unroll
    for (int j = 0; j < 8; ++j) t8[j] = t8[j] + quad_xor1(t8[j]);
    const float ss = ((t8[0] + t8[4]) + (t8[2] + t8[6])) + ((t8[1] + t8[5]) + (t8[3] + t8[7]));
    const float nrm = sqrtf(ss);
    const float safe = fmaxf(nrm, 1e-8f);
    const float rinv = 1.0f / safe;
    // a norm that overflowed to infinity: x / inf is 0 for every finite x, which q = x * 0 already is; the
    // correction term must then not multiply infinity by that zero
    const float nsafe = (safe == INFINITY) ? 0.0f : -safe;
    // ---- unit vector
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (kMix) {
          const uint32_t h2 = hw[k][j >> 1];
          const float q0 = (j & 1) ? mix_mul<1>(h2, rinv, negzero) : mix_mul<0>(h2, rinv, negzero);
          const float rem = (j & 1) ? mix_fma_addend<1>(nsafe, q0, h2) : mix_fma_addend<0>(nsafe, q0, h2);
          xs[k][j] = __fmaf_rn(rem, rinv, q0);
        } else {
          const float q0 = xs[k][j] * rinv;
          const float rem = __fmaf_rn(nsafe, q0, xs[k][j]);
          xs[k][j] = __fmaf_rn(rem, rinv, q0);
        }
      }
    butterfly_4lane_neg12(xs, m1, m2);
    // ---- levels, 8 * BITS bits per chunk
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      uint32_t bits24 = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float w = xs[k][j];
        const uint32_t off = __float_as_uint(__fmaf_rn(w, gs.alpha, gs.beta)) & (uint32_t)((kCells - 1) << 3);
        const uint2 lv = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned char*>(lvl_s) + off);
        const uint32_t idx = lv.y + ((w > __uint_as_float(lv.x)) ? 1u : 0u);
        bits24 |= idx << (BITS * j);
      }
      chunks[v * 16 + ls + 4 * k] = (nrm != nrm) ? 0u : bits24;
    }
    // ---- words.  Three bits: word wd of a row holds elements 10wd .. 10wd+9 = chunks (5wd)/4 and the next;
    // four bits: a chunk is a word; two bits / one bit: two / four chunks make a word
    uint32_t* prow = packed + ((int64_t)grp * rm.packed_group_stride + rin) * kPd;
#pragma unroll
    for (int it = 0; it < (kEncVecs * kPd + 63) / 64; ++it) {
      const int id = it * 64 + lane;
      if (id < kEncVecs * kPd) {
        const int vv = id / kPd, wd = id - kPd * vv;
        uint32_t word;
        if (BITS == 3) {
          const int a = (5 * wd) >> 2, sh = 3 * ((10 * wd) & 7);
          const uint32_t lo = chunks[vv * 16 + a], hi = chunks[vv * 16 + a + 1];
          word = ((lo >> sh) | (hi << (24 - sh))) & (wd == 12 ? 0xFFFFFFu : 0x3FFFFFFFu);
        } else if (BITS == 4) {
          word = chunks[vv * 16 + wd];
        } else if (BITS == 2) {
          word = chunks[vv * 16 + 2 * wd] | (chunks[vv * 16 + 2 * wd + 1] << 16);
        } else {
          word = chunks[vv * 16 + 4 * wd] | (chunks[vv * 16 + 4 * wd + 1] << 8) | (chunks[vv * 16 + 4 * wd + 2] << 16) |
                 (chunks[vv * 16 + 4 * wd + 3] << 24);
        }
        prow[id] = word;
      }
    }
    if (ls == 0) norms[(int64_t)grp * rm.norms_group_stride + rin + v] = nrm;
    row0 += kEncVecs;
    rin += kEncVecs;
    if (rin >= (uint32_t)rm.rows_per_group) { rin = 0; ++grp; }
  }
}

// ---------------------------------------------------------------- dequant
template <int D, int BITS>
__device__ __forceinline__ void load_centroid_values(const uint32_t* __restrict__ prow, const float* cb,
                                                     int lane, float s, float (&v)[Lay<D>::EPL]) {
  constexpr int EPL = Lay<D>::EPL;
  constexpr int VPW = Pk<BITS>::VPW;
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    int e = lane + 64 * i;
    float val = 0.0f;
    if (e < D) {
      uint32_t word = prow[e / VPW];
      uint32_t idx = (word >> ((e % VPW) * BITS)) & Pk<BITS>::MASK;
      val = cb[idx] * s;
    }
    v[i] = val;
  }
}

template <int D, int BITS, typename TO>
__global__ __launch_bounds__(kBlock) void dequant_kernel(const uint32_t* __restrict__ packed,
                                                         const float* __restrict__ norms, Codebook cbk,
                                                         const float* __restrict__ signs, float s,
                                                         TO* __restrict__ out, RowMap rm) {
  constexpr int EPL = Lay<D>::EPL;
  constexpr int PDIM = Pk<BITS>::pdim(D);
  __shared__ float cb[16];
  if (threadIdx.x < 16) cb[threadIdx.x] = cbk.c[threadIdx.x];
  __syncthreads();
  const int lane = threadIdx.x & (TQ_WAVE - 1);
  const int wave = threadIdx.x >> 6;
  float sg[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    int e = lane + 64 * i;
    sg[i] = (e < D) ? signs[e] : 0.0f;
  }
  const int64_t rows_per_sweep = (int64_t)gridDim.x * kWavesPerBlock;
  for (int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + wave; row < rm.n_rows; row += rows_per_sweep) {
    const int64_t g = row / rm.rows_per_group;
    const int64_t r = row - g * rm.rows_per_group;
    const uint32_t* prow = packed + (g * rm.packed_group_stride + r) * PDIM;
    const float nrm = norms[g * rm.norms_group_stride + r];
    float v[EPL];
    load_centroid_values<D, BITS>(prow, cb, lane, s, v);
    raw_butterfly<D>(v, lane);
    TO* orow = out + (g * rm.out_group_stride + r) * D;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      int e = lane + 64 * i;
      if (e < D) store_from_float<TO>(orow + e, ((v[i] * s) * sg[i]) * nrm);
    }
  }
}

// ---------------------------------------------------------------- dequant, d = 128
// Same four-lanes-per-vector layout as encode128x3_kernel, every width.  The packed words of a pass (208 at
// three bits) are read with coalesced loads into LDS; a lane cuts the 8 * BITS bits of each of its chunks out
// of one or two words and looks centroid pairs up in a table of 4^BITS entries (c[a]*s, c[b]*s).  Arithmetic per
// element, in this order, as in dequant_kernel: butterfly, * s, * sign, * norm, round to TO.
template <typename TO, int BITS = 3>
__global__ __launch_bounds__(kBlock) void dequant128x3_kernel(const uint32_t* __restrict__ packed,
                                                              const float* __restrict__ norms, Codebook cbk,
                                                              const float* __restrict__ signs, float s,
                                                              TO* __restrict__ out, RowMap rm, int passes) {
  using CK = Chunk<BITS>;
  constexpr int kPd = CK::kPd;
  constexpr int kPairs = 1 << (2 * BITS);                      // entries of the centroid-pair table
  constexpr int kWordLoads = (kEncVecs * kPd + 63) / 64;       // wave-wide loads of a pass's packed words
  __shared__ __align__(16) float sg_s[128];
  // centroid pairs, and after them the same pairs negated: lanes 1 and 2 of a vector read those (butterfly_4lane_neg12)
  __shared__ __align__(8) float2 pair_s[2 * kPairs];
  __shared__ uint32_t words_s[kWavesPerBlock][kEncVecs * kPd + 3];
  // Outputs leave through LDS: 16 rows of 256 (16-bit) or 512 (float32) bytes at a padded pitch (conflict-free
  // 16-byte writes per lane and reads per row segment), so that every store instruction writes 1 KB of
  // contiguous memory
  constexpr int kPitch = sizeof(TO) == 2 ? 320 : 528;          // row of 256 / 512 bytes plus padding
  __shared__ __align__(16) unsigned char orow_s[kWavesPerBlock][kEncVecs * kPitch];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ls = lane & 3, v = lane >> 2;
  if (tid < kPairs) {                                          // kBlock = 256 threads cover the largest table
    float clo = 0.0f, chi = 0.0f;
#pragma unroll
    for (int i = 0; i < (1 << BITS); ++i) {
      clo = ((tid & ((1 << BITS) - 1)) == i) ? cbk.c[i] : clo;
      chi = ((tid >> BITS) == i) ? cbk.c[i] : chi;
    }
    pair_s[tid] = make_float2(clo * s, chi * s);
    pair_s[kPairs + tid] = make_float2(-(clo * s), -(chi * s));
  }
  if (tid >= 128) sg_s[tid - 128] = signs[tid - 128];
  __syncthreads();

  uint32_t sm[4][8];                                           // sign bit of each element of this lane
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float4 a = *reinterpret_cast<const float4*>(&sg_s[32 * k + 8 * ls]);
    const float4 b = *reinterpret_cast<const float4*>(&sg_s[32 * k + 8 * ls + 4]);
    const float sv[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) sm[k][j] = __float_as_uint(sv[j]) & 0x80000000u;
  }
  const float m1 = (ls & 1) ? 1.0f : -1.0f, m2 = (ls & 2) ? 1.0f : -1.0f;
  const float2* my_pairs = pair_s + ((ls == 1 || ls == 2) ? kPairs : 0);
  uint32_t* words = words_s[wave];
  // words / shifts of the bits of chunk c = ls + 4k (elements 8c .. 8c+7)
  int cw[4], csl[4], csh[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) CK::pos(ls + 4 * k, cw[k], csl[k], csh[k]);

  const uint32_t batch0 = ((uint32_t)blockIdx.x * kWavesPerBlock + wave) * (uint32_t)passes;
  uint32_t row0 = batch0 * kEncVecs;
  uint32_t grp = row0 / (uint32_t)rm.rows_per_group;
  uint32_t rin = row0 - grp * (uint32_t)rm.rows_per_group;

  // the packed words and the norm of the next pass are fetched while the current one is computed
  uint32_t pw[kWordLoads];
  float pn = 0.0f;
  auto fetch = [&](uint32_t g_, uint32_t r_) {
    const uint32_t* prow = packed + ((int64_t)g_ * rm.packed_group_stride + r_) * kPd;
    pn = norms[(int64_t)g_ * rm.norms_group_stride + r_ + v];
#pragma unroll
    for (int it = 0; it < kWordLoads; ++it) {
      const int id = it * 64 + lane;
      pw[it] = (id < kEncVecs * kPd) ? prow[id] : 0u;
    }
  };
  if (row0 < (uint32_t)rm.n_rows) fetch(grp, rin);
  for (int pass = 0; pass < passes; ++pass) {
    if (row0 >= (uint32_t)rm.n_rows) break;                    // uniform over the wavefront
    const float nrm = pn;
#pragma unroll
    for (int it = 0; it < kWordLoads; ++it) {
      const int id = it * 64 + lane;
      if (id < kEncVecs * kPd) words[id] = pw[it];
    }
    uint32_t nrin = rin + kEncVecs, ngrp = grp;
    if (nrin >= (uint32_t)rm.rows_per_group) { nrin = 0; ++ngrp; }
    if (pass + 1 < passes && row0 + kEncVecs < (uint32_t)rm.n_rows) fetch(ngrp, nrin);
    float xs[4][8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t f = CK::field(words + v * kPd + cw[k], csl[k], csh[k]);
#pragma unroll
      for (int jp = 0; jp < 4; ++jp) {
        const float2 c2 = my_pairs[(f >> (2 * BITS * jp)) & CK::kPairMask];
        xs[k][2 * jp] = c2.x;
        xs[k][2 * jp + 1] = c2.y;
      }
    }
    butterfly_4lane_neg12(xs, m1, m2);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float r[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float t = (xs[k][j] * s) * nrm;
        asm volatile("" : "+v"(t));                            // keep the multiply out of the narrowing convert
        r[j] = t;
      }
      if (sizeof(TO) == 4) {
        uint4 a, b;
        a.x = __float_as_uint(r[0]) ^ sm[k][0]; a.y = __float_as_uint(r[1]) ^ sm[k][1];
        a.z = __float_as_uint(r[2]) ^ sm[k][2]; a.w = __float_as_uint(r[3]) ^ sm[k][3];
        b.x = __float_as_uint(r[4]) ^ sm[k][4]; b.y = __float_as_uint(r[5]) ^ sm[k][5];
        b.z = __float_as_uint(r[6]) ^ sm[k][6]; b.w = __float_as_uint(r[7]) ^ sm[k][7];
        *reinterpret_cast<uint4*>(&orow_s[wave][v * kPitch + 128 * k + 32 * ls]) = a;
        *reinterpret_cast<uint4*>(&orow_s[wave][v * kPitch + 128 * k + 32 * ls + 16]) = b;
      } else {
        uint32_t w[4];
#pragma unroll
        for (int jp = 0; jp < 4; ++jp) {
          uint32_t lo, hi;
          if (__is_same(TO, __half)) {
            lo = __half_as_ushort(__float2half_rn(r[2 * jp]));
            hi = __half_as_ushort(__float2half_rn(r[2 * jp + 1]));
          } else {
            lo = __bfloat16_as_ushort(__float2bfloat16(r[2 * jp]));
            hi = __bfloat16_as_ushort(__float2bfloat16(r[2 * jp + 1]));
          }
          w[jp] = (lo | (hi << 16)) ^ ((sm[k][2 * jp] >> 16) | sm[k][2 * jp + 1]);
        }
        *reinterpret_cast<uint4*>(&orow_s[wave][v * kPitch + 64 * k + 16 * ls]) = make_uint4(w[0], w[1], w[2], w[3]);
      }
    }
    {
      unsigned char* oblock = reinterpret_cast<unsigned char*>(out + ((int64_t)grp * rm.out_group_stride + rin) * 128);
      constexpr int kPiecesPerRow = 8 * (int)sizeof(TO);           // 16-byte pieces in a row: 16 or 32
#pragma unroll
      for (int i = 0; i < (int)(2 * sizeof(TO)); ++i) {            // 4 or 8 KB per pass
        const int piece = i * 64 + lane;
        // a streaming store (the "nt" hint): the rows are not read again by this kernel and a pass writes more than the
        // caches hold -- 115 -> 99 us per 1 M float32 rows, 75 -> 66 us for fp16
        typedef uint32_t piece_t __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(
            *reinterpret_cast<const piece_t*>(&orow_s[wave][(piece / kPiecesPerRow) * kPitch + (piece % kPiecesPerRow) * 16]),
            reinterpret_cast<piece_t*>(oblock + piece * 16));
      }
    }
    row0 += kEncVecs;
    rin = nrin;
    grp = ngrp;
  }
}

// ---------------------------------------------------------------- prerotate query
template <int D, typename T>
__global__ __launch_bounds__(kBlock) void prerotate_kernel(const T* __restrict__ q,
                                                           const float* __restrict__ signs,
                                                           float* __restrict__ q_rot, int64_t n_heads) {
  constexpr int EPL = Lay<D>::EPL;
  const int lane = threadIdx.x & (TQ_WAVE - 1);
  const int wave = threadIdx.x >> 6;
  const int64_t h = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  if (h >= n_heads) return;
  float v[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    int e = lane + 64 * i;
    v[i] = (e < D) ? load_as_float<T>(q + h * D + e) * signs[e] : 0.0f;
  }
  raw_butterfly<D>(v, lane);
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    int e = lane + 64 * i;
    if (e < D) q_rot[h * D + e] = v[i];
  }
}

// ---------------------------------------------------------------- per-row-butterfly QK scores (MHA)
template <int D, int BITS>
__global__ __launch_bounds__(kBlock) void packed_qk_kernel(const float* __restrict__ query,
                                                           const uint32_t* __restrict__ packed,
                                                           const float* __restrict__ norms, Codebook cbk,
                                                           const float* __restrict__ signs, float s,
                                                           float* __restrict__ scores, int64_t seq_len,
                                                           int64_t p_head_stride, int64_t n_head_stride) {
  constexpr int EPL = Lay<D>::EPL;
  constexpr int PDIM = Pk<BITS>::pdim(D);
  __shared__ float cb[16];
  if (threadIdx.x < 16) cb[threadIdx.x] = cbk.c[threadIdx.x];
  __syncthreads();
  const int lane = threadIdx.x & (TQ_WAVE - 1);
  const int wave = threadIdx.x >> 6;
  const int head = blockIdx.y;
  float sg[EPL], qv[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    int e = lane + 64 * i;
    sg[i] = (e < D) ? signs[e] : 0.0f;
    qv[i] = (e < D) ? query[(int64_t)head * D + e] : 0.0f;
  }
  const int64_t sweep = (int64_t)gridDim.x * kWavesPerBlock;
  for (int64_t pos = (int64_t)blockIdx.x * kWavesPerBlock + wave; pos < seq_len; pos += sweep) {
    const uint32_t* prow = packed + ((int64_t)head * p_head_stride + pos) * PDIM;
    const float nrm = norms[(int64_t)head * n_head_stride + pos];
    float v[EPL];
    load_centroid_values<D, BITS>(prow, cb, lane, s, v);
    raw_butterfly<D>(v, lane);
    float part[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) part[i] = (((v[i] * s) * sg[i]) * nrm) * qv[i];
    const float tot = tree_sum<D>(part);
    if (lane == 0) scores[(int64_t)head * seq_len + pos] = tot;
  }
}

// ---------------------------------------------------------------- host helpers

// order-preserving map float <-> uint32 for bisection over all finite floats
inline uint32_t f2ord(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
inline float ord2f(uint32_t o) {
  uint32_t u = (o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

// The pure-array quantiser compares z = fl(fl(w*s)/s) with each boundary b, w being the raw
// butterfly output and s = float32(1/sqrt(dim)).  z is a non-decreasing function of w, so
// {w : z(w) > b} = {w : w > t} with t the largest float whose z is <= b; t is found by
// bisection over the ordered floats.  Comparing w with t gives the same index for every w,
// NaN included (both comparisons are false), without the multiply and divide per element.
float double_rounding_threshold(float b, float s) {
  auto z_le_b = [&](float w) {
    volatile float y = w * s;
    volatile float z = y / s;
    return z <= b;
  };
  uint32_t lo = f2ord(-3.4028234663852886e38f), hi = f2ord(3.4028234663852886e38f);
  if (!z_le_b(ord2f(lo))) return -INFINITY;
  if (z_le_b(ord2f(hi))) return ord2f(hi);
  while (hi - lo > 1) {  // invariant: z(lo) <= b < z(hi)
    uint32_t mid = lo + (hi - lo) / 2;
    if (z_le_b(ord2f(mid))) lo = mid; else hi = mid;
  }
  return ord2f(lo);
}

// Finds alpha, beta with  j + 1/16 < alpha * t[j] + beta < j + 1 - 1/16  for every threshold j (and a
// further margin of 0.01), beta a multiple of 1/8.  The kernel evaluates v = fma(w, alpha, beta + 2^20 + 32)
// in float: one rounding, to a multiple of 1/8, i.e. at most 1/16 away from alpha*w + beta, so
// floor(v) - 2^20 - 32 is the count of thresholds below w or one less for every w.  |w| <= sqrt(128)
// (raw butterfly of a unit vector), so the guess must stay within +-32 of zero for the 64-entry table (three bits).
// False when no such line exists (then the generic kernel counts the thresholds one by one).
bool level_guess_search(const float* t, int nb, EncodeGuess& out);

// Widths other than three bits: any line u = alpha * t + beta0 (beta0 a multiple of 1/8) under which no cell
// [c, c + 1) of u holds two thresholds and every threshold keeps the margin above from both edges of its cell.
// The kernel's cell of w is floor(alpha * w + beta0) or, for w within 1/16 below a cell edge, the next one; with no
// threshold that close below an edge the count "thresholds below the cell + (w > the threshold inside it)" is the
// count of thresholds below w either way.  The candidate with the widest margin is taken.
bool level_cells_search(const float* t, int nb, EncodeGuess& out) {
  for (int i = 0; i < nb; ++i)
    if (!std::isfinite(t[i]) || (i > 0 && !(t[i] > t[i - 1]))) return false;
  const int half = nb == 15 ? 64 : 32;                              // the kernel's table has 2 * half cells
  const double margin = 1.0 / 16.0 + 0.01;
  double best = -1.0, best_b = 0.0;
  float best_a = 0.0f;
  for (int ai = 4000; ai >= 100; --ai) {
    const float af = (float)(ai * ((half - 1) / 11.4 / 4000.0));    // up to (half - 1) / 11.4 cells per unit of w
    const double a = (double)af;
    for (int bi = -64; bi <= 64; ++bi) {
      const double b = bi / 8.0;
      if (!(a * 11.4 + std::fabs(b) < half - 1.0)) continue;
      double slack = 1e9, prev_cell = -1e9;
      bool ok = true;
      for (int j = 0; j < nb && ok; ++j) {
        const double u = a * (double)t[j] + b;
        const double c = std::floor(u), f = u - c;
        if (f < margin || f > 1.0 - margin || c <= prev_cell) ok = false;
        prev_cell = c;
        slack = std::fmin(slack, std::fmin(f - margin, 1.0 - margin - f));
      }
      if (ok && slack > best) { best = slack; best_a = af; best_b = b; }
    }
    if (best > 0.15) break;                                         // good enough: finer cells gain nothing
  }
  if (best < 0.0) return false;
  out.alpha = best_a;
  out.beta0 = (float)best_b;
  out.beta = (float)(best_b + 1048576.0 + (double)half);            // exact: a multiple of 1/8 below 2^21
  return true;
}

// Search results are kept for the last few threshold sets seen (a process that alternates widths or threshold
// rules between calls -- caches of different bits, keys and values under different rules -- would otherwise repeat
// a search of several milliseconds at every switch).  The lock covers the table only, not the search: two threads
// that miss on the same set both search and store the same result.
bool level_guess(const float* t, int nb, EncodeGuess& out) {
  constexpr int kSlots = 8;
  struct Slot { float t[15]; int nb; bool ok; EncodeGuess g; };
  static std::mutex mu;
  static Slot slots[kSlots];
  static int n_used = 0, next = 0;
  {
    std::lock_guard<std::mutex> lock(mu);
    for (int i = 0; i < n_used; ++i)
      if (slots[i].nb == nb && memcmp(slots[i].t, t, nb * sizeof(float)) == 0) {
        out = slots[i].g;
        return slots[i].ok;
      }
  }
  Slot s{};
  s.nb = nb;
  memcpy(s.t, t, nb * sizeof(float));
  s.ok = (nb == 7) ? level_guess_search(t, nb, s.g) : level_cells_search(t, nb, s.g);
  {
    std::lock_guard<std::mutex> lock(mu);
    slots[next] = s;
    next = (next + 1) % kSlots;
    if (n_used < kSlots) ++n_used;
  }
  out = s.g;
  return s.ok;
}

bool level_guess_search(const float* t, int nb, EncodeGuess& out) {
  for (int i = 0; i < nb; ++i)
    if (!std::isfinite(t[i]) || (i > 0 && !(t[i] > t[i - 1]))) return false;
  const double span = (double)t[nb - 1] - (double)t[0];
  if (!(span > 0)) return false;
  double best_w = 0.0, best_a = 0.0, best_b = 0.0;
  for (int s = 1; s <= 4000; ++s) {
    const double a = (double)(nb + 1) * s / (1000.0 * span);       // up to 4x the mean level density
    double lo = -1e300, hi = 1e300;
    for (int j = 0; j < nb; ++j) {
      lo = std::fmax(lo, j - a * (double)t[j]);
      hi = std::fmin(hi, j + 1 - a * (double)t[j]);
    }
    if (hi - lo > best_w) { best_w = hi - lo; best_a = a; best_b = 0.5 * (lo + hi); }
  }
  if (best_w < 0.2) return false;
  out.alpha = (float)best_a;
  const double a = (double)out.alpha;
  double lo = -1e300, hi = 1e300;
  for (int j = 0; j < nb; ++j) {
    lo = std::fmax(lo, j - a * (double)t[j]);
    hi = std::fmin(hi, j + 1 - a * (double)t[j]);
  }
  const double b = std::floor(0.5 * (lo + hi) * 8.0 + 0.5) / 8.0;
  const double margin = 1.0 / 16.0 + 0.01;
  if (!(b - lo >= margin && hi - b >= margin)) return false;
  if (!(a * 11.4 + std::fabs(b) < 31.0)) return false;
  out.beta = (float)(b + 1048576.0 + 32.0);                  // exact: a multiple of 1/8 below 2^21
  out.beta0 = (float)b;
  return true;
}

// Passes per wavefront of the four-lanes-per-vector kernels: several, to spread the set-up cost,
// once every CU has a few workgroups anyway.
int fast_passes(int64_t n_rows) {
  const int64_t rows_per_block_pass = (int64_t)kEncVecs * kWavesPerBlock;
  return (n_rows >= rows_per_block_pass * kEncPasses * 256 * 4) ? kEncPasses : 1;
}

int grid_for_rows(int64_t rows) {
  int64_t blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
  const int64_t cap = 256 * 16;  // 16 blocks of 4 waves per CU keeps every SIMD supplied
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

}  // namespace

// Key and value rows of one decode step in one launch (d = 128, BITS bits, one wavefront per row): rows
// 0 .. n_rows - 1 are the keys (signs, destination 0), rows n_rows .. 2 n_rows - 1 the values.  Same
// arithmetic, operation for operation, as encode_kernel.
struct PairSide {
  const void* x;
  const float* signs;
  uint32_t* packed;
  float* norms;
  int dtype;
};

// With pos_dev set the destination row of group g is g * group_stride + *pos_dev (read when the kernel runs;
// nothing is stored when that position is outside 0 .. group_stride - 1).
template <int BITS>
__global__ __launch_bounds__(kBlock) void encode_pair_kernel(PairSide k, PairSide v, Thresholds thr, int64_t n_rows,
                                                             int64_t group_stride, const int64_t* pos_dev) {
  constexpr int D = 128, PDIM = BITS == 3 ? 13 : 4 * BITS, VPW = BITS == 3 ? 10 : 32 / BITS, NB = (1 << BITS) - 1;
  const int lane = threadIdx.x & (TQ_WAVE - 1);
  const int wave = threadIdx.x >> 6;
  const int64_t slot = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  if (slot >= 2 * n_rows) return;                          // no barriers below: a wavefront may leave alone
  const bool is_v = slot >= n_rows;
  const PairSide& s = is_v ? v : k;
  const int64_t row = is_v ? slot - n_rows : slot;
  float xv[2], sq[2], sg[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int64_t at = row * D + lane + 64 * i;
    xv[i] = s.dtype == TQ_F16 ? __half2float(((const __half*)s.x)[at])
          : s.dtype == TQ_F32 ? ((const float*)s.x)[at] : __bfloat162float(((const __hip_bfloat16*)s.x)[at]);
    sg[i] = s.signs[lane + 64 * i];
    sq[i] = xv[i] * xv[i];
  }
  const float ss = tree_sum<D>(sq);
  const float nrm = sqrtf(ss);
  const float safe = fmaxf(nrm, 1e-8f);
  float w[2] = {(xv[0] / safe) * sg[0], (xv[1] / safe) * sg[1]};
  raw_butterfly<D>(w, lane);
  int idx[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    uint32_t n = 0;
#pragma unroll
    for (int b = 0; b < NB; ++b) n += (w[i] > thr.t[b]) ? 1u : 0u;
    idx[i] = (int)n;
  }
  uint32_t word = 0;                                       // word `lane`: elements VPW * lane .. VPW * lane + VPW - 1
#pragma unroll
  for (int i = 0; i < VPW; ++i) {
    const int e = min(VPW * lane + i, D - 1);
    const int lo = __shfl(idx[0], e & 63), hi = __shfl(idx[1], e & 63);
    const uint32_t fld = (uint32_t)((e >> 6) ? hi : lo);
    if (VPW * lane + i < D) word |= fld << (BITS * i);
  }
  int64_t dst = row * group_stride;
  if (pos_dev) {
    const int64_t pos = *pos_dev;
    if (pos < 0 || pos >= group_stride) return;
    dst += pos;
  }
  if (lane < PDIM) s.packed[dst * PDIM + lane] = word;
  if (lane == 0) s.norms[dst] = nrm;
}

namespace tq {
int encode_pair(const void* k_new, int k_dtype, const float* k_signs, uint32_t* k_packed, float* k_norms,
                const void* v_new, int v_dtype, const float* v_signs, uint32_t* v_packed, float* v_norms,
                const float* boundaries, int bits, int64_t n_rows, int64_t group_stride, int variant, tq_stream_t stream_,
                const int64_t* pos_dev) {
  Thresholds thr;
  for (int i = 0; i < 15; ++i) thr.t[i] = INFINITY;
  encode_thresholds(boundaries, 128, bits, variant, thr.t);
  PairSide k{k_new, k_signs, k_packed, k_norms, k_dtype}, v{v_new, v_signs, v_packed, v_norms, v_dtype};
  const int grid = (int)((2 * n_rows + kWavesPerBlock - 1) / kWavesPerBlock);
  TQ_DISPATCH_BITS(bits, (encode_pair_kernel<B_><<<grid, kBlock, 0, (hipStream_t)stream_>>>(k, v, thr, n_rows, group_stride, pos_dev)));
  TQ_CHECK_LAUNCH("encode_pair launch");
  return TQ_OK;
}

void encode_thresholds(const float* boundaries, int dim, int bits, int variant, float* thr_out) {
  const float s = (float)(1.0 / sqrt((double)dim));
  const int nb = (1 << bits) - 1;
  for (int i = 0; i < nb; ++i)
    thr_out[i] = (variant == TQ_ENCODE_MLX) ? double_rounding_threshold(boundaries[i], s) : boundaries[i];
}
}  // namespace tq

// ------------------------------------------------------------------ C ABI

extern "C" int tq_version(void) { return TQ_VERSION; }

extern "C" const char* tq_last_error(void) { return tq::err_buf(); }

extern "C" const char* tq_status_string(int status) {
  switch (status) {
    case TQ_OK: return "ok";
    case TQ_ERR_NULL: return "null pointer";
    case TQ_ERR_DIM: return "bad dim";
    case TQ_ERR_BITS: return "bad bits";
    case TQ_ERR_NREP: return "bad n_rep";
    case TQ_ERR_ALIGN: return "misaligned pointer";
    case TQ_ERR_DTYPE: return "bad dtype";
    case TQ_ERR_BLOCK: return "bad block_size";
    case TQ_ERR_WORKSPACE: return "workspace too small";
    case TQ_ERR_ARG: return "bad argument";
    case TQ_ERR_UNSUPPORTED: return "unsupported";
  }
  return status <= TQ_ERR_HIP ? "hip error" : "unknown";
}

extern "C" int tq_encode(const void* x, int x_dtype, const float* signs, const float* boundaries,
                         uint32_t* packed, float* norms, int64_t n_groups, int64_t rows_per_group,
                         int64_t packed_group_stride, int64_t norms_group_stride, int dim, int bits,
                         int variant, tq_stream_t stream_) {
  if (int rc = tq::check_dim_bits(dim, bits)) return rc;
  if (tq::check_dtype(x_dtype)) return tq::fail(TQ_ERR_DTYPE, "tq_encode: unknown x_dtype %d", x_dtype);
  if (variant != TQ_ENCODE_MLX && variant != TQ_ENCODE_METAL)
    return tq::fail(TQ_ERR_ARG, "tq_encode: unknown variant %d", variant);
  if (n_groups < 0 || rows_per_group < 0) return tq::fail(TQ_ERR_ARG, "tq_encode: negative row count");
  const int64_t n_rows = n_groups * rows_per_group;
  if (n_rows == 0) return TQ_OK;
  if (!x || !signs || !boundaries || !packed || !norms) return tq::fail(TQ_ERR_NULL, "tq_encode: null pointer");
  if (!tq::aligned(x, tq::dtype_size(x_dtype)) || !tq::aligned(signs, 4) || !tq::aligned(packed, 4) ||
      !tq::aligned(norms, 4))
    return tq::fail(TQ_ERR_ALIGN, "tq_encode: misaligned pointer");
  const int nb = (1 << bits) - 1;
  Thresholds thr;
  const float s = (float)(1.0 / sqrt((double)dim));
  for (int i = 0; i < 15; ++i) thr.t[i] = INFINITY;
  for (int i = 0; i < nb; ++i)
    thr.t[i] = (variant == TQ_ENCODE_MLX) ? double_rounding_threshold(boundaries[i], s) : boundaries[i];
  RowMap rm{n_rows, rows_per_group, packed_group_stride, norms_group_stride, 0};
  hipStream_t stream = (hipStream_t)stream_;
  const int grid = grid_for_rows(n_rows);
  EncodeGuess gs{};
  if (dim == 128 && rows_per_group % kEncVecs == 0 && n_rows < (int64_t)1 << 31 &&
      tq::aligned(x, 16) && level_guess(thr.t, nb, gs)) {
    const int passes = fast_passes(n_rows);
    const int64_t rows_per_block = (int64_t)kEncVecs * passes * kWavesPerBlock;
    const int fgrid = (int)((n_rows + rows_per_block - 1) / rows_per_block);
#define LAUNCH_ENC128(T)                                                                                          \
    TQ_DISPATCH_BITS(bits, (encode128x3_kernel<T, B_><<<fgrid, kBlock, 0, stream>>>((const T*)x, signs, thr, gs, packed, \
                                                                                   norms, rm, passes)))
    if (x_dtype == TQ_F32) { LAUNCH_ENC128(float); }
    else if (x_dtype == TQ_F16) { LAUNCH_ENC128(__half); }
    else { LAUNCH_ENC128(__hip_bfloat16); }
#undef LAUNCH_ENC128
    TQ_CHECK_LAUNCH("tq_encode launch");
    return TQ_OK;
  }
#define LAUNCH_ENC(T)                                                                               \
  TQ_DISPATCH_DIM(dim, TQ_DISPATCH_BITS(bits, (encode_kernel<D_, B_, T><<<grid, kBlock, 0, stream>>>( \
                                                  (const T*)x, signs, thr, packed, norms, rm, RowCopy{}))))
  if (x_dtype == TQ_F32) { LAUNCH_ENC(float); }
  else if (x_dtype == TQ_F16) { LAUNCH_ENC(__half); }
  else { LAUNCH_ENC(__hip_bfloat16); }
#undef LAUNCH_ENC
  TQ_CHECK_LAUNCH("tq_encode launch");
  return TQ_OK;
}

namespace {
int vonly_append(const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                               const float* v_signs, const float* boundaries, void* k_f16, void* v_raw,
                               uint32_t* v_packed, float* v_norms, int64_t n_groups, int64_t rows_per_group,
                               int64_t k_group_stride, int64_t v_raw_group_stride, int64_t packed_group_stride,
                               int64_t norms_group_stride, int dim, int bits, int variant, const int64_t* pos_dev,
                               int64_t pos_cap, tq_stream_t stream_) {
  if (int rc = tq::check_dim_bits(dim, bits)) return rc;
  if (tq::check_dtype(k_dtype) || tq::check_dtype(v_dtype))
    return tq::fail(TQ_ERR_DTYPE, "tq_vonly_append: unknown dtype %d / %d", k_dtype, v_dtype);
  if (variant != TQ_ENCODE_MLX && variant != TQ_ENCODE_METAL)
    return tq::fail(TQ_ERR_ARG, "tq_vonly_append: unknown variant %d", variant);
  if (n_groups < 0 || rows_per_group < 0) return tq::fail(TQ_ERR_ARG, "tq_vonly_append: negative row count");
  const int64_t n_rows = n_groups * rows_per_group;
  if (n_rows == 0) return TQ_OK;
  if (!k_new || !v_new || !v_signs || !boundaries || !k_f16 || !v_packed || !v_norms)
    return tq::fail(TQ_ERR_NULL, "tq_vonly_append: null pointer");
  if (!tq::aligned(k_new, tq::dtype_size(k_dtype)) || !tq::aligned(v_new, tq::dtype_size(v_dtype)) ||
      !tq::aligned(v_signs, 4) || !tq::aligned(k_f16, 2) || !tq::aligned(v_packed, 4) || !tq::aligned(v_norms, 4) ||
      (v_raw && !tq::aligned(v_raw, tq::dtype_size(v_dtype))))
    return tq::fail(TQ_ERR_ALIGN, "tq_vonly_append: misaligned pointer");
  const int nb = (1 << bits) - 1;
  Thresholds thr;
  const float s = (float)(1.0 / sqrt((double)dim));
  for (int i = 0; i < 15; ++i) thr.t[i] = INFINITY;
  for (int i = 0; i < nb; ++i)
    thr.t[i] = (variant == TQ_ENCODE_MLX) ? double_rounding_threshold(boundaries[i], s) : boundaries[i];
  RowMap rm{n_rows, rows_per_group, packed_group_stride, norms_group_stride, 0};
  if (pos_dev && (!tq::aligned(pos_dev, 8) || pos_cap < 1))
    return tq::fail(TQ_ERR_ARG, "tq_vonly_append_at: position_dev must be 8-byte aligned and t_alloc >= 1");
  RowCopy rc{k_new, (__half*)k_f16, v_raw, k_group_stride, v_raw_group_stride, k_dtype, pos_dev, pos_cap};
  hipStream_t stream = (hipStream_t)stream_;
  const int grid = grid_for_rows(n_rows);
#define LAUNCH_APP(T)                                                                               \
  TQ_DISPATCH_DIM(dim, TQ_DISPATCH_BITS(bits, (encode_kernel<D_, B_, T><<<grid, kBlock, 0, stream>>>( \
                                                  (const T*)v_new, v_signs, thr, v_packed, v_norms, rm, rc))))
  if (v_dtype == TQ_F32) { LAUNCH_APP(float); }
  else if (v_dtype == TQ_F16) { LAUNCH_APP(__half); }
  else { LAUNCH_APP(__hip_bfloat16); }
#undef LAUNCH_APP
  TQ_CHECK_LAUNCH("tq_vonly_append launch");
  return TQ_OK;
}
}  // namespace

extern "C" int tq_vonly_append(const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                               const float* v_signs, const float* boundaries, void* k_f16, void* v_raw,
                               uint32_t* v_packed, float* v_norms, int64_t n_groups, int64_t rows_per_group,
                               int64_t k_group_stride, int64_t v_raw_group_stride, int64_t packed_group_stride,
                               int64_t norms_group_stride, int dim, int bits, int variant, tq_stream_t stream_) {
  return vonly_append(k_new, k_dtype, v_new, v_dtype, v_signs, boundaries, k_f16, v_raw, v_packed, v_norms, n_groups,
                      rows_per_group, k_group_stride, v_raw_group_stride, packed_group_stride, norms_group_stride, dim,
                      bits, variant, nullptr, 0, stream_);
}

extern "C" int tq_vonly_append_at(const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                                  const float* v_signs, const float* boundaries, void* k_f16, void* v_raw,
                                  uint32_t* v_packed, float* v_norms, int64_t n_groups, int64_t rows_per_group,
                                  int64_t t_alloc, int dim, int bits, int variant, const int64_t* position_dev,
                                  tq_stream_t stream_) {
  if (!position_dev) return tq::fail(TQ_ERR_NULL, "tq_vonly_append_at: null position_dev");
  if (rows_per_group > t_alloc)
    return tq::fail(TQ_ERR_ARG, "tq_vonly_append_at: %lld new rows per group do not fit %lld positions",
                    (long long)rows_per_group, (long long)t_alloc);
  return vonly_append(k_new, k_dtype, v_new, v_dtype, v_signs, boundaries, k_f16, v_raw, v_packed, v_norms, n_groups,
                      rows_per_group, t_alloc, t_alloc, t_alloc, t_alloc, dim, bits, variant, position_dev, t_alloc,
                      stream_);
}

extern "C" int tq_dequant(const uint32_t* packed, const float* norms, const float* centroids,
                          const float* signs, void* out, int out_dtype, int64_t n_groups,
                          int64_t rows_per_group, int64_t packed_group_stride, int64_t norms_group_stride,
                          int64_t out_group_stride, int dim, int bits, tq_stream_t stream_) {
  if (int rc = tq::check_dim_bits(dim, bits)) return rc;
  if (tq::check_dtype(out_dtype)) return tq::fail(TQ_ERR_DTYPE, "tq_dequant: unknown out_dtype %d", out_dtype);
  if (n_groups < 0 || rows_per_group < 0) return tq::fail(TQ_ERR_ARG, "tq_dequant: negative row count");
  const int64_t n_rows = n_groups * rows_per_group;
  if (n_rows == 0) return TQ_OK;
  if (!packed || !norms || !centroids || !signs || !out) return tq::fail(TQ_ERR_NULL, "tq_dequant: null pointer");
  if (!tq::aligned(packed, 4) || !tq::aligned(norms, 4) || !tq::aligned(signs, 4) ||
      !tq::aligned(out, tq::dtype_size(out_dtype)))
    return tq::fail(TQ_ERR_ALIGN, "tq_dequant: misaligned pointer");
  Codebook cb;
  for (int i = 0; i < 16; ++i) cb.c[i] = i < (1 << bits) ? centroids[i] : 0.0f;
  const float s = (float)(1.0 / sqrt((double)dim));
  RowMap rm{n_rows, rows_per_group, packed_group_stride, norms_group_stride, out_group_stride};
  hipStream_t stream = (hipStream_t)stream_;
  const int grid = grid_for_rows(n_rows);
  if (dim == 128 && rows_per_group % kEncVecs == 0 && n_rows < (int64_t)1 << 31 &&
      tq::aligned(out, 16) && (out_group_stride * 128 * (int64_t)tq::dtype_size(out_dtype)) % 16 == 0) {
    const int passes = fast_passes(n_rows);
    const int64_t rows_per_block = (int64_t)kEncVecs * passes * kWavesPerBlock;
    const int fgrid = (int)((n_rows + rows_per_block - 1) / rows_per_block);
#define LAUNCH_DEQ128(TO)                                                                                       \
    TQ_DISPATCH_BITS(bits, (dequant128x3_kernel<TO, B_><<<fgrid, kBlock, 0, stream>>>(packed, norms, cb, signs, s, \
                                                                                     (TO*)out, rm, passes)))
    if (out_dtype == TQ_F32) { LAUNCH_DEQ128(float); }
    else if (out_dtype == TQ_F16) { LAUNCH_DEQ128(__half); }
    else { LAUNCH_DEQ128(__hip_bfloat16); }
#undef LAUNCH_DEQ128
    TQ_CHECK_LAUNCH("tq_dequant launch");
    return TQ_OK;
  }
#define LAUNCH_DEQ(T)                                                                                 \
  TQ_DISPATCH_DIM(dim, TQ_DISPATCH_BITS(bits, (dequant_kernel<D_, B_, T><<<grid, kBlock, 0, stream>>>( \
                                                  packed, norms, cb, signs, s, (T*)out, rm))))
  if (out_dtype == TQ_F32) { LAUNCH_DEQ(float); }
  else if (out_dtype == TQ_F16) { LAUNCH_DEQ(__half); }
  else { LAUNCH_DEQ(__hip_bfloat16); }
#undef LAUNCH_DEQ
  TQ_CHECK_LAUNCH("tq_dequant launch");
  return TQ_OK;
}

extern "C" int tq_prerotate_query(const void* q, int q_dtype, const float* signs, float* q_rot,
                                  int64_t n_heads, int dim, tq_stream_t stream_) {
  if (!tq::is_pow2(dim)) return tq::fail(TQ_ERR_DIM, "dim must be a power of 2, got %d", dim);
  if (dim < 32 || dim > 256) return tq::fail(TQ_ERR_DIM, "dim %d outside the supported range 32..256", dim);
  if (tq::check_dtype(q_dtype)) return tq::fail(TQ_ERR_DTYPE, "tq_prerotate_query: unknown q_dtype %d", q_dtype);
  if (n_heads < 0) return tq::fail(TQ_ERR_ARG, "tq_prerotate_query: negative n_heads");
  if (n_heads == 0) return TQ_OK;
  if (!q || !signs || !q_rot) return tq::fail(TQ_ERR_NULL, "tq_prerotate_query: null pointer");
  hipStream_t stream = (hipStream_t)stream_;
  const int grid = (int)((n_heads + kWavesPerBlock - 1) / kWavesPerBlock);
#define LAUNCH_PRE(T) \
  TQ_DISPATCH_DIM(dim, (prerotate_kernel<D_, T><<<grid, kBlock, 0, stream>>>((const T*)q, signs, q_rot, n_heads)))
  if (q_dtype == TQ_F32) { LAUNCH_PRE(float); }
  else if (q_dtype == TQ_F16) { LAUNCH_PRE(__half); }
  else { LAUNCH_PRE(__hip_bfloat16); }
#undef LAUNCH_PRE
  TQ_CHECK_LAUNCH("tq_prerotate_query launch");
  return TQ_OK;
}

extern "C" int tq_packed_qk_scores(const float* query, const uint32_t* k_packed, const float* k_norms,
                                   const float* centroids, const float* signs, float* scores, int n_heads,
                                   int64_t seq_len, int64_t packed_head_stride, int64_t norms_head_stride,
                                   int dim, int bits, tq_stream_t stream_) {
  if (int rc = tq::check_dim_bits(dim, bits)) return rc;
  if (n_heads < 0 || seq_len < 0) return tq::fail(TQ_ERR_ARG, "tq_packed_qk_scores: negative size");
  if (n_heads == 0 || seq_len == 0) return TQ_OK;
  if (!query || !k_packed || !k_norms || !centroids || !signs || !scores)
    return tq::fail(TQ_ERR_NULL, "tq_packed_qk_scores: null pointer");
  Codebook cb;
  for (int i = 0; i < 16; ++i) cb.c[i] = i < (1 << bits) ? centroids[i] : 0.0f;
  const float s = (float)(1.0 / sqrt((double)dim));
  hipStream_t stream = (hipStream_t)stream_;
  dim3 grid(grid_for_rows(seq_len), n_heads);
  TQ_DISPATCH_DIM(dim, TQ_DISPATCH_BITS(bits, (packed_qk_kernel<D_, B_><<<grid, kBlock, 0, stream>>>(
                                                  query, k_packed, k_norms, cb, signs, s, scores, seq_len,
                                                  packed_head_stride, norms_head_stride))));
  TQ_CHECK_LAUNCH("tq_packed_qk_scores launch");
  return TQ_OK;
}
