// Matrix-core tile pass at float32 fidelity for the two wrappers the reference names: pre-rotated scores over packed
// keys (tq_prerot_qk_scores) and the weighted value sum with given weights (tq_sparse_v_matvec), d = 128, 1 to 4 bits,
// n_rep <= 16.  Included by tq_attn.hip after tq_packed_mfma.h, whose layout it shares (a workgroup of 8 waves owns
// 512 positions of one kv head, a wave 64 of them).
//
// Every float32 operand enters as TWO fp16 numbers, its rounded value and the rounded remainder of that rounding
// (x = hi + lo to about 2^-22 |x|), and a product a * b is formed as hi_a hi_b + hi_a lo_b + lo_a hi_b: three
// v_mfma_f32_16x16x32_f16 per tile instead of one.  An fp16 x fp16 product has 22 significant bits and is exact in the
// float32 accumulator; what is dropped is lo_a lo_b, 2^-22 of the product.  So the result differs from a float32
// evaluation only by the order of the float32 additions: the reference's own bars for these two functions
// (1e-5 relative for the value sum, 1e-4 absolute for scores) hold with two orders of magnitude to spare, which the
// single-fp16 path (3e-4) does not meet.
//
//   centroids  scaled by 2^10 (exact) so that the remainders stay normal fp16 numbers; the pair table holds
//              {half2(hi, hi), half2(lo, lo)} per index: one 8-byte look-up per pair of elements;
//   queries    q_rot as hi / lo halves in LDS (as the fp16-operand pass already does);
//   weights    p = w * norm in float32 (the reference's order, (w * norm) * c), positions below the threshold
//              dropped, then scaled per wave by a power of two that puts the wave's largest p near 2^13 -- so that
//              weights many decades below the largest still have normal hi and lo parts -- and split.
#pragma once

#include "tq_packed_mfma.h"

namespace tqm {

constexpr float kSplitTableScale = 1024.0f;
constexpr float kSplitTableUnscale = 1.0f / 1024.0f;

// this lane's entries of the split pair table: entry i = {half2(hi[i & mask], hi[i >> BITS]), half2(lo[..], lo[..])}
template <int BITS>
__device__ __forceinline__ void fill_split_table(uint2* lut, const Codebook& cb, int lane) {
  using VF = VField<BITS>;
#pragma unroll
  for (int base = 0; base < VF::kLut; base += 64) {
    const int idx = base + lane;
    float c0 = 0.0f, c1 = 0.0f;
#pragma unroll
    for (int i = 0; i < (1 << BITS); ++i) {
      c0 = ((idx & ((1 << BITS) - 1)) == i) ? cb.c[i] : c0;
      c1 = ((idx >> BITS) == i) ? cb.c[i] : c1;
    }
    c0 *= kSplitTableScale;
    c1 *= kSplitTableScale;
    const __half h0 = __float2half_rn(c0), h1 = __float2half_rn(c1);
    const uint32_t hi = pack_h2(__half2float(h0), __half2float(h1));
    const uint32_t lo = pack_h2(c0 - __half2float(h0), c1 - __half2float(h1));
    if (VF::kLut >= 64 || idx < VF::kLut) lut[idx] = make_uint2(hi, lo);
  }
}

struct SplitArgs {
  const float* q_rot;         // scores: [n_q, 128] f32, pre-rotated
  const float* weights;       // values: [n_q, w_stride] f32
  int64_t w_stride;
  const uint32_t* packed;     // keys (scores) or values
  const float* norms;
  float* scores;              // scores: [n_q, seq_len] f32
  float* ws_S;                // values: partial sums [n_kv, n_tiles, n_rep, 128]
  float* ws_ml;               //         their (0, sum of weights) pairs
  int64_t seq_len;
  int64_t head_stride, norms_head_stride;   // rows / floats between kv heads
  int32_t n_kv, n_rep, n_tiles;
  float scale;                // scores: 1 / dim
  float threshold;            // values
};

// MODE = kScores or kWeights.  grid = (n_tiles, n_kv), 512 threads.
template <int MODE, int BITS>
__global__ __launch_bounds__(kMfmaThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
void split_tile_kernel(SplitArgs a, Codebook cb) {
  using VF = VField<BITS>;
  constexpr int kPd = VF::kPd;
  constexpr bool SCORES = MODE == kScores;
  __shared__ __align__(16) unsigned char big_s[32768];      // per-wave 4 KB areas, later the merge deposits
  __shared__ __align__(16) uint2 lut_s[VF::kLut < 64 ? 64 : VF::kLut];
  __shared__ __align__(16) uint32_t q_s[kHeadsMax][kD / 2];
  __shared__ __align__(16) uint32_t ql_s[kHeadsMax][kD / 2];
  __shared__ __align__(16) float n_s[kWaves][kWavePos];
  __shared__ __align__(16) MergeLds<kWaves> mg_s;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n16 = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x, kvh = blockIdx.y;
  const int n_rep = a.n_rep;
  const int64_t q_row0 = (int64_t)kvh * n_rep;
  const int64_t len = a.seq_len;
  const int64_t tile_p0 = (int64_t)tile * kTilePos;
  if (tile_p0 >= len) return;
  const int rows_here = (int)min((int64_t)kTilePos, len - tile_p0);
  const int last_row = rows_here - 1;
  const int wrow0 = wave * kWavePos;
  int crow = wrow0 + lane;
  crow = crow < last_row ? crow : last_row;

  // ---- loads ----------------------------------------------------------------------------------------------------
  float2 my_q[2];
  if (SCORES) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int w = tid + i * kMfmaThreads;
      my_q[i] = (w < n_rep * (kD / 2)) ? reinterpret_cast<const float2*>(a.q_rot + q_row0 * kD)[w] : make_float2(0.f, 0.f);
    }
  }
  const float my_n = a.norms[(int64_t)kvh * a.norms_head_stride + tile_p0 + crow];
  PackedBlockT<kPd> blk;
  load_block<MODE == kWeights>(blk, a.packed + ((int64_t)kvh * a.head_stride + tile_p0 + wrow0) * kPd, lane, wrow0, rows_here);
  // given weights: lane (head n16, group g) takes positions 16t + 4g + j
  float wgt[4][4];
  if (!SCORES) {
    const bool vec_ok = ((a.w_stride & 3) == 0) && ((reinterpret_cast<uintptr_t>(a.weights) & 15) == 0);   // uniform
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int row0 = wrow0 + 16 * t + 4 * g;
      const float* src = a.weights + (q_row0 + n16) * a.w_stride + tile_p0 + row0;
#pragma unroll
      for (int j = 0; j < 4; ++j) wgt[t][j] = 0.0f;
      if (n16 < n_rep) {
        if (vec_ok && row0 + 4 <= rows_here) {
          const f4 v = *reinterpret_cast<const f4*>(src);
          wgt[t][0] = v[0]; wgt[t][1] = v[1]; wgt[t][2] = v[2]; wgt[t][3] = v[3];
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (row0 + j < rows_here) wgt[t][j] = src[j];
        }
      }
    }
  }
  if (tid < 64) fill_split_table<BITS>(lut_s, cb, tid);
  if (SCORES) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const __half2 h = __floats2half2_rn(my_q[i].x, my_q[i].y);
      const float2 back = __half22float2(h);
      (&q_s[0][0])[tid + i * kMfmaThreads] = *reinterpret_cast<const uint32_t*>(&h);
      (&ql_s[0][0])[tid + i * kMfmaThreads] = pack_h2(my_q[i].x - back.x, my_q[i].y - back.y);
    }
  }
  n_s[wave][lane] = SCORES ? my_n * (a.scale * kSplitTableUnscale) : my_n;
  __syncthreads();

  uint32_t* stage = reinterpret_cast<uint32_t*>(big_s) + wave * 1024;
  stage_block(blk, stage, lane);

  if constexpr (SCORES) {
    // ---- scores: A = centroids of 16 positions x 32 elements (hi, lo), B = query columns (hi, lo)
    u4 qreg[4], qlow[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      qreg[kb] = *reinterpret_cast<const u4*>(&q_s[n16][(4 * kb + g) * 4]);
      qlow[kb] = *reinterpret_cast<const u4*>(&ql_s[n16][(4 * kb + g) * 4]);
    }
    int kw0[4], ksl[4], ksh[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) VF::pos(4 * kb + g, kw0[kb], ksl[kb], ksh[kb]);
    float s[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      f4 acc = {0.f, 0.f, 0.f, 0.f};
      const uint32_t* krow = stage + (16 * t + n16) * kPd;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const uint32_t f = VF::field_raw(krow + kw0[kb], ksl[kb], ksh[kb]);
        u4 kh, kl;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const uint2 e = lut_s[VF::index(f, k)];
          kh[k] = e.x;
          kl[k] = e.y;
        }
        // smallest terms first
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, kl), __builtin_bit_cast(h8, qreg[kb]), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, kh), __builtin_bit_cast(h8, qlow[kb]), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, kh), __builtin_bit_cast(h8, qreg[kb]), acc, 0, 0, 0);
      }
      const float4 kn4 = *reinterpret_cast<const float4*>(&n_s[wave][16 * t + 4 * g]);
      s[t][0] = acc[0] * kn4.x; s[t][1] = acc[1] * kn4.y; s[t][2] = acc[2] * kn4.z; s[t][3] = acc[3] * kn4.w;
    }
    // The wave's 64 x n_rep scores leave through its LDS area (the key image has been consumed): a store
    // instruction then writes whole 256-byte runs of a head's row.  Area = [16 heads][16 units of 4 positions],
    // the unit index xor-ed with the head (conflict-free 16-byte accesses both ways).
    f4* sc = reinterpret_cast<f4*>(stage);
#pragma unroll
    for (int t = 0; t < 4; ++t) sc[n16 * 16 + ((4 * t + g) ^ n16)] = f4{s[t][0], s[t][1], s[t][2], s[t][3]};
    const bool vec_ok = ((len & 3) == 0) && ((reinterpret_cast<uintptr_t>(a.scores) & 15) == 0);   // uniform
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int h = 4 * i + g, unit = n16;
      if (h < n_rep) {
        const f4 v = sc[h * 16 + (unit ^ h)];
        const int row0 = wrow0 + 4 * unit;
        float* dst = a.scores + (q_row0 + h) * len + tile_p0 + row0;
        if (vec_ok && row0 + 4 <= rows_here) {
          __builtin_nontemporal_store(v, reinterpret_cast<f4*>(dst));     // streaming store: 10.9 -> 10.3 us at 65 536 positions
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (row0 + j < rows_here) dst[j] = v[j];
        }
      }
    }
  } else {
    // ---- values: p = w * norm (weights below the threshold dropped), scaled per wave, split into hi and lo
    float p[4][4];
    float pmax = 0.0f, l = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float4 n4 = *reinterpret_cast<const float4*>(&n_s[wave][16 * t + 4 * g]);
      const float nv[4] = {n4.x, n4.y, n4.z, n4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float w = (wgt[t][j] < a.threshold) ? 0.0f : wgt[t][j];
        l += w;
        p[t][j] = w * nv[j];
        pmax = fmaxf(pmax, fabsf(p[t][j]));
      }
    }
    pmax = wave_max(pmax);
    // 2^e with pmax * 2^e in [2^13, 2^14); exponents clamped so that both 2^e and 2^-e are normal floats
    int ex = (int)((__float_as_uint(pmax) >> 23) & 0xFF);                 // biased exponent of pmax (0: pmax is 0 or denormal)
    ex = ex < 40 ? (ex < 1 ? 140 : 40) : (ex > 230 ? 230 : ex);
    const float up = __uint_as_float((uint32_t)(254 - ex + 13) << 23);   // 2^(127 - ex + 13)
    const float inv_tscale = __uint_as_float((uint32_t)(ex - 13) << 23); // its inverse
    uint32_t pa_hi[2][4], pa_lo[2][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      float hi[4], lo[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float ps = p[t][j] * up;
        hi[j] = __half2float(__float2half_rn(ps));
        lo[j] = ps - hi[j];
      }
      pa_hi[t >> 1][2 * (t & 1)] = pack_h2(hi[0], hi[1]);
      pa_hi[t >> 1][2 * (t & 1) + 1] = pack_h2(hi[2], hi[3]);
      pa_lo[t >> 1][2 * (t & 1)] = pack_h2(lo[0], lo[1]);
      pa_lo[t >> 1][2 * (t & 1) + 1] = pack_h2(lo[2], lo[3]);
    }
    l = sum_over_rows(l);

    int w0, sh_lo, sh_hi;
    VF::pos(n16, w0, sh_lo, sh_hi);
    f4 accS[8];
#pragma unroll
    for (int et = 0; et < 8; ++et) accS[et] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb2 = 0; kb2 < 2; ++kb2) {
      uint32_t VI[8];
      value_indices<BITS, false>(stage, kb2, g, w0, sh_lo, sh_hi, VI);
      const u4 Ah = {pa_hi[kb2][0], pa_hi[kb2][1], pa_hi[kb2][2], pa_hi[kb2][3]};
      const u4 Al = {pa_lo[kb2][0], pa_lo[kb2][1], pa_lo[kb2][2], pa_lo[kb2][3]};
#pragma unroll
      for (int et = 0; et < 8; ++et) {
        u4 Bh, Bl;
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          const uint2 e = lut_s[VF::index(VI[(et & 1) * 4 + qd], et >> 1)];
          Bh[qd] = e.x;
          Bl[qd] = e.y;
        }
        accS[et] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, Al), __builtin_bit_cast(h8, Bh), accS[et], 0, 0, 0);
        accS[et] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, Ah), __builtin_bit_cast(h8, Bl), accS[et], 0, 0, 0);
        accS[et] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, Ah), __builtin_bit_cast(h8, Bh), accS[et], 0, 0, 0);
      }
    }
    float* pS = a.ws_S + ((int64_t)kvh * a.n_tiles + tile) * (int64_t)(n_rep * kD);
    float* pml = a.ws_ml + ((int64_t)kvh * a.n_tiles + tile) * (int64_t)(n_rep * 2);
    merge_waves<kWaves>(mg_s, big_s, 4096, accS, 0.0f, l, inv_tscale, kSplitTableUnscale, n_rep, pS, pml);
  }
}

template <int BITS>
void launch_split_tiles(int mode, dim3 grid, const SplitArgs& a, const Codebook& cb, hipStream_t stream) {
  if (mode == kScores) split_tile_kernel<kScores, BITS><<<grid, kMfmaThreads, 0, stream>>>(a, cb);
  else split_tile_kernel<kWeights, BITS><<<grid, kMfmaThreads, 0, stream>>>(a, cb);
}
#ifndef TQ_WIDTH_HERE
extern template void launch_split_tiles<1>(int, dim3, const SplitArgs&, const Codebook&, hipStream_t);
extern template void launch_split_tiles<2>(int, dim3, const SplitArgs&, const Codebook&, hipStream_t);
extern template void launch_split_tiles<4>(int, dim3, const SplitArgs&, const Codebook&, hipStream_t);
#endif

}  // namespace tqm
