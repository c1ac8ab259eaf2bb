// Shared host/device helpers for libtqhip (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <cmath>
#include <cstring>
#include <mutex>

#include "../../include/tqhip.h"

#define TQ_WAVE 64
#define TQ_VERSION 100

// ------------------------------------------------------------------ host side

namespace tq {

// thread-local message of the last failure
inline char* err_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}

inline int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(err_buf(), 512, fmt, ap);
  va_end(ap);
  return status;
}

inline int hip_fail(hipError_t e, const char* what) {
  return fail(TQ_ERR_HIP - (int)e, "%s: %s", what, hipGetErrorString(e));
}

inline int vals_per_word(int bits) {
  switch (bits) { case 1: return 32; case 2: return 16; case 3: return 10; case 4: return 8; }
  return 0;
}

inline int packed_dim(int dim, int bits) {
  int vpw = vals_per_word(bits);
  return (dim + vpw - 1) / vpw;
}

inline bool is_pow2(int d) { return d > 0 && (d & (d - 1)) == 0; }

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

inline int check_dtype(int dt) { return (dt == TQ_F32 || dt == TQ_F16 || dt == TQ_BF16) ? 0 : 1; }

// Decision thresholds of the encoder in the domain of the raw butterfly output for `nb` = 2^bits - 1
// boundaries (defined beside the encoder): TQ_ENCODE_MLX reproduces the comparison of
// fl(fl(w * s) / s) with the boundary, TQ_ENCODE_METAL compares w itself.
void encode_thresholds(const float* boundaries, int dim, int bits, int variant, float* thr_out);

// One new key row and one new value row per group (d = 128, `bits` bits) encoded by ONE launch: row g of either
// tensor goes to packed + g * group_stride rows and norms + g * group_stride (defined beside the
// encoder; the caller has validated pointers, dtypes and the width).
int encode_pair(const void* k_new, int k_dtype, const float* k_signs, uint32_t* k_packed, float* k_norms,
                const void* v_new, int v_dtype, const float* v_signs, uint32_t* v_packed, float* v_norms,
                const float* boundaries, int bits, int64_t n_rows, int64_t group_stride, int variant, tq_stream_t stream,
                const int64_t* pos_dev = nullptr);   // set: row g goes to g * group_stride + *pos_dev (device value)

inline size_t dtype_size(int dt) { return dt == TQ_F32 ? 4 : 2; }

inline int check_dim_bits(int dim, int bits) {
  if (bits < 1 || bits > 4) return fail(TQ_ERR_BITS, "Unsupported bit width: %d. Use 1-4.", bits);
  if (!is_pow2(dim)) return fail(TQ_ERR_DIM, "dim must be a power of 2, got %d", dim);
  if (dim < 32 || dim > 256) return fail(TQ_ERR_DIM, "dim %d outside the supported range 32..256", dim);
  return 0;
}

#define TQ_DISPATCH_DIM(dim, ...)                                  \
  switch (dim) {                                                   \
    case 32: { constexpr int D_ = 32; __VA_ARGS__; } break;        \
    case 64: { constexpr int D_ = 64; __VA_ARGS__; } break;        \
    case 128: { constexpr int D_ = 128; __VA_ARGS__; } break;      \
    case 256: { constexpr int D_ = 256; __VA_ARGS__; } break;      \
  }
#define TQ_DISPATCH_BITS(bits, ...)                                \
  switch (bits) {                                                  \
    case 1: { constexpr int B_ = 1; __VA_ARGS__; } break;          \
    case 2: { constexpr int B_ = 2; __VA_ARGS__; } break;          \
    case 3: { constexpr int B_ = 3; __VA_ARGS__; } break;          \
    case 4: { constexpr int B_ = 4; __VA_ARGS__; } break;          \
  }

#define TQ_CHECK_LAUNCH(what)                                   \
  do {                                                          \
    hipError_t e__ = hipGetLastError();                         \
    if (e__ != hipSuccess) return tq::hip_fail(e__, what);      \
  } while (0)

}  // namespace tq

// ------------------------------------------------------------------ device side

namespace tqd {

// centroid table passed to kernels by value
struct Codebook { float c[16]; };

template <int BITS> struct Pk {
  static constexpr int VPW = BITS == 1 ? 32 : BITS == 2 ? 16 : BITS == 3 ? 10 : 8;
  static constexpr uint32_t MASK = (1u << BITS) - 1u;
  static constexpr int pdim(int d) { return (d + VPW - 1) / VPW; }
};

// A 128-float (or shorter) vector is spread over one wavefront: lane l, slot i holds
// element l + 64*i.  EPL = slots per lane.
template <int D> struct Lay { static constexpr int EPL = (D >= 64) ? D / 64 : 1; };

__device__ __forceinline__ float shfl_xor_f(float v, int m) { return __shfl_xor(v, m, TQ_WAVE); }

// Value of lane (own ^ H): lanes 1 and 2 apart through a quad permute folded into the consuming
// instruction, 4 to 16 apart through ds_swizzle (no address register), 32 apart through a permute.
template <int H>
__device__ __forceinline__ float lane_xor(float v) {
  if constexpr (H == 1) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));
  } else if constexpr (H == 2) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));
  } else if constexpr (H <= 16) {
    return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (H << 10) | 0x1F));   // xor mask, and mask 31
  } else {
    return __shfl_xor(v, H, TQ_WAVE);
  }
}

// One lane-exchange stage: the element whose lane has bit H clear receives own + partner, the
// other partner - own (= partner + (-own): the same single rounding).
template <int H, int EPL>
__device__ __forceinline__ void butterfly_lane_stage(float (&v)[EPL], int lane) {
  const uint32_t flip = (lane & H) ? 0x80000000u : 0u;
#pragma unroll
  for (int i = 0; i < EPL; ++i) v[i] = lane_xor<H>(v[i]) + __uint_as_float(__float_as_uint(v[i]) ^ flip);
}

// Raw (un-normalised) Walsh-Hadamard butterfly, stages h = 1, 2, ..., D/2; the element whose
// index has bit h clear receives a+b, its partner a-b.  Stages below 64 exchange lanes, stages
// from 64 up are register-to-register.  Float adds only, so the result is the same expression
// tree as a serial loop over h.
template <int D>
__device__ __forceinline__ void raw_butterfly(float (&v)[Lay<D>::EPL], int lane) {
  constexpr int EPL = Lay<D>::EPL;
  if constexpr (D > 1) butterfly_lane_stage<1, EPL>(v, lane);
  if constexpr (D > 2) butterfly_lane_stage<2, EPL>(v, lane);
  if constexpr (D > 4) butterfly_lane_stage<4, EPL>(v, lane);
  if constexpr (D > 8) butterfly_lane_stage<8, EPL>(v, lane);
  if constexpr (D > 16) butterfly_lane_stage<16, EPL>(v, lane);
  if constexpr (D > 32) butterfly_lane_stage<32, EPL>(v, lane);
#pragma unroll
  for (int h = 64; h < D; h <<= 1) {
    const int hs = h / 64;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      if ((i & hs) == 0) {
        float a = v[i], b = v[i + hs];
        v[i] = a + b;
        v[i + hs] = a - b;
      }
    }
  }
}

// Sum over the D elements in stride-halving tree order: ns[e] += ns[e + stride] for
// stride = D/2, D/4, ..., 1.  Every lane ends with the value of ns[0].
template <int D>
__device__ __forceinline__ float tree_sum(float (&s)[Lay<D>::EPL]) {
  constexpr int EPL = Lay<D>::EPL;
#pragma unroll
  for (int hs = EPL / 2; hs >= 1; hs >>= 1) {
#pragma unroll
    for (int i = 0; i < hs; ++i) s[i] = s[i] + s[i + hs];
  }
  float v = s[0];
#pragma unroll
  for (int m = (D >= 64 ? 32 : D / 2); m >= 1; m >>= 1) v = v + shfl_xor_f(v, m);
  return v;
}

template <typename T> __device__ __forceinline__ float load_as_float(const T* p);
template <> __device__ __forceinline__ float load_as_float<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_as_float<__half>(const __half* p) { return __half2float(*p); }
template <> __device__ __forceinline__ float load_as_float<__hip_bfloat16>(const __hip_bfloat16* p) {
  return __bfloat162float(*p);
}

template <typename T> __device__ __forceinline__ void store_from_float(T* p, float v);
template <> __device__ __forceinline__ void store_from_float<float>(float* p, float v) { *p = v; }
// The value is rounded to float32 first and to the 16-bit type second, as a cast of a float
// variable does.  The empty asm keeps the compiler from folding the producing multiply into a
// mixed-precision multiply-convert, which would round only once.
template <> __device__ __forceinline__ void store_from_float<__half>(__half* p, float v) {
  asm volatile("" : "+v"(v));
  *p = __float2half_rn(v);
}
template <> __device__ __forceinline__ void store_from_float<__hip_bfloat16>(__hip_bfloat16* p, float v) {
  asm volatile("" : "+v"(v));
  *p = __float2bfloat16(v);
}

__device__ __forceinline__ float quad_xor1(float v) {
  return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));   // lanes 1,0,3,2
}
__device__ __forceinline__ float quad_xor2(float v) {
  return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));   // lanes 2,3,0,1
}

// Raw butterfly of a 128-vector spread over four lanes (element e = 32k + 8*ls + j in xs[k][j] of
// lane ls), stages in the order of strides 1, 2, ..., 64.  flip1 / flip2 are 0x80000000 in the
// lanes whose ls has bit 0 / bit 1 set (the upper element of a pair computes partner - own).
__device__ __forceinline__ void butterfly_4lane(float (&xs)[4][8], uint32_t flip1, uint32_t flip2) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (!(j & h)) {
          const float a = xs[k][j], b = xs[k][j + h];
          xs[k][j] = a + b;
          xs[k][j + h] = a - b;
        }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float a = xs[k][j];
      xs[k][j] = quad_xor1(a) + __uint_as_float(__float_as_uint(a) ^ flip1);
    }
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float a = xs[k][j];
      xs[k][j] = quad_xor2(a) + __uint_as_float(__float_as_uint(a) ^ flip2);
    }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float a0 = xs[0][j] + xs[1][j], a1 = xs[0][j] - xs[1][j];
    const float a2 = xs[2][j] + xs[3][j], a3 = xs[2][j] - xs[3][j];
    xs[0][j] = a0 + a2; xs[2][j] = a0 - a2;
    xs[1][j] = a1 + a3; xs[3][j] = a1 - a3;
  }
}

// butterfly_4lane for inputs that the lanes with ls = 1 and ls = 2 hold NEGATED -- a sign the caller folds into the
// sign flip or the table it applies to its inputs anyway.  Each of the two lane-exchange stages is then ONE fused
// multiply-add, own + partner * (+-1), instead of a sign flip and an add: with the value a of the lower lane and b
// of the upper lane of a pair, (own, partner, factor) = (a, -b, -1) gives a + b and (-b, a, +1) gives a - b; in the
// pairs whose results the next stage wants negated, (-a, b, -1) gives -(a + b) and (b, -a, +1) gives -(a - b).  A
// product with +-1 is exact, so every output is the same single rounding of the same sum as in butterfly_4lane:
// identical bits (the sign of a zero aside, which no consumer looks at).  m1 = (ls & 1) ? 1 : -1,
// m2 = (ls & 2) ? 1 : -1.  Outputs are not negated in any lane.
__device__ __forceinline__ void butterfly_4lane_neg12(float (&xs)[4][8], float m1, float m2) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (!(j & h)) {
          const float a = xs[k][j], b = xs[k][j + h];
          xs[k][j] = a + b;
          xs[k][j + h] = a - b;
        }
  }
  // v_fmac_f32 with the partner lane's value as its DPP operand, eight registers per statement (the compiler does
  // not form this instruction from a quad permute and a fused multiply-add: it leaves the permute a move of its
  // own).  A DPP read of a register that a vector instruction has just written needs two wait states, which the
  // compiler does not count across an asm statement: each statement starts with them.
#define TQ_FMAC8(PERM, M, R)                                                                                        \
  asm("s_nop 1\n\t"                                                                                                \
      "v_fmac_f32_dpp %0, %0, %8 quad_perm:" PERM " row_mask:0xf bank_mask:0xf\n\t"                                 \
      "v_fmac_f32_dpp %1, %1, %8 quad_perm:" PERM " row_mask:0xf bank_mask:0xf\n\t"                                 \
      "v_fmac_f32_dpp %2, %2, %8 quad_perm:" PERM " row_mask:0xf bank_mask:0xf\n\t"                                 \
      "v_fmac_f32_dpp %3, %3, %8 quad_perm:" PERM " row_mask:0xf bank_mask:0xf\n\t"                                 \
      "v_fmac_f32_dpp %4, %4, %8 quad_perm:" PERM " row_mask:0xf bank_mask:0xf\n\t"                                 \
      "v_fmac_f32_dpp %5, %5, %8 quad_perm:" PERM " row_mask:0xf bank_mask:0xf\n\t"                                 \
      "v_fmac_f32_dpp %6, %6, %8 quad_perm:" PERM " row_mask:0xf bank_mask:0xf\n\t"                                 \
      "v_fmac_f32_dpp %7, %7, %8 quad_perm:" PERM " row_mask:0xf bank_mask:0xf"                                      \
      : "+v"(R[0]), "+v"(R[1]), "+v"(R[2]), "+v"(R[3]), "+v"(R[4]), "+v"(R[5]), "+v"(R[6]), "+v"(R[7])              \
      : "v"(M))
#pragma unroll
  for (int k = 0; k < 4; ++k) TQ_FMAC8("[1,0,3,2]", m1, xs[k]);
#pragma unroll
  for (int k = 0; k < 4; ++k) TQ_FMAC8("[2,3,0,1]", m2, xs[k]);
#undef TQ_FMAC8
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float a0 = xs[0][j] + xs[1][j], a1 = xs[0][j] - xs[1][j];
    const float a2 = xs[2][j] + xs[3][j], a3 = xs[2][j] - xs[3][j];
    xs[0][j] = a0 + a2; xs[2][j] = a0 - a2;
    xs[1][j] = a1 + a3; xs[3][j] = a1 - a3;
  }
}

// Reductions over the four 16-lane rows of a wave (lanes l, l ^ 16, l ^ 32, l ^ 48), result in every lane: row
// swaps in the vector ALU (v_permlane16_swap: rows 1, 3 of the first operand change places with rows 0, 2 of the
// second; v_permlane32_swap: the upper half of the first with the lower half of the second) instead of two trips
// through the LDS permute path.  Both operands start as the value itself, so after a swap the two results hold the
// value of this lane's row and of its partner row in some order; max and + do not care which.
__device__ __forceinline__ float max_over_rows(float v) {
  typedef unsigned int u2_t __attribute__((ext_vector_type(2)));
  u2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_over_rows(float v) {
  typedef unsigned int u2_t __attribute__((ext_vector_type(2)));
  u2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, shfl_xor_f(v, m));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += shfl_xor_f(v, m);
  return v;
}

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
  __half2 h = __floats2half2_rn(a, b);
  return *reinterpret_cast<uint32_t*>(&h);
}

// Packed rows of one bit width (d = 128): words per row, and how a lane gets at the 8 * BITS bits that hold
// elements 8 pc .. 8 pc + 7 of a row.  Three-bit rows hold ten fields per word, so a piece may straddle two
// words; the other widths divide the word.
template <int BITS>
struct PackedField {
  static constexpr int kPd = BITS == 3 ? 13 : 4 * BITS;                  // words per packed row
  static constexpr uint32_t kEven = BITS == 3 ? 0x1C71C7u : BITS == 4 ? 0x0F0F0F0Fu : BITS == 2 ? 0x3333u : 0x55u;   // fields 0, 2, 4, 6
  static constexpr int kLut = 1 << (2 * BITS);                            // entries of the centroid-pair table
  __device__ static __forceinline__ void pos(int pc, int& w0, int& sh_lo, int& sh_hi) {
    if (BITS == 3) {
      w0 = (pc == 15) ? 11 : (8 * pc) / 10;                               // piece 15: word 11 >> 30 is 0, all of word 12
      const int s0 = (pc == 15) ? 10 : (8 * pc) % 10;
      sh_lo = 3 * s0;
      sh_hi = 30 - 3 * s0;
    } else {
      constexpr int kPerWord = 4 / BITS;                                  // pieces per word: 1, 2, 4 for 4, 2, 1 bits
      w0 = pc / kPerWord;
      sh_lo = (pc % kPerWord) * 8 * BITS;
      sh_hi = 0;
    }
  }
  __device__ static __forceinline__ uint32_t field(const uint32_t* at_w0, int sh_lo, int sh_hi) {
    if (BITS == 3) return ((at_w0[0] >> sh_lo) | (at_w0[1] << sh_hi)) & 0xFFFFFFu;
    if (BITS == 4) return at_w0[0];
    return (at_w0[0] >> sh_lo) & ((1u << (8 * BITS)) - 1u);
  }
  // even / odd fields of two rows interleaved into table indices at bit offsets 0, 2 BITS, 4 BITS, 6 BITS
  __device__ static __forceinline__ void interleave(uint32_t fa, uint32_t fb, uint32_t& X, uint32_t& Y) {
    X = (fa & kEven) | ((fb & kEven) << BITS);
    Y = ((fa >> BITS) & kEven) | (fb & (kEven << BITS));
  }
  __device__ static __forceinline__ uint32_t index(uint32_t src, int i) { return (src >> (2 * BITS * i)) & (uint32_t)(kLut - 1); }

  // bits of a packed row that start in word at_w0[0] at bit sh_lo, NOT cut to the 8 * BITS bits of the piece: for
  // consumers that mask every index they take out anyway
  __device__ static __forceinline__ uint32_t field_raw(const uint32_t* at_w0, int sh_lo, int sh_hi) {
    if (BITS == 3) return (at_w0[1] << sh_hi) | (at_w0[0] >> sh_lo);
    if (BITS == 4) return at_w0[0];
    return at_w0[0] >> sh_lo;
  }
  // interleave() on raw fields: bits of X / Y above 8 * BITS are garbage; four operations (two shifts, two selects
  // under the mask of the even fields)
  __device__ static __forceinline__ void interleave_raw(uint32_t fa, uint32_t fb, uint32_t& X, uint32_t& Y) {
    X = (fa & kEven) | ((fb << BITS) & ~kEven);
    Y = ((fa >> BITS) & kEven) | (fb & ~kEven);
  }

  // this lane's entries of a table of kLut centroid pairs half2(c[i & mask], c[i >> BITS]); selects, not a dynamic
  // index into kernel arguments
  __device__ static __forceinline__ void fill(uint32_t* lut, const Codebook& cb, int lane) {
#pragma unroll
    for (int base = 0; base < kLut; base += 64) {
      const int idx = base + lane;
      float clo = 0.0f, chi = 0.0f;
#pragma unroll
      for (int i = 0; i < (1 << BITS); ++i) {
        clo = ((idx & ((1 << BITS) - 1)) == i) ? cb.c[i] : clo;
        chi = ((idx >> BITS) == i) ? cb.c[i] : chi;
      }
      if (kLut >= 64 || idx < kLut) lut[idx] = pack_h2(clo, chi);
    }
  }

  // ---- centroid QUADS: one 8-byte look-up decodes four fields ----------------------------------------------------
  // Entry i of the quad table is {pair[i mod kLut], pair[i / kLut]}: the four centroids of four adjacent fields of a
  // source word (keys: four consecutive elements of a row; values: the same two elements of two rows, interleaved).
  // 16 / 256 / 4096 entries at 1 / 2 / 3 bits (32 KB at three bits, one table for keys and values when their
  // codebooks are equal); four bits would need 65536 entries and stay with pairs.  Per four fields: two vector
  // instructions (bit-field extract, shift) and one 8-byte LDS read, against four and two 4-byte reads with pairs.
  static constexpr bool kQuad = BITS <= 3;
  static constexpr int kQuadBits = 4 * BITS;
  static constexpr int kQuadEntries = kQuad ? (1 << kQuadBits) : 1;
  // built by the whole workgroup from the pair table (which must be visible: barrier before, barrier after)
  __device__ static __forceinline__ void fill_quad(uint2* qlut, const uint32_t* pair_lut, int tid, int n_threads) {
    for (int i = tid; i < kQuadEntries; i += n_threads)
      qlut[i] = make_uint2(pair_lut[i & (kLut - 1)], pair_lut[i >> (2 * BITS)]);
  }
  // Value side: four positions a, b, c, d interleaved so that the 4 * BITS bits of ONE element at the four positions
  // are adjacent (a lowest): from the raw fields of the four rows, Z[0] holds elements 0 and 4 (quads 0 and 1), Z[1]
  // elements 2 and 6, Z[2] elements 1 and 5, Z[3] elements 3 and 7.  Two levels of interleave_raw's shift-and-select:
  // 16 operations for 32 fields.  Bits above 8 * BITS are garbage.
  static constexpr uint32_t kEven2 = BITS == 3 ? 0x03F03Fu : BITS == 2 ? 0x0F0Fu : BITS == 1 ? 0x33u : 0x00FF00FFu;
  __device__ static __forceinline__ void interleave4_raw(uint32_t fa, uint32_t fb, uint32_t fc, uint32_t fd, uint32_t (&Z)[4]) {
    uint32_t Xab, Yab, Xcd, Ycd;
    interleave_raw(fa, fb, Xab, Yab);
    interleave_raw(fc, fd, Xcd, Ycd);
    Z[0] = (Xab & kEven2) | ((Xcd << (2 * BITS)) & ~kEven2);
    Z[1] = ((Xab >> (2 * BITS)) & kEven2) | (Xcd & ~kEven2);
    Z[2] = (Yab & kEven2) | ((Ycd << (2 * BITS)) & ~kEven2);
    Z[3] = ((Yab >> (2 * BITS)) & kEven2) | (Ycd & ~kEven2);
  }
  // element et (0 .. 7) of the piece: which Z word and which quad of it
  __device__ static constexpr int z_word(int et) { return ((et & 1) << 1) | ((et >> 1) & 1); }
  __device__ static constexpr int z_quad(int et) { return et >> 2; }
  __device__ static __forceinline__ uint2 quad_lookup(const uint2* qlut, uint32_t src, int j) {
    const uint32_t off = __builtin_amdgcn_ubfe(src, kQuadBits * j, kQuadBits) << 3;
    return *reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(qlut) + off);
  }
};

}  // namespace tqd

namespace tq {

// The matrix-core kernels hold the codebook as fp16.  Rounding the 2^bits levels to fp16 is a
// systematic error (the same few values at every position, so it does not average out over a
// sequence); multiplying the table by a scale a in [1, 2) first and dividing the result by a
// afterwards (in float32) leaves the mathematics alone, and a can be chosen so that every a*c[i]
// lies within a few 2^-16 of an fp16 value.  Returns 1/a; search results are kept for the last few
// tables seen.
inline float fill_codebook_fp16(tqd::Codebook& cb, const float* c, int bits) {
  constexpr int kSlots = 4;                                   // one per width in use
  struct Slot { float c[16]; int n; float scale; };
  static std::mutex mu;
  static Slot slots[kSlots];
  static int n_used = 0, next = 0;
  const int n = 1 << bits;
  float scale = 0.0f;
  {
    std::lock_guard<std::mutex> lock(mu);
    for (int i = 0; i < n_used; ++i)
      if (slots[i].n == n && std::memcmp(slots[i].c, c, n * sizeof(float)) == 0) scale = slots[i].scale;
  }
  if (scale == 0.0f) {                                        // the search runs outside the lock
    scale = 1.0f;
    double best = 1e30;
    for (int j = 0; j < 65536; ++j) {
      const float a = 1.0f + (float)j * (1.0f / 65536.0f);
      double worst = 0.0;
      for (int i = 0; i < n && worst < best; ++i) {
        const float v = a * c[i];
        if (v == 0.0f) continue;
        const float r = (float)(_Float16)v;
        worst = std::fmax(worst, std::fabs(((double)r - (double)v) / (double)v));
      }
      if (worst < best) { best = worst; scale = a; }
    }
    std::lock_guard<std::mutex> lock(mu);
    Slot& s = slots[next];
    std::memcpy(s.c, c, n * sizeof(float));
    s.n = n;
    s.scale = scale;
    next = (next + 1) % kSlots;
    if (n_used < kSlots) ++n_used;
  }
  for (int i = 0; i < 16; ++i) cb.c[i] = (i < n) ? scale * c[i] : 0.0f;
  return 1.0f / scale;
}

}  // namespace tq
