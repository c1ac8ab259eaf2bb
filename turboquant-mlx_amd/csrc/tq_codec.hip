// PolarQuant codec kernels for gfx950: fused encode, dequantise, query pre-rotation and the
// per-row-butterfly QK scoring.  One wavefront owns one vector; the Walsh-Hadamard butterfly
// and the norm reduction run on lane exchanges, never through LDS barriers.
#include "tq_common.h"

#include <math.h>
#include <string.h>

namespace {

using namespace tqd;

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * TQ_WAVE;

struct Thresholds { float t[15]; };

struct RowMap {
  int64_t n_rows, rows_per_group, packed_group_stride, norms_group_stride, out_group_stride;
};

// ---------------------------------------------------------------- encode
// Per vector: sum of squares in stride-halving tree order, sqrt, divide by max(n, 1e-8), sign
// flip, raw butterfly, count of thresholds exceeded (strict >), pack.  `thr` holds the decision
// thresholds in the domain of the raw butterfly output (see encode_thresholds below).
template <int D, int BITS, typename T>
__global__ __launch_bounds__(kBlock) void encode_kernel(const T* __restrict__ x,
                                                        const float* __restrict__ signs,
                                                        Thresholds thr, uint32_t* __restrict__ packed,
                                                        float* __restrict__ norms, RowMap rm) {
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
      const int64_t r = row - g * rm.rows_per_group;
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
    }
    __syncthreads();
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

int grid_for_rows(int64_t rows) {
  int64_t blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
  const int64_t cap = 256 * 16;  // 16 blocks of 4 waves per CU keeps every SIMD supplied
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

}  // namespace

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
#define LAUNCH_ENC(T)                                                                               \
  TQ_DISPATCH_DIM(dim, TQ_DISPATCH_BITS(bits, (encode_kernel<D_, B_, T><<<grid, kBlock, 0, stream>>>( \
                                                  (const T*)x, signs, thr, packed, norms, rm))))
  if (x_dtype == TQ_F32) { LAUNCH_ENC(float); }
  else if (x_dtype == TQ_F16) { LAUNCH_ENC(__half); }
  else { LAUNCH_ENC(__hip_bfloat16); }
#undef LAUNCH_ENC
  TQ_CHECK_LAUNCH("tq_encode launch");
  return TQ_OK;
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
