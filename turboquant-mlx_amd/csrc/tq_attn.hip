// Decode-attention kernels over packed PolarQuant K/V for gfx950, float32 vector-ALU path.
//
// KV positions are the parallel axis: a workgroup owns one tile of kTile positions of ONE kv
// head and serves all n_rep query heads of that kv head from a single read of the tile.  The
// V side accumulates sum_p w_p * norm_p * c[idx_p] in the rotated domain (no butterfly per
// position); partial sums (and the online-softmax statistics m, l) go to a workspace and a
// second pass merges the tiles, applies the ONE Walsh-Hadamard butterfly per output row, the
// signs and the 1/dim factor.
#include "tq_common.h"
#include "tq_decode_mfma.h"
#include "tq_packed_mfma.h"
#include "tq_split_mfma.h"

#include <math.h>
#include <cmath>
#include <cstring>
#include <mutex>

namespace {

using namespace tqd;

constexpr int kTile = 256;          // positions per workgroup, one per thread in the score phase
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / TQ_WAVE;
constexpr int kRMax = 8;            // query heads per kv head served by one workgroup

enum KMode { kWeights = 0, kPackedK = 1, kDenseK = 2 };

struct DecodeArgs {
  // query side
  const void* q;                // kPackedK: q_rot f32; kDenseK: q (dtype QT); kWeights: weights f32 [n_q, T]
  // key side
  const uint32_t* k_packed;
  const float* k_norms;
  const __half* k_dense;
  // value side
  const uint32_t* v_packed;
  const float* v_norms;
  const int32_t* seq_offsets;
  const float* mask;
  float* ws_S;                  // [n_seq*n_q, n_tiles_max, D]
  float* ws_ml;                 // [n_seq*n_q, n_tiles_max, 2]
  int64_t seq_len;
  int64_t k_seq_stride, k_head_stride, kn_seq_stride, kn_head_stride;
  int64_t v_seq_stride, v_head_stride, vn_seq_stride, vn_head_stride;
  int64_t mask_seq_stride, mask_head_stride;
  int32_t n_kv, n_rep, n_rgroups, n_tiles_max;
  float attn_scale, inv_dim, threshold;
};

__device__ __forceinline__ void seq_range(const int32_t* seq_offsets, int64_t seq_len, int seq,
                                          int64_t& first, int64_t& len) {
  if (seq_offsets) {
    first = seq_offsets[seq];
    len = (int64_t)seq_offsets[seq + 1] - first;
  } else {
    first = 0;
    len = seq_len;
  }
}

// ---- score of one position against up to kRMax query heads, fp16 keys: acc[r] = sum_e K[e] * q[r][e]
//      (q_s is [D][kRMax] in LDS)
template <int D>
__device__ __forceinline__ void score_dense(const __half* __restrict__ krow, const float (*q_s)[kRMax],
                                            float (&acc)[kRMax]) {
#pragma unroll
  for (int r = 0; r < kRMax; ++r) acc[r] = 0.0f;
#pragma unroll 1
  for (int e0 = 0; e0 < D; e0 += 8) {
    const uint4 raw = *reinterpret_cast<const uint4*>(krow + e0);
    const __half2* h2 = reinterpret_cast<const __half2*>(&raw);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float2 kf = __half22float2(h2[j]);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float kv = u ? kf.y : kf.x;
        const int e = e0 + 2 * j + u;
        const float4 qa = *reinterpret_cast<const float4*>(&q_s[e][0]);
        const float4 qb = *reinterpret_cast<const float4*>(&q_s[e][4]);
        acc[0] += kv * qa.x; acc[1] += kv * qa.y; acc[2] += kv * qa.z; acc[3] += kv * qa.w;
        acc[4] += kv * qb.x; acc[5] += kv * qb.y; acc[6] += kv * qb.z; acc[7] += kv * qb.w;
      }
    }
  }
}

template <typename QT, int D>
__device__ __forceinline__ void load_q_tile(const QT* __restrict__ q, int64_t q_row0, int n_local,
                                            float (*q_s)[kRMax]) {
  for (int i = threadIdx.x; i < D * kRMax; i += kThreads) {
    const int r = i / D, e = i % D;
    q_s[e][r] = (r < n_local) ? load_as_float<QT>(q + (q_row0 + r) * D + e) : 0.0f;
  }
}

// ---------------------------------------------------------------- stand-alone score kernels
// Packed rows of a wave's 64 consecutive positions, fetched with coalesced loads (instruction i reads words
// 64 i .. 64 i + 63 of the contiguous block) into LDS at an odd row pitch, so that every lane then reads its own
// row without bank conflicts.  Rows at or past rows_here are not fetched.
template <int PDIM>
__device__ __forceinline__ void stage_rows(const uint32_t* __restrict__ block, int rows_here, uint32_t* dst, int lane) {
  constexpr int PSTR = PDIM | 1;
  const int valid = rows_here * PDIM;
#pragma unroll
  for (int i = 0; i < PDIM; ++i) {
    const int idx = i * 64 + lane;
    if (idx < valid) {
      const int row = idx / PDIM;
      dst[row * PSTR + (idx - row * PDIM)] = block[idx];
    }
  }
}

// acc[u][r] = sum_e c[idx_e(row u)] * q[r][e] over NP packed rows in LDS (rows `pitch` words apart), element order
// e = 0, 1, ...: one fused multiply-add per (row, head, element).  The query rows are read at wave-uniform
// addresses, which the compiler turns into scalar loads: the vector ALU sees them as scalar-register operands and
// no LDS bandwidth goes into re-reading the query for every position; NP rows per lane share each of them.
// qrow[r] points at row min(r, n_local - 1).
template <int D, int BITS, int NP>
__device__ __forceinline__ void score_packed_uniform_q(const uint32_t* row, int pitch, const float* cb,
                                                       const float* const (&qrow)[kRMax], float (&acc)[NP][kRMax]) {
  constexpr int VPW = Pk<BITS>::VPW;
  constexpr int PDIM = Pk<BITS>::pdim(D);
#pragma unroll
  for (int u = 0; u < NP; ++u)
#pragma unroll
    for (int r = 0; r < kRMax; ++r) acc[u][r] = 0.0f;
  // Full words in a rolled loop (few live registers, so many waves per SIMD hide the scalar-load latency),
  // the last, partly filled word unrolled with its element count known at compile time.
  constexpr int FULL = D / VPW;
#pragma unroll 1
  for (int w = 0; w < FULL; ++w) {
    uint32_t word[NP];
#pragma unroll
    for (int u = 0; u < NP; ++u) word[u] = row[u * pitch + w];
#pragma unroll
    for (int i = 0; i < VPW; ++i) {
      float c[NP];
#pragma unroll
      for (int u = 0; u < NP; ++u) c[u] = cb[(word[u] >> (i * BITS)) & Pk<BITS>::MASK];
#pragma unroll
      for (int r = 0; r < kRMax; ++r) {
        const float qv = qrow[r][w * VPW + i];
#pragma unroll
        for (int u = 0; u < NP; ++u) acc[u][r] = __builtin_fmaf(c[u], qv, acc[u][r]);
      }
    }
  }
  if (FULL < PDIM) {
    uint32_t word[NP];
#pragma unroll
    for (int u = 0; u < NP; ++u) word[u] = row[u * pitch + FULL];
#pragma unroll
    for (int i = 0; i < D - FULL * VPW; ++i) {
      float c[NP];
#pragma unroll
      for (int u = 0; u < NP; ++u) c[u] = cb[(word[u] >> (i * BITS)) & Pk<BITS>::MASK];
#pragma unroll
      for (int r = 0; r < kRMax; ++r) {
        const float qv = qrow[r][FULL * VPW + i];
#pragma unroll
        for (int u = 0; u < NP; ++u) acc[u][r] = __builtin_fmaf(c[u], qv, acc[u][r]);
      }
    }
  }
}

// grid = (ceil(seq_len / kScoreTile), n_kv * n_rgroups): a wave takes 128 consecutive positions, a lane the
// positions lane and lane + 64 of them.
constexpr int kScoreNP = 1;
constexpr int kScoreTile = kThreads * kScoreNP;

template <int D, int BITS>
__global__ __launch_bounds__(kThreads) void prerot_scores_kernel(const float* __restrict__ q_rot,
                                                                 const uint32_t* __restrict__ k_packed,
                                                                 const float* __restrict__ k_norms,
                                                                 Codebook cbk, float* __restrict__ scores,
                                                                 int n_rep, int n_rgroups, int64_t seq_len,
                                                                 int64_t p_head_stride, int64_t n_head_stride,
                                                                 float inv_dim) {
  constexpr int PDIM = Pk<BITS>::pdim(D);
  constexpr int PSTR = PDIM | 1;
  __shared__ float cb[16];
  __shared__ uint32_t rows_s[kWaves][kScoreNP * 64 * PSTR];
  const int kvh = blockIdx.y / n_rgroups;
  const int r0 = (blockIdx.y % n_rgroups) * kRMax;
  const int n_local = min(kRMax, n_rep - r0);
  const int64_t q_row0 = (int64_t)kvh * n_rep + r0;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x < 16) cb[threadIdx.x] = cbk.c[threadIdx.x];
  const int64_t wp0 = (int64_t)blockIdx.x * kScoreTile + wave * (64 * kScoreNP);    // first position of this wave
  const int rows_here = (int)max((int64_t)0, min((int64_t)(64 * kScoreNP), seq_len - wp0));
#pragma unroll
  for (int u = 0; u < kScoreNP; ++u)
    stage_rows<PDIM>(k_packed + ((int64_t)kvh * p_head_stride + wp0 + 64 * u) * PDIM, rows_here - 64 * u,
                     rows_s[wave] + u * 64 * PSTR, lane);
  __syncthreads();
  if (lane >= rows_here) return;
  const float* qrow[kRMax];
#pragma unroll
  for (int r = 0; r < kRMax; ++r) qrow[r] = q_rot + (q_row0 + min(r, n_local - 1)) * D;
  float acc[kScoreNP][kRMax];
  score_packed_uniform_q<D, BITS, kScoreNP>(&rows_s[wave][lane * PSTR], 64 * PSTR, cb, qrow, acc);
#pragma unroll
  for (int u = 0; u < kScoreNP; ++u) {
    const int64_t p = wp0 + 64 * u + lane;
    if (p < seq_len) {
      const float nrm = k_norms[(int64_t)kvh * n_head_stride + p];
#pragma unroll
      for (int r = 0; r < kRMax; ++r)
        if (r < n_local) __builtin_nontemporal_store((acc[u][r] * nrm) * inv_dim, &scores[(q_row0 + r) * seq_len + p]);
    }
  }
}

template <int D, typename QT>
__global__ __launch_bounds__(kThreads) void dense_scores_kernel(const QT* __restrict__ q,
                                                                const __half* __restrict__ k,
                                                                float* __restrict__ scores, int n_rep,
                                                                int n_rgroups, int64_t seq_len,
                                                                int64_t k_head_stride, float scale) {
  __shared__ __align__(16) float q_s[D][kRMax];
  const int kvh = blockIdx.y / n_rgroups;
  const int r0 = (blockIdx.y % n_rgroups) * kRMax;
  const int n_local = min(kRMax, n_rep - r0);
  const int64_t q_row0 = (int64_t)kvh * n_rep + r0;
  load_q_tile<QT, D>(q, q_row0, n_local, q_s);
  __syncthreads();
  const int64_t p = (int64_t)blockIdx.x * kTile + threadIdx.x;
  if (p >= seq_len) return;
  float acc[kRMax];
  score_dense<D>(k + ((int64_t)kvh * k_head_stride + p) * D, q_s, acc);
#pragma unroll
  for (int r = 0; r < kRMax; ++r)
    if (r < n_local) scores[(q_row0 + r) * seq_len + p] = acc[r] * scale;
}

// ---------------------------------------------------------------- row softmax
// grid = (n_rows, n_chunks).  Every workgroup takes the maximum and the sum of exponentials over the WHOLE row in
// ONE sweep (online: a running maximum per thread, the sum rescaled when it moves) and then writes the weights of
// its own chunk, so a few long rows still fill the chip with one launch and without scratch memory.  With
// several chunks per row the row is read n_chunks times (from L2 for all but the first reader): the host keeps
// n_chunks at about one workgroup per CU, since that re-reading is what bounds the launch.  Logits are kept in
// log2 units (scale and mask times log2 e) so that e^x is one v_exp_f32.  16-byte accesses where the row is aligned.
constexpr int kSmThreads = 256;
constexpr int kSmWaves = kSmThreads / 64;

__global__ __launch_bounds__(kSmThreads) void softmax_rows_kernel(const float* __restrict__ scores,
                                                                const float* __restrict__ mask,
                                                                int64_t mask_row_stride,
                                                                float* __restrict__ weights, int64_t seq_len,
                                                                float scale, int64_t chunk_len) {
  __shared__ float red_m[kSmWaves], red_l[kSmWaves];
  constexpr float kLog2eF = 1.44269504088896340736f;
  const float scale2 = scale * kLog2eF;
  const int64_t row = blockIdx.x;
  const float* s = scores + row * seq_len;
  const float* mk = mask ? mask + row * mask_row_stride : nullptr;
  float* w = weights + row * seq_len;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool vec = ((seq_len & 3) == 0) && ((reinterpret_cast<uintptr_t>(scores) & 15) == 0) &&
                   ((reinterpret_cast<uintptr_t>(weights) & 15) == 0) && ((chunk_len & 3) == 0) &&
                   (!mask || (((reinterpret_cast<uintptr_t>(mask) & 15) == 0) && ((mask_row_stride & 3) == 0)));
  auto logits4 = [&](int64_t p, float (&v)[4]) {                      // four consecutive logits (vec only)
    const float4 x = *reinterpret_cast<const float4*>(s + p);
    v[0] = x.x * scale2; v[1] = x.y * scale2; v[2] = x.z * scale2; v[3] = x.w * scale2;
    if (mk) {
      const float4 m4 = *reinterpret_cast<const float4*>(mk + p);
      v[0] = __builtin_fmaf(m4.x, kLog2eF, v[0]); v[1] = __builtin_fmaf(m4.y, kLog2eF, v[1]);
      v[2] = __builtin_fmaf(m4.z, kLog2eF, v[2]); v[3] = __builtin_fmaf(m4.w, kLog2eF, v[3]);
    }
  };
  auto logit = [&](int64_t p) {
    float v = s[p] * scale2;
    if (mk) v = __builtin_fmaf(mk[p], kLog2eF, v);
    return v;
  };
  // ---- one sweep: per-thread running maximum m and sum l of 2^(x - m); kSweep 16-byte pieces per step, all
  // loads of a step issued before any is used
  constexpr int kSweep = 8;
  float m = -INFINITY, l = 0.0f;
  if (vec) {
    // the pieces of step i + 1 are requested before those of step i are reduced
    float4 nx[kSweep], nm[kSweep];
    auto fetch = [&](int64_t p) {
#pragma unroll
      for (int u = 0; u < kSweep; ++u) {
        const int64_t pu = p + (int64_t)u * 4 * kSmThreads;
        const bool ok = pu < seq_len;
        nx[u] = ok ? *reinterpret_cast<const float4*>(s + pu) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        if (mk) nm[u] = ok ? *reinterpret_cast<const float4*>(mk + pu) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    };
    const int64_t step = 4 * (int64_t)kSmThreads * kSweep;
    int64_t p = 4 * (int64_t)threadIdx.x;
    if (p < seq_len) fetch(p);
    for (; p < seq_len; p += step) {
      float v[kSweep][4];
#pragma unroll
      for (int u = 0; u < kSweep; ++u) {
        v[u][0] = nx[u].x * scale2; v[u][1] = nx[u].y * scale2; v[u][2] = nx[u].z * scale2; v[u][3] = nx[u].w * scale2;
        if (mk) {
          v[u][0] = __builtin_fmaf(nm[u].x, kLog2eF, v[u][0]); v[u][1] = __builtin_fmaf(nm[u].y, kLog2eF, v[u][1]);
          v[u][2] = __builtin_fmaf(nm[u].z, kLog2eF, v[u][2]); v[u][3] = __builtin_fmaf(nm[u].w, kLog2eF, v[u][3]);
        }
      }
      if (p + step < seq_len) fetch(p + step);
      float mb = m;
#pragma unroll
      for (int u = 0; u < kSweep; ++u) mb = fmaxf(mb, fmaxf(fmaxf(v[u][0], v[u][1]), fmaxf(v[u][2], v[u][3])));
      if (mb != -INFINITY) {
        float add = 0.0f;
#pragma unroll
        for (int u = 0; u < kSweep; ++u)
          add += (__builtin_amdgcn_exp2f(v[u][0] - mb) + __builtin_amdgcn_exp2f(v[u][1] - mb)) +
                 (__builtin_amdgcn_exp2f(v[u][2] - mb) + __builtin_amdgcn_exp2f(v[u][3] - mb));
        l = l * __builtin_amdgcn_exp2f(m - mb) + add;          // m = -inf: l is 0 and 2^-inf = 0
        m = mb;
      }
    }
  } else {
    for (int64_t p = threadIdx.x; p < seq_len; p += kSmThreads) {
      const float v = logit(p);
      const float mb = fmaxf(m, v);
      if (mb != -INFINITY) {
        l = l * __builtin_amdgcn_exp2f(m - mb) + __builtin_amdgcn_exp2f(v - mb);
        m = mb;
      }
    }
  }
  // ---- combine the threads: maximum first, then the sums rescaled to it
  float M = wave_max(m);
  if (lane == 0) red_m[wave] = M;
  __syncthreads();
  M = red_m[0];
#pragma unroll
  for (int i = 1; i < kSmWaves; ++i) M = fmaxf(M, red_m[i]);
  if (M == -INFINITY) M = 0.0f;                                  // a fully masked row: l = 0 and every weight is 0 * inf = NaN, as a softmax over nothing is
  l = (m == -INFINITY) ? 0.0f : l * __builtin_amdgcn_exp2f(m - M);
  l = wave_sum(l);
  if (lane == 0) red_l[wave] = l;
  __syncthreads();
  l = 0.0f;
#pragma unroll
  for (int i = 0; i < kSmWaves; ++i) l += red_l[i];
  const float inv_l = 1.0f / l;
  const int64_t p_lo = (int64_t)blockIdx.y * chunk_len;
  const int64_t p_hi = p_lo + chunk_len < seq_len ? p_lo + chunk_len : seq_len;
  if (vec) {
    constexpr int kWr = 4;                               // pieces per thread and step, loaded before any is used
    for (int64_t p = p_lo + 4 * (int64_t)threadIdx.x; p < p_hi; p += 4 * kSmThreads * kWr) {
      float v[kWr][4];
#pragma unroll
      for (int u = 0; u < kWr; ++u) {
        const int64_t pu = p + (int64_t)u * 4 * kSmThreads;
        if (pu < p_hi) logits4(pu, v[u]);
      }
#pragma unroll
      for (int u = 0; u < kWr; ++u) {
        const int64_t pu = p + (int64_t)u * 4 * kSmThreads;
        if (pu < p_hi)
          *reinterpret_cast<float4*>(w + pu) =
              make_float4(__builtin_amdgcn_exp2f(v[u][0] - M) * inv_l, __builtin_amdgcn_exp2f(v[u][1] - M) * inv_l,
                          __builtin_amdgcn_exp2f(v[u][2] - M) * inv_l, __builtin_amdgcn_exp2f(v[u][3] - M) * inv_l);
      }
    }
  } else {
    for (int64_t p = p_lo + threadIdx.x; p < p_hi; p += kSmThreads) w[p] = __builtin_amdgcn_exp2f(logit(p) - M) * inv_l;
  }
}

// ---------------------------------------------------------------- fused tile pass
// grid = (n_tiles_max, n_kv * n_rgroups, n_seq)
template <int D, int BITS, int KMODE, typename QT>
__global__ __launch_bounds__(kThreads) void decode_tile_kernel(DecodeArgs a, Codebook kcb, Codebook vcb) {
  constexpr int EPL = Lay<D>::EPL;
  constexpr int VPW = Pk<BITS>::VPW;
  constexpr int PDIM = Pk<BITS>::pdim(D);
  __shared__ float cbk_s[16], cbv_s[16];
  __shared__ __align__(16) float q_s[KMODE == kDenseK ? D : 1][kRMax];
  __shared__ uint32_t vrows_s[kWaves][66 * (PDIM | 1)];      // 64 rows + two that the pipelined loop reads ahead
  __shared__ float red_s[kWaves][kRMax];
  __shared__ float acc_s[kWaves][kRMax][D >= 64 ? D : 64];

  const int tile = blockIdx.x;
  const int kvh = blockIdx.y / a.n_rgroups;
  const int r0 = (blockIdx.y % a.n_rgroups) * kRMax;
  const int n_local = min(kRMax, a.n_rep - r0);
  const int seq = blockIdx.z;
  const int n_q = a.n_kv * a.n_rep;
  const int64_t q_row0 = (int64_t)seq * n_q + (int64_t)kvh * a.n_rep + r0;   // row in [n_seq*n_q]
  int64_t first, len;
  seq_range(a.seq_offsets, a.seq_len, seq, first, len);
  const int64_t p0 = (int64_t)tile * kTile;
  if (p0 >= len) return;     // tile past the end of this sequence: the merge pass never reads it
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  if (threadIdx.x < 16) {
    cbk_s[threadIdx.x] = kcb.c[threadIdx.x];
    cbv_s[threadIdx.x] = vcb.c[threadIdx.x];
  }
  if (KMODE == kDenseK) load_q_tile<QT, D>(reinterpret_cast<const QT*>(a.q), q_row0, n_local, q_s);
  const float* qrow[kRMax];                                // kPackedK: rows of the pre-rotated query, wave-uniform
  if (KMODE == kPackedK) {
#pragma unroll
    for (int r = 0; r < kRMax; ++r) qrow[r] = reinterpret_cast<const float*>(a.q) + (q_row0 + min(r, n_local - 1)) * D;
    // packed key rows of this wave's 64 positions (thread t of the workgroup owns position p0 + t)
    const int k_here = (int)max((int64_t)0, min((int64_t)TQ_WAVE, len - p0 - wave * TQ_WAVE));
    stage_rows<PDIM>(a.k_packed + ((int64_t)seq * a.k_seq_stride + (int64_t)kvh * a.k_head_stride + first + p0 +
                                  wave * TQ_WAVE) * PDIM, k_here, vrows_s[wave], lane);
  }
  __syncthreads();

  // ---- phase 1: one position per thread -> up to kRMax scores / weights
  const int64_t p = p0 + threadIdx.x;
  const bool live = p < len;
  float sc[kRMax];
  float pw[kRMax];                    // weight of this thread's position for each head (0 past the end)
  if (KMODE == kWeights) {
    const float* wts = reinterpret_cast<const float*>(a.q);
#pragma unroll
    for (int r = 0; r < kRMax; ++r) {
      float w = 0.0f;
      if (live && r < n_local) {
        w = wts[(q_row0 + r) * len + p];
        if (w < a.threshold) w = 0.0f;
      }
      pw[r] = w;
    }
  } else {
    if (live) {
      if (KMODE == kPackedK) {
        float acc1[1][kRMax];
        score_packed_uniform_q<D, BITS, 1>(&vrows_s[wave][lane * (PDIM | 1)], 0, cbk_s, qrow, acc1);
#pragma unroll
        for (int r = 0; r < kRMax; ++r) sc[r] = acc1[0][r];
        const float nrm = a.k_norms[(int64_t)seq * a.kn_seq_stride + (int64_t)kvh * a.kn_head_stride + first + p];
#pragma unroll
        for (int r = 0; r < kRMax; ++r) sc[r] = ((sc[r] * nrm) * a.inv_dim) * a.attn_scale;
      } else {
        const int64_t row = (int64_t)seq * a.k_seq_stride + (int64_t)kvh * a.k_head_stride + first + p;
        score_dense<D>(a.k_dense + row * D, q_s, sc);
#pragma unroll
        for (int r = 0; r < kRMax; ++r) sc[r] = sc[r] * a.attn_scale;
      }
      if (a.mask) {
#pragma unroll
        for (int r = 0; r < kRMax; ++r)
          if (r < n_local)
            sc[r] += a.mask[(int64_t)seq * a.mask_seq_stride +
                            ((int64_t)kvh * a.n_rep + r0 + r) * a.mask_head_stride + p];
      }
    } else {
#pragma unroll
      for (int r = 0; r < kRMax; ++r) sc[r] = -INFINITY;
    }
    // ---- phase 2: tile-local softmax statistics
    float mx[kRMax];
#pragma unroll
    for (int r = 0; r < kRMax; ++r) {
      float m = wave_max(sc[r]);
      if (lane == 0) red_s[wave][r] = m;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kRMax; ++r)
      mx[r] = fmaxf(fmaxf(red_s[0][r], red_s[1][r]), fmaxf(red_s[2][r], red_s[3][r]));
    __syncthreads();
    float ls[kRMax];
#pragma unroll
    for (int r = 0; r < kRMax; ++r) {
      const float e = (mx[r] == -INFINITY) ? 0.0f : expf(sc[r] - mx[r]);
      pw[r] = e;
      ls[r] = wave_sum(e);
      if (lane == 0) red_s[wave][r] = ls[r];
    }
    __syncthreads();
    if (threadIdx.x < kRMax && threadIdx.x < n_local) {
      const int r = threadIdx.x;
      const float l = (red_s[0][r] + red_s[1][r]) + (red_s[2][r] + red_s[3][r]);
      float* ml = a.ws_ml + ((q_row0 + r) * a.n_tiles_max + tile) * 2;
      ml[0] = mx[r];
      ml[1] = l;
    }
  }
  __syncthreads();

  // ---- phase 3: V accumulation in the rotated domain; wave w walks positions [64w, 64w+64).
  // The wave's packed rows come in with coalesced loads and are read back from LDS; the weight of position
  // 64w + j (held by lane j of this same wave) and its norm reach the arithmetic as scalar operands through
  // v_readlane, so the loop has no global load and no LDS read of weights.
  float acc[kRMax][EPL];
#pragma unroll
  for (int r = 0; r < kRMax; ++r)
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[r][i] = 0.0f;
  int widx[EPL], wsh[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + 64 * i;
    widx[i] = (e < D) ? e / VPW : 0;
    wsh[i] = (e % VPW) * BITS;
  }
  const int t_begin = wave * TQ_WAVE;
  const int n_here = (int)max((int64_t)0, min((int64_t)TQ_WAVE, len - p0 - t_begin));       // uniform over the wave
  const int64_t vrow0 = (int64_t)seq * a.v_seq_stride + (int64_t)kvh * a.v_head_stride + first + p0;
  const int64_t vnrow0 = (int64_t)seq * a.vn_seq_stride + (int64_t)kvh * a.vn_head_stride + first + p0;
  stage_rows<PDIM>(a.v_packed + (vrow0 + t_begin) * PDIM, n_here, vrows_s[wave], lane);
  const float my_nrm = (lane < n_here) ? a.v_norms[vnrow0 + t_begin + lane] : 0.0f;
  __builtin_amdgcn_wave_barrier();                      // the rows are read back by this wave only; LDS operations of a wave complete in order
  // The norm of a position rides on its weights (same lane): (w * norm) * centroid, the order of
  // sparse_v.py:64.  Software pipeline: the packed words of position j + 2 and the centroids of position j + 1
  // are fetched from LDS while the multiply-adds of position j run (rows 64 and 65 of the wave's area exist and
  // are never used).  Four positions per trip with a wave-uniform trip count: positions past n_here carry
  // weight 0 and whatever codes their rows hold select finite centroids.
#pragma unroll
  for (int r = 0; r < kRMax; ++r) pw[r] *= my_nrm;
  const uint32_t* vrows = vrows_s[wave];
  uint32_t wnext[EPL];
  float cnext[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) cnext[i] = cbv_s[(vrows[widx[i]] >> wsh[i]) & Pk<BITS>::MASK];
#pragma unroll
  for (int i = 0; i < EPL; ++i) wnext[i] = vrows[(PDIM | 1) + widx[i]];
  const int n_trips = __builtin_amdgcn_readfirstlane((n_here + 3) >> 2);
  for (int jj = 0; jj < n_trips; ++jj) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = 4 * jj + u;
      float cn[EPL];
#pragma unroll
      for (int i = 0; i < EPL; ++i) cn[i] = cnext[i];
#pragma unroll
      for (int i = 0; i < EPL; ++i) cnext[i] = cbv_s[(wnext[i] >> wsh[i]) & Pk<BITS>::MASK];
#pragma unroll
      for (int i = 0; i < EPL; ++i) wnext[i] = vrows[(u + 2) * (PDIM | 1) + widx[i]];
#pragma unroll
      for (int r = 0; r < kRMax; ++r) {
        const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, pw[r]), j));
#pragma unroll
        for (int i = 0; i < EPL; ++i) acc[r][i] = __builtin_fmaf(w, cn[i], acc[r][i]);
      }
    }
    vrows += 4 * (PDIM | 1);
  }
#pragma unroll
  for (int r = 0; r < kRMax; ++r)
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int e = lane + 64 * i;
      if (e < D) acc_s[wave][r][e] = acc[r][i];
    }
  __syncthreads();
  // ---- phase 4: merge the four waves, fixed order, and emit the tile partial
  for (int i = threadIdx.x; i < n_local * D; i += kThreads) {
    const int r = i / D, e = i % D;
    const float v = ((acc_s[0][r][e] + acc_s[1][r][e]) + acc_s[2][r][e]) + acc_s[3][r][e];
    a.ws_S[((q_row0 + r) * a.n_tiles_max + tile) * D + e] = v;
  }
}

// ---------------------------------------------------------------- merge pass
// grid = (n_q, n_seq), 256 threads.  Lane group ph = tid / (D/4) folds tiles ph, ph + P, ... (4
// elements per lane, P = 1024 / D groups) -- with a running maximum for the softmax modes, a plain
// sum for given weights -- the groups are combined through LDS in a fixed order and wave 0 applies
// the one butterfly, the signs, 1/dim (and 1/l).
template <int D, int KMODE, typename TO>
__global__ __launch_bounds__(kThreads) void decode_merge_kernel(const float* __restrict__ ws_S,
                                                                const float* __restrict__ ws_ml,
                                                                const int32_t* __restrict__ seq_offsets,
                                                                int64_t seq_len, int n_tiles_max,
                                                                const float* __restrict__ signs, float inv_dim,
                                                                TO* __restrict__ out) {
  constexpr int EPL = Lay<D>::EPL;
  constexpr int LPG = D / 4;                 // lanes per group
  constexpr int P = kThreads / LPG;          // groups
  typedef float f4 __attribute__((ext_vector_type(4)));
  __shared__ __align__(16) float acc_s[P][D];
  __shared__ float ml_s[P][2];
  const int tid = threadIdx.x, lane = tid & 63;
  const int eq = tid % LPG, ph = tid / LPG;
  const int64_t row = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
  int64_t first, len;
  seq_range(seq_offsets, seq_len, blockIdx.y, first, len);
  const int n_tiles = (int)((len + kTile - 1) / kTile);
  const float* S = ws_S + row * n_tiles_max * D + 4 * eq;
  const float* ml = ws_ml + row * n_tiles_max * 2;
  float M = -INFINITY, L = 0.0f;
  f4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int t0 = ph; t0 < n_tiles; t0 += 4 * P) {
    f4 x[4];
    float2 st[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int t = min(t0 + u * P, n_tiles - 1);
      x[u] = *reinterpret_cast<const f4*>(S + (int64_t)t * D);
      st[u] = (KMODE == kWeights) ? make_float2(0.f, 0.f) : *reinterpret_cast<const float2*>(ml + 2 * t);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (t0 + u * P >= n_tiles) continue;
      if (KMODE == kWeights) {
        acc += x[u];
      } else if (st[u].x != -INFINITY) {
        const float Mn = fmaxf(M, st[u].x);
        const float fo = (M == -INFINITY) ? 0.0f : expf(M - Mn);
        const float fc = expf(st[u].x - Mn);
        acc = acc * fo + x[u] * fc;
        L = L * fo + st[u].y * fc;
        M = Mn;
      }
    }
  }
  *reinterpret_cast<f4*>(&acc_s[ph][4 * eq]) = acc;
  if (eq == 0) { ml_s[ph][0] = M; ml_s[ph][1] = L; }
  __syncthreads();
  if (tid >= TQ_WAVE) return;
  float Mt = -INFINITY, Lt = 1.0f;
  float v[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) v[i] = 0.0f;
  if (KMODE != kWeights) {
    for (int p = 0; p < P; ++p) Mt = fmaxf(Mt, ml_s[p][0]);
    Lt = 0.0f;
  }
  for (int p = 0; p < P; ++p) {
    float f = 1.0f;
    if (KMODE != kWeights) {
      f = (ml_s[p][0] == -INFINITY) ? 0.0f : expf(ml_s[p][0] - Mt);
      Lt += f * ml_s[p][1];
    }
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int e = lane + 64 * i;
      if (e < D) v[i] += f * acc_s[p][e];
    }
  }
  raw_butterfly<D>(v, lane);
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + 64 * i;
    if (e < D) {
      float o = (v[i] * signs[e]) * inv_dim;
      if (KMODE != kWeights) o = (Lt > 0.0f) ? o / Lt : 0.0f;
      store_from_float<TO>(out + row * D + e, o);
    }
  }
}

// ---------------------------------------------------------------- host side

int n_tiles_for(int64_t len) { return (int)((len + kTile - 1) / kTile); }

size_t ws_bytes(int n_seq, int n_q, int64_t max_len, int dim) {
  const size_t tiles = (size_t)(n_tiles_for(max_len) > 0 ? n_tiles_for(max_len) : 1);
  return (size_t)n_seq * n_q * tiles * ((size_t)dim + 2) * sizeof(float);
}

void fill_codebook(Codebook& cb, const float* c, int bits) {
  for (int i = 0; i < 16; ++i) cb.c[i] = (c && i < (1 << bits)) ? c[i] : 0.0f;
}

int check_heads(int n_kv, int n_rep, const char* who) {
  if (n_kv < 1) return tq::fail(TQ_ERR_ARG, "%s: n_kv_heads must be >= 1, got %d", who, n_kv);
  if (n_rep < 1) return tq::fail(TQ_ERR_NREP, "%s: n_rep must be >= 1, got %d", who, n_rep);
  return 0;
}

template <int KMODE>
int launch_decode(const void* q, int q_dtype, const uint32_t* k_packed, const float* k_norms,
                  const void* k_dense, const uint32_t* v_packed, const float* v_norms,
                  const float* k_centroids, const float* v_centroids, const float* v_signs, void* out,
                  void* workspace, size_t workspace_bytes, const tq_decode_shape& sh, float threshold,
                  hipStream_t stream, const char* who, int phases = 3) {
  const int n_q = sh.n_kv_heads * sh.n_rep;
  const size_t need = ws_bytes(sh.n_seq, n_q, sh.seq_len, sh.dim);
  if (!workspace || workspace_bytes < need)
    return tq::fail(TQ_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
  if (!tq::aligned(workspace, 16)) return tq::fail(TQ_ERR_ALIGN, "%s: workspace must be 16-byte aligned", who);
  const int n_tiles = n_tiles_for(sh.seq_len);
  const int n_tiles_max = n_tiles > 0 ? n_tiles : 1;
  DecodeArgs a{};
  a.q = q;
  a.k_packed = k_packed; a.k_norms = k_norms; a.k_dense = (const __half*)k_dense;
  a.v_packed = v_packed; a.v_norms = v_norms;
  a.seq_offsets = sh.seq_offsets; a.mask = sh.mask;
  a.ws_S = (float*)workspace;
  a.ws_ml = a.ws_S + (size_t)sh.n_seq * n_q * n_tiles_max * sh.dim;
  a.seq_len = sh.seq_len;
  a.k_seq_stride = sh.k_seq_stride; a.k_head_stride = sh.k_head_stride;
  a.kn_seq_stride = sh.kn_seq_stride; a.kn_head_stride = sh.kn_head_stride;
  a.v_seq_stride = sh.v_seq_stride; a.v_head_stride = sh.v_head_stride;
  a.vn_seq_stride = sh.vn_seq_stride; a.vn_head_stride = sh.vn_head_stride;
  a.mask_seq_stride = sh.mask_seq_stride; a.mask_head_stride = sh.mask_head_stride;
  a.n_kv = sh.n_kv_heads; a.n_rep = sh.n_rep;
  a.n_rgroups = (sh.n_rep + kRMax - 1) / kRMax;
  a.n_tiles_max = n_tiles_max;
  a.attn_scale = sh.attn_scale;
  a.inv_dim = 1.0f / (float)sh.dim;
  a.threshold = threshold;
  Codebook kcb, vcb;
  fill_codebook(kcb, k_centroids, sh.bits);
  fill_codebook(vcb, v_centroids, sh.bits);
  if (n_tiles > 0 && (phases & 1)) {
    dim3 grid(n_tiles, sh.n_kv_heads * a.n_rgroups, sh.n_seq);
#define LAUNCH_TILE(QT)                                                                              \
  TQ_DISPATCH_DIM(sh.dim, TQ_DISPATCH_BITS(sh.bits, (decode_tile_kernel<D_, B_, KMODE, QT>            \
                                                        <<<grid, kThreads, 0, stream>>>(a, kcb, vcb))))
    if (KMODE == kDenseK && q_dtype == TQ_F16) { LAUNCH_TILE(__half); }
    else if (KMODE == kDenseK && q_dtype == TQ_BF16) { LAUNCH_TILE(__hip_bfloat16); }
    else { LAUNCH_TILE(float); }
#undef LAUNCH_TILE
    TQ_CHECK_LAUNCH(who);
  }
  if (!(phases & 2)) return TQ_OK;
  dim3 mgrid(n_q, sh.n_seq);
#define LAUNCH_MERGE(TO)                                                                              \
  TQ_DISPATCH_DIM(sh.dim, (decode_merge_kernel<D_, KMODE, TO><<<mgrid, kThreads, 0, stream>>>(         \
                              a.ws_S, a.ws_ml, sh.seq_offsets, sh.seq_len, n_tiles_max, v_signs,       \
                              a.inv_dim, (TO*)out)))
  if (sh.out_dtype == TQ_F16) { LAUNCH_MERGE(__half); }
  else if (sh.out_dtype == TQ_BF16) { LAUNCH_MERGE(__hip_bfloat16); }
  else { LAUNCH_MERGE(float); }
#undef LAUNCH_MERGE
  TQ_CHECK_LAUNCH(who);
  return TQ_OK;
}

// Matrix-core path: tile pass (partials of 512-position tiles) + merge pass.
int launch_vonly_mfma(const void* q, int q_dtype, const void* k_f16, const uint32_t* v_packed, const float* v_norms,
                      const float* v_centroids, const float* v_signs, void* out, void* workspace,
                      size_t workspace_bytes, const tq_decode_shape& sh, hipStream_t stream, int phases,
                      const int64_t* len_dev = nullptr, int64_t len_bias = 0, const tqm::FreshToken* fresh = nullptr) {
  const char* who = "tq_vonly_decode_attn";
  const int n_q = sh.n_kv_heads * sh.n_rep;
  // no mask, no ragged offsets, 16-byte aligned V rows of every tile: with full tiles on top, the PLAIN variants apply
  // (a length read on the device rules them out as well: sh.seq_len is then only its upper bound)
  const bool plain_any = !sh.mask && !sh.seq_offsets && sh.attn_scale > 0.0f && tq::aligned(v_packed, 16) &&
                         sh.v_seq_stride % 4 == 0 && sh.v_head_stride % 4 == 0;
  const bool plain_base = plain_any && !len_dev;
  const bool plain = plain_base && sh.seq_len % tqm::kTilePos == 0;
  // Long unmasked caches: several consecutive 512-position blocks per workgroup, as many as still leave
  // one workgroup per CU (256) and divide the length.
  int n_blocks = 1;
  const int64_t wgs8 = ((sh.seq_len + tqm::kTilePos - 1) / tqm::kTilePos) * sh.n_kv_heads * sh.n_seq;
  bool ragged_stream = false;
  if (plain) {
    for (int nb = (int)(wgs8 / 256 < 8 ? wgs8 / 256 : 8); nb > 1; --nb)
      if ((sh.seq_len / tqm::kTilePos) % nb == 0) { n_blocks = nb; break; }
    // A divisor may leave a short second round (36 blocks x 32 (sequence, kv head) pairs in fours: 288 workgroups, so
    // 32 CUs carry two): a count that does not divide the length takes the any-length form of the pass when it needs
    // fewer rounds of 256 workgroups times blocks (there: five blocks, 256 workgroups -- 46.2 -> 36 us).
    if (n_blocks > 1) {
      const int64_t blocks = sh.seq_len / tqm::kTilePos, groups = (int64_t)sh.n_kv_heads * sh.n_seq;
      auto cost = [&](int nb) { return ((((blocks + nb - 1) / nb) * groups + 255) / 256) * nb; };
      int64_t best = cost(n_blocks);
      for (int nb = 2; nb <= 8; ++nb)
        if (cost(nb) < best) { best = cost(nb); n_blocks = nb; ragged_stream = true; }
    }
  }
  const int64_t wgs4 = ((sh.seq_len + 255) / 256) * sh.n_kv_heads * sh.n_seq;
  if (n_blocks == 1 && plain_base && wgs4 > 768) {
    // Long caches of any length: the streaming pass with a ragged end.  Blocks per workgroup: the count that
    // minimises rounds of 256 workgroups times blocks per workgroup (ties: fewer blocks, more workgroups).
    const int64_t blocks = (sh.seq_len + tqm::kTilePos - 1) / tqm::kTilePos;
    int64_t best_cost = INT64_MAX;
    for (int nb = 2; nb <= 8; ++nb) {
      const int64_t wgs = ((blocks + nb - 1) / nb) * sh.n_kv_heads * sh.n_seq;
      const int64_t cost = ((wgs + 255) / 256) * nb;
      if (cost < best_cost) { best_cost = cost; n_blocks = nb; }
    }
    ragged_stream = true;
  }
  // Ragged batches (unmasked): the streaming pass as well, once the longest sequence alone would give every CU three
  // four-wave tiles.  True lengths are not known here, so at most 4 blocks per workgroup (a short tail), the count
  // with the fewest rounds for the longest sequence.  Three-bit rows start at any multiple of 4 bytes; rows of the
  // other widths are multiples of 16 bytes and need a 16-byte aligned tensor.
  const bool ragged_batch = sh.seq_offsets && !sh.mask && !len_dev && sh.attn_scale > 0.0f &&
                            (sh.bits == 3 || tq::aligned(v_packed, 16));
  if (ragged_batch && wgs4 > 768) {
    const int64_t blocks = (sh.seq_len + tqm::kTilePos - 1) / tqm::kTilePos;
    int64_t best_cost = INT64_MAX;
    for (int nb = 2; nb <= 4; ++nb) {
      const int64_t wgs = ((blocks + nb - 1) / nb) * sh.n_kv_heads * sh.n_seq;
      const int64_t cost = ((wgs + 255) / 256) * nb;
      if (cost <= best_cost) { best_cost = cost; n_blocks = nb; }         // ties: fewer workgroups, fewer set-ups
    }
    ragged_stream = true;
  }
  // One tile per workgroup, as measured over lengths from 4 096 to 65 537 (28/4 heads): eight-wave workgroups
  // (512 positions, one per CU) are the faster shape when they fill between half and all of the CUs in one round;
  // four-wave workgroups (256 positions, up to three per CU) fill more CUs on short caches and, from 257 to 768
  // of them, avoid the nearly empty second round of the eight-wave shape; beyond that the eight-wave shape again.
  int nw = 8;
  if (n_blocks == 1 && (wgs8 <= 128 || (wgs8 > 256 && wgs4 <= 768))) nw = 4;
  // Just above one full round of eight-wave workgroups (32 769 ... 49 152 positions at 28/4 heads) the four-wave shape pays
  // for a short last round: workgroups of ten or twelve waves (640 / 768 positions, three waves per SIMD, still one
  // workgroup per CU) cover such a cache in ONE round.  Any-length kernel only (unmasked, no offsets).
  if (n_blocks == 1 && plain_any && wgs8 > 256 && wgs4 <= 768) {
    for (int cand = 10; cand <= 12; cand += 2) {
      const int64_t tiles = (sh.seq_len + cand * tqm::kWavePos - 1) / (cand * tqm::kWavePos);
      if (tiles * sh.n_kv_heads * sh.n_seq <= 256) { nw = cand; break; }
    }
  }
  // The streaming pass in more than one round of eight-wave workgroups: four-wave workgroups over the same ranges
  // (twice the blocks of half the size), two to a CU, so that the set-up and the merge of one run under the steps of
  // the other.
  if (n_blocks > 1) {
    const int64_t blocks = (sh.seq_len + tqm::kTilePos - 1) / tqm::kTilePos;
    if (((blocks + n_blocks - 1) / n_blocks) * sh.n_kv_heads * sh.n_seq > 256) { nw = 4; n_blocks *= 2; }
  }
  const int tile_pos = nw * tqm::kWavePos * n_blocks;
  const int n_tiles_real = (int)((sh.seq_len + tile_pos - 1) / tile_pos);     // 0: an empty cache, merge pass only
  const int n_tiles = n_tiles_real > 0 ? n_tiles_real : 1;
  const size_t need = (size_t)sh.n_seq * n_q * n_tiles * (tqm::kD + 2) * sizeof(float);
  if (!workspace || workspace_bytes < need)
    return tq::fail(TQ_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
  if (!tq::aligned(workspace, 16)) return tq::fail(TQ_ERR_ALIGN, "%s: workspace must be 16-byte aligned", who);
  tqm::MfmaArgs a{};
  a.q = (const __half*)q; a.k = (const __half*)k_f16; a.q_bf16 = q_dtype == TQ_BF16 ? 1 : 0;
  const bool q_f32 = q_dtype == TQ_F32;
  a.v_packed = v_packed; a.v_norms = v_norms;
  a.seq_offsets = sh.seq_offsets; a.mask = sh.mask;
  a.len_dev = len_dev; a.len_bias = len_bias;
  a.ws_S = (float*)workspace;
  a.ws_ml = a.ws_S + (size_t)sh.n_seq * n_q * n_tiles * tqm::kD;
  a.seq_len = sh.seq_len;
  a.k_seq_stride = sh.k_seq_stride; a.k_head_stride = sh.k_head_stride;
  a.v_seq_stride = sh.v_seq_stride; a.v_head_stride = sh.v_head_stride;
  a.vn_seq_stride = sh.vn_seq_stride; a.vn_head_stride = sh.vn_head_stride;
  a.mask_seq_stride = sh.mask_seq_stride; a.mask_head_stride = sh.mask_head_stride;
  a.n_kv = sh.n_kv_heads; a.n_rep = sh.n_rep; a.n_tiles_max = n_tiles;
  a.attn_scale = sh.attn_scale;
  Codebook vcb;
  a.v_unscale = tq::fill_codebook_fp16(vcb, v_centroids, sh.bits);
  if ((phases & 1) && n_tiles_real > 0) {
    dim3 grid(n_tiles, sh.n_kv_heads, sh.n_seq);
    tqm::VonlyTileChoice ch{};
    ch.nw = nw; ch.n_blocks = n_blocks; ch.ragged_stream = ragged_stream; ch.plain = plain;
    ch.plain4 = plain_base && sh.seq_len % 256 == 0;                    // full 256-position tiles
    ch.plain_any = plain_any; ch.q_f32 = q_f32;
    switch (sh.bits) {
      case 1: tqm::launch_vonly_tiles<1>(grid, ch, a, vcb, stream); break;
      case 2: tqm::launch_vonly_tiles<2>(grid, ch, a, vcb, stream); break;
      case 4: tqm::launch_vonly_tiles<4>(grid, ch, a, vcb, stream); break;
      default: tqm::launch_vonly_tiles<3>(grid, ch, a, vcb, stream); break;
    }
    TQ_CHECK_LAUNCH(who);
  }
  if (!(phases & 2)) return TQ_OK;
  dim3 mgrid(n_q, sh.n_seq);
  const float inv_dim = 1.0f / (float)sh.dim;
#define LAUNCH_MERGE_U(TO, U_)                                                                            \
  tqm::decode_merge_rows_kernel<TO, true, U_><<<mgrid, tqm::kMergeThreads, 0, stream>>>(                    \
      a.ws_S, a.ws_ml, sh.seq_offsets, sh.seq_len, n_tiles, sh.n_kv_heads, sh.n_rep, v_signs, inv_dim, (TO*)out, tile_pos, \
      len_dev, len_bias)
  // tiles per lane group and round: one round of loads where 64, 128 or 256 tiles cover the sequence
#define LAUNCH_MERGE_M(TO)                                                                                \
  do {                                                                                                    \
    if (n_tiles <= 64) LAUNCH_MERGE_U(TO, 8);                                                             \
    else if (n_tiles <= 128) LAUNCH_MERGE_U(TO, 16);                                                      \
    else LAUNCH_MERGE_U(TO, 32);                                                                          \
  } while (0)
#define LAUNCH_FRESH_U(TO, U_)                                                                            \
  tqm::decode_merge_fresh_kernel<TO, U_><<<mgrid, tqm::kMergeThreads + 64, 0, stream>>>(                    \
      a.ws_S, a.ws_ml, sh.seq_len, n_tiles, sh.n_kv_heads, sh.n_rep, v_signs, inv_dim, (TO*)out, tile_pos, len_dev, *fresh)
#define LAUNCH_FRESH_M(TO)                                                                                \
  do {                                                                                                    \
    if (n_tiles <= 64) LAUNCH_FRESH_U(TO, 8);                                                             \
    else if (n_tiles <= 128) LAUNCH_FRESH_U(TO, 16);                                                      \
    else LAUNCH_FRESH_U(TO, 32);                                                                          \
  } while (0)
  if (fresh) {
    if (sh.out_dtype == TQ_F16) { LAUNCH_FRESH_M(__half); }
    else if (sh.out_dtype == TQ_BF16) { LAUNCH_FRESH_M(__hip_bfloat16); }
    else { LAUNCH_FRESH_M(float); }
  } else if (sh.out_dtype == TQ_F16) { LAUNCH_MERGE_M(__half); }
  else if (sh.out_dtype == TQ_BF16) { LAUNCH_MERGE_M(__hip_bfloat16); }
  else { LAUNCH_MERGE_M(float); }
#undef LAUNCH_FRESH_M
#undef LAUNCH_FRESH_U
#undef LAUNCH_MERGE_M
#undef LAUNCH_MERGE_U
  TQ_CHECK_LAUNCH(who);
  return TQ_OK;
}

// the width as a run-time value
void launch_packed_tiles_bits(int bits, int mode, int shape, dim3 grid, const tqm::PackedArgs& a, const Codebook& kcb,
                              const Codebook& vcb, hipStream_t stream) {
  switch (bits) {
    case 1: tqm::launch_packed_tiles<1>(mode, shape, grid, a, kcb, vcb, stream); break;
    case 2: tqm::launch_packed_tiles<2>(mode, shape, grid, a, kcb, vcb, stream); break;
    case 4: tqm::launch_packed_tiles<4>(mode, shape, grid, a, kcb, vcb, stream); break;
    default: tqm::launch_packed_tiles<3>(mode, shape, grid, a, kcb, vcb, stream); break;
  }
}


void launch_split_tiles_bits(int bits, int mode, dim3 grid, const tqm::SplitArgs& a, const Codebook& cb, hipStream_t stream) {
  switch (bits) {
    case 1: tqm::launch_split_tiles<1>(mode, grid, a, cb, stream); break;
    case 2: tqm::launch_split_tiles<2>(mode, grid, a, cb, stream); break;
    case 4: tqm::launch_split_tiles<4>(mode, grid, a, cb, stream); break;
    default: tqm::launch_split_tiles<3>(mode, grid, a, cb, stream); break;
  }
}

void launch_packed_stream_scores_bits(int bits, dim3 grid, const tqm::PackedArgs& a, const Codebook& kcb, int n_steps,
                                      hipStream_t stream) {
  switch (bits) {
    case 1: tqm::launch_packed_stream_scores<1>(grid, a, kcb, n_steps, stream); break;
    case 2: tqm::launch_packed_stream_scores<2>(grid, a, kcb, n_steps, stream); break;
    case 4: tqm::launch_packed_stream_scores<4>(grid, a, kcb, n_steps, stream); break;
    default: tqm::launch_packed_stream_scores<3>(grid, a, kcb, n_steps, stream); break;
  }
}

void launch_packed_stream_weights_bits(int bits, dim3 grid, const tqm::PackedArgs& a, const Codebook& vcb, int n_steps,
                                       hipStream_t stream) {
  switch (bits) {
    case 1: tqm::launch_packed_stream_weights<1>(grid, a, vcb, n_steps, stream); break;
    case 2: tqm::launch_packed_stream_weights<2>(grid, a, vcb, n_steps, stream); break;
    case 4: tqm::launch_packed_stream_weights<4>(grid, a, vcb, n_steps, stream); break;
    default: tqm::launch_packed_stream_weights<3>(grid, a, vcb, n_steps, stream); break;
  }
}

void launch_packed_stream_bits(int bits, dim3 grid, const tqm::PackedArgs& a, const Codebook& kcb, const Codebook& vcb,
                               int n_steps, hipStream_t stream) {
  switch (bits) {
    case 1: tqm::launch_packed_stream<1>(grid, a, kcb, vcb, n_steps, stream); break;
    case 2: tqm::launch_packed_stream<2>(grid, a, kcb, vcb, n_steps, stream); break;
    case 4: tqm::launch_packed_stream<4>(grid, a, kcb, vcb, n_steps, stream); break;
    default: tqm::launch_packed_stream<3>(grid, a, kcb, vcb, n_steps, stream); break;
  }
}


// Steps of 256 positions that one workgroup of the streaming flash pass runs through, or 0 for the
// single-tile pass (at most 512 steps in all).  A step of a wave that has its SIMD to itself (at most
// one four-wave workgroup per CU, 256 on this part) takes about 2.7 us, a step that shares it (up to two
// per CU) about 4.2 us, and with more workgroups than that the launch runs in rounds whose set-up overlaps.
// So: the smallest step count that brings the launch down to 256 workgroups, or the smallest that brings it
// down to 512, whichever costs less; at most 8 steps, and at most 4 for ragged batches (true lengths
// unknown on the host, max_seq_len is an upper bound), which keeps the tail of the launch short.  Measured,
// one sequence of 32 / 8 heads: 24 576 positions 16.7 us with 3 steps (256 workgroups) against 17.9 with 2
// (384) and 22.4 as single tiles; 18 432 positions 17.0 with 3 steps, 18.2 with 2, 22.0 as single tiles; 36 864
// positions 21.7 with 3 (384 workgroups), 26.5 with 2 (576), 22.3 with 5 (232).
int flash_stream_steps(int n_seq, int n_kv, int64_t max_seq_len, bool ragged) {
  const int64_t steps = (max_seq_len + tqm::kSStepPos - 1) / tqm::kSStepPos;
  const int64_t groups = (int64_t)n_seq * n_kv;
  if (groups * steps <= 512) return 0;            // up to 256 eight-wave tiles: the tile pass is as fast (14.7 against 14.9 us)
  const int cap = ragged ? 4 : 8;
  int alone = 0, shared = 0;                      // step counts that leave at most 256 / 512 workgroups
  for (int n = 2; n <= cap; ++n) {
    const int64_t wgs = groups * ((steps + n - 1) / n);
    if (!alone && wgs <= 256) alone = n;
    if (!shared && wgs <= 512) shared = n;
  }
  if (!shared) {
    // More than two workgroups per CU even at the cap: the launch runs in rounds of 512 workgroups.  A full round costs
    // the steps of a workgroup at the shared rate (4.2 us each) plus a set-up of about 5 us (the stamps of the kernel; a
    // sweep of the count over a ragged batch of 16 sequences: 116 / 117 / 108 / 108 us at 2 / 3 / 4 / 6 steps); a last round of at most 256
    // workgroups runs its steps at the rate of a wave that has its SIMD to itself.  The cheapest count, ties to the
    // larger.  16 sequences x 8 kv heads x 40 steps: five steps (1024 workgroups, two full rounds) instead of eight
    // (640: a second round that is a quarter full), 61 -> 54 us on one box.
    int best_n = cap;
    int64_t best = INT64_MAX;
    for (int n = 2; n <= cap; ++n) {
      const int64_t wgs = groups * ((steps + n - 1) / n);
      const int64_t rest = wgs % 512;
      const int64_t cost = (wgs / 512) * (42 * n + 50) + (rest == 0 ? 0 : (rest <= 256 ? 27 : 42) * n + 50);
      if (cost <= best) { best = cost; best_n = n; }
    }
    return best_n;
  }
  return (alone && alone * 27 <= shared * 42) ? alone : shared;
}

// Matrix-core path over packed keys/values: MODE = tqm::kFlash (tq_flash_decode) or tqm::kWeights
// (tq_sparse_v_matvec): tile pass + merge pass.
template <int MODE>
int launch_packed_mfma(const float* q_rot_or_weights, const uint32_t* k_packed, const float* k_norms,
                       const uint32_t* v_packed, const float* v_norms, const float* k_centroids,
                       const float* v_centroids, const float* v_signs, void* out, void* workspace,
                       size_t workspace_bytes, const tq_decode_shape& sh, float threshold, hipStream_t stream,
                       const char* who, const void* q_raw = nullptr, int q_dtype = TQ_F32,
                       const float* k_signs = nullptr, const int64_t* len_dev = nullptr, int64_t len_bias = 0,
                       const tqm::FreshToken* fresh = nullptr) {
  const int n_q = sh.n_kv_heads * sh.n_rep;
  const int n_tiles_real = (int)((sh.seq_len + tqm::kTilePos - 1) / tqm::kTilePos);   // 0: empty cache, merge pass only (fresh)
  const int n_tiles = n_tiles_real > 0 ? n_tiles_real : 1;
  const size_t need = (size_t)sh.n_seq * n_q * n_tiles * (tqm::kD + 2) * sizeof(float);
  if (!workspace || workspace_bytes < need)
    return tq::fail(TQ_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
  if (!tq::aligned(workspace, 16)) return tq::fail(TQ_ERR_ALIGN, "%s: workspace must be 16-byte aligned", who);
  tqm::PackedArgs a{};
  if (MODE == tqm::kWeights) a.weights = q_rot_or_weights; else a.q_rot = q_rot_or_weights;
  a.q_raw = q_raw; a.q_dtype = q_dtype; a.k_signs = k_signs;      // set: the kernel rotates the query itself
  a.k_packed = k_packed; a.k_norms = k_norms; a.v_packed = v_packed; a.v_norms = v_norms;
  a.seq_offsets = sh.seq_offsets; a.mask = sh.mask;
  a.ws_S = (float*)workspace;
  a.ws_ml = a.ws_S + (size_t)sh.n_seq * n_q * n_tiles * tqm::kD;
  a.seq_len = sh.seq_len;
  a.k_seq_stride = sh.k_seq_stride; a.k_head_stride = sh.k_head_stride;
  a.kn_seq_stride = sh.kn_seq_stride; a.kn_head_stride = sh.kn_head_stride;
  a.v_seq_stride = sh.v_seq_stride; a.v_head_stride = sh.v_head_stride;
  a.vn_seq_stride = sh.vn_seq_stride; a.vn_head_stride = sh.vn_head_stride;
  a.mask_seq_stride = sh.mask_seq_stride; a.mask_head_stride = sh.mask_head_stride;
  a.n_kv = sh.n_kv_heads; a.n_rep = sh.n_rep; a.n_tiles_max = n_tiles;
  a.score_scale = sh.attn_scale / (float)sh.dim;
  a.threshold = threshold;
  a.w_stride = sh.seq_len;                               // given weights: one sequence, rows of seq_len floats
  Codebook kcb, vcb;
  fill_codebook(kcb, nullptr, sh.bits);
  if (MODE != tqm::kWeights) a.score_scale *= tq::fill_codebook_fp16(kcb, k_centroids, sh.bits);
  a.v_unscale = tq::fill_codebook_fp16(vcb, v_centroids, sh.bits);
  int tile_pos = tqm::kTilePos;
  a.len_dev = len_dev; a.len_bias = len_bias;             // a length read on the device: an upper bound on the host, like a ragged batch
  // the streaming pass takes rows at any 4-byte offset at three bits only (the other widths: 16-byte aligned tensors)
  const bool stream_ok = MODE == tqm::kFlash && !sh.mask &&
                         (sh.bits == 3 || (tq::aligned(k_packed, 16) && tq::aligned(v_packed, 16)));
  const int n_steps = stream_ok ? flash_stream_steps(sh.n_seq, sh.n_kv_heads, sh.seq_len,
                                                     sh.seq_offsets != nullptr || len_dev != nullptr) : 0;
  if (n_steps >= 2) {
    tile_pos = tqm::kSStepPos * n_steps;
    a.n_tiles_max = (int)((sh.seq_len + tile_pos - 1) / tile_pos);
    dim3 grid(a.n_tiles_max, sh.n_kv_heads, sh.n_seq);
    launch_packed_stream_bits(sh.bits, grid, a, kcb, vcb, n_steps, stream);
  } else if (n_tiles_real > 0) {
    const int64_t wgs8 = (int64_t)n_tiles * sh.n_kv_heads * sh.n_seq;
    // Short caches (the eight-wave tiles fill at most half of the CUs): workgroups of FOUR waves over tiles of 256
    // positions, so that a wave has its SIMD to itself -- a tile's time is one wave's chain of key decode, softmax and
    // value decode, which a second wave on the SIMD stretches.  The partials of the finer tiles must fit the workspace.
    const int n_tiles4 = (int)((sh.seq_len + 4 * tqm::kWavePos - 1) / (4 * tqm::kWavePos));
    const size_t need4 = (size_t)sh.n_seq * n_q * n_tiles4 * (tqm::kD + 2) * sizeof(float);
    if (MODE == tqm::kFlash && wgs8 <= 128 && workspace_bytes >= need4) {
      tile_pos = 4 * tqm::kWavePos;
      a.n_tiles_max = n_tiles4;
      a.ws_ml = a.ws_S + (size_t)sh.n_seq * n_q * n_tiles4 * tqm::kD;
      dim3 grid(n_tiles4, sh.n_kv_heads, sh.n_seq);
      launch_packed_tiles_bits(sh.bits, MODE, tqm::kTilesFourWaves, grid, a, kcb, vcb, stream);
    } else {
      dim3 grid(n_tiles, sh.n_kv_heads, sh.n_seq);
      // at most one workgroup per CU: the flash variant without spills
      launch_packed_tiles_bits(sh.bits, MODE, wgs8 <= 256 ? tqm::kTilesOnePerCu : tqm::kTilesDefault, grid, a, kcb, vcb, stream);
    }
  }
  TQ_CHECK_LAUNCH(who);
  dim3 mgrid(n_q, sh.n_seq);
  const float inv_dim = 1.0f / (float)sh.dim;
  const int n_parts = a.n_tiles_max;
  if (fresh) {                                             // kFlash only: the merge pass inserts the token
#define LAUNCH_FRESH_P(TO, U_)                                                                                \
  tqm::decode_merge_fresh_kernel<TO, U_><<<mgrid, tqm::kMergeThreads + 64, 0, stream>>>(                        \
      a.ws_S, a.ws_ml, sh.seq_len, n_parts, sh.n_kv_heads, sh.n_rep, v_signs, inv_dim, (TO*)out, tile_pos, len_dev, *fresh)
#define LAUNCH_FRESH_PM(TO)                                                                                   \
  do {                                                                                                        \
    if (n_parts <= 64) LAUNCH_FRESH_P(TO, 8);                                                                 \
    else if (n_parts <= 128) LAUNCH_FRESH_P(TO, 16);                                                          \
    else LAUNCH_FRESH_P(TO, 32);                                                                              \
  } while (0)
    if (sh.out_dtype == TQ_F16) { LAUNCH_FRESH_PM(__half); }
    else if (sh.out_dtype == TQ_BF16) { LAUNCH_FRESH_PM(__hip_bfloat16); }
    else { LAUNCH_FRESH_PM(float); }
#undef LAUNCH_FRESH_PM
#undef LAUNCH_FRESH_P
    TQ_CHECK_LAUNCH(who);
    return TQ_OK;
  }
#define LAUNCH_MERGE_P(TO)                                                                                    \
  tqm::decode_merge_rows_kernel<TO, MODE == tqm::kFlash><<<mgrid, tqm::kMergeThreads, 0, stream>>>(            \
      a.ws_S, a.ws_ml, sh.seq_offsets, sh.seq_len, n_parts, sh.n_kv_heads, sh.n_rep, v_signs, inv_dim, (TO*)out, tile_pos, \
      len_dev, len_bias)
  if (sh.out_dtype == TQ_F16) { LAUNCH_MERGE_P(__half); }
  else if (sh.out_dtype == TQ_BF16) { LAUNCH_MERGE_P(__hip_bfloat16); }
  else { LAUNCH_MERGE_P(float); }
#undef LAUNCH_MERGE_P
  TQ_CHECK_LAUNCH(who);
  return TQ_OK;
}

// Second and third pass of the thresholded decode steps: weights 2^(s - M) / L from the scores and per-tile
// statistics, weights below the threshold dropped, value sums per tile; then the merge pass.
int launch_soft_weights(const float* scores, const float* stats, int stats_tile_pos, float* ws_S, float* ws_ml, int64_t t_pad, int n_tiles,
                        const uint32_t* v_packed, const float* v_norms, const float* v_centroids, const float* v_signs,
                        float threshold, void* out, const tq_decode_shape& sh, hipStream_t stream, const char* who) {
  const int n_q = sh.n_kv_heads * sh.n_rep;
  dim3 grid(n_tiles, sh.n_kv_heads, sh.n_seq);
  tqm::PackedArgs a{};
  a.weights = scores; a.stats = stats; a.w_stride = t_pad;
  a.stats_tile_pos = stats_tile_pos;
  a.n_stats_max = (int)((sh.seq_len + stats_tile_pos - 1) / stats_tile_pos);
  a.v_packed = v_packed; a.v_norms = v_norms;
  a.seq_offsets = sh.seq_offsets;
  a.ws_S = ws_S; a.ws_ml = ws_ml;
  a.seq_len = sh.seq_len;
  a.v_seq_stride = sh.v_seq_stride; a.v_head_stride = sh.v_head_stride;
  a.vn_seq_stride = sh.vn_seq_stride; a.vn_head_stride = sh.vn_head_stride;
  a.n_kv = sh.n_kv_heads; a.n_rep = sh.n_rep; a.n_tiles_max = n_tiles;
  a.threshold = threshold;
  Codebook kcb, vcb;
  fill_codebook(kcb, nullptr, sh.bits);
  a.v_unscale = tq::fill_codebook_fp16(vcb, v_centroids, sh.bits);
  // Large calls (more than 1024 steps of 256 positions in all: below that the tile pass is level or ahead, 35.0 against
  // 38.2 us for one sequence of 28 / 4 heads at 65 536 positions, while four sequences of 32 / 8 heads gain from 10 240
  // positions up, 181 -> 161 us at 65 536): the streaming form with the step rule of the dense flash step (a mask only
  // concerns the scores pass), one partial per workgroup range -- fewer than the tile pass would write, so they fit the
  // same workspace section.
  const int64_t steps_in_all = (int64_t)sh.n_seq * sh.n_kv_heads * ((sh.seq_len + tqm::kSStepPos - 1) / tqm::kSStepPos);
  const int n_steps = (steps_in_all > 1024 && (sh.bits == 3 || tq::aligned(v_packed, 16)))
                          ? flash_stream_steps(sh.n_seq, sh.n_kv_heads, sh.seq_len, sh.seq_offsets != nullptr) : 0;
  int tile_pos = tqm::kTilePos, n_parts = n_tiles;
  if (n_steps >= 2) {
    tile_pos = tqm::kSStepPos * n_steps;
    n_parts = (int)((sh.seq_len + tile_pos - 1) / tile_pos);
    a.n_tiles_max = n_parts;
    a.ws_ml = ws_ml = ws_S + (size_t)sh.n_seq * n_q * n_parts * tqm::kD;
    dim3 sgrid(n_parts, sh.n_kv_heads, sh.n_seq);
    launch_packed_stream_weights_bits(sh.bits, sgrid, a, vcb, n_steps, stream);
  } else {
    launch_packed_tiles_bits(sh.bits, tqm::kSoftWeights, tqm::kTilesDefault, grid, a, kcb, vcb, stream);
  }
  TQ_CHECK_LAUNCH(who);

  dim3 mgrid(n_q, sh.n_seq);
  const float inv_dim = 1.0f / (float)sh.dim;
  // partials per lane group and round: one round of loads where 64, 128 or 256 partials cover the sequence
#define LAUNCH_MERGE_SU(TO, U_)                                                                             \
  tqm::decode_merge_rows_kernel<TO, false, U_><<<mgrid, tqm::kMergeThreads, 0, stream>>>(                     \
      ws_S, ws_ml, sh.seq_offsets, sh.seq_len, n_parts, sh.n_kv_heads, sh.n_rep, v_signs, inv_dim, (TO*)out, tile_pos)
#define LAUNCH_MERGE_S(TO)                                                                                  \
  do {                                                                                                      \
    if (n_parts <= 64) LAUNCH_MERGE_SU(TO, 8);                                                              \
    else if (n_parts <= 128) LAUNCH_MERGE_SU(TO, 16);                                                       \
    else LAUNCH_MERGE_SU(TO, 32);                                                                           \
  } while (0)
  if (sh.out_dtype == TQ_F16) { LAUNCH_MERGE_S(__half); }
  else if (sh.out_dtype == TQ_BF16) { LAUNCH_MERGE_S(__hip_bfloat16); }
  else { LAUNCH_MERGE_S(float); }
#undef LAUNCH_MERGE_S
#undef LAUNCH_MERGE_SU
  TQ_CHECK_LAUNCH(who);
  return TQ_OK;
}

// Thresholded V-only decode on the matrix cores: scores pass (fp16 keys -> scores in log2 units + per-tile
// softmax statistics), weights pass (2^(s - M) / L, weights below the threshold dropped, value sums per tile),
// merge pass.  Workspace: scores | statistics | partial sums | their (0, l) pairs.
constexpr int kSparseStatsPos = 256;     // finest granularity of the per-tile statistics (scores pass of the fp16-key step)

size_t vonly_sparse_ws_bytes(int n_seq, int n_q, int64_t seq_len) {
  const int64_t t_pad = (seq_len + 3) & ~(int64_t)3;
  const int64_t n_tiles = (seq_len + tqm::kTilePos - 1) / tqm::kTilePos;
  const int64_t n_stats = (seq_len + kSparseStatsPos - 1) / kSparseStatsPos;
  // every section starts 16-byte aligned: the statistics are padded to a multiple of four floats
  return ((size_t)n_seq * n_q * t_pad + (((size_t)n_seq * n_q * n_stats * 2 + 3) & ~(size_t)3) +
          (size_t)n_seq * n_q * n_tiles * (tqm::kD + 2)) * sizeof(float);
}

int launch_vonly_sparse(const void* q, int q_dtype, const void* k_f16, const uint32_t* v_packed, const float* v_norms,
                        const float* v_centroids, const float* v_signs, float threshold, void* out, void* workspace,
                        size_t workspace_bytes, const tq_decode_shape& sh, hipStream_t stream) {
  const char* who = "tq_vonly_sparse_decode_attn";
  const int n_q = sh.n_kv_heads * sh.n_rep;
  const int64_t t_pad = (sh.seq_len + 3) & ~(int64_t)3;
  const int n_tiles = (int)((sh.seq_len + tqm::kTilePos - 1) / tqm::kTilePos);
  const size_t need = vonly_sparse_ws_bytes(sh.n_seq, n_q, sh.seq_len);
  if (!workspace || workspace_bytes < need)
    return tq::fail(TQ_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
  if (!tq::aligned(workspace, 16)) return tq::fail(TQ_ERR_ALIGN, "%s: workspace must be 16-byte aligned", who);
  const int n_stats = (int)((sh.seq_len + kSparseStatsPos - 1) / kSparseStatsPos);
  float* scores = (float*)workspace;                                    // [n_seq * n_q, t_pad]
  float* stats = scores + (size_t)sh.n_seq * n_q * t_pad;               // [n_seq * n_kv, n_stats, n_rep, 2]
  float* ws_S = stats + (((size_t)sh.n_seq * n_q * n_stats * 2 + 3) & ~(size_t)3);   // [n_seq * n_kv, n_tiles, n_rep, 128]
  float* ws_ml = ws_S + (size_t)sh.n_seq * n_q * n_tiles * tqm::kD;

  tqm::MfmaArgs m{};
  m.q = (const __half*)q; m.k = (const __half*)k_f16; m.q_bf16 = q_dtype == TQ_BF16 ? 1 : 0;
  m.seq_offsets = sh.seq_offsets; m.mask = sh.mask;
  m.ws_ml = stats; m.scores = scores; m.scores_stride = t_pad;
  m.seq_len = sh.seq_len;
  m.k_seq_stride = sh.k_seq_stride; m.k_head_stride = sh.k_head_stride;
  m.mask_seq_stride = sh.mask_seq_stride; m.mask_head_stride = sh.mask_head_stride;
  m.n_kv = sh.n_kv_heads; m.n_rep = sh.n_rep; m.n_tiles_max = n_stats;
  m.attn_scale = sh.attn_scale;
  // workgroups of four waves (256 positions), several per CU: the loads of one overlap the arithmetic and stores of another
  dim3 sgrid(n_stats, sh.n_kv_heads, sh.n_seq);
  if (q_dtype == TQ_F32) tqm::vonly_scores_kernel<true, 4><<<sgrid, 256, 0, stream>>>(m);
  else tqm::vonly_scores_kernel<false, 4><<<sgrid, 256, 0, stream>>>(m);
  TQ_CHECK_LAUNCH(who);

  return launch_soft_weights(scores, stats, kSparseStatsPos, ws_S, ws_ml, t_pad, n_tiles, v_packed, v_norms, v_centroids,
                             v_signs, threshold, out, sh, stream, who);
}

// The same over packed keys: scores pass = the packed-key score kernel with the attention scale, the mask and
// the per-tile statistics (tq_flash_sparse_decode).
int launch_flash_sparse(const float* q_rot, const uint32_t* k_packed, const float* k_norms, const uint32_t* v_packed,
                        const float* v_norms, const float* k_centroids, const float* v_centroids, const float* v_signs,
                        float threshold, void* out, void* workspace, size_t workspace_bytes, const tq_decode_shape& sh,
                        hipStream_t stream, const void* q_raw = nullptr, int q_dtype = TQ_F32,
                        const float* k_signs = nullptr) {
  const char* who = "tq_flash_sparse_decode";
  const int n_q = sh.n_kv_heads * sh.n_rep;
  const int64_t t_pad = (sh.seq_len + 3) & ~(int64_t)3;
  const int n_tiles = (int)((sh.seq_len + tqm::kTilePos - 1) / tqm::kTilePos);
  const size_t need = vonly_sparse_ws_bytes(sh.n_seq, n_q, sh.seq_len);
  if (!workspace || workspace_bytes < need)
    return tq::fail(TQ_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
  if (!tq::aligned(workspace, 16)) return tq::fail(TQ_ERR_ALIGN, "%s: workspace must be 16-byte aligned", who);
  float* scores = (float*)workspace;
  float* stats = scores + (size_t)sh.n_seq * n_q * t_pad;
  float* ws_S = stats + (((size_t)sh.n_seq * n_q * n_tiles * 2 + 3) & ~(size_t)3);
  float* ws_ml = ws_S + (size_t)sh.n_seq * n_q * n_tiles * tqm::kD;

  tqm::PackedArgs a{};
  a.q_rot = q_rot; a.k_packed = k_packed; a.k_norms = k_norms;
  a.q_raw = q_raw; a.q_dtype = q_dtype; a.k_signs = k_signs;
  a.seq_offsets = sh.seq_offsets; a.mask = sh.mask;
  a.scores = scores; a.stats_out = stats; a.w_stride = t_pad;
  a.seq_len = sh.seq_len;
  a.k_seq_stride = sh.k_seq_stride; a.k_head_stride = sh.k_head_stride;
  a.kn_seq_stride = sh.kn_seq_stride; a.kn_head_stride = sh.kn_head_stride;
  a.mask_seq_stride = sh.mask_seq_stride; a.mask_head_stride = sh.mask_head_stride;
  a.n_kv = sh.n_kv_heads; a.n_rep = sh.n_rep; a.n_tiles_max = n_tiles;
  Codebook kcb;
  a.score_scale = sh.attn_scale / (float)sh.dim * tq::fill_codebook_fp16(kcb, k_centroids, sh.bits);
  // Large unmasked calls: the scores pass in its streaming form (the rule of the dense step), one statistics entry per
  // workgroup range of n_steps * 256 positions -- at most as many entries as the tile pass would write.
  const bool stream_ok = !sh.mask && (sh.bits == 3 || tq::aligned(k_packed, 16));
  const int n_steps = stream_ok ? flash_stream_steps(sh.n_seq, sh.n_kv_heads, sh.seq_len, sh.seq_offsets != nullptr) : 0;
  int stats_pos = tqm::kTilePos;
  if (n_steps >= 2) {
    stats_pos = tqm::kSStepPos * n_steps;
    a.n_tiles_max = (int)((sh.seq_len + stats_pos - 1) / stats_pos);
    dim3 grid(a.n_tiles_max, sh.n_kv_heads, sh.n_seq);
    launch_packed_stream_scores_bits(sh.bits, grid, a, kcb, n_steps, stream);
  } else {
    dim3 grid(n_tiles, sh.n_kv_heads, sh.n_seq);
    launch_packed_tiles_bits(sh.bits, tqm::kSoftScores, tqm::kTilesDefault, grid, a, kcb, kcb, stream);
  }
  TQ_CHECK_LAUNCH(who);
  return launch_soft_weights(scores, stats, stats_pos, ws_S, ws_ml, t_pad, n_tiles, v_packed, v_norms, v_centroids,
                             v_signs, threshold, out, sh, stream, who);
}

// the matrix-core tile passes exist for d = 128 at every width
bool mma_shape(const tq_decode_shape& sh) {
  return sh.allow_mma && sh.dim == 128 && sh.bits >= 1 && sh.bits <= 4 && sh.n_rep <= tqm::kHeadsMax && sh.seq_len > 0;
}

bool vonly_mma_shape(const tq_decode_shape& sh) { return mma_shape(sh); }

int check_shape(const tq_decode_shape* sh, const char* who, int max_dim) {
  if (!sh) return tq::fail(TQ_ERR_NULL, "%s: null shape", who);
  if (int rc = tq::check_dim_bits(sh->dim, sh->bits)) return rc;
  if (sh->dim > max_dim)
    return tq::fail(TQ_ERR_DIM, "dim must be a power of 2 and <= %d, got %d", max_dim, sh->dim);
  if (int rc = check_heads(sh->n_kv_heads, sh->n_rep, who)) return rc;
  if (sh->n_seq < 1) return tq::fail(TQ_ERR_ARG, "%s: n_seq must be >= 1, got %d", who, sh->n_seq);
  if (sh->n_seq > 65535 || sh->n_kv_heads > 65535)         // sequences and kv heads are grid dimensions z and y
    return tq::fail(TQ_ERR_ARG, "%s: at most 65535 sequences and 65535 kv heads per call, got %d and %d", who,
                    sh->n_seq, sh->n_kv_heads);
  if (sh->seq_len < 0) return tq::fail(TQ_ERR_ARG, "%s: negative seq_len", who);
  if (sh->block_size < 1 || sh->block_size > 32)
    return tq::fail(TQ_ERR_BLOCK, "block_size must be in 1..32, got %d", sh->block_size);
  if (tq::check_dtype(sh->out_dtype)) return tq::fail(TQ_ERR_DTYPE, "%s: unknown out_dtype %d", who, sh->out_dtype);
  return 0;
}

}  // namespace

// ------------------------------------------------------------------ C ABI

extern "C" size_t tq_workspace_bytes(int op, int n_seq, int n_q_heads, int64_t max_seq_len, int dim) {
  if (n_seq < 1 || n_q_heads < 1 || max_seq_len < 0 || dim < 1) return 0;
  // Partials of the float32 kernels (tiles of kTile positions) bound those of the matrix-core
  // kernels (larger tiles), so one size serves every op.
  (void)op;
  return ws_bytes(n_seq, n_q_heads, max_seq_len, dim);
}

extern "C" int tq_prerot_qk_scores(const float* q_rot, const uint32_t* k_packed, const float* k_norms,
                                   const float* centroids, float* scores, int n_kv_heads, int n_rep,
                                   int64_t seq_len, int64_t packed_head_stride, int64_t norms_head_stride,
                                   int dim, int bits, int allow_mma, tq_stream_t stream_) {
  if (int rc = tq::check_dim_bits(dim, bits)) return rc;
  if (int rc = check_heads(n_kv_heads, n_rep, "tq_prerot_qk_scores")) return rc;
  if (seq_len < 0) return tq::fail(TQ_ERR_ARG, "tq_prerot_qk_scores: negative seq_len");
  if (seq_len == 0) return TQ_OK;
  if (!q_rot || !k_packed || !k_norms || !centroids || !scores)
    return tq::fail(TQ_ERR_NULL, "tq_prerot_qk_scores: null pointer");
  Codebook cb;
  fill_codebook(cb, centroids, bits);
  if (allow_mma == TQ_MMA_SPLIT && dim == 128 && bits >= 1 && bits <= 4 && n_rep <= tqm::kHeadsMax && tq::aligned(q_rot, 8)) {
    // split operands (value + remainder, three matrix instructions per tile): float32 fidelity
    tqm::SplitArgs a{};
    a.q_rot = q_rot; a.packed = k_packed; a.norms = k_norms; a.scores = scores;
    a.seq_len = seq_len; a.head_stride = packed_head_stride; a.norms_head_stride = norms_head_stride;
    a.n_kv = n_kv_heads; a.n_rep = n_rep; a.scale = 1.0f / (float)dim;
    dim3 grid((unsigned)((seq_len + tqm::kTilePos - 1) / tqm::kTilePos), n_kv_heads);
    a.n_tiles = (int)grid.x;
    launch_split_tiles_bits(bits, tqm::kScores, grid, a, cb, (hipStream_t)stream_);
    TQ_CHECK_LAUNCH("tq_prerot_qk_scores launch");
    return TQ_OK;
  }
  if (allow_mma && dim == 128 && bits >= 1 && bits <= 4 && n_rep <= tqm::kHeadsMax && tq::aligned(q_rot, 8)) {
    tqm::PackedArgs a{};
    a.q_rot = q_rot; a.k_packed = k_packed; a.k_norms = k_norms; a.scores = scores;
    a.seq_len = seq_len; a.k_head_stride = packed_head_stride; a.kn_head_stride = norms_head_stride;
    a.n_kv = n_kv_heads; a.n_rep = n_rep; a.n_tiles_max = 1;
    Codebook cbh;
    a.score_scale = tq::fill_codebook_fp16(cbh, centroids, bits) / (float)dim;
    dim3 grid((unsigned)((seq_len + tqm::kTilePos - 1) / tqm::kTilePos), n_kv_heads, 1);
    launch_packed_tiles_bits(bits, tqm::kScores, tqm::kTilesDefault, grid, a, cbh, cbh, (hipStream_t)stream_);
    TQ_CHECK_LAUNCH("tq_prerot_qk_scores launch");
    return TQ_OK;
  }
  const int n_rgroups = (n_rep + kRMax - 1) / kRMax;
  dim3 grid((unsigned)((seq_len + kScoreTile - 1) / kScoreTile), n_kv_heads * n_rgroups);
  hipStream_t stream = (hipStream_t)stream_;
  TQ_DISPATCH_DIM(dim, TQ_DISPATCH_BITS(bits, (prerot_scores_kernel<D_, B_><<<grid, kThreads, 0, stream>>>(
                                                  q_rot, k_packed, k_norms, cb, scores, n_rep, n_rgroups,
                                                  seq_len, packed_head_stride, norms_head_stride,
                                                  1.0f / (float)dim))));
  TQ_CHECK_LAUNCH("tq_prerot_qk_scores launch");
  return TQ_OK;
}

extern "C" int tq_dense_qk_scores(const void* q, int q_dtype, const void* k_f16, float* scores, int n_kv_heads,
                                  int n_rep, int64_t seq_len, int64_t k_head_stride, int dim, float scale,
                                  tq_stream_t stream_) {
  if (int rc = tq::check_dim_bits(dim, 3)) return rc;
  if (int rc = check_heads(n_kv_heads, n_rep, "tq_dense_qk_scores")) return rc;
  if (tq::check_dtype(q_dtype)) return tq::fail(TQ_ERR_DTYPE, "tq_dense_qk_scores: unknown q_dtype %d", q_dtype);
  if (seq_len < 0) return tq::fail(TQ_ERR_ARG, "tq_dense_qk_scores: negative seq_len");
  if (seq_len == 0) return TQ_OK;
  if (!q || !k_f16 || !scores) return tq::fail(TQ_ERR_NULL, "tq_dense_qk_scores: null pointer");
  if (!tq::aligned(k_f16, 16)) return tq::fail(TQ_ERR_ALIGN, "tq_dense_qk_scores: k must be 16-byte aligned");
  const int n_rgroups = (n_rep + kRMax - 1) / kRMax;
  dim3 grid(n_tiles_for(seq_len), n_kv_heads * n_rgroups);
  hipStream_t stream = (hipStream_t)stream_;
#define LAUNCH_DS(QT)                                                                                   \
  TQ_DISPATCH_DIM(dim, (dense_scores_kernel<D_, QT><<<grid, kThreads, 0, stream>>>(                       \
                           (const QT*)q, (const __half*)k_f16, scores, n_rep, n_rgroups, seq_len,         \
                           k_head_stride, scale)))
  if (q_dtype == TQ_F32) { LAUNCH_DS(float); }
  else if (q_dtype == TQ_F16) { LAUNCH_DS(__half); }
  else { LAUNCH_DS(__hip_bfloat16); }
#undef LAUNCH_DS
  TQ_CHECK_LAUNCH("tq_dense_qk_scores launch");
  return TQ_OK;
}

extern "C" int tq_softmax_rows(const float* scores, const float* mask, int64_t mask_row_stride, float* weights,
                               int64_t n_rows, int64_t seq_len, float scale, tq_stream_t stream_) {
  if (n_rows < 0 || seq_len < 0) return tq::fail(TQ_ERR_ARG, "tq_softmax_rows: negative size");
  if (n_rows == 0 || seq_len == 0) return TQ_OK;
  if (!scores || !weights) return tq::fail(TQ_ERR_NULL, "tq_softmax_rows: null pointer");
  if (n_rows > 0x7FFFFFFF) return tq::fail(TQ_ERR_ARG, "tq_softmax_rows: too many rows");
  // chunks per row: enough workgroups to fill the chip when the rows are few and long (at least 4096 positions each)
  int64_t n_chunks = (256 + n_rows - 1) / n_rows;      // about one workgroup per CU: every chunk re-reads its whole row
  if (n_chunks > seq_len / 4096) n_chunks = seq_len / 4096;
  if (n_chunks < 1) n_chunks = 1;
  int64_t chunk_len = (seq_len + n_chunks - 1) / n_chunks;
  chunk_len = (chunk_len + 3) & ~(int64_t)3;
  n_chunks = (seq_len + chunk_len - 1) / chunk_len;
  softmax_rows_kernel<<<dim3((unsigned)n_rows, (unsigned)n_chunks), kSmThreads, 0, (hipStream_t)stream_>>>(
      scores, mask, mask_row_stride, weights, seq_len, scale, chunk_len);
  TQ_CHECK_LAUNCH("tq_softmax_rows launch");
  return TQ_OK;
}

extern "C" int tq_sparse_v_matvec(const float* weights, const uint32_t* v_packed, const float* v_norms,
                                  const float* centroids, const float* signs, float* out, void* workspace,
                                  size_t workspace_bytes, int n_kv_heads, int n_rep, int64_t seq_len,
                                  int64_t packed_head_stride, int64_t norms_head_stride, int dim, int bits,
                                  float threshold, int allow_mma, tq_stream_t stream_) {
  if (!tq::is_pow2(dim)) return tq::fail(TQ_ERR_DIM, "dim must be a power of 2, got %d", dim);
  if (dim > 256) return tq::fail(TQ_ERR_DIM, "dim > 256 not supported by threadgroup layout, got %d", dim);
  tq_decode_shape sh{};
  sh.n_seq = 1; sh.n_kv_heads = n_kv_heads; sh.n_rep = n_rep; sh.dim = dim; sh.bits = bits;
  sh.block_size = 16; sh.seq_len = seq_len;
  sh.v_head_stride = packed_head_stride; sh.vn_head_stride = norms_head_stride;
  sh.out_dtype = TQ_F32;
  if (int rc = check_shape(&sh, "tq_sparse_v_matvec", 256)) return rc;
  if (!signs || !out || !centroids) return tq::fail(TQ_ERR_NULL, "tq_sparse_v_matvec: null pointer");
  if (seq_len > 0 && (!weights || !v_packed || !v_norms))
    return tq::fail(TQ_ERR_NULL, "tq_sparse_v_matvec: null pointer");
  const float thr = threshold > 0.0f ? threshold : 0.0f;
  sh.allow_mma = allow_mma;
  if (allow_mma == TQ_MMA_SPLIT && vonly_mma_shape(sh)) {
    // split operands (value + remainder, three matrix instructions per tile): float32 fidelity
    const int n_q = n_kv_heads * n_rep;
    const int n_tiles = (int)((seq_len + tqm::kTilePos - 1) / tqm::kTilePos);
    const size_t need = (size_t)n_q * n_tiles * (tqm::kD + 2) * sizeof(float);
    if (!workspace || workspace_bytes < need)
      return tq::fail(TQ_ERR_WORKSPACE, "tq_sparse_v_matvec: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    if (!tq::aligned(workspace, 16)) return tq::fail(TQ_ERR_ALIGN, "tq_sparse_v_matvec: workspace must be 16-byte aligned");
    tqm::SplitArgs a{};
    a.weights = weights; a.w_stride = seq_len; a.packed = v_packed; a.norms = v_norms;
    a.ws_S = (float*)workspace; a.ws_ml = a.ws_S + (size_t)n_q * n_tiles * tqm::kD;
    a.seq_len = seq_len; a.head_stride = packed_head_stride; a.norms_head_stride = norms_head_stride;
    a.n_kv = n_kv_heads; a.n_rep = n_rep; a.n_tiles = n_tiles; a.threshold = thr;
    Codebook cb;
    fill_codebook(cb, centroids, bits);
    hipStream_t stream = (hipStream_t)stream_;
    launch_split_tiles_bits(bits, tqm::kWeights, dim3(n_tiles, n_kv_heads), a, cb, stream);
    TQ_CHECK_LAUNCH("tq_sparse_v_matvec launch");
    tqm::decode_merge_rows_kernel<float, false><<<dim3(n_q, 1), tqm::kMergeThreads, 0, stream>>>(
        a.ws_S, a.ws_ml, nullptr, seq_len, n_tiles, n_kv_heads, n_rep, signs, 1.0f / (float)dim, out, tqm::kTilePos);
    TQ_CHECK_LAUNCH("tq_sparse_v_matvec merge launch");
    return TQ_OK;
  }
  if (vonly_mma_shape(sh))                                   // packed values only: every width
    return launch_packed_mfma<tqm::kWeights>(weights, nullptr, nullptr, v_packed, v_norms, centroids, centroids,
                                             signs, out, workspace, workspace_bytes, sh, thr,
                                             (hipStream_t)stream_, "tq_sparse_v_matvec");
  return launch_decode<kWeights>(weights, TQ_F32, nullptr, nullptr, nullptr, v_packed, v_norms, nullptr,
                                 centroids, signs, out, workspace, workspace_bytes, sh, thr,
                                 (hipStream_t)stream_, "tq_sparse_v_matvec");
}

extern "C" int tq_flash_decode_plan(int n_seq, int n_kv_heads, int64_t max_seq_len, int ragged, int masked) {
  if (n_seq < 1 || n_kv_heads < 1 || max_seq_len < 0) return 0;
  return masked ? 0 : flash_stream_steps(n_seq, n_kv_heads, max_seq_len, ragged != 0);
}

extern "C" int tq_flash_decode(const float* q_rot, const uint32_t* k_packed, const float* k_norms,
                               const uint32_t* v_packed, const float* v_norms, const float* k_centroids,
                               const float* v_centroids, const float* v_signs, void* out, void* workspace,
                               size_t workspace_bytes, const tq_decode_shape* shape, tq_stream_t stream_) {
  if (int rc = check_shape(shape, "tq_flash_decode", 128)) return rc;
  if (!q_rot || !k_centroids || !v_centroids || !v_signs || !out)
    return tq::fail(TQ_ERR_NULL, "tq_flash_decode: null pointer");
  if (shape->seq_len > 0 && (!k_packed || !k_norms || !v_packed || !v_norms))
    return tq::fail(TQ_ERR_NULL, "tq_flash_decode: null pointer");
  if (mma_shape(*shape) && tq::aligned(q_rot, 8))
    return launch_packed_mfma<tqm::kFlash>(q_rot, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids,
                                           v_signs, out, workspace, workspace_bytes, *shape, 0.0f,
                                           (hipStream_t)stream_, "tq_flash_decode");
  return launch_decode<kPackedK>(q_rot, TQ_F32, k_packed, k_norms, nullptr, v_packed, v_norms, k_centroids,
                                 v_centroids, v_signs, out, workspace, workspace_bytes, *shape, 0.0f,
                                 (hipStream_t)stream_, "tq_flash_decode");
}

extern "C" int tq_vonly_decode_attn_phases(const void* q, int q_dtype, const void* k_f16, const uint32_t* v_packed,
                                           const float* v_norms, const float* v_centroids, const float* v_signs,
                                           void* out, void* workspace, size_t workspace_bytes,
                                           const tq_decode_shape* shape, int phases, tq_stream_t stream_) {
  if (int rc = check_shape(shape, "tq_vonly_decode_attn", 256)) return rc;
  if (phases < 1 || phases > 3) return tq::fail(TQ_ERR_ARG, "tq_vonly_decode_attn: phases must be 1, 2 or 3");
  if (tq::check_dtype(q_dtype)) return tq::fail(TQ_ERR_DTYPE, "tq_vonly_decode_attn: unknown q_dtype %d", q_dtype);
  if (!q || !v_centroids || !v_signs || !out) return tq::fail(TQ_ERR_NULL, "tq_vonly_decode_attn: null pointer");
  if (shape->seq_len > 0 && (!k_f16 || !v_packed || !v_norms))
    return tq::fail(TQ_ERR_NULL, "tq_vonly_decode_attn: null pointer");
  if (!tq::aligned(k_f16, 16)) return tq::fail(TQ_ERR_ALIGN, "tq_vonly_decode_attn: k must be 16-byte aligned");
  // d = 128, at most 16 query heads per kv head: matrix-core tile pass (float32 queries as fp16 value + remainder).
  if (vonly_mma_shape(*shape) && tq::aligned(q, 16))
    return launch_vonly_mfma(q, q_dtype, k_f16, v_packed, v_norms, v_centroids, v_signs, out, workspace, workspace_bytes,
                             *shape, (hipStream_t)stream_, phases);
  return launch_decode<kDenseK>(q, q_dtype, nullptr, nullptr, k_f16, v_packed, v_norms, nullptr, v_centroids,
                                v_signs, out, workspace, workspace_bytes, *shape, 0.0f, (hipStream_t)stream_,
                                "tq_vonly_decode_attn", phases);
}

extern "C" int tq_vonly_decode_attn(const void* q, int q_dtype, const void* k_f16, const uint32_t* v_packed,
                                    const float* v_norms, const float* v_centroids, const float* v_signs,
                                    void* out, void* workspace, size_t workspace_bytes,
                                    const tq_decode_shape* shape, tq_stream_t stream_) {
  return tq_vonly_decode_attn_phases(q, q_dtype, k_f16, v_packed, v_norms, v_centroids, v_signs, out, workspace,
                                     workspace_bytes, shape, 3, stream_);
}

// ---- the entry point that allocates nothing -------------------------------------------------------------
// Per-tile partial sums of tq_vonly_decode_attn_static live in this array instead of a caller's workspace.
// Every GPU the library runs on holds its own copy at its own address until the process ends; in host code
// the array's name is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t kStaticScratchBytes = TQ_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];      // device address of `scratch` per device ordinal, resolved once
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device: hipGetSymbolAddress on the first call per device.
int static_scratch(void** ptr, const char* who) {
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return tq::hip_fail(e, who);
  if (dev < 0 || dev >= kMaxDevices) return tq::fail(TQ_ERR_ARG, "%s: device ordinal %d outside 0..%d", who, dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)); e != hipSuccess) return tq::hip_fail(e, who);
    if (!p) return tq::fail(TQ_ERR_HIP, "%s: hipGetSymbolAddress returned a null address", who);
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return TQ_OK;
}
}  // namespace

extern "C" int tq_vonly_decode_attn_static(const void* q, int q_dtype, const void* k_f16, const uint32_t* v_packed,
                                           const float* v_norms, const float* v_centroids, const float* v_signs,
                                           void* out, const tq_decode_shape* shape, tq_stream_t stream_) {
  const char* who = "tq_vonly_decode_attn_static";
  if (int rc = check_shape(shape, who, 256)) return rc;
  const size_t need = ws_bytes(shape->n_seq, shape->n_kv_heads * shape->n_rep, shape->seq_len, shape->dim);
  if (need > kStaticScratchBytes)
    return tq::fail(TQ_ERR_WORKSPACE,
                    "%s: this shape needs %zu bytes of per-tile partial sums, the static scratch holds %zu; "
                    "call tq_vonly_decode_attn with a workspace instead", who, need, kStaticScratchBytes);
  void* ptr = nullptr;
  if (int rc = static_scratch(&ptr, who)) return rc;
  return tq_vonly_decode_attn_phases(q, q_dtype, k_f16, v_packed, v_norms, v_centroids, v_signs, out, ptr,
                                     kStaticScratchBytes, shape, 3, stream_);
}

namespace {
constexpr int kNotFused = 1;   // not an error: the caller takes the append + attention route

// A decode step as two launches: the tile pass over the positions before the new one, and a merge pass that
// encodes and stores the new token itself (tqm::FreshToken).  dim 128, values of any width, n_rep <= 16.
int vonly_step_fused(const tq_vonly_cache_desc* c, const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                     const void* q, int q_dtype, void* out, int out_dtype, int64_t position, const int64_t* position_dev,
                     float attn_scale, tq_stream_t stream_, const char* who) {
  if (!(c->dim == 128 && c->bits >= 1 && c->bits <= 4 && c->n_rep >= 1 && c->n_rep <= tqm::kHeadsMax && c->allow_mma &&
        tq::aligned(q, 16) && tq::aligned(c->k_f16, 16)))
    return kNotFused;
  if (tq::check_dtype(k_dtype) || tq::check_dtype(v_dtype) || tq::check_dtype(q_dtype) || tq::check_dtype(out_dtype))
    return tq::fail(TQ_ERR_DTYPE, "%s: unknown dtype", who);
  if (c->variant != TQ_ENCODE_MLX && c->variant != TQ_ENCODE_METAL)
    return tq::fail(TQ_ERR_ARG, "%s: unknown variant %d", who, c->variant);
  if (!k_new || !v_new || !q || !out || !c->v_signs) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (!tq::aligned(k_new, tq::dtype_size(k_dtype)) || !tq::aligned(v_new, tq::dtype_size(v_dtype)) ||
      !tq::aligned(c->v_packed, 4) || !tq::aligned(c->v_norms, 4) || !tq::aligned(c->v_signs, 4) ||
      (c->v_raw && !tq::aligned(c->v_raw, tq::dtype_size(v_dtype))))
    return tq::fail(TQ_ERR_ALIGN, "%s: misaligned pointer", who);
  if (c->n_seq > 65535) return tq::fail(TQ_ERR_ARG, "%s: at most 65535 sequences per call", who);
  tqm::FreshToken f{};
  f.k_new = k_new; f.v_new = v_new; f.q = q;
  f.k_f16 = (__half*)c->k_f16; f.v_raw = c->v_raw; f.v_packed = c->v_packed; f.v_norms = c->v_norms;
  f.pos_dev = position_dev; f.pos = position; f.t_alloc = c->t_alloc;
  for (int i = 0; i < 15; ++i) f.thr[i] = INFINITY;         // past the width: never exceeded
  tq::encode_thresholds(c->boundaries, c->dim, c->bits, c->variant, f.thr);
  for (int i = 0; i < 16; ++i) f.cent[i] = i < (1 << c->bits) ? c->centroids[i] : 0.0f;
  f.bits = c->bits;
  f.cs = attn_scale * tqm::kLog2e;
  f.k_dtype = k_dtype; f.v_dtype = v_dtype; f.q_dtype = q_dtype;
  tq_decode_shape sh{};
  sh.n_seq = c->n_seq; sh.n_kv_heads = c->n_kv_heads; sh.n_rep = c->n_rep; sh.dim = c->dim; sh.bits = c->bits;
  sh.block_size = 16;
  sh.seq_len = position_dev ? c->t_alloc : position;        // positions before the new one (device: upper bound)
  sh.k_head_stride = sh.v_head_stride = sh.vn_head_stride = c->t_alloc;
  sh.k_seq_stride = sh.v_seq_stride = sh.vn_seq_stride = c->t_alloc * c->n_kv_heads;
  sh.attn_scale = attn_scale; sh.out_dtype = out_dtype; sh.allow_mma = 1;
  return launch_vonly_mfma(q, q_dtype, c->k_f16, c->v_packed, c->v_norms, c->centroids, c->v_signs, out, c->workspace,
                           c->workspace_bytes, sh, (hipStream_t)stream_, 3, position_dev, 0, &f);
}
}  // namespace

extern "C" int tq_vonly_decode_step(const tq_vonly_cache_desc* c, const void* k_new, int k_dtype, const void* v_new,
                                    int v_dtype, const void* q, int q_dtype, void* out, int out_dtype,
                                    int64_t position, float attn_scale, tq_stream_t stream_) {
  const char* who = "tq_vonly_decode_step";
  if (!c) return tq::fail(TQ_ERR_NULL, "%s: null cache descriptor", who);
  if (int rc = tq::check_dim_bits(c->dim, c->bits)) return rc;
  if (c->n_seq < 1 || c->n_kv_heads < 1 || c->t_alloc < 1)
    return tq::fail(TQ_ERR_ARG, "%s: empty cache descriptor (n_seq %d, n_kv_heads %d, t_alloc %lld)", who, c->n_seq,
                    c->n_kv_heads, (long long)c->t_alloc);
  if (position < 0 || position >= c->t_alloc)
    return tq::fail(TQ_ERR_ARG, "%s: position %lld outside the storage of %lld positions", who, (long long)position,
                    (long long)c->t_alloc);
  if (!c->k_f16 || !c->v_packed || !c->v_norms) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (int rc = vonly_step_fused(c, k_new, k_dtype, v_new, v_dtype, q, q_dtype, out, out_dtype, position, nullptr,
                                attn_scale, stream_, who); rc != kNotFused)
    return rc;
  const int pdim = tq::packed_dim(c->dim, c->bits);
  const int64_t groups = (int64_t)c->n_seq * c->n_kv_heads;
  if (int rc = tq_vonly_append(
          k_new, k_dtype, v_new, v_dtype, c->v_signs, c->boundaries, (__half*)c->k_f16 + position * c->dim,
          c->v_raw ? (char*)c->v_raw + position * c->dim * (int64_t)tq::dtype_size(v_dtype) : nullptr,
          c->v_packed + position * pdim, c->v_norms + position, groups, 1, c->t_alloc, c->t_alloc, c->t_alloc,
          c->t_alloc, c->dim, c->bits, c->variant, stream_))
    return rc;
  tq_decode_shape sh{};
  sh.n_seq = c->n_seq; sh.n_kv_heads = c->n_kv_heads; sh.n_rep = c->n_rep; sh.dim = c->dim; sh.bits = c->bits;
  sh.block_size = 16;
  sh.seq_len = position + 1;
  sh.k_head_stride = sh.v_head_stride = sh.vn_head_stride = c->t_alloc;
  sh.k_seq_stride = sh.v_seq_stride = sh.vn_seq_stride = c->t_alloc * c->n_kv_heads;
  sh.attn_scale = attn_scale; sh.out_dtype = out_dtype; sh.allow_mma = c->allow_mma;
  return tq_vonly_decode_attn(q, q_dtype, c->k_f16, c->v_packed, c->v_norms, c->centroids, c->v_signs, out,
                              c->workspace, c->workspace_bytes, &sh, stream_);
}

extern "C" size_t tq_vonly_sparse_workspace_bytes(int n_seq, int n_q_heads, int64_t max_seq_len) {
  if (n_seq < 1 || n_q_heads < 1 || max_seq_len < 0) return 0;
  return vonly_sparse_ws_bytes(n_seq, n_q_heads, max_seq_len);
}

extern "C" int tq_vonly_sparse_decode_attn(const void* q, int q_dtype, const void* k_f16, const uint32_t* v_packed,
                                           const float* v_norms, const float* v_centroids, const float* v_signs,
                                           float threshold, void* out, void* workspace, size_t workspace_bytes,
                                           const tq_decode_shape* shape, tq_stream_t stream_) {
  const char* who = "tq_vonly_sparse_decode_attn";
  if (int rc = check_shape(shape, who, 256)) return rc;
  if (tq::check_dtype(q_dtype)) return tq::fail(TQ_ERR_DTYPE, "%s: unknown q_dtype %d", who, q_dtype);
  if (!q || !v_centroids || !v_signs || !out) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (shape->seq_len > 0 && (!k_f16 || !v_packed || !v_norms)) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (!tq::aligned(k_f16, 16)) return tq::fail(TQ_ERR_ALIGN, "%s: k must be 16-byte aligned", who);
  if (!(threshold >= 0.0f)) return tq::fail(TQ_ERR_ARG, "%s: threshold must be >= 0", who);
  if (!(shape->dim == 128 && shape->n_rep <= tqm::kHeadsMax && shape->seq_len > 0 && tq::aligned(q, 16)))
    return tq::fail(TQ_ERR_UNSUPPORTED, "%s: dim 128, n_rep <= 16, a non-empty cache and a 16-byte aligned q only "
                                        "(compose tq_dense_qk_scores, tq_softmax_rows and tq_sparse_v_matvec otherwise)", who);
  return launch_vonly_sparse(q, q_dtype, k_f16, v_packed, v_norms, v_centroids, v_signs, threshold, out, workspace,
                             workspace_bytes, *shape, (hipStream_t)stream_);
}

extern "C" int tq_flash_sparse_decode(const float* q_rot, const uint32_t* k_packed, const float* k_norms,
                                      const uint32_t* v_packed, const float* v_norms, const float* k_centroids,
                                      const float* v_centroids, const float* v_signs, float threshold, void* out,
                                      void* workspace, size_t workspace_bytes, const tq_decode_shape* shape,
                                      tq_stream_t stream_) {
  const char* who = "tq_flash_sparse_decode";
  if (int rc = check_shape(shape, who, 128)) return rc;
  if (!q_rot || !k_centroids || !v_centroids || !v_signs || !out) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (shape->seq_len > 0 && (!k_packed || !k_norms || !v_packed || !v_norms))
    return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (!(threshold >= 0.0f)) return tq::fail(TQ_ERR_ARG, "%s: threshold must be >= 0", who);
  if (!(shape->dim == 128 && shape->bits >= 1 && shape->bits <= 4 && shape->n_rep <= tqm::kHeadsMax && shape->seq_len > 0 &&
        tq::aligned(q_rot, 8)))
    return tq::fail(TQ_ERR_UNSUPPORTED, "%s: dim 128, n_rep <= 16 and a non-empty cache only "
                                        "(compose tq_prerot_qk_scores, tq_softmax_rows and tq_sparse_v_matvec otherwise)", who);
  return launch_flash_sparse(q_rot, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids, v_signs, threshold,
                             out, workspace, workspace_bytes, *shape, (hipStream_t)stream_);
}

extern "C" int tq_flash_decode_from_q(const void* q, int q_dtype, const float* k_signs, const uint32_t* k_packed,
                                      const float* k_norms, const uint32_t* v_packed, const float* v_norms,
                                      const float* k_centroids, const float* v_centroids, const float* v_signs,
                                      float threshold, void* out, void* workspace, size_t workspace_bytes,
                                      const tq_decode_shape* shape, tq_stream_t stream_) {
  const char* who = "tq_flash_decode_from_q";
  if (int rc = check_shape(shape, who, 128)) return rc;
  if (tq::check_dtype(q_dtype)) return tq::fail(TQ_ERR_DTYPE, "%s: unknown q_dtype %d", who, q_dtype);
  if (!q || !k_signs || !k_centroids || !v_centroids || !v_signs || !out) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (shape->seq_len > 0 && (!k_packed || !k_norms || !v_packed || !v_norms))
    return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (!(threshold >= 0.0f)) return tq::fail(TQ_ERR_ARG, "%s: threshold must be >= 0", who);
  if (!(shape->dim == 128 && shape->bits >= 1 && shape->bits <= 4 && shape->n_rep <= tqm::kHeadsMax && shape->seq_len > 0 &&
        tq::aligned(q, (int)tq::dtype_size(q_dtype))))
    return tq::fail(TQ_ERR_UNSUPPORTED, "%s: dim 128, n_rep <= 16 and a non-empty cache only "
                                        "(call tq_prerotate_query and tq_flash_decode otherwise)", who);
  hipStream_t stream = (hipStream_t)stream_;
  if (threshold > 0.0f)
    return launch_flash_sparse(nullptr, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids, v_signs, threshold,
                               out, workspace, workspace_bytes, *shape, stream, q, q_dtype, k_signs);
  tq_decode_shape sh = *shape;
  sh.allow_mma = 1;
  return launch_packed_mfma<tqm::kFlash>(nullptr, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids, v_signs,
                                         out, workspace, workspace_bytes, sh, 0.0f, stream, who, q, q_dtype, k_signs);
}

extern "C" int tq_vonly_decode_step_at(const tq_vonly_cache_desc* c, const void* k_new, int k_dtype, const void* v_new,
                                       int v_dtype, const void* q, int q_dtype, void* out, int out_dtype,
                                       const int64_t* position_dev, float attn_scale, tq_stream_t stream_) {
  const char* who = "tq_vonly_decode_step_at";
  if (!c || !position_dev) return tq::fail(TQ_ERR_NULL, "%s: null cache descriptor or position_dev", who);
  if (c->n_seq < 1 || c->n_kv_heads < 1 || c->t_alloc < 1)
    return tq::fail(TQ_ERR_ARG, "%s: empty cache descriptor (n_seq %d, n_kv_heads %d, t_alloc %lld)", who, c->n_seq,
                    c->n_kv_heads, (long long)c->t_alloc);
  if (!c->k_f16 || !c->v_packed || !c->v_norms || !q || !out || !c->v_signs)
    return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  tq_decode_shape sh{};
  sh.n_seq = c->n_seq; sh.n_kv_heads = c->n_kv_heads; sh.n_rep = c->n_rep; sh.dim = c->dim; sh.bits = c->bits;
  sh.block_size = 16;
  sh.seq_len = c->t_alloc;                                 // upper bound: sizes the grid and the workspace
  sh.k_head_stride = sh.v_head_stride = sh.vn_head_stride = c->t_alloc;
  sh.k_seq_stride = sh.v_seq_stride = sh.vn_seq_stride = c->t_alloc * c->n_kv_heads;
  sh.attn_scale = attn_scale; sh.out_dtype = out_dtype; sh.allow_mma = 1;
  if (int rc = check_shape(&sh, who, 256)) return rc;
  if (tq::check_dtype(q_dtype)) return tq::fail(TQ_ERR_DTYPE, "%s: unknown q_dtype %d", who, q_dtype);
  if (!(vonly_mma_shape(sh) && tq::aligned(q, 16) && tq::aligned(c->k_f16, 16)))
    return tq::fail(TQ_ERR_UNSUPPORTED, "%s: dim 128, n_rep <= 16 and aligned q / k only", who);
  const int n_q = c->n_kv_heads * c->n_rep;
  if (c->workspace_bytes < tq_workspace_bytes(TQ_OP_VONLY_DECODE, c->n_seq, n_q, c->t_alloc, c->dim))
    return tq::fail(TQ_ERR_WORKSPACE, "%s: workspace too small for %lld positions", who, (long long)c->t_alloc);
  if (!tq::aligned(position_dev, 8)) return tq::fail(TQ_ERR_ALIGN, "%s: position_dev must be 8-byte aligned", who);
  if (int rc = vonly_step_fused(c, k_new, k_dtype, v_new, v_dtype, q, q_dtype, out, out_dtype, 0, position_dev,
                                attn_scale, stream_, who); rc != kNotFused)
    return rc;
  return tq::fail(TQ_ERR_UNSUPPORTED, "%s: shape not covered", who);
}

namespace {
int packed_step(const tq_packed_cache_desc* c, const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                const void* q, int q_dtype, void* out, int out_dtype, int64_t position, const int64_t* position_dev,
                float attn_scale, tq_stream_t stream_, const char* who) {
  if (!c) return tq::fail(TQ_ERR_NULL, "%s: null cache descriptor", who);
  if (int rc = tq::check_dim_bits(c->dim, c->bits)) return rc;
  if (c->n_seq < 1 || c->n_kv_heads < 1 || c->t_alloc < 1)
    return tq::fail(TQ_ERR_ARG, "%s: empty cache descriptor (n_seq %d, n_kv_heads %d, t_alloc %lld)", who, c->n_seq,
                    c->n_kv_heads, (long long)c->t_alloc);
  if (position < 0 || position >= c->t_alloc)
    return tq::fail(TQ_ERR_ARG, "%s: position %lld outside the storage of %lld positions", who, (long long)position,
                    (long long)c->t_alloc);
  if (!c->k_packed || !c->k_norms || !c->v_packed || !c->v_norms) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (!(c->dim == 128 && c->bits >= 1 && c->bits <= 4 && c->n_rep >= 1 && c->n_rep <= tqm::kHeadsMax))
    return tq::fail(TQ_ERR_UNSUPPORTED, "%s: dim 128 and n_rep <= 16 only (call tq_encode, "
                                        "tq_prerotate_query and tq_flash_decode otherwise)", who);
  const int pdim = tq::packed_dim(c->dim, c->bits);
  const int64_t groups = (int64_t)c->n_seq * c->n_kv_heads;
  if (tq::check_dtype(k_dtype) || tq::check_dtype(v_dtype))
    return tq::fail(TQ_ERR_DTYPE, "%s: unknown dtype %d / %d", who, k_dtype, v_dtype);
  if (c->variant != TQ_ENCODE_MLX && c->variant != TQ_ENCODE_METAL)
    return tq::fail(TQ_ERR_ARG, "%s: unknown variant %d", who, c->variant);
  if (!k_new || !v_new || !c->k_signs || !c->v_signs) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (!tq::aligned(k_new, tq::dtype_size(k_dtype)) || !tq::aligned(v_new, tq::dtype_size(v_dtype)) ||
      !tq::aligned(c->k_signs, 4) || !tq::aligned(c->v_signs, 4) || !tq::aligned(c->k_packed, 4) ||
      !tq::aligned(c->v_packed, 4) || !tq::aligned(c->k_norms, 4) || !tq::aligned(c->v_norms, 4))
    return tq::fail(TQ_ERR_ALIGN, "%s: misaligned pointer", who);
  if (q && out && !tq::check_dtype(q_dtype) && !tq::check_dtype(out_dtype) && tq::aligned(q, (int)tq::dtype_size(q_dtype)) &&
      (!position_dev || tq::aligned(position_dev, 8)) && c->n_seq <= 65535 && c->n_kv_heads <= 65535) {
    // two launches: the tile pass over the positions before the new one, and a merge pass that encodes both new
    // rows, scores the new key and stores them (tqm::FreshToken with packed keys)
    tqm::FreshToken f{};
    f.k_new = k_new; f.v_new = v_new; f.q = q;
    f.v_packed = c->v_packed; f.v_norms = c->v_norms; f.k_packed = c->k_packed; f.k_norms = c->k_norms;
    f.k_signs = c->k_signs;
    f.pos_dev = position_dev; f.pos = position; f.t_alloc = c->t_alloc;
    for (int i = 0; i < 15; ++i) f.thr[i] = INFINITY;
    tq::encode_thresholds(c->boundaries, c->dim, c->bits, c->variant, f.thr);
    for (int i = 0; i < 16; ++i) f.cent[i] = i < (1 << c->bits) ? c->centroids[i] : 0.0f;
    f.bits = c->bits;
    f.cs = attn_scale * tqm::kLog2e;
    f.k_dtype = k_dtype; f.v_dtype = v_dtype; f.q_dtype = q_dtype;
    tq_decode_shape fs{};
    fs.n_seq = c->n_seq; fs.n_kv_heads = c->n_kv_heads; fs.n_rep = c->n_rep; fs.dim = c->dim; fs.bits = c->bits;
    fs.block_size = 16;
    fs.seq_len = position_dev ? c->t_alloc : position;     // positions before the new one (device: upper bound)
    fs.k_head_stride = fs.kn_head_stride = fs.v_head_stride = fs.vn_head_stride = c->t_alloc;
    fs.k_seq_stride = fs.kn_seq_stride = fs.v_seq_stride = fs.vn_seq_stride = c->t_alloc * c->n_kv_heads;
    fs.attn_scale = attn_scale; fs.out_dtype = out_dtype; fs.allow_mma = 1;
    return launch_packed_mfma<tqm::kFlash>(nullptr, c->k_packed, c->k_norms, c->v_packed, c->v_norms, c->centroids,
                                           c->centroids, c->v_signs, out, c->workspace, c->workspace_bytes, fs, 0.0f,
                                           (hipStream_t)stream_, who, q, q_dtype, c->k_signs, position_dev, 0, &f);
  }
  if (int rc = tq::encode_pair(k_new, k_dtype, c->k_signs, c->k_packed + position * pdim, c->k_norms + position, v_new,
                               v_dtype, c->v_signs, c->v_packed + position * pdim, c->v_norms + position, c->boundaries,
                               c->bits, groups, c->t_alloc, c->variant, stream_, position_dev))
    return rc;
  tq_decode_shape sh{};
  sh.n_seq = c->n_seq; sh.n_kv_heads = c->n_kv_heads; sh.n_rep = c->n_rep; sh.dim = c->dim; sh.bits = c->bits;
  sh.block_size = 16;
  sh.seq_len = position_dev ? c->t_alloc : position + 1;   // device position: upper bound that sizes grid and workspace
  sh.k_head_stride = sh.kn_head_stride = sh.v_head_stride = sh.vn_head_stride = c->t_alloc;
  sh.k_seq_stride = sh.kn_seq_stride = sh.v_seq_stride = sh.vn_seq_stride = c->t_alloc * c->n_kv_heads;
  sh.attn_scale = attn_scale; sh.out_dtype = out_dtype; sh.allow_mma = 1;
  if (!position_dev)
    return tq_flash_decode_from_q(q, q_dtype, c->k_signs, c->k_packed, c->k_norms, c->v_packed, c->v_norms, c->centroids,
                                  c->centroids, c->v_signs, 0.0f, out, c->workspace, c->workspace_bytes, &sh, stream_);
  if (int rc = check_shape(&sh, who, 128)) return rc;
  if (tq::check_dtype(q_dtype)) return tq::fail(TQ_ERR_DTYPE, "%s: unknown q_dtype %d", who, q_dtype);
  if (!q || !out) return tq::fail(TQ_ERR_NULL, "%s: null pointer", who);
  if (!tq::aligned(q, (int)tq::dtype_size(q_dtype)) || !tq::aligned(position_dev, 8))
    return tq::fail(TQ_ERR_ALIGN, "%s: misaligned pointer", who);
  return launch_packed_mfma<tqm::kFlash>(nullptr, c->k_packed, c->k_norms, c->v_packed, c->v_norms, c->centroids,
                                         c->centroids, c->v_signs, out, c->workspace, c->workspace_bytes, sh, 0.0f,
                                         (hipStream_t)stream_, who, q, q_dtype, c->k_signs, position_dev, 1);
}
}  // namespace

extern "C" int tq_packed_decode_step(const tq_packed_cache_desc* c, const void* k_new, int k_dtype, const void* v_new,
                                     int v_dtype, const void* q, int q_dtype, void* out, int out_dtype,
                                     int64_t position, float attn_scale, tq_stream_t stream_) {
  if (c && (position < 0 || position >= c->t_alloc))
    return tq::fail(TQ_ERR_ARG, "tq_packed_decode_step: position %lld outside the storage of %lld positions",
                    (long long)position, (long long)c->t_alloc);
  return packed_step(c, k_new, k_dtype, v_new, v_dtype, q, q_dtype, out, out_dtype, position, nullptr, attn_scale,
                     stream_, "tq_packed_decode_step");
}

extern "C" int tq_packed_decode_step_at(const tq_packed_cache_desc* c, const void* k_new, int k_dtype, const void* v_new,
                                        int v_dtype, const void* q, int q_dtype, void* out, int out_dtype,
                                        const int64_t* position_dev, float attn_scale, tq_stream_t stream_) {
  if (!position_dev) return tq::fail(TQ_ERR_NULL, "tq_packed_decode_step_at: null position_dev");
  return packed_step(c, k_new, k_dtype, v_new, v_dtype, q, q_dtype, out, out_dtype, 0, position_dev, attn_scale,
                     stream_, "tq_packed_decode_step_at");
}
