/*
 * tqhip.h -- C ABI of libtqhip.so: the PolarQuant KV-cache hot path on MI355X (gfx950).
 *
 * One entry point per GPU kernel launcher of the reference (each of which is a
 * Python wrapper around mx.fast.metal_kernel); the citation on each declaration
 * is the reference interface it replaces.  A reference-side binding is a ctypes
 * stub that passes device pointers and sizes.
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless the comment says "host"; the two small tables,
 *    `boundaries` and `centroids` (at most 16 floats), are always HOST pointers: they travel
 *    to the kernels by value;
 *  - the library never allocates or frees device memory: outputs and workspace
 *    are caller-owned;
 *  - launches are asynchronous on `stream` (a hipStream_t passed as void*);
 *  - every function returns 0 on success or a negative tq_status; the text of
 *    the last failure on the calling thread is tq_last_error();
 *  - packed layout: element e of a vector lives in uint32 word e / vpw at bit
 *    offset (e % vpw) * bits, vpw = 32/16/10/8 for bits = 1/2/3/4
 *    (reference turboquant_mlx/packing.py:16-56);
 *  - "KV addressing": sequence s, kv head h, position p of a packed / norm / fp16-K
 *    tensor is the row  s * seq_stride + h * head_stride + (first[s] + p)
 *    where strides are counted in ROWS (a row = pdim words, 1 norm, or dim halfs),
 *    first[s] = seq_offsets ? seq_offsets[s] : 0 and the sequence length is
 *    seq_offsets ? seq_offsets[s+1] - seq_offsets[s] : seq_len.
 *    A cache tensor [B, H, T_alloc, *] uses seq_stride = H*T_alloc, head_stride =
 *    T_alloc, seq_offsets = NULL; a ragged batch [H, sum(L), *] uses seq_stride = 0,
 *    head_stride = sum(L) and seq_offsets[n_seq+1].
 */
#ifndef TQHIP_H
#define TQHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* tq_stream_t;

enum tq_dtype { TQ_F32 = 0, TQ_F16 = 1, TQ_BF16 = 2 };

enum tq_status {
  TQ_OK = 0,
  TQ_ERR_NULL = -1,       /* a required pointer is NULL */
  TQ_ERR_DIM = -2,        /* dim not a power of two or out of range */
  TQ_ERR_BITS = -3,       /* bits not in 1..4 */
  TQ_ERR_NREP = -4,       /* n_q_heads != n_kv_heads * n_rep, or n_rep < 1 */
  TQ_ERR_ALIGN = -5,      /* pointer not aligned for its element type */
  TQ_ERR_DTYPE = -6,      /* unknown tq_dtype */
  TQ_ERR_BLOCK = -7,      /* block_size outside 1..32 */
  TQ_ERR_WORKSPACE = -8,  /* workspace too small */
  TQ_ERR_ARG = -9,        /* other invalid argument (negative size, ...) */
  TQ_ERR_UNSUPPORTED = -10, /* valid request this build has no kernel for */
  TQ_ERR_HIP = -100       /* a HIP call failed; tq_last_error() holds hipGetErrorString */
};

/* encode variants */
enum tq_encode_variant {
  TQ_ENCODE_MLX = 0,   /* bits equal to PolarQuantizer.quantize (quantizer.py:85-106):
                          compares (w*s)/s, s = float32(1/sqrt(dim)) */
  TQ_ENCODE_METAL = 1  /* bits equal to the fused Metal encoder (metal.py:66-77):
                          compares the raw butterfly output w */
};

/* values of the `allow_mma` argument of tq_prerot_qk_scores and tq_sparse_v_matvec */
enum tq_mma_mode {
  TQ_MMA_OFF = 0,      /* float32 vector kernels */
  TQ_MMA_FP16 = 1,     /* matrix cores, operands rounded to fp16 */
  TQ_MMA_SPLIT = 2     /* matrix cores, operands as fp16 value + fp16 remainder: float32 fidelity */
};

/* which fused decode kernel a workspace query is for */
enum tq_op {
  TQ_OP_SPARSE_V = 0,
  TQ_OP_FLASH_DECODE = 1,
  TQ_OP_VONLY_DECODE = 2
};

int tq_version(void);
const char* tq_last_error(void);            /* host string, valid until the next failing call on this thread */
const char* tq_status_string(int status);   /* host string */

/*
 * Fused encode: per-vector L2 norm -> x/max(n,1e-8) -> sign flip -> Walsh-Hadamard
 * butterfly -> Lloyd-Max boundary count -> bit packing.
 * Replaces fused_quantize (reference turboquant_mlx/metal.py:147-196, kernel 14-101) and,
 * with TQ_ENCODE_MLX, PolarQuantizer.quantize + pack_indices (quantizer.py:75-106,
 * packing.py:26-56).
 *   x          [n_groups*rows_per_group, dim] contiguous, dtype x_dtype
 *   signs      [dim] float, +-1 (device);  boundaries [2^bits - 1] float, ascending (HOST)
 *   packed     row r = (g, i) is written at packed + (g*packed_group_stride + i) * pdim words
 *   norms      row r is written at norms + g*norms_group_stride + i   (float32, un-clamped norm)
 * With n_groups = 1 this is the plain (n_vecs, dim) -> (n_vecs, pdim), (n_vecs,) call.
 */
int tq_encode(const void* x, int x_dtype, const float* signs, const float* boundaries,
              uint32_t* packed, float* norms,
              int64_t n_groups, int64_t rows_per_group,
              int64_t packed_group_stride, int64_t norms_group_stride,
              int dim, int bits, int variant, tq_stream_t stream);

/*
 * Append new tokens to a cache that keeps float16 keys beside PolarQuant values, in ONE launch:
 * every new value row is encoded exactly as tq_encode does (bit-identical words and norms), and
 * the wavefront that encodes row (g, i) also stores the key row, converted to float16 with
 * round-to-nearest-even, and (when v_raw is not null) the value row unchanged.
 * Replaces the insert of VOnlyTurboQuantCache.update_and_fetch (reference
 * turboquant_mlx/v_only_cache.py:52-53,74: KVCache.update_and_fetch(keys, values) followed by the
 * encode on insert of TurboQuantKVCache, cache.py:141-160), which is three slice assignments and
 * one kernel there.
 *   k_new, v_new  [n_groups*rows_per_group, dim] contiguous, dtypes k_dtype / v_dtype
 *   k_f16         row (g, i) at k_f16 + (g*k_group_stride + i) * dim halves
 *   v_raw         row (g, i) at v_raw + (g*v_raw_group_stride + i) * dim elements of v_dtype, or NULL
 *   v_packed, v_norms, strides, boundaries (HOST), variant: as in tq_encode
 * The destination pointers already point at the first free position of group 0.
 */
int tq_vonly_append(const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                    const float* v_signs, const float* boundaries,
                    void* k_f16, void* v_raw, uint32_t* v_packed, float* v_norms,
                    int64_t n_groups, int64_t rows_per_group,
                    int64_t k_group_stride, int64_t v_raw_group_stride,
                    int64_t packed_group_stride, int64_t norms_group_stride,
                    int dim, int bits, int variant, tq_stream_t stream);

/*
 * Dequantise packed rows: out = ((butterfly(c[idx]*s) * s) * signs) * norm, s = 1/sqrt(dim).
 * Replaces packed_dequantize (kernels.py:123-155, kernel 14-55; out_dtype TQ_F32) and
 * dequant_fp16 (metal.py:199-232, kernel 104-141; out_dtype TQ_F16).  TQ_BF16 also accepted.
 * Row addressing as in tq_encode, plus out_group_stride (rows of dim elements).
 */
int tq_dequant(const uint32_t* packed, const float* norms, const float* centroids,
               const float* signs, void* out, int out_dtype,
               int64_t n_groups, int64_t rows_per_group,
               int64_t packed_group_stride, int64_t norms_group_stride, int64_t out_group_stride,
               int dim, int bits, tq_stream_t stream);

/*
 * q_rot[h] = butterfly(q[h] * signs), no 1/sqrt(dim).
 * Replaces prerotate_query (metal_kernels_v4.py:119-150, kernel 37-62).
 *   q [n_heads, dim] dtype q_dtype -> q_rot [n_heads, dim] float32
 */
int tq_prerotate_query(const void* q, int q_dtype, const float* signs, float* q_rot,
                       int64_t n_heads, int dim, tq_stream_t stream);

/*
 * scores[h, p] = (sum_e c[idx[h/n_rep, p, e]] * q_rot[h, e]) * k_norms[h/n_rep, p] * (1/dim).
 * Replaces prerot_fused_qk_scores (metal_kernels_v4.py:153-221, kernel 71-113).
 *   q_rot [n_kv*n_rep, dim] f32; k_packed / k_norms: one sequence, head_stride in rows;
 *   scores [n_kv*n_rep, seq_len] f32 contiguous.
 * allow_mma = TQ_MMA_OFF (0): float32 vector arithmetic throughout (the reference's operation
 * order); TQ_MMA_FP16 (1): q_rot and the centroids are rounded to fp16 and multiplied on the matrix
 * cores with float32 accumulation (about 3e-4 relative per score); TQ_MMA_SPLIT (2): matrix cores
 * with every operand as an fp16 value plus the fp16 remainder of its rounding (three matrix
 * instructions per tile, products exact in float32: float32 fidelity, ~1e-6 relative, inside the
 * reference's own bar of 1e-4 absolute, tests/test_prerot.py:90-95).  The matrix-core forms need
 * d = 128, n_rep <= 16 (any width); other shapes run the float32 vector kernels whatever the flag.
 */
int tq_prerot_qk_scores(const float* q_rot, const uint32_t* k_packed, const float* k_norms,
                        const float* centroids, float* scores,
                        int n_kv_heads, int n_rep, int64_t seq_len,
                        int64_t packed_head_stride, int64_t norms_head_stride,
                        int dim, int bits, int allow_mma, tq_stream_t stream);

/*
 * scores[h, p] = <dequant(K[h, p]), query[h]>, one butterfly per K row (MHA only).
 * Replaces packed_fused_qk_scores (kernels.py:158-196, kernel 58-117); kept because the
 * reference uses it as the cross-check of the pre-rotated path (tests/test_prerot.py:81-88).
 */
int tq_packed_qk_scores(const float* query, const uint32_t* k_packed, const float* k_norms,
                        const float* centroids, const float* signs, float* scores,
                        int n_heads, int64_t seq_len,
                        int64_t packed_head_stride, int64_t norms_head_stride,
                        int dim, int bits, tq_stream_t stream);

/*
 * scores[h, p] = <q[h], K[h/n_rep, p]> * scale for fp16 keys (the K side of a V-only cache,
 * v_only_cache.py:24-38; the reference computes this inside the stock SDPA).
 *   q [n_kv*n_rep, dim] dtype q_dtype; k fp16 rows of dim halfs, head_stride in rows.
 */
int tq_dense_qk_scores(const void* q, int q_dtype, const void* k_f16, float* scores,
                       int n_kv_heads, int n_rep, int64_t seq_len, int64_t k_head_stride,
                       int dim, float scale, tq_stream_t stream);

/*
 * weights[r, :] = softmax(scores[r, :] * scale + mask[r * mask_row_stride, :]).
 * Replaces the `* attn_scale`, `+ mask`, mx.softmax steps of turboquant_attention
 * (fused_attention.py:78-94).  mask may be NULL; mask_row_stride is 0 for a mask shared by
 * all rows or seq_len for one row per score row.  In-place (weights == scores) is allowed.
 */
int tq_softmax_rows(const float* scores, const float* mask, int64_t mask_row_stride,
                    float* weights, int64_t n_rows, int64_t seq_len, float scale,
                    tq_stream_t stream);

/*
 * out[h] = butterfly(sum_{p: !(w[h,p] < thr)} w[h,p] * norm[h/n_rep,p] * c[idx[h/n_rep,p,:]])
 *          * signs * (1/dim),   thr = max(threshold, 0).
 * Replaces sparse_v_matvec (sparse_v.py:94-186, kernel 32-88).  KV positions are split
 * across workgroups; partial sums go through `workspace` and a second pass applies the one
 * butterfly.   weights [n_kv*n_rep, seq_len] f32; out [n_kv*n_rep, dim] f32.
 * allow_mma as in tq_prerot_qk_scores (TQ_MMA_FP16: weights * norm and centroids rounded to fp16;
 * TQ_MMA_SPLIT: both as value + remainder, within the reference's bar of 1e-5 of the largest
 * output, tests/test_sparse_v.py:70-75).
 */
int tq_sparse_v_matvec(const float* weights, const uint32_t* v_packed, const float* v_norms,
                       const float* centroids, const float* signs, float* out,
                       void* workspace, size_t workspace_bytes,
                       int n_kv_heads, int n_rep, int64_t seq_len,
                       int64_t packed_head_stride, int64_t norms_head_stride,
                       int dim, int bits, float threshold, int allow_mma, tq_stream_t stream);

/* Shapes and addressing shared by the two fused decode-attention entry points. */
typedef struct tq_decode_shape {
  int32_t n_seq;             /* sequences in the batch (>= 1) */
  int32_t n_kv_heads;
  int32_t n_rep;             /* query heads per kv head */
  int32_t dim;               /* head dimension */
  int32_t bits;
  int32_t block_size;        /* accepted for interface parity (1..32); the result does not depend on it */
  int64_t seq_len;           /* uniform length, or the maximum length when seq_offsets != NULL */
  const int32_t* seq_offsets;/* device, [n_seq+1], or NULL */
  int64_t k_seq_stride, k_head_stride;   /* rows; K packed and K fp16 share the row count */
  int64_t kn_seq_stride, kn_head_stride; /* K norms (unused by the V-only kernel) */
  int64_t v_seq_stride, v_head_stride;   /* V packed */
  int64_t vn_seq_stride, vn_head_stride; /* V norms */
  const float* mask;         /* optional additive mask, device, or NULL */
  int64_t mask_seq_stride;   /* floats between sequences */
  int64_t mask_head_stride;  /* floats between query heads (0 = shared) */
  float attn_scale;
  int32_t out_dtype;         /* TQ_F32, TQ_F16 or TQ_BF16 */
  int32_t allow_mma;         /* 1: use the fp16 matrix-core kernels where the shape allows (d = 128,
                                n_rep <= 16, every width 1-4; operands rounded to fp16, float32
                                accumulation);
                                0: float32 vector-ALU kernels only */
} tq_decode_shape;

/*
 * Single-pass SDPA for one query token per head over packed K and packed V, online softmax in
 * float32:  s = (sum_e c_k[idx_k] * q_rot) * k_norm * (1/dim) * attn_scale (+ mask),
 *           out = butterfly(sum_p e^{s-m} * v_norm * c_v[idx_v]) * v_signs * (1/dim) / l.
 * Replaces flash_attention_turboquant (flash_attention.py:168-274, kernel 36-163), extended
 * with a batch of sequences of ragged length.
 *   q_rot [n_seq, n_kv*n_rep, dim] f32;  out [n_seq, n_kv*n_rep, dim] out_dtype.
 */
int tq_flash_decode(const float* q_rot,
                    const uint32_t* k_packed, const float* k_norms,
                    const uint32_t* v_packed, const float* v_norms,
                    const float* k_centroids, const float* v_centroids, const float* v_signs,
                    void* out, void* workspace, size_t workspace_bytes,
                    const tq_decode_shape* shape /* host */, tq_stream_t stream);

/*
 * Which tile pass tq_flash_decode takes on the matrix-core path for a batch of this shape:
 * 0 = one workgroup per 512-position tile; n >= 2 = the streaming pass, one workgroup per
 * n * 256 consecutive positions (large unmasked batches).  Informational: lets a caller or a test
 * know which kernel a shape exercises.  No counterpart in the reference (one kernel per call,
 * flash_attention.py:168-274).  The plan sees no pointers: it describes three-bit tensors (rows at any
 * 4-byte offset) and tensors of widths 1, 2 and 4 that are 16-byte aligned; tq_flash_decode sends a
 * tensor of width 1, 2 or 4 at another offset to the tile pass whatever the plan says.
 */
int tq_flash_decode_plan(int n_seq, int n_kv_heads, int64_t max_seq_len, int ragged, int masked);

/*
 * Decode attention for a V-only cache: fp16 keys, packed values, dense softmax (threshold 0):
 *   out = butterfly(sum_p softmax_p(<q,K_p>*attn_scale + mask) * v_norm * c_v[idx_v]) * v_signs / dim.
 * The composition dense-K scores -> softmax -> sparse_v_matvec of hybrid_attention.py:52-88 /
 * fused_attention.py:50-121 in one launch for the cache of v_only_cache.py:24-127.
 *   q [n_seq, n_kv*n_rep, dim] dtype q_dtype;  k_f16 rows of dim halfs;  out as tq_flash_decode.
 * With allow_mma, d = 128 and n_rep <= 16 the tile pass runs on the matrix cores for values of every
 * width (bits 1-4, as adaptive.py:26 / v_only_cache.py:41 take them); other shapes take the float32 kernels.
 * Alignment: k_f16 16 bytes (TQ_ERR_ALIGN otherwise).  The matrix-core pass reads q in 16-byte pieces: a q
 * that is not 16-byte aligned (a view at an odd element offset) is served by the float32 kernels instead,
 * same result to their rounding, several times slower.
 */
int tq_vonly_decode_attn(const void* q, int q_dtype, const void* k_f16,
                         const uint32_t* v_packed, const float* v_norms,
                         const float* v_centroids, const float* v_signs,
                         void* out, void* workspace, size_t workspace_bytes,
                         const tq_decode_shape* shape /* host */, tq_stream_t stream);

/*
 * tq_vonly_decode_attn without a workspace argument and without any allocation.  No counterpart in the
 * reference (its runtime allocates every kernel output, e.g. sparse_v.py:169-185): this entry point is for
 * callers that cannot allocate device memory -- code under HIP-graph capture, tight serving loops,
 * harnesses that forbid it.  The per-tile partial sums that tq_vonly_decode_attn keeps in the caller's
 * workspace go to an array of TQ_STATIC_SCRATCH_BYTES bytes inside the library (one copy per GPU, held
 * until the process ends; its address is looked up on the first call on a device, so make that call
 * outside a capture).  Arguments, kernels and results are those of tq_vonly_decode_attn (bit-identical
 * output).  Fails with TQ_ERR_WORKSPACE when tq_workspace_bytes(TQ_OP_VONLY_DECODE, n_seq, n_q_heads,
 * seq_len, dim) exceeds TQ_STATIC_SCRATCH_BYTES (e.g. more than 8065 tiles of 256 positions x query heads
 * at dim 128).  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
 * streams, two threads) race; order them on one stream.  Nothing in the array has to be cleared
 * between calls -- every partial that a call's merge pass reads has been written by its tile pass.
 */
#define TQ_STATIC_SCRATCH_BYTES ((size_t)4 << 20)
int tq_vonly_decode_attn_static(const void* q, int q_dtype, const void* k_f16,
                                const uint32_t* v_packed, const float* v_norms,
                                const float* v_centroids, const float* v_signs,
                                void* out, const tq_decode_shape* shape /* host */, tq_stream_t stream);

/*
 * A V-only cache as the library sees it between two growths of its storage: what a caller fills in
 * once and reuses for every decode step (all four tensors share n_seq, n_kv_heads and t_alloc).
 */
typedef struct tq_vonly_cache_desc {
  void* k_f16;               /* [n_seq, n_kv_heads, t_alloc, dim] float16, device */
  void* v_raw;               /* [n_seq, n_kv_heads, t_alloc, dim] in the dtype of the new values, or NULL */
  uint32_t* v_packed;        /* [n_seq, n_kv_heads, t_alloc, pdim] */
  float* v_norms;            /* [n_seq, n_kv_heads, t_alloc] */
  const float* v_signs;      /* [dim], device */
  float boundaries[15];      /* 2^bits - 1 used */
  float centroids[16];       /* 2^bits used */
  void* workspace;           /* device, tq_workspace_bytes(TQ_OP_VONLY_DECODE, n_seq, n_q, t_alloc, dim) */
  size_t workspace_bytes;
  int64_t t_alloc;
  int32_t n_seq, n_kv_heads, n_rep, dim, bits;
  int32_t variant;           /* TQ_ENCODE_MLX / TQ_ENCODE_METAL */
  int32_t allow_mma;         /* as in tq_decode_shape */
} tq_vonly_cache_desc;

/*
 * One decode step of a V-only cache in one library call: ONE new token per sequence is inserted at
 * time index `position` and the query token attends over positions 0 .. position.  For dim 128
 * (values of any width, bits 1-4) and n_rep <= 16 that is two launches: the tile pass over positions 0 .. position - 1,
 * and a merge pass that encodes the new value row with the encoder's own arithmetic, scores the new
 * key, folds both in and stores the key row, the raw value row, the packed words and the norm (the
 * stored state is bit-identical to tq_vonly_append's, the output agrees with the two calls to the
 * rounding of one score); other shapes run tq_vonly_append followed by tq_vonly_decode_attn.
 * Replaces, for a single-token step, VOnlyTurboQuantCache.update_and_fetch followed by the
 * attention of hybrid_attention.py:52-88 / fused_attention.py:50-121 (v_only_cache.py:52-78).
 *   k_new, v_new [n_seq, n_kv_heads, dim];  q [n_seq, n_kv_heads*n_rep, dim];  out likewise, out_dtype
 * Fails with TQ_ERR_ARG when position is outside 0 .. t_alloc - 1.
 * Alignment: the two-launch path needs q and cache->k_f16 16-byte aligned; with another q (or k_f16) the
 * call runs tq_vonly_append followed by tq_vonly_decode_attn, whose own rules then apply.
 */
int tq_vonly_decode_step(const tq_vonly_cache_desc* cache /* host */,
                         const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                         const void* q, int q_dtype, void* out, int out_dtype,
                         int64_t position, float attn_scale, tq_stream_t stream);

/*
 * tq_vonly_append with the insert position read from DEVICE memory when the kernel runs: row (g, i)
 * goes to time index *position_dev + i of group g, the destination pointers point at time index 0
 * and all four tensors hold t_alloc positions per group; rows that would land outside 0 .. t_alloc - 1
 * are dropped.  For a decode step recorded once in a HIP graph and replayed while a device counter
 * advances; the reference's insert position is a host integer (cache.offset, v_only_cache.py:80-82).
 */
int tq_vonly_append_at(const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                       const float* v_signs, const float* boundaries,
                       void* k_f16, void* v_raw, uint32_t* v_packed, float* v_norms,
                       int64_t n_groups, int64_t rows_per_group, int64_t t_alloc,
                       int dim, int bits, int variant, const int64_t* position_dev, tq_stream_t stream);

/*
 * tq_vonly_decode_step with the position read from device memory: inserts ONE token per sequence at
 * *position_dev and attends over positions 0 .. *position_dev (clamped to the storage).  Grids and the
 * workspace are sized for t_alloc positions, so the same recorded launches serve every step until the
 * storage is reallocated; the caller advances the counter between steps (on the same stream).
 * dim 128 (values of any width), n_rep <= 16 and 16-byte aligned q and cache->k_f16 only (TQ_ERR_UNSUPPORTED
 * otherwise: there is no fallback that reads the position on the device); position_dev 8-byte aligned.
 */
int tq_vonly_decode_step_at(const tq_vonly_cache_desc* cache /* host */,
                            const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                            const void* q, int q_dtype, void* out, int out_dtype,
                            const int64_t* position_dev /* device */, float attn_scale, tq_stream_t stream);

/*
 * A cache with packed keys AND values as the library sees it between two growths of its storage
 * (all four tensors share n_seq, n_kv_heads and t_alloc; keys and values share dim and bits, hence
 * the tables, and differ in their sign vectors: seeds s and s + 1 of cache.py:92,96).
 */
typedef struct tq_packed_cache_desc {
  uint32_t* k_packed;        /* [n_seq, n_kv_heads, t_alloc, pdim] */
  float* k_norms;            /* [n_seq, n_kv_heads, t_alloc] */
  uint32_t* v_packed;
  float* v_norms;
  const float* k_signs;      /* [dim], device */
  const float* v_signs;
  float boundaries[15];      /* 2^bits - 1 used */
  float centroids[16];       /* 2^bits used */
  void* workspace;           /* device, tq_workspace_bytes(TQ_OP_FLASH_DECODE, n_seq, n_q, t_alloc, dim) */
  size_t workspace_bytes;
  int64_t t_alloc;
  int32_t n_seq, n_kv_heads, n_rep, dim, bits;
  int32_t variant;           /* TQ_ENCODE_MLX / TQ_ENCODE_METAL */
} tq_packed_cache_desc;

/*
 * One decode step of a packed cache in one library call: ONE new key and value row per sequence
 * and kv head is encoded and stored at time index `position` and the query token attends over
 * positions 0 .. position (no mask, no threshold).  Two launches: the packed tile pass over
 * positions 0 .. position - 1, and a merge pass that encodes both new rows with the encoder's own
 * arithmetic, rotates the query, scores the new key from its codes and folds both in (stored state
 * bit-identical to tq_encode's, output equal to the separate calls up to the rounding of one score).
 * Replaces, for a single-token step, TurboQuantKVCache.update_and_fetch (cache.py:131-165) followed
 * by turboquant_attention (fused_attention.py:20-125).  Shapes and errors as tq_vonly_decode_step;
 * TQ_ERR_UNSUPPORTED where tq_flash_decode_from_q has no kernel (it needs dim 128 and n_rep <= 16).
 */
int tq_packed_decode_step(const tq_packed_cache_desc* cache /* host */,
                          const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                          const void* q, int q_dtype, void* out, int out_dtype,
                          int64_t position, float attn_scale, tq_stream_t stream);

/*
 * tq_packed_decode_step with the position read from device memory (see tq_vonly_decode_step_at): encodes
 * the new key and value rows at *position_dev and attends over positions 0 .. *position_dev; grids and the
 * workspace are sized for t_alloc positions; an insert outside the storage is dropped.
 */
int tq_packed_decode_step_at(const tq_packed_cache_desc* cache /* host */,
                             const void* k_new, int k_dtype, const void* v_new, int v_dtype,
                             const void* q, int q_dtype, void* out, int out_dtype,
                             const int64_t* position_dev /* device */, float attn_scale, tq_stream_t stream);

/*
 * The same call with its two passes selectable: phases = 1 runs only the tile pass (per-tile
 * partial sums and softmax statistics into `workspace`), phases = 2 only the merge pass (workspace
 * -> out), phases = 3 both (= tq_vonly_decode_attn).  For callers that time or overlap the passes;
 * the reference has a single kernel per call (sparse_v.py:169-185) and no counterpart to the split.
 */
int tq_vonly_decode_attn_phases(const void* q, int q_dtype, const void* k_f16,
                                const uint32_t* v_packed, const float* v_norms,
                                const float* v_centroids, const float* v_signs,
                                void* out, void* workspace, size_t workspace_bytes,
                                const tq_decode_shape* shape /* host */, int phases, tq_stream_t stream);

/*
 * Decode attention for a V-only cache with the sparse-V threshold: weights of the softmax over the whole
 * sequence that are below `threshold` contribute nothing,
 *   w_p = softmax_p(<q,K_p>*attn_scale + mask);   out = butterfly(sum_{p: !(w_p < threshold)} w_p * v_norm * c_v[idx_v]) * v_signs / dim,
 * i.e. dense-K scores -> softmax -> sparse_v_matvec(threshold) of hybrid_attention.py:52-88 (threshold rule of
 * sparse_v.py:59-65, 163-164; the call with sparse_v_threshold of fused_attention.py:109-121) in one call:
 * a scores pass, a weights-and-values pass and the merge pass, with the scores of the step held in `workspace`
 * (tq_vonly_sparse_workspace_bytes) instead of three tensors of the caller.  Arguments as tq_vonly_decode_attn;
 * threshold >= 0 (0 = dense: every position contributes).  Rows whose positions are all masked out yield zeros.
 * Matrix-core shape only: dim 128, values of any width (bits 1-4), n_rep <= 16, non-empty cache, 16-byte
 * aligned q (TQ_ERR_UNSUPPORTED otherwise: compose tq_dense_qk_scores, tq_softmax_rows and tq_sparse_v_matvec
 * for those); k_f16 16-byte aligned (TQ_ERR_ALIGN otherwise).
 */
int tq_vonly_sparse_decode_attn(const void* q, int q_dtype, const void* k_f16,
                                const uint32_t* v_packed, const float* v_norms,
                                const float* v_centroids, const float* v_signs, float threshold,
                                void* out, void* workspace, size_t workspace_bytes,
                                const tq_decode_shape* shape /* host */, tq_stream_t stream);

size_t tq_vonly_sparse_workspace_bytes(int n_seq, int n_q_heads, int64_t max_seq_len);

/*
 * The thresholded decode step over packed keys AND packed values: turboquant_attention with
 * sparse_v_threshold > 0 (fused_attention.py:70-121: prerot_fused_qk_scores -> * attn_scale + mask -> softmax
 * -> sparse_v_matvec(threshold)) in one call of three passes, for batches and ragged lengths as
 * tq_flash_decode.  q_rot is the pre-rotated query (tq_prerotate_query).  Workspace:
 * tq_vonly_sparse_workspace_bytes (same layout).  Same shape limits and error as tq_vonly_sparse_decode_attn
 * (compose tq_prerot_qk_scores, tq_softmax_rows and tq_sparse_v_matvec for other shapes).
 */
int tq_flash_sparse_decode(const float* q_rot,
                           const uint32_t* k_packed, const float* k_norms,
                           const uint32_t* v_packed, const float* v_norms,
                           const float* k_centroids, const float* v_centroids, const float* v_signs,
                           float threshold, void* out, void* workspace, size_t workspace_bytes,
                           const tq_decode_shape* shape /* host */, tq_stream_t stream);

/*
 * turboquant_attention in one call, from the query itself (fused_attention.py:56-121: prerotate_query ->
 * prerot_fused_qk_scores -> * attn_scale + mask -> softmax -> sparse_v_matvec): tq_flash_decode
 * (threshold == 0) or tq_flash_sparse_decode (threshold > 0) with the pre-rotation q_rot = butterfly(q * k_signs)
 * of tq_prerotate_query done inside the kernels (same bits), which saves the separate launch and the q_rot
 * tensor.  q [n_seq, n_kv*n_rep, dim] of q_dtype; k_signs [dim] f32 on the device.  Workspace:
 * tq_workspace_bytes(TQ_OP_FLASH_DECODE, ...) for threshold == 0, tq_vonly_sparse_workspace_bytes otherwise.
 * Matrix-core shape only (dim 128, n_rep <= 16, non-empty cache; TQ_ERR_UNSUPPORTED otherwise: call
 * tq_prerotate_query and tq_flash_decode).
 */
int tq_flash_decode_from_q(const void* q, int q_dtype, const float* k_signs,
                           const uint32_t* k_packed, const float* k_norms,
                           const uint32_t* v_packed, const float* v_norms,
                           const float* k_centroids, const float* v_centroids, const float* v_signs,
                           float threshold, void* out, void* workspace, size_t workspace_bytes,
                           const tq_decode_shape* shape /* host */, tq_stream_t stream);

/*
 * Bytes of workspace the op needs for this shape (host computation, no GPU call).  The workspace
 * holds per-tile partial results between the two passes of a call; its contents need not be
 * preserved or cleared between calls.  Calls that share a workspace must be ordered (same stream);
 * concurrent calls need separate workspaces.
 */
size_t tq_workspace_bytes(int op, int n_seq, int n_q_heads, int64_t max_seq_len, int dim);

/*
 * Chunked-prefill attention: n_rows query rows per q head (positions q_pos0 .. q_pos0 + n_rows - 1)
 * against kv_len cached positions held PACKED (K and V), causal when `causal` != 0 (row i sees
 * positions <= q_pos0 + i).  No kernel of the reference does this: its prefill dequantises the
 * whole cache to fp16 and runs stock SDPA over it (cache.py:125-129, 209-210 feeding
 * mlx-lm's scaled_dot_product_attention); the arithmetic here is flash_attention.py:79-162
 * (rotated-domain scores and value sum, one butterfly per output row) applied to many rows.
 *   q   [n_kv*n_rep, n_rows, dim] q_dtype, contiguous, NOT pre-rotated (k_signs are applied here)
 *   k_packed / v_packed [n_kv, *_head_stride rows, pdim], k_norms / v_norms [n_kv, *_head_stride]
 *   out [n_kv*n_rep, n_rows, dim] out_dtype, contiguous
 * Matrix-core kernel: q_rot, the centroids and softmax weights * value norm are fp16 operands,
 * accumulation is float32.  dim 128 only, every width (TQ_ERR_UNSUPPORTED otherwise).  The workspace
 * (tq_prefill_workspace_bytes, 256-byte aligned) is scratch as for the decode ops.
 * flags: TQ_PREFILL_CAUSAL (row i sees positions <= q_pos0 + i); TQ_PREFILL_FP16_QUERY: the rotated
 * query enters as ONE fp16 number per element instead of value + remainder (a third fewer matrix
 * instructions).  The logit error of that rounding (~4e-4) is harmless on ordinary data but reaches
 * 1e-2 of an output row when an outlier channel of V cancels in the average, so it is off unless
 * the caller sets it.
 */
enum tq_prefill_flags { TQ_PREFILL_CAUSAL = 1, TQ_PREFILL_FP16_QUERY = 2 };

int tq_prefill_attn(const void* q, int q_dtype,
                    const uint32_t* k_packed, const float* k_norms,
                    const uint32_t* v_packed, const float* v_norms,
                    const float* k_centroids /* host */, const float* v_centroids /* host */,
                    const float* k_signs, const float* v_signs,
                    void* out, int out_dtype, void* workspace, size_t workspace_bytes,
                    int n_kv_heads, int n_rep, int64_t n_rows, int64_t kv_len, int64_t q_pos0,
                    int64_t k_head_stride, int64_t kn_head_stride,
                    int64_t v_head_stride, int64_t vn_head_stride,
                    int dim, int bits, float attn_scale, int flags, tq_stream_t stream);

size_t tq_prefill_workspace_bytes(int n_q_heads, int64_t n_rows, int64_t kv_len, int dim);

/*
 * Measurement aid, no counterpart in the reference (its benches time whole kernels with mx.eval,
 * scripts/bench_sparse_v.py:49-57): ONE launch that streams `bytes` bytes from `src` (16-byte aligned,
 * a multiple of 16) through n_workgroups workgroups (256 threads with eight loads in flight each; 512 threads with
 * every load requested up front when a workgroup's share is between 32 and 160 KB) -- the practical ceiling for a launch
 * that reads this much on the machine at hand, launch overhead and tail included.  With
 * store_bytes_per_workgroup > 0 (a multiple of 16, at most 4096) every workgroup ends with a store of that
 * many bytes at sink + 16 + workgroup * store_bytes_per_workgroup, as a split-KV tile pass ends with the
 * store of its partial result; `sink` (device, 16-byte aligned) must then hold 16 + n_workgroups *
 * store_bytes_per_workgroup bytes, else 4 bytes suffice (never written in practice) and it may be NULL.
 * bytes == 0 launches an empty kernel (the cost of a launch alone).  bench.py --calibrate-read times these
 * beside the decode step.
 */
int tq_probe_read(const void* src, size_t bytes, uint32_t* sink, int n_workgroups,
                  size_t store_bytes_per_workgroup, tq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TQHIP_H */
