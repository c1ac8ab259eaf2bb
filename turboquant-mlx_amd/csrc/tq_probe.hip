// Measurement aids of the library: a plain streaming read and an empty launch.  They give the
// practical ceiling for ONE launch that reads a given number of bytes on the machine at hand (launch
// overhead, ramp-up and tail included), which is what a decode step of a few tens of megabytes is
// measured against; they take no part in any result.
#include "tq_common.h"

namespace {

constexpr int kProbeThreads = 256;
constexpr int kProbeUnroll = 8;
constexpr int kProbeWideThreads = 512;   // the shape of a decode tile pass: one pass, every load of a thread
constexpr int kProbeWideUnroll = 20;     // requested up front (512 threads x 20 x 16 B = 160 KB per workgroup)

// every workgroup reads one contiguous slice in 16-byte pieces, kProbeUnroll loads in flight per thread;
// the xor of everything read is stored only if it equals a value it cannot have by construction of the test
// buffers' use (the store keeps the loads alive, the branch keeps the write out of the traffic)
// store16 > 0: every workgroup ends with a store of store16 16-byte pieces (derived from what it read) at
// sink + 16 + workgroup * store16 * 16, as a tile pass ends with the store of its partial result.
template <int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void probe_read_kernel(const uint4* __restrict__ p, size_t n16,
                                                             uint32_t* __restrict__ sink, int store16) {
  const size_t per_wg = (n16 + gridDim.x - 1) / gridDim.x;
  const size_t b = (size_t)blockIdx.x * per_wg;
  const size_t e = b + per_wg < n16 ? b + per_wg : n16;
  uint32_t acc = 0;
  for (size_t i = b + threadIdx.x; i < e; i += (size_t)THREADS * UNROLL) {
    uint4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const size_t j = i + (size_t)u * THREADS;
      if (j < e) {                                             // streaming loads, as the decode kernels read K and V
        typedef uint32_t piece_t __attribute__((ext_vector_type(4)));
        const piece_t w = __builtin_nontemporal_load(reinterpret_cast<const piece_t*>(p + j));
        v[u] = make_uint4(w[0], w[1], w[2], w[3]);
      } else {
        v[u] = make_uint4(0, 0, 0, 0);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9E3779B9u && sink) sink[0] = acc;
  if ((int)threadIdx.x < store16)
    reinterpret_cast<uint4*>(sink + 4)[(size_t)blockIdx.x * store16 + threadIdx.x] = make_uint4(acc, 0u, 0u, 0u);
}

__global__ void probe_empty_kernel(uint32_t* sink) {
  if (sink == reinterpret_cast<uint32_t*>(1)) sink[0] = 1;
}

}  // namespace

extern "C" int tq_probe_read(const void* src, size_t bytes, uint32_t* sink, int n_workgroups,
                             size_t store_bytes_per_workgroup, tq_stream_t stream_) {
  if (bytes == 0) {
    probe_empty_kernel<<<1, 64, 0, (hipStream_t)stream_>>>(sink);
    TQ_CHECK_LAUNCH("tq_probe_read (empty launch)");
    return TQ_OK;
  }
  if (!src) return tq::fail(TQ_ERR_NULL, "tq_probe_read: null pointer");
  if (!tq::aligned(src, 16) || bytes % 16) return tq::fail(TQ_ERR_ALIGN, "tq_probe_read: src and bytes must be multiples of 16");
  if (n_workgroups < 1 || n_workgroups > 65535) return tq::fail(TQ_ERR_ARG, "tq_probe_read: n_workgroups must be in 1..65535");
  if (store_bytes_per_workgroup % 16 || store_bytes_per_workgroup > (size_t)kProbeThreads * 16)
    return tq::fail(TQ_ERR_ARG, "tq_probe_read: store_bytes_per_workgroup must be a multiple of 16 up to %d", kProbeThreads * 16);
  if (store_bytes_per_workgroup && (!sink || !tq::aligned(sink, 16)))
    return tq::fail(TQ_ERR_ALIGN, "tq_probe_read: a sink for stores must be 16-byte aligned");
  // workgroups with more than one pass of the narrow shape (32 KB) and at most 160 KB each take the launch shape of a
  // decode tile pass (512 threads, everything requested up front); otherwise 256 threads, eight loads in flight each
  const size_t per_wg = (bytes / 16 + n_workgroups - 1) / n_workgroups * 16;
  if (per_wg > (size_t)kProbeThreads * kProbeUnroll * 16 && per_wg <= (size_t)kProbeWideThreads * kProbeWideUnroll * 16)
    probe_read_kernel<kProbeWideThreads, kProbeWideUnroll><<<n_workgroups, kProbeWideThreads, 0, (hipStream_t)stream_>>>(
        (const uint4*)src, bytes / 16, sink, (int)(store_bytes_per_workgroup / 16));
  else
    probe_read_kernel<kProbeThreads, kProbeUnroll><<<n_workgroups, kProbeThreads, 0, (hipStream_t)stream_>>>(
        (const uint4*)src, bytes / 16, sink, (int)(store_bytes_per_workgroup / 16));
  TQ_CHECK_LAUNCH("tq_probe_read");
  return TQ_OK;
}
