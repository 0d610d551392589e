// Measurement aid: the memory traffic of the pack kernel with no arithmetic.
// Every lane reads 64 bytes of an fp32 stream (four 16-byte loads, a load
// instruction covering 1 KB contiguous per wavefront) and writes 0, 2, 4, 8 or
// 16 bytes (what 1, 2, 4, 8 bits per element pack 16 elements into), coalesced.
// What this kernel reaches is what the memory system of the device delivers
// for that mix of reads and writes: the bar the pack kernel is held against.

#include "exact_common.hpp"

namespace exact {

template <int OUT_BYTES>
__global__ __launch_bounds__(kBlock) void stream_probe_kernel(const f32x4* __restrict__ in, uint8_t* __restrict__ out) {
  constexpr int kQuads = 4;  // 16-byte loads per lane
  const int t = threadIdx.x;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kBlock * kQuads);
  f32x4 v[kQuads];
#pragma unroll
  for (int u = 0; u < kQuads; ++u) v[u] = __builtin_nontemporal_load(in + base + u * kBlock + t);
  uint32_t w = 0;
#pragma unroll
  for (int u = 0; u < kQuads; ++u)
    w ^= __float_as_uint(v[u].x) ^ __float_as_uint(v[u].y) ^ __float_as_uint(v[u].z) ^ __float_as_uint(v[u].w);
  const int64_t lane_id = static_cast<int64_t>(blockIdx.x) * kBlock + t;
  if constexpr (OUT_BYTES == 0) {
    // keeps the loads alive; a word of these bits does not come out of finite inputs in practice, and the
    // store is to valid memory if it does
    if (w == 0x7FC12345u) *reinterpret_cast<uint32_t*>(out) = w;
  } else if constexpr (OUT_BYTES == 2) {
    reinterpret_cast<uint16_t*>(out)[lane_id] = static_cast<uint16_t>(w);
  } else if constexpr (OUT_BYTES == 4) {
    reinterpret_cast<uint32_t*>(out)[lane_id] = w;
  } else if constexpr (OUT_BYTES == 8) {
    reinterpret_cast<uint2*>(out)[lane_id] = make_uint2(w, ~w);
  } else {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 q = {w, ~w, w + 1u, w - 1u};
    reinterpret_cast<u32x4*>(out)[lane_id] = q;
  }
}

}  // namespace exact

using namespace exact;

extern "C" int exact_stream_probe_f32(const float* x, int64_t n, int out_bytes, void* out, void* stream) {
  if (n < 0 || n > (int64_t{1} << 40)) return EXACT_E_SHAPE;
  if (out_bytes != 0 && out_bytes != 2 && out_bytes != 4 && out_bytes != 8 && out_bytes != 16) return EXACT_E_ARG;
  const int64_t tiles = n / (kBlock * 16);  // whole workgroup tiles of 4096 floats; the rest is not touched
  if (tiles == 0) return EXACT_OK;
  if (!x || !out) return EXACT_E_NULL;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15u) return EXACT_E_ALIGN;
  if (tiles > 0x7FFFFFFF) return EXACT_E_SHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tiles));
  const f32x4* in = reinterpret_cast<const f32x4*>(x);
  uint8_t* o = static_cast<uint8_t*>(out);
  switch (out_bytes) {
    case 0: hipLaunchKernelGGL(stream_probe_kernel<0>, grid, dim3(kBlock), 0, s, in, o); break;
    case 2: hipLaunchKernelGGL(stream_probe_kernel<2>, grid, dim3(kBlock), 0, s, in, o); break;
    case 4: hipLaunchKernelGGL(stream_probe_kernel<4>, grid, dim3(kBlock), 0, s, in, o); break;
    case 8: hipLaunchKernelGGL(stream_probe_kernel<8>, grid, dim3(kBlock), 0, s, in, o); break;
    default: hipLaunchKernelGGL(stream_probe_kernel<16>, grid, dim3(kBlock), 0, s, in, o); break;
  }
  return launch_status();
}
