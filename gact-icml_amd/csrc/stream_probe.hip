// Compute-free kernels with the memory traffic of the quantize and dequantize kernels: what this GPU's memory system gives a
// read stream with a minority of writes (and the reverse) when nothing else is in the way.  Measurement aids for bench.py -
// the compression library does not use them.
//
//   quantize-like:   a wave reads IN_KB KB with 16-byte loads and writes OUT_DW dwords per lane (256 * OUT_DW bytes), both
//                    contiguous per wave: 8 float groups are 8 KB in and 256 * bits bytes out, 8 half groups 4 KB in.
//   dequantize-like: a wave reads IN_DW dwords per lane and then writes OUT_KB KB with 16-byte stores through the policy the
//                    dequantize kernels use (nontemporal, written through): 8 float groups are 256 * bits bytes in and 8 KB out.
// The values written depend on the values read, so that no load can be dropped.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

// the tile order of the library's kernels: each of the 8 XCDs gets runs of consecutive tiles
__device__ __forceinline__ uint32_t xcd_tile(uint32_t b, uint32_t nb, uint32_t run) {
  const uint32_t round = 8 * run;
  if (b >= nb / round * round) return b;
  const uint32_t q = b / 8, x = b % 8;
  return ((q / run) * 8 + x) * run + q % run;
}

template <int N>
__device__ __forceinline__ void load_dwords(const uint8_t* p, uint32_t (&c)[N]) {
  if constexpr (N == 1) {
    c[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
  } else if constexpr (N == 2) {
    const u32x2 q = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    c[0] = q.x; c[1] = q.y;
  } else {
#pragma unroll
    for (int j = 0; j < N / 4; j++) {
      const u32x4 q = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p) + j);
      c[4 * j] = q.x; c[4 * j + 1] = q.y; c[4 * j + 2] = q.z; c[4 * j + 3] = q.w;
    }
  }
}
template <int N>
__device__ __forceinline__ void store_dwords(uint8_t* p, const uint32_t (&c)[N]) {
  if constexpr (N == 1) {
    __builtin_nontemporal_store(c[0], reinterpret_cast<uint32_t*>(p));
  } else if constexpr (N == 2) {
    __builtin_nontemporal_store(u32x2{c[0], c[1]}, reinterpret_cast<u32x2*>(p));
  } else {
#pragma unroll
    for (int j = 0; j < N / 4; j++)
      __builtin_nontemporal_store(u32x4{c[4 * j], c[4 * j + 1], c[4 * j + 2], c[4 * j + 3]}, reinterpret_cast<u32x4*>(p) + j);
  }
}

template <int IN_KB, int OUT_DW>
__global__ void __launch_bounds__(256)
quantize_like_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int64_t tiles) {
  const int64_t t = (int64_t)xcd_tile(blockIdx.x, gridDim.x, 128) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (t >= tiles) return;
  const int lane = threadIdx.x & 63;
  u32x4 v[IN_KB];
#pragma unroll
  for (int k = 0; k < IN_KB; k++)
    v[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(in + t * (IN_KB * 1024) + k * 1024 + lane * 16));
  uint32_t o[OUT_DW];
#pragma unroll
  for (int j = 0; j < OUT_DW; j++) o[j] = 0;
#pragma unroll
  for (int k = 0; k < IN_KB; k++) {
    o[(4 * k + 0) % OUT_DW] = (o[(4 * k + 0) % OUT_DW] << 1) ^ v[k].x;
    o[(4 * k + 1) % OUT_DW] = (o[(4 * k + 1) % OUT_DW] << 1) ^ v[k].y;
    o[(4 * k + 2) % OUT_DW] = (o[(4 * k + 2) % OUT_DW] << 1) ^ v[k].z;
    o[(4 * k + 3) % OUT_DW] = (o[(4 * k + 3) % OUT_DW] << 1) ^ v[k].w;
  }
  store_dwords<OUT_DW>(out + t * (256 * OUT_DW) + lane * 4 * OUT_DW, o);
}

template <int IN_DW, int OUT_KB>
__global__ void __launch_bounds__(256)
dequantize_like_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int64_t tiles) {
  const int64_t t = (int64_t)xcd_tile(blockIdx.x, gridDim.x, 16) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (t >= tiles) return;
  const int lane = threadIdx.x & 63;
  uint32_t c[IN_DW];
  load_dwords<IN_DW>(in + t * (256 * IN_DW) + lane * 4 * IN_DW, c);
  uint8_t* base = out + t * (OUT_KB * 1024);
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(base, 0, OUT_KB * 1024, 0x00020000);
#pragma unroll
  for (int k = 0; k < OUT_KB; k++) {
    const u32x4 v = {c[k % IN_DW] + (uint32_t)k, c[(k + 1) % IN_DW], c[0] ^ (uint32_t)k, c[IN_DW - 1] + 7u};
    __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, k * 1024 + lane * 16, 0, 19 /* sc0 sc1 nt */);
  }
}

template <int IN_KB>
int launch_quantize_like(int out_dw, const uint8_t* in, uint8_t* out, int64_t tiles, hipStream_t s) {
  const dim3 grid((unsigned)((tiles + 3) / 4)), block(256);
  switch (out_dw) {
    case 1: hipLaunchKernelGGL((quantize_like_kernel<IN_KB, 1>), grid, block, 0, s, in, out, tiles); break;
    case 2: hipLaunchKernelGGL((quantize_like_kernel<IN_KB, 2>), grid, block, 0, s, in, out, tiles); break;
    case 4: hipLaunchKernelGGL((quantize_like_kernel<IN_KB, 4>), grid, block, 0, s, in, out, tiles); break;
    case 8: hipLaunchKernelGGL((quantize_like_kernel<IN_KB, 8>), grid, block, 0, s, in, out, tiles); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -4;
}
template <int OUT_KB>
int launch_dequantize_like(int in_dw, const uint8_t* in, uint8_t* out, int64_t tiles, hipStream_t s) {
  const dim3 grid((unsigned)((tiles + 3) / 4)), block(256);
  switch (in_dw) {
    case 1: hipLaunchKernelGGL((dequantize_like_kernel<1, OUT_KB>), grid, block, 0, s, in, out, tiles); break;
    case 2: hipLaunchKernelGGL((dequantize_like_kernel<2, OUT_KB>), grid, block, 0, s, in, out, tiles); break;
    case 4: hipLaunchKernelGGL((dequantize_like_kernel<4, OUT_KB>), grid, block, 0, s, in, out, tiles); break;
    case 8: hipLaunchKernelGGL((dequantize_like_kernel<8, OUT_KB>), grid, block, 0, s, in, out, tiles); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

}  // namespace

extern "C" {

// Reads in_bytes / (in_kb * 1024) whole tiles of `in` (in_kb: 4 or 8) and writes 256 * out_dwords bytes per tile to `out`
// (out_dwords: 1, 2, 4 or 8), both 16-byte aligned.  Returns 0, -1 for arguments it does not know, -4 for a failed launch.
int gact_probe_quantize_like(const void* in, void* out, int64_t in_bytes, int in_kb, int out_dwords, void* stream) {
  if (!in || !out || in_bytes < 0 || ((uintptr_t)in & 15u) || ((uintptr_t)out & 15u)) return -1;
  if (in_kb != 4 && in_kb != 8) return -1;
  const int64_t tiles = in_bytes / (in_kb * 1024);
  if (tiles == 0) return 0;
  if (tiles > 0x7fffffffLL) return -1;
  (void)hipGetLastError();
  return in_kb == 4 ? launch_quantize_like<4>(out_dwords, (const uint8_t*)in, (uint8_t*)out, tiles, (hipStream_t)stream)
                    : launch_quantize_like<8>(out_dwords, (const uint8_t*)in, (uint8_t*)out, tiles, (hipStream_t)stream);
}

// Writes out_bytes / (out_kb * 1024) whole tiles of `out` (out_kb: 4 or 8), reading 256 * in_dwords bytes of `in` per tile
// (in_dwords: 1, 2, 4 or 8) first.
int gact_probe_dequantize_like(const void* in, void* out, int64_t out_bytes, int in_dwords, int out_kb, void* stream) {
  if (!in || !out || out_bytes < 0 || ((uintptr_t)in & 15u) || ((uintptr_t)out & 15u)) return -1;
  if (out_kb != 4 && out_kb != 8) return -1;
  const int64_t tiles = out_bytes / (out_kb * 1024);
  if (tiles == 0) return 0;
  if (tiles > 0x7fffffffLL) return -1;
  (void)hipGetLastError();
  return out_kb == 4 ? launch_dequantize_like<4>(in_dwords, (const uint8_t*)in, (uint8_t*)out, tiles, (hipStream_t)stream)
                     : launch_dequantize_like<8>(in_dwords, (const uint8_t*)in, (uint8_t*)out, tiles, (hipStream_t)stream);
}

}  // extern "C"
