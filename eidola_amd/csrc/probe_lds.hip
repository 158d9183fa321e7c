// Measurement probe (not part of the attention ABI): what do 16-byte LDS reads in the MFMA
// fragment pattern sustain per CU?  Every wave reads 16 KiB per iteration with ds_read_b128
// (lane (i16, g) = (lane % 16, lane / 16) takes 16 bytes of row i16 of a 16-row tile) from its
// own 2 KiB slice of a 96 KiB array, in one of three layouts:
//   0  linear: lane l reads bytes 16 l .. 16 l + 15 (the best the port can do)
//   1  128-byte rows, the row's 16-byte segments permuted by (row / 2) % 8 (the layout the
//      direct global -> LDS loads of the projection and prefill kernels write)
//   2  144-byte rows, unpermuted (the padded layout of the register-staged kernels)
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
constexpr int kLdsBytes = 96 * 1024;

template <int MODE>
__global__ __launch_bounds__(1024) void lds_probe_kernel(uint32_t *sink, const int iters) {
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < kLdsBytes / 4; i += blockDim.x) ((uint32_t *)lds)[i] = i;
  __syncthreads();
  const int i16 = lane & 15, g = lane >> 4;
  const uint32_t off = MODE == 0   ? lane * 16
                       : MODE == 1 ? i16 * 128 + ((g ^ ((i16 >> 1) & 7)) * 16)
                                   : i16 * 144 + g * 16;
  const uint8_t *p = lds + off + (tid >> 6) * 2048;
  u32x4 acc = {0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const u32x4 v = *(const u32x4 *)(p + ((j + it) & 7) * 4096);  // (the address moves: no hoisting)
      acc[0] ^= v[0];
      acc[1] ^= v[1];
      acc[2] ^= v[2];
      acc[3] ^= v[3];
    }
    asm volatile("" ::"v"(acc[0]));
  }
  if (acc[0] == 0x12345u && acc[1] == 7u && acc[2] == 9u && acc[3] == 11u) sink[0] = 1;
}

}  // namespace

// One workgroup of `threads` (256, 512 or 1024) per CU, `iters` iterations of 16 reads per wave.
extern "C" int eid_probe_lds_read(int mode, int nwg, int threads, int iters, unsigned *sink, void *stream) {
  if (mode < 0 || mode > 2 || nwg < 1 || threads < 64 || threads > 1024 || threads % 64 || iters < 1) return -1;
  auto kern = mode == 0 ? lds_probe_kernel<0> : mode == 1 ? lds_probe_kernel<1> : lds_probe_kernel<2>;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                          kLdsBytes) != hipSuccess)
    return -4;
  kern<<<nwg, threads, kLdsBytes, static_cast<hipStream_t>(stream)>>>(sink, iters);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}
