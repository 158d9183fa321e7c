// Measurement probe (not part of the attention ABI): what does a pure gather of 16 KiB KV
// pages sustain on this machine, with the decode kernel's access pattern and nothing else?
// 512-thread workgroups; workgroup b walks pages table[b * pages_per_wg ..] four at a time,
// from a K pool and a V pool; wave w reads its 128-byte slice (KV head w) of each of a page's
// 16 token rows with two 16-byte loads per lane, as attend() does, and XORs what arrives
// (`whole_rows` instead gives each wave two whole 1 KiB token rows of a page: the pattern a
// kernel staging pages through LDS could use).
// `delay` dependent integer multiply-adds per wave and batch stand in for the kernel's own
// arithmetic per 64-token chunk (one link is ~36 core cycles).  A table of consecutive page
// ids turns the gather into a linear read of the pools.  `lds_bytes` of dynamic LDS (unused)
// set how many workgroups a CU holds: 75 KiB gives the decode kernel's two.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

template <bool NT>
__device__ __forceinline__ u32x4 ld16(const uint8_t *p) {
  if (NT) return __builtin_nontemporal_load((const u32x4 *)p);  // (streaming: no reuse expected)
  return *(const u32x4 *)p;
}

template <bool ROWS, bool NT>
__device__ __forceinline__ void load_batch(const uint8_t *pool, const int *tb, const int p0,
                                           const int n, const int lane, const int wave,
                                           u32x4 (&r)[8]) {
  const int i16 = lane & 15, g = lane >> 4;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int page = tb[p0 + (b < n ? b : n - 1)];  // (clamped: every load is issued)
    if (ROWS) {  // wave w takes token rows 2w, 2w+1 whole: 1 KiB contiguous per load instruction
      const size_t off = (size_t)page * 16384 + wave * 2048 + lane * 16;
      r[2 * b] = ld16<NT>(pool + off);
      r[2 * b + 1] = ld16<NT>(pool + off + 1024);
    } else {  // wave w takes KV head w of all 16 rows: 16 slices of 128 bytes, 1 KiB apart
      const size_t off = (size_t)page * 16384 + i16 * 1024 + wave * 128 + g * 32;
      r[2 * b] = ld16<NT>(pool + off);
      r[2 * b + 1] = ld16<NT>(pool + off + 16);
    }
  }
}

template <bool ROWS, bool NT>
__global__ __launch_bounds__(512, 4) void gather_probe_kernel(const uint8_t *k, const uint8_t *v,
                                                              const int *table, const int pages_per_wg,
                                                              const int delay, uint32_t *sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int *tb = table + (size_t)blockIdx.x * pages_per_wg;
  uint32_t acc = 0;
  for (int p0 = 0; p0 < pages_per_wg; p0 += 4) {
    const int n = min(4, pages_per_wg - p0);
    u32x4 a[8], b[8];
    load_batch<ROWS, NT>(k, tb, p0, n, lane, wave, a);
    load_batch<ROWS, NT>(v, tb, p0, n, lane, wave, b);
    uint32_t x = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) x ^= a[i][0] ^ a[i][1] ^ a[i][2] ^ a[i][3] ^ b[i][0] ^ b[i][1] ^ b[i][2] ^ b[i][3];
    for (int i = 0; i < delay; ++i) x = x * 1664525u + 1013904223u;
    acc ^= x;
  }
  if (acc == 0x12345678u) sink[0] = acc;  // (keeps the loads alive)
}

}  // namespace

// k, v: pools of 16 KiB pages; table: nwg * pages_per_wg page ids (device); sink: one word.
extern "C" int eid_probe_gather(const void *k, const void *v, const int *table, int nwg,
                                int pages_per_wg, int delay, int lds_bytes, int whole_rows,
                                unsigned *sink, void *stream) {
  if (nwg < 1 || pages_per_wg < 1 || delay < 0 || lds_bytes < 0 || lds_bytes > 160 * 1024) return -1;
  // whole_rows: 0 head slices, 1 whole rows, 2 whole rows with non-temporal loads, 3 head slices with them
  auto kern = whole_rows == 1 ? gather_probe_kernel<true, false> : whole_rows == 2 ? gather_probe_kernel<true, true>
              : whole_rows == 3 ? gather_probe_kernel<false, true> : gather_probe_kernel<false, false>;
  if (lds_bytes > 64 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                          lds_bytes) != hipSuccess)
    return -4;
  kern<<<nwg, 512, lds_bytes, static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint8_t *>(k), static_cast<const uint8_t *>(v), table, pages_per_wg, delay, sink);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}
