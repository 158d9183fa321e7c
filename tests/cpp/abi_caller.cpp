// A C++ caller of the C ABI, with no Python and no torch in the process: reads one decode
// batch from a file, writes the new K/V rows with eid_kv_write, attends with eid_attn_decode
// and writes the attention output and the touched cache rows back to a file.  Built by
// tests/cpp/Makefile; tests/test_gpu_cpp_caller.py prepares the input and checks the output
// against the CPU oracle.
//
// Input file: int32 header {num_seqs, max_blocks_per_seq, num_blocks, window, max_kv_len},
// then q [S,64,64] bf16, k_new / v_new [S,8,64] bf16, k_cache / v_cache [num_blocks,16,8,64] bf16,
// block_table [S,max_blocks] i32, seq_lens [S] i32, slot_mapping [S] i64, sinks [64] f32.
// Output file: out [S,64,64] bf16, then the S written K rows and the S written V rows.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "eidola_attn.h"

#define HIP_OK(x)                                                                    \
  do {                                                                               \
    hipError_t e_ = (x);                                                             \
    if (e_ != hipSuccess) {                                                          \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                   \
      return 2;                                                                      \
    }                                                                                \
  } while (0)
#define EID_CHECK(x)                                                                 \
  do {                                                                               \
    if ((x) != EID_OK) {                                                             \
      std::fprintf(stderr, "%s: %s\n", #x, eid_last_error());                        \
      return 3;                                                                      \
    }                                                                                \
  } while (0)

template <typename T>
static bool read_vec(std::FILE *f, std::vector<T> &v, size_t n) {
  v.resize(n);
  return std::fread(v.data(), sizeof(T), n, f) == n;
}
template <typename T>
static hipError_t to_device(const std::vector<T> &h, T **d) {
  hipError_t e = hipMalloc(reinterpret_cast<void **>(d), h.size() * sizeof(T));
  return e != hipSuccess ? e : hipMemcpy(*d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice);
}

int main(int argc, char **argv) {
  if (argc != 3) return 1;
  std::FILE *f = std::fopen(argv[1], "rb");
  if (!f) return 1;
  int32_t hdr[5];
  if (std::fread(hdr, sizeof(int32_t), 5, f) != 5) return 1;
  const int S = hdr[0], MB = hdr[1], NB = hdr[2];
  std::vector<uint16_t> q, kn, vn, kc, vc;
  std::vector<int32_t> bt, sl;
  std::vector<int64_t> slot;
  std::vector<float> sinks;
  const size_t row = 8 * 64, cache = (size_t)NB * 16 * row;
  if (!read_vec(f, q, (size_t)S * 64 * 64) || !read_vec(f, kn, S * row) || !read_vec(f, vn, S * row) ||
      !read_vec(f, kc, cache) || !read_vec(f, vc, cache) || !read_vec(f, bt, (size_t)S * MB) ||
      !read_vec(f, sl, S) || !read_vec(f, slot, S) || !read_vec(f, sinks, 64))
    return 1;
  std::fclose(f);

  eid_attn_desc d{};
  d.struct_size = sizeof d;
  d.num_seqs = d.num_q_tokens = S;
  d.max_q_len = 1;
  d.max_kv_len = hdr[4];
  d.num_q_heads = 64;
  d.num_kv_heads = 8;
  d.head_dim = 64;
  d.block_size = 16;
  d.max_blocks_per_seq = MB;
  d.num_blocks = NB;
  d.softmax_scale = 0.125f;
  d.window = hdr[3];
  d.kv_dtype = EID_KV_BF16;

  uint16_t *dq, *dkn, *dvn, *dkc, *dvc, *dout;
  int32_t *dbt, *dsl;
  int64_t *dslot;
  float *dsinks;
  void *ws;
  HIP_OK(to_device(q, &dq));
  HIP_OK(to_device(kn, &dkn));
  HIP_OK(to_device(vn, &dvn));
  HIP_OK(to_device(kc, &dkc));
  HIP_OK(to_device(vc, &dvc));
  HIP_OK(to_device(bt, &dbt));
  HIP_OK(to_device(sl, &dsl));
  HIP_OK(to_device(slot, &dslot));
  HIP_OK(to_device(sinks, &dsinks));
  HIP_OK(hipMalloc(reinterpret_cast<void **>(&dout), q.size() * sizeof(uint16_t)));
  const size_t ws_bytes = eid_workspace_bytes(&d);
  HIP_OK(hipMalloc(&ws, ws_bytes ? ws_bytes : 256));
  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));

  EID_CHECK(eid_kv_write(&d, dkn, dvn, dkc, dvc, dslot, S, nullptr, nullptr, st));
  eid_attn_args a{};
  a.q = dq;
  a.out = dout;
  a.k_cache = dkc;
  a.v_cache = dvc;
  a.block_table = dbt;
  a.seq_lens = dsl;
  a.sinks = dsinks;
  a.workspace = ws;
  a.workspace_bytes = ws_bytes;
  a.seq_lens_host = sl.data();
  EID_CHECK(eid_attn_decode(&d, &a, st));
  HIP_OK(hipStreamSynchronize(st));

  std::vector<uint16_t> out(q.size()), krows(S * row), vrows(S * row);
  HIP_OK(hipMemcpy(out.data(), dout, out.size() * sizeof(uint16_t), hipMemcpyDeviceToHost));
  for (int s = 0; s < S; ++s) {
    HIP_OK(hipMemcpy(&krows[s * row], dkc + slot[s] * row, row * sizeof(uint16_t), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(&vrows[s * row], dvc + slot[s] * row, row * sizeof(uint16_t), hipMemcpyDeviceToHost));
  }
  std::FILE *g = std::fopen(argv[2], "wb");
  if (!g) return 1;
  std::fwrite(out.data(), sizeof(uint16_t), out.size(), g);
  std::fwrite(krows.data(), sizeof(uint16_t), krows.size(), g);
  std::fwrite(vrows.data(), sizeof(uint16_t), vrows.size(), g);
  std::fclose(g);
  std::printf("abi_caller: %d sequences, library version %u\n", S, eid_version());
  return 0;
}
